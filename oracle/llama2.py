"""ctypes front end of liboracle_llama2.so plus the llama2.c ``.bin`` writer.

TEST INFRASTRUCTURE ONLY (parity checker + timed CPU baseline).

The checkpoint layout written by :func:`write_checkpoint_v1` is the one the
reference reads in CudaExtension.llm32.llama2/Files/llama2_cpu.cpp:108-159
(magic 0x616b3432, version 1, seven int32 config fields, one shared-classifier
byte, zero padding to 256 bytes, then fp32 tensors in the order of
memory_map_weights, llama2_cpu.cpp:74-106).
"""
import ctypes
import os
import struct
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle_llama2.so")

CONFIG_FIELDS = ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len")


class OrcConfig(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in CONFIG_FIELDS]


def build(force=False):
    """Compile the checker library with the committed Makefile."""
    if force or not os.path.exists(_LIB):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle_llama2.so"])
    return _LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB)
        fp = ctypes.POINTER(ctypes.c_float)
        ip = ctypes.POINTER(ctypes.c_int)
        L.orc_set_threads.argtypes = [ctypes.c_int]
        L.orc_set_threads.restype = ctypes.c_int
        L.orc_set_kv_bf16.argtypes = [ctypes.c_int]
        L.orc_round_bf16.argtypes = [fp, ctypes.c_int]
        L.orc_rmsnorm.argtypes = [fp, fp, fp, ctypes.c_int]
        L.orc_softmax.argtypes = [fp, ctypes.c_int]
        L.orc_matvec.argtypes = [fp, fp, fp, ctypes.c_int, ctypes.c_int]
        L.orc_rope_pairs.argtypes = [ctypes.c_int, ctypes.c_int, fp, fp, fp, fp, ctypes.c_int]
        L.orc_freq_tables.argtypes = [ctypes.c_int, ctypes.c_int, fp, fp]
        L.orc_argmax.argtypes = [fp, ctypes.c_int]
        L.orc_argmax.restype = ctypes.c_int
        L.orc_llama_weight_count.argtypes = [ctypes.POINTER(OrcConfig), ctypes.c_int]
        L.orc_llama_weight_count.restype = ctypes.c_size_t
        L.orc_llama_create.argtypes = [ctypes.POINTER(OrcConfig), fp, ctypes.c_int]
        L.orc_llama_create.restype = ctypes.c_void_p
        L.orc_llama_destroy.argtypes = [ctypes.c_void_p]
        L.orc_llama_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        L.orc_llama_forward.restype = fp
        L.orc_llama_generate_greedy.argtypes = [ctypes.c_void_p, ip, ctypes.c_int, ctypes.c_int, ip, fp]
        L.orc_llama_generate_greedy.restype = ctypes.c_int
        u64p = ctypes.POINTER(ctypes.c_ulonglong)
        L.orc_random_u32.argtypes = [u64p]
        L.orc_random_u32.restype = ctypes.c_uint
        L.orc_random_f32.argtypes = [u64p]
        L.orc_random_f32.restype = ctypes.c_float
        L.orc_sample_mult.argtypes = [fp, ctypes.c_int, ctypes.c_float]
        L.orc_sample_mult.restype = ctypes.c_int
        L.orc_sample_topp.argtypes = [fp, ctypes.c_int, ctypes.c_float, ctypes.c_float]
        L.orc_sample_topp.restype = ctypes.c_int
        L.orc_sample.argtypes = [fp, ctypes.c_int, ctypes.c_float, ctypes.c_float, u64p]
        L.orc_sample.restype = ctypes.c_int
        L.orc_llama_generate_sampled.argtypes = [ctypes.c_void_p, ip, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float,
                                                 u64p, ip]
        L.orc_llama_generate_sampled.restype = ctypes.c_int
        _lib = L
    return _lib


def _fp(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def rmsnorm(x, w):
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    o = np.empty_like(x)
    lib().orc_rmsnorm(_fp(o), _fp(x), _fp(w), x.size)
    return o


def softmax(x):
    x = np.array(x, np.float32, copy=True)
    lib().orc_softmax(_fp(x), x.size)
    return x


def matvec(w, x):
    w = np.ascontiguousarray(w, np.float32)
    x = np.ascontiguousarray(x, np.float32)
    d, n = w.shape
    o = np.empty(d, np.float32)
    lib().orc_matvec(_fp(o), _fp(x), _fp(w), n, d)
    return o


def freq_tables(hs, seq_len):
    c = np.empty((seq_len, hs // 2), np.float32)
    s = np.empty((seq_len, hs // 2), np.float32)
    lib().orc_freq_tables(hs, seq_len, _fp(c), _fp(s))
    return c, s


def rope_pairs(q, k, fcos, fsin, pos):
    """q, k: (n_heads, hs) rotated at position ``pos``; returns new arrays."""
    q = np.array(q, np.float32, copy=True)
    k = np.array(k, np.float32, copy=True)
    nh, hs = q.shape
    fcos = np.ascontiguousarray(fcos, np.float32)
    fsin = np.ascontiguousarray(fsin, np.float32)
    lib().orc_rope_pairs(nh, hs, _fp(q), _fp(k), _fp(fcos), _fp(fsin), pos * hs // 2)
    return q, k


def set_threads(n):
    """Limit the checker's parallel loops to ``n`` threads; returns the previous limit."""
    return int(lib().orc_set_threads(int(n)))


def set_kv_bf16(on):
    """Checker-only option (no counterpart in the reference): every forward from now on rounds the rotated key and the
    value of the current position to bfloat16 before they enter the cache and the attention."""
    lib().orc_set_kv_bf16(int(bool(on)))


def round_bf16(x):
    """fp32 -> nearest bfloat16 (ties to even), as fp32."""
    x = np.array(x, np.float32).ravel().copy()
    lib().orc_round_bf16(_fp(x), x.size)
    return x


def argmax(p):
    p = np.ascontiguousarray(p, np.float32)
    return int(lib().orc_argmax(_fp(p), p.size))


class Sampler:
    """llama2_sampler.cpp: build_sampler / sample with the xorshift64* state kept across calls."""

    def __init__(self, temperature, topp, seed):
        self.temperature, self.topp = float(temperature), float(topp)
        self.state = ctypes.c_ulonglong(int(seed) & 0xFFFFFFFFFFFFFFFF)

    def random_u32(self):
        return int(lib().orc_random_u32(ctypes.byref(self.state)))

    def random_f32(self):
        return float(lib().orc_random_f32(ctypes.byref(self.state)))

    def sample(self, logits):
        lg = np.array(logits, np.float32)   # copy: the routine overwrites its input
        return int(lib().orc_sample(_fp(lg), lg.size, self.temperature, self.topp, ctypes.byref(self.state)))


def sample_mult(p, coin):
    p = np.ascontiguousarray(p, np.float32)
    return int(lib().orc_sample_mult(_fp(p), p.size, float(coin)))


def sample_topp(p, topp, coin):
    p = np.ascontiguousarray(p, np.float32)
    return int(lib().orc_sample_topp(_fp(p), p.size, float(topp), float(coin)))


# ----------------------------------------------------------------------------
# synthetic checkpoints
# ----------------------------------------------------------------------------

def tensor_shapes(cfg, shared_classifier):
    """Tensor names and shapes in file order."""
    dim, hid, L = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"]
    hs = dim // cfg["n_heads"]
    kvd = hs * cfg["n_kv_heads"]
    V = cfg["vocab_size"]
    shapes = [
        ("rms_att", (L, dim)), ("rms_ffn", (L, dim)), ("rms_final", (dim,)),
        ("tok_emb", (V, dim)),
        ("wq", (L, dim, dim)), ("wk", (L, kvd, dim)), ("wv", (L, kvd, dim)), ("wo", (L, dim, dim)),
        ("w1", (L, hid, dim)), ("w2", (L, dim, hid)), ("w3", (L, hid, dim)),
    ]
    if not shared_classifier:
        shapes.append(("wcls", (V, dim)))
    return shapes


def random_weights(cfg, seed, shared_classifier=False, std=0.02):
    """N(0, std) matrices, RMSNorm weights = 1, as one flat fp32 blob + views."""
    rng = np.random.default_rng(seed)
    shapes = tensor_shapes(cfg, shared_classifier)
    total = sum(int(np.prod(s)) for _, s in shapes)
    blob = np.empty(total, np.float32)
    views, off = {}, 0
    for name, shp in shapes:
        n = int(np.prod(shp))
        v = blob[off:off + n].reshape(shp)
        if name.startswith("rms"):
            v[...] = 1.0
        else:
            v[...] = rng.standard_normal(shp, dtype=np.float32) * np.float32(std)
        views[name] = v
        off += n
    return blob, views


def write_checkpoint_v1(path, cfg, blob, shared_classifier=False):
    with open(path, "wb") as f:
        f.write(struct.pack("<I", 0x616B3432))
        f.write(struct.pack("<i", 1))
        f.write(struct.pack("<7i", *[cfg[k] for k in CONFIG_FIELDS]))
        f.write(struct.pack("<B", 1 if shared_classifier else 0))
        f.write(b"\0" * (256 - f.tell()))
        blob.astype(np.float32, copy=False).tofile(f)


class Llama:
    """The checker model: fp32 decode with a KV cache, one token at a time."""

    def __init__(self, cfg, blob, shared_classifier=False):
        self.cfg = dict(cfg)
        self._c = OrcConfig(*[cfg[k] for k in CONFIG_FIELDS])
        need = lib().orc_llama_weight_count(ctypes.byref(self._c), int(shared_classifier))
        self._blob = np.ascontiguousarray(blob, np.float32)
        if self._blob.size != need:
            raise ValueError("weight blob has %d floats, config needs %d" % (self._blob.size, need))
        self._h = lib().orc_llama_create(ctypes.byref(self._c), _fp(self._blob), int(shared_classifier))

    def forward(self, token, pos):
        p = lib().orc_llama_forward(self._h, int(token), int(pos))
        return np.ctypeslib.as_array(p, shape=(self.cfg["vocab_size"],)).copy()

    def generate_greedy(self, prompt, n_steps, want_logits=False):
        prompt = np.ascontiguousarray(prompt, np.int32)
        out = np.empty(n_steps, np.int32)
        lg = np.empty((n_steps, self.cfg["vocab_size"]), np.float32) if want_logits else None
        ip = ctypes.POINTER(ctypes.c_int)
        lib().orc_llama_generate_greedy(self._h, prompt.ctypes.data_as(ip), prompt.size, n_steps,
                                        out.ctypes.data_as(ip), _fp(lg) if want_logits else None)
        return (out, lg) if want_logits else out

    def generate_sampled(self, prompt, n_steps, sampler):
        """The generate loop with ``sampler`` (its state advances at every position, prompt included)."""
        prompt = np.ascontiguousarray(prompt, np.int32)
        out = np.empty(n_steps, np.int32)
        ip = ctypes.POINTER(ctypes.c_int)
        lib().orc_llama_generate_sampled(self._h, prompt.ctypes.data_as(ip), prompt.size, n_steps, sampler.temperature,
                                         sampler.topp, ctypes.byref(sampler.state), out.ctypes.data_as(ip))
        return out

    def close(self):
        if self._h:
            lib().orc_llama_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
