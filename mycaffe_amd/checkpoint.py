"""llama2.c checkpoint files, version 1, as the extension's ``LOAD`` reads them (llama2_cpu.cpp:108-170): a 256-byte
header (magic 0x616B3432, version 1, seven int32 config fields, one flag byte: classifier shared with the embedding) and
the fp32 tensors in the order of ``tensor_shapes``.  Used to write synthetic models of a given shape for benchmarks."""
import struct

import numpy as np

CONFIG_FIELDS = ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads", "vocab_size", "seq_len")


def tensor_shapes(cfg, shared_classifier):
    """Tensor names and shapes in file order."""
    dim, hid, L = cfg["dim"], cfg["hidden_dim"], cfg["n_layers"]
    kvd = dim // cfg["n_heads"] * cfg["n_kv_heads"]
    V = cfg["vocab_size"]
    shapes = [("rms_att", (L, dim)), ("rms_ffn", (L, dim)), ("rms_final", (dim,)), ("tok_emb", (V, dim)),
              ("wq", (L, dim, dim)), ("wk", (L, kvd, dim)), ("wv", (L, kvd, dim)), ("wo", (L, dim, dim)),
              ("w1", (L, hid, dim)), ("w2", (L, dim, hid)), ("w3", (L, hid, dim))]
    if not shared_classifier:
        shapes.append(("wcls", (V, dim)))
    return shapes


def random_model(cfg, seed, shared_classifier=False, std=0.02):
    """One flat fp32 array in file order: matrices ~ N(0, std) from ``numpy.random.default_rng(seed)``, drawn tensor
    by tensor in file order; the RMSNorm weights are 1."""
    rng = np.random.default_rng(seed)
    parts = []
    for name, shape in tensor_shapes(cfg, shared_classifier):
        if name.startswith("rms"):
            parts.append(np.ones(shape, np.float32).ravel())
        else:
            parts.append((rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).ravel())
    return np.concatenate(parts)


def write_v1(path, cfg, weights, shared_classifier=False):
    with open(path, "wb") as f:
        f.write(struct.pack("<Ii", 0x616B3432, 1))
        f.write(struct.pack("<7i", *[cfg[k] for k in CONFIG_FIELDS]))
        f.write(struct.pack("<B", 1 if shared_classifier else 0))
        f.write(b"\0" * (256 - f.tell()))
        np.asarray(weights, np.float32).tofile(f)
