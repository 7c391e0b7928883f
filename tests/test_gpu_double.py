"""The double base type of the C ABI (DLL_InvokeDouble / DLL_InvokeDoubleEx2; CudaDnnDLL.cpp:494-853): the function ids of
the attention path on a kernel whose memory and arithmetic are double, against the checker in float64.  The reference's
own tests run every case once per base type (TestBase.cs:107-115); the bar here is what double arithmetic gives, 1e-12
relative, so a path that went through fp32 anywhere (2^-24) cannot pass it.  The rotary tables are the exception: the
reference builds them with powf / cosf / sinf for either base type (rope.cu:535-553), the checker's library calls may
differ from the C library's by an ulp of a float."""
import numpy as np
import pytest

from tests.conftest import assert_close
from mycaffe_amd.cudadnn import CUDAFN, CudaDnn, CudaDnnDouble, CudaDnnError
from mycaffe_amd.layers import Blob, CausalSelfAttentionLayer, InnerProductLayer, SoftmaxLayer, TransposeLayer
from oracle import attention_ref as R

pytestmark = pytest.mark.gpu

F64_RTOL = 1e-12
ROPE_RTOL = 2e-6


class DevD:
    def __init__(self):
        self.cuda = CudaDnnDouble(0)

    def put(self, a):
        return self.cuda.AllocMemory(np.asarray(a, np.float64))

    def zeros(self, n):
        return self.cuda.AllocMemory(int(n))

    def get(self, h, shape=None):
        a = self.cuda.GetMemoryFloat(h)
        assert a.dtype == np.float64
        return a.reshape(shape) if shape is not None else a


@pytest.fixture()
def devd():
    d = DevD()
    yield d
    d.cuda.Dispose()


def test_double_memory_keeps_every_bit(devd):
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(1000), [1.0 + 2.0 ** -52, 1e-300, -1e300, 2.0 ** -1074, np.pi]])
    h = devd.put(x)
    assert devd.get(h).tobytes() == x.tobytes()
    y = rng.standard_normal(x.size)
    devd.cuda.SetMemory(h, y)
    assert devd.get(h).tobytes() == y.tobytes()
    assert devd.cuda.GetMemoryFloat(h, 7).tobytes() == y[:7].tobytes()     # fits the caller's buffer
    h2 = devd.zeros(x.size)
    assert not devd.get(h2).any()
    devd.cuda.copy(100, h, h2, 5, 10)
    assert np.array_equal(devd.get(h2)[10:110], y[5:105])
    devd.cuda.set(x.size, h2, 1.0 / 3.0)
    assert np.all(devd.get(h2) == 1.0 / 3.0)
    devd.cuda.set(1, h2, 7.0, 3)
    assert devd.get(h2)[3] == 7.0 and devd.get(h2)[4] == 1.0 / 3.0
    devd.cuda.FreeMemory(h)
    with pytest.raises(CudaDnnError):
        devd.cuda.GetMemoryFloat(h)
    # the float table does not know the double table's kernels and the other way round: separate index spaces
    f = CudaDnn(0)
    hf = f.AllocMemory(np.float32([1, 2, 3]))
    assert f.GetMemoryFloat(hf).dtype == np.float32
    f.Dispose()


@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
def test_double_gemm_inline_vectors_and_random(devd, tA, tB):
    """The 2x3 . 3x4 case of TestCudaDnn.cs:5586-5686 in the four transpose combinations, then a random product."""
    A = np.arange(1, 7, dtype=np.float64).reshape(2, 3)
    B = np.arange(1, 13, dtype=np.float64).reshape(3, 4)
    hA, hB, hC = devd.put(A.T if tA else A), devd.put(B.T if tB else B), devd.zeros(8)
    devd.cuda.gemm(tA, tB, 2, 4, 3, 1.0, hA, hB, 0.0, hC)
    assert np.array_equal(devd.get(hC), [38, 44, 50, 56, 83, 98, 113, 128])
    rng = np.random.default_rng(5)
    m, n, k = 70, 45, 130
    A, B, C = rng.standard_normal((m, k)), rng.standard_normal((k, n)), rng.standard_normal((m, n))
    hA, hB, hC = devd.put(A.T if tA else A), devd.put(B.T if tB else B), devd.put(C)
    devd.cuda.gemm(tA, tB, m, n, k, 0.7, hA, hB, -1.3, hC)
    assert_close(devd.get(hC, (m, n)), 0.7 * A @ B - 1.3 * C, F64_RTOL, "gemm")


def test_double_gemm_is_double(devd, dev):
    # the same product on the float base type is off by 2^-24 and more; on the double base type by 2^-50
    rng = np.random.default_rng(6)
    A, B = rng.standard_normal((64, 256)), rng.standard_normal((256, 64))
    ref = A @ B
    hA, hB, hC = devd.put(A), devd.put(B), devd.zeros(64 * 64)
    devd.cuda.gemm(False, False, 64, 64, 256, 1.0, hA, hB, 0.0, hC)
    err_d = np.abs(devd.get(hC, (64, 64)) - ref).max() / np.abs(ref).max()
    fA, fB, fC = dev.put(A), dev.put(B), dev.zeros(64 * 64)
    dev.cuda.gemm(False, False, 64, 64, 256, 1.0, fA, fB, 0.0, fC)
    err_f = np.abs(dev.get(fC, (64, 64)) - ref).max() / np.abs(ref).max()
    assert err_d < 1e-14 and err_f > 1e-9


def test_double_matmul_gemv_and_vector_updates(devd):
    rng = np.random.default_rng(7)
    outer, m, n, k = 6, 33, 20, 17
    A, B = rng.standard_normal((outer, m, k)), rng.standard_normal((outer, k, n))
    hA, hB, hC = devd.put(A), devd.put(B), devd.zeros(outer * m * n)
    devd.cuda.matmul(outer, m, n, k, hA, hB, hC, 0.25)
    assert_close(devd.get(hC, (outer, m, n)), 0.25 * A @ B, F64_RTOL, "matmul")
    Bt = np.ascontiguousarray(B.transpose(0, 2, 1))
    hBt = devd.put(Bt)
    devd.cuda.matmul(outer, m, n, k, hA, hBt, hC, 1.0, False, True)
    assert_close(devd.get(hC, (outer, m, n)), A @ B, F64_RTOL, "matmul with B transposed")
    W, x, y = rng.standard_normal((40, 30)), rng.standard_normal(30), rng.standard_normal(40)
    hW, hx, hy = devd.put(W), devd.put(x), devd.put(y)
    devd.cuda.gemv(False, 40, 30, 2.0, hW, hx, 0.5, hy)
    assert_close(devd.get(hy), 2.0 * W @ x + 0.5 * y, F64_RTOL, "gemv")
    hy2 = devd.zeros(30)
    devd.cuda.gemv(True, 40, 30, 1.0, hW, hy, 0.0, hy2)
    assert_close(devd.get(hy2), W.T @ devd.get(hy), F64_RTOL, "gemv transposed")
    a, b = rng.standard_normal(1001), rng.standard_normal(1001)
    ha, hb, hc = devd.put(a), devd.put(b), devd.zeros(1001)
    devd.cuda.axpy(1001, 1.0 / 3.0, ha, hb)
    b2 = a / 3.0 + b
    assert_close(devd.get(hb), b2, F64_RTOL, "axpy")
    devd.cuda.scal(1001, 1.0 / 7.0, hb)
    assert_close(devd.get(hb), b2 / 7.0, F64_RTOL, "scal")
    devd.cuda.scale(1001, -2.5, ha, hc)
    assert np.array_equal(devd.get(hc), -2.5 * a)
    devd.cuda.add(1001, ha, hb, hc)
    assert_close(devd.get(hc), a + b2 / 7.0, F64_RTOL, "add")
    devd.cuda.add(1001, ha, hb, hc, 0.1)
    assert_close(devd.get(hc), a + 0.1 * (b2 / 7.0), F64_RTOL, "add with a factor")
    devd.cuda.mul(1001, ha, ha, hc)
    assert np.array_equal(devd.get(hc), a * a)
    devd.cuda.silu_fwd(1001, ha, hc)
    assert_close(devd.get(hc), R.silu(a, np.float64), F64_RTOL, "silu")


def test_double_mask_layout_ops_softmax_embed(devd):
    rng = np.random.default_rng(8)
    B, H, T = 2, 3, 16
    x = rng.standard_normal((B, H, T, T))
    causal = np.tril(np.ones((T, T)))
    hx, hm, hy = devd.put(x), devd.put(causal), devd.zeros(x.size)
    devd.cuda.mask(x.size, T * T, 0.0, -1e29, hx, hm, hy)
    assert np.array_equal(devd.get(hy), R.mask(x.size, T * T, 0.0, -1e29, x, causal, np.float64).reshape(-1))
    keym = (rng.random((B, T)) > 0.3).astype(np.float64)
    hk = devd.put(keym)
    devd.cuda.mask_batch(x.size, B, B * T, 0.0, -1e29, hx, hk, hy)
    want = R.mask_batch(x.size, B, B * T, 0.0, -1e29, x, keym, np.float64)
    assert np.array_equal(devd.get(hy), want.reshape(-1))
    # softmax through the descriptors, over the last axis (rows) and over channels
    sm = SoftmaxLayer(devd.cuda, -1)
    bx, by = Blob(devd.cuda, x.shape), Blob(devd.cuda)
    bx.mutable_cpu_data = want.reshape(x.shape)
    sm.Forward(bx, by)
    assert_close(by.mutable_cpu_data, R.softmax_lastaxis(want.reshape(x.shape), np.float64), F64_RTOL, "softmax rows")
    sm1 = SoftmaxLayer(devd.cuda, 1)
    bx.mutable_cpu_data = x
    sm1.Forward(bx, by)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    assert_close(by.mutable_cpu_data, e / e.sum(axis=1, keepdims=True), F64_RTOL, "softmax over channels")
    # transposes and channel copy as the layer uses them
    t = TransposeLayer(devd.cuda, (0, 2, 1, 3))
    z = rng.standard_normal((2, 5, 3, 4))
    bz, bt = Blob(devd.cuda, z.shape), Blob(devd.cuda)
    bz.mutable_cpu_data = z
    t.Forward(bz, bt)
    assert np.array_equal(bt.mutable_cpu_data.reshape(2, 3, 5, 4), z.transpose(0, 2, 1, 3))
    hz, hz2 = devd.put(z), devd.zeros(z.size)
    devd.cuda.transposeHW(2, 5, 3, 4, hz, hz2)
    assert np.array_equal(devd.get(hz2, (2, 5, 4, 3)), z.transpose(0, 1, 3, 2))
    ip = rng.standard_normal((2, 7, 3 * 8))
    hip_, hq = devd.put(ip), devd.zeros(2 * 7 * 8)
    devd.cuda.channel_copy(2 * 7 * 8, 2, 7, 3, 8, 1, hip_, hq, 0)
    assert np.array_equal(devd.get(hq, (2, 7, 8)), ip[:, :, 8:16])
    ids = rng.integers(0, 11, 9).astype(np.float64)
    w = rng.standard_normal((11, 6))
    hi, hw, ht = devd.put(ids), devd.put(w), devd.zeros(9 * 6)
    devd.cuda.embed_fwd(9 * 6, hi, hw, 9, 6, 11, ht)
    assert np.array_equal(devd.get(ht, (9, 6)), w[ids.astype(int)])


@pytest.mark.parametrize("B,T,H,hs,off", [(2, 16, 3, 8, -1), (1, 9, 2, 64, -1), (1, 1, 2, 16, 5)])
def test_double_rope_forward(devd, B, T, H, hs, off):
    S = 16
    rng = np.random.default_rng(T)
    x = rng.standard_normal((B, T, H, hs))
    hr = devd.cuda.CreateRope(0, 0, x.size, B, S, H, hs, 10000.0)
    hx, hy = devd.put(x), devd.zeros(x.size)
    devd.cuda.RopeForward(hr, x.size, hx, hy, off)
    want = R.rope_forward(x, S, H, hs, 10000.0, off, np.float64, base_double=True)
    assert_close(devd.get(hy), want, ROPE_RTOL, "rope")
    # the rotation keeps the length of every pair: a property no table error can hide
    got = devd.get(hy).reshape(-1, 2)
    assert_close((got ** 2).sum(axis=1), (x.reshape(-1, 2) ** 2).sum(axis=1), 1e-6, "pair norms")
    devd.cuda.FreeRope(hr)


@pytest.mark.parametrize("kind", ["causal", "none", "keys", "per_sequence"])
def test_double_attention_forward(devd, kind):
    B, H, T, hs = 2, 3, 40, 16
    rng = np.random.default_rng(3)
    q, k, v = (rng.standard_normal((B, H, T, hs)) for _ in range(3))
    hc, ha = devd.cuda.CreateCuDNN(), devd.cuda.CreateAttn()
    devd.cuda.SetAttn(hc, ha, 0, False, B, 64, H, hs, 0.0)
    hq, hk, hv, hy = devd.put(q), devd.put(k), devd.put(v), devd.zeros(q.size)
    if kind == "causal":
        m = np.tril(np.ones((T, T)))
        hm, bm = devd.put(m), 0
        full = np.broadcast_to(m, (B, H, T, T))
    elif kind == "none":
        hm, bm, full = 0, 0, np.ones((B, H, T, T))
    elif kind == "keys":
        m = (rng.random((B, T)) > 0.4).astype(np.float64)
        m[1, :] = 0                                        # a sequence with every key masked: uniform weights
        hm, bm = devd.put(m), 1
        full = np.broadcast_to(m[:, None, None, :], (B, H, T, T))
    else:
        m = (rng.random((B, T, T)) > 0.4).astype(np.float64)
        hm, bm = devd.put(m), 2
        full = np.broadcast_to(m[:, None], (B, H, T, T))
    devd.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, bm)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) / np.sqrt(hs)
    s = np.where(full == 0, -1e29, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    assert_close(devd.get(hy, q.shape), np.einsum("bhqk,bhkd->bhqd", p, v), F64_RTOL, "attention, " + kind)
    if kind == "causal":
        ref, _ = R.attn_forward(q, k, v, R.causal_mask(T, np.float64), False, np.float64)
        assert_close(devd.get(hy, q.shape), ref, F64_RTOL, "attention vs the checker")
    devd.cuda.FreeAttn(ha)
    devd.cuda.FreeCuDNN(hc)


@pytest.mark.parametrize("sdpa", [True, False])
@pytest.mark.parametrize("rope", [False, True])
def test_double_causal_self_attention_layer(devd, sdpa, rope):
    """CausalSelfAttentionLayer.forward (CausalSelfAttentionLayer.cs:526-605) on the double base type, through the fused
    attention handle and through the explicit chain (transposes, MatMul, scale, mask, softmax, MatMul), against the
    checker in float64."""
    B, T, C, H = 2, 24, 48, 3
    rng = np.random.default_rng(11)
    x = rng.standard_normal((B, T, C))
    wa, wp = rng.standard_normal((3 * C, C)) * 0.1, rng.standard_normal((C, C)) * 0.1
    ba, bp = rng.standard_normal(3 * C) * 0.1, rng.standard_normal(C) * 0.1
    layer = CausalSelfAttentionLayer(devd.cuda, H, C, T, True, sdpa, enable_rotary_positional_embedding=rope)
    bottom, top = Blob(devd.cuda, x.shape), Blob(devd.cuda)
    bottom.mutable_cpu_data = x
    layer.Setup(bottom, wa, ba, wp, bp)
    layer.Forward(bottom, top)
    y = top.mutable_cpu_data
    assert y.dtype == np.float64
    ref = R.causal_self_attention(x, wa, ba, wp, bp, H, rope=(T, 10000.0) if rope else None, dtype=np.float64)["y"]
    assert_close(y, ref, ROPE_RTOL if rope else F64_RTOL, "layer output")


def test_double_activations_softmax_rope_gradients(devd):
    rng = np.random.default_rng(22)
    n = 5001
    x, g = rng.standard_normal(n) * 3, rng.standard_normal(n)
    hx, hg, hy, hdx = devd.put(x), devd.put(g), devd.zeros(n), devd.zeros(n)
    for bert in (True, False):
        devd.cuda.gelu_fwd(n, hx, hy, bert)
        assert_close(devd.get(hy), R.gelu(x, bert, np.float64), F64_RTOL, "gelu bert=%s" % bert)
        devd.cuda.gelu_bwd(n, hg, hy, hdx, hx, bert)
        assert_close(devd.get(hdx), R.gelu_grad(x, g, bert, np.float64), F64_RTOL, "gelu grad bert=%s" % bert)
    devd.cuda.silu_bwd(n, hg, hy, hdx, hx)
    assert_close(devd.get(hdx), R.silu_grad(x, g, np.float64), F64_RTOL, "silu grad")
    for slope in (0.0, 0.1):
        devd.cuda.relu_fwd(n, hx, hy, slope)
        y = devd.get(hy)
        assert_close(y, R.relu(x, slope, np.float64), F64_RTOL, "relu")
        devd.cuda.relu_bwd(n, hg, hy, hdx, slope)
        assert_close(devd.get(hdx), R.relu_grad(y, g, slope, np.float64), F64_RTOL, "relu grad")
    devd.cuda.SwigluForward(n, hx, hg, hy)
    assert_close(devd.get(hy), R.silu(x, np.float64) * g, F64_RTOL, "swiglu")
    # softmax gradient through the layer (cuDNN engine ids 111 / 112)
    z, dz = rng.standard_normal((3, 4, 5, 33)), rng.standard_normal((3, 4, 5, 33))
    sm = SoftmaxLayer(devd.cuda, -1)
    bz, bt = Blob(devd.cuda, z.shape), Blob(devd.cuda)
    bz.mutable_cpu_data = z
    sm.Forward(bz, bt)
    bt.mutable_cpu_diff = dz
    sm.Backward(bt, bz)
    yy = R.softmax_lastaxis(z, np.float64)
    assert_close(bz.mutable_cpu_diff, R.softmax_backward(yy, dz, -1, False, np.float64), F64_RTOL, "softmax gradient")
    # rope backward undoes rope forward
    B, T, H, hs = 2, 12, 3, 16
    r = rng.standard_normal((B, T, H, hs))
    hr = devd.cuda.CreateRope(0, 0, r.size, B, T, H, hs, 10000.0)
    h1, h2, h3 = devd.put(r), devd.zeros(r.size), devd.zeros(r.size)
    devd.cuda.RopeForward(hr, r.size, h1, h2)
    devd.cuda.RopeBackward(hr, r.size, h1, h2, h3)
    assert_close(devd.get(h3), r, 1e-6, "rope round trip")
    assert_close(devd.get(h3), R.rope_backward(devd.get(h2), T, H, hs, dtype=np.float64), ROPE_RTOL, "rope gradient")


@pytest.mark.parametrize("kind", ["causal", "keys", "cross"])
def test_double_attention_backward(devd, kind):
    B, H, hs = 2, 2, 16
    Tq, Tk = (24, 40) if kind == "cross" else (32, 32)
    rng = np.random.default_rng(9)
    q = rng.standard_normal((B, H, Tq, hs))
    k, v = rng.standard_normal((B, H, Tk, hs)), rng.standard_normal((B, H, Tk, hs))
    dy = rng.standard_normal((B, H, Tq, hs))
    hc, ha = devd.cuda.CreateCuDNN(), devd.cuda.CreateAttn()
    devd.cuda.SetAttn(hc, ha, 0, True, B, 64, H, hs, 0.0)
    if kind == "causal":
        m = np.tril(np.ones((Tq, Tk)))
        hm, bm, full = devd.put(m), 0, np.broadcast_to(m, (B, H, Tq, Tk))
    elif kind == "keys":
        m = (rng.random((B, Tk)) > 0.4).astype(np.float64)
        hm, bm, full = devd.put(m), 1, np.broadcast_to(m[:, None, None, :], (B, H, Tq, Tk))
    else:
        hm, bm, full = 0, 0, np.ones((B, H, Tq, Tk))
    hq, hk, hv, hy, hdy = devd.put(q), devd.put(k), devd.put(v), devd.zeros(q.size), devd.put(dy)
    hdq, hdk, hdv = devd.zeros(q.size), devd.zeros(k.size), devd.zeros(v.size)
    devd.cuda.AttnScaledDotProductForward(hc, ha, Tq, hq, hk, hv, hm, hy, bm, Tk)
    devd.cuda.AttnScaledDotProductBackward(hc, ha, hq, hdq, hk, hdk, hv, hdv, 0, hy, hdy)
    s = np.einsum("bhqd,bhkd->bhqk", q, k) / np.sqrt(hs)
    s = np.where(full == 0, -1e29, s)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    dv = np.einsum("bhqk,bhqd->bhkd", p, dy)
    dp = np.einsum("bhqd,bhkd->bhqk", dy, v)
    ds = p * (dp - (p * dp).sum(-1, keepdims=True)) / np.sqrt(hs)
    assert_close(devd.get(hdv, v.shape), dv, F64_RTOL, "dV")
    assert_close(devd.get(hdq, q.shape), np.einsum("bhqk,bhkd->bhqd", ds, k), 1e-11, "dQ")
    assert_close(devd.get(hdk, k.shape), np.einsum("bhqk,bhqd->bhkd", ds, q), 1e-11, "dK")


@pytest.mark.parametrize("sdpa", [True, False])
@pytest.mark.parametrize("name,heads", [("gpt-pico-blk3", 3), ("gpt-pico-blk3B", 3)])
def test_double_transformer_block_forward_and_backward_golden(devd, name, heads, sdpa, golden_dir):
    """The reference's own dump of a GPT block (layer norm handle, attention, ReLU MLP, residuals): activations and
    gradients, the C# call sequence replayed on the double base type - what its test base does for T = double."""
    import os
    from mycaffe_amd.layers import TransformerBlockLayer
    from tests.conftest import load_txt
    d = os.path.join(golden_dir, name)
    g = os.path.join(d, "iter_0")
    p = {k: load_txt(os.path.join(d, k + ".txt")) for k in ("attn_weight", "attn_bias", "attn_proj_weight", "attn_proj_bias",
                                                             "fc_weight", "fc_bias", "proj_weight", "proj_bias")}
    x = load_txt(os.path.join(d, "1_x.txt"))
    B, T, C = x.shape
    layer = TransformerBlockLayer(devd.cuda, heads, C, T, "relu", True, 1e-10, sdpa, training=True)
    bx, top = Blob(devd.cuda, x.shape), Blob(devd.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    assert_close(top.mutable_cpu_data, load_txt(os.path.join(d, "10_y.txt")), 2e-6, "block y")
    top.mutable_cpu_diff = load_txt(os.path.join(g, "grad_1_y.txt"))
    layer.Backward(top, bx)
    assert_close(layer.b["Norm2"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_6_x_ln2.txt")), 2e-5, "grad ln2 out")
    assert_close(bx.mutable_cpu_diff, load_txt(os.path.join(g, "grad_10_x.txt")), 5e-5, "grad x")
    # and against the checker in float64, where the bar is double's
    ref = R.transformer_block_gpt(x, p, heads, "relu", 1e-10, np.float64)
    assert_close(top.mutable_cpu_data, ref["y"], 1e-10, "block y vs the float64 checker")


@pytest.mark.parametrize("fused_rmsnorm,sdpa", [(False, False), (True, True)])
def test_double_llama_style_block_and_its_gradient(devd, fused_rmsnorm, sdpa):
    """The Llama-style block (RMSNorm chain of primitives or the fused id, rotary attention, SiLU-gated MLP) on the double
    base type: forward against the checker, input gradient against central differences of the checker."""
    from mycaffe_amd.layers import TransformerBlockLayer
    rng = np.random.default_rng(85)
    B, T, C, H = 2, 6, 16, 2
    layer = TransformerBlockLayer(devd.cuda, H, C, T, "silu", False, 1e-5, sdpa, training=not fused_rmsnorm, enable_llama_style_head=True,
                                  multiple_of=8, fused_rmsnorm=fused_rmsnorm)
    hid = layer.fc1.N
    p = {"rms1_weight": 1 + 0.1 * rng.standard_normal(C), "rms2_weight": 1 + 0.1 * rng.standard_normal(C),
         "attn_weight": rng.standard_normal((3 * C, C)) * 0.3, "attn_proj_weight": rng.standard_normal((C, C)) * 0.3,
         "fc_weight": rng.standard_normal((hid, C)) * 0.3, "fc2_weight": rng.standard_normal((hid, C)) * 0.3,
         "proj_weight": rng.standard_normal((C, hid)) * 0.3}
    x, dy = rng.standard_normal((B, T, C)), rng.standard_normal((B, T, C))
    bx, top = Blob(devd.cuda, x.shape), Blob(devd.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    assert_close(top.mutable_cpu_data, R.transformer_block_llama(x, p, H, T, 10000.0, 1e-5, np.float64), ROPE_RTOL, "llama block")
    if fused_rmsnorm:
        return
    top.mutable_cpu_diff = dy
    layer.Backward(top, bx)
    got = bx.mutable_cpu_diff.reshape(x.shape)

    def loss(xx):
        return float((R.transformer_block_llama(xx, p, H, T, 10000.0, 1e-5, np.float64) * dy).sum())

    num, h = np.zeros(x.shape), 1e-6
    for i in np.ndindex(*x.shape):
        xp, xm = x.copy(), x.copy()
        xp[i] += h
        xm[i] -= h
        num[i] = (loss(xp) - loss(xm)) / (2 * h)
    assert_close(got, num, 1e-5, "llama block dx")


def test_double_memory_pointers_alias_the_allocation(devd):
    x = np.arange(100, dtype=np.float64)
    h = devd.put(x)
    v = devd.cuda.CreateMemoryPointer(h, 10, 20)
    assert np.array_equal(devd.get(v), x[10:30])
    devd.cuda.set(20, v, -1.0)
    assert np.array_equal(devd.get(h)[10:30], np.full(20, -1.0)) and devd.get(h)[9] == 9 and devd.get(h)[30] == 30
    v2 = devd.cuda.CreateMemoryPointer(v, 5, 5)              # a view of a view aliases the allocation
    devd.cuda.set(5, v2, 2.0)
    assert np.array_equal(devd.get(h)[15:20], np.full(5, 2.0))
    with pytest.raises(CudaDnnError):
        devd.cuda.CreateMemoryPointer(h, 90, 20)
    devd.cuda.FreeMemoryPointer(v2)
    assert devd.get(h)[15] == 2.0                             # freeing a view frees nothing else
    devd.cuda.FreeMemory(h)
    with pytest.raises(CudaDnnError):
        devd.cuda.GetMemoryFloat(v)                           # views go with their allocation


@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("m,n,k", [(37, 53, 29), (128, 96, 64), (1, 7, 300)])
def test_double_linear_forward(devd, bias, m, n, k):
    rng = np.random.default_rng(m + n)
    x, W, b = rng.standard_normal((m, k)), rng.standard_normal((n, k)), rng.standard_normal(n)
    hx, hW, hb, hy = devd.put(x), devd.put(W), devd.put(b), devd.put(np.full(m * n, 9.0))
    devd.cuda.LinearForward(m, n, k, hx, hW, hb if bias else 0, hy)
    assert_close(devd.get(hy, (m, n)), x @ W.T + (b if bias else 0.0), F64_RTOL, "linear forward")
    with pytest.raises(CudaDnnError):
        devd.cuda.LinearForward(m, n + 1, k, hx, hW, hb, hy)


@pytest.mark.parametrize("rope", [False, True])
@pytest.mark.parametrize("bias", [True, False])
def test_double_qkv_proj_heads(devd, rope, bias):
    B, T, H, hs = 2, 12, 3, 8
    C = H * hs
    rng = np.random.default_rng(4)
    x, W, b = rng.standard_normal((B, T, C)), rng.standard_normal((3 * C, C)) * 0.2, rng.standard_normal(3 * C)
    hx, hW, hb = devd.put(x), devd.put(W), devd.put(b)
    hq, hk, hv = (devd.zeros(B * T * C) for _ in range(3))
    hr = devd.cuda.CreateRope(0, 0, B * T * C, B, T, H, hs, 10000.0) if rope else 0
    devd.cuda.QkvProjHeads(B, T, H, hs, hx, hW, hb if bias else 0, hq, hk, hv, hr)
    ip = x.reshape(B * T, C) @ W.T + (b if bias else 0.0)
    for i, h in enumerate((hq, hk, hv)):
        part = ip[:, i * C:(i + 1) * C].reshape(B, T, H, hs)
        if rope and i < 2:
            part = np.asarray(R.rope_forward(part, T, H, hs, 10000.0, -1, np.float64, base_double=True)).reshape(B, T, H, hs)
        assert_close(devd.get(h, (B, H, T, hs)), part.transpose(0, 2, 1, 3), ROPE_RTOL if rope else F64_RTOL, "qkv part %d" % i)
    if rope:
        other = devd.cuda.CreateRope(0, 0, B * T * C, B, T, H + 1, hs, 10000.0)
        with pytest.raises(CudaDnnError):
            devd.cuda.QkvProjHeads(B, T, H, hs, hx, hW, hb, hq, hk, hv, other)


def test_double_causal_self_attention_layer_as_three_calls(devd):
    B, T, C, H = 2, 24, 48, 3
    rng = np.random.default_rng(12)
    x = rng.standard_normal((B, T, C))
    wa, wp = rng.standard_normal((3 * C, C)) * 0.1, rng.standard_normal((C, C)) * 0.1
    ba, bp = rng.standard_normal(3 * C) * 0.1, rng.standard_normal(C) * 0.1
    for rope in (False, True):
        layer = CausalSelfAttentionLayer(devd.cuda, H, C, T, True, True, enable_rotary_positional_embedding=rope, fused_qkv_heads=True)
        bottom, top = Blob(devd.cuda, x.shape), Blob(devd.cuda)
        bottom.mutable_cpu_data = x
        layer.Setup(bottom, wa, ba, wp, bp)
        layer.Forward(bottom, top)
        ref = R.causal_self_attention(x, wa, ba, wp, bp, H, rope=(T, 10000.0) if rope else None, dtype=np.float64)["y"]
        assert_close(top.mutable_cpu_data, ref, ROPE_RTOL if rope else F64_RTOL, "three-call layer, double")


@pytest.mark.parametrize("kvH", [4, 2])
@pytest.mark.parametrize("append", [False, True])
def test_double_attn_decode_forward(devd, kvH, append):
    """Id 2001 on the double base type: one query per (sequence, head) over a cache with padded strides, grouped heads,
    with and without the rotate-and-append step, against the plain float64 formulas."""
    B, H, hs, L, S = 3, 4, 16, 37, 48
    rng = np.random.default_rng(kvH + 2 * append)
    sT, sH = hs + 8, S * (hs + 8) + 16
    sB = kvH * sH + 32
    kc, vc = rng.standard_normal(B * sB), rng.standard_normal(B * sB)
    q, kn, vn = rng.standard_normal((B, H, hs)), rng.standard_normal((B, kvH, hs)), rng.standard_normal((B, kvH, hs))
    hq, hkc, hvc, hy = devd.put(q), devd.put(kc), devd.put(vc), devd.zeros(B * H * hs)
    hkn, hvn = devd.put(kn), devd.put(vn)
    hr = devd.cuda.CreateRope(0, 0, B * S * H * hs, B, S, H, hs, 10000.0)
    if append:
        devd.cuda.AttnDecodeForward(B, H, kvH, hs, L, hq, hkc, hvc, hy, sB, sH, sT, 0.0, hr, hkn, hvn)
    else:
        devd.cuda.AttnDecodeForward(B, H, kvH, hs, L, hq, hkc, hvc, hy, sB, sH, sT)
    fcos, fsin = R.rope_tables(S, hs, 10000.0, base_double=True)

    def rot(a, pos):
        a = a.reshape(-1, hs // 2, 2)
        c, sn = fcos[pos], fsin[pos]
        return np.stack([a[..., 0] * c - a[..., 1] * sn, a[..., 0] * sn + a[..., 1] * c], -1).reshape(-1, hs)

    qq = q.reshape(B * H, hs)
    K = np.zeros((B, kvH, L, hs)); V = np.zeros((B, kvH, L, hs))
    for b in range(B):
        for g in range(kvH):
            for t in range(L):
                o = b * sB + g * sH + t * sT
                K[b, g, t], V[b, g, t] = kc[o:o + hs], vc[o:o + hs]
    if append:
        qq = rot(qq, L - 1)
        K[:, :, L - 1] = rot(kn.reshape(-1, hs), L - 1).reshape(B, kvH, hs)
        V[:, :, L - 1] = vn
    qq = qq.reshape(B, H, hs)
    want = np.zeros((B, H, hs))
    for b in range(B):
        for h in range(H):
            g = h // (H // kvH)
            sc = K[b, g] @ qq[b, h] / np.sqrt(hs)
            p = np.exp(sc - sc.max())
            want[b, h] = (p / p.sum()) @ V[b, g]
    assert_close(devd.get(hy, (B, H, hs)), want, ROPE_RTOL if append else F64_RTOL, "decode attention, double")
    if append:
        # q and the new key were rotated in place and the caches hold the new rows
        assert_close(devd.get(hq, (B * H, hs)), rot(q.reshape(-1, hs), L - 1), ROPE_RTOL, "q rotated in place")
        got_kc, got_vc = devd.get(hkc), devd.get(hvc)
        o = 1 * sB + (kvH - 1) * sH + (L - 1) * sT
        assert_close(got_kc[o:o + hs], K[1, kvH - 1, L - 1], ROPE_RTOL, "appended key")
        assert np.array_equal(got_vc[o:o + hs], vn[1, kvH - 1])
        untouched = np.ones(B * sB, bool)
        for b in range(B):
            for g in range(kvH):
                o = b * sB + g * sH + (L - 1) * sT
                untouched[o:o + hs] = False
        assert np.array_equal(got_kc[untouched], kc[untouched]) and np.array_equal(got_vc[untouched], vc[untouched])
    with pytest.raises(CudaDnnError):
        devd.cuda.AttnDecodeForward(B, H, 3, hs, L, hq, hkc, hvc, hy, sB, sH, sT)          # heads not a multiple of kv heads
    with pytest.raises(CudaDnnError):
        devd.cuda.AttnDecodeForward(B, H, kvH, hs, S + 40, hq, hkc, hvc, hy, sB, sH, sT)    # past the cache


def test_double_ids_outside_the_built_set_say_so(devd):
    h = devd.zeros(16)
    with pytest.raises(CudaDnnError) as e:
        devd.cuda._ex2(CUDAFN.CUDA_BLOBLOADER_LOAD, None, [1, 4, h, 0])
    assert e.value.code == 90009 and "double" in str(e.value)
    with pytest.raises(CudaDnnError) as e:
        devd.cuda.CreateExtension("libmycaffe_hip_llama2.so")
    assert e.value.code == 90009
    # dropout in the handle is a float-only feature
    hc, ha = devd.cuda.CreateCuDNN(), devd.cuda.CreateAttn()
    with pytest.raises(CudaDnnError) as e:
        devd.cuda.SetAttn(hc, ha, 0, True, 1, 8, 1, 8, 0.1)
    assert e.value.code == 90009
