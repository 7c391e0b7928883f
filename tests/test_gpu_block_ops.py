"""GPU parity of the per-block ops around attention (LayerNorm handle, GELU / ReLU / SiLU and their gradients, RoPE
gradient, the GPT transformer block) through the C ABI, against the numpy checker and the reference-held fixtures."""
import os

import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnnError, DIR, ERROR
from mycaffe_amd.layers import Blob, TransformerBlockLayer
from oracle import attention_ref as R
from tests.conftest import BF16_RTOL, FP32_RTOL, GOLDEN, assert_close, bf16_round, load_txt

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["gpt-pico-ln", "gpt-pico-ln3", "gpt-pico-ln3B"])
def test_layernorm_handle_golden(dev, name):
    d = os.path.join(GOLDEN, name)
    x = load_txt(os.path.join(d, "x.txt"))
    B, T, C = x.shape
    h = dev.cuda.CreateLayerNorm(0, x.size, B, T, C, 1e-10)
    hx, hy = dev.put(x), dev.zeros(x.size)
    dev.cuda.LayerNormForward(h, hx, hy)
    y = dev.get(hy)
    assert_close(y, load_txt(os.path.join(d, "y.txt")), 2e-6, "layernorm fwd")
    hdy, hdx = dev.put(load_txt(os.path.join(d, "grad_1a_y.txt"))), dev.zeros(x.size)
    dev.cuda.LayerNormBackward(h, hy, hdy, hdx)
    assert_close(dev.get(hdx), load_txt(os.path.join(d, "grad_9_x.txt")), 2e-5, "layernorm bwd")
    dev.cuda.FreeLayerNorm(h)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.LayerNormForward(h, hx, hy)
    assert e.value.code == ERROR.LAYERNORM_NOT_INITIALIZED


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("shape", [(3, 7, 768), (2, 5, 1000), (4, 3, 24), (1, 2, 5000)])
def test_layernorm_vs_checker(dev, shape, half):
    rng = np.random.default_rng(21)
    x = bf16_round((rng.standard_normal(shape) * 2 + 0.5).astype(np.float32))
    dy = bf16_round(rng.standard_normal(shape).astype(np.float32))
    B, T, C = shape
    eps = 1e-5
    h = dev.cuda.CreateLayerNorm(0, x.size, B, T, C, eps)
    hx, hy, hdy, hdx = dev.put(x, half), dev.zeros(x.size, half), dev.put(dy, half), dev.zeros(x.size, half)
    dev.cuda.LayerNormForward(h, hx, hy)
    y, sd = R.layernorm_forward(x, C, eps, np.float64)
    tol = BF16_RTOL if half else 1e-5
    got_y = dev.get(hy)
    assert_close(got_y, y, tol, "layernorm fwd")
    # the gradient is checked on the y the device holds (bf16 storage rounds it)
    yy = got_y.reshape(shape).astype(np.float64)
    for calls in (1, 2):   # the divisor of the first rows grows by eps per backward call until the next forward
        dev.cuda.LayerNormBackward(h, hy, hdy, hdx)
        ref = R.layernorm_backward(yy, dy, sd, C, eps, calls, np.float64)
        assert_close(dev.get(hdx), ref, tol, "layernorm bwd call %d" % calls)
    dev.cuda.LayerNormForward(h, hx, hy)
    dev.cuda.LayerNormBackward(h, hy, hdy, hdx)
    assert_close(dev.get(hdx), R.layernorm_backward(yy, dy, sd, C, eps, 1, np.float64), tol, "layernorm bwd after forward")
    dev.cuda.FreeLayerNorm(h)


def test_layernorm_bad_arguments(dev):
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.CreateLayerNorm(0, 100, 2, 5, 11, 1e-5)   # count != outer*channels*inner
    assert e.value.code == ERROR.PARAM_OUT_OF_RANGE
    h = dev.cuda.CreateLayerNorm(0, 110, 2, 5, 11, 1e-5)
    hx, hy = dev.zeros(100), dev.zeros(110)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.LayerNormForward(h, hx, hy)
    assert e.value.code == ERROR.MEMORY_RANGE_EXCEEDED
    dev.cuda.FreeLayerNorm(h)


def test_gelu_golden(dev):
    d = os.path.join(GOLDEN, "gpt-pico-gelu")
    x = load_txt(os.path.join(d, "1_x.txt"))
    hx, hy = dev.put(x), dev.zeros(x.size)
    dev.cuda.gelu_fwd(x.size, hx, hy, True)
    assert_close(dev.get(hy), load_txt(os.path.join(d, "2_y.txt")), 1e-6, "gelu fwd")
    hdy, hdx = dev.put(load_txt(os.path.join(d, "grad_1_y.txt"))), dev.zeros(x.size)
    dev.cuda.gelu_bwd(x.size, hdy, hy, hdx, hx, True)
    assert_close(dev.get(hdx), load_txt(os.path.join(d, "grad_2_x.txt")), 1e-6, "gelu bwd")


@pytest.mark.parametrize("half", [False, True])
def test_activations_and_gradients_vs_checker(dev, half):
    rng = np.random.default_rng(22)
    n = 70001
    x = bf16_round((rng.standard_normal(n) * 3).astype(np.float32))
    g = bf16_round(rng.standard_normal(n).astype(np.float32))
    hx, hg, hy, hdx = dev.put(x, half), dev.put(g, half), dev.zeros(n, half), dev.zeros(n, half)
    tol = BF16_RTOL if half else 2e-6
    for bert in (True, False):
        dev.cuda.gelu_fwd(n, hx, hy, bert)
        assert_close(dev.get(hy), R.gelu(x, bert, np.float64), tol, "gelu bert=%s" % bert)
        dev.cuda.gelu_bwd(n, hg, hy, hdx, hx, bert)
        assert_close(dev.get(hdx), R.gelu_grad(x, g, bert, np.float64), tol, "gelu grad bert=%s" % bert)
    dev.cuda.silu_bwd(n, hg, hy, hdx, hx)
    assert_close(dev.get(hdx), R.silu_grad(x, g, np.float64), tol, "silu grad")
    for slope in (0.0, 0.1):
        dev.cuda.relu_fwd(n, hx, hy, slope)
        y = dev.get(hy)
        assert_close(y, R.relu(x, slope, np.float64), tol, "relu")
        dev.cuda.relu_bwd(n, hg, hy, hdx, slope)
        assert_close(dev.get(hdx), R.relu_grad(y, g, slope, np.float64), tol, "relu grad")


@pytest.mark.parametrize("half", [False, True])
def test_rope_backward_vs_checker(dev, half):
    rng = np.random.default_rng(23)
    B, T, H, hs = 2, 12, 3, 16
    x = bf16_round(rng.standard_normal((B, T, H, hs)).astype(np.float32))
    dy = bf16_round(rng.standard_normal((B, T, H, hs)).astype(np.float32))
    h = dev.cuda.CreateRope(0, 0, x.size, B, T, H, hs, 10000.0)
    hx, hdy, hdx = dev.put(x, half), dev.put(dy, half), dev.zeros(x.size, half)
    dev.cuda.RopeBackward(h, x.size, hx, hdy, hdx)
    assert_close(dev.get(hdx), R.rope_backward(dy, T, H, hs, dtype=np.float64), BF16_RTOL if half else 2e-6, "rope bwd")
    if not half:   # backward undoes forward
        hy = dev.zeros(x.size)
        dev.cuda.RopeForward(h, x.size, hx, hy)
        dev.cuda.RopeBackward(h, x.size, hx, hy, hdx)
        assert_close(dev.get(hdx), x, 2e-6, "rope round trip")
    dev.cuda.FreeRope(h)


@pytest.mark.parametrize("sdpa", [True, False])
@pytest.mark.parametrize("name,heads", [("gpt-pico-blk", 1), ("gpt-pico-blk3", 3), ("gpt-pico-blk3B", 3)])
def test_transformer_block_golden(dev, name, heads, sdpa):
    d = os.path.join(GOLDEN, name)
    p = {k: load_txt(os.path.join(d, k + ".txt")) for k in ("attn_weight", "attn_bias", "attn_proj_weight", "attn_proj_bias",
                                                             "fc_weight", "fc_bias", "proj_weight", "proj_bias")}
    x = load_txt(os.path.join(d, "1_x.txt"))
    B, T, C = x.shape
    layer = TransformerBlockLayer(dev.cuda, heads, C, T, "relu", True, 1e-10, sdpa)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    assert_close(top.mutable_cpu_data, load_txt(os.path.join(d, "10_y.txt")), 2e-6, "block y")
    assert_close(layer.b["Norm1"].mutable_cpu_data, load_txt(os.path.join(d, "2_x_ln11.txt")), 2e-6, "ln1")
    assert_close(layer.b["X"].mutable_cpu_data, load_txt(os.path.join(d, "4_x_p_attn.txt")), 2e-6, "x + attn")
    assert_close(layer.b["MlpOut"].mutable_cpu_data, load_txt(os.path.join(d, "8_x_c_proj.txt")), 2e-5, "mlp")


@pytest.mark.parametrize("activation", ["gelu_bert", "gelu", "relu"])
def test_transformer_block_gpt2_shape_vs_checker(dev, activation):
    rng = np.random.default_rng(24)
    B, T, C, H = 2, 64, 128, 2
    p = {"attn_weight": rng.standard_normal((3 * C, C)) * 0.05, "attn_bias": rng.standard_normal(3 * C) * 0.02,
         "attn_proj_weight": rng.standard_normal((C, C)) * 0.05, "attn_proj_bias": rng.standard_normal(C) * 0.02,
         "fc_weight": rng.standard_normal((4 * C, C)) * 0.05, "fc_bias": rng.standard_normal(4 * C) * 0.02,
         "proj_weight": rng.standard_normal((C, 4 * C)) * 0.05, "proj_bias": rng.standard_normal(C) * 0.02}
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    layer = TransformerBlockLayer(dev.cuda, H, C, T, activation, True, 1e-5, True)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    ref = R.transformer_block_gpt(x, {k: v.astype(np.float32) for k, v in p.items()}, H, activation, 1e-5, np.float64)
    assert_close(top.mutable_cpu_data, ref["y"], FP32_RTOL, "block %s" % activation)


def test_blob_loader_reads_a_llama_checkpoint_like_the_model_builder(dev, tmp_path):
    """The call sequence of LlamaModelBuilder.loadWeights_kpth0 (MyCaffe.model/LlamaModelBuilder.cs:239-420) against the
    legacy llama2.c file layout: 28-byte header, then tok_emb, rms_att, wq, wk, wv, wo, rms_ffn, w1, w2, w3, rms_final."""
    import struct
    rng = np.random.default_rng(61)
    dim, hid, L, H, V, S = 24, 40, 3, 4, 50, 16
    order = [("tok_emb", (V, dim)), ("rms_att", (L, dim)), ("wq", (L, dim, dim)), ("wk", (L, dim, dim)), ("wv", (L, dim, dim)),
             ("wo", (L, dim, dim)), ("rms_ffn", (L, dim)), ("w1", (L, hid, dim)), ("w2", (L, dim, hid)), ("w3", (L, hid, dim)),
             ("rms_final", (dim,))]
    w = {n: rng.standard_normal(s).astype(np.float32) for n, s in order}
    path = str(tmp_path / "legacy.bin")
    with open(path, "wb") as f:
        f.write(struct.pack("<7i", dim, hid, L, H, H, V, S))
        for n, _ in order:
            w[n].tofile(f)
    cuda = dev.cuda
    hdr = 28
    h = cuda.CreateBlobLoader(path)
    cuda.BlobLoaderResetOffset(h, hdr)
    hemb = dev.zeros(V * dim)
    cuda.LoadBlob(h, V * dim, hemb, 0)
    assert np.array_equal(dev.get(hemb, (V, dim)), w["tok_emb"])
    start = hdr + V * dim * 4
    per_layer = ["rms_att", "wq", "wk", "wv", "wo", "rms_ffn", "w1", "w2", "w3"]
    for i in range(L):
        cuda.BlobLoaderResetOffset(h, start)
        for n in per_layer:
            total = w[n].size
            one = total // L
            hd = dev.zeros(one, half=(n == "w1"))          # one blob kept in 16-bit storage
            cuda.LoadBlob(h, one, hd, i * one)
            cuda.BlobLoaderAddToOffset(h, total)
            got = dev.get(hd).reshape(w[n][i].shape)
            if n == "w1":
                assert np.array_equal(got, bf16_round(w[n][i])), (i, n)
            else:
                assert np.array_equal(got, w[n][i]), (i, n)
        hf = dev.zeros(dim)
        cuda.LoadBlob(h, dim, hf, 0)                          # after the last AddToOffset the cursor is at rms_final
        assert np.array_equal(dev.get(hf), w["rms_final"])
    # error behaviour
    with pytest.raises(CudaDnnError) as e:
        cuda.LoadBlob(h, dim + 1, hf, 0)                      # blob smaller than the request
    assert e.value.code == ERROR.INSUFFICIENT_BUFFER
    with pytest.raises(CudaDnnError) as e:
        cuda.LoadBlob(h, dim, hf, -1)
    assert e.value.code == ERROR.INVALID_PARAMETER
    with pytest.raises(CudaDnnError) as e:
        cuda.LoadBlob(h, dim, hf, 1)                          # one item past the end of the file
    assert e.value.code == ERROR.MEMORY_RANGE_EXCEEDED
    cuda.FreeBlobLoader(h)
    with pytest.raises(CudaDnnError) as e:
        cuda.LoadBlob(h, dim, hf, 0)
    assert e.value.code == ERROR.BLOBLOADER_NOT_INITIALIZED
    with pytest.raises(CudaDnnError) as e:
        cuda.CreateBlobLoader(str(tmp_path / "missing.bin"))
    assert e.value.code == ERROR.FILE_NOT_FOUND


def _csa_params(d):
    return [load_txt(os.path.join(d, k + ".txt")) for k in ("attn_weight", "attn_bias", "attn_proj_weight", "attn_proj_bias")]


@pytest.mark.parametrize("sdpa", [True, False])
@pytest.mark.parametrize("name,heads", [("gpt-pico-csa", 1), ("gpt-pico-csa3", 3), ("gpt-pico-csa3B", 3), ("gpt-pico-csaB", 1)])
def test_causal_self_attention_layer_backward_golden(dev, name, heads, sdpa):
    """Forward + backward of the layer through the C ABI against the reference's dump of the same layer: grad_y in, grad_x
    out, with the gradients of q / k / v checked on the way; with the fused attention handle and with the layer's default
    chain (MatMul gradients around the softmax gradient, id 112)."""
    from mycaffe_amd.layers import CausalSelfAttentionLayer
    d = os.path.join(GOLDEN, name)
    g = os.path.join(d, "iter_0")
    x = load_txt(os.path.join(d, "x.txt"))
    B, T, C = x.shape
    layer = CausalSelfAttentionLayer(dev.cuda, heads, C, T, True, sdpa, training=True)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, *_csa_params(d))
    layer.Forward(bx, top)
    assert_close(top.mutable_cpu_data, load_txt(os.path.join(d, "y.txt")), 2e-6, "y")
    top.mutable_cpu_diff = load_txt(os.path.join(g, "grad_y.txt"))
    layer.Backward(top, bx)
    assert_close(layer.b["Qt"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_qt.txt")), 2e-5, "grad q")
    assert_close(layer.b["Kt"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_kt.txt")), 2e-5, "grad k")
    assert_close(layer.b["Vt"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_vt.txt")), 2e-5, "grad v")
    assert_close(bx.mutable_cpu_diff, load_txt(os.path.join(g, "grad_x.txt")), 2e-5, "grad x")
    if not sdpa:
        # the explicit chain's own intermediates: gradient of the probabilities, of the (scaled) scores, of k^T
        assert_close(layer.b["AttB"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_att_after_softmax.txt")), 2e-5, "grad att")
        assert_close(layer.b["AttA"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_qkt.txt")), 2e-5, "grad q k^T")
        assert_close(layer.b["Kt1"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_kt1.txt")), 2e-5, "grad k^T")


@pytest.mark.parametrize("half", [False, True])
def test_causal_self_attention_layer_backward_at_a_tiled_shape(dev, half):
    """Forward and backward of the layer at B = 2, T = 256, C = 256, four heads, in fp32 and in 16-bit storage, where the
    attention gradient runs on the tiled kernels and the inner products' data and weight gradients (InnerProductLayer.cs:
    429-494) on the A B^T kernels with a turned operand; against the float64 formulas of the same layer."""
    from mycaffe_amd.layers import CausalSelfAttentionLayer
    B, T, C, H = 2, 256, 256, 4
    hs = C // H
    rng = np.random.default_rng(77)
    x = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    wa = bf16_round((rng.standard_normal((3 * C, C)) * 0.05).astype(np.float32))
    wp = bf16_round((rng.standard_normal((C, C)) * 0.05).astype(np.float32))
    ba = bf16_round((rng.standard_normal(3 * C) * 0.1).astype(np.float32))
    bp = bf16_round((rng.standard_normal(C) * 0.1).astype(np.float32))
    dy = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, True, half=half, training=True)
    bx, top = Blob(dev.cuda, x.shape, half=half), Blob(dev.cuda, half=half)
    bx.mutable_cpu_data = x
    layer.Setup(bx, wa, ba, wp, bp)
    layer.Forward(bx, top)
    f = R.causal_self_attention(x, wa, ba, wp, bp, H, dtype=np.float64)
    tol = BF16_RTOL if half else 2e-5
    assert_close(top.mutable_cpu_data, f["y"], tol, "y")
    top.mutable_cpu_diff = dy
    layer.Backward(top, bx)
    # the layer's gradients in float64
    d = dy.astype(np.float64).reshape(B * T, C)
    merged = f["work"].transpose(0, 2, 1, 3).reshape(B * T, C)
    dwp, dbp = d.T @ merged, d.sum(0)
    dwork = (d @ wp.astype(np.float64)).reshape(B, T, H, hs).transpose(0, 2, 1, 3)
    dq, dk, dv = R.attn_backward(f["qt"], f["kt"], f["vt"], f["att"], dwork, np.float64)
    dqkv = np.concatenate([g.transpose(0, 2, 1, 3).reshape(B * T, C) for g in (dq, dk, dv)], axis=1)
    dwa, dba = dqkv.T @ x.astype(np.float64).reshape(B * T, C), dqkv.sum(0)
    dx = (dqkv @ wa.astype(np.float64)).reshape(B, T, C)
    assert_close(bx.mutable_cpu_diff, dx, tol, "grad x")
    assert_close(layer.c_attn.blobs[0].mutable_cpu_diff, dwa, tol, "grad w_attn")
    assert_close(layer.c_attn.blobs[1].mutable_cpu_diff, dba, tol, "grad b_attn")
    assert_close(layer.c_proj.blobs[0].mutable_cpu_diff, dwp, tol, "grad w_proj")
    assert_close(layer.c_proj.blobs[1].mutable_cpu_diff, dbp, tol, "grad b_proj")


@pytest.mark.parametrize("sdpa", [True, False])
@pytest.mark.parametrize("name,heads", [("gpt-pico-blk", 1), ("gpt-pico-blk3", 3), ("gpt-pico-blk3B", 3)])
def test_transformer_block_backward_golden(dev, name, heads, sdpa):
    d = os.path.join(GOLDEN, name)
    g = os.path.join(d, "iter_0")
    p = {k: load_txt(os.path.join(d, k + ".txt")) for k in ("attn_weight", "attn_bias", "attn_proj_weight", "attn_proj_bias",
                                                             "fc_weight", "fc_bias", "proj_weight", "proj_bias")}
    x = load_txt(os.path.join(d, "1_x.txt"))
    B, T, C = x.shape
    layer = TransformerBlockLayer(dev.cuda, heads, C, T, "relu", True, 1e-10, sdpa, training=True)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    top.mutable_cpu_diff = load_txt(os.path.join(g, "grad_1_y.txt"))
    layer.Backward(top, bx)
    assert_close(layer.b["Mlp1"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_5_x_c_fc.txt")), 2e-5, "grad fc out")
    assert_close(layer.b["Norm2"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_6_x_ln2.txt")), 2e-5, "grad ln2 out")
    assert_close(layer.b["Norm1"].mutable_cpu_diff, load_txt(os.path.join(g, "grad_9_ln1.txt")), 5e-5, "grad ln1 out")
    assert_close(bx.mutable_cpu_diff, load_txt(os.path.join(g, "grad_10_x.txt")), 5e-5, "grad x")


def test_norm_chain_primitives_vs_numpy(dev):
    """The elementwise / per-row ids the C# RMSNormLayer and LayerNormLayer chains call, each against its index rule."""
    rng = np.random.default_rng(81)
    cuda = dev.cuda
    outer, ch, inner = 3, 5, 48
    n = outer * ch * inner
    x = rng.standard_normal(n).astype(np.float32)
    x[7] = 0.0
    hx, hy = dev.put(x), dev.zeros(n)
    cuda.powx(n, hx, 2.0, hy)
    assert np.array_equal(dev.get(hy), x * x)
    cuda.powx(n, hx, 3.0, hy)
    assert_close(dev.get(hy), x.astype(np.float64) ** 3, 1e-6, "powx 3")
    cuda.sqrt(n, hy, hy)                                   # of negative values: NaN, as sqrtf gives
    cuda.powx(n, hx, 2.0, hy)
    cuda.sqrt(n, hy, hy, 0.25)
    assert_close(dev.get(hy), np.sqrt(x.astype(np.float64) ** 2 + 0.25), 1e-6, "sqrt eps")
    cuda.invert(n, hx, hy)
    ref = np.where(x == 0, 0, 1.0 / np.where(x == 0, 1, x))
    assert_close(dev.get(hy), ref, 1e-6, "invert")
    cuda.invert(n, hx, hy, 0, 0, 3.0, 2.0)
    assert_close(dev.get(hy), 1.5 * ref, 1e-6, "invert n/d")
    cuda.invert(n, hx, hy, 0, 0, -1.0)
    assert_close(dev.get(hy), -ref, 1e-6, "invert -1")
    hm = dev.zeros(outer * ch)
    cuda.channel_mean(n, outer, ch, inner, hx, hm)
    assert_close(dev.get(hm), x.reshape(outer * ch, inner).astype(np.float64).mean(1), 1e-6, "channel_mean")
    cuda.channel_fillfrom(n, outer, ch, inner, hm, hy, 0)
    assert np.array_equal(dev.get(hy), np.repeat(dev.get(hm), inner))
    hb = dev.zeros(outer * ch)
    cuda.channel_fillfrom(n, outer, ch, inner, hb, hx, 1)  # backward: picks the first value of every row
    assert np.array_equal(dev.get(hb), x.reshape(outer * ch, inner)[:, 0])
    cuda.channel_duplicate(n, outer * ch, 1, inner, hm, hy)
    assert np.array_equal(dev.get(hy), np.repeat(dev.get(hm), inner))
    w = rng.standard_normal(inner).astype(np.float32)
    hw = dev.put(w)
    cuda.channel_copyall(n, outer * ch, 1, inner, hw, hy)
    assert np.array_equal(dev.get(hy), np.tile(w, outer * ch))
    d2 = rng.standard_normal((2, 3, 4)).astype(np.float32)   # duplicate with more than one channel: (num, dup, channels)
    hd, hd2 = dev.put(d2[:, 0, :].copy()), dev.zeros(d2.size)
    cuda.channel_duplicate(d2.size, 2, 4, 3, hd, hd2)
    assert np.array_equal(dev.get(hd2, d2.shape), np.broadcast_to(d2[:, :1, :], d2.shape))
    a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    b[11] = 0.0
    ha, hb2 = dev.put(a), dev.put(b)
    cuda.sub(n, ha, hb2, hy)
    assert np.array_equal(dev.get(hy), a - b)
    cuda.sub(n, ha, hb2, hy, 0, 0, 0, inner)
    assert np.array_equal(dev.get(hy), a - np.tile(b[:inner], outer * ch))
    cuda.div(n, ha, hb2, hy)
    assert_close(dev.get(hy), np.where(b == 0, 0, a / np.where(b == 0, 1, b)), 1e-6, "div")
    cuda.add_scalar(n, 0.5, ha)
    assert np.array_equal(dev.get(ha), a + np.float32(0.5))
    cuda.add_scalar(10, 1.0, ha, 5)
    exp = a + np.float32(0.5)
    exp[5:15] += 1
    assert np.array_equal(dev.get(ha), exp)


@pytest.mark.parametrize("half", [False, True])
def test_channel_sum_forms_vs_numpy(dev, half):
    """Ids 292 and 309: sums across the channels and within every channel, and the backward forms that spread the sums."""
    rng = np.random.default_rng(83)
    cuda = dev.cuda
    tol = BF16_RTOL if half else 1e-6
    for outer, ch, inner in [(3, 5, 48), (2, 1024, 70), (4, 7, 1), (1, 1, 300), (2, 130, 64), (1, 4096, 768), (1, 300, 70), (1, 1000, 36)]:
        n = outer * ch * inner
        x = bf16_round(rng.standard_normal((outer, ch, inner)).astype(np.float32))
        hx, ha, hw = dev.put(x, half), dev.zeros(outer * inner, half), dev.zeros(outer * ch, half)
        cuda.channel_sum(n, outer, ch, inner, hx, ha)
        assert_close(dev.get(ha, (outer, inner)), x.astype(np.float64).sum(1), tol, "channel_sum %s" % ((outer, ch, inner),))
        cuda.channel_sumEx(n, outer, ch, inner, hx, ha, True, DIR.FWD)
        assert_close(dev.get(ha, (outer, inner)), x.astype(np.float64).sum(1), tol, "channel_sumEx across")
        cuda.channel_sumEx(n, outer, ch, inner, hx, hw, False, DIR.FWD)
        assert_close(dev.get(hw, (outer, ch)), x.astype(np.float64).sum(2), tol, "channel_sumEx within")
        across, within = dev.get(ha, (outer, 1, inner)), dev.get(hw, (outer, ch, 1))
        cuda.channel_sumEx(n, outer, ch, inner, hx, ha, True, DIR.BWD)
        assert np.array_equal(dev.get(hx, x.shape), np.broadcast_to(across, x.shape))
        cuda.channel_sumEx(n, outer, ch, inner, hx, hw, False, DIR.BWD)
        assert np.array_equal(dev.get(hx, x.shape), np.broadcast_to(within, x.shape))
    # a destination that holds one row of `inner` sums although outer > 1 (the weight gradient of RMSNormLayer): the
    # first entry's sums, nothing written past the end
    x = rng.standard_normal((3, 6, 40)).astype(np.float32)
    hx, hy = dev.put(x), dev.put(np.zeros(40 + 8, np.float32))
    hv = cuda.CreateMemoryPointer(hy, 0, 40)
    cuda.channel_sum(x.size, 3, 6, 40, hx, hv)
    got = dev.get(hy)
    assert_close(got[:40], x[0].astype(np.float64).sum(0), 1e-6, "channel_sum into one row")
    assert np.array_equal(got[40:], np.zeros(8, np.float32))
    cuda.FreeMemoryPointer(hv)
    with pytest.raises(CudaDnnError):
        cuda.channel_sum(x.size, 3, 6, 40, hx, dev.zeros(39))
    with pytest.raises(CudaDnnError) as e:
        cuda.channel_sumEx(x.size, 3, 6, 40, hx, dev.zeros(3 * 40), True, DIR.BWD, 1)
    assert e.value.code == ERROR.NOT_IMPLEMENTED


def test_rmsnorm_layer_backward_chain_vs_checker(dev):
    """RMSNormLayer.backward as the C# layer issues it (mul, channel_sum, channel_sumEx, powx, invert, channel_duplicate,
    scal, scale, add) against the checker's gradients, for one and for several leading entries."""
    from mycaffe_amd.layers import RMSNormLayer
    rng = np.random.default_rng(84)
    for shape in [(1, 9, 288), (3, 5, 64)]:
        x = rng.standard_normal(shape).astype(np.float32)
        w = (rng.standard_normal(shape[-1]) + 1.0).astype(np.float32)
        dy = rng.standard_normal(shape).astype(np.float32)
        layer = RMSNormLayer(dev.cuda, 1e-5, True, False)
        bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
        bx.mutable_cpu_data = x
        layer.Setup(bx, w)
        layer.Forward(bx, top)
        top.mutable_cpu_diff = dy
        layer.Backward(top, bx)
        dx, dw = R.rmsnorm_layer_backward(x, w, dy, 1e-5, np.float64)
        assert_close(bx.mutable_cpu_diff, dx, 1e-5, "rmsnorm dx %s" % (shape,))
        assert_close(layer.blobs[0].mutable_cpu_diff, dw, 1e-5, "rmsnorm dw %s" % (shape,))


@pytest.mark.parametrize("fused", [False, True])
def test_rmsnorm_layer_chain_vs_checker(dev, fused):
    from mycaffe_amd.layers import RMSNormLayer
    rng = np.random.default_rng(82)
    x = rng.standard_normal((2, 9, 288)).astype(np.float32)
    w = rng.standard_normal(288).astype(np.float32)
    for weights in (True, False):
        layer = RMSNormLayer(dev.cuda, 1e-5, weights, fused)
        bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
        bx.mutable_cpu_data = x
        layer.Setup(bx, w)
        layer.Forward(bx, top)
        assert_close(top.mutable_cpu_data, R.rmsnorm_layer(x, w if weights else None, 1e-5, np.float64), 1e-5, "rmsnorm layer")


def test_layernorm_layer_chain_equals_handle(dev):
    from mycaffe_amd.layers import LayerNormLayer
    rng = np.random.default_rng(83)
    x = (rng.standard_normal((2, 6, 96)) * 3 + 1).astype(np.float32)
    bx = Blob(dev.cuda, x.shape)
    bx.mutable_cpu_data = x
    outs = []
    for impl in (True, False):
        top = Blob(dev.cuda)
        LayerNormLayer(dev.cuda, 1e-5, impl).Forward(bx, top)
        outs.append(top.mutable_cpu_data)
    ref, _ = R.layernorm_forward(x, 96, 1e-5, np.float64)
    assert_close(outs[0], ref, 1e-5, "handle")
    assert_close(outs[1], ref, 1e-5, "chain")


@pytest.mark.parametrize("fused_rmsnorm,sdpa", [(False, False), (True, True)])
def test_transformer_block_llama_style_vs_checker(dev, fused_rmsnorm, sdpa):
    """The Llama-style block (RMSNorm chain or the fused id, rotary attention without bias, SiLU-gated MLP) through the
    layer mirrors, against the checker."""
    rng = np.random.default_rng(84)
    B, T, C, H = 2, 32, 128, 2
    layer = TransformerBlockLayer(dev.cuda, H, C, T, "silu", False, 1e-5, sdpa, enable_llama_style_head=True, multiple_of=32,
                                  fused_rmsnorm=fused_rmsnorm)
    hid = layer.fc1.N
    assert hid == 352    # 2 * (4 * 128) / 3 = 341 rounded up to a multiple of 32
    p = {"rms1_weight": 1 + 0.1 * rng.standard_normal(C), "rms2_weight": 1 + 0.1 * rng.standard_normal(C),
         "attn_weight": rng.standard_normal((3 * C, C)) * 0.05, "attn_proj_weight": rng.standard_normal((C, C)) * 0.05,
         "fc_weight": rng.standard_normal((hid, C)) * 0.05, "fc2_weight": rng.standard_normal((hid, C)) * 0.05,
         "proj_weight": rng.standard_normal((C, hid)) * 0.05}
    p = {k: v.astype(np.float32) for k, v in p.items()}
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    ref = R.transformer_block_llama(x, p, H, T, 10000.0, 1e-5, np.float64)
    assert_close(top.mutable_cpu_data, ref, FP32_RTOL, "llama block")


@pytest.mark.parametrize("sdpa", [True, False])
def test_transformer_block_llama_style_backward_vs_finite_differences(dev, sdpa):
    """Backward of the Llama-style block through the layer mirrors (RMSNorm chain, rotary attention, gated MLP): the input
    gradient against central differences of the fp64 checker's forward pass, every input element perturbed."""
    rng = np.random.default_rng(85)
    B, T, C, H = 2, 6, 16, 2
    layer = TransformerBlockLayer(dev.cuda, H, C, T, "silu", False, 1e-5, sdpa, training=True, enable_llama_style_head=True,
                                  multiple_of=8)
    hid = layer.fc1.N
    p = {"rms1_weight": 1 + 0.1 * rng.standard_normal(C), "rms2_weight": 1 + 0.1 * rng.standard_normal(C),
         "attn_weight": rng.standard_normal((3 * C, C)) * 0.3, "attn_proj_weight": rng.standard_normal((C, C)) * 0.3,
         "fc_weight": rng.standard_normal((hid, C)) * 0.3, "fc2_weight": rng.standard_normal((hid, C)) * 0.3,
         "proj_weight": rng.standard_normal((C, hid)) * 0.3}
    p = {k: v.astype(np.float32) for k, v in p.items()}
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    dy = rng.standard_normal((B, T, C)).astype(np.float32)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, p)
    layer.Forward(bx, top)
    top.mutable_cpu_diff = dy
    layer.Backward(top, bx)
    got = bx.mutable_cpu_diff.reshape(x.shape)

    def loss(xx):
        return float((R.transformer_block_llama(xx, p, H, T, 10000.0, 1e-5, np.float64) * dy).sum())

    x64, num, h = x.astype(np.float64), np.zeros(x.shape, np.float64), 1e-5
    for i in np.ndindex(*x.shape):
        xp, xm = x64.copy(), x64.copy()
        xp[i] += h
        xm[i] -= h
        num[i] = (loss(xp) - loss(xm)) / (2 * h)
    assert_close(got, num, 2e-4, "llama block dx")


def test_layernorm_layer_chain_intermediates_and_backward_golden(dev):
    """LayerNormLayer's own chain (no handle) against the reference's dump of every intermediate of a minGPT LayerNorm
    (mean, x - mean, its square, variance, standard deviation, y) and of its gradient."""
    from mycaffe_amd.layers import LayerNormLayer
    d = os.path.join(GOLDEN, "gpt-pico-ln-blk")
    x = load_txt(os.path.join(d, "x.txt"))
    layer = LayerNormLayer(dev.cuda, 1e-10, False)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Forward(bx, top)
    for blob, f, tol in (("Mu", "mean", 2e-6), ("Xmu", "xmu", 2e-6), ("XmuSq", "xmusq", 2e-6), ("Var", "var1", 2e-6), ("Stdev", "std", 2e-6)):
        assert_close(layer.b[blob].mutable_cpu_data, load_txt(os.path.join(d, f + ".txt")), tol, f)
    assert_close(top.mutable_cpu_data, load_txt(os.path.join(d, "y.txt")), 2e-6, "y")
    top.mutable_cpu_diff = load_txt(os.path.join(d, "iter_0", "grad_1a_y.txt"))
    layer.Backward(top, bx)
    assert_close(bx.mutable_cpu_diff, load_txt(os.path.join(d, "iter_0", "grad_9_x.txt")), 2e-5, "grad x")


def test_explicit_chain_with_held_back_calls_matches_the_fused_handle_at_a_large_shape(dev):
    """A score tensor of two million elements: the layer's scal / mask / softmax sequence runs through the held-back
    path (one pass), forward twice in a row (the second MatMul overwrites the tensor that is still masked on record)
    and backward; everything agrees with the checker and with the same layer on the fused attention handle."""
    from mycaffe_amd.layers import CausalSelfAttentionLayer
    rng = np.random.default_rng(91)
    B, T, C, H = 2, 512, 128, 4
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    dy = rng.standard_normal((B, T, C)).astype(np.float32)
    wa, ba = (rng.standard_normal((3 * C, C)) * 0.1).astype(np.float32), (rng.standard_normal(3 * C) * 0.1).astype(np.float32)
    wp, bp = (rng.standard_normal((C, C)) * 0.1).astype(np.float32), (rng.standard_normal(C) * 0.1).astype(np.float32)
    ref = R.causal_self_attention(x, wa, ba, wp, bp, H, dtype=np.float64)["y"]
    grads = {}
    for sdpa in (False, True):
        layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, sdpa, training=True)
        bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
        bx.mutable_cpu_data = x
        layer.Setup(bx, wa, ba, wp, bp)
        for _ in range(2):
            layer.Forward(bx, top)
            assert_close(top.mutable_cpu_data, ref, FP32_RTOL, "layer forward, sdpa=%s" % sdpa)
        top.mutable_cpu_diff = dy
        layer.Backward(top, bx)
        grads[sdpa] = bx.mutable_cpu_diff.copy()
        if not sdpa:
            # the score tensor, read after everything else: masked and scaled, as the immediate calls would have left it
            att = layer.b["AttA"].mutable_cpu_data.reshape(B, H, T, T)
            assert np.all(att[:, :, 0, 1:] == np.float32(-1e29))
    assert_close(grads[False], grads[True], 5e-5, "input gradient, explicit chain against fused handle")
