"""GPU parity of the fused attention paths through the C ABI: the attention handle
(ids 160-163), the layer mirrors on the reference's golden tensors, and the
single-call KV-cache decode attention."""
import os

import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnnError, ERROR
from mycaffe_amd.layers import Blob, CausalSelfAttentionLayer, MultiheadAttentionLayer
from oracle import attention_ref as R
from tests.conftest import BF16_RTOL, FP32_RTOL, GOLDEN, assert_close, bf16_round, load_txt

pytestmark = pytest.mark.gpu


def _attn(dev, q, k, v, mask, batch_mask, half=False, block=None):
    B, H, T, hs = q.shape
    Tk = k.shape[2]
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    dev.cuda.SetAttn(hc, ha, 0, False, B, block or max(T, Tk), H, hs, 0.0)
    hq, hk, hv, hy = dev.put(q, half), dev.put(k, half), dev.put(v, half), dev.zeros(q.size, half)
    hm = dev.put(mask) if mask is not None else 0
    dev.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, batch_mask, Tk if Tk != T else None)
    out = dev.get(hy, q.shape)
    dev.cuda.FreeAttn(ha)
    dev.cuda.FreeCuDNN(hc)
    return out


@pytest.mark.parametrize("B,H,T,hs", [(3, 8, 200, 64), (2, 4, 128, 64), (1, 2, 77, 48), (2, 2, 256, 128), (1, 1, 1, 64), (2, 3, 130, 32), (1, 4, 777, 64), (2, 2, 1000, 64),
                                      (12, 32, 160, 64)])
def test_attn_forward_causal_fp32(dev, B, H, T, hs):
    # the shape (3,8,200,64) is the one TestCudaAttentionForward uses (TestGPT_MultiheadAttentionLayer.cs:945-1036)
    rng = np.random.default_rng(T)
    q, k, v = (rng.standard_normal((B, H, T, hs)).astype(np.float32) for _ in range(3))
    out = _attn(dev, q, k, v, R.causal_mask(T), False)
    ref, _ = R.attn_forward(q, k, v, R.causal_mask(T, np.float64), False, np.float64)
    assert_close(out, ref, FP32_RTOL, "attn causal fp32")
    if T == 1:
        assert_close(out, v, 1e-6, "T=1 returns V")


@pytest.mark.parametrize("B,H,T,hs", [(3, 8, 200, 64), (2, 4, 256, 64), (2, 2, 256, 128), (2, 3, 777, 128), (1, 2, 1024, 128),
                                      (1, 2, 33, 128), (1, 1, 300, 128)])
def test_attn_forward_causal_bf16(dev, B, H, T, hs):
    # head size 128 takes the software-pipelined kernel: 256-row workgroups, so T = 777 has full, diagonal, ragged and
    # idle wavefronts, T = 33 never reaches a steady-state phase
    rng = np.random.default_rng(T + 1)
    q, k, v = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(3))
    out = _attn(dev, q, k, v, R.causal_mask(T), False, half=True)
    ref, _ = R.attn_forward(q, k, v, R.causal_mask(T, np.float64), False, np.float64)
    assert_close(out, ref, BF16_RTOL, "attn causal bf16")


@pytest.mark.parametrize("half", [False, True])
def test_attn_forward_key_padding_mask_and_fully_masked_rows(dev, half):
    rng = np.random.default_rng(11)
    B, H, T, hs = 4, 8, 256, 64
    q, k, v = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(3))
    lens = [256, 32, 100, 0]          # the last sequence is masked everywhere: uniform weights, not NaN
    km = np.zeros((B, T), np.float32)
    for b, n in enumerate(lens):
        km[b, :n] = 1
    out = _attn(dev, q, k, v, km, True, half)
    ref, _ = R.attn_forward(q, k, v, km, True, np.float64)
    assert_close(out, ref, BF16_RTOL if half else FP32_RTOL, "attn key mask")
    assert_close(out[3], np.broadcast_to(v[3].mean(axis=1, keepdims=True), v[3].shape), BF16_RTOL if half else FP32_RTOL, "uniform row")


def test_attn_forward_arbitrary_qk_mask_and_no_mask(dev):
    rng = np.random.default_rng(12)
    B, H, T, hs = 2, 3, 96, 64
    q, k, v = (rng.standard_normal((B, H, T, hs)).astype(np.float32) for _ in range(3))
    m = (rng.random((T, T)) > 0.3).astype(np.float32)
    out = _attn(dev, q, k, v, m, False)
    ref, _ = R.attn_forward(q, k, v, m, False, np.float64)
    assert_close(out, ref, FP32_RTOL, "attn (T,T) mask")
    out = _attn(dev, q, k, v, None, False)
    ref, _ = R.attn_forward(q, k, v, None, False, np.float64)
    assert_close(out, ref, FP32_RTOL, "attn no mask")


@pytest.mark.parametrize("half", [True, False])
@pytest.mark.parametrize("B,H,Tq,Tk,hs", [(2, 3, 64, 64, 64), (1, 2, 100, 100, 64), (2, 2, 257, 257, 64), (1, 4, 1024, 1024, 64),
                                          (2, 2, 128, 320, 64), (1, 2, 33, 500, 64), (1, 2, 192, 192, 128), (2, 2, 700, 700, 128),
                                          (1, 3, 130, 777, 128), (1, 2, 520, 95, 128)])
def test_attn_forward_unmasked(dev, half, B, H, Tq, Tk, hs):
    # no mask: bf16 / head size 64 takes the software-pipelined kernel (steady-state phases need > 3 key steps,
    # ragged lengths end in its sequential phases); T_q != T_k is cross attention
    rng = np.random.default_rng(Tq + Tk)
    q = bf16_round(rng.standard_normal((B, H, Tq, hs)).astype(np.float32))
    k, v = (bf16_round(rng.standard_normal((B, H, Tk, hs)).astype(np.float32)) for _ in range(2))
    out = _attn(dev, q, k, v, None, False, half)
    ref, _ = R.attn_forward(q, k, v, None, False, np.float64)
    assert_close(out, ref, BF16_RTOL if half else FP32_RTOL, "attn unmasked")


def test_attn_forward_large_scores_rescale_in_the_pipelined_head_size_128_kernel(dev):
    # as below for bf16, head size 128: a key far above the running maximum late in the range forces the rescale of the
    # output accumulators inside a steady-state phase of the pipelined kernel
    rng = np.random.default_rng(6)
    B, H, T, hs = 1, 2, 640, 128
    q = bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32))
    k = bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32))
    v = bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32))
    k[:, :, 401] = bf16_round(6.0 * q[:, :, 500])      # a large score for the rows near 500 (and a wide spread elsewhere)
    k[:, :, 130] = bf16_round(-5.0 * q[:, :, 200])
    for mask in (None, R.causal_mask(T)):
        out = _attn(dev, q, k, v, mask, False, True)
        ref, _ = R.attn_forward(q, k, v, None if mask is None else R.causal_mask(T, np.float64), False, np.float64)
        assert_close(out, ref, BF16_RTOL, "attn hs128 with score jumps")


def test_attn_forward_large_scores_lazy_rescale(dev):
    # a score that jumps far above the running maximum late in the key range forces the rescale of the output
    # accumulators; scores within the slack must not
    rng = np.random.default_rng(5)
    B, H, T, hs = 1, 2, 512, 64
    q = rng.standard_normal((B, H, T, hs)).astype(np.float32)
    k = rng.standard_normal((B, H, T, hs)).astype(np.float32)
    v = rng.standard_normal((B, H, T, hs)).astype(np.float32)
    k[:, :, 300] = 6.0 * q[:, :, 17]          # huge score for query 17 (and large ones for similar queries) at key 300
    k[:, :, 40] = 0.6 * q[:, :, 99]
    for half in (False, True):
        qq, kk, vv = (bf16_round(x) for x in (q, k, v))
        out = _attn(dev, qq, kk, vv, None, False, half)
        ref, _ = R.attn_forward(qq, kk, vv, None, False, np.float64)
        assert_close(out, ref, BF16_RTOL if half else FP32_RTOL, "attn with late large scores")
        out = _attn(dev, qq, kk, vv, R.causal_mask(T), False, half)
        ref, _ = R.attn_forward(qq, kk, vv, R.causal_mask(T, np.float64), False, np.float64)
        assert_close(out, ref, BF16_RTOL if half else FP32_RTOL, "causal attn with late large scores")


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("B,H,T,hs", [(1, 2, 512, 64), (2, 2, 513, 64), (1, 3, 777, 64), (1, 2, 1000, 128), (2, 1, 1024, 64), (1, 1, 1100, 128),
                                      (1, 2, 1536, 64), (1, 1, 2000, 128), (1, 2, 575, 128), (1, 1, 640, 64)])
def test_attn_forward_two_tiles_per_wavefront_kernel(dev, causal, B, H, T, hs):
    # bf16 with 512 keys or more, no mask or the causal one, takes the kernel with two 32-row tiles per wavefront and
    # 256-row workgroups: the lengths give workgroups with idle tiles (513, 575), a last block of 1 .. 63 keys (513, 777,
    # 1000, 1100, 2000: the pinned phases stop four blocks before it), whole blocks only (512, 1024, 1536) and an odd
    # number of 32-key steps (1000 -> 32 steps, 1100 -> 35)
    rng = np.random.default_rng(T + hs + causal)
    q, k, v = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(3))
    out = _attn(dev, q, k, v, R.causal_mask(T) if causal else None, False, half=True)
    ref, _ = R.attn_forward(q, k, v, R.causal_mask(T, np.float64) if causal else None, False, np.float64)
    assert_close(out, ref, BF16_RTOL, "attn bf16, two tiles per wavefront")


@pytest.mark.parametrize("hs", [64, 128])
@pytest.mark.parametrize("scale", [1.5, 2.0, 3.0, 6.0])
def test_attn_forward_two_tiles_per_wavefront_kernel_hands_large_scores_to_its_plain_pass(dev, hs, scale):
    # That kernel takes exp2 of the scaled scores with the reference 0 and accepts a row whose sum of weights ends inside
    # [2^-18, 2^18]; a workgroup with a row outside computes its rows again with running maxima.  Inputs scaled by 1.5 stay
    # inside (scaled scores up to about 15), by 2 and more leave it (up to 25 .. 200 and far beyond what exp2 can hold).
    rng = np.random.default_rng(int(10 * scale) + hs)
    B, H, T = 1, 2, 640
    q, k, v = (bf16_round(scale * rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(3))
    for causal in (True, False):
        out = _attn(dev, q, k, v, R.causal_mask(T) if causal else None, False, half=True)
        ref, _ = R.attn_forward(q, k, v, R.causal_mask(T, np.float64) if causal else None, False, np.float64)
        assert np.isfinite(out).all()
        assert_close(out, ref, BF16_RTOL, "attn bf16, large scores")
    # one row far below the range, the others ordinary: every key of query 100 scores about -60
    q2, k2, v2 = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(3))
    k2[..., 0] = 8.0
    q2[:, :, 100, 0] = -60.0 * np.sqrt(hs) / 8.0 / 1.4426950408889634
    q2, k2 = bf16_round(q2), bf16_round(k2)
    out = _attn(dev, q2, k2, v2, None, False, half=True)
    ref, _ = R.attn_forward(q2, k2, v2, None, False, np.float64)
    assert_close(out, ref, BF16_RTOL, "attn bf16, one row of tiny weights")


def test_attn_mask_content_change_is_seen(dev):
    # a causal mask that is later overwritten through the ABI must stop being treated as causal
    rng = np.random.default_rng(13)
    B, H, T, hs = 1, 2, 64, 64
    q, k, v = (rng.standard_normal((B, H, T, hs)).astype(np.float32) for _ in range(3))
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    dev.cuda.SetAttn(hc, ha, 0, False, B, T, H, hs, 0.0)
    hq, hk, hv, hy = dev.put(q), dev.put(k), dev.put(v), dev.zeros(q.size)
    hm = dev.put(R.causal_mask(T))
    dev.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, False)
    assert_close(dev.get(hy), R.attn_forward(q, k, v, R.causal_mask(T), False, np.float64)[0], FP32_RTOL, "causal")
    full = np.ones((T, T), np.float32)
    dev.cuda.SetMemory(hm, full)
    dev.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, False)
    assert_close(dev.get(hy), R.attn_forward(q, k, v, full, False, np.float64)[0], FP32_RTOL, "after overwrite")


def test_attn_cross_attention_lengths_differ(dev):
    rng = np.random.default_rng(14)
    B, H, Tq, Tk, hs = 2, 8, 128, 256, 64
    q = rng.standard_normal((B, H, Tq, hs)).astype(np.float32)
    k, v = (rng.standard_normal((B, H, Tk, hs)).astype(np.float32) for _ in range(2))
    km = np.ones((B, Tk), np.float32)
    km[0, 40:] = 0
    km[1, 200:] = 0
    out = _attn(dev, q, k, v, km, True)
    s = np.einsum("bhqd,bhkd->bhqk", q.astype(np.float64), k) / 8.0
    s = np.where(km[:, None, None, :] == 0, -1e29, s)
    ref = R.softmax_lastaxis(s, np.float64) @ v
    assert_close(out, ref, FP32_RTOL, "cross attention")


def test_attn_error_codes(dev):
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    h = dev.zeros(2 * 2 * 16 * 8)
    with pytest.raises(CudaDnnError) as e:   # forward before Set
        dev.cuda.AttnScaledDotProductForward(hc, ha, 16, h, h, h, 0, h, False)
    assert e.value.code == ERROR.ATTN_NOT_INITIALIZED
    dev.cuda.SetAttn(hc, ha, 0, False, 2, 16, 2, 8, 0.0)
    with pytest.raises(CudaDnnError) as e:   # attn.cu:531-532
        dev.cuda.AttnScaledDotProductForward(hc, ha, 32, h, h, h, 0, h, False)
    assert e.value.code == ERROR.ATTN_INVALID_BLOCK_SIZE
    small = dev.zeros(10)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.AttnScaledDotProductForward(hc, ha, 16, small, h, h, 0, h, False)
    assert e.value.code == ERROR.ATTN_INCOMPATIBLE_BLOB_SIZE


# ---- layer mirrors on the reference's golden tensors ---------------------------------

@pytest.mark.parametrize("name,heads", [("gpt-pico-csa", 1), ("gpt-pico-csa3", 3), ("gpt-pico-csa3B", 3), ("gpt-pico-csaB", 1)])
@pytest.mark.parametrize("sdpa", [True, False])
def test_causal_self_attention_layer_golden(dev, name, heads, sdpa):
    d = os.path.join(GOLDEN, name)
    x = load_txt(os.path.join(d, "x.txt"))
    B, T, C = x.shape
    layer = CausalSelfAttentionLayer(dev.cuda, heads, C, T, True, enable_cuda_scaled_dot_product_attention=sdpa)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, load_txt(os.path.join(d, "attn_weight.txt")), load_txt(os.path.join(d, "attn_bias.txt")),
                load_txt(os.path.join(d, "attn_proj_weight.txt")), load_txt(os.path.join(d, "attn_proj_bias.txt")))
    layer.Forward(bx, top)
    y = load_txt(os.path.join(d, "y.txt")).reshape(B, T, C)
    assert_close(top.mutable_cpu_data, y, FP32_RTOL, name + " y")
    qt = load_txt(os.path.join(d, "qt.txt"))
    assert_close(layer.b["Qt"].mutable_cpu_data, qt.reshape(layer.b["Qt"].shape_), FP32_RTOL, name + " qt")
    if os.path.exists(os.path.join(d, "var_y.npy")):
        assert_close(layer.b["Work"].mutable_cpu_data, np.load(os.path.join(d, "var_y.npy")), FP32_RTOL, name + " att@v")
        if not sdpa:
            att = np.load(os.path.join(d, "var_att.npy"))
            got = layer.b["AttB"].mutable_cpu_data
            assert_close(got, att, FP32_RTOL, name + " softmax")
            assert np.all(np.triu(got, 1) == 0)


@pytest.mark.parametrize("sdpa", [True, False])
@pytest.mark.parametrize("rope", [False, True])
def test_causal_self_attention_layer_random(dev, sdpa, rope):
    rng = np.random.default_rng(21)
    B, T, C, H = 2, 64, 192, 6      # the 6-head / 192-embed layer of TestGPT_CausalSelfAttentionLayer.cs:179-271
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    wa, ba = (rng.standard_normal((3 * C, C)) * 0.02).astype(np.float32), (rng.standard_normal(3 * C) * 0.02).astype(np.float32)
    wp, bp = (rng.standard_normal((C, C)) * 0.02).astype(np.float32), (rng.standard_normal(C) * 0.02).astype(np.float32)
    layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, sdpa, enable_rotary_positional_embedding=rope)
    bx, top = Blob(dev.cuda, x.shape), Blob(dev.cuda)
    bx.mutable_cpu_data = x
    layer.Setup(bx, wa, ba, wp, bp)
    layer.Forward(bx, top)
    ref = R.causal_self_attention(x, wa, ba, wp, bp, H, rope=(T, 10000.0) if rope else None, dtype=np.float64)
    assert_close(top.mutable_cpu_data, ref["y"], FP32_RTOL, "csa random")


def test_causal_self_attention_layer_bf16(dev):
    rng = np.random.default_rng(22)
    B, T, C, H = 2, 128, 256, 4
    x = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    wa = bf16_round((rng.standard_normal((3 * C, C)) * 0.02).astype(np.float32))
    wp = bf16_round((rng.standard_normal((C, C)) * 0.02).astype(np.float32))
    layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, False, True, half=True)
    bx, top = Blob(dev.cuda, x.shape, half=True), Blob(dev.cuda, half=True)
    bx.mutable_cpu_data = x
    layer.Setup(bx, wa, None, wp, None)
    layer.Forward(bx, top)
    ref = R.causal_self_attention(x, wa, None, wp, None, H, dtype=np.float64)
    assert_close(top.mutable_cpu_data, ref["y"], BF16_RTOL, "csa bf16")


@pytest.mark.parametrize("rope", [False, True])
def test_multihead_attention_cached_decode_branch_of_the_layer(dev, rope):
    """The reference layer's own cached decode (MultiheadAttentionLayer.cs:713-730, 759-777: one token per call with the
    "position" option, a copy / MatMul / channel_copy / add loop over the cached positions) through the unchanged call
    sequence: the output for token p equals row p of the causal forward over the whole sequence."""
    rng = np.random.default_rng(29)
    B, T, C, H = 1, 10, 96, 3
    W = {k: (rng.standard_normal((C, C)) * 0.2).astype(np.float32) for k in ("wq", "wk", "wv", "wo")}
    W.update({k: (rng.standard_normal(C) * 0.1).astype(np.float32) for k in ("bq", "bk", "bv", "bo")})
    x = rng.standard_normal((B, T, C)).astype(np.float32)
    ref = R.multihead_attention(x, x, x, W["wq"], W["bq"], W["wk"], W["bk"], W["wv"], W["bv"], W["wo"], W["bo"], H,
                                R.causal_mask(T), "causal", rope=(T, 10000.0) if rope else None, dtype=np.float64)["y"]
    layer = MultiheadAttentionLayer(dev.cuda, H, C, T, True, False, enable_rotary_positional_embedding=rope,
                                    enable_key_value_cache=True)
    tok, top = Blob(dev.cuda, (B, 1, C)), Blob(dev.cuda)
    tok.mutable_cpu_data = x[:, :1]
    layer.Setup(tok, tok, tok, W)
    for p in range(T):
        tok.mutable_cpu_data = x[:, p:p + 1]
        layer.SetLayerOption("position", p)
        layer.Forward(tok, tok, tok, None, top)
        assert_close(top.mutable_cpu_data.reshape(B, C), ref[:, p], FP32_RTOL, "cached decode, position %d" % p)


@pytest.mark.parametrize("sdpa", [True, False])
def test_multihead_attention_encoder_decoder_masks(dev, sdpa):
    # scaled-down encoder / decoder / cross attention with padding masks (valid lengths per sequence)
    rng = np.random.default_rng(23)
    B, Ts, Tt, C, H = 4, 64, 32, 128, 8
    W = {k: (rng.standard_normal((C, C)) * 0.05).astype(np.float32) for k in ("wq", "wk", "wv", "wo")}
    W.update({k: (rng.standard_normal(C) * 0.05).astype(np.float32) for k in ("bq", "bk", "bv", "bo")})
    src = rng.standard_normal((B, Ts, C)).astype(np.float32)
    tgt = rng.standard_normal((B, Tt, C)).astype(np.float32)
    slen, tlen = rng.integers(8, Ts + 1, B), rng.integers(4, Tt + 1, B)
    enc_mask = (np.arange(Ts)[None, :] < slen[:, None]).astype(np.float32)                       # (B,Ts) key padding
    dec_mask = ((np.arange(Tt)[None, :] < tlen[:, None])[:, None, :] * np.tril(np.ones((Tt, Tt)))[None]).astype(np.float32)
    bs, bt, top = Blob(dev.cuda, src.shape), Blob(dev.cuda, tgt.shape), Blob(dev.cuda)
    bs.mutable_cpu_data, bt.mutable_cpu_data = src, tgt
    # encoder self attention, key-padding mask through mask_batch / batch-mask handle
    enc = MultiheadAttentionLayer(dev.cuda, H, C, Ts, True, sdpa)
    enc.Setup(bs, bs, bs, W)
    bm = Blob(dev.cuda, (B, Ts, 1, 1))
    bm.mutable_cpu_data = enc_mask
    enc.Forward(bs, bs, bs, bm, top)
    ref = R.multihead_attention(src, src, src, W["wq"], W["bq"], W["wk"], W["bk"], W["wv"], W["bv"], W["wo"], W["bo"], H,
                                enc_mask, "key", dtype=np.float64)
    assert_close(top.mutable_cpu_data, ref["y"], FP32_RTOL, "encoder self attention")
    # decoder self attention, (B,T,T) causal-and-padding mask
    dec = MultiheadAttentionLayer(dev.cuda, H, C, Tt, True, sdpa)
    dec.Setup(bt, bt, bt, W)
    bdm = Blob(dev.cuda, (B, Tt, Tt, 1))
    bdm.mutable_cpu_data = dec_mask
    dec.Forward(bt, bt, bt, bdm, top)
    ref = R.multihead_attention(tgt, tgt, tgt, W["wq"], W["bq"], W["wk"], W["bk"], W["wv"], W["bv"], W["wo"], W["bo"], H,
                                dec_mask, "full", dtype=np.float64)
    assert_close(top.mutable_cpu_data, ref["y"], FP32_RTOL, "decoder self attention")
    if sdpa:
        # the same (B,T,T) mask kept on the fused handle (batch-mask code 2)
        dec2 = MultiheadAttentionLayer(dev.cuda, H, C, Tt, True, True, fuse_batch_qk_mask=True)
        dec2.Setup(bt, bt, bt, W)
        dec2.Forward(bt, bt, bt, bdm, top)
        assert_close(top.mutable_cpu_data, ref["y"], FP32_RTOL, "decoder self attention, fused per-sequence mask")
    # cross attention: queries from the target, keys / values from the source, source key padding
    if sdpa:
        cross = MultiheadAttentionLayer(dev.cuda, H, C, Ts, True, True)
        cross.Setup(bt, bs, bs, W)
        cross.Forward(bt, bs, bs, bm, top)
        ref = R.multihead_attention(tgt, src, src, W["wq"], W["bq"], W["wk"], W["bk"], W["wv"], W["bv"], W["wo"], W["bo"], H,
                                    enc_mask, "key", dtype=np.float64)
        assert_close(top.mutable_cpu_data, ref["y"], FP32_RTOL, "cross attention")


# ---- KV-cache decode attention -----------------------------------------------------------

@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,H,L,hs", [(1, 32, 512, 128), (8, 32, 2048, 128), (2, 6, 200, 48), (3, 12, 777, 64), (1, 4, 1, 64), (2, 2, 33, 20)])
def test_attn_decode_vs_checker(dev, half, B, H, L, hs):
    rng = np.random.default_rng(L)
    q = bf16_round(rng.standard_normal((B, H, hs)).astype(np.float32))
    k, v = (bf16_round(rng.standard_normal((B, H, L, hs)).astype(np.float32)) for _ in range(2))
    hq, hk, hv, hy = dev.put(q, half), dev.put(k, half), dev.put(v, half), dev.zeros(q.size, half)
    dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq, hk, hv, hy, H * L * hs, L * hs, hs)
    ref = R.kv_cache_attention(q, k, v, np.float64)
    assert_close(dev.get(hy, q.shape), ref, BF16_RTOL if half else FP32_RTOL, "decode attention")


def test_attn_decode_position_major_cache_and_gqa(dev):
    # cache laid out (L, kvHeads*hs) per sequence, as the llama2 engine keeps it, 4 query heads per kv head
    rng = np.random.default_rng(31)
    B, H, KVH, L, hs, S = 2, 8, 2, 150, 64, 256
    q = rng.standard_normal((B, H, hs)).astype(np.float32)
    kc = rng.standard_normal((B, S, KVH, hs)).astype(np.float32)
    vc = rng.standard_normal((B, S, KVH, hs)).astype(np.float32)
    hq, hk, hv, hy = dev.put(q), dev.put(kc), dev.put(vc), dev.zeros(q.size)
    dev.cuda.AttnDecodeForward(B, H, KVH, hs, L, hq, hk, hv, hy, S * KVH * hs, hs, KVH * hs)
    kk = np.repeat(kc[:, :L].transpose(0, 2, 1, 3), H // KVH, axis=1)
    vv = np.repeat(vc[:, :L].transpose(0, 2, 1, 3), H // KVH, axis=1)
    assert_close(dev.get(hy, q.shape), R.kv_cache_attention(q, kk, vv, np.float64), FP32_RTOL, "decode gqa")


def test_attn_decode_with_rope_and_append(dev):
    # RoPE (theta 10000) applied to q and the newest key at position L-1, key / value appended, then attention
    rng = np.random.default_rng(32)
    B, H, L, hs, S = 2, 4, 40, 64, 64
    q = rng.standard_normal((B, H, hs)).astype(np.float32)
    kn, vn = (rng.standard_normal((B, H, hs)).astype(np.float32) for _ in range(2))
    kc = rng.standard_normal((B, H, S, hs)).astype(np.float32)
    vc = rng.standard_normal((B, H, S, hs)).astype(np.float32)
    hr = dev.cuda.CreateRope(0, 0, B * H * hs, B, S, H, hs, 10000.0)
    hq, hkn, hvn, hk, hv, hy = dev.put(q), dev.put(kn), dev.put(vn), dev.put(kc), dev.put(vc), dev.zeros(q.size)
    dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq, hk, hv, hy, H * S * hs, S * hs, hs, 0.0, hr, hkn, hvn)
    cos, sin = R.rope_tables(S, hs)

    def rot(x):
        o = x.copy()
        o[..., 0::2] = x[..., 0::2] * cos[L - 1] - x[..., 1::2] * sin[L - 1]
        o[..., 1::2] = x[..., 0::2] * sin[L - 1] + x[..., 1::2] * cos[L - 1]
        return o

    kc2, vc2 = kc.copy(), vc.copy()
    kc2[:, :, L - 1], vc2[:, :, L - 1] = rot(kn), vn
    ref = R.kv_cache_attention(rot(q), kc2[:, :, :L], vc2[:, :, :L], np.float64)
    assert_close(dev.get(hy, q.shape), ref, FP32_RTOL, "decode with rope")
    assert_close(dev.get(hk, kc.shape), kc2, 1e-6, "key cache after append")
    assert np.array_equal(dev.get(hv, vc.shape), vc2)


# ---- fused QKV projection (id 2004) and head-merged attention output -----------------------

@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,T,H,hs,bias", [(2, 128, 4, 64, True), (3, 100, 3, 64, True), (1, 257, 2, 128, False), (2, 40, 3, 16, True),
                                           (2, 64, 5, 24, True)])
def test_qkv_proj_heads_against_the_call_sequence_it_replaces(dev, half, B, T, H, hs, bias):
    """One call against InnerProduct + bias GEMM + three channel copies + three head transposes
    (CausalSelfAttentionLayer.cs:526-557): bit for bit in fp32, within the 16-bit bar otherwise, and against the checker."""
    C = H * hs
    rng = np.random.default_rng(B * 1000 + T)
    x = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    w = bf16_round((rng.standard_normal((3 * C, C)) * 0.05).astype(np.float32))
    bv = bf16_round((rng.standard_normal(3 * C) * 0.1).astype(np.float32)) if bias else None
    hx, hw = dev.put(x, half), dev.put(w, half)
    hb = dev.put(bv, half) if bias else 0
    hq, hk, hv = (dev.zeros(B * T * C, half) for _ in range(3))
    dev.cuda.QkvProjHeads(B, T, H, hs, hx, hw, hb, hq, hk, hv)
    got = [dev.get(h, (B, H, T, hs)) for h in (hq, hk, hv)]
    # the sequence it replaces, through the layer mirror's own pieces
    layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, bias, True, half=half)
    bottom, top = Blob(dev.cuda, x.shape, half=half), Blob(dev.cuda, half=half)
    bottom.mutable_cpu_data = x
    layer.Setup(bottom, w, bv if bias else None, np.eye(C, dtype=np.float32), np.zeros(C, np.float32) if bias else None)
    layer.Forward(bottom, top)
    seq = [layer.b[n].mutable_cpu_data.reshape(B, H, T, hs) for n in ("Qt", "Kt", "Vt")]
    ref = R.inner_product(x, w, bv, np.float64).reshape(B, T, 3, H, hs).transpose(2, 0, 3, 1, 4)
    for i, name in enumerate("qkv"):
        assert_close(got[i], ref[i], BF16_RTOL if half else FP32_RTOL, name + " vs checker")
        if not half:
            assert np.array_equal(got[i], seq[i]), name + " differs from the call sequence"
        else:
            assert_close(got[i], seq[i], BF16_RTOL, name + " vs the call sequence")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,T,H,hs", [(2, 128, 4, 64), (3, 100, 3, 64), (1, 257, 2, 128), (2, 40, 3, 16), (2, 64, 5, 24)])
def test_qkv_proj_heads_with_the_rotary_embedding(dev, half, B, T, H, hs):
    """The eleventh argument: q and k leave the projection rotated, as the two RopeForward calls between the channel
    copies and the head transposes leave them (CausalSelfAttentionLayer.cs:538-545).  Against the layer's own call
    sequence (the same products, roundings and tables; the rotation's multiply-adds may contract differently, hence a
    few ulps and not bit for bit) and against the checker; v must not be touched."""
    C = H * hs
    rng = np.random.default_rng(B * 1000 + T + 7)
    x = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    w = bf16_round((rng.standard_normal((3 * C, C)) * 0.05).astype(np.float32))
    bv = bf16_round((rng.standard_normal(3 * C) * 0.1).astype(np.float32))
    layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, True, enable_rotary_positional_embedding=True, half=half)
    bottom, top = Blob(dev.cuda, x.shape, half=half), Blob(dev.cuda, half=half)
    bottom.mutable_cpu_data = x
    layer.Setup(bottom, w, bv, np.eye(C, dtype=np.float32), np.zeros(C, np.float32))
    layer.Forward(bottom, top)
    seq = [layer.b[n].mutable_cpu_data.reshape(B, H, T, hs) for n in ("Qt", "Kt", "Vt")]
    hx, hw, hb = dev.put(x, half), dev.put(w, half), dev.put(bv, half)
    hq, hk, hv = (dev.zeros(B * T * C, half) for _ in range(3))
    dev.cuda.QkvProjHeads(B, T, H, hs, hx, hw, hb, hq, hk, hv, layer.hRope)
    got = [dev.get(h, (B, H, T, hs)) for h in (hq, hk, hv)]
    qkv = R.inner_product(x, w, bv, np.float64).reshape(B, T, 3, H, hs)
    ref = [R.rope_forward(qkv[:, :, i], T, H, hs, dtype=np.float64).reshape(B, T, H, hs) if i < 2 else qkv[:, :, i] for i in range(3)]
    for i, name in enumerate("qkv"):
        assert_close(got[i], ref[i].transpose(0, 2, 1, 3), BF16_RTOL if half else FP32_RTOL, name + " vs checker")
        assert_close(got[i], seq[i], BF16_RTOL if half else 1e-6, name + " vs the call sequence")
    assert np.array_equal(got[2], seq[2]) or half
    # the handle has to fit the projection
    other = dev.cuda.CreateRope(0, 0, B * T * C, B, T, H + 1, hs, 10000.0)
    with pytest.raises(Exception):
        dev.cuda.QkvProjHeads(B, T, H, hs, hx, hw, hb, hq, hk, hv, other)
    dev.cuda.FreeRope(other)


@pytest.mark.parametrize("half", [False, True])
def test_causal_self_attention_layer_with_rotary_embedding_as_three_calls(dev, half):
    B, T, C, H = 2, 128, 256, 4
    rng = np.random.default_rng(T + 1)
    x = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    wa = bf16_round((rng.standard_normal((3 * C, C)) * 0.05).astype(np.float32))
    wp = bf16_round((rng.standard_normal((C, C)) * 0.05).astype(np.float32))
    ba = bf16_round((rng.standard_normal(3 * C) * 0.1).astype(np.float32))
    bp = bf16_round((rng.standard_normal(C) * 0.1).astype(np.float32))
    outs = []
    for fused in (False, True):
        layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, True, enable_rotary_positional_embedding=True, half=half,
                                         fused_qkv_heads=fused)
        bottom, top = Blob(dev.cuda, x.shape, half=half), Blob(dev.cuda, half=half)
        bottom.mutable_cpu_data = x
        layer.Setup(bottom, wa, ba, wp, bp)
        layer.Forward(bottom, top)
        outs.append(top.mutable_cpu_data.copy())
    ref = R.causal_self_attention(x, wa, ba, wp, bp, H, rope=(T, 10000.0), dtype=np.float64)["y"]
    assert_close(outs[1], ref, BF16_RTOL if half else FP32_RTOL, "three-call layer vs checker")
    assert_close(outs[1], outs[0], BF16_RTOL if half else 1e-5, "three-call layer vs the nineteen-call sequence")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,T,C,H", [(2, 128, 256, 4), (1, 200, 192, 3), (2, 96, 256, 2), (2, 50, 48, 3)])
def test_causal_self_attention_layer_as_three_calls(dev, half, B, T, C, H):
    rng = np.random.default_rng(T)
    x = bf16_round(rng.standard_normal((B, T, C)).astype(np.float32))
    wa = bf16_round((rng.standard_normal((3 * C, C)) * 0.05).astype(np.float32))
    wp = bf16_round((rng.standard_normal((C, C)) * 0.05).astype(np.float32))
    ba = bf16_round((rng.standard_normal(3 * C) * 0.1).astype(np.float32))
    bp = bf16_round((rng.standard_normal(C) * 0.1).astype(np.float32))
    outs = []
    for fused in (False, True):
        layer = CausalSelfAttentionLayer(dev.cuda, H, C, T, True, True, half=half, fused_qkv_heads=fused)
        bottom, top = Blob(dev.cuda, x.shape, half=half), Blob(dev.cuda, half=half)
        bottom.mutable_cpu_data = x
        layer.Setup(bottom, wa, ba, wp, bp)
        layer.Forward(bottom, top)
        outs.append(top.mutable_cpu_data.copy())
    ref = R.causal_self_attention(x, wa, ba, wp, bp, H, dtype=np.float64)["y"]
    assert_close(outs[1], ref, BF16_RTOL if half else FP32_RTOL, "three-call layer vs checker")
    if not half:
        assert np.array_equal(outs[0], outs[1]), "three-call layer differs from the seventeen-call sequence"
