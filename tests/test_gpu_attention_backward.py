"""GPU parity of the attention handle's backward pass (id 164) through the C ABI, against the numpy checker (fp64) and
the gradient tensors the reference's test data holds for minGPT's CausalSelfAttention."""
import os

import numpy as np
import pytest

from oracle import attention_ref as R
from tests.conftest import BF16_RTOL, FP32_RTOL, GOLDEN, assert_close, bf16_round, load_txt

pytestmark = pytest.mark.gpu


def _probs(q, k, mask, batch_mask):
    """fp64 probabilities of the checker; batch_mask 2 = (B,Tq,Tk) mask broadcast over heads."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    att = (q @ np.swapaxes(k, -1, -2)) / np.sqrt(float(q.shape[-1]))
    if mask is not None:
        m = np.asarray(mask)
        if batch_mask == 2:
            m = m[:, None, :, :]
        elif batch_mask == 1:
            m = m[:, None, None, :]
        att = np.where(np.broadcast_to(m, att.shape) == 0, R.MASKED, att)
    return R.softmax_lastaxis(att, np.float64)


def _fwd_bwd(dev, q, k, v, dy, mask, batch_mask, half=False, training=True):
    B, H, T, hs = q.shape
    Tk = k.shape[2]
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    dev.cuda.SetAttn(hc, ha, 0, training, B, max(T, Tk), H, hs, 0.0)
    hq, hk, hv, hy, hdy = dev.put(q, half), dev.put(k, half), dev.put(v, half), dev.zeros(q.size, half), dev.put(dy, half)
    hdq, hdk, hdv = dev.zeros(q.size, half), dev.zeros(k.size, half), dev.zeros(k.size, half)
    hm = dev.put(mask) if mask is not None else 0
    dev.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, batch_mask, Tk if Tk != T else None)
    dev.cuda.AttnScaledDotProductBackward(hc, ha, hq, hdq, hk, hdk, hv, hdv, hm, hy, hdy)
    out = dev.get(hy, q.shape), dev.get(hdq, q.shape), dev.get(hdk, k.shape), dev.get(hdv, k.shape)
    dev.cuda.FreeAttn(ha)
    dev.cuda.FreeCuDNN(hc)
    return out


def _check(out, q, k, v, dy, mask, batch_mask, tol, what):
    p = _probs(q, k, mask, batch_mask)
    dq, dk, dv = R.attn_backward(q, k, v, p, dy, np.float64)
    assert_close(out[0], p @ np.asarray(v, np.float64), tol, what + " y")
    for got, exp, name in ((out[1], dq, "dq"), (out[2], dk, "dk"), (out[3], dv, "dv")):
        # a gradient that is exactly zero (one key: the softmax is constant) is compared on the scale of the inputs
        floor = 1e-2 * float(np.abs(dy).max())
        if float(np.abs(exp).max()) < floor:
            assert float(np.abs(got - exp).max()) <= tol * floor, what + " " + name
        else:
            assert_close(got, exp, tol, what + " " + name)


@pytest.mark.parametrize("name,heads", [("gpt-pico-csa", 1), ("gpt-pico-csa3", 3), ("gpt-pico-csa3B", 3), ("gpt-pico-csaB", 1)])
def test_attn_backward_golden(dev, name, heads):
    d = os.path.join(GOLDEN, name)
    ref = R.causal_self_attention(
        load_txt(os.path.join(d, "x.txt")), load_txt(os.path.join(d, "attn_weight.txt")), load_txt(os.path.join(d, "attn_bias.txt")),
        load_txt(os.path.join(d, "attn_proj_weight.txt")), load_txt(os.path.join(d, "attn_proj_bias.txt")), heads, dtype=np.float64)
    g = os.path.join(d, "iter_0")
    q, k, v = ref["qt"], ref["kt"], ref["vt"]
    dy = load_txt(os.path.join(g, "grad_y_pre_transpose.txt")).reshape(q.shape)
    T = q.shape[2]
    out = _fwd_bwd(dev, q, k, v, dy, R.causal_mask(T), 0)
    for got, f in ((out[1], "grad_qt.txt"), (out[2], "grad_kt.txt"), (out[3], "grad_vt.txt")):
        assert_close(got, load_txt(os.path.join(g, f)), 2e-5, name + " " + f)


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,H,T,hs", [(2, 3, 200, 64), (1, 2, 77, 48), (2, 2, 256, 128), (1, 1, 1, 64), (2, 3, 130, 32),
                                      (1, 4, 512, 64), (1, 2, 384, 128)])
def test_attn_backward_causal(dev, B, H, T, hs, half):
    rng = np.random.default_rng(T + hs)
    q, k, v, dy = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(4))
    out = _fwd_bwd(dev, q, k, v, dy, R.causal_mask(T), 0, half)
    _check(out, q, k, v, dy, R.causal_mask(T), 0, BF16_RTOL if half else FP32_RTOL, "causal")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,H,Tq,Tk,hs", [(2, 3, 64, 64, 64), (1, 2, 100, 100, 64), (2, 2, 257, 257, 64), (2, 3, 128, 256, 64),
                                          (1, 2, 200, 72, 128), (2, 2, 33, 65, 20)])
def test_attn_backward_unmasked_and_cross(dev, B, H, Tq, Tk, hs, half):
    rng = np.random.default_rng(Tq + Tk)
    q, dy = (bf16_round(rng.standard_normal((B, H, Tq, hs)).astype(np.float32)) for _ in range(2))
    k, v = (bf16_round(rng.standard_normal((B, H, Tk, hs)).astype(np.float32)) for _ in range(2))
    out = _fwd_bwd(dev, q, k, v, dy, None, 0, half)
    _check(out, q, k, v, dy, None, 0, BF16_RTOL if half else FP32_RTOL, "unmasked")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("hs", [64, 128, 40])
def test_attn_backward_masks(dev, hs, half):
    rng = np.random.default_rng(31 + hs)
    B, H, T = 3, 2, 160
    q, k, v, dy = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(4))
    tol = BF16_RTOL if half else FP32_RTOL
    # key-padding mask (B,T); the last sequence is masked everywhere: uniform weights there, in both directions
    km = np.zeros((B, T), np.float32)
    km[0, :] = 1
    km[1, :57] = 1
    out = _fwd_bwd(dev, q, k, v, dy, km, 1, half)
    _check(out, q, k, v, dy, km, 1, tol, "key mask")
    # per-sequence (B,T,T) mask: causal and padded
    bm = np.tril(np.ones((T, T), np.float32))[None] * np.stack([np.ones(T), (np.arange(T) < 90), (np.arange(T) < 33)])[:, None, :]
    out = _fwd_bwd(dev, q, k, v, dy, bm.astype(np.float32), 2, half)
    _check(out, q, k, v, dy, bm, 2, tol, "batch mask")
    # arbitrary (T,T) mask shared by all sequences
    m = (rng.random((T, T)) > 0.3).astype(np.float32)
    out = _fwd_bwd(dev, q, k, v, dy, m, 0, half)
    _check(out, q, k, v, dy, m, 0, tol, "(T,T) mask")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("causal", [True, False])
def test_attn_backward_gpt2_sequence_length(dev, causal, half):
    """T = 1024, 64-wide heads (the shape the prefill benchmark uses), fewer sequences so the fp64 checker stays small."""
    rng = np.random.default_rng(51)
    B, H, T, hs = 1, 3, 1024, 64
    q, k, v, dy = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(4))
    mask = R.causal_mask(T) if causal else None
    out = _fwd_bwd(dev, q, k, v, dy, mask, 0, half)
    _check(out, q, k, v, dy, mask, 0, BF16_RTOL if half else FP32_RTOL, "T=1024")


def test_attn_backward_without_training_forward_recomputes_row_statistics(dev):
    rng = np.random.default_rng(41)
    B, H, T, hs = 2, 2, 96, 64
    q, k, v, dy = (rng.standard_normal((B, H, T, hs)).astype(np.float32) for _ in range(4))
    out = _fwd_bwd(dev, q, k, v, dy, R.causal_mask(T), 0, False, training=False)
    _check(out, q, k, v, dy, R.causal_mask(T), 0, FP32_RTOL, "no saved statistics")


def test_attn_backward_large_scores(dev):
    rng = np.random.default_rng(42)
    B, H, T, hs = 1, 2, 128, 64
    q, k, v, dy = (rng.standard_normal((B, H, T, hs)).astype(np.float32) for _ in range(4))
    q *= 6.0   # scores in the hundreds: probabilities are nearly one-hot
    out = _fwd_bwd(dev, q, k, v, dy, R.causal_mask(T), 0)
    _check(out, q, k, v, dy, R.causal_mask(T), 0, FP32_RTOL, "large scores")


@pytest.mark.parametrize("half", [False, True])
def test_causal_launch_order_does_not_change_results(dev, half):
    """A causal launch large enough for the reordered dispatch rounds (384 workgroups: the second round of 32 per XCD is
    dealt backwards) gives, head by head, exactly what small launches of the same heads give (which keep the plain
    order), forward and backward."""
    rng = np.random.default_rng(61)
    B, H, T, hs = 4, 12, 1024, 64
    q, k, v, dy = (bf16_round(rng.standard_normal((B, H, T, hs)).astype(np.float32)) for _ in range(4))
    mask = R.causal_mask(T)
    big = _fwd_bwd(dev, q, k, v, dy, mask, 0, half)
    for b, h0 in ((0, 0), (3, 9), (2, 5)):
        sl = (slice(b, b + 1), slice(h0, h0 + 3))
        small = _fwd_bwd(dev, q[sl], k[sl], v[sl], dy[sl], mask, 0, half)
        for got, exp, name in zip(big, small, ("y", "dq", "dk", "dv")):
            assert np.array_equal(got[sl], exp), name
