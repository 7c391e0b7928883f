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


# ---- attention dropout: training mode of the handle with a ratio (attn.cu:455-486, 578-583, 637-640) ---------------

def _dropout_case(dev, B, H, Tq, Tk, hs, ratio, seed, mask, batch_mask, half, calls=1):
    rng = np.random.default_rng(seed)
    rnd = bf16_round if half else (lambda a: a)
    q, dy = (rnd(rng.standard_normal((B, H, Tq, hs)).astype(np.float32)) for _ in range(2))
    k, v = (rnd(rng.standard_normal((B, H, Tk, hs)).astype(np.float32)) for _ in range(2))
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    dev.cuda.SetAttn(hc, ha, 0, True, B, max(Tq, Tk), H, hs, ratio, seed)
    hq, hk, hv, hy, hdy = dev.put(q, half), dev.put(k, half), dev.put(v, half), dev.zeros(q.size, half), dev.put(dy, half)
    hdq, hdk, hdv = dev.zeros(q.size, half), dev.zeros(k.size, half), dev.zeros(k.size, half)
    hm = dev.put(mask) if mask is not None else 0
    ys = []
    for _ in range(calls):
        dev.cuda.AttnScaledDotProductForward(hc, ha, Tq, hq, hk, hv, hm, hy, batch_mask, Tk if Tk != Tq else None)
        ys.append(dev.get(hy, q.shape))
    dev.cuda.AttnScaledDotProductBackward(hc, ha, hq, hdq, hk, hdk, hv, hdv, hm, hy, hdy)
    got = ys, dev.get(hdq, q.shape), dev.get(hdk, k.shape), dev.get(hdv, k.shape)
    dev.cuda.FreeAttn(ha)
    dev.cuda.FreeCuDNN(hc)
    # checker: probabilities in fp64, the library's mask generator, the reference's step sequence
    p = _probs(q, k, mask, batch_mask)
    exp_y, keep = [], None
    for c in range(1, calls + 1):
        keep = R.attn_dropout_keep(seed, B, H, Tq, Tk, ratio, forward_calls=c)
        pd = p * keep / (1.0 - float(np.float32(ratio)))
        exp_y.append(pd @ np.asarray(v, np.float64))
    grads = R.attn_backward_dropout(q, k, v, pd, keep, ratio, dy, np.float64)
    return got, exp_y, grads


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("B,H,Tq,Tk,hs,ratio,kind", [(2, 3, 70, 70, 64, 0.1, "causal"), (1, 2, 130, 130, 128, 0.5, "causal"),
                                                     (2, 2, 33, 50, 48, 0.25, "none"), (3, 2, 40, 40, 64, 0.3, "key"),
                                                     (2, 2, 24, 24, 16, 0.2, "bqk")])
def test_attn_dropout_forward_and_backward(dev, B, H, Tq, Tk, hs, ratio, kind, half):
    rng = np.random.default_rng(3)
    mask, bm = None, 0
    if kind == "causal":
        mask = np.tril(np.ones((Tq, Tk), np.float32))
    elif kind == "key":
        mask, bm = (rng.random((B, Tk)) > 0.3).astype(np.float32), 1
        mask[:, 0] = 1
    elif kind == "bqk":
        mask, bm = (rng.random((B, Tq, Tk)) > 0.3).astype(np.float32), 2
        mask[:, :, 0] = 1
    tol = BF16_RTOL if half else FP32_RTOL
    (ys, dq, dk, dv), exp_y, (edq, edk, edv) = _dropout_case(dev, B, H, Tq, Tk, hs, ratio, 1234, mask, bm, half)
    what = "dropout %.2f %s hs %d" % (ratio, kind, hs)
    assert_close(ys[0], exp_y[0], tol, what + " y")
    assert_close(dq, edq, tol, what + " dq")
    assert_close(dk, edk, tol, what + " dk")
    assert_close(dv, edv, tol, what + " dv")


def test_attn_dropout_draws_a_new_mask_per_forward_call_and_backward_repeats_the_last(dev):
    (ys, dq, dk, dv), exp_y, (edq, edk, edv) = _dropout_case(dev, 2, 2, 48, 48, 64, 0.4, 77, np.tril(np.ones((48, 48), np.float32)), 0,
                                                              False, calls=3)
    for c in range(3):
        assert_close(ys[c], exp_y[c], FP32_RTOL, "forward call %d" % (c + 1))
    assert np.abs(ys[0] - ys[1]).max() > 1e-2 and np.abs(ys[1] - ys[2]).max() > 1e-2
    assert_close(dq, edq, FP32_RTOL, "dq after three forward calls")
    assert_close(dk, edk, FP32_RTOL, "dk after three forward calls")
    assert_close(dv, edv, FP32_RTOL, "dv after three forward calls")


def test_attn_dropout_is_ignored_outside_training_and_checked_at_set(dev):
    rng = np.random.default_rng(5)
    B, H, T, hs = 2, 2, 40, 64
    q, k, v = (rng.standard_normal((B, H, T, hs)).astype(np.float32) for _ in range(3))
    m = np.tril(np.ones((T, T), np.float32))
    hc, ha = dev.cuda.CreateCuDNN(), dev.cuda.CreateAttn()
    dev.cuda.SetAttn(hc, ha, 0, False, B, T, H, hs, 0.5, 9)   # inference: the ratio has no effect (attn.cu:578)
    hq, hk, hv, hy, hm = dev.put(q), dev.put(k), dev.put(v), dev.zeros(q.size), dev.put(m)
    dev.cuda.AttnScaledDotProductForward(hc, ha, T, hq, hk, hv, hm, hy, False)
    assert_close(dev.get(hy, q.shape), _probs(q, k, m, 0) @ v.astype(np.float64), FP32_RTOL, "inference with a ratio set")
    from mycaffe_amd.cudadnn import CudaDnnError
    with pytest.raises(CudaDnnError):
        dev.cuda.SetAttn(hc, ha, 0, True, B, T, H, hs, 1.0, 9)
    dev.cuda.FreeAttn(ha)
    dev.cuda.FreeCuDNN(hc)
