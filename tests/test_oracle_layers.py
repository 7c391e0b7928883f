"""Pins the numpy checker (oracle/attention_ref.py) against reference-held
golden vectors, library routines and closed forms.  CPU only."""
import json
import os

import numpy as np
import pytest

from oracle import attention_ref as R
from tests.conftest import GOLDEN, load_txt

INL = json.load(open(os.path.join(GOLDEN, "inline_vectors.json")))


# ---- inline known-answer vectors of TestCudaDnn.cs --------------------------------

def test_gemm_inline_all_transposes():
    g = INL["gemm"]
    A, B = g["data"][:6], g["data"]
    exp = np.array(g["result"], np.float32).reshape(2, 4)
    for tA, tB, a, b in [(0, 0, A, B), (1, 0, g["A_T"], B), (1, 1, g["A_T"], g["B_T"]), (0, 1, A, g["B_T"])]:
        out = R.gemm(bool(tA), bool(tB), 2, 4, 3, 1.0, a, b, 0.0)
        assert np.array_equal(out, exp), (tA, tB)


def test_gemv_inline():
    g = INL["gemv"]
    assert np.array_equal(R.gemv(False, 2, 3, 1.0, g["data"], g["data"][:3], 0.0), np.array(g["result_notrans"], np.float32))
    assert np.array_equal(R.gemv(True, 2, 3, 1.0, g["data"], g["data"][:2], 0.0), np.array(g["result_trans"], np.float32))


def test_mask_inline():
    x = np.array(INL["mask"]["x"], np.float32)
    n = x.size
    for i in range(n):
        m = np.ones(n, np.float32)
        m[i:] = 0
        exp = x.copy()
        exp[i:] = -np.inf
        assert np.array_equal(R.mask(n, n, 0.0, -np.inf, x, m), exp)


def test_mask2_inline_wraps_mask():
    x = np.array(INL["mask2"]["x"], np.float32)
    n, nm = x.size, x.size // 2
    for i in range(n):
        m = np.ones(nm, np.float32)
        m[i:] = 0
        exp = x.copy()
        for j in range(i, n):
            if m[j % nm] == 0:
                exp[j] = -np.inf
        assert np.array_equal(R.mask(n, nm, 0.0, -np.inf, x, m), exp)


def test_mask_batch_inline():
    g = INL["mask_batch"]
    x = np.array(g["x"], np.float32)
    exp = x.copy()
    exp[g["masked_positions"]] = -np.inf
    out = R.mask_batch(x.size, g["batch"], len(g["mask"]), 0.0, -np.inf, x, g["mask"])
    assert np.array_equal(out, exp)


def test_channel_copy_inline():
    g = INL["channel_copy"]
    cnt = g["num"] * g["channels"] * g["inner"]
    allx = np.array(g["all"], np.float32)
    rebuilt = np.zeros_like(allx)
    for off, key in enumerate("ABC"):
        y = R.channel_copy_fwd(cnt, g["num"], g["channels"], g["blocks"], g["inner"], off, allx)
        assert np.array_equal(y, np.array(g[key], np.float32))
        rebuilt = R.channel_copy_bwd(cnt, g["num"], g["channels"], g["blocks"], g["inner"], off, rebuilt, y)
    assert np.array_equal(rebuilt, allx)


# ---- library routines / closed forms ----------------------------------------------

def test_gemm2_matmul_matches_numpy():
    rng = np.random.default_rng(0)
    A = rng.standard_normal((6, 5, 7))
    B = rng.standard_normal((6, 7, 3))
    out = R.matmul(6, 5, 3, 7, A, B, scale=0.5, dtype=np.float64)
    assert np.allclose(out, 0.5 * (A @ B), rtol=1e-13, atol=1e-13)
    Bt = B.transpose(0, 2, 1).copy()
    out = R.matmul(6, 5, 3, 7, A, Bt, transB=True, dtype=np.float64)
    assert np.allclose(out, A @ B, rtol=1e-13, atol=1e-13)
    At = A.transpose(0, 2, 1).copy()
    out = R.matmul(6, 5, 3, 7, At, B, transA=True, dtype=np.float64)
    assert np.allclose(out, A @ B, rtol=1e-13, atol=1e-13)


def test_rmsnorm_layer_backward_matches_torch_autograd():
    import torch
    rng = np.random.default_rng(6)
    x = torch.tensor(rng.standard_normal((1, 5, 24)), dtype=torch.float64, requires_grad=True)
    w = torch.tensor(rng.standard_normal(24) + 1.0, dtype=torch.float64, requires_grad=True)
    dy = rng.standard_normal((1, 5, 24))
    y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w
    y.backward(torch.tensor(dy))
    dx, dw = R.rmsnorm_layer_backward(x.detach().numpy(), w.detach().numpy(), dy, 1e-5, np.float64)
    assert np.allclose(dx, x.grad.numpy(), rtol=1e-11, atol=1e-13)
    assert np.allclose(dw, w.grad.numpy(), rtol=1e-11, atol=1e-13)
    # more than one leading entry: the input gradient is still the full one, the weight gradient is the first entry's
    x3 = rng.standard_normal((3, 5, 24))
    dy3 = rng.standard_normal((3, 5, 24))
    xt = torch.tensor(x3, requires_grad=True)
    (xt * torch.rsqrt((xt * xt).mean(-1, keepdim=True) + 1e-5) * w.detach()).backward(torch.tensor(dy3))
    dx3, dw3 = R.rmsnorm_layer_backward(x3, w.detach().numpy(), dy3, 1e-5, np.float64)
    assert np.allclose(dx3, xt.grad.numpy(), rtol=1e-11, atol=1e-13)
    _, dw0 = R.rmsnorm_layer_backward(x3[:1], w.detach().numpy(), dy3[:1], 1e-5, np.float64)
    assert np.allclose(dw3, dw0)


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("axis", [-1, 1])
def test_softmax_backward_matches_torch_autograd(axis, log):
    import torch
    rng = np.random.default_rng(5)
    x = torch.tensor(rng.standard_normal((3, 7, 11)) * 3, dtype=torch.float64, requires_grad=True)
    dy = rng.standard_normal((3, 7, 11))
    y = torch.log_softmax(x, dim=axis) if log else torch.softmax(x, dim=axis)
    y.backward(torch.tensor(dy))
    got = R.softmax_backward(y.detach().numpy(), dy, axis, log, np.float64)
    assert np.allclose(got, x.grad.numpy(), rtol=1e-11, atol=1e-13)


def test_softmax_matches_scipy():
    from scipy.special import softmax
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, 4, 9)) * 5
    assert np.allclose(R.softmax_lastaxis(x, np.float64), softmax(x, axis=-1), rtol=1e-13)


def test_transpose_matches_numpy_permute():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 5, 3, 4)).astype(np.float32)
    perm = (0, 2, 1, 3)
    y = np.transpose(x, perm)
    xs = [5 * 3 * 4, 3 * 4, 4, 1]
    ys = [int(np.prod(y.shape[i + 1:])) for i in range(4)]
    out = R.transpose(x, xs, ys, perm)
    assert np.array_equal(out.reshape(y.shape), y)
    assert np.array_equal(R.transpose_hw(2, 5, 3, 4, x).reshape(2, 5, 4, 3), x.transpose(0, 1, 3, 2))


def test_rope_is_complex_rotation_with_explicit_positions():
    # closed form: (re + i im) * exp(i * pos * theta^(-2j/hs)); T == seq_len so the
    # kernel's index-derived position equals the true token position for every batch
    B, T, H, hs, theta = 2, 6, 3, 8, 10000.0
    rng = np.random.default_rng(3)
    x = rng.standard_normal((B, T, H, hs))
    out = R.rope_forward(x, T, H, hs, theta, dtype=np.float64).reshape(B, T, H, hs // 2, 2)
    z = x.reshape(B, T, H, hs // 2, 2)
    zc = z[..., 0] + 1j * z[..., 1]
    j = np.arange(hs // 2)
    ang = np.arange(T)[:, None] * theta ** (-2.0 * j / hs)[None, :]
    rot = zc * np.exp(1j * ang)[None, :, None, :]
    # tables are built in fp32 by the reference host code
    assert np.allclose(out[..., 0], rot.real, atol=2e-6)
    assert np.allclose(out[..., 1], rot.imag, atol=2e-6)
    # invariants: pair norms preserved; position 0 is the identity
    assert np.allclose(np.hypot(out[..., 0], out[..., 1]), np.abs(zc), atol=1e-6)
    assert np.allclose(out[:, 0].reshape(B, H, hs), x[:, 0], atol=0)


def test_rope_freq_offset_selects_position_row():
    H, hs, S = 2, 8, 16
    rng = np.random.default_rng(4)
    x = rng.standard_normal((1, 1, H, hs))
    full = rng.standard_normal((1, S, H, hs))
    full[0, 5] = x[0, 0]
    whole = R.rope_forward(full, S, H, hs, dtype=np.float64).reshape(1, S, H, hs)
    one = R.rope_forward(x, S, H, hs, freq_offset=5 * hs // 2, dtype=np.float64).reshape(H, hs)
    assert np.allclose(one, whole[0, 5], atol=1e-12)
    # offset <= 0 means "no shift" (rope.cu:808-814)
    assert np.array_equal(R.rope_forward(x, S, H, hs, freq_offset=0), R.rope_forward(x, S, H, hs, freq_offset=-1))


def test_attention_matches_torch_sdpa():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(5)
    B, H, T, hs = 2, 3, 7, 8
    q, k, v = (rng.standard_normal((B, H, T, hs)) for _ in range(3))
    y, p = R.attn_forward(q, k, v, R.causal_mask(T, np.float64), False, np.float64)
    ref = F.scaled_dot_product_attention(*(torch.from_numpy(a) for a in (q, k, v)), is_causal=True).numpy()
    assert np.allclose(y, ref, rtol=1e-12, atol=1e-12)
    assert np.all(np.triu(p, 1) == 0) and np.allclose(p.sum(-1), 1)
    # key-padding mask (B,T): torch boolean mask broadcast over heads and rows
    lens = [4, 7]
    km = np.zeros((B, T))
    for b, n in enumerate(lens):
        km[b, :n] = 1
    y2, _ = R.attn_forward(q, k, v, km, True, np.float64)
    ref2 = F.scaled_dot_product_attention(*(torch.from_numpy(a) for a in (q, k, v)),
                                          attn_mask=torch.from_numpy(km.astype(bool))[:, None, None, :]).numpy()
    assert np.allclose(y2, ref2, rtol=1e-12, atol=1e-12)


def test_fully_masked_row_is_uniform_not_nan():
    q = np.zeros((1, 1, 2, 4), np.float32)
    k = np.ones((1, 1, 2, 4), np.float32)
    v = np.arange(8, dtype=np.float32).reshape(1, 1, 2, 4)
    y, p = R.attn_forward(q, k, v, np.zeros((1, 2), np.float32), True)
    assert np.allclose(p, 0.5) and np.allclose(y[0, 0, 0], v[0, 0].mean(0))


def test_kv_cache_attention_equals_last_row_of_causal():
    rng = np.random.default_rng(6)
    B, H, L, hs = 2, 3, 9, 8
    q, k, v = (rng.standard_normal((B, H, L, hs)) for _ in range(3))
    full, _ = R.attn_forward(q, k, v, R.causal_mask(L, np.float64), False, np.float64)
    dec = R.kv_cache_attention(q[:, :, -1], k, v, np.float64)
    assert np.allclose(dec, full[:, :, -1], rtol=1e-12, atol=1e-12)


def test_rmsnorm_silu_match_torch():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(7)
    x = rng.standard_normal((3, 5, 16))
    w = rng.standard_normal(16)
    ref = F.rms_norm(torch.from_numpy(x), (16,), torch.from_numpy(w), eps=1e-5).numpy()
    assert np.allclose(R.rmsnorm_layer(x, w, 1e-5, np.float64), ref, rtol=1e-12)
    assert np.allclose(R.silu(x, np.float64), F.silu(torch.from_numpy(x)).numpy(), rtol=1e-12)


# ---- reference-held golden tensors (minGPT CausalSelfAttention dumps) --------------

@pytest.mark.parametrize("name,heads", [("gpt-pico-csa", 1), ("gpt-pico-csa3", 3), ("gpt-pico-csa3B", 3), ("gpt-pico-csaB", 1)])
def test_causal_self_attention_golden(name, heads):
    d = os.path.join(GOLDEN, name)
    x = load_txt(os.path.join(d, "x.txt"))
    out = R.causal_self_attention(
        x, load_txt(os.path.join(d, "attn_weight.txt")), load_txt(os.path.join(d, "attn_bias.txt")),
        load_txt(os.path.join(d, "attn_proj_weight.txt")), load_txt(os.path.join(d, "attn_proj_bias.txt")),
        heads, dtype=np.float64)
    y = load_txt(os.path.join(d, "y.txt"))
    assert np.abs(out["y"] - y.reshape(out["y"].shape)).max() < 2e-7
    qt = load_txt(os.path.join(d, "qt.txt"))
    assert np.abs(out["qt"] - qt.reshape(out["qt"].shape)).max() < 2e-7
    if os.path.exists(os.path.join(d, "var_att.npy")):
        att = np.load(os.path.join(d, "var_att.npy"))
        assert np.abs(out["att"] - att).max() < 2e-7
        assert np.all(np.triu(att, 1) == 0)
        assert np.abs(out["vt"] - np.load(os.path.join(d, "var_vt.npy"))).max() < 2e-7
        assert np.abs(out["work"] - np.load(os.path.join(d, "var_y.npy"))).max() < 2e-7
    # fp32 arithmetic stays within the fp32 parity tolerance of the fp64 result
    out32 = R.causal_self_attention(
        x, load_txt(os.path.join(d, "attn_weight.txt")), load_txt(os.path.join(d, "attn_bias.txt")),
        load_txt(os.path.join(d, "attn_proj_weight.txt")), load_txt(os.path.join(d, "attn_proj_bias.txt")), heads)
    assert np.abs(out32["y"] - out["y"]).max() < 1e-6


# ---- remaining primitives against independent library routines -----------------------

def test_gemm2_colmajor_matches_blas_sgemm_strided():
    """Column-major strided-batched semantics against scipy's BLAS dgemm on Fortran-ordered views,
    with padded leading dimensions, both transposes and beta != 0."""
    from scipy.linalg import blas
    rng = np.random.default_rng(5)
    m, n, k, batch = 4, 3, 5, 3
    for tA in (False, True):
        for tB in (False, True):
            ar, ac = (k, m) if tA else (m, k)
            br, bc = (n, k) if tB else (k, n)
            lda, ldb, ldc = ar + 2, br + 1, m + 3
            sA, sB, sC = lda * ac + 4, ldb * bc + 2, ldc * n + 1
            A = rng.standard_normal(sA * batch)
            B = rng.standard_normal(sB * batch)
            C = rng.standard_normal(sC * batch)
            out = R.gemm2_colmajor(tA, tB, m, n, k, 0.7, A, B, -0.3, C, lda, ldb, ldc, sA, sB, sC, batch, dtype=np.float64)
            exp = C.copy()
            for b in range(batch):
                a = A[b * sA:b * sA + lda * ac].reshape((lda, ac), order="F")[:ar]
                bb = B[b * sB:b * sB + ldb * bc].reshape((ldb, bc), order="F")[:br]
                c = exp[b * sC:b * sC + ldc * n].reshape((ldc, n), order="F")
                c[:m] = blas.dgemm(0.7, a, bb, beta=-0.3, c=np.asfortranarray(c[:m]), trans_a=tA, trans_b=tB)
            assert np.allclose(out, exp, rtol=1e-13, atol=1e-13), (tA, tB)


def test_embed_inner_product_match_torch():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(6)
    w = rng.standard_normal((11, 5)).astype(np.float32)
    ids = np.array([3.0, 0.0, 10.0, 3.0, 7.0], np.float32)   # the reference passes indices as floats
    assert np.array_equal(R.embed_fwd(ids, w), F.embedding(torch.tensor(ids).long(), torch.tensor(w)).numpy())
    x = rng.standard_normal((2, 3, 5))
    wt = rng.standard_normal((4, 5))
    b = rng.standard_normal(4)
    exp = F.linear(torch.tensor(x), torch.tensor(wt), torch.tensor(b)).numpy()
    assert np.allclose(R.inner_product(x, wt, b, dtype=np.float64), exp, rtol=1e-13, atol=1e-13)
    assert np.allclose(R.inner_product(x, wt, None, dtype=np.float64), exp - b, rtol=1e-12, atol=1e-12)


def test_rope_tables_closed_form():
    """cos/sin(pos * theta^(-2j/hs)) in float64; the fp32 table may differ by the rounding of the angle
    (|d angle| <= 2^-24 * pos), nothing more."""
    S, hs, theta = 64, 16, 10000.0
    c, s = R.rope_tables(S, hs, theta)
    assert c.shape == (S, hs // 2) and s.shape == (S, hs // 2)
    pos = np.arange(S, dtype=np.float64)[:, None]
    ang = pos * theta ** (-np.arange(0, hs, 2, dtype=np.float64) / hs)[None, :]
    tol = 4e-7 * (1 + pos)
    assert np.all(np.abs(c - np.cos(ang)) <= tol) and np.all(np.abs(s - np.sin(ang)) <= tol)
    assert np.all(c[0] == 1) and np.all(s[0] == 0)
    assert c[1, 0] == np.float32(np.cos(np.float32(1.0))) and s[1, 0] == np.float32(np.sin(np.float32(1.0)))


@pytest.mark.parametrize("kind", ["none", "causal", "key", "full"])
def test_multihead_attention_matches_torch_mha(kind):
    """The whole layer (four projections, head split, scaled scores, mask fill, softmax, merge) against
    torch.nn.functional.multi_head_attention_forward with separate projection weights; self attention for
    the causal / full masks, cross attention (T_q != T_k) with a key padding mask."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(8)
    B, Tq, C, H = 3, 5, 8, 2
    Tk = 7 if kind in ("none", "key") else Tq
    xq = rng.standard_normal((B, Tq, C))
    xk = rng.standard_normal((B, Tk, C)) if Tk != Tq else xq
    W = [rng.standard_normal((C, C)) * 0.4 for _ in range(4)]
    b = [rng.standard_normal(C) * 0.1 for _ in range(4)]
    mask_data = None
    attn_mask = None
    kpm = None
    if kind == "causal":
        mask_data = R.causal_mask(Tq, np.float64)
        attn_mask = torch.tensor(mask_data.reshape(Tq, Tq) == 0)
    elif kind == "key":
        lens = np.array([7, 3, 5])
        mask_data = (np.arange(Tk)[None, :] < lens[:, None]).astype(np.float64)
        kpm = torch.tensor(mask_data == 0)
    elif kind == "full":
        lens = np.array([5, 2, 4])
        keep = (np.arange(Tq)[None, None, :] < lens[:, None, None]) & np.tril(np.ones((Tq, Tq), bool))[None]
        mask_data = keep.astype(np.float64)
        attn_mask = torch.tensor(np.repeat(~keep, H, axis=0))           # (B*H, Tq, Tk), batch-major like torch
    out = R.multihead_attention(xq, xk, xk, W[0], b[0], W[1], b[1], W[2], b[2], W[3], b[3], H, mask_data, kind, dtype=np.float64)
    t = lambda a: torch.tensor(a)
    exp, _ = F.multi_head_attention_forward(
        t(xq).transpose(0, 1), t(xk).transpose(0, 1), t(xk).transpose(0, 1), C, H, None,
        torch.cat([t(b[0]), t(b[1]), t(b[2])]), None, None, False, 0.0, t(W[3]), t(b[3]), training=False,
        key_padding_mask=kpm, need_weights=False, attn_mask=attn_mask, use_separate_proj_weight=True,
        q_proj_weight=t(W[0]), k_proj_weight=t(W[1]), v_proj_weight=t(W[2]))
    assert np.allclose(out["y"], exp.transpose(0, 1).numpy(), rtol=1e-10, atol=1e-10)
    assert np.allclose(out["att"].sum(-1), 1.0)


# ---- LayerNorm / GELU / SiLU / RoPE / attention gradients -----------------------------------

@pytest.mark.parametrize("name", ["gpt-pico-ln", "gpt-pico-ln3", "gpt-pico-ln3B", "gpt-pico-ln-blk"])
def test_layernorm_golden_forward_backward(name):
    d = os.path.join(GOLDEN, name)
    x = load_txt(os.path.join(d, "x.txt"))
    y, sd = R.layernorm_forward(x, x.shape[-1], 1e-10, np.float64)
    assert np.abs(y - load_txt(os.path.join(d, "y.txt"))).max() < 3e-7
    g = os.path.join(d, "iter_0") if name == "gpt-pico-ln-blk" else d   # that set keeps its gradients one level down
    dx = R.layernorm_backward(y, load_txt(os.path.join(g, "grad_1a_y.txt")), sd, x.shape[-1], 1e-10, 1, np.float64)
    assert np.abs(dx - load_txt(os.path.join(g, "grad_9_x.txt"))).max() < 3e-8


def test_layernorm_matches_torch_and_autograd():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 5, 24))
    dy = rng.standard_normal((2, 5, 24))
    eps = 1e-5
    xt = torch.tensor(x, requires_grad=True)
    yt = F.layer_norm(xt, (24,), eps=eps)
    yt.backward(torch.tensor(dy))
    y, sd = R.layernorm_forward(x, 24, eps, np.float64)
    assert np.allclose(y, yt.detach().numpy(), rtol=1e-12, atol=1e-13)
    # eps = 0 in the divisor bump: the exact gradient
    dx = R.layernorm_backward(y, dy, sd, 24, eps, 0, np.float64)
    assert np.allclose(dx, xt.grad.numpy(), rtol=1e-10, atol=1e-12)
    # the bump touches the first rows (=10) flat entries only, once per backward call
    dx2 = R.layernorm_backward(y, dy, sd, 24, eps, 2, np.float64)
    flat, flat2 = dx.reshape(-1), dx2.reshape(-1)
    assert np.array_equal(flat[10:], flat2[10:])
    assert np.allclose(flat2[:10], flat[:10] * sd[0] / (sd[0] + 2 * eps), rtol=1e-12)


def test_gelu_golden_and_library():
    import torch
    import torch.nn.functional as F
    d = os.path.join(GOLDEN, "gpt-pico-gelu")
    x = load_txt(os.path.join(d, "1_x.txt"))
    y = load_txt(os.path.join(d, "2_y.txt"))
    dy = load_txt(os.path.join(d, "grad_1_y.txt"))
    dx = load_txt(os.path.join(d, "grad_2_x.txt"))
    assert np.abs(R.gelu(x, True, np.float64) - y).max() < 1e-8
    assert np.abs(R.gelu_grad(x, dy, True, np.float64) - dx).max() < 1e-8
    rng = np.random.default_rng(4)
    x = rng.standard_normal(500) * 3
    g = rng.standard_normal(500)
    for bert, approx in ((True, "tanh"), (False, "none")):
        xt = torch.tensor(x, requires_grad=True)
        yt = F.gelu(xt, approximate=approx)
        yt.backward(torch.tensor(g))
        assert np.allclose(R.gelu(x, bert, np.float64), yt.detach().numpy(), rtol=1e-7, atol=1e-9)
        # the reference's gradient constants are rounded to six digits
        assert np.allclose(R.gelu_grad(x, g, bert, np.float64), xt.grad.numpy(), rtol=2e-5, atol=2e-6)
        assert np.allclose(R.gelu(x, bert), R.gelu(x, bert, np.float64), rtol=1e-6, atol=1e-7)


def test_silu_grad_and_rope_backward():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(6)
    x = rng.standard_normal(300) * 4
    g = rng.standard_normal(300)
    xt = torch.tensor(x, requires_grad=True)
    F.silu(xt).backward(torch.tensor(g))
    assert np.allclose(R.silu_grad(x, g, np.float64), xt.grad.numpy(), rtol=1e-12)
    # the rotation is orthogonal: <rope(x), dy> == <x, rope_backward(dy)> and backward(forward(x)) == x
    B, T, H, hs = 2, 5, 3, 8
    x = rng.standard_normal((B, T, H, hs))
    dy = rng.standard_normal((B, T, H, hs))
    y = R.rope_forward(x, T, H, hs, dtype=np.float64)
    dx = R.rope_backward(dy, T, H, hs, dtype=np.float64)
    assert abs((y * dy.reshape(y.shape)).sum() - (x * dx.reshape(x.shape)).sum()) < 1e-6
    assert np.allclose(R.rope_backward(y, T, H, hs, dtype=np.float64).reshape(x.shape), x, atol=1e-6)


@pytest.mark.parametrize("name,heads", [("gpt-pico-csa", 1), ("gpt-pico-csa3", 3), ("gpt-pico-csa3B", 3), ("gpt-pico-csaB", 1)])
def test_attention_backward_golden(name, heads):
    d = os.path.join(GOLDEN, name)
    out = R.causal_self_attention(
        load_txt(os.path.join(d, "x.txt")), load_txt(os.path.join(d, "attn_weight.txt")), load_txt(os.path.join(d, "attn_bias.txt")),
        load_txt(os.path.join(d, "attn_proj_weight.txt")), load_txt(os.path.join(d, "attn_proj_bias.txt")), heads, dtype=np.float64)
    g = os.path.join(d, "iter_0")
    dy = load_txt(os.path.join(g, "grad_y_pre_transpose.txt"))
    dq, dk, dv = R.attn_backward(out["qt"], out["kt"], out["vt"], out["att"], dy, np.float64)
    for got, f in ((dq, "grad_qt.txt"), (dk, "grad_kt.txt"), (dv, "grad_vt.txt")):
        exp = load_txt(os.path.join(g, f))
        assert np.abs(got - exp.reshape(got.shape)).max() < 1e-8 + 2e-7 * np.abs(exp).max(), f


def test_attention_backward_matches_autograd():
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(8)
    B, H, T, hs = 2, 3, 9, 8
    q, k, v, dy = (rng.standard_normal((B, H, T, hs)) for _ in range(4))
    for causal in (True, False):
        qt, kt, vt = (torch.tensor(a, requires_grad=True) for a in (q, k, v))
        F.scaled_dot_product_attention(qt, kt, vt, is_causal=causal).backward(torch.tensor(dy))
        _, att = R.attn_forward(q, k, v, R.causal_mask(T, np.float64) if causal else None, False, np.float64)
        dq, dk, dv = R.attn_backward(q, k, v, att, dy, np.float64)
        assert np.allclose(dq, qt.grad.numpy(), rtol=1e-9, atol=1e-11)
        assert np.allclose(dk, kt.grad.numpy(), rtol=1e-9, atol=1e-11)
        assert np.allclose(dv, vt.grad.numpy(), rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("name,heads", [("gpt-pico-blk", 1), ("gpt-pico-blk3", 3), ("gpt-pico-blk3B", 3)])
def test_transformer_block_golden(name, heads):
    d = os.path.join(GOLDEN, name)
    p = {k: load_txt(os.path.join(d, k + ".txt")) for k in ("attn_weight", "attn_bias", "attn_proj_weight", "attn_proj_bias",
                                                             "fc_weight", "fc_bias", "proj_weight", "proj_bias")}
    out = R.transformer_block_gpt(load_txt(os.path.join(d, "1_x.txt")), p, heads, "relu", 1e-10, np.float64)
    for key, f in (("ln1", "2_x_ln11"), ("attn", "3_x_attn"), ("xb", "4_x_p_attn"), ("ln2", "5_x_ln2"), ("fc", "6_x_c_fc"),
                   ("act", "7_x_act"), ("mlp", "8_x_c_proj"), ("y", "10_y")):
        exp = load_txt(os.path.join(d, f + ".txt"))
        assert np.abs(out[key] - exp.reshape(out[key].shape)).max() < 5e-7, f


def test_transformer_block_llama_matches_torch_composition():
    """The Llama-style block of the checker against torch library routines: rms_norm, linear, SDPA (causal), silu, with
    the rotary embedding applied as a complex rotation of adjacent pairs."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(12)
    B, T, C, H, hid = 2, 7, 24, 3, 40
    hs = C // H
    p = {"rms1_weight": rng.standard_normal(C), "rms2_weight": rng.standard_normal(C),
         "attn_weight": rng.standard_normal((3 * C, C)) * 0.2, "attn_proj_weight": rng.standard_normal((C, C)) * 0.2,
         "fc_weight": rng.standard_normal((hid, C)) * 0.2, "fc2_weight": rng.standard_normal((hid, C)) * 0.2,
         "proj_weight": rng.standard_normal((C, hid)) * 0.2}
    x = rng.standard_normal((B, T, C))
    got = R.transformer_block_llama(x, p, H, T, 10000.0, 1e-5, np.float64)
    t = {k: torch.tensor(v) for k, v in p.items()}
    xt = torch.tensor(x)

    def rope(v):    # (B,T,H,hs): pairs (2j, 2j+1) rotated by pos * theta^(-2j/hs)
        vc = torch.view_as_complex(v.reshape(B, T, H, hs // 2, 2).contiguous())
        ang = torch.arange(T, dtype=torch.float64)[:, None] * (10000.0 ** (-torch.arange(0, hs, 2, dtype=torch.float64) / hs))[None, :]
        return torch.view_as_real(vc * torch.polar(torch.ones_like(ang), ang)[None, :, None, :]).reshape(B, T, H, hs)

    n1 = F.rms_norm(xt, (C,), t["rms1_weight"], 1e-5)
    q, k, v = F.linear(n1, t["attn_weight"]).split(C, dim=2)
    q, k, v = rope(q.reshape(B, T, H, hs)), rope(k.reshape(B, T, H, hs)), v.reshape(B, T, H, hs)
    att = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True)
    xb = xt + F.linear(att.transpose(1, 2).reshape(B, T, C), t["attn_proj_weight"])
    n2 = F.rms_norm(xb, (C,), t["rms2_weight"], 1e-5)
    want = xb + F.linear(F.silu(F.linear(n2, t["fc_weight"])) * F.linear(n2, t["fc2_weight"]), t["proj_weight"])
    # the table frequencies are rounded to fp32 in the reference (rope.cu:535-553), hence 1e-6 and not 1e-12
    assert np.allclose(got, want.numpy(), rtol=1e-5, atol=1e-6)


# ---- CAFFE-engine softmax chain (SoftmaxLayer.cs:230-273) -------------------------------------

def test_channel_primitives_against_numpy_and_a_worked_case():
    # worked by hand: num 1, channels 3, spatial 2, x[c][s] = [[1, 5], [4, 2], [4, -1]]
    x = np.array([1, 5, 4, 2, 4, -1], np.float32)
    assert R.channel_max(x, 1, 3, 2).tolist() == [4, 5]
    assert R.channel_max(x, 1, 3, 2, return_idx=True).tolist() == [1, 0]          # first maximum wins (strict '>')
    assert R.channel_sub(x, [1, 2], 1, 3, 2).tolist() == [0, 3, 3, 0, 3, -3]
    assert R.channel_div(x, [2, 4], 1, 3, 2).tolist() == [0.5, 1.25, 2, 0.5, 2, -0.25]
    assert R.channel_dot(x, x, 1, 3, 2).tolist() == [33, 30]
    # within a channel: the kernel's own index rule, num * spatial rows of `spatial` values
    assert R.channel_max(np.arange(8, dtype=np.float32), 2, 1, 2, across=False).tolist() == [1, 3, 5, 7]
    rng = np.random.default_rng(0)
    v = rng.standard_normal((3, 5, 7)).astype(np.float32)
    assert np.array_equal(R.channel_max(v, 3, 5, 7), v.max(1).reshape(-1))
    assert np.allclose(R.channel_dot(v, 2 * v, 3, 5, 7), np.einsum("ncs,ncs->ns", v, 2 * v).reshape(-1), rtol=1e-6)


@pytest.mark.parametrize("axis", [1, 2, -1])
def test_softmax_chain_equals_scipy(axis):
    from scipy.special import log_softmax, softmax
    x = np.random.default_rng(1).standard_normal((4, 6, 5)).astype(np.float32) * 3
    assert np.allclose(R.softmax_caffe_chain(x, axis, dtype=np.float64), softmax(x.astype(np.float64), axis=axis), rtol=1e-12)
    assert np.allclose(R.softmax_caffe_chain(x, axis, log=True, dtype=np.float64), log_softmax(x.astype(np.float64), axis=axis), rtol=1e-10, atol=1e-12)


# ---- attention dropout (training mode of the attention handle) ------------------------------------------------------

def test_splitmix64_known_answers():
    # the generator's published outputs for seed 1234567 (first five draws; the state advances by the golden increment)
    G = 0x9E3779B97F4A7C15
    st = np.array([(1234567 + i * G) & (2 ** 64 - 1) for i in range(5)], np.uint64)
    assert [int(x) for x in R.splitmix64(st)] == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                                  4593380528125082431, 16408922859458223821]


@pytest.mark.parametrize("ratio", [0.1, 0.25, 0.5])
def test_attn_dropout_mask_statistics(ratio):
    keep = R.attn_dropout_keep(99, 4, 6, 64, 80, ratio)
    n = keep.size
    sigma = np.sqrt(ratio * (1 - ratio) / n)
    assert abs(keep.mean() - (1 - ratio)) < 4 * sigma
    # rows and columns are not correlated with each other, and another call of the forward pass draws another mask
    assert abs(np.corrcoef(keep[..., :-1].ravel(), keep[..., 1:].ravel())[0, 1]) < 0.01
    assert abs(np.corrcoef(keep[:, :, :-1].ravel(), keep[:, :, 1:].ravel())[0, 1]) < 0.01
    again = R.attn_dropout_keep(99, 4, 6, 64, 80, ratio, forward_calls=2)
    assert abs(np.corrcoef(keep.ravel(), again.ravel())[0, 1]) < 0.01
    assert np.array_equal(R.attn_dropout_keep(99, 4, 6, 64, 80, ratio), keep)


def test_attn_forward_dropout_is_unbiased_and_reduces_to_the_plain_forward():
    rng = np.random.default_rng(0)
    B, H, T, hs = 1, 2, 24, 8
    q, k, v = (rng.standard_normal((B, H, T, hs)) for _ in range(3))
    m = R.causal_mask(T, np.float64)
    y0, p0 = R.attn_forward(q, k, v, m, False, np.float64)
    y, p, pd = R.attn_forward_dropout(q, k, v, np.ones((B, H, T, T), bool), 0.0, m, False, np.float64)
    assert np.array_equal(y, y0) and np.array_equal(p, p0) and np.array_equal(pd, p0)
    acc = np.zeros_like(y0)
    n = 600
    for seed in range(n):
        acc += R.attn_forward_dropout(q, k, v, R.attn_dropout_keep(seed, B, H, T, T, 0.3), 0.3, m, False, np.float64)[0]
    # the mean over masks is the undropped output (error shrinks as 1 / sqrt(n))
    assert np.abs(acc / n - y0).max() < 6 * np.abs(v).max() * np.sqrt(0.3 / 0.7 / n)


def test_attn_backward_dropout_sequence_and_its_closed_form():
    """The reference's step sequence (softmax backward on the probabilities dropout was applied to in place) collapses to
    dS = keep / (1 - r)^2 * P * (dP - dY.Y), dV = (P keep / (1 - r))^T dY, which is what the HIP kernels compute from the
    regenerated mask; with no dropout it is the plain backward pass (itself pinned on torch autograd)."""
    rng = np.random.default_rng(1)
    B, H, T, hs, r = 2, 2, 20, 8, 0.25
    q, k, v, dy = (rng.standard_normal((B, H, T, hs)) for _ in range(4))
    m = R.causal_mask(T, np.float64)
    keep = R.attn_dropout_keep(5, B, H, T, T, r)
    y, p, pd = R.attn_forward_dropout(q, k, v, keep, r, m, False, np.float64)
    dq, dk, dv = R.attn_backward_dropout(q, k, v, pd, keep, r, dy, np.float64)
    dP = dy @ np.swapaxes(v, -1, -2)
    D = (dy * y).sum(-1, keepdims=True)
    dS = keep / (1 - r) ** 2 * p * (dP - D) / np.sqrt(hs)
    assert np.allclose(dq, dS @ k, rtol=1e-12, atol=1e-12)
    assert np.allclose(dk, np.swapaxes(dS, -1, -2) @ q, rtol=1e-12, atol=1e-12)
    assert np.allclose(dv, np.swapaxes(pd, -1, -2) @ dy, rtol=1e-12, atol=1e-12)
    ones = np.ones_like(keep)
    y1, p1, pd1 = R.attn_forward_dropout(q, k, v, ones, 0.0, m, False, np.float64)
    for a, b in zip(R.attn_backward_dropout(q, k, v, pd1, ones, 0.0, dy, np.float64), R.attn_backward(q, k, v, p1, dy, np.float64)):
        assert np.allclose(a, b, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("slope", [0.0, 0.1])
def test_relu_and_its_gradient_against_torch(slope):
    """relu_fwd / relu_bwd of the checker against torch.nn.functional.leaky_relu and its autograd gradient.  The
    reference's backward reads its gate from the TOP data (math.cu:12072-12078); for slope >= 0 the output has the sign
    of the input, so that gate equals the one autograd takes from the input."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(31)
    x = rng.standard_normal((7, 33)).astype(np.float32)
    x[0, :4] = [0.0, -0.0, 1e-30, -1e-30]
    dy = rng.standard_normal(x.shape).astype(np.float32)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = torch.nn.functional.leaky_relu(xt, negative_slope=slope)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    y = R.relu(x, slope, np.float64)
    assert np.allclose(y, yt.detach().numpy(), rtol=0, atol=1e-12)
    nz = x != 0        # at exactly zero the subgradient is a convention
    assert np.allclose(R.relu_grad(y, dy, slope, np.float64)[nz], xt.grad.numpy()[nz], rtol=0, atol=1e-12)
