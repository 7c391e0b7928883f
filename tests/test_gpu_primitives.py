"""GPU parity of the CudaDnn primitives on the attention path, called through the
C ABI exactly as the C# host packs them, checked against the CPU checker and the
reference's inline known-answer vectors."""
import json
import os

import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnnError, DIR, ERROR, SOFTMAX_ALGORITHM, SOFTMAX_MODE
from mycaffe_amd.layers import Blob, SoftmaxLayer
from oracle import attention_ref as R
from tests.conftest import BF16_RTOL, FP32_RTOL, GOLDEN, assert_close, bf16_round

pytestmark = pytest.mark.gpu
INL = json.load(open(os.path.join(GOLDEN, "inline_vectors.json")))


def test_device_name_and_alloc_is_zero_filled(dev):
    assert "gfx950" in dev.cuda.GetDeviceName(0)
    h = dev.zeros(1000)
    assert np.all(dev.get(h) == 0)
    hh = dev.zeros(1000, half=True)
    assert np.all(dev.get(hh) == 0)


def test_set_get_memory_round_trip_and_half_storage(dev):
    x = np.random.default_rng(0).standard_normal(5000).astype(np.float32)
    h = dev.put(x)
    assert np.array_equal(dev.get(h), x)
    dev.cuda.SetMemory(h, x[::-1].copy())
    assert np.array_equal(dev.get(h), x[::-1])
    assert np.array_equal(dev.cuda.GetMemoryFloat(h, 7), x[::-1][:7])
    hh = dev.put(x, half=True)
    assert np.array_equal(dev.get(hh), bf16_round(x))
    # copy converts between storage types
    h2 = dev.zeros(5000)
    dev.cuda.copy(5000, hh, h2)
    assert np.array_equal(dev.get(h2), bf16_round(x))
    dev.cuda.copy(100, h, h2, 10, 20)
    exp = bf16_round(x)
    exp[20:120] = x[::-1][10:110]
    assert np.array_equal(dev.get(h2), exp)


def test_memory_pointer_views_alias_the_allocation(dev):
    x = np.arange(64, dtype=np.float32)
    h = dev.put(x)
    v = dev.cuda.CreateMemoryPointer(h, 16, 8)
    assert np.array_equal(dev.cuda.GetMemoryFloat(v), x[16:24])
    dev.cuda.set(8, v, 5.0)
    assert np.array_equal(dev.get(h)[16:24], np.full(8, 5, np.float32))
    dev.cuda.FreeMemoryPointer(v)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.CreateMemoryPointer(h, 60, 8)
    assert e.value.code == ERROR.MEMORY_RANGE_EXCEEDED


def test_error_codes_bad_handle_and_arg_count(dev):
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.GetMemoryFloat(9999)
    assert e.value.code == ERROR.MEMORY_NOT_FOUND
    with pytest.raises(CudaDnnError) as e:   # mask needs exactly 7 longs (device.cu:2108)
        dev.cuda._ex2(264, [0.0, 1.0], [4, 4, 0, 0, 1, 1])
    assert e.value.code == ERROR.PARAM_OUT_OF_RANGE
    with pytest.raises(CudaDnnError) as e:   # Ex2-style id through the legacy entry point has no long array
        dev.cuda.RunFloat(dev.cuda.m_hKernel, 264, [0.0, 1.0])
    assert e.value.code == ERROR.PARAM_OUT_OF_RANGE
    with pytest.raises(CudaDnnError) as e:
        dev.cuda._ex2(321, None, [1])
    assert e.value.code == ERROR.NOT_IMPLEMENTED
    h = dev.put(np.zeros(4, np.float32))
    hh = dev.put(np.zeros(4, np.float32), half=True)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.add(4, h, hh, h)
    assert e.value.code == ERROR.MEMORY_MIXED_HALF_TYPES
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.add(5, h, h, h)
    assert e.value.code == ERROR.MEMORY_RANGE_EXCEEDED


def test_gemm_inline_vectors_all_transposes(dev):
    g = INL["gemm"]
    exp = np.array(g["result"], np.float32)
    hC = dev.zeros(8)
    for tA, tB, a, b in [(0, 0, g["data"][:6], g["data"]), (1, 0, g["A_T"], g["data"]), (1, 1, g["A_T"], g["B_T"]),
                         (0, 1, g["data"][:6], g["B_T"])]:
        hA, hB = dev.put(a), dev.put(b)
        for _ in range(2):
            dev.cuda.gemm(bool(tA), bool(tB), 2, 4, 3, 1.0, hA, hB, 0.0, hC)
            assert np.array_equal(dev.get(hC), exp), (tA, tB)


def test_gemv_inline_vectors(dev):
    g = INL["gemv"]
    hA = dev.put(g["data"])
    hx, hy = dev.put(g["data"][:3]), dev.zeros(2)
    dev.cuda.gemv(False, 2, 3, 1.0, hA, hx, 0.0, hy)
    assert np.array_equal(dev.get(hy), np.float32(g["result_notrans"]))
    hy2, hx2 = dev.put(g["data"][:2]), dev.zeros(3)
    dev.cuda.gemv(True, 2, 3, 1.0, hA, hy2, 0.0, hx2)
    assert np.array_equal(dev.get(hx2), np.float32(g["result_trans"]))


@pytest.mark.parametrize("tA,tB", [(False, True), (False, False), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k", [(200, 136, 96), (128, 128, 64), (37, 53, 29), (8, 2304, 768), (513, 260, 20)])
def test_gemm_fp32_vs_checker(dev, tA, tB, m, n, k):
    rng = np.random.default_rng(m * 7 + n)
    A = rng.standard_normal((k, m) if tA else (m, k)).astype(np.float32)
    B = rng.standard_normal((n, k) if tB else (k, n)).astype(np.float32)
    C0 = rng.standard_normal((m, n)).astype(np.float32)
    hA, hB, hC = dev.put(A), dev.put(B), dev.put(C0)
    dev.cuda.gemm(tA, tB, m, n, k, 0.5, hA, hB, 2.0, hC)
    ref = R.gemm(tA, tB, m, n, k, 0.5, A, B, 2.0, C0, dtype=np.float64)
    assert_close(dev.get(hC), ref, FP32_RTOL, "gemm fp32")


@pytest.mark.parametrize("m,n,k", [(256, 384, 128), (200, 136, 96), (100, 72, 40)])
def test_gemm_bf16_inner_product_shape(dev, m, n, k):
    rng = np.random.default_rng(n)
    A = bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    B = bf16_round((rng.standard_normal((n, k)) * 0.02).astype(np.float32))
    hA, hB, hC = dev.put(A, True), dev.put(B, True), dev.zeros(m * n, True)
    dev.cuda.gemm(False, True, m, n, k, 1.0, hA, hB, 0.0, hC)
    ref = R.gemm(False, True, m, n, k, 1.0, A, B, 0.0, dtype=np.float64)
    assert_close(dev.get(hC), ref, BF16_RTOL, "gemm bf16")


@pytest.mark.parametrize("m,n,k,alpha,beta", [
    (300, 200, 128, 1.0, 0.0),      # edge tiles in both directions
    (512, 768, 192, 0.5, 0.0),      # interior only, 128 x 192 tiles, alpha
    (384, 256, 64, 1.0, 2.0),       # beta != 0: read-modify-write epilogue
    (1024, 1024, 2048, 1.0, 0.0),   # fewer 128 x 128 tiles than CUs and fewer than 200 tiles of 64 x 128: 64 x 64 tiles
    (2048, 768, 2048, 1.0, 0.0),    # the same dispatch at the w2 shape of the batched prompt pass
    (2048, 1024, 512, 1.0, 0.0),    # 128 tiles of 128 x 128, 256 of 64 x 128: the 64 x 128 tile
    (2000, 1000, 512, 0.5, 1.0),    # the 64 x 128 tile with ragged edges and a read-modify-write epilogue
    (260, 132, 64, 0.25, -1.0),     # ragged, both scalars
])
def test_gemm_fp32_large_tile_paths(dev, m, n, k, alpha, beta):
    rng = np.random.default_rng(m + n + k + 1)
    A = rng.standard_normal((m, k)).astype(np.float32)
    B = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    C0 = rng.standard_normal((m, n)).astype(np.float32)
    hA, hB, hC = dev.put(A), dev.put(B), dev.put(C0)
    dev.cuda.gemm(False, True, m, n, k, alpha, hA, hB, beta, hC)
    ref = R.gemm(False, True, m, n, k, alpha, A, B, beta, C0, dtype=np.float64)
    assert_close(dev.get(hC, (m, n)), ref, FP32_RTOL, "gemm fp32 large tiles")


@pytest.mark.parametrize("m,n,k,alpha,beta", [
    (300, 200, 128, 1.0, 0.0),
    (512, 768, 192, 0.5, 0.0),
    (384, 256, 64, 1.0, 2.0),
    (1024, 1024, 2048, 1.0, 0.0),   # 64 x 64 tiles (see the fp32 list)
    (2048, 768, 2048, 1.0, 0.0),    # 64 x 64 tiles
    (2048, 1024, 512, 1.0, 0.0),    # 64 x 128 tiles
    (2000, 1000, 512, 0.5, 1.0),    # 64 x 128 tiles, ragged, beta != 0
    (260, 132, 64, 0.25, -1.0),
])
def test_gemm_bf16_large_tile_paths(dev, m, n, k, alpha, beta):
    rng = np.random.default_rng(m + n + k)
    A = bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    B = bf16_round((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    C0 = bf16_round(rng.standard_normal((m, n)).astype(np.float32))
    hA, hB, hC = dev.put(A, True), dev.put(B, True), dev.put(C0, True)
    dev.cuda.gemm(False, True, m, n, k, alpha, hA, hB, beta, hC)
    ref = R.gemm(False, True, m, n, k, alpha, A, B, beta, C0, dtype=np.float64)
    assert_close(dev.get(hC, (m, n)), ref, BF16_RTOL, "gemm bf16 large tiles")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("tA,tB", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("m,n,k,beta", [
    (1024, 768, 512, 0.0),      # data gradient shape: large enough in fp32 for the operand to be turned in scratch memory
    (768, 512, 2048, 1.0),      # weight gradient shape, accumulated into the result (beta = 1)
    (264, 200, 136, 0.5),       # ragged tiles, multiples of eight
    (260, 132, 72, 0.0),        # multiples of four only: 16-bit storage keeps the strided kernel
])
def test_gemm_backward_transpose_combinations(dev, half, tA, tB, m, n, k, beta):
    """The transpose combinations of InnerProductLayer.backward (InnerProductLayer.cs:429-494) at sizes where an operand
    is turned in scratch memory and the product runs on the A B^T kernels, against the float64 checker."""
    rng = np.random.default_rng(m + n + k + 2 * tA + tB)
    A = bf16_round(rng.standard_normal((k, m) if tA else (m, k)).astype(np.float32))
    B = bf16_round((rng.standard_normal((n, k) if tB else (k, n)) * 0.05).astype(np.float32))
    C0 = bf16_round(rng.standard_normal((m, n)).astype(np.float32))
    hA, hB, hC = dev.put(A, half), dev.put(B, half), dev.put(C0, half)
    dev.cuda.gemm(tA, tB, m, n, k, 1.0, hA, hB, beta, hC)
    ref = R.gemm(tA, tB, m, n, k, 1.0, A, B, beta, C0, dtype=np.float64)
    assert_close(dev.get(hC, (m, n)), ref, BF16_RTOL if half else FP32_RTOL, "gemm, transposed operands")
    # the operands are left as they were
    assert np.array_equal(dev.get(hA), A.reshape(-1)) and np.array_equal(dev.get(hB), B.reshape(-1))


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("tA,tB", [(False, True), (True, False)])
@pytest.mark.parametrize("m,n,k,alpha,beta", [
    (768, 512, 4096, 1.0, 0.0),     # 24 tiles of 128 x 128: eight parts of 512
    (300, 260, 2048, 0.5, 1.0),     # ragged tiles, two parts, both scalars
    (1536, 1152, 2048, 1.0, 1.0),   # 108 tiles: two parts
])
def test_gemm_long_contraction_split_over_workgroups(dev, half, tA, tB, m, n, k, alpha, beta):
    """Weight-gradient shapes (few tiles, the token count as the contraction): partial products of equal slices of K by
    rows of workgroups, summed in fp32 by a second kernel; against the float64 checker."""
    rng = np.random.default_rng(m + n + k + tA)
    A = bf16_round(rng.standard_normal((k, m) if tA else (m, k)).astype(np.float32))
    B = bf16_round((rng.standard_normal((n, k) if tB else (k, n)) * 0.05).astype(np.float32))
    C0 = bf16_round(rng.standard_normal((m, n)).astype(np.float32))
    hA, hB, hC = dev.put(A, half), dev.put(B, half), dev.put(C0, half)
    dev.cuda.gemm(tA, tB, m, n, k, alpha, hA, hB, beta, hC)
    ref = R.gemm(tA, tB, m, n, k, alpha, A, B, beta, C0, dtype=np.float64)
    assert_close(dev.get(hC, (m, n)), ref, BF16_RTOL if half else FP32_RTOL, "gemm, split contraction")
    # the same call again gives the same bits: the parts are summed in a fixed order
    hC2 = dev.put(C0, half)
    dev.cuda.gemm(tA, tB, m, n, k, alpha, hA, hB, beta, hC2)
    assert np.array_equal(dev.get(hC2), dev.get(hC))


def test_gemm_offsets_and_bias_rank1_update(dev):
    # InnerProductLayer.cs:411-415: y = x W^T, then y += ones(M,1) * bias(1,N) through gemm with K = 1
    rng = np.random.default_rng(3)
    M, N, K = 96, 80, 64
    x, W, b = rng.standard_normal((M, K)), rng.standard_normal((N, K)), rng.standard_normal(N)
    hx, hW, hb, hones, hy = dev.put(x), dev.put(W), dev.put(b), dev.put(np.ones(M)), dev.zeros(M * N)
    dev.cuda.gemm(False, True, M, N, K, 1.0, hx, hW, 0.0, hy)
    dev.cuda.gemm(False, False, M, N, 1, 1.0, hones, hb, 1.0, hy)
    assert_close(dev.get(hy), R.inner_product(x, W, b, np.float64), FP32_RTOL, "inner product")
    # offsets: second half of A rows
    hy2 = dev.zeros(M * N)
    dev.cuda.gemm(False, True, M // 2, N, K, 1.0, hx, hW, 0.0, hy2, nAOffset=(M // 2) * K, nCOffset=(M // 2) * N)
    out = dev.get(hy2, (M, N))
    assert np.all(out[:M // 2] == 0)
    assert_close(out[M // 2:], (x @ W.T)[M // 2:], FP32_RTOL, "gemm offsets")


def test_scores_product_is_held_back_without_changing_any_result(dev):
    """Q K^T of the explicit attention chain (CausalSelfAttentionLayer.cs:583-603) waits for the calls that follow it: the
    scaling becomes its alpha and, under a causal mask, the softmax pass has only the tiles that touch the lower triangle
    computed.  Whatever reads or changes the scores, or an operand, in between sees what the immediate calls would have
    left.  Every variant against numpy."""
    rng = np.random.default_rng(8)
    cuda = dev.cuda
    outer, T, hs = 16, 512, 64
    n = outer * T * T
    q = rng.standard_normal((outer, T, hs)).astype(np.float32)
    kt = rng.standard_normal((outer, hs, T)).astype(np.float32)
    tril = np.tril(np.ones((T, T), np.float32))
    hm = dev.put(tril)
    hc, d = cuda.CreateCuDNN(), cuda.CreateTensorDesc()
    cuda.SetTensorDesc(d, outer * T, T, 1, 1, False)
    sc = q.astype(np.float64) @ kt.astype(np.float64)
    masked = np.where(tril == 0, -1e29, sc * 0.125)
    p = np.exp(masked - masked.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)

    def chain(hq, hkt, hatt, mask=hm):
        cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
        cuda.scal(n, 0.125, hatt)
        cuda.mask(n, T * T, 0.0, -1e29, hatt, mask, hatt)

    # the whole chain: probabilities, and afterwards the scores tensor itself (masked and scaled, also where no tile was computed)
    hq, hkt, hatt, hp = dev.put(q), dev.put(kt), dev.put(np.full(n, 7.0, np.float32)), dev.zeros(n)
    chain(hq, hkt, hatt)
    cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hatt, 0.0, d, hp)
    assert_close(dev.get(hp, p.shape), p, FP32_RTOL, "probabilities")
    got = dev.get(hatt, sc.shape)
    assert np.all(got[:, tril == 0] == np.float32(-1e29))
    assert_close(got[:, tril == 1], (sc * 0.125)[:, tril == 1], FP32_RTOL, "masked, scaled scores")
    # read right after the product, after the scaling, after the mask
    hatt = dev.zeros(n)
    cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
    assert_close(dev.get(hatt, sc.shape), sc, FP32_RTOL, "scores")
    cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
    cuda.scal(n, 0.125, hatt)
    assert_close(dev.get(hatt, sc.shape), sc * 0.125, FP32_RTOL, "scaled scores")
    chain(hq, hkt, hatt)
    assert_close(dev.get(hatt, sc.shape), np.where(tril == 0, -1e29, sc * 0.125), FP32_RTOL, "masked scores")
    # an operand changes, or goes, while the product waits: the values of the moment of the call count
    hq2 = dev.put(q)
    cuda.matmul(outer, T, T, hs, hq2, hkt, hatt)
    cuda.set(q.size, hq2, 0.0)
    assert_close(dev.get(hatt, sc.shape), sc, FP32_RTOL, "scores after q was overwritten")
    hq3 = dev.put(q)
    chain(hq3, hkt, hatt)
    cuda.FreeMemory(hq3)
    cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hatt, 0.0, d, hp)
    assert_close(dev.get(hp, p.shape), p, FP32_RTOL, "probabilities after q was freed")
    # a mask that is not the causal one: the whole product
    m2 = (rng.random((T, T)) > 0.3).astype(np.float32)
    m2[:, 0] = 1
    hm2 = dev.put(m2)
    chain(hq, hkt, hatt, hm2)
    cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hatt, 0.0, d, hp)
    mk2 = np.where(m2 == 0, -1e29, sc * 0.125)
    p2 = np.exp(mk2 - mk2.max(-1, keepdims=True))
    p2 /= p2.sum(-1, keepdims=True)
    assert_close(dev.get(hp, p.shape), p2, FP32_RTOL, "probabilities under another mask")
    # softmax with no mask call in between
    cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
    cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hatt, 0.0, d, hp)
    p3 = np.exp(sc - sc.max(-1, keepdims=True))
    p3 /= p3.sum(-1, keepdims=True)
    assert_close(dev.get(hp, p.shape), p3, FP32_RTOL, "probabilities without a mask")
    # a second product into the same tensor replaces the first; the result freed while its product waits
    cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
    cuda.matmul(outer, T, T, hs, hq, hkt, hatt, 2.0)
    assert_close(dev.get(hatt, sc.shape), 2.0 * sc, FP32_RTOL, "second product")
    cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
    cuda.FreeMemory(hatt)
    assert_close(dev.get(hq, q.shape), q, 0.0, "q untouched")


@pytest.mark.parametrize("scale", [0.125, 0.3])
def test_matmul_by_a_tensor_whose_scaling_is_held_back(dev, scale):
    """Blob.MatMulGrad (Blob.cs:4304-4311) scales a gradient and multiplies by it twice.  The scaling of a large tensor
    waits; a power of two then goes into the products' alpha and keeps waiting - every partial product and sum is the
    same number times that power, so the products come out bit for bit as with the tensor scaled in memory - and any
    other factor is applied before the first product.  Reading the tensor, or overwriting it through the softmax
    gradient, afterwards shows the scaled values, or the new ones."""
    from mycaffe_amd.cudadnn import SOFTMAX_ALGORITHM, SOFTMAX_MODE
    rng = np.random.default_rng(3)
    cuda = dev.cuda
    outer, T, hs = 8, 512, 64
    n = outer * T * T
    assert n >= 1 << 20
    g = rng.standard_normal((outer, T, T)).astype(np.float32)
    kt = rng.standard_normal((outer, hs, T)).astype(np.float32)
    q = rng.standard_normal((outer, T, hs)).astype(np.float32)

    def products(hg, immediate):
        hdq, hdkt = dev.zeros(outer * T * hs), dev.zeros(outer * T * hs)
        cuda.scal(n, scale, hg)
        if immediate:
            dev.get(hg)          # a read in between: the scaling is applied in memory first
        # dq = dS k (dS times kt transposed), dkt = q^T dS
        cuda.matmul(outer, T, hs, T, hg, hkt_, hdq, 1.0, False, True)
        cuda.matmul(outer, hs, T, T, hq_, hg, hdkt, 1.0, True, False)
        return dev.get(hdq, (outer, T, hs)), dev.get(hdkt, (outer, hs, T))

    hkt_, hq_ = dev.put(kt), dev.put(q)
    a1, b1 = products(dev.put(g), True)
    hg = dev.put(g)
    a2, b2 = products(hg, False)
    gs = g.astype(np.float64) * np.float32(scale)
    assert_close(a1, gs @ kt.astype(np.float64).transpose(0, 2, 1), FP32_RTOL, "dS k")
    assert_close(b1, q.astype(np.float64).transpose(0, 2, 1) @ gs, FP32_RTOL, "q^T dS")
    if scale == 0.125:
        assert np.array_equal(a1, a2) and np.array_equal(b1, b2)
    else:
        assert_close(a2, a1, FP32_RTOL, "dS k, factor applied first")
        assert_close(b2, b1, FP32_RTOL, "q^T dS, factor applied first")
    assert np.array_equal(dev.get(hg, g.shape), g * np.float32(scale))
    # the scaled tensor overwritten by a softmax gradient: nothing of the old factor is left on it
    cuda.scal(n, scale, hg)
    y = rng.random((outer * T, T)).astype(np.float32)
    y /= y.sum(-1, keepdims=True)
    dy = rng.standard_normal((outer * T, T)).astype(np.float32)
    hy, hdy = dev.put(y), dev.put(dy)
    hc, d = cuda.CreateCuDNN(), cuda.CreateTensorDesc()
    cuda.SetTensorDesc(d, outer * T, T, 1, 1, False)
    cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d, hdy, 0.0, d, hg)
    want = y.astype(np.float64) * (dy - (y.astype(np.float64) * dy).sum(-1, keepdims=True))
    assert_close(dev.get(hg, want.shape), want, FP32_RTOL, "softmax gradient over a tensor with a factor outstanding")


@pytest.mark.parametrize("M,N,K", [(2048, 768, 768), (1024, 1024, 96), (4096, 264, 40), (512, 2304, 8192)])
def test_inner_product_and_its_bias_update_run_as_one_launch_without_changing_any_result(dev, M, N, K):
    """The forward pass of an inner product layer (InnerProductLayer.cs:372-417) is two gemm calls: Y = X W^T, then the rank-1
    update ones (M) x bias (N) added to Y.  The first waits for the second and both run as one launch; with Y read in
    between, a multiplier that is not all ones, other factors, or an operand changed while the product waits, the calls
    run as they are.  Every variant against numpy, and the fused result bit for bit against the two-launch one."""
    rng = np.random.default_rng(M + N + K)
    cuda = dev.cuda
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    hx, hw, hb, hy, hone = dev.put(x), dev.put(w), dev.put(b), dev.put(np.full(M * N, 3.0, np.float32)), dev.put(np.ones(M, np.float32))

    def product(hy=hy, hx=hx):
        cuda.gemm(False, True, M, N, K, 1.0, hx, hw, 0.0, hy)

    def bias(hone=hone, alpha=1.0, beta=1.0, hy=hy):
        cuda.gemm(False, False, M, N, 1, alpha, hone, hb, beta, hy)

    # two launches: the result is read in between
    product()
    assert_close(dev.get(hy, ref.shape), ref, FP32_RTOL, "product")
    bias()
    two = dev.get(hy, ref.shape)
    assert_close(two, ref + b, FP32_RTOL, "product + bias, two launches")
    # one launch, twice over (the second time the multiplier is known to be ones)
    for _ in range(2):
        cuda.set(M * N, hy, 5.0)
        product()
        bias()
        assert np.array_equal(dev.get(hy, ref.shape), two)
    # the product alone, read later
    product()
    cuda.set(N, hb, 0.0)
    assert_close(dev.get(hy, ref.shape), ref, FP32_RTOL, "product read after another blob was written")
    cuda.SetMemory(hb, b)
    # a multiplier that is not all ones, or becomes ones only later
    m2 = np.ones(M, np.float32)
    m2[M // 3] = 0.5
    hm2 = dev.put(m2)
    product()
    bias(hm2)
    assert_close(dev.get(hy, ref.shape), ref + np.outer(m2, b), FP32_RTOL, "multiplier with another entry")
    cuda.SetMemory(hm2, np.ones(M, np.float32))
    product()
    bias(hm2)
    assert np.array_equal(dev.get(hy, ref.shape), two)
    cuda.SetMemory(hm2, m2)
    product()
    bias(hm2)
    assert_close(dev.get(hy, ref.shape), ref + np.outer(m2, b), FP32_RTOL, "multiplier changed back")
    # other factors on the update
    product()
    bias(alpha=2.0)
    assert_close(dev.get(hy, ref.shape), ref + 2 * b, FP32_RTOL, "alpha 2")
    product()
    bias(beta=0.5)
    assert_close(dev.get(hy, ref.shape), 0.5 * ref + b, FP32_RTOL, "beta 0.5")
    # the input changes, or goes, while the product waits: the values of the moment of the call count
    hx2 = dev.put(x)
    product(hx=hx2)
    cuda.set(M * K, hx2, 0.0)
    bias()
    assert_close(dev.get(hy, ref.shape), ref + b, FP32_RTOL, "input overwritten before the bias call")
    hx3 = dev.put(x)
    product(hx=hx3)
    cuda.FreeMemory(hx3)
    bias()
    assert_close(dev.get(hy, ref.shape), ref + b, FP32_RTOL, "input freed before the bias call")
    # the update on another tensor leaves the waiting product alone; a second product replaces the first
    hy2 = dev.put(np.zeros(M * N, np.float32))
    product()
    bias(hy=hy2)
    assert_close(dev.get(hy2, ref.shape), np.broadcast_to(b, ref.shape), FP32_RTOL, "update of another tensor")
    assert_close(dev.get(hy, ref.shape), ref, FP32_RTOL, "product after an update elsewhere")
    product()
    product()
    bias()
    assert np.array_equal(dev.get(hy, ref.shape), two)
    # the result is the input of the next product (two layers in a row, N == K only for the first shape)
    if N == K:
        product()
        bias()
        hy3 = dev.zeros(M * N)
        product(hy=hy3, hx=hy)
        bias(hy=hy3)
        y1 = (ref + b).astype(np.float32).astype(np.float64)
        assert_close(dev.get(hy3, ref.shape), y1 @ w.astype(np.float64).T + b, 5e-4, "second layer on the first one's result")
    # the result freed while its product waits
    hy4 = dev.zeros(M * N)
    product(hy=hy4)
    cuda.FreeMemory(hy4)
    cuda.SynchronizeDevice()
    for h in (hx, hw, hb, hy, hone, hm2, hx2, hy2):
        cuda.FreeMemory(h)


@pytest.mark.parametrize("replace", [-1e29, -3.0])
def test_matmul_after_a_causal_softmax_stops_at_the_diagonal_only_when_the_masked_weights_are_zero(dev, replace):
    """The explicit attention chain (CausalSelfAttentionLayer.cs:583-603): scale, mask, softmax, MatMul with v.  The softmax
    pass that folds the causal mask in leaves word that the weights above the diagonal are exact zeros, and the MatMul
    then stops each block of queries at its diagonal.  With a replacement value that leaves those weights non-zero
    (-3), or after anything else has written to the weights, the whole contraction runs.  Either way against numpy."""
    rng = np.random.default_rng(5)
    cuda = dev.cuda
    outer, T, hs = 6, 512, 64
    n = outer * T * T
    sc = rng.standard_normal((outer, T, T)).astype(np.float32) * 3
    v = rng.standard_normal((outer, T, hs)).astype(np.float32)
    tril = np.tril(np.ones((T, T), np.float32))
    hm, hv = dev.put(tril), dev.put(v)
    hc, d = cuda.CreateCuDNN(), cuda.CreateTensorDesc()
    cuda.SetTensorDesc(d, outer * T, T, 1, 1, False)
    masked = np.where(tril == 0, np.float64(replace), sc.astype(np.float64) * 0.125)
    p = np.exp(masked - masked.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)

    def weights():
        h, hp = dev.put(sc), dev.zeros(n)
        cuda.scal(n, 0.125, h)
        cuda.mask(n, T * T, 0.0, replace, h, hm, h)
        cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, h, 0.0, d, hp)
        return hp

    hp, hy = weights(), dev.zeros(outer * T * hs)
    cuda.matmul(outer, T, hs, T, hp, hv, hy)
    assert_close(dev.get(hy, v.shape), p @ v, FP32_RTOL, "weights @ v")
    assert_close(dev.get(hp, p.shape), p, FP32_RTOL, "weights")
    # the weights are written to before the MatMul (one of them above the diagonal set to one): the whole row counts
    hp = weights()
    cuda.set(1, hp, 1.0, 5 * T + 300)          # sequence 0, query 5, key 300
    p2 = p.copy()
    p2[0, 5, 300] = 1.0
    cuda.matmul(outer, T, hs, T, hp, hv, hy)
    assert_close(dev.get(hy, v.shape), p2 @ v, FP32_RTOL, "changed weights @ v")
    # a product with other operands of the same shape is untouched by the record
    hq = dev.put(rng.standard_normal((outer, T, T)).astype(np.float32))
    cuda.matmul(outer, T, hs, T, hq, hv, hy)
    assert_close(dev.get(hy, v.shape), dev.get(hq, p.shape).astype(np.float64) @ v, FP32_RTOL, "other weights @ v")
    # the backward pass multiplies by the transposed weights (Blob.MatMulGrad, Blob.cs:4304-4311: v' = weights^T y'): that
    # contraction, over the queries, begins at the diagonal; with an entry above the diagonal written, the whole column counts
    hp = weights()
    cuda.matmul(outer, T, hs, T, hp, hv, hy, 1.0, True, False)
    assert_close(dev.get(hy, v.shape), p.transpose(0, 2, 1) @ v, FP32_RTOL, "weights^T @ y'")
    cuda.set(1, hp, 1.0, 5 * T + 300)
    cuda.matmul(outer, T, hs, T, hp, hv, hy, 1.0, True, False)
    assert_close(dev.get(hy, v.shape), p2.transpose(0, 2, 1) @ v, FP32_RTOL, "changed weights^T @ y'")
    cuda.matmul(outer, T, hs, T, hq, hv, hy, 1.0, True, False)
    assert_close(dev.get(hy, v.shape), dev.get(hq, p.shape).astype(np.float64).transpose(0, 2, 1) @ v, FP32_RTOL, "other weights^T @ y'")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("m,n,k", [
    (96, 80, 64),           # fewer tiles than CUs, ragged edges
    (300, 200, 128),        # edge tiles in both directions
    (512, 768, 192),        # 128 x 192 tiles, interior only
    (2048, 768, 768),       # the attention layer's output projection
    (1024, 1024, 2048),     # long contraction
    (1536, 1152, 2048),     # wide tiles in 16-bit storage
    (4096, 4096, 2048),     # 256 x 256 tiles in both storage types
    (37, 53, 29),           # no tile kernel takes it: product in the workspace, then one pass
    (260, 132, 64),
])
def test_linear_forward_is_the_inner_product_with_its_bias(dev, half, bias, m, n, k):
    """Id 2005 against the float64 checker and against the two calls it replaces (InnerProductLayer.cs:372-417)."""
    rng = np.random.default_rng(m + n + k + 5)
    x = bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    W = bf16_round((rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    b = bf16_round(rng.standard_normal(n).astype(np.float32))
    hx, hW, hb, hy = dev.put(x, half), dev.put(W, half), dev.put(b, half), dev.put(np.full(m * n, 7.0, np.float32), half)
    dev.cuda.LinearForward(m, n, k, hx, hW, hb if bias else 0, hy)
    got = dev.get(hy, (m, n))
    ref = x.astype(np.float64) @ W.astype(np.float64).T + (b.astype(np.float64) if bias else 0.0)
    assert_close(got, ref, BF16_RTOL if half else FP32_RTOL, "linear forward vs checker")
    hy2, hones = dev.zeros(m * n, half), dev.put(np.ones(m, np.float32), half)
    dev.cuda.gemm(False, True, m, n, k, 1.0, hx, hW, 0.0, hy2)
    if bias:
        dev.cuda.gemm(False, False, m, n, 1, 1.0, hones, hb, 1.0, hy2)
    two = dev.get(hy2, (m, n))
    # 16-bit storage: the two calls round the product and then the sum, the one call rounds once
    assert_close(got, two, BF16_RTOL if half else 1e-5, "linear forward vs gemm and bias gemm")


def test_linear_forward_checks_its_arguments(dev):
    hx, hW, hb, hy = dev.zeros(64 * 32), dev.zeros(48 * 32), dev.zeros(48), dev.zeros(64 * 48)
    dev.cuda.LinearForward(64, 48, 32, hx, hW, hb, hy)
    with pytest.raises(CudaDnnError):
        dev.cuda.LinearForward(64, 49, 32, hx, hW, hb, hy)          # weight, bias and y are too short
    with pytest.raises(CudaDnnError):
        dev.cuda.LinearForward(0, 48, 32, hx, hW, hb, hy)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.LinearForward(64, 48, 32, hx, hW, dev.zeros(48, half=True), hy)
    assert e.value.code == ERROR.MEMORY_MIXED_HALF_TYPES
    with pytest.raises(CudaDnnError):
        dev.cuda._ex2(2005, None, [64, 48, 32, hx, hW, hb])


def test_matmul_batched_is_gemm2_with_swapped_operands(dev):
    rng = np.random.default_rng(4)
    outer, m, n, k = 6, 50, 24, 40
    A, B = rng.standard_normal((outer, m, k)), rng.standard_normal((outer, k, n))
    hA, hB, hC = dev.put(A), dev.put(B), dev.zeros(outer * m * n)
    dev.cuda.matmul(outer, m, n, k, hA, hB, hC, 0.125)
    assert_close(dev.get(hC), 0.125 * (A @ B), FP32_RTOL, "matmul")
    Bt = B.transpose(0, 2, 1).copy()
    hBt = dev.put(Bt)
    dev.cuda.matmul(outer, m, n, k, hA, hBt, hC, 1.0, bTransB=True)
    assert_close(dev.get(hC), A @ B, FP32_RTOL, "matmul transB")
    assert_close(dev.get(hC), R.matmul(outer, m, n, k, A, Bt, transB=True, dtype=np.float64), FP32_RTOL, "matmul vs checker")


@pytest.mark.parametrize("tA", [False, True])
@pytest.mark.parametrize("tB", [False, True])
@pytest.mark.parametrize("m,n,k,batch", [(64, 256, 64, 6), (256, 64, 256, 4), (132, 200, 76, 3), (36, 36, 8, 2), (128, 128, 20, 2)])
def test_gemm2_strided_batched_blas_semantics(dev, tA, tB, m, n, k, batch):
    """Column-major strided-batched gemm with padded leading dimensions and strides (cublasSgemmStridedBatched
    semantics, math.cu:1750-1788), alpha / beta, every transpose combination; sizes that take the matrix-core kernel
    (all extents multiples of 4) including ragged tiles."""
    rng = np.random.default_rng(m + n + k)
    ar, ac = (k, m) if tA else (m, k)
    br, bc = (n, k) if tB else (k, n)
    lda, ldb, ldc = ar + 4, br + 8, m + 4
    sA, sB, sC = lda * ac + 8, ldb * bc + 4, ldc * n + 4
    A = rng.standard_normal(sA * batch).astype(np.float32)
    B = rng.standard_normal(sB * batch).astype(np.float32)
    C = rng.standard_normal(sC * batch).astype(np.float32)
    hA, hB, hC = dev.put(A), dev.put(B), dev.put(C)
    dev.cuda.gemm2(tA, tB, m, n, k, 0.7, hA, hB, -0.3, hC, lda, ldb, ldc, sA, sB, sC, batch)
    ref = R.gemm2_colmajor(tA, tB, m, n, k, 0.7, A, B, -0.3, C, lda, ldb, ldc, sA, sB, sC, batch, dtype=np.float64)
    assert_close(dev.get(hC), ref, FP32_RTOL, "gemm2 tA=%s tB=%s" % (tA, tB))
    # the padding of C between columns and batches is untouched
    got = dev.get(hC)
    for b in range(batch):
        blk = got[b * sC:(b + 1) * sC]
        assert np.array_equal(blk[ldc * n:], C[b * sC + ldc * n:(b + 1) * sC])
        assert np.array_equal(blk[:ldc * n].reshape(n, ldc)[:, m:], C[b * sC:b * sC + ldc * n].reshape(n, ldc)[:, m:])


@pytest.mark.parametrize("beta", [0.0, 1.0, 0.5])
@pytest.mark.parametrize("tA,tB", [(True, False), (False, False)])
def test_gemm_fp32_long_contraction_few_tiles(dev, tA, tB, beta):
    """Weight-gradient shape (InnerProductLayer.cs:445-447): few output tiles, a long contraction; the contraction is split
    over workgroups there, so the result is checked for every beta (the accumulate case is the layer's)."""
    rng = np.random.default_rng(45)
    m, n, k = 192, 160, 4096
    A = rng.standard_normal((k, m) if tA else (m, k)).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    C = rng.standard_normal((m, n)).astype(np.float32)
    hA, hB, hC = dev.put(A), dev.put(B), dev.put(C)
    dev.cuda.gemm(tA, tB, m, n, k, 0.5, hA, hB, beta, hC)
    ref = 0.5 * ((A.T if tA else A).astype(np.float64) @ B) + beta * C
    assert_close(dev.get(hC, (m, n)), ref, FP32_RTOL, "long K")


def test_matmul_attention_chain_shapes(dev):
    """The two MatMul calls of the explicit attention chain (CausalSelfAttentionLayer.cs:583-603) at 64-wide heads."""
    rng = np.random.default_rng(44)
    outer, T, hs = 6, 256, 64
    q, kt, v = rng.standard_normal((outer, T, hs)), rng.standard_normal((outer, hs, T)), rng.standard_normal((outer, T, hs))
    hq, hkt, hv, hatt, hy = dev.put(q), dev.put(kt), dev.put(v), dev.zeros(outer * T * T), dev.zeros(outer * T * hs)
    dev.cuda.matmul(outer, T, T, hs, hq, hkt, hatt)
    att = q @ kt
    assert_close(dev.get(hatt), att, FP32_RTOL, "q @ k^T")
    dev.cuda.matmul(outer, T, hs, T, hatt, hv, hy)
    assert_close(dev.get(hy), att @ v, FP32_RTOL, "att @ v")


@pytest.mark.parametrize("hs", [32, 64, 128])
@pytest.mark.parametrize("Tq,Tk", [(512, 512), (300, 260), (129, 1028)])
def test_matmul_scores_of_the_attention_chain_with_the_query_panel_in_registers(dev, hs, Tq, Tk):
    """Q K^T of the explicit attention chain (CausalSelfAttentionLayer.cs:583-590: MatMul of q with the transposed keys)
    at sizes that take the kernel built for short contractions: whole and ragged tiles, the three head sizes, then the
    BLAS form of the same call with both scalars."""
    rng = np.random.default_rng(hs + Tq)
    outer = 64
    q, kt = rng.standard_normal((outer, Tq, hs)).astype(np.float32), rng.standard_normal((outer, hs, Tk)).astype(np.float32)
    hq, hkt, hatt = dev.put(q), dev.put(kt), dev.put(np.full(outer * Tq * Tk, 3.0, np.float32))
    dev.cuda.matmul(outer, Tq, Tk, hs, hq, hkt, hatt)
    want = q.astype(np.float64) @ kt.astype(np.float64)
    assert_close(dev.get(hatt, want.shape), want, FP32_RTOL, "q @ k^T")
    # C = alpha A B + beta C through id 219 itself (column-major: C^T = K^T-operand first)
    c0 = rng.standard_normal((outer, Tq, Tk)).astype(np.float32)
    hc = dev.put(c0)
    dev.cuda._ex2(219, [0.5, -2.0], [0, 0, Tk, Tq, hs, 0, hkt, hq, 0, hc, Tk, hs, Tk, hs * Tk, Tq * hs, Tq * Tk, outer])
    assert_close(dev.get(hc, want.shape), 0.5 * want - 2.0 * c0, FP32_RTOL, "gemm2 with both scalars")


@pytest.mark.parametrize("half", [False, True])
def test_gemv_decode_shapes(dev, half):
    rng = np.random.default_rng(5)
    for d, n in [(288, 288), (768, 288), (288, 768), (1000, 52), (3, 7)]:
        W = (rng.standard_normal((d, n)) * 0.02).astype(np.float32)
        if half:
            W = bf16_round(W)
        x = rng.standard_normal(n).astype(np.float32)
        y0 = rng.standard_normal(d).astype(np.float32)
        hW, hx, hy = dev.put(W, half), dev.put(x), dev.put(y0)
        dev.cuda.gemv(False, d, n, 1.0, hW, hx, 0.0, hy)
        assert_close(dev.get(hy), W.astype(np.float64) @ x, FP32_RTOL, "gemv")
        dev.cuda.gemv(False, d, n, 2.0, hW, hx, 1.0, hy)
        assert_close(dev.get(hy), 3 * (W.astype(np.float64) @ x), FP32_RTOL, "gemv beta")
        hx2 = dev.zeros(n)
        dev.cuda.gemv(True, d, n, 1.0, hW, hy, 0.0, hx2)
        assert_close(dev.get(hx2), W.astype(np.float64).T @ dev.get(hy), FP32_RTOL, "gemv transposed")


@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("m,n", [(8192, 2304), (4096, 770), (1000, 52), (256, 4), (5000, 1)])
def test_gemv_transposed_over_many_rows(dev, half, m, n):
    """y = alpha A^T x + beta y with many rows (the bias gradient of an inner product layer, InnerProductLayer.cs:473-478:
    A = the output gradient, x = ones): rows dealt over workgroups, partial sums added in a fixed order, so two runs give
    the same bits.  Column counts that allow 16-byte loads and ones that do not; matrix in fp32 and in 16-bit storage."""
    rng = np.random.default_rng(m + n)
    A = rng.standard_normal((m, n)).astype(np.float32)
    if half:
        A = bf16_round(A)
    x = rng.standard_normal(m).astype(np.float32)
    y0 = rng.standard_normal(n).astype(np.float32)
    hA, hx = dev.put(A, half), dev.put(x)
    ref = A.astype(np.float64).T @ x
    # sums of m products of N(0,1) numbers: compare on the scale of the sum's terms
    tol = 2e-6 * np.sqrt(m) * 4
    outs = []
    for _ in range(2):
        hy = dev.put(y0)
        dev.cuda.gemv(True, m, n, 0.5, hA, hx, 2.0, hy)
        got = dev.get(hy)
        assert np.max(np.abs(got - (0.5 * ref + 2.0 * y0))) < tol * 0.5 + 1e-5
        outs.append(got)
    assert np.array_equal(outs[0], outs[1])
    hy = dev.put(y0)
    dev.cuda.gemv(True, m, n, 1.0, hA, dev.put(np.ones(m, np.float32)), 0.0, hy)
    assert np.max(np.abs(dev.get(hy) - A.astype(np.float64).sum(0))) < tol


@pytest.mark.parametrize("tA", [False, True])
def test_gemv_in_16_bit_storage(dev, tA):
    """Matrix and both vectors in 16-bit storage (the bias gradient of an inner product kept that way); a 16-bit vector with
    an fp32 matrix stays refused."""
    m, n = 300, 136
    rng = np.random.default_rng(9 + tA)
    A = bf16_round(rng.standard_normal((m, n)).astype(np.float32))
    x = bf16_round(rng.standard_normal(m if tA else n).astype(np.float32))
    y0 = bf16_round(rng.standard_normal(n if tA else m).astype(np.float32))
    hA, hx, hy = dev.put(A, True), dev.put(x, True), dev.put(y0, True)
    dev.cuda.gemv(tA, m, n, 0.5, hA, hx, 1.0, hy)
    want = 0.5 * ((A.T if tA else A).astype(np.float64) @ x) + y0
    assert_close(dev.get(hy), want, BF16_RTOL, "gemv, 16-bit storage")
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.gemv(tA, m, n, 1.0, dev.put(A), hx, 0.0, hy)
    assert e.value.code == ERROR.MEMORY_HALF_TYPE_NOT_SUPPORTED


def test_timed_dispatch_over_argument_sets_takes_them_in_turn(dev):
    """MCH_TimeInvokeFloatEx2Sets: dispatch i runs with the i-th list of long arguments (modulo the number of lists)."""
    from mycaffe_amd.cudadnn import CUDAFN
    n = 1000
    src = dev.put(np.arange(n, dtype=np.float32))
    dsts = [dev.zeros(n) for _ in range(3)]
    sets = [[n, src, d, 0, 0, -1, -1, -1] for d in dsts]
    ms = dev.cuda.TimeFunctionSets(CUDAFN.CUDA_COPY, None, sets, 0, 2)      # two dispatches: sets 0 and 1
    assert ms > 0
    assert np.array_equal(dev.get(dsts[0]), np.arange(n)) and np.array_equal(dev.get(dsts[1]), np.arange(n))
    assert not dev.get(dsts[2]).any()
    dev.cuda.TimeFunctionSets(CUDAFN.CUDA_COPY, None, sets, 1, 2)           # one warm-up and two timed: sets 0, 1, 2
    assert np.array_equal(dev.get(dsts[2]), np.arange(n))
    with pytest.raises(ValueError):
        dev.cuda.TimeFunctionSets(CUDAFN.CUDA_COPY, None, [sets[0], sets[1][:5]], 0, 1)
    # one list is the plain timing call
    assert dev.cuda.TimeFunctionSets(CUDAFN.CUDA_COPY, None, sets[:1], 1, 3) > 0


def test_mask_inline_vectors(dev):
    x = np.array(INL["mask"]["x"], np.float32)
    n = x.size
    hx, hm, hy = dev.put(x), dev.zeros(n), dev.zeros(n)
    for i in range(n):
        m = np.ones(n, np.float32)
        m[i:] = 0
        dev.cuda.SetMemory(hm, m)
        dev.cuda.set(n, hy, 0)
        dev.cuda.mask(n, n, 0.0, -np.inf, hx, hm, hy)
        exp = x.copy()
        exp[i:] = -np.inf
        assert np.array_equal(dev.get(hy), exp)
    x2 = np.array(INL["mask2"]["x"], np.float32)
    hx2, hm2, hy2 = dev.put(x2), dev.put([1, 0, 1, 0]), dev.zeros(8)
    dev.cuda.mask(8, 4, 0.0, -1e29, hx2, hm2, hy2)
    assert np.array_equal(dev.get(hy2), R.mask(8, 4, 0.0, -1e29, x2, [1, 0, 1, 0]))


def test_mask_batch_inline_vectors(dev):
    g = INL["mask_batch"]
    x = np.array(g["x"], np.float32)
    hx, hm, hy = dev.put(x), dev.put(g["mask"]), dev.zeros(x.size)
    dev.cuda.mask_batch(x.size, g["batch"], len(g["mask"]), 0.0, -np.inf, hx, hm, hy)
    exp = x.copy()
    exp[g["masked_positions"]] = -np.inf
    assert np.array_equal(dev.get(hy), exp)


def test_channel_copy_inline_vectors(dev):
    g = INL["channel_copy"]
    cnt = g["num"] * g["channels"] * g["inner"]
    hall = dev.put(g["all"])
    hs = []
    for off, key in enumerate("ABC"):
        h = dev.zeros(cnt)
        dev.cuda.channel_copy(cnt, g["num"], g["channels"], g["blocks"], g["inner"], off, hall, h, DIR.FWD)
        assert np.array_equal(dev.get(h), np.float32(g[key]))
        hs.append(h)
    hback = dev.zeros(len(g["all"]))
    for off, h in enumerate(hs):
        dev.cuda.channel_copy(cnt, g["num"], g["channels"], g["blocks"], g["inner"], off, hback, h, DIR.BWD)
    assert np.array_equal(dev.get(hback), np.float32(g["all"]))


def test_channel_copy_splits_fused_qkv(dev):
    # CausalSelfAttentionLayer.cs:537-539: (B,T,3C) -> q,k,v (B,T,C)
    rng = np.random.default_rng(6)
    B, T, Cc = 3, 17, 48
    x = rng.standard_normal((B, T, 3 * Cc)).astype(np.float32)
    hx = dev.put(x)
    for off in range(3):
        h = dev.zeros(B * T * Cc)
        dev.cuda.channel_copy(B * T * Cc, B, T, 3, Cc, off, hx, h, DIR.FWD)
        assert np.array_equal(dev.get(h, (B, T, Cc)), x[..., off * Cc:(off + 1) * Cc])


@pytest.mark.parametrize("half", [False, True])
def test_transpose_head_split_and_generic(dev, half):
    rng = np.random.default_rng(7)
    shape = (2, 9, 4, 16)
    x = bf16_round(rng.standard_normal(shape).astype(np.float32))
    for perm in [(0, 2, 1, 3), (0, 1, 3, 2), (3, 2, 1, 0)]:
        y = np.transpose(x, perm)
        xs = [int(np.prod(shape[i + 1:])) for i in range(4)]
        ys = [int(np.prod(y.shape[i + 1:])) for i in range(4)]
        hx, hy = dev.put(x, half), dev.zeros(x.size, half)
        hxc, hyc, hmap, hbuf = dev.put(xs), dev.put(ys), dev.put(perm), dev.zeros(x.size * 4)
        dev.cuda.transpose(x.size, hx, hy, hxc, hyc, hmap, 4, hbuf)
        assert np.array_equal(dev.get(hy, y.shape), y), perm
        assert np.array_equal(dev.get(hy), R.transpose(x, xs, ys, perm))
    hx, hy = dev.put(x, half), dev.zeros(x.size, half)
    dev.cuda.transposeHW(2, 9, 4, 16, hx, hy)
    assert np.array_equal(dev.get(hy, (2, 9, 16, 4)), x.transpose(0, 1, 3, 2))
    big = rng.standard_normal((3, 2, 70, 45)).astype(np.float32)
    hb, hb2 = dev.put(big), dev.zeros(big.size)
    dev.cuda.transposeHW(3, 2, 70, 45, hb, hb2)
    assert np.array_equal(dev.get(hb2, (3, 2, 45, 70)), big.transpose(0, 1, 3, 2))


@pytest.mark.parametrize("half", [False, True])
def test_softmax_backward_through_tensor_descriptors(dev, half):
    """Id 112 against the checker: row lengths on the one-wavefront path (multiples of four up to 2048) and off it,
    channel mode with an inner axis, the log form, and the gradient written over dy."""
    rng = np.random.default_rng(18)
    hc = dev.cuda.CreateCuDNN()
    tol = BF16_RTOL if half else FP32_RTOL
    d = dev.cuda.CreateTensorDesc()
    for rows, length in [(24, 200), (9, 1024), (3, 2048), (7, 3000), (5, 1), (6, 37), (130, 64)]:
        y = bf16_round(R.softmax_lastaxis((rng.standard_normal((rows, length)) * 3).astype(np.float32)))
        dy = bf16_round(rng.standard_normal((rows, length)).astype(np.float32))
        hy, hg, hx = dev.put(y, half), dev.put(dy, half), dev.zeros(y.size, half)
        dev.cuda.SetTensorDesc(d, rows, length, 1, 1, half)
        dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d, hg, 0.0, d, hx)
        assert_close(dev.get(hx, y.shape), R.softmax_backward(y, dy, dtype=np.float64), tol, "softmax backward %dx%d" % (rows, length))
        # in place over the incoming gradient
        dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d, hg, 0.0, d, hg)
        assert np.array_equal(dev.get(hg, y.shape), dev.get(hx, y.shape))
    # channel mode: series along c for every (n, h)
    y = bf16_round(R.softmax_lastaxis(rng.standard_normal((3, 6, 10)).astype(np.float32)).transpose(0, 2, 1).copy())   # (3, 10, 6)
    dy = bf16_round(rng.standard_normal(y.shape).astype(np.float32))
    hy, hg, hx = dev.put(y, half), dev.put(dy, half), dev.zeros(y.size, half)
    dev.cuda.SetTensorDesc(d, 3, 10, 6, 1, half)
    dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.CHANNEL, 1.0, d, hy, d, hg, 0.0, d, hx)
    assert_close(dev.get(hx, y.shape), R.softmax_backward(y, dy, axis=1, dtype=np.float64), tol, "softmax backward channel")
    # log form
    x = (rng.standard_normal((11, 96)) * 2).astype(np.float64)
    ylog = bf16_round((x - np.log(np.exp(x).sum(-1, keepdims=True))).astype(np.float32))
    dy = bf16_round(rng.standard_normal(ylog.shape).astype(np.float32))
    hy, hg, hx = dev.put(ylog, half), dev.put(dy, half), dev.zeros(ylog.size, half)
    dev.cuda.SetTensorDesc(d, 11, 96, 1, 1, half)
    dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.LOG, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d, hg, 0.0, d, hx)
    assert_close(dev.get(hx, ylog.shape), R.softmax_backward(ylog, dy, log=True, dtype=np.float64), tol, "log softmax backward")
    # argument checks: scaling factors other than (1, 0), a descriptor of another shape, a short buffer
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d, hg, 1.0, d, hx)
    assert e.value.code == ERROR.NOT_IMPLEMENTED
    d2 = dev.cuda.CreateTensorDesc()
    dev.cuda.SetTensorDesc(d2, 11, 95, 1, 1, half)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d2, hg, 0.0, d, hx)
    assert e.value.code == ERROR.PARAM_OUT_OF_RANGE
    dev.cuda.SetTensorDesc(d, 12, 96, 1, 1, half)
    with pytest.raises(CudaDnnError):
        dev.cuda.SoftmaxBackward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, hy, d, hg, 0.0, d, hx)
    dev.cuda.FreeTensorDesc(d)
    dev.cuda.FreeTensorDesc(d2)
    dev.cuda.FreeCuDNN(hc)


def test_softmax_forward_through_tensor_descriptors(dev):
    rng = np.random.default_rng(8)
    hc = dev.cuda.CreateCuDNN()
    for rows, length in [(24, 200), (7, 3000), (5, 1), (9, 1024), (3, 2048), (130, 64), (6, 37)]:
        x = (rng.standard_normal((rows, length)) * 4).astype(np.float32)
        hx, hy = dev.put(x), dev.zeros(x.size)
        bd, td = dev.cuda.CreateTensorDesc(), dev.cuda.CreateTensorDesc()
        dev.cuda.SetTensorDesc(bd, rows, length, 1, 1)
        dev.cuda.SetTensorDesc(td, rows, length, 1, 1)
        dev.cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, bd, hx, 0.0, td, hy)
        assert_close(dev.get(hy), R.softmax_lastaxis(x, np.float64), FP32_RTOL, "softmax")
        dev.cuda.FreeTensorDesc(bd)
        dev.cuda.FreeTensorDesc(td)
    # channel mode with an inner axis: softmax over c for every (n, h)
    x = rng.standard_normal((3, 10, 6)).astype(np.float32)
    hx, hy = dev.put(x), dev.zeros(x.size)
    bd, td = dev.cuda.CreateTensorDesc(), dev.cuda.CreateTensorDesc()
    dev.cuda.SetTensorDesc(bd, 3, 10, 6, 1)
    dev.cuda.SetTensorDesc(td, 3, 10, 6, 1)
    dev.cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.CHANNEL, 1.0, bd, hx, 0.0, td, hy)
    ref = R.softmax_lastaxis(x.transpose(0, 2, 1), np.float64).transpose(0, 2, 1)
    assert_close(dev.get(hy), ref, FP32_RTOL, "softmax channel")
    # masked rows of -1e29 stay finite and uniform
    x = np.full((2, 8), -1e29, np.float32)
    hx, hy = dev.put(x), dev.zeros(16)
    dev.cuda.SetTensorDesc(bd, 2, 8, 1, 1)
    dev.cuda.SetTensorDesc(td, 2, 8, 1, 1)
    dev.cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, bd, hx, 0.0, td, hy)
    assert np.allclose(dev.get(hy), 0.125)
    dev.cuda.FreeCuDNN(hc)


@pytest.mark.parametrize("half", [False, True])
def test_rope_forward_vs_checker(dev, half):
    rng = np.random.default_rng(9)
    B, T, H, hs = 2, 12, 3, 16
    x = bf16_round(rng.standard_normal((B, T, H, hs)).astype(np.float32))
    h = dev.cuda.CreateRope(0, 0, x.size, B, T, H, hs, 10000.0)
    hx, hy = dev.put(x, half), dev.zeros(x.size, half)
    dev.cuda.RopeForward(h, x.size, hx, hy)
    ref = R.rope_forward(x, T, H, hs, 10000.0)
    assert_close(dev.get(hy), ref, BF16_RTOL if half else 2e-6, "rope")
    # in place, as the layers call it
    dev.cuda.RopeForward(h, x.size, hx, hx)
    assert_close(dev.get(hx), ref, BF16_RTOL if half else 2e-6, "rope in place")
    # decode form: one position, table offset pos*hs/2 (MultiheadAttentionLayer.cs:678-683)
    one = x[:1, 5:6].copy()
    h1, h1y = dev.put(one, half), dev.zeros(one.size, half)
    dev.cuda.RopeForward(h, one.size, h1, h1y, 5 * hs // 2)
    assert_close(dev.get(h1y), ref.reshape(B, T, H, hs)[0, 5], BF16_RTOL if half else 2e-6, "rope offset")
    with pytest.raises(CudaDnnError) as e:   # offset that would leave the table
        dev.cuda.RopeForward(h, one.size, h1, h1y, T * hs // 2)
    assert e.value.code == ERROR.PARAM_OUT_OF_RANGE
    dev.cuda.FreeRope(h)
    with pytest.raises(CudaDnnError) as e:
        dev.cuda.RopeForward(h, one.size, h1, h1y)
    assert e.value.code == ERROR.ROPE_NOT_INITIALIZED


@pytest.mark.parametrize("half", [False, True])
def test_rope_forward_shorter_than_the_handle_keeps_the_reference_index_rule(dev, half):
    # The reference derives a pair's position from its flat index modulo the HANDLE's sequence length
    # (rope.cu:741-744), so with T < seq_len and more than one sequence the second sequence does not restart at
    # position 0: its first rows continue at position T.  Reproduced, not corrected.
    rng = np.random.default_rng(19)
    B, T, S, H, hs = 2, 12, 16, 3, 16
    x = bf16_round(rng.standard_normal((B, T, H, hs)).astype(np.float32))
    h = dev.cuda.CreateRope(0, 0, B * S * H * hs, B, S, H, hs, 10000.0)
    hx, hy = dev.put(x, half), dev.zeros(x.size, half)
    dev.cuda.RopeForward(h, x.size, hx, hy)
    ref = R.rope_forward(x, S, H, hs, 10000.0)
    assert_close(dev.get(hy), ref, BF16_RTOL if half else 2e-6, "rope with T < seq_len")
    # what the quirk amounts to: sequence 1, row 0 is rotated as position 12, and row 4 wraps to position 0
    per_pos = R.rope_forward(np.broadcast_to(x[1, 0], (S, H, hs)).copy(), S, H, hs, 10000.0).reshape(S, H, hs)
    assert_close(ref.reshape(B, T, H, hs)[1, 0], per_pos[12], 1e-6, "sequence 1 row 0 sits at position 12")
    per_pos = R.rope_forward(np.broadcast_to(x[1, 4], (S, H, hs)).copy(), S, H, hs, 10000.0).reshape(S, H, hs)
    assert_close(ref.reshape(B, T, H, hs)[1, 4], per_pos[0], 1e-6, "sequence 1 row 4 wraps to position 0")
    dev.cuda.FreeRope(h)


def test_elementwise_family(dev):
    rng = np.random.default_rng(10)
    n = 10007
    a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    ha, hb, hy = dev.put(a), dev.put(b), dev.zeros(n)
    dev.cuda.add(n, ha, hb, hy)
    assert np.array_equal(dev.get(hy), a + b)
    dev.cuda.add(n, ha, hb, hy, 0.5)
    assert_close(dev.get(hy), a + 0.5 * b, 1e-6, "add alpha")
    dev.cuda.mul(n, ha, hb, hy)
    assert np.array_equal(dev.get(hy), a * b)
    dev.cuda.scale(n, 3.0, ha, hy)
    assert np.array_equal(dev.get(hy), 3 * a)
    dev.cuda.scal(n, 0.25, hy)
    assert np.array_equal(dev.get(hy), 0.75 * a)
    dev.cuda.axpy(n, 2.0, hb, hy)
    assert_close(dev.get(hy), 0.75 * a + 2 * b, 1e-6, "axpy")
    dev.cuda.silu_fwd(n, ha, hy)
    assert_close(dev.get(hy), R.silu(a, np.float64), 1e-6, "silu")
    dev.cuda.SwigluForward(n, ha, hb, hy)
    assert_close(dev.get(hy), R.silu(a, np.float64) * b, 1e-6, "swiglu")
    dev.cuda.set(n, hy, 7.0)
    assert np.all(dev.get(hy) == 7)
    dev.cuda.set(1, hy, 9.0, 3)
    out = dev.get(hy)
    assert out[3] == 9 and out[2] == 7 and out[4] == 7


def test_embed_and_rmsnorm(dev):
    rng = np.random.default_rng(11)
    V, D = 50, 24
    W = rng.standard_normal((V, D)).astype(np.float32)
    ids = rng.integers(0, V, 13)
    hW, hi, ht = dev.put(W), dev.put(ids.astype(np.float32)), dev.zeros(13 * D)
    dev.cuda.embed_fwd(13 * D, hi, hW, 13, D, V, ht)
    assert np.array_equal(dev.get(ht, (13, D)), W[ids])
    x = rng.standard_normal((9, 288)).astype(np.float32)
    w = rng.standard_normal(288).astype(np.float32)
    hx, hw, hy = dev.put(x), dev.put(w), dev.zeros(x.size)
    dev.cuda.RmsNormForward(9, 288, hx, hw, hy, 1e-5)
    assert_close(dev.get(hy), R.rmsnorm_layer(x, w, 1e-5, np.float64), 1e-5, "rmsnorm")
    dev.cuda.RmsNormForward(9, 288, hx, 0, hy, 1e-5)
    assert_close(dev.get(hy), R.rmsnorm_layer(x, None, 1e-5, np.float64), 1e-5, "rmsnorm no weight")


@pytest.mark.parametrize("half", [False, True])
def test_whole_tensor_scal_is_deferred_without_changing_any_result(dev, half):
    """A SCAL over a large whole tensor is held back until the tensor is next touched (the mask calls fold it into their
    pass).  Whatever touches the tensor afterwards sees exactly what an immediate multiplication would have left."""
    rng = np.random.default_rng(71)
    cuda = dev.cuda
    n, md = 1 << 20, 4096
    x = bf16_round(rng.standard_normal(n).astype(np.float32))
    m = (rng.random(md) > 0.3).astype(np.float32)
    alpha = np.float32(0.125) if half else np.float32(0.3)
    scaled = bf16_round(x * alpha) if half else x * alpha
    hm = dev.put(m, half)

    def fresh():
        return dev.put(x, half)

    # read back
    h = fresh()
    cuda.scal(n, float(alpha), h)
    assert np.array_equal(dev.get(h), scaled)
    # mask in place: one pass
    h = fresh()
    cuda.scal(n, float(alpha), h)
    cuda.mask(n, md, 0.0, -1e29, h, hm, h)
    exp = np.where(np.tile(m, n // md) == 0, np.float32(-1e29), scaled)
    if half:
        exp = bf16_round(exp)
    assert np.array_equal(dev.get(h), exp)
    # mask_batch in place
    h = fresh()
    cuda.scal(n, float(alpha), h)
    mb = (rng.random(2 * md) > 0.3).astype(np.float32)
    hmb = dev.put(mb, half)
    cuda.mask_batch(n, 2, 2 * md, 0.0, -1e29, h, hmb, h)
    idx = np.arange(n) % md + (np.arange(n) // (n // 2)) * md
    exp = np.where(mb[idx] == 0, np.float32(-1e29), scaled)
    assert np.array_equal(dev.get(h), bf16_round(exp) if half else exp)
    # mask into another tensor: the source ends up scaled as well
    h, hy = fresh(), dev.zeros(n, half)
    cuda.scal(n, float(alpha), h)
    cuda.mask(n, md, 0.0, 7.0, h, hm, hy)
    assert np.array_equal(dev.get(hy), np.where(np.tile(m, n // md) == 0, np.float32(7.0), scaled))
    assert np.array_equal(dev.get(h), scaled)
    # two in a row, a copy, a memory pointer created afterwards, an element-wise consumer
    h, hc = fresh(), dev.zeros(n, half)
    cuda.scal(n, float(alpha), h)
    cuda.scal(n, 2.0, h)
    twice = bf16_round(scaled * np.float32(2.0)) if half else scaled * np.float32(2.0)
    cuda.copy(n, h, hc)
    assert np.array_equal(dev.get(hc), twice)
    h = fresh()
    cuda.scal(n, float(alpha), h)
    hv = cuda.CreateMemoryPointer(h, 16, 64)
    assert np.array_equal(dev.get(hv), scaled[16:80])
    # with a memory pointer alive the multiplication is immediate, and visible through the pointer
    cuda.scal(n, 2.0, h)
    assert np.array_equal(dev.get(hv), twice[16:80])
    cuda.FreeMemoryPointer(hv)
    h, hb = fresh(), dev.put(np.ones(n, np.float32), half)
    cuda.scal(n, float(alpha), h)
    cuda.mul(n, h, hb, hb)
    assert np.array_equal(dev.get(hb), scaled)
    # freed while the multiplication is still pending
    h = fresh()
    cuda.scal(n, float(alpha), h)
    cuda.FreeMemory(h)


def test_nothing_is_held_back_on_a_tensor_whose_device_address_was_handed_out(dev):
    """Internal_GetPointerFloat (CudaDnnDLL.cpp:57-75) gives an extension library the device address behind a memory
    handle, and the extension then reads that memory on its own: a SCAL and an in-place mask over such a tensor have
    to be in the stream when the call returns, where the same calls on an ordinary tensor wait for the next access."""
    import ctypes
    rng = np.random.default_rng(73)
    cuda = dev.cuda
    n, md = 1 << 20, 4096
    x = rng.standard_normal(n).astype(np.float32)
    m = (rng.random(md) > 0.3).astype(np.float32)
    h, hm = dev.put(x, False), dev.put(m, False)
    lib = cuda._lib
    lib.Internal_GetPointerFloat.argtypes = [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_void_p)]
    lib.Internal_GetPointerFloat.restype = ctypes.c_int32
    p = ctypes.c_void_p()
    assert lib.Internal_GetPointerFloat(0, cuda.m_hKernel, h, ctypes.byref(p)) == 0 and p.value
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    hip.hipMemcpy.restype = ctypes.c_int

    def raw():
        cuda.SynchronizeDevice()
        out = np.empty(n, np.float32)
        assert hip.hipMemcpy(out.ctypes.data, p, 4 * n, 2) == 0   # device to host, straight from the address
        return out

    assert np.array_equal(raw(), x)
    cuda.scal(n, 0.5, h)
    assert np.array_equal(raw(), x * np.float32(0.5))
    cuda.mask(n, md, 0.0, -1e29, h, hm, h)
    assert np.array_equal(raw(), np.where(np.tile(m, n // md) == 0, np.float32(-1e29), x * np.float32(0.5)))


def test_held_back_causal_mask_is_not_read_and_still_follows_the_mask_blob(dev):
    """A held-back (T,T) mask that keeps exactly the lower triangle is recognised once per content version: the
    softmax then reads neither the mask nor the scores above the diagonal.  Its output equals, bit for bit, that of the
    immediate calls (forced here by a memory pointer on the tensor, which rules out holding anything back), and a
    change to the mask blob is seen by the next call."""
    rng = np.random.default_rng(74)
    cuda = dev.cuda
    rows, T = 4096, 256
    n = rows * T
    x = (rng.standard_normal((rows, T)) * 4).astype(np.float32)
    tril = np.tril(np.ones((T, T), np.float32))
    alpha = np.float32(0.125)
    hm = dev.put(tril)
    hc, d = cuda.CreateCuDNN(), cuda.CreateTensorDesc()
    cuda.SetTensorDesc(d, rows, T, 1, 1, False)

    def run(immediate):
        h, hp = dev.put(x), dev.zeros(n)
        hv = cuda.CreateMemoryPointer(h, 0, n) if immediate else 0
        cuda.scal(n, float(alpha), h)
        cuda.mask(n, T * T, 0.0, -1e29, h, hm, h)
        cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, h, 0.0, d, hp)
        p, kept = dev.get(hp, x.shape), dev.get(h, x.shape)
        if hv:
            cuda.FreeMemoryPointer(hv)
        cuda.FreeMemory(h)
        cuda.FreeMemory(hp)
        return p, kept

    def expect(m):
        masked = np.where(np.tile(m, (rows // T, 1)) == 0, np.float32(-1e29), x * alpha)
        return masked, R.softmax_lastaxis(masked, np.float64)

    for m in (tril, None):
        if m is None:   # one more key kept in row 3 of the same blob: no longer a triangle
            m = tril.copy()
            m[3, 200] = 1.0
            cuda.SetMemory(hm, m)
        masked, want = expect(m)
        p_held, kept_held = run(False)
        p_now, kept_now = run(True)
        assert np.array_equal(p_held, p_now)
        assert np.array_equal(kept_held, masked) and np.array_equal(kept_now, masked)
        assert_close(p_held, want, FP32_RTOL, "softmax of the held-back causal mask")
    assert p_held[3, 200] > 0 and p_held[4, 200] == 0


@pytest.mark.parametrize("half", [False, True])
def test_in_place_mask_is_held_back_for_the_softmax_without_changing_any_result(dev, half):
    """An in-place mask call over a large whole tensor waits for the next call: a softmax forward over the tensor does
    mask, folded-in scaling and softmax in one pass; whatever else touches the tensor (or the mask blob) first sees
    exactly what the immediate call would have left; a MatMul that overwrites the tensor cancels it."""
    rng = np.random.default_rng(72)
    cuda = dev.cuda
    rows, length = 1024, 1024
    n = rows * length
    tol = BF16_RTOL if half else FP32_RTOL
    x = bf16_round(rng.standard_normal((rows, length)).astype(np.float32) * 4)
    tril = np.tril(np.ones((length, length), np.float32))
    alpha = np.float32(0.125)
    hm = dev.put(tril, half)
    hc, d = cuda.CreateCuDNN(), cuda.CreateTensorDesc()
    cuda.SetTensorDesc(d, rows, length, 1, 1, half)
    masked = np.where(tril == 0, np.float32(-1e29), x * alpha)
    if half:
        masked = bf16_round(masked)

    def prepared():
        h = dev.put(x, half)
        cuda.scal(n, float(alpha), h)
        cuda.mask(n, length * length, 0.0, -1e29, h, hm, h)
        return h

    # softmax straight after: one pass; the probabilities are those of the masked, scaled scores
    h, hp = prepared(), dev.zeros(n, half)
    cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, h, 0.0, d, hp)
    assert_close(dev.get(hp, x.shape), R.softmax_lastaxis(masked, np.float64), tol, "softmax of the held-back mask")
    # ... and the tensor itself, read afterwards, holds the masked scores
    assert np.array_equal(dev.get(h, x.shape), masked)
    # read back without a softmax
    h = prepared()
    assert np.array_equal(dev.get(h, x.shape), masked)
    # consumed by another call first
    h, hy = prepared(), dev.zeros(n, half)
    cuda.copy(n, h, hy)
    assert np.array_equal(dev.get(hy, x.shape), masked)
    # the mask blob changes before anything reads the tensor: the old mask values count
    hm2 = dev.put(tril, half)
    h = dev.put(x, half)
    cuda.mask(n, length * length, 0.0, -1e29, h, hm2, h)
    cuda.set(length * length, hm2, 1.0)
    exp = np.where(tril == 0, np.float32(-1e29), x)
    assert np.array_equal(dev.get(h, x.shape), bf16_round(exp) if half else exp)
    # the mask blob is freed first
    hm3 = dev.put(tril, half)
    h = dev.put(x, half)
    cuda.mask(n, length * length, 0.0, -1e29, h, hm3, h)
    cuda.FreeMemory(hm3)
    assert np.array_equal(dev.get(h, x.shape), bf16_round(exp) if half else exp)
    # two tensors in a row: the first call runs when the second arrives
    h1, h2 = dev.put(x, half), dev.put(x, half)
    cuda.mask(n, length * length, 0.0, -1e29, h1, hm, h1)
    cuda.mask(n, length * length, 0.0, 5.0, h2, hm, h2)
    assert np.array_equal(dev.get(h2, x.shape), np.where(tril == 0, np.float32(5.0), x))
    assert np.array_equal(dev.get(h1, x.shape), bf16_round(exp) if half else exp)
    # per-sequence masks (mask_batch), two sequences
    mb = (rng.random((2, length // 2, length)) > 0.3).astype(np.float32)
    hmb = dev.put(mb, half)
    h, hp = dev.put(x, half), dev.zeros(n, half)
    cuda.mask_batch(n, 2, mb.size, 0.0, -1e29, h, hmb, h)
    cuda.SoftmaxForward(hc, SOFTMAX_ALGORITHM.ACCURATE, SOFTMAX_MODE.INSTANCE, 1.0, d, h, 0.0, d, hp)
    mexp = np.where(mb.reshape(rows, length) == 0, np.float32(-1e29), x)
    assert_close(dev.get(hp, x.shape), R.softmax_lastaxis(mexp, np.float64), tol, "softmax of a held-back mask_batch")
    assert np.array_equal(dev.get(h, x.shape), bf16_round(mexp) if half else mexp)
    # freed while the mask call is outstanding
    h = prepared()
    cuda.FreeMemory(h)
    if not half:
        # a MatMul that rewrites the whole tensor cancels the call: (rows x 8) @ (8 x length)
        a, b = rng.standard_normal((1, 1, rows, 8)).astype(np.float32), rng.standard_normal((1, 1, 8, length)).astype(np.float32)
        ha, hb = dev.put(a), dev.put(b)
        h = prepared()
        cuda.matmul(1, rows, length, 8, ha, hb, h)
        assert_close(dev.get(h, x.shape), a[0, 0].astype(np.float64) @ b[0, 0].astype(np.float64), FP32_RTOL, "overwritten")
    cuda.FreeTensorDesc(d)
    cuda.FreeCuDNN(hc)


# ---- CAFFE-engine softmax chain: exp, log, channel_max / sub / div / dot ----------------------

@pytest.mark.parametrize("half", [False, True])
@pytest.mark.parametrize("num,ch,sp", [(5, 37, 19), (33, 200, 1), (7, 1024, 1), (9, 67, 1)])
def test_channel_primitives_of_the_softmax_chain(dev, half, num, ch, sp):
    """Channel axis in the middle, and as the last axis (spatial = 1: rows of consecutive values, which take the
    one-wavefront-a-row kernels from 64 channels on), with ties for the index of the maximum."""
    rng = np.random.default_rng(3)
    x = bf16_round(rng.standard_normal((num, ch, sp)).astype(np.float32))
    x[0, ch // 3] = x[0, ch - 1] = x[0].max(0) + 1        # equal maxima: the first index counts
    x[1, 0] = x[1, ch // 2] = x[1].max(0) + 1
    x = bf16_round(x)
    a = bf16_round(rng.standard_normal((num, ch, sp)).astype(np.float32))
    r = bf16_round((rng.random((num, sp)) + 0.5).astype(np.float32))
    tol = BF16_RTOL if half else 1e-6
    hx, ha, hr = dev.put(x, half), dev.put(a, half), dev.put(r, half)
    hy, hfull = dev.zeros(num * sp, half), dev.zeros(x.size, half)
    n, full = num * sp, x.size
    dev.cuda.channel_max(n, num, ch, sp, hx, hy)
    assert np.array_equal(dev.get(hy), R.channel_max(x, num, ch, sp))
    dev.cuda.channel_max(n, num, ch, sp, hx, hy, True)
    want_idx = R.channel_max(x, num, ch, sp, return_idx=True)
    assert np.array_equal(dev.get(hy), bf16_round(want_idx) if half else want_idx)     # the index is stored as a number
    dev.cuda.channel_max(n, num, 1, sp, hx, hy, False, False)                      # within-channel index rule
    assert np.array_equal(dev.get(hy), R.channel_max(x, num, 1, sp, across=False))
    dev.cuda.channel_sub(full, num, ch, sp, hr, hfull, ha)
    assert_close(dev.get(hfull), R.channel_sub(a, r, num, ch, sp), tol, "channel_sub a - x")
    dev.cuda.copy(full, hx, hfull)
    dev.cuda.channel_sub(full, num, ch, sp, hr, hfull)
    assert_close(dev.get(hfull), R.channel_sub(x, r, num, ch, sp), tol, "channel_sub in place")
    for method, count in ((1, full), (2, n)):
        dev.cuda.copy(full, hx, hfull)
        dev.cuda.channel_div(count, num, ch, sp, hr, hfull, method)
        assert_close(dev.get(hfull), R.channel_div(x, r, num, ch, sp), tol, "channel_div method %d" % method)
    # a partial count: method 1 divides the first `count` elements; method 2 would divide all channels of the first
    # `count` (n, s) pairs (math.cu:7171-7183), a different set, and is refused rather than silently run as method 1
    dev.cuda.copy(full, hx, hfull)
    part = (num - 1) * ch * sp
    dev.cuda.channel_div(part, num, ch, sp, hr, hfull, 1)
    want = R.channel_div(x, r, num, ch, sp).reshape(-1).copy()
    want[part:] = x.reshape(-1)[part:]
    assert_close(dev.get(hfull), want, tol, "channel_div method 1, partial count")
    with pytest.raises(CudaDnnError) as ei:
        dev.cuda.channel_div(n - sp, num, ch, sp, hr, hfull, 2)
    assert ei.value.code == ERROR.PARAM_OUT_OF_RANGE
    dev.cuda.copy(full, hx, hfull)
    part = (num - 1) * ch * sp - 3                       # not a whole number of rows
    dev.cuda.channel_sub(part, num, ch, sp, hr, hfull)
    want = R.channel_sub(x, r, num, ch, sp).reshape(-1).copy()
    want[part:] = x.reshape(-1)[part:]
    assert_close(dev.get(hfull), want, tol, "channel_sub in place, partial count")
    dev.cuda.channel_dot(n, num, ch, sp, hx, ha, hy)
    ref_dot = R.channel_dot(x, a, num, ch, sp)
    assert np.max(np.abs(dev.get(hy).reshape(ref_dot.shape) - ref_dot)) < (2e-2 if half else 1e-5) * np.sqrt(ch)
    dev.cuda.exp(full, hx, hfull, 0, 0, 0.5)
    assert_close(dev.get(hfull), np.exp(0.5 * x.astype(np.float64)).reshape(-1), tol, "exp")
    dev.cuda.log(n, hr, hy, 2.0, 0.25)
    assert_close(dev.get(hy), np.log(2.0 * (r.astype(np.float64) + 0.25)).reshape(-1), tol, "log")


@pytest.mark.parametrize("shape,axis", [((6, 50), -1), ((3, 4, 64, 64), -1), ((4, 9, 33), 1)])
@pytest.mark.parametrize("algorithm", ["ACCURATE", "LOG"])
def test_softmax_layer_caffe_engine_chain(dev, shape, axis, algorithm):
    """SoftmaxLayer with engine CAFFE (SoftmaxLayer.cs:230-330): forward against scipy and against the cuDNN-engine
    call (id 111), gradient of the ACCURATE form against the softmax gradient id (112)."""
    from scipy.special import log_softmax, softmax
    rng = np.random.default_rng(9)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    outs = {}
    for engine in ("CAFFE", "CUDNN"):
        if engine == "CUDNN" and algorithm == "LOG":
            continue
        layer = SoftmaxLayer(dev.cuda, axis, engine, algorithm)
        bottom, top = Blob(dev.cuda, shape), Blob(dev.cuda)
        bottom.mutable_cpu_data = x
        layer.Forward(bottom, top)
        y = top.mutable_cpu_data.copy()
        dx = None
        if algorithm == "ACCURATE":
            top.mutable_cpu_diff = dy
            layer.Backward(top, bottom)
            dx = bottom.mutable_cpu_diff.copy()
        outs[engine] = (y, dx)
    ref = (log_softmax if algorithm == "LOG" else softmax)(x.astype(np.float64), axis=axis)
    assert_close(outs["CAFFE"][0], ref, FP32_RTOL, "CAFFE-engine forward")
    assert_close(outs["CAFFE"][0], R.softmax_caffe_chain(x, axis, algorithm == "LOG"), 1e-6, "forward vs the checker's chain")
    if algorithm == "ACCURATE":
        assert_close(outs["CAFFE"][0], outs["CUDNN"][0], 1e-6, "CAFFE vs cuDNN engine forward")
        refdx = R.softmax_backward(ref, dy.astype(np.float64), axis=axis, dtype=np.float64)
        assert_close(outs["CAFFE"][1], refdx, FP32_RTOL, "CAFFE-engine gradient")
        assert_close(outs["CAFFE"][1], outs["CUDNN"][1], 1e-5, "CAFFE vs cuDNN engine gradient")
