"""The entry point that allocates nothing (MCH_AttnDecodeForwardNoAlloc) against the ordinary one
(ATTN_DECODE_FWD, id 2001): same arguments, split partials in the library's fixed device array.  Two calls in a
row, the second on a smaller input, so that whatever the first call left in the array is in the way of the second."""
import numpy as np
import pytest

from mycaffe_amd.cudadnn import CudaDnnError, ERROR
from oracle import attention_ref as R
from tests.conftest import BF16_RTOL, FP32_RTOL, assert_close, bf16_round

pytestmark = pytest.mark.gpu


def _case(dev, half, B, H, KVH, L, hs, seed, tag):
    rng = np.random.default_rng(seed)
    q = bf16_round(rng.standard_normal((B, H, hs)).astype(np.float32))
    k, v = (bf16_round(rng.standard_normal((B, KVH, L, hs)).astype(np.float32)) for _ in range(2))
    hq, hk, hv = dev.put(q, half), dev.put(k, half), dev.put(v, half)
    hy0, hy1 = dev.zeros(q.size, half), dev.zeros(q.size, half)
    print("no-alloc decode attention:", tag, "half" if half else "fp32", (B, H, KVH, L, hs), flush=True)
    dev.cuda.AttnDecodeForward(B, H, KVH, hs, L, hq, hk, hv, hy0, KVH * L * hs, L * hs, hs)
    dev.cuda.AttnDecodeForwardNoAlloc(B, H, KVH, hs, L, hq, hk, hv, hy1, KVH * L * hs, L * hs, hs)
    y0, y1 = dev.get(hy0, q.shape), dev.get(hy1, q.shape)
    # same kernels, same split plan: the two entry points agree to the bit
    assert np.array_equal(y0, y1), tag
    kk, vv = (np.repeat(a, H // KVH, axis=1) for a in (k, v))
    assert_close(y1, R.kv_cache_attention(q, kk, vv, np.float64), BF16_RTOL if half else FP32_RTOL, tag)


@pytest.mark.parametrize("half", [False, True])
def test_no_alloc_entry_point_matches_the_allocating_one_twice_in_a_row(dev, half):
    # first call: many splits per head (batch 1), 258-float partials; second: smaller cache, fewer heads, other head size
    _case(dev, half, 1, 32, 32, 2048, 128, 11, "first call")
    _case(dev, half, 2, 6, 3, 300, 64, 12, "second, smaller call")


def test_no_alloc_entry_point_with_rope_and_append(dev):
    rng = np.random.default_rng(5)
    B, H, L, hs, S = 2, 4, 40, 64, 64
    q = rng.standard_normal((B, H, hs)).astype(np.float32)
    kn, vn = (rng.standard_normal((B, H, hs)).astype(np.float32) for _ in range(2))
    kc = rng.standard_normal((B, H, S, hs)).astype(np.float32)
    vc = rng.standard_normal((B, H, S, hs)).astype(np.float32)
    hr = dev.cuda.CreateRope(0, 0, B * H * hs, B, S, H, hs, 10000.0)
    outs = []
    for fn in (dev.cuda.AttnDecodeForward, dev.cuda.AttnDecodeForwardNoAlloc):
        hq, hkn, hvn, hk, hv, hy = dev.put(q), dev.put(kn), dev.put(vn), dev.put(kc), dev.put(vc), dev.zeros(q.size)
        fn(B, H, H, hs, L, hq, hk, hv, hy, H * S * hs, S * hs, hs, 0.0, hr, hkn, hvn)
        outs.append((dev.get(hy, q.shape), dev.get(hk, kc.shape), dev.get(hv, vc.shape)))
    for a, b in zip(*outs):
        assert np.array_equal(a, b)


def test_no_alloc_entry_point_rejects_sizes_beyond_its_array(dev):
    # 4097 (batch x head) pairs: one more than the fixed array holds tickets for
    B, H, hs, L = 4097, 1, 8, 4
    hq, hk, hv, hy = dev.zeros(B * H * hs), dev.zeros(B * H * L * hs), dev.zeros(B * H * L * hs), dev.zeros(B * H * hs)
    with pytest.raises(CudaDnnError) as ei:
        dev.cuda.AttnDecodeForwardNoAlloc(B, H, H, hs, L, hq, hk, hv, hy, H * L * hs, L * hs, hs)
    assert ei.value.code == ERROR.PARAM_OUT_OF_RANGE
    assert "4096" in str(ei.value)
    # the ordinary entry point takes the same call
    dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq, hk, hv, hy, H * L * hs, L * hs, hs)


def test_no_alloc_entry_point_refuses_an_oversize_call_before_it_rotates_or_appends(dev):
    # 15-argument form (rotary embedding + new key / value) beyond the array's 4096 (batch x head) pairs: the refusal has
    # to come before the rotate-and-append kernel, or a caller that falls back to id 2001 would rotate q and k twice
    rng = np.random.default_rng(9)
    B, H, hs, L, S = 4097, 1, 8, 3, 4
    q = rng.standard_normal((B, H, hs)).astype(np.float32)
    kn, vn = (rng.standard_normal((B, H, hs)).astype(np.float32) for _ in range(2))
    kc, vc = (rng.standard_normal((B, H, S, hs)).astype(np.float32) for _ in range(2))
    hr = dev.cuda.CreateRope(0, 0, B * H * hs, B, S, H, hs, 10000.0)
    hq, hkn, hvn, hk, hv, hy = dev.put(q), dev.put(kn), dev.put(vn), dev.put(kc), dev.put(vc), dev.zeros(q.size)
    with pytest.raises(CudaDnnError) as ei:
        dev.cuda.AttnDecodeForwardNoAlloc(B, H, H, hs, L, hq, hk, hv, hy, H * S * hs, S * hs, hs, 0.0, hr, hkn, hvn)
    assert ei.value.code == ERROR.PARAM_OUT_OF_RANGE
    for h, ref, name in ((hq, q, "q"), (hkn, kn, "new key"), (hk, kc, "key cache"), (hv, vc, "value cache")):
        assert np.array_equal(dev.get(h, ref.shape), ref), name + " changed by a refused call"
    # the fallback the header names: the same call through id 2001 equals a fresh id 2001 call
    dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq, hk, hv, hy, H * S * hs, S * hs, hs, 0.0, hr, hkn, hvn)
    hq2, hkn2, hvn2, hk2, hv2, hy2 = dev.put(q), dev.put(kn), dev.put(vn), dev.put(kc), dev.put(vc), dev.zeros(q.size)
    dev.cuda.AttnDecodeForward(B, H, H, hs, L, hq2, hk2, hv2, hy2, H * S * hs, S * hs, hs, 0.0, hr, hkn2, hvn2)
    assert np.array_equal(dev.get(hy, q.shape), dev.get(hy2, q.shape))
