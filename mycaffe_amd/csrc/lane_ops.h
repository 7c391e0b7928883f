// Cross-lane exchanges of a 64-wide wavefront without the LDS crossbar: DPP inside a row of 16 lanes, the row-swapping
// permutes of gfx950 across rows.  A __shfl_xor step costs a lone wavefront some 50 ns (ds_bpermute round trip); these
// run at vector-ALU latency, which is what matters at the tail of kernels that are a few microseconds long.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mch {

template <int CTRL, int BANK> __device__ __forceinline__ uint32_t dpp_take(uint32_t old, uint32_t v)
{
    return __builtin_amdgcn_update_dpp(old, v, CTRL, 0xf, BANK, false);
}

// {a, b} = the lane's own value and that of lane ^ O (one bit of the lane index).  For O < 16, a is the own value; for
// O = 16 and 32 the two come out of a swap and which is which depends on the lane - use them symmetrically.
template <int O> __device__ __forceinline__ void lane_xor_pair(uint32_t v, uint32_t& a, uint32_t& b)
{
    static_assert(O == 1 || O == 2 || O == 4 || O == 8 || O == 16 || O == 32, "one bit of the lane index");
    a = v;
    if constexpr (O == 1) b = dpp_take<0xB1, 0xf>(0u, v);          // quad_perm [1,0,3,2]
    else if constexpr (O == 2) b = dpp_take<0x4E, 0xf>(0u, v);     // quad_perm [2,3,0,1]
    else if constexpr (O == 4) {
        // lanes 0-3 and 8-11 of a row take the lane four above (row_shl:4), the others the lane four below (row_shr:4)
        b = dpp_take<0x104, 0x5>(0u, v);
        b = dpp_take<0x114, 0xA>(b, v);
    } else if constexpr (O == 8) b = dpp_take<0x128, 0xf>(0u, v);  // row_ror:8
    else if constexpr (O == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);   // odd rows of one copy <-> even rows of the other
        a = r[0]; b = r[1];
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);   // upper half of one copy <-> lower half of the other
        a = r[0]; b = r[1];
    }
}

template <int O> __device__ __forceinline__ float add_lane_xor(float v)
{
    uint32_t a, b;
    lane_xor_pair<O>(__float_as_uint(v), a, b);
    return __uint_as_float(a) + __uint_as_float(b);
}

// Sum over each group of LPR adjacent lanes (a power of two), widest step first: the sums of the xor butterfly
// `for (o = LPR / 2; o > 0; o >>= 1) v += __shfl_xor(v, o)`, bit for bit, in every lane of the group.
template <int LPR> __device__ __forceinline__ float group_sum(float v)
{
    if constexpr (LPR >= 64) v = add_lane_xor<32>(v);
    if constexpr (LPR >= 32) v = add_lane_xor<16>(v);
    if constexpr (LPR >= 16) v = add_lane_xor<8>(v);
    if constexpr (LPR >= 8) v = add_lane_xor<4>(v);
    if constexpr (LPR >= 4) v = add_lane_xor<2>(v);
    if constexpr (LPR >= 2) v = add_lane_xor<1>(v);
    return v;
}

template <int O> __device__ __forceinline__ float max_lane_xor(float v)
{
    uint32_t a, b;
    lane_xor_pair<O>(__float_as_uint(v), a, b);
    return fmaxf(__uint_as_float(a), __uint_as_float(b));
}
// maximum over each group of LPR adjacent lanes, in every lane of the group
template <int LPR> __device__ __forceinline__ float group_max(float v)
{
    if constexpr (LPR >= 64) v = max_lane_xor<32>(v);
    if constexpr (LPR >= 32) v = max_lane_xor<16>(v);
    if constexpr (LPR >= 16) v = max_lane_xor<8>(v);
    if constexpr (LPR >= 8) v = max_lane_xor<4>(v);
    if constexpr (LPR >= 4) v = max_lane_xor<2>(v);
    if constexpr (LPR >= 2) v = max_lane_xor<1>(v);
    return v;
}

// Largest value of the wavefront with the smallest index among equals, in every lane.
template <int O> __device__ __forceinline__ void argmax_lane_xor(float& v, int& i)
{
    uint32_t va, vb, ia, ib;
    lane_xor_pair<O>(__float_as_uint(v), va, vb);
    lane_xor_pair<O>((uint32_t)i, ia, ib);
    const float fa = __uint_as_float(va), fb = __uint_as_float(vb);
    const bool takeB = fb > fa || (fb == fa && (int)ib < (int)ia);
    v = takeB ? fb : fa;
    i = takeB ? (int)ib : (int)ia;
}
__device__ __forceinline__ void wave_argmax_first(float& v, int& i)
{
    argmax_lane_xor<32>(v, i);
    argmax_lane_xor<16>(v, i);
    argmax_lane_xor<8>(v, i);
    argmax_lane_xor<4>(v, i);
    argmax_lane_xor<2>(v, i);
    argmax_lane_xor<1>(v, i);
}

}  // namespace mch
