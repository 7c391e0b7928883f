// MFMA operand fragments shared by the attention forward and backward kernels (gfx950).
//
// One fragment is 16 bytes per lane.  bf16: v_mfma_f32_32x32x16_bf16, a fragment covers 16 contraction indices (lane half
// h holds 8 of them).  fp32: v_mfma_f32_32x32x2_f32 four times per fragment; lane half h holds indices 4h..4h+3 of an
// 8-index group and step e contracts the pair {e, 4+e}, which is legal because the slot-to-index assignment only has to
// agree between the A and the B operand.  Accumulator register v of a lane holds row 8*(v/4) + 4*(lane/32) + v%4,
// column lane%32 of the 32x32 result.
#pragma once
#include "kernels.h"

namespace mch {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // one 16-byte MFMA operand fragment

__device__ inline uint32_t pack_bf16x2(float a, float b)
{
    floatx2 f = {a, b};
    bf16x2 r = __builtin_convertvector(f, bf16x2);
    return *reinterpret_cast<uint32_t*>(&r);
}

// Transposing LDS read of gfx950 (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane i supplies the address of
// four consecutive 16-bit elements; the 64 elements form a 4 x 16 matrix whose row r comes from lanes 4r .. 4r+3, and
// lane c of the group receives column c: {row 0, row 1, row 2, row 3}[c].  A row-major [key][dim] tile is thus read as
// the [dim][key] fragments the matrix cores want without ever being stored transposed.
typedef short short4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint2 lds_read_tr16(const bf16_t* p)
{
    const short4v r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4v __attribute__((address_space(3)))*)(p));
    return *reinterpret_cast<const uint2*>(&r);
}

template <typename T> struct FlashTraits;
template <> struct FlashTraits<bf16_t> {
    static constexpr int EPC = 8;    // elements per 16-byte chunk
    static constexpr int CPF = 16;   // contraction indices covered by one fragment (both lane halves)
    __device__ static inline floatx16 mma(u32x4 a, u32x4 b, floatx16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8*>(&a), *reinterpret_cast<bf16x8*>(&b), c, 0, 0, 0);
    }
    // V^T fragment t of a 32-key step: keys 16t + 4h .. +3 and 16t + 8 + 4h .. +3
    __device__ static inline u32x4 load_vt(const bf16_t* row, int t, int half)
    {
        const bf16_t* p = row + 16 * t + 4 * half;
        uint2 lo = *(const uint2*)p, hi = *(const uint2*)(p + 8);
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    }
    // The same fragment from a ROW-MAJOR [key][dim] tile (row stride ld elements): `tile` points at key 0, first dim of
    // the 32-dim tile.  Lane (group g = lane / 16, i = lane % 16) supplies row 4 half + i / 4 of the four-key run, dims
    // 16 (g & 1) + 4 (i % 4) .. + 3, and receives its own dim lane % 32 for the four keys; the second read is the run
    // eight keys further on.
    __device__ static inline u32x4 load_vt_rowmajor(const bf16_t* tile, int ld, int t, int lane)
    {
        const int i = lane & 15, half = lane >> 5;
        const bf16_t* p = tile + (16 * t + 4 * half + (i >> 2)) * ld + 16 * ((lane >> 4) & 1) + 4 * (i & 3);
        const uint2 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 8 * ld);
        return u32x4{lo.x, lo.y, hi.x, hi.y};
    }
    // P^T fragment t: the weights held in accumulator registers 8t .. 8t+7
    __device__ static inline u32x4 pack_p(const floatx16& p, int t)
    {
        return u32x4{pack_bf16x2(p[8 * t], p[8 * t + 1]), pack_bf16x2(p[8 * t + 2], p[8 * t + 3]),
                     pack_bf16x2(p[8 * t + 4], p[8 * t + 5]), pack_bf16x2(p[8 * t + 6], p[8 * t + 7])};
    }
    // sum of the eight products of two fragments
    __device__ static inline float dot(u32x4 a, u32x4 b)
    {
        float r = 0.f;
        const uint32_t av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r += __uint_as_float(av[i] << 16) * __uint_as_float(bv[i] << 16);
            r += __uint_as_float(av[i] & 0xffff0000u) * __uint_as_float(bv[i] & 0xffff0000u);
        }
        return r;
    }
    __device__ static inline void store4(bf16_t* dst, float a, float b, float c, float d)
    {
        uint2 w;
        w.x = pack_bf16x2(a, b);
        w.y = pack_bf16x2(c, d);
        *(uint2*)dst = w;
    }
    __device__ static inline void scatter_chunk(bf16_t* d, int ld, u32x4 r)
    {
        d[0 * ld] = (bf16_t)(r.x & 0xffffu); d[1 * ld] = (bf16_t)(r.x >> 16);
        d[2 * ld] = (bf16_t)(r.y & 0xffffu); d[3 * ld] = (bf16_t)(r.y >> 16);
        d[4 * ld] = (bf16_t)(r.z & 0xffffu); d[5 * ld] = (bf16_t)(r.z >> 16);
        d[6 * ld] = (bf16_t)(r.w & 0xffffu); d[7 * ld] = (bf16_t)(r.w >> 16);
    }
};
template <> struct FlashTraits<float> {
    static constexpr int EPC = 4;
    static constexpr int CPF = 8;
    __device__ static inline floatx16 mma(u32x4 a, u32x4 b, floatx16 c)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
        return c;
    }
    // V^T fragment t of a 32-key step: keys 8t + 4h .. +3
    __device__ static inline u32x4 load_vt(const float* row, int t, int half) { return *(const u32x4*)(row + 8 * t + 4 * half); }
    __device__ static inline u32x4 load_vt_rowmajor(const float*, int, int, int) { return u32x4{0u, 0u, 0u, 0u}; }   // 16-bit storage only
    // P^T fragment t: the weights held in accumulator registers 4t .. 4t+3
    __device__ static inline u32x4 pack_p(const floatx16& p, int t)
    {
        return u32x4{__float_as_uint(p[4 * t]), __float_as_uint(p[4 * t + 1]), __float_as_uint(p[4 * t + 2]),
                     __float_as_uint(p[4 * t + 3])};
    }
    __device__ static inline float dot(u32x4 a, u32x4 b)
    {
        return __uint_as_float(a.x) * __uint_as_float(b.x) + __uint_as_float(a.y) * __uint_as_float(b.y) +
               __uint_as_float(a.z) * __uint_as_float(b.z) + __uint_as_float(a.w) * __uint_as_float(b.w);
    }
    __device__ static inline void store4(float* dst, float a, float b, float c, float d) { *(float4*)dst = make_float4(a, b, c, d); }
    __device__ static inline void scatter_chunk(float* d, int ld, u32x4 r)
    {
        d[0 * ld] = __uint_as_float(r.x); d[1 * ld] = __uint_as_float(r.y);
        d[2 * ld] = __uint_as_float(r.z); d[3 * ld] = __uint_as_float(r.w);
    }
};

// offset of output row `row` of head (b, h) in y
__device__ __forceinline__ size_t attn_y_row(int yMerged, int b, int h, int H, int Tq, int row, int hs)
{
    return yMerged ? (((size_t)b * Tq + row) * H + h) * hs : (((size_t)b * H + h) * Tq + row) * hs;
}

// arguments of the matrix-core attention forward kernels (attn_prefill.hip, attn_flash2.hip)
struct FlashArgs {
    const void* q; const void* k; const void* v; void* y;
    const float* mask;   // (B, Tk) key mask for KIND 2, (B, Tq, Tk) mask for KIND 3
    int maskBatch;       // KIND 3: 1 = one (Tq, Tk) mask per sequence, 0 = one mask shared by all sequences
    int B, H, Tq, Tk;
    float c;             // softmax scale * log2(e)
    float maskedRaw;     // raw (unscaled) score that stands for the reference's -1e29
    float lazy;          // raw-score slack of the running maximum: 8 / c, so weights stay below 2^8
    float* lse2;         // optional [B*H*Tq]: log2 of the softmax denominator of every row, kept for the backward pass
    int yMerged;         // y laid out (B,Tq,H,hs) instead of (B,H,Tq,hs)
    int causalGroup;     // causal launches: heads per group of the workgroup order (0: all heads in one group)
};

// Rank of a workgroup of a causal launch in the heaviest-first order.  Workgroup i goes to XCD i % 8 and, within it, the
// first launches land on its 32 CUs in turn, `occ` rounds of 32 before the XCD is full.  A CU keeps what it was given in
// those rounds, so every second one of them is walked backwards: the CU that got the heaviest block of one round gets
// the lightest of the next.  Later rounds start as slots free up, where plain heaviest-first is the better order.
// Ranks stay congruent to the workgroup index mod 8 (same XCD, same L2).
__device__ __forceinline__ int flash_causal_rank(int occ)
{
    if ((gridDim.x & 7) != 0) return (int)blockIdx.x;
    const int x = blockIdx.x & 7, j = blockIdx.x >> 3, per = gridDim.x >> 3;
    if (occ == 2 && per > 32 && per < 64) {
        // Less than two rounds: the XCD's CUs 0 .. per - 33 get a second workgroup, the others stay alone.  The heaviest
        // blocks go to the CUs that stay alone; the paired CUs take the next heaviest, and as partners the lightest ones,
        // lightest to the heaviest - so that no CU holds much more than the heaviest single block.
        const int nPair = per - 32, nLone = 32 - nPair;
        const int r = j >= 32 ? per - 1 - (j - 32) : j >= nPair ? j - nPair : nLone + j;
        return (r << 3) + x;
    }
    const int r = j >> 5, c = j & 31;
    if (!(r & 1) || r >= occ) return (int)blockIdx.x;
    const int rest = per - (r << 5);
    const int width = rest < 32 ? rest : 32;   // the last round may be short
    return (((r << 5) + width - 1 - c) << 3) + x;
}

// (query block, head index) of rank r of a causal launch.  Heads are taken in groups of `group` (a multiple of 8, so a
// head keeps its die): within a group heaviest query block first across the group's heads, then the next group.  Fewer
// heads in flight at a time keep their K and V in the caches while their query blocks run; with at most four groups the
// last group's heaviest blocks still start early enough not to stick out at the end.  group >= nbh is the plain
// heaviest-first order over all heads.
__device__ __forceinline__ void flash_causal_map(int rank, int nbh, int nqb, int group, int* qblock, int* ibh)
{
    if (group <= 0 || group >= nbh) {
        *qblock = nqb - 1 - rank / nbh;
        *ibh = rank % nbh;
        return;
    }
    const int per = group * nqb;
    const int g = rank / per, r = rank - g * per;
    const int width = min(group, nbh - g * group);   // the last group may be short
    *qblock = nqb - 1 - r / width;
    *ibh = g * group + r % width;
}

}  // namespace mch
