// Fused scaled-dot-product attention forward for gfx950:
//   Y = softmax(mask(Q K^T * scale)) V   without materialising the (Tq,Tk) scores.
//
// Masked entries take the value -1e29 (not -inf), exactly like the reference's
// mask kernels: a fully masked row therefore yields the uniform distribution
// over all Tk keys, never NaN.
//
// Two implementations:
//  * attn_rows_kernel  - any head size / mask kind / Tq != Tk: one wavefront per
//    query row, lanes over keys, online softmax with wavefront reductions.
//  * flash kernels (attn_flash_*.inc) - MFMA tiles for hs in {64, 128}.
#include <stdlib.h>

#include "kernels.h"

namespace mch {

static constexpr float MASKED = -1e29f;

template <typename T> __device__ inline float ldp(const T* p, size_t i);
template <> __device__ inline float ldp<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ inline float ldp<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ inline void stp(T* p, size_t i, float v);
template <> __device__ inline void stp<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ inline void stp<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

struct AttnArgs {
    const void* q; const void* k; const void* v; void* y;
    const float* mask;
    int B, H, Tq, Tk, hs, kind;
    float scale;
};

// 4 wavefronts per workgroup, one query row each
template <typename T> __global__ __launch_bounds__(256) void attn_rows_kernel(AttnArgs a)
{
    constexpr int DPL = 4;  // hs <= 256
    __shared__ float qs[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;
    const int h = blockIdx.y, b = blockIdx.z;
    const bool valid = row < a.Tq;
    const size_t bh = (size_t)b * a.H + h;
    const T* q = (const T*)a.q + (bh * a.Tq + (valid ? row : 0)) * a.hs;
    const T* k = (const T*)a.k + bh * a.Tk * a.hs;
    const T* v = (const T*)a.v + bh * a.Tk * a.hs;
    for (int d = lane; d < a.hs; d += 64) qs[wave][d] = ldp(q, d) * a.scale;
    __syncthreads();
    if (!valid) return;
    // causal: keys beyond the row contribute exp(-1e29 - max) == 0 exactly, skip them
    const int kend = (a.kind == MASK_CAUSAL) ? min(a.Tk, row + 1) : a.Tk;
    float m = -INFINITY, l = 0.f, acc[DPL] = {0.f, 0.f, 0.f, 0.f};
    for (int kb = 0; kb < kend; kb += 64) {
        const int j = kb + lane;
        float s = -INFINITY;
        if (j < kend) {
            const T* kr = k + (size_t)j * a.hs;
            float d = 0.f;
            for (int i = 0; i < a.hs; i++) d += qs[wave][i] * ldp(kr, i);
            s = d;
            float mv = 1.f;
            if (a.kind == MASK_QK) mv = a.mask[(size_t)row * a.Tk + j];
            else if (a.kind == MASK_KEY) mv = a.mask[(size_t)b * a.Tk + j];
            else if (a.kind == MASK_BQK) mv = a.mask[((size_t)b * a.Tq + row) * a.Tk + j];
            if (mv == 0.f) s = MASKED;
        }
        float mx = s;
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float mn = fmaxf(m, mx);
        const float corr = __expf(m - mn);
        const float p = (j < kend) ? __expf(s - mn) : 0.f;
        float ps = p;
        for (int o = 32; o > 0; o >>= 1) ps += __shfl_xor(ps, o, 64);
        l = l * corr + ps;
        for (int i = 0; i < DPL; i++) acc[i] *= corr;
        const int cnt = min(64, kend - kb);
        for (int jj = 0; jj < cnt; jj++) {
            const float pj = __shfl(p, jj, 64);
            const T* vr = v + (size_t)(kb + jj) * a.hs;
            for (int i = 0; i < DPL; i++) {
                int d = lane + i * 64;
                if (d < a.hs) acc[i] += pj * ldp(vr, d);
            }
        }
        m = mn;
    }
    T* y = (T*)a.y + (bh * a.Tq + row) * a.hs;
    for (int i = 0; i < DPL; i++) {
        int d = lane + i * 64;
        if (d < a.hs) stp(y, d, acc[i] / l);
    }
}

hipError_t attn_flash_launch(hipStream_t s, DType dt, const AttnArgs& a, bool* handled);

hipError_t k_attn_prefill(hipStream_t s, DType dt, const void* q, const void* k, const void* v, void* y, int B, int H,
                          int Tq, int Tk, int hs, float scale, const float* mask, MaskKind kind)
{
    if (B <= 0 || H <= 0 || Tq <= 0 || Tk <= 0 || hs <= 0) return hipSuccess;
    if (B > 65535 || H > 65535) return hipErrorInvalidValue;
    if (kind != MASK_NONE && kind != MASK_CAUSAL && mask == nullptr) return hipErrorInvalidValue;
    AttnArgs a;
    a.q = q; a.k = k; a.v = v; a.y = y; a.mask = mask;
    a.B = B; a.H = H; a.Tq = Tq; a.Tk = Tk; a.hs = hs; a.kind = (int)kind; a.scale = scale;
    bool handled = false;
    hipError_t e = attn_flash_launch(s, dt, a, &handled);
    if (e != hipSuccess || handled) return e;
    if (hs > 256) return hipErrorInvalidValue;
    dim3 grid((Tq + 3) / 4, H, B);
    if (dt == F32) hipLaunchKernelGGL(attn_rows_kernel<float>, grid, 256, 0, s, a);
    else hipLaunchKernelGGL(attn_rows_kernel<bf16_t>, grid, 256, 0, s, a);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// MFMA flash attention, bf16 storage, head size 64.
//
// One workgroup = NW wavefronts; each wavefront owns QT tiles of 32 query rows and walks
// the keys in LDS blocks of 64, consumed as two 32-key online-softmax steps.  Per step:
//
//   S^T = K Q^T   v_mfma_f32_32x32x16_bf16, A = K rows from LDS (128-bit reads), B = Q
//                 fragments held in registers for the whole kernel.  Computing the
//                 TRANSPOSED scores puts one query per lane (lane%32) and its keys
//                 in that lane's accumulator registers, so the row max / row sum of
//                 the online softmax are in-register reductions plus ONE cross-lane
//                 exchange (lane ^ 32), and the per-row rescale factor is a per-lane
//                 scalar.
//   P^T           exp2 with the softmax scale folded into one fma per score, packed
//                 to bf16 in registers in exactly the order the next MFMA wants.
//   O^T += V^T P^T  A = V^T from LDS (V is transposed while it is stored to LDS, two
//                 64-bit reads per fragment), B = P^T from registers.
//
// K and V blocks are shared by the wavefronts of a workgroup through LDS and prefetched
// into registers one block ahead.  The kernel is bound by the softmax VALU work (about
// eight issue slots per score against 256 MFMA flops per score at head size 64), so the
// configuration is chosen for wavefronts per SIMD: that is what lets one wavefront's MFMAs
// run under another's exp2/fma/add stream.  Causal: key blocks past the workgroup's last
// row are never visited, wavefronts skip steps past their own rows, only diagonal steps
// pay for the element mask, and the heaviest query blocks are scheduled first.
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

struct FlashArgs {
    const bf16_t* q; const bf16_t* k; const bf16_t* v; bf16_t* y;
    const float* mask;   // (B, Tk) key mask for KIND 2
    int B, H, Tq, Tk;
    float c;             // softmax scale * log2(e)
    float maskedRaw;     // raw (unscaled) score that stands for the reference's -1e29
};

__device__ inline uint32_t pack_bf16x2(float a, float b)
{
    floatx2 f = {a, b};
    bf16x2 r = __builtin_convertvector(f, bf16x2);
    return *reinterpret_cast<uint32_t*>(&r);
}

// One 32-key online-softmax step for all query tiles of a wavefront, written as a single
// branch-free block (apart from the wavefront-uniform rescale test) so the tiles'
// dependency chains interleave.  MASKED: scores equal to `sentinel` stand for the
// reference's -1e29 fill; their weight is decided by comparison (1 while the row maximum
// is still the sentinel, else exactly 0) because exp2 of a difference of two huge
// products would not cancel exactly.
template <bool MASKED, int DT, int QT>
__device__ __forceinline__ void flash_softmax_step(floatx16 (&s)[QT], floatx16 (&o)[DT][QT], float (&m)[QT], float (&l)[QT],
                                                   bf16x8 (&pf)[QT][2], float c, float sentinel)
{
    float mx[QT], mnew[QT], alpha[QT], mc[QT];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        mx[qt] = s[qt][0];
#pragma unroll
        for (int v = 1; v < 16; v++) mx[qt] = fmaxf(mx[qt], s[qt][v]);
    }
#pragma unroll
    for (int qt = 0; qt < QT; qt++) mx[qt] = fmaxf(mx[qt], __shfl_xor(mx[qt], 32, 64));
    bool same = true;
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        mnew[qt] = fmaxf(m[qt], mx[qt]);
        alpha[qt] = __builtin_amdgcn_exp2f((m[qt] - mnew[qt]) * c);
        mc[qt] = mnew[qt] * c;
        m[qt] = mnew[qt];
        same = same && (alpha[qt] == 1.0f);
    }
    float p[QT][16];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        float rs = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            p[qt][v] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qt][v], c, -mc[qt]));
            if (MASKED && s[qt][v] == sentinel) p[qt][v] = (mnew[qt] == sentinel) ? 1.0f : 0.0f;
            rs += p[qt][v];
        }
        l[qt] = l[qt] * alpha[qt] + rs;
    }
    if (!__all(same)) {
#pragma unroll
        for (int qt = 0; qt < QT; qt++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int v = 0; v < 16; v++) o[dt][qt][v] *= alpha[qt];
    }
    // MFMA step t contracts the 16 keys held in registers 8t..8t+7
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; j++) w[j] = pack_bf16x2(p[qt][8 * t + 2 * j], p[qt][8 * t + 2 * j + 1]);
            pf[qt][t] = *reinterpret_cast<bf16x8*>(w);
        }
}

// KIND: 0 no mask, 1 causal, 2 per-key mask (B, Tk).  OCC: workgroups per CU the register budget is set for.
template <int KIND, int QT, int NW, int OCC>
__global__ __launch_bounds__(NW * 64, OCC) void flash_fwd_bf16_hs64_kernel(FlashArgs a)
{
    constexpr int HS = 64, NT = NW * 64, BM = NW * 32 * QT, BN = 64;
    constexpr int KS = HS / 16, DT = HS / 32;
    constexpr int LDK = HS + 8, LDV = BN + 8;
    constexpr int KPT = (BN * HS / 8) / NT;   // 16-byte K chunks per thread (512 chunks per block)
    constexpr int VPW = 8 / NW;               // 8-dim V chunks per wavefront
    static_assert(KPT >= 1 && VPW >= 1, "at most 8 wavefronts");
    __shared__ __attribute__((aligned(16))) bf16_t Ks[BN * LDK];
    __shared__ __attribute__((aligned(16))) bf16_t Vt[HS * LDV];
    __shared__ float Ms[BN];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int qblock = gridDim.x - 1 - blockIdx.x;   // heavy (late) query blocks first
    const int h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const int q0 = qblock * BM + wave * 32 * QT;      // first row of this wavefront
    const bf16_t* qp = a.q + bh * a.Tq * HS;
    const bf16_t* kp = a.k + bh * a.Tk * HS;
    const bf16_t* vp = a.v + bh * a.Tk * HS;

    // Q fragments: lane (query l32 of tile qt, half) holds dims 16*ks + 8*half .. +7
    bf16x8 qf[QT][KS];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        int row = min(q0 + qt * 32 + l32, a.Tq - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qf[qt][ks] = *(const bf16x8*)(qp + (size_t)row * HS + ks * 16 + half * 8);
    }
    floatx16 o[DT][QT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int qt = 0; qt < QT; qt++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[dt][qt][v] = 0.f;
    float m[QT], l[QT];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) { m[qt] = -INFINITY; l[qt] = 0.f; }

    int kend = a.Tk;
    if (KIND == 1) kend = min(a.Tk, qblock * BM + BM);
    const int nkb = (kend + BN - 1) / BN;

    // global -> register prefetch of one K / V block.  K: 8 threads per key row; V: one key per
    // lane and 8-dim chunks per wavefront, so that the transposing 16-bit LDS stores of a
    // wavefront hit consecutive addresses.
    uint4 kreg[KPT], vreg[VPW];
    auto gload = [&](int kb) {
        const int kbase = kb * BN;
#pragma unroll
        for (int i = 0; i < KPT; i++) {
            const int e = tid + i * NT;
            kreg[i] = *(const uint4*)(kp + (size_t)min(kbase + (e >> 3), a.Tk - 1) * HS + (e & 7) * 8);
        }
        const size_t vrow = (size_t)min(kbase + lane, a.Tk - 1) * HS;
#pragma unroll
        for (int i = 0; i < VPW; i++) vreg[i] = *(const uint4*)(vp + vrow + (wave + NW * i) * 8);
    };
    auto sstore = [&](int kb) {
#pragma unroll
        for (int i = 0; i < KPT; i++) {
            const int e = tid + i * NT;
            *(uint4*)(&Ks[(e >> 3) * LDK + (e & 7) * 8]) = kreg[i];
        }
#pragma unroll
        for (int i = 0; i < VPW; i++) {
            bf16_t* d = &Vt[(wave + NW * i) * 8 * LDV + lane];
            const uint4 r = vreg[i];
            d[0 * LDV] = (bf16_t)(r.x & 0xffffu); d[1 * LDV] = (bf16_t)(r.x >> 16);
            d[2 * LDV] = (bf16_t)(r.y & 0xffffu); d[3 * LDV] = (bf16_t)(r.y >> 16);
            d[4 * LDV] = (bf16_t)(r.z & 0xffffu); d[5 * LDV] = (bf16_t)(r.z >> 16);
            d[6 * LDV] = (bf16_t)(r.w & 0xffffu); d[7 * LDV] = (bf16_t)(r.w >> 16);
        }
        if (KIND == 2 && tid < BN) {
            const int key = kb * BN + tid;
            Ms[tid] = key < a.Tk ? a.mask[(size_t)b * a.Tk + key] : 1.f;
        }
    };

    gload(0);
    sstore(0);
    // make the Q fragments "used" here, so the wait for their loads sits before the loop and the
    // loop body never waits on the memory counter that the next block's prefetch shares
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int ks = 0; ks < KS; ks++) asm volatile("" : "+v"(qf[qt][ks]));
    __syncthreads();

    const float c = a.c;
    for (int kb = 0; kb < nkb; kb++) {
        if (kb + 1 < nkb) gload(kb + 1);
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            const int k0 = kb * BN + 32 * sub;
            // causal: this wavefront's last row is q0 + 32*QT - 1; keys past it contribute nothing
            const bool active = (KIND != 1) || (k0 <= q0 + 32 * QT - 1);
            if (active && k0 < a.Tk) {
                floatx16 s[QT];
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
#pragma unroll
                    for (int v = 0; v < 16; v++) s[qt][v] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    bf16x8 kf = *(const bf16x8*)(&Ks[(sub * 32 + l32) * LDK + ks * 16 + half * 8]);
#pragma unroll
                    for (int qt = 0; qt < QT; qt++) s[qt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[qt][ks], s[qt], 0, 0, 0);
                }
                // register v holds key k0 + 8*(v/4) + 4*half + v%4 for query q0 + 32*qt + l32
                const bool maskedBlock = ((KIND == 1) && (k0 + 31 > q0)) || (k0 + 32 > a.Tk) || KIND == 2;   // wavefront-uniform
                bf16x8 pf[QT][2];
                if (maskedBlock) {
#pragma unroll
                    for (int qt = 0; qt < QT; qt++) {
                        const int qrow = q0 + qt * 32 + l32;
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            const int kl = 8 * (v >> 2) + 4 * half + (v & 3);
                            const int key = k0 + kl;
                            float sv = s[qt][v];
                            if (KIND == 1 && key > qrow) sv = a.maskedRaw;
                            if (KIND == 2 && Ms[32 * sub + kl] == 0.f) sv = a.maskedRaw;
                            if (key >= a.Tk) sv = -INFINITY;
                            s[qt][v] = sv;
                        }
                    }
                    flash_softmax_step<true, DT, QT>(s, o, m, l, pf, c, a.maskedRaw);
                } else {
                    flash_softmax_step<false, DT, QT>(s, o, m, l, pf, c, a.maskedRaw);
                }
                // O^T += V^T P^T; slot j of step t is key 16t + 4*half + j (j < 4) or 16t + 8 + 4*half + j - 4
#pragma unroll
                for (int t = 0; t < 2; t++)
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        const bf16_t* vrow = &Vt[(dt * 32 + l32) * LDV + 32 * sub + 16 * t + 4 * half];
                        uint2 lo = *(const uint2*)vrow;
                        uint2 hi = *(const uint2*)(vrow + 8);
                        uint32_t w[4] = {lo.x, lo.y, hi.x, hi.y};
                        bf16x8 vf = *reinterpret_cast<bf16x8*>(w);
#pragma unroll
                        for (int qt = 0; qt < QT; qt++) o[dt][qt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[qt][t], o[dt][qt], 0, 0, 0);
                    }
            }
        }
        __syncthreads();
        if (kb + 1 < nkb) sstore(kb + 1);
        __syncthreads();
    }

    // epilogue: y[query, dim] = O^T[dim, query] / l; register v of tile dt is dim 32*dt + 8*(v/4) + 4*half + v%4
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        const int qrow = q0 + qt * 32 + l32;
        const float lt = l[qt] + __shfl_xor(l[qt], 32, 64);
        const float inv = 1.0f / lt;
        if (qrow < a.Tq) {
            bf16_t* yr = a.y + (bh * a.Tq + qrow) * HS;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    uint2 w;
                    w.x = pack_bf16x2(o[dt][qt][4 * g] * inv, o[dt][qt][4 * g + 1] * inv);
                    w.y = pack_bf16x2(o[dt][qt][4 * g + 2] * inv, o[dt][qt][4 * g + 3] * inv);
                    *(uint2*)(yr + 32 * dt + 8 * g + 4 * half) = w;
                }
        }
    }
}

template <int QT, int NW, int OCC>
static hipError_t flash_launch_cfg(hipStream_t s, const FlashArgs& f, int kind)
{
    constexpr int BM = NW * 32 * QT;
    dim3 grid((f.Tq + BM - 1) / BM, f.H, f.B);
    if (kind == MASK_NONE) hipLaunchKernelGGL((flash_fwd_bf16_hs64_kernel<0, QT, NW, OCC>), grid, NW * 64, 0, s, f);
    else if (kind == MASK_CAUSAL) hipLaunchKernelGGL((flash_fwd_bf16_hs64_kernel<1, QT, NW, OCC>), grid, NW * 64, 0, s, f);
    else hipLaunchKernelGGL((flash_fwd_bf16_hs64_kernel<2, QT, NW, OCC>), grid, NW * 64, 0, s, f);
    return hipGetLastError();
}

hipError_t attn_flash_launch(hipStream_t s, DType dt, const AttnArgs& a, bool* handled)
{
    *handled = false;
    if (dt != BF16 || a.hs != 64) return hipSuccess;
    if (a.kind != MASK_NONE && a.kind != MASK_CAUSAL && a.kind != MASK_KEY) return hipSuccess;
    if ((((uintptr_t)a.q | (uintptr_t)a.k | (uintptr_t)a.v | (uintptr_t)a.y) & 15) != 0) return hipSuccess;
    FlashArgs f;
    f.q = (const bf16_t*)a.q; f.k = (const bf16_t*)a.k; f.v = (const bf16_t*)a.v; f.y = (bf16_t*)a.y;
    f.mask = a.mask; f.B = a.B; f.H = a.H; f.Tq = a.Tq; f.Tk = a.Tk;
    f.c = a.scale * 1.4426950408889634f;
    f.maskedRaw = MASKED / a.scale;
    *handled = true;
    static int cfg = getenv("MCH_FLASH_CFG") ? atoi(getenv("MCH_FLASH_CFG")) : 0;
    switch (cfg) {
    case 1: return flash_launch_cfg<1, 4, 3>(s, f, a.kind);
    case 2: return flash_launch_cfg<1, 4, 4>(s, f, a.kind);
    case 3: return flash_launch_cfg<1, 8, 2>(s, f, a.kind);
    case 4: return flash_launch_cfg<2, 8, 1>(s, f, a.kind);
    case 5: return flash_launch_cfg<1, 8, 1>(s, f, a.kind);
    case 6: return flash_launch_cfg<2, 2, 4>(s, f, a.kind);
    default: return flash_launch_cfg<2, 4, 2>(s, f, a.kind);
    }
}

}  // namespace mch
