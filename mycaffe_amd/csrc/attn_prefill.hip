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

#include <type_traits>

#include "flash_traits.h"
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
    float* lse2;   // optional [B*H*Tq]: log2 of the row's softmax denominator (-inf marks a fully masked row)
    int yMerged;   // 1: y is written head-merged, (B,Tq,H,hs), the layout the output projection reads; 0: (B,H,Tq,hs)
    int useDropout;
    AttnDropout drop;
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
        // dropout acts on the normalised probabilities: the denominator keeps every key, the output only the survivors
        float pd = p;
        if (a.useDropout && j < kend)
            pd = attn_dropout_keep(a.drop.seed, (uint64_t)(bh * a.Tq + row) * a.Tk + j, a.drop.threshold) ? p * a.drop.keepScale : 0.f;
        const int cnt = min(64, kend - kb);
        for (int jj = 0; jj < cnt; jj++) {
            const float pj = __shfl(pd, jj, 64);
            const T* vr = v + (size_t)(kb + jj) * a.hs;
            for (int i = 0; i < DPL; i++) {
                int d = lane + i * 64;
                if (d < a.hs) acc[i] += pj * ldp(vr, d);
            }
        }
        m = mn;
    }
    T* y = (T*)a.y + attn_y_row(a.yMerged, b, h, a.H, a.Tq, row, a.hs);
    for (int i = 0; i < DPL; i++) {
        int d = lane + i * 64;
        if (d < a.hs) stp(y, d, acc[i] / l);
    }
    // a causal row's maximum is never the fill value, so the shortened key range above changes nothing here
    if (a.lse2 && lane == 0) a.lse2[bh * a.Tq + row] = (m == MASKED) ? -INFINITY : (m + __logf(l)) * 1.4426950408889634f;
}

hipError_t attn_flash_launch(hipStream_t s, DType dt, const AttnArgs& a, bool* handled);
hipError_t attn_flash2_launch(hipStream_t s, const FlashArgs& f, int hs, bool causal, bool* handled);

hipError_t k_attn_prefill(hipStream_t s, DType dt, const void* q, const void* k, const void* v, void* y, int B, int H,
                          int Tq, int Tk, int hs, float scale, const float* mask, MaskKind kind, float* lse2, bool yMerged,
                          const AttnDropout* dropout)
{
    if (B <= 0 || H <= 0 || Tq <= 0 || Tk <= 0 || hs <= 0) return hipSuccess;
    if (B > 65535 || H > 65535) return hipErrorInvalidValue;
    if (kind != MASK_NONE && kind != MASK_CAUSAL && mask == nullptr) return hipErrorInvalidValue;
    AttnArgs a;
    a.q = q; a.k = k; a.v = v; a.y = y; a.mask = mask;
    a.B = B; a.H = H; a.Tq = Tq; a.Tk = Tk; a.hs = hs; a.kind = (int)kind; a.scale = scale; a.lse2 = lse2;
    a.yMerged = yMerged ? 1 : 0;
    a.useDropout = dropout ? 1 : 0;
    if (dropout) a.drop = *dropout;
    bool handled = false;
    if (!dropout) {   // the matrix-core kernels have no dropout: training with a non-zero ratio takes the row kernel
        hipError_t e = attn_flash_launch(s, dt, a, &handled);
        if (e != hipSuccess || handled) return e;
    }
    if (hs > 256) return hipErrorInvalidValue;
    dim3 grid((Tq + 3) / 4, H, B);
    if (dt == F32) hipLaunchKernelGGL(attn_rows_kernel<float>, grid, 256, 0, s, a);
    else hipLaunchKernelGGL(attn_rows_kernel<bf16_t>, grid, 256, 0, s, a);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// MFMA flash attention for head sizes 64 and 128, bf16 and fp32 storage.
//
// One workgroup = NW wavefronts; each wavefront owns QT tiles of 32 query rows and walks
// the keys in LDS blocks of 64, consumed as two 32-key online-softmax steps.  Per step:
//
//   S^T = K Q^T   A = K rows from LDS (128-bit reads), B = Q fragments held in registers for
//                 the whole kernel.  Computing the TRANSPOSED scores puts one query per
//                 lane (lane%32) and its keys in that lane's accumulator registers, so the
//                 row max / row sum of the online softmax are in-register reductions plus
//                 ONE cross-lane exchange (lane ^ 32), and the per-row rescale factor is a
//                 per-lane scalar.
//   P^T           exp2 with the softmax scale folded into one fma per score; for bf16 the
//                 weights are packed in registers in exactly the order the next MFMA wants.
//   O^T += V^T P^T  A = V^T from LDS (V is transposed while it is stored to LDS), B = P^T
//                 straight from registers.
//
// bf16 uses v_mfma_f32_32x32x16_bf16 (a 16-byte fragment per lane covers 16 contraction
// indices); fp32 uses v_mfma_f32_32x32x2_f32 four times per 16-byte fragment: lane half h
// holds indices 4h..4h+3 of an 8-index group and step e contracts the pair {e, 4+e}, which
// is legal because the slot-to-index assignment only has to agree between A and B.
//
// The bf16 kernel is bound by the softmax VALU work (v_exp_f32 is quarter rate: about 27
// cycles per score against 8 MFMA cycles per score at head size 64); the fp32 kernel is
// MFMA bound.  Causal: key blocks past the workgroup's last row are never visited,
// wavefronts skip steps past their own rows, only diagonal steps pay for the element mask,
// and workgroups are launched heaviest query block first across all heads.

__device__ __forceinline__ float flash_half_max(float v)
{
    // v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// One 32-key online-softmax step for all query tiles of a wavefront, written as a single
// branch-free block (apart from the wavefront-uniform rescale test) so the tiles'
// dependency chains interleave.  On return s holds the weights p.  MASKED: scores equal to
// `sentinel` stand for the reference's -1e29 fill; their weight is decided by comparison (1
// while the row maximum is still the sentinel, else exactly 0) because exp2 of a difference
// of two huge products would not cancel exactly.
template <bool MASKED, int DT, int QT>
__device__ __forceinline__ void flash_softmax_step(floatx16 (&s)[QT], floatx16 (&o)[DT][QT], float (&m)[QT], float (&l)[QT],
                                                   float c, float sentinel, float lazy)
{
    float mx[QT], mnew[QT], alpha[QT], mc[QT];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        mx[qt] = s[qt][0];
#pragma unroll
        for (int v = 1; v < 16; v++) mx[qt] = fmaxf(mx[qt], s[qt][v]);
    }
    // the other lane half's maximum comes through a register swap, not a trip through LDS
#pragma unroll
    for (int qt = 0; qt < QT; qt++) mx[qt] = flash_half_max(mx[qt]);
    bool same = true;
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        // the reference maximum only moves when a score exceeds it by more than the slack: weights are then
        // at most 2^8 (exact in the final normalisation, since l uses the same reference) and the rescale of
        // the output accumulators below is skipped on most steps
        mnew[qt] = (mx[qt] > m[qt] + lazy) ? mx[qt] : m[qt];
        alpha[qt] = __builtin_amdgcn_exp2f((m[qt] - mnew[qt]) * c);
        mc[qt] = mnew[qt] * c;
        m[qt] = mnew[qt];
        same = same && (alpha[qt] == 1.0f);
    }
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        float rs = 0.f;
#pragma unroll
        for (int v = 0; v < 16; v++) {
            float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qt][v], c, -mc[qt]));
            if (MASKED && s[qt][v] == sentinel) pv = (mnew[qt] == sentinel) ? 1.0f : 0.0f;
            s[qt][v] = pv;
            rs += pv;
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
}

// KIND: 0 no mask, 1 causal, 2 per-key mask (B, Tk), 3 per-sequence mask (B, Tq, Tk).  OCC: workgroups per CU the register budget is set for.
// PREFETCH: hold the next K / V block in registers while computing on the current one.
template <typename T, int HS, int KIND, int QT, int NW, int OCC, bool PREFETCH>
__global__ __launch_bounds__(NW * 64, OCC) void flash_fwd_kernel(FlashArgs a)
{
    typedef FlashTraits<T> TR;
    constexpr int NT = NW * 64, BM = NW * 32 * QT, BN = 64;
    constexpr int EPC = TR::EPC, CPF = TR::CPF;
    constexpr int KF = HS / CPF;              // fragments along the head dimension (S^T contraction)
    constexpr int PF = 32 / CPF;              // fragments along a 32-key step (P V contraction)
    constexpr int DT = HS / 32;
    constexpr int PAD = 16 / (int)sizeof(T);
    constexpr int LDK = HS + PAD, LDV = BN + PAD;
    // Row stride of the row-major V tile.  The transposing read takes 32 contiguous bytes from each of four rows per
    // 16 lanes, so rows must start 8 banks (32 bytes) apart modulo the bank count: 144 bytes (head size 64) does, 272
    // (head size 128 with the K padding) puts neighbouring rows 4 banks apart and halves the read rate; 288 does not.
    constexpr int LDVR = (HS * (int)sizeof(T)) % 256 == 0 ? HS + 2 * PAD : HS + PAD;
    constexpr int CHR = HS / EPC;             // 16-byte chunks per K / V row
    constexpr int KPT = (BN * CHR) / NT;      // K chunks per thread per block
    // 16-bit storage keeps V row-major in LDS, staged exactly like K, and reads the V^T fragments with the transposing
    // LDS read; fp32 stores V transposed (4-byte scatter stores, which do not collide)
    constexpr bool VROW = sizeof(T) == 2;
    constexpr int VPW = VROW ? KPT : CHR / NW;   // V chunks per thread (row-major) / per wavefront, one key per lane (transposed)
    static_assert(KPT >= 1 && VPW >= 1 && (BN * CHR) % NT == 0 && (VROW || CHR % NW == 0), "tile / thread mismatch");
    __shared__ __attribute__((aligned(16))) T Ks[BN * LDK];
    __shared__ __attribute__((aligned(16))) T Vt[VROW ? BN * LDVR : HS * LDV];
    __shared__ float Ms[BN];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    // Causal work grows with the query block, so the launch is one-dimensional and ordered heaviest block
    // first across ALL (batch, head) pairs: workgroups are dispatched in index order as slots free up, which
    // makes the hardware dispatcher a longest-job-first scheduler.  Consecutive indices share a query block
    // and differ in (batch, head), so with B*H a multiple of 8 every head's blocks land on one XCD's L2.
    int qblock, h, b;
    if (KIND == 1) {
        const int nbh = a.B * a.H;
        const int nqb = (a.Tq + BM - 1) / BM;
        const int rank = flash_causal_rank(OCC);
        int ibh;
        flash_causal_map(rank, nbh, nqb, a.causalGroup, &qblock, &ibh);
        b = ibh / a.H;
        h = ibh % a.H;
    } else {
        qblock = blockIdx.x;
        h = blockIdx.y;
        b = blockIdx.z;
    }
    const size_t bh = (size_t)b * a.H + h;
    const int q0 = qblock * BM + wave * 32 * QT;      // first row of this wavefront
    const T* qp = (const T*)a.q + bh * a.Tq * HS;
    const T* kp = (const T*)a.k + bh * a.Tk * HS;
    const T* vp = (const T*)a.v + bh * a.Tk * HS;

    // Q fragments: lane (query l32 of tile qt, half) holds elements f*CPF + half*CPF/2 .. of its row
    u32x4 qf[QT][KF];
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        int row = min(q0 + qt * 32 + l32, a.Tq - 1);
#pragma unroll
        for (int f = 0; f < KF; f++) qf[qt][f] = *(const u32x4*)(qp + (size_t)row * HS + f * CPF + half * (CPF / 2));
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

    // global -> (register ->) LDS movement of one K / V block.  K: consecutive threads take
    // consecutive 16-byte chunks; V: one key per lane and whole chunks per wavefront, so that the
    // transposing LDS stores of a wavefront hit consecutive addresses.
    u32x4 kreg[KPT], vreg[VPW];
    auto gload = [&](int kb) {
        const int kbase = kb * BN;
#pragma unroll
        for (int i = 0; i < KPT; i++) {
            const int e = tid + i * NT;
            kreg[i] = *(const u32x4*)(kp + (size_t)min(kbase + e / CHR, a.Tk - 1) * HS + (e % CHR) * EPC);
        }
        if (VROW) {
#pragma unroll
            for (int i = 0; i < VPW; i++) {
                const int e = tid + i * NT;
                vreg[i] = *(const u32x4*)(vp + (size_t)min(kbase + e / CHR, a.Tk - 1) * HS + (e % CHR) * EPC);
            }
        } else {
            const size_t vrow = (size_t)min(kbase + lane, a.Tk - 1) * HS;
#pragma unroll
            for (int i = 0; i < VPW; i++) vreg[i] = *(const u32x4*)(vp + vrow + (wave + NW * i) * EPC);
        }
    };
    auto sstore = [&](int kb) {
#pragma unroll
        for (int i = 0; i < KPT; i++) {
            const int e = tid + i * NT;
            *(u32x4*)(&Ks[(e / CHR) * LDK + (e % CHR) * EPC]) = kreg[i];
        }
        if (VROW) {
#pragma unroll
            for (int i = 0; i < VPW; i++) {
                const int e = tid + i * NT;
                *(u32x4*)(&Vt[(e / CHR) * LDVR + (e % CHR) * EPC]) = vreg[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < VPW; i++) TR::scatter_chunk(&Vt[(wave + NW * i) * EPC * LDV + lane], LDV, vreg[i]);
        }
        if (KIND == 2 && tid < BN) {
            const int key = kb * BN + tid;
            Ms[tid] = key < a.Tk ? a.mask[(size_t)b * a.Tk + key] : 1.f;
        }
    };

    // Key-padding masks: a 32-key step whose keys are all masked adds exact zeros once the sequence has a valid key
    // anywhere (its weights underflow against any real maximum), so such steps are skipped, and steps without a masked
    // key take the unmasked path.  A sequence with no valid key at all keeps every step (uniform weights, as the
    // reference's -1e29 fill gives).
    bool seqValid = false;
    gload(0);   // requested before the mask scan, so that the two trips to memory overlap
    if (KIND == 2) {
        int any = 0;
        for (int t = tid; t < a.Tk; t += NT) any |= a.mask[(size_t)b * a.Tk + t] != 0.f;
        seqValid = __syncthreads_or(any) != 0;
    }
    sstore(0);
    // make the Q fragments "used" here, so the wait for their loads sits before the loop and the
    // loop body never waits on the memory counter that the next block's prefetch shares
#pragma unroll
    for (int qt = 0; qt < QT; qt++)
#pragma unroll
        for (int f = 0; f < KF; f++) asm volatile("" : "+v"(qf[qt][f]));
    __syncthreads();

    const float c = a.c;
    for (int kb = 0; kb < nkb; kb++) {
        if (PREFETCH && kb + 1 < nkb) gload(kb + 1);
        unsigned long long zeros = 0;      // bit = key of this block is masked (KIND 2)
        if (KIND == 2) zeros = __ballot(Ms[lane] == 0.f);
#pragma unroll
        for (int sub = 0; sub < 2; sub++) {
            const int k0 = kb * BN + 32 * sub;
            // causal: this wavefront's last row is q0 + 32*QT - 1; keys past it contribute nothing
            const bool active = (KIND != 1) || (k0 <= q0 + 32 * QT - 1);
            const unsigned subZeros = (unsigned)(zeros >> (32 * sub));
            const bool skip = KIND == 2 && seqValid && subZeros == 0xffffffffu;
            if (active && k0 < a.Tk && !skip) {
                floatx16 s[QT];
#pragma unroll
                for (int qt = 0; qt < QT; qt++)
#pragma unroll
                    for (int v = 0; v < 16; v++) s[qt][v] = 0.f;
#pragma unroll
                for (int f = 0; f < KF; f++) {
                    const u32x4 kf = *(const u32x4*)(&Ks[(sub * 32 + l32) * LDK + f * CPF + half * (CPF / 2)]);
#pragma unroll
                    for (int qt = 0; qt < QT; qt++) s[qt] = TR::mma(kf, qf[qt][f], s[qt]);
                }
                // register v holds key k0 + 8*(v/4) + 4*half + v%4 for query q0 + 32*qt + l32
                const bool maskedBlock = ((KIND == 1) && (k0 + 31 > q0)) || (k0 + 32 > a.Tk) || KIND == 3 ||
                                         (KIND == 2 && subZeros != 0);   // wavefront-uniform
                if (maskedBlock) {
#pragma unroll
                    for (int qt = 0; qt < QT; qt++) {
                        const int qrow = q0 + qt * 32 + l32;
                        // KIND 3: the lane's 16 keys are four runs of four; with whole, aligned runs each is one
                        // 16-byte load of the mask row instead of four scalar ones
                        float mk[16];
                        if (KIND == 3) {
                            const float* mrow = a.mask + ((size_t)b * a.maskBatch * a.Tq + min(qrow, a.Tq - 1)) * a.Tk;
                            const bool vec = (a.Tk & 3) == 0 && k0 + 32 <= a.Tk && (((uintptr_t)a.mask) & 15) == 0;
#pragma unroll
                            for (int g = 0; g < 4; g++) {
                                const int kq = k0 + 8 * g + 4 * half;
                                if (vec) {
                                    const float4 t = *(const float4*)(mrow + kq);
                                    mk[4 * g] = t.x; mk[4 * g + 1] = t.y; mk[4 * g + 2] = t.z; mk[4 * g + 3] = t.w;
                                } else {
#pragma unroll
                                    for (int e = 0; e < 4; e++) mk[4 * g + e] = kq + e < a.Tk ? mrow[kq + e] : 1.f;
                                }
                            }
                        }
#pragma unroll
                        for (int v = 0; v < 16; v++) {
                            const int kl = 8 * (v >> 2) + 4 * half + (v & 3);
                            const int key = k0 + kl;
                            float sv = s[qt][v];
                            // causal: every row of a diagonal step keeps at least its own key, so the masked scores
                            // can simply be -inf (weight exactly 0) and the step takes the plain softmax path
                            if (KIND == 1 && key > qrow) sv = -INFINITY;
                            if (KIND == 2 && Ms[32 * sub + kl] == 0.f) sv = a.maskedRaw;
                            if (KIND == 3 && qrow < a.Tq && key < a.Tk && mk[v] == 0.f) sv = a.maskedRaw;
                            if (key >= a.Tk) sv = -INFINITY;
                            s[qt][v] = sv;
                        }
                    }
                    if (KIND == 1) flash_softmax_step<false, DT, QT>(s, o, m, l, c, a.maskedRaw, a.lazy);
                    else flash_softmax_step<true, DT, QT>(s, o, m, l, c, a.maskedRaw, a.lazy);
                } else {
                    flash_softmax_step<false, DT, QT>(s, o, m, l, c, a.maskedRaw, a.lazy);
                }
                // O^T += V^T P^T
                u32x4 pf[QT][PF];
#pragma unroll
                for (int qt = 0; qt < QT; qt++) {
#pragma unroll
                    for (int t = 0; t < PF; t++) pf[qt][t] = TR::pack_p(s[qt], t);
                }
#pragma unroll
                for (int t = 0; t < PF; t++)
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        const u32x4 vf = VROW ? TR::load_vt_rowmajor(&Vt[32 * sub * LDVR + dt * 32], LDVR, t, lane)
                                              : TR::load_vt(&Vt[(dt * 32 + l32) * LDV + 32 * sub], t, half);
#pragma unroll
                        for (int qt = 0; qt < QT; qt++) o[dt][qt] = TR::mma(vf, pf[qt][t], o[dt][qt]);
                    }
            }
        }
        __syncthreads();
        if (kb + 1 < nkb) {
            if (!PREFETCH) gload(kb + 1);
            sstore(kb + 1);
        }
        __syncthreads();
    }

    // epilogue: y[query, dim] = O^T[dim, query] / l; register v of tile dt is dim 32*dt + 8*(v/4) + 4*half + v%4
#pragma unroll
    for (int qt = 0; qt < QT; qt++) {
        const int qrow = q0 + qt * 32 + l32;
        const float lt = l[qt] + __shfl_xor(l[qt], 32, 64);
        const float inv = 1.0f / lt;
        if (a.lse2 && qrow < a.Tq && half == 0)
            a.lse2[bh * a.Tq + qrow] = (m[qt] == a.maskedRaw) ? -INFINITY : __builtin_fmaf(m[qt], a.c, __log2f(lt));
        if (qrow < a.Tq) {
            T* yr = (T*)a.y + attn_y_row(a.yMerged, b, h, a.H, a.Tq, qrow, HS);
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    TR::store4(yr + 32 * dt + 8 * g + 4 * half, o[dt][qt][4 * g] * inv, o[dt][qt][4 * g + 1] * inv,
                               o[dt][qt][4 * g + 2] * inv, o[dt][qt][4 * g + 3] * inv);
        }
    }
}

// ---------------------------------------------------------------------------
// Software-pipelined kernel for bf16 inference without mask or with the causal one, head sizes 64 and 128.
//
// Same data flow as flash_fwd_kernel with one 32-row tile per wavefront, but the three parts of a 32-key step run
// in different phases so that matrix and vector instructions of ONE wavefront overlap (those of different
// wavefronts on a SIMD do not): during phase t a wavefront issues
//     O^T += V^T P^T of step t - 1     (HS / 16 MFMAs, V^T fragments through the transposing LDS read)
//     S^T of step t + 1                (HS / 16 MFMAs, K fragments from LDS)
//     the softmax of step t            (vector ALU: max, exp2, sum, pack)
// in a fixed issue order: a phase is NSLOT MFMA slots, each followed by a slice of the softmax, the fragment
// read two slots ahead and a slice of the K / V staging traffic, every slice in a scheduling region of its own
// so that the order is kept.  K and V blocks of 64 keys are row-major and double buffered in dynamic LDS; a
// block is requested from memory three phases before it is written to LDS, while the other buffer is being
// read.  Phases that are not in steady state (the first, the last, diagonal or ragged steps) take a plain
// sequential path built from the same pieces.
template <int KIND, int NW, int HS, int OCC>
__global__ __launch_bounds__(NW * 64, OCC) void flash_pipe_bf16_kernel(FlashArgs a)
{
    typedef FlashTraits<bf16_t> TR;
    constexpr int BN = 64, NT = NW * 64, BM = NW * 32, LDK = HS + 8, LDVR = (HS * 2) % 256 == 0 ? HS + 16 : HS + 8;
    constexpr int KF = HS / 16, DT = HS / 32, NPV = 2 * DT, NSLOT = NPV + KF;   // 16 slots at head size 128, 8 at 64
    constexpr int CPR = HS / 8;                  // 16-byte chunks per K (or V) row
    constexpr int CPT = BN * CPR / NT;           // chunks of a block per thread
    // slots of the softmax slices: maxima in 0 and 1, new maximum in 2, the exponentials from 3 on, then the packing,
    // the row sum in the last slot
    constexpr int NEXP = NSLOT == 16 ? 8 : 3, EPS = NSLOT == 16 ? 2 : 6;   // exponential slots, scores per slot
    constexpr int PACK0 = 3 + NEXP, NPACK = NSLOT == 16 ? 4 : 1, WPS = 8 / NPACK;   // packing slots, words per slot
    static_assert(PACK0 + NPACK < NSLOT && 2 * CPT <= NSLOT - 2, "slices do not fit the slots");
    constexpr int KBUF = BN * LDK, VBUF = BN * LDVR;
    extern __shared__ __attribute__((aligned(16))) unsigned char pipe_smem[];
    bf16_t* Ks = reinterpret_cast<bf16_t*>(pipe_smem);   // [2][KBUF]
    bf16_t* Vs = Ks + 2 * KBUF;                          // [2][VBUF]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    int qblock, h, b;
    if (KIND == 1) {
        const int nbh = a.B * a.H;
        const int nqb = (a.Tq + BM - 1) / BM;
        const int rank = flash_causal_rank(OCC);
        int ibh;
        flash_causal_map(rank, nbh, nqb, a.causalGroup, &qblock, &ibh);
        b = ibh / a.H;
        h = ibh % a.H;
    } else {
        qblock = blockIdx.x;
        h = blockIdx.y;
        b = blockIdx.z;
    }
    const size_t bh = (size_t)b * a.H + h;
    const int q0 = qblock * BM + wave * 32;
    const bf16_t* qp = (const bf16_t*)a.q + bh * a.Tq * HS;
    const bf16_t* kp = (const bf16_t*)a.k + bh * a.Tk * HS;
    const bf16_t* vp = (const bf16_t*)a.v + bh * a.Tk * HS;

    u32x4 qf[KF];
    {
        const int row = min(q0 + l32, a.Tq - 1);
#pragma unroll
        for (int f = 0; f < KF; f++) qf[f] = *(const u32x4*)(qp + (size_t)row * HS + f * 16 + half * 8);
    }
    int kend = a.Tk;
    if (KIND == 1) kend = min(a.Tk, qblock * BM + BM);
    const int nkb = (kend + BN - 1) / BN;
    int nstw = min(2 * nkb, (a.Tk + 31) / 32);             // steps this wavefront computes
    if (KIND == 1) nstw = min(nstw, (q0 + 31) / 32 + 1);
    if (q0 >= a.Tq) nstw = 0;

    // staging: chunk e = tid + NT i of a block -> key e / CPR, 16-byte chunk e % CPR (K and V alike)
    // two register sets per operand (set = block & 1): a block is requested three phases before it is written to LDS
    u32x4 kreg[2][CPT], vreg[2][CPT];
    int srow[CPT];
#pragma unroll
    for (int i = 0; i < CPT; i++) srow[i] = (tid + i * NT) / CPR;
    const int scol = (tid % CPR) * 8;
    auto gaddr = [&](const bf16_t* base, int kb, int i) { return base + (size_t)min(kb * BN + srow[i], a.Tk - 1) * HS + scol; };
    auto kstore = [&](int buf, const u32x4 (&r)[CPT]) {
#pragma unroll
        for (int i = 0; i < CPT; i++) *(u32x4*)(Ks + buf * KBUF + srow[i] * LDK + scol) = r[i];
    };
    auto vstore = [&](int buf, const u32x4 (&r)[CPT]) {
#pragma unroll
        for (int i = 0; i < CPT; i++) *(u32x4*)(Vs + buf * VBUF + srow[i] * LDVR + scol) = r[i];
    };

    floatx16 o[DT][1];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[dt][0][v] = 0.f;
    float m[1] = {-INFINITY}, l[1] = {0.f};
    const float c = a.c, lazy = a.lazy;
    const floatx16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const bf16_t* kfrag = Ks + l32 * LDK + half * 8;

    // fragment j of a phase around step t: 0 .. NPV - 1 = V^T fragments of step t - 1 (key half j / DT, dim tile j % DT),
    // the rest = K fragments of step t + 1
    auto frag = [&](int j, int t) -> u32x4 {
        if (j < NPV) {
            const int tv = t - 1;
            return TR::load_vt_rowmajor(Vs + ((tv >> 1) & 1) * VBUF + 32 * (tv & 1) * LDVR + (j % DT) * 32, LDVR, j / DT, lane);
        }
        const int ts = t + 1;
        return *(const u32x4*)(kfrag + ((ts >> 1) & 1) * KBUF + (ts & 1) * 32 * LDK + (j - NPV) * 16);
    };
    auto smma = [&](int t, floatx16& sn) {      // S^T of step t
        const bf16_t* kb_ = kfrag + ((t >> 1) & 1) * KBUF + (t & 1) * 32 * LDK;
        sn = TR::mma(*(const u32x4*)(kb_), qf[0], zero16);
#pragma unroll
        for (int f = 1; f < KF; f++) sn = TR::mma(*(const u32x4*)(kb_ + 16 * f), qf[f], sn);
    };
    auto pvmma = [&](int t, const u32x4 (&pp)[2]) {   // O^T += V^T P^T of step t
        const bf16_t* vb_ = Vs + ((t >> 1) & 1) * VBUF + 32 * (t & 1) * LDVR;
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) o[dt][0] = TR::mma(TR::load_vt_rowmajor(vb_ + dt * 32, LDVR, tt, lane), pp[tt], o[dt][0]);
    };
    // sequential softmax of step t (any masking), leaves the packed weights in pc
    auto soft_slow = [&](int t, floatx16 (&sc)[1], u32x4 (&pc)[2]) {
        const int k0 = t * 32;
        const bool masked = ((KIND == 1) && (k0 + 31 > q0)) || (k0 + 32 > a.Tk);
        if (masked) {
            const int qrow = q0 + l32;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int key = k0 + 8 * (v >> 2) + 4 * half + (v & 3);
                // every row of such a step keeps at least one key (its own, or key k0 < Tk), so -inf is safe
                if ((KIND == 1 && key > qrow) || key >= a.Tk) sc[0][v] = -INFINITY;
            }
        }
        flash_softmax_step<false, DT, 1>(sc, o, m, l, c, a.maskedRaw, lazy);
        pc[0] = TR::pack_p(sc[0], 0);
        pc[1] = TR::pack_p(sc[0], 1);
    };

    // prologue: K(0), V(0) in LDS, K(1), K(2) and V(1) in registers, S^T of step 0
#pragma unroll
    for (int i = 0; i < CPT; i++) { kreg[0][i] = *(const u32x4*)gaddr(kp, 0, i); vreg[0][i] = *(const u32x4*)gaddr(vp, 0, i); }
    kstore(0, kreg[0]);
    vstore(0, vreg[0]);
#pragma unroll
    for (int i = 0; i < CPT; i++) {
        kreg[1][i] = *(const u32x4*)gaddr(kp, 1, i);
        kreg[0][i] = *(const u32x4*)gaddr(kp, 2, i);
        vreg[1][i] = *(const u32x4*)gaddr(vp, 1, i);
    }
#pragma unroll
    for (int f = 0; f < KF; f++) asm volatile("" : "+v"(qf[f]));
    __syncthreads();
    floatx16 sA[1], sB[1];
    u32x4 pA[2], pB[2];
    sA[0] = zero16;
    sB[0] = zero16;
    pA[0] = pA[1] = pB[0] = pB[1] = u32x4{0u, 0u, 0u, 0u};
    if (nstw > 0) smma(0, sA[0]);

    // One phase of block kb = t / 2, P = kb & 1.  ROLE 0 (even phase 2 kb): request V(kb + 2) into set P, write K(kb + 1)
    // from set 1 - P to LDS; ROLE 1 (odd phase 2 kb + 1): request K(kb + 3) into set 1 - P (just written out), write
    // V(kb + 1) from set 1 - P.  sc: scores of step t (in), sn: scores of step t + 1 (out), pp: packed weights of step
    // t - 1 (in), pc: packed weights of step t (out).  Blocks past the end re-read the last rows (never consumed).
    auto phase = [&](auto role_, auto par_, int t, floatx16 (&sc)[1], floatx16 (&sn)[1], const u32x4 (&pp)[2], u32x4 (&pc)[2]) {
        constexpr int ROLE = decltype(role_)::value, P = decltype(par_)::value;
        const int kbn = (ROLE == 0) ? (t >> 1) + 2 : (t >> 1) + 3;     // block requested in this phase
        const int wbuf = ((t >> 1) + 1) & 1;                           // LDS buffer written in this phase: block kb + 1
        u32x4 (&fetch)[CPT] = ROLE == 0 ? vreg[P] : kreg[1 - P];
        const u32x4 (&put)[CPT] = ROLE == 0 ? kreg[1 - P] : vreg[1 - P];
        const bool doSoft = t < nstw, doS = t + 1 < nstw, doPV = t >= 1 && t - 1 < nstw;
        const bool plain = !((KIND == 1) && (t * 32 + 31 > q0)) && (t * 32 + 32 <= a.Tk);
        if (doSoft && doS && doPV && plain) {
            u32x4 fr[NSLOT];
            fr[0] = frag(0, t);
            fr[1] = frag(1, t);
            float m1 = 0.f, m2 = 0.f, m3 = 0.f, m4 = 0.f, mx = 0.f, alpha = 1.f, mc = 0.f, rs = 0.f, pw[16];
            uint32_t pk[8];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NSLOT; j++) {
                if (j < NPV) o[j % DT][0] = TR::mma(fr[j], pp[j / DT], o[j % DT][0]);
                else sn[0] = TR::mma(fr[j], qf[j - NPV], j == NPV ? zero16 : sn[0]);
                if (j + 2 < NSLOT) fr[j + 2] = frag(j + 2, t);
                // softmax of step t, one slice per slot
                if (j == 0) {
                    m1 = fmaxf(fmaxf(sc[0][0], sc[0][1]), sc[0][2]);
                    m2 = fmaxf(fmaxf(sc[0][3], sc[0][4]), sc[0][5]);
                    m3 = fmaxf(fmaxf(sc[0][6], sc[0][7]), sc[0][8]);
                    m4 = fmaxf(fmaxf(sc[0][9], sc[0][10]), sc[0][11]);
                    asm volatile("" : "+v"(m1), "+v"(m2), "+v"(m3), "+v"(m4));
                } else if (j == 1) {
                    const float m5 = fmaxf(fmaxf(sc[0][12], sc[0][13]), sc[0][14]);
                    mx = fmaxf(fmaxf(m1, m2), m3);
                    mx = fmaxf(fmaxf(mx, m4), m5);
                    mx = fmaxf(mx, sc[0][15]);
                    mx = flash_half_max(mx);
                    asm volatile("" : "+v"(mx));
                } else if (j == 2) {
                    const float mnew = (mx > m[0] + lazy) ? mx : m[0];
                    alpha = __builtin_amdgcn_exp2f((m[0] - mnew) * c);
                    mc = mnew * c;
                    m[0] = mnew;
                    asm volatile("" : "+v"(alpha), "+v"(mc), "+v"(m[0]));
                } else if (j < 3 + NEXP) {
#pragma unroll
                    for (int e = EPS * (j - 3); e < EPS * (j - 2) && e < 16; e += 2) {
                        pw[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[0][e], c, -mc));
                        pw[e + 1] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[0][e + 1], c, -mc));
                        rs += pw[e] + pw[e + 1];
                        asm volatile("" : "+v"(pw[e]), "+v"(pw[e + 1]), "+v"(rs));
                    }
                } else if (j < PACK0 + NPACK) {
#pragma unroll
                    for (int w = WPS * (j - PACK0); w < WPS * (j - PACK0 + 1); w++) {
                        pk[w] = pack_bf16x2(pw[2 * w], pw[2 * w + 1]);
                        asm volatile("" : "+v"(pk[w]));
                    }
                } else if (j == NSLOT - 1) {
                    l[0] = l[0] * alpha + rs;
                    asm volatile("" : "+v"(l[0]));
                }
                // K / V staging traffic of this phase
                if (j >= NSLOT - 2 * CPT && j < NSLOT - CPT) {
                    const int i = j - (NSLOT - 2 * CPT);
                    if (ROLE == 0) *(u32x4*)(Ks + wbuf * KBUF + srow[i] * LDK + scol) = put[i];
                    else *(u32x4*)(Vs + wbuf * VBUF + srow[i] * LDVR + scol) = put[i];
                } else if (j >= NSLOT - CPT) {
                    // the set that ROLE 1 refills is the one ROLE 0 emptied a phase ago; ROLE 0 refills a set that the
                    // previous odd phase emptied: requests go after this phase's LDS writes in program order
                    fetch[j - (NSLOT - CPT)] = *(const u32x4*)gaddr(ROLE == 0 ? vp : kp, kbn, j - (NSLOT - CPT));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            pc[0] = u32x4{pk[0], pk[1], pk[2], pk[3]};
            pc[1] = u32x4{pk[4], pk[5], pk[6], pk[7]};
            if (!__all(alpha == 1.0f)) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int v = 0; v < 16; v++) o[dt][0][v] *= alpha;
            }
        } else {
            if (doPV) pvmma(t - 1, pp);
            if (doSoft) soft_slow(t, sc, pc);
            if (doS) smma(t + 1, sn[0]);
            if (ROLE == 1) vstore(wbuf, put);
            else kstore(wbuf, put);
#pragma unroll
            for (int i = 0; i < CPT; i++) fetch[i] = *(const u32x4*)gaddr(ROLE == 0 ? vp : kp, kbn, i);
        }
        __syncthreads();
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    for (int kb = 0; kb <= nkb; kb += 2) {
        phase(I0{}, I0{}, 2 * kb, sA, sB, pB, pA);
        if (kb < nkb) phase(I1{}, I0{}, 2 * kb + 1, sB, sA, pA, pB);
        if (kb + 1 <= nkb) phase(I0{}, I1{}, 2 * kb + 2, sA, sB, pB, pA);
        if (kb + 1 < nkb) phase(I1{}, I1{}, 2 * kb + 3, sB, sA, pA, pB);
    }

    // epilogue: y[query, dim] = O^T[dim, query] / l
    const int qrow = q0 + l32;
    const float lt = l[0] + __shfl_xor(l[0], 32, 64);
    const float inv = 1.0f / lt;
    if (qrow < a.Tq) {
        bf16_t* yr = (bf16_t*)a.y + attn_y_row(a.yMerged, b, h, a.H, a.Tq, qrow, HS);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                TR::store4(yr + 32 * dt + 8 * g + 4 * half, o[dt][0][4 * g] * inv, o[dt][0][4 * g + 1] * inv,
                           o[dt][0][4 * g + 2] * inv, o[dt][0][4 * g + 3] * inv);
    }
}

// ---------------------------------------------------------------------------
// Short causal sequences in fp32, head size 64 (the one-sequence prompt pass of the decode engine: 128 positions, 12
// heads).  flash_fwd_kernel gives such a launch one workgroup per head, and the wavefront that owns the last 32 rows runs
// its four 32-key steps - 256 fp32 MFMAs of 64 cycles - one after the other.  Here a workgroup owns 32 query rows and
// its four wavefronts take the 32-key steps in turn (step w, w + 4, ...), each with its own running maximum, sum and
// output tile; the partial results meet in LDS and are combined as the splits of a decode step are.  K and V go from
// global memory straight into the fragments (a step's tiles are read by one wavefront only, so LDS would add a
// round trip and nothing else).
__global__ __launch_bounds__(256) void flash_short_causal_f32_kernel(FlashArgs a)
{
    typedef FlashTraits<float> TR;
    constexpr int HS = 64, CPF = TR::CPF, KF = HS / CPF, PF = 32 / CPF, DT = HS / 32, LDO = HS + 4;
    __shared__ __attribute__((aligned(16))) float Os[4][32 * LDO];
    __shared__ float Ms[4][32], Ls[4][32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int qtile = (int)gridDim.x - 1 - (int)blockIdx.x;   // heaviest first
    const int h = blockIdx.y, b = blockIdx.z;
    const size_t bh = (size_t)b * a.H + h;
    const int q0 = qtile * 32;
    const float* qp = (const float*)a.q + bh * a.Tq * HS;
    const float* kp = (const float*)a.k + bh * a.Tk * HS;
    const float* vp = (const float*)a.v + bh * a.Tk * HS;
    const int qrow = q0 + l32;

    u32x4 qf[1][KF];
    {
        const int row = min(qrow, a.Tq - 1);
#pragma unroll
        for (int f = 0; f < KF; f++) qf[0][f] = *(const u32x4*)(qp + (size_t)row * HS + f * CPF + half * (CPF / 2));
    }
    floatx16 o[DT][1];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[dt][0][v] = 0.f;
    float m[1] = {-INFINITY}, l[1] = {0.f};

    const int lastStep = min(qtile, (a.Tk - 1) / 32);   // causal: keys past the tile's last row contribute nothing
    for (int step = wave; step <= lastStep; step += 4) {
        const int k0 = step * 32;
        floatx16 s[1];
#pragma unroll
        for (int v = 0; v < 16; v++) s[0][v] = 0.f;
        const float* krow = kp + (size_t)min(k0 + l32, a.Tk - 1) * HS + half * (CPF / 2);
        u32x4 kf[KF];
#pragma unroll
        for (int f = 0; f < KF; f++) kf[f] = *(const u32x4*)(krow + f * CPF);
        // V^T fragments: lane (d = 32 dt + l32, half) holds keys k0 + 8 t + 4 half .. + 3 of column d
        u32x4 vf[PF][DT];
#pragma unroll
        for (int t = 0; t < PF; t++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                const float* vc = vp + dt * 32 + l32;
                const int kb = k0 + 8 * t + 4 * half;
                vf[t][dt] = u32x4{__float_as_uint(vc[(size_t)min(kb, a.Tk - 1) * HS]), __float_as_uint(vc[(size_t)min(kb + 1, a.Tk - 1) * HS]),
                                  __float_as_uint(vc[(size_t)min(kb + 2, a.Tk - 1) * HS]), __float_as_uint(vc[(size_t)min(kb + 3, a.Tk - 1) * HS])};
            }
#pragma unroll
        for (int f = 0; f < KF; f++) s[0] = TR::mma(kf[f], qf[0][f], s[0]);
        // register v holds key k0 + 8 (v / 4) + 4 half + v % 4 for query q0 + l32
        if (k0 + 31 > q0 || k0 + 32 > a.Tk) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int key = k0 + 8 * (v >> 2) + 4 * half + (v & 3);
                if (key > qrow || key >= a.Tk) s[0][v] = -INFINITY;
            }
        }
        flash_softmax_step<false, DT, 1>(s, o, m, l, a.c, a.maskedRaw, a.lazy);
#pragma unroll
        for (int t = 0; t < PF; t++) {
            const u32x4 pf = TR::pack_p(s[0], t);
#pragma unroll
            for (int dt = 0; dt < DT; dt++) o[dt][0] = TR::mma(vf[t][dt], pf, o[dt][0]);
        }
    }
    // partial results to LDS: register v of tile dt is dim 32 dt + 8 (v / 4) + 4 half + v % 4 of query l32
    const float lsum = l[0] + __shfl_xor(l[0], 32, 64);
    if (half == 0) { Ms[wave][l32] = m[0]; Ls[wave][l32] = lsum; }
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *(float4*)&Os[wave][l32 * LDO + 32 * dt + 8 * g + 4 * half] =
                make_float4(o[dt][0][4 * g], o[dt][0][4 * g + 1], o[dt][0][4 * g + 2], o[dt][0][4 * g + 3]);
    __syncthreads();
    // thread t combines eight dims of query t / 8.  Wavefront 0 always has a step (key 0 is visible to every row), so
    // the common maximum is finite; a wavefront without steps has maximum -inf and weight exp2(-inf) = 0.
    const int q = tid >> 3, d8 = (tid & 7) * 8;
    float mw[4], M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; w++) { mw[w] = Ms[w][q]; M = fmaxf(M, mw[w]); }
    float L = 0.f, acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const float sc = __builtin_amdgcn_exp2f((mw[w] - M) * a.c);
        L += Ls[w][q] * sc;
        const float4 x0 = *(const float4*)&Os[w][q * LDO + d8], x1 = *(const float4*)&Os[w][q * LDO + d8 + 4];
        acc[0] += x0.x * sc; acc[1] += x0.y * sc; acc[2] += x0.z * sc; acc[3] += x0.w * sc;
        acc[4] += x1.x * sc; acc[5] += x1.y * sc; acc[6] += x1.z * sc; acc[7] += x1.w * sc;
    }
    if (q0 + q < a.Tq) {
        const float inv = 1.0f / L;
        float* yr = (float*)a.y + attn_y_row(a.yMerged, b, h, a.H, a.Tq, q0 + q, HS) + d8;
        *(float4*)yr = make_float4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
        *(float4*)(yr + 4) = make_float4(acc[4] * inv, acc[5] * inv, acc[6] * inv, acc[7] * inv);
    }
}

template <typename T, int HS, int QT, int NW, int OCC, bool PREFETCH>
static hipError_t flash_launch_cfg(hipStream_t s, const FlashArgs& f, int kind)
{
    constexpr int BM = NW * 32 * QT;
    dim3 grid((f.Tq + BM - 1) / BM, f.H, f.B);
    if (kind == MASK_CAUSAL) grid = dim3(((f.Tq + BM - 1) / BM) * f.H * f.B, 1, 1);
    if (kind == MASK_NONE) hipLaunchKernelGGL((flash_fwd_kernel<T, HS, 0, QT, NW, OCC, PREFETCH>), grid, NW * 64, 0, s, f);
    else if (kind == MASK_CAUSAL) hipLaunchKernelGGL((flash_fwd_kernel<T, HS, 1, QT, NW, OCC, PREFETCH>), grid, NW * 64, 0, s, f);
    else if (kind == MASK_KEY) hipLaunchKernelGGL((flash_fwd_kernel<T, HS, 2, QT, NW, OCC, PREFETCH>), grid, NW * 64, 0, s, f);
    else hipLaunchKernelGGL((flash_fwd_kernel<T, HS, 3, QT, NW, OCC, PREFETCH>), grid, NW * 64, 0, s, f);   // MASK_BQK, MASK_QK
    return hipGetLastError();
}

hipError_t attn_flash_launch(hipStream_t s, DType dt, const AttnArgs& a, bool* handled)
{
    *handled = false;
    if (a.hs != 64 && a.hs != 128) return hipSuccess;
    if ((((uintptr_t)a.q | (uintptr_t)a.k | (uintptr_t)a.v | (uintptr_t)a.y) & 15) != 0) return hipSuccess;
    FlashArgs f;
    f.maskBatch = a.kind == MASK_QK ? 0 : 1;   // a shared (Tq,Tk) mask is the per-sequence form with batch stride 0
    f.q = a.q; f.k = a.k; f.v = a.v; f.y = a.y;
    f.mask = a.mask; f.B = a.B; f.H = a.H; f.Tq = a.Tq; f.Tk = a.Tk;
    f.c = a.scale * 1.4426950408889634f;
    f.maskedRaw = MASKED / a.scale;
    f.lazy = 8.0f / f.c;
    f.lse2 = a.lse2;
    f.yMerged = a.yMerged;
    f.causalGroup = 0;
    if (a.kind == MASK_CAUSAL && a.hs == 128 && dt == BF16) {
        // when K and V of all heads together exceed what the caches hold (128 MB taken as the line), walk the heads in
        // at most four groups of a multiple of 8 heads
        const long long nbh = (long long)a.B * a.H;
        const double kvBytes = 2.0 * nbh * a.Tk * a.hs * 2;
        if (kvBytes > 128e6 && nbh % 8 == 0) f.causalGroup = (int)(((nbh + 3) / 4 + 7) / 8 * 8);
    }
    *handled = true;
    // Tile shapes picked by measurement on MI355X.  Head size 64: four wavefronts with one 32-row tile each
    // (128-row workgroups) give enough equal-sized workgroups to balance 256 CUs at T = 1024; head size 128
    // keeps eight wavefronts per workgroup so that each staged K / V block serves more rows.
    if (dt == BF16) {
        // 512 keys and more, no mask or the causal one: the kernel with two query tiles per wavefront (attn_flash2.hip),
        // 7 .. 30 % ahead of the ones below from that length on (B = 8, T = 1024, 12 heads of 64, causal: 26.4 against
        // 28.6 us; B = 4, T = 4096, 32 heads of 128, causal: 0.52 against 0.62 ms).  Its workgroups own 256 query rows,
        // too coarse a grain for shorter sequences.
        if (f.Tk >= 512 && (a.kind == MASK_NONE || a.kind == MASK_CAUSAL)) {
            bool took = false;
            const hipError_t e = attn_flash2_launch(s, f, a.hs, a.kind == MASK_CAUSAL, &took);
            if (e != hipSuccess || took) return e;
        }
        if (a.hs == 64) {
            // Unmasked attention runs the software-pipelined kernel (B = 8, T = 1024, 12 heads: 45.7 us; B = 4,
            // T = 4096, 32 heads: 0.79 ms).  Causal launches measure the same (T = 1024) or up to 10 % slower
            // (T >= 2048) with it - ragged per-wavefront ranges leave the pipeline in its sequential phases more
            // often - so they stay with the plain kernel.
            if (a.kind == MASK_NONE && !a.lse2) {   // the pipelined kernel does not keep the row statistics
                constexpr int LDSB = 2 * (64 * 72 + 64 * 72) * 2;
                hipLaunchKernelGGL((flash_pipe_bf16_kernel<0, 4, 64, 3>), dim3((f.Tq + 127) / 128, f.H, f.B), 256, LDSB, s, f);
                return hipGetLastError();
            }
            return flash_launch_cfg<bf16_t, 64, 1, 4, 3, true>(s, f, a.kind);
        }
        // no mask or causal, inference: the software-pipelined kernel (it does not keep the row statistics).  Measured at
        // B=4, T=4096, 32 heads: unmasked 1.57 -> 1.31 ms; causal the same as the plain kernel (0.77 - 0.80 ms).
        if ((a.kind == MASK_NONE || a.kind == MASK_CAUSAL) && !a.lse2) {
            constexpr int LDSB = 2 * (64 * 136 + 64 * 144) * 2;
            static bool attr = false;
            if (!attr) {
                hipError_t e = hipFuncSetAttribute((const void*)flash_pipe_bf16_kernel<0, 8, 128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, LDSB);
                if (e == hipSuccess) e = hipFuncSetAttribute((const void*)flash_pipe_bf16_kernel<1, 8, 128, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, LDSB);
                if (e == hipSuccess) e = hipFuncSetAttribute((const void*)flash_pipe_bf16_kernel<1, 4, 128, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, LDSB);
                if (e != hipSuccess) return e;
                attr = true;
            }
            // launches that leave CUs empty with 256-row workgroups take four wavefronts per workgroup (T = 777, 6 heads:
            // 28.9 -> 23.8 us); at full size the larger workgroup wins (0.77 against 0.81 ms)
            if (a.kind == MASK_CAUSAL && (long long)((f.Tq + 255) / 256) * f.H * f.B < 256) {
                hipLaunchKernelGGL((flash_pipe_bf16_kernel<1, 4, 128, 2>), dim3(((f.Tq + 127) / 128) * f.H * f.B), 256, LDSB, s, f);
                return hipGetLastError();
            }
            const int nqb = (f.Tq + 255) / 256;
            if (a.kind == MASK_CAUSAL) hipLaunchKernelGGL((flash_pipe_bf16_kernel<1, 8, 128, 1>), dim3(nqb * f.H * f.B), 512, LDSB, s, f);
            else hipLaunchKernelGGL((flash_pipe_bf16_kernel<0, 8, 128, 1>), dim3(nqb, f.H, f.B), 512, LDSB, s, f);
            return hipGetLastError();
        }
        return flash_launch_cfg<bf16_t, 128, 1, 8, 1, true>(s, f, a.kind);
    }
    if (a.hs == 64) {
        // causal self attention whose 128-row blocks would not give every CU a workgroup: one workgroup per 32 rows,
        // the key steps dealt to its wavefronts
        if (a.kind == MASK_CAUSAL && !a.lse2 && a.Tq == a.Tk && (long long)((a.Tq + 127) / 128) * a.H * a.B < 256) {
            hipLaunchKernelGGL(flash_short_causal_f32_kernel, dim3((a.Tq + 31) / 32, a.H, a.B), 256, 0, s, f);
            return hipGetLastError();
        }
        return flash_launch_cfg<float, 64, 1, 4, 2, false>(s, f, a.kind);
    }
    return flash_launch_cfg<float, 128, 1, 8, 1, false>(s, f, a.kind);
}

}  // namespace mch
