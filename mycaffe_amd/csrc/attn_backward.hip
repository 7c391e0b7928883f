// Scaled-dot-product attention backward for gfx950.
//
// The reference keeps the (B,H,T,T) probabilities of the forward pass and runs four batched GEMMs and a cuDNN
// softmax gradient over them (attnHandle::Backward, CudaDnnDLL/Cuda Files/attn.cu:608-661).  Here nothing of size
// T x T ever reaches memory: the probabilities are recomputed tile by tile from Q, K and one number per query row,
//     lse2[row] = log2( sum_k exp(score[row,k]) )        (scores already scaled, masked ones at -1e29),
// which the forward pass stores when the attention handle is in training mode, together with
//     D[row] = sum_d dY[row,d] * Y[row,d]                ( = sum_k P[row,k] dP[row,k] ).
// With P = exp2(score * log2e - lse2):
//     dV = P^T dY,   dP = dY V^T,   dS = P * (dP - D) * scale,   dQ = dS K,   dK = dS^T Q.
// A masked entry has P exactly 0, as exp(-1e29 - max) is in the reference; a row whose every key is masked is uniform
// over all keys there (all scores equal) and is marked here by lse2 = -inf.
//
// Kernels:
//  * attn_bwd_stats_kernel: D for every row and, when the forward pass left no lse2, lse2 as well (one wavefront a row);
//    skipped when the MFMA kernels run on a stored lse2 (the dQ kernel then computes D on the way).
//  * attn_bwd_dq_rows_kernel / attn_bwd_dkv_rows_kernel: any head size up to 256, any mask kind, Tq != Tk: one wavefront
//    per query row (per key row), lanes over the other sequence axis.  No atomics: every output row has one owner, so
//    results do not depend on scheduling.
//  * MFMA tiles for head sizes 64 and 128 (further down).
#include "flash_traits.h"
#include "kernels.h"

namespace mch {

static constexpr float MASKED_SCORE = -1e29f;
static constexpr float LOG2E = 1.4426950408889634f;

template <typename T> __device__ inline float ldb(const T* p, size_t i);
template <> __device__ inline float ldb<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ inline float ldb<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ inline void stb(T* p, size_t i, float v);
template <> __device__ inline void stb<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ inline void stb<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

struct AttnBwdArgs {
    const void *q, *k, *v, *y, *dy;
    void *dq, *dk, *dv;
    const float* mask;
    float* lse2;      // [B*H*Tq]
    float* dsum;      // [B*H*Tq]
    int B, H, Tq, Tk, hs, kind;
    float scale;
    int computeLse;
    int computeD;     // MFMA path: the dQ kernel computes D itself (no statistics kernel ran)
    int useDropout;   // row kernels only
    AttnDropout drop;
};

// factors of probability (bh, row, key) under dropout: pf multiplies P for dV, sf multiplies dS
__device__ inline void attn_drop_factors(const AttnBwdArgs& a, size_t bh, int row, int key, float* pf, float* sf)
{
    *pf = 1.f;
    *sf = 1.f;
    if (!a.useDropout) return;
    const bool keep = attn_dropout_keep(a.drop.seed, (uint64_t)(bh * a.Tq + row) * a.Tk + key, a.drop.threshold);
    *pf = keep ? a.drop.keepScale : 0.f;
    *sf = keep ? a.drop.keepScale * a.drop.keepScale : 0.f;
}

__device__ inline bool attn_masked(const AttnBwdArgs& a, int b, int row, int key)
{
    switch (a.kind) {
    case MASK_CAUSAL: return key > row;
    case MASK_QK: return a.mask[(size_t)row * a.Tk + key] == 0.f;
    case MASK_KEY: return a.mask[(size_t)b * a.Tk + key] == 0.f;
    case MASK_BQK: return a.mask[((size_t)b * a.Tq + row) * a.Tk + key] == 0.f;
    default: return false;
    }
}

__device__ inline float wave_sum_f(float v)
{
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ inline float wave_max_f(float v)
{
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// probability of (row, key) given the scaled score and the row's lse2
__device__ inline float attn_prob(float s, bool masked, float lse2, float uniform)
{
    if (lse2 == -INFINITY) return uniform;
    return masked ? 0.f : exp2f(s * LOG2E - lse2);
}

// 4 wavefronts per workgroup, one query row each
template <typename T> __global__ __launch_bounds__(256) void attn_bwd_stats_kernel(AttnBwdArgs a)
{
    __shared__ float qs[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;
    const int h = blockIdx.y, b = blockIdx.z;
    const bool valid = row < a.Tq;
    const size_t bh = (size_t)b * a.H + h;
    const size_t ro = (bh * a.Tq + (valid ? row : 0)) * a.hs;
    const T* q = (const T*)a.q + ro;
    for (int d = lane; d < a.hs; d += 64) qs[wave][d] = ldb(q, d) * a.scale;
    __syncthreads();
    if (!valid) return;
    float dsum = 0.f;
    for (int d = lane; d < a.hs; d += 64) dsum += ldb((const T*)a.dy + ro, d) * ldb((const T*)a.y + ro, d);
    dsum = wave_sum_f(dsum);
    if (lane == 0) a.dsum[bh * a.Tq + row] = dsum;
    if (!a.computeLse) return;
    const T* k = (const T*)a.k + bh * a.Tk * a.hs;
    float m = -INFINITY, l = 0.f;
    for (int kb = 0; kb < a.Tk; kb += 64) {
        const int j = kb + lane;
        float s = -INFINITY;
        if (j < a.Tk) {
            const T* kr = k + (size_t)j * a.hs;
            float d = 0.f;
            for (int i = 0; i < a.hs; i++) d += qs[wave][i] * ldb(kr, i);
            s = attn_masked(a, b, row, j) ? MASKED_SCORE : d;
        }
        const float mn = fmaxf(m, wave_max_f(s));
        const float p = (j < a.Tk) ? expf(s - mn) : 0.f;
        l = l * expf(m - mn) + wave_sum_f(p);
        m = mn;
    }
    if (lane == 0) a.lse2[bh * a.Tq + row] = (m == MASKED_SCORE) ? -INFINITY : (m + logf(l)) * LOG2E;
}

// dQ: one wavefront per query row, lanes over keys
template <typename T> __global__ __launch_bounds__(256) void attn_bwd_dq_rows_kernel(AttnBwdArgs a)
{
    constexpr int DPL = 4;  // hs <= 256
    __shared__ float qs[4][256], gs[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row = blockIdx.x * 4 + wave;
    const int h = blockIdx.y, b = blockIdx.z;
    const bool valid = row < a.Tq;
    const size_t bh = (size_t)b * a.H + h;
    const size_t ro = (bh * a.Tq + (valid ? row : 0)) * a.hs;
    for (int d = lane; d < a.hs; d += 64) {
        qs[wave][d] = ldb((const T*)a.q + ro, d) * a.scale;
        gs[wave][d] = ldb((const T*)a.dy + ro, d);
    }
    __syncthreads();
    if (!valid) return;
    const T* k = (const T*)a.k + bh * a.Tk * a.hs;
    const T* v = (const T*)a.v + bh * a.Tk * a.hs;
    const float lse2 = a.lse2[bh * a.Tq + row], dsum = a.dsum[bh * a.Tq + row];
    const float uniform = 1.0f / a.Tk;
    // causal rows that are not fully masked have zero probability past the diagonal
    const int kend = (a.kind == MASK_CAUSAL && lse2 != -INFINITY) ? min(a.Tk, row + 1) : a.Tk;
    float acc[DPL] = {0.f, 0.f, 0.f, 0.f};
    for (int kb = 0; kb < kend; kb += 64) {
        const int j = kb + lane;
        float ds = 0.f;
        if (j < kend) {
            const T* kr = k + (size_t)j * a.hs;
            const T* vr = v + (size_t)j * a.hs;
            float s = 0.f, dp = 0.f;
            for (int i = 0; i < a.hs; i++) {
                s += qs[wave][i] * ldb(kr, i);
                dp += gs[wave][i] * ldb(vr, i);
            }
            const float p = attn_prob(s, attn_masked(a, b, row, j), lse2, uniform);
            float pf, sf;
            attn_drop_factors(a, bh, row, j, &pf, &sf);
            ds = sf * p * (dp - dsum) * a.scale;
        }
        const int cnt = min(64, kend - kb);
        for (int jj = 0; jj < cnt; jj++) {
            const float dj = __shfl(ds, jj, 64);
            const T* kr = k + (size_t)(kb + jj) * a.hs;
            for (int i = 0; i < DPL; i++) {
                const int d = lane + i * 64;
                if (d < a.hs) acc[i] += dj * ldb(kr, d);
            }
        }
    }
    for (int i = 0; i < DPL; i++) {
        const int d = lane + i * 64;
        if (d < a.hs) stb((T*)a.dq + ro, d, acc[i]);
    }
}

// dK, dV: one wavefront per key row, lanes over queries
template <typename T> __global__ __launch_bounds__(256) void attn_bwd_dkv_rows_kernel(AttnBwdArgs a)
{
    constexpr int DPL = 4;
    __shared__ float ks[4][256], vs[4][256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int key = blockIdx.x * 4 + wave;
    const int h = blockIdx.y, b = blockIdx.z;
    const bool valid = key < a.Tk;
    const size_t bh = (size_t)b * a.H + h;
    const size_t ko = (bh * a.Tk + (valid ? key : 0)) * a.hs;
    for (int d = lane; d < a.hs; d += 64) {
        ks[wave][d] = ldb((const T*)a.k + ko, d) * a.scale;
        vs[wave][d] = ldb((const T*)a.v + ko, d);
    }
    __syncthreads();
    if (!valid) return;
    const T* q = (const T*)a.q + bh * a.Tq * a.hs;
    const T* g = (const T*)a.dy + bh * a.Tq * a.hs;
    const float* lse = a.lse2 + bh * a.Tq;
    const float* dsm = a.dsum + bh * a.Tq;
    const float uniform = 1.0f / a.Tk;
    float accK[DPL] = {0.f, 0.f, 0.f, 0.f}, accV[DPL] = {0.f, 0.f, 0.f, 0.f};
    // causal: queries before the key never see it (no causal row is fully masked: the diagonal is kept)
    const int qstart = (a.kind == MASK_CAUSAL) ? (key / 64) * 64 : 0;
    for (int qb = qstart; qb < a.Tq; qb += 64) {
        const int i = qb + lane;
        float p = 0.f, ds = 0.f;
        if (i < a.Tq) {
            const T* qr = q + (size_t)i * a.hs;
            const T* gr = g + (size_t)i * a.hs;
            float s = 0.f, dp = 0.f;
            for (int d = 0; d < a.hs; d++) {
                s += ks[wave][d] * ldb(qr, d);
                dp += vs[wave][d] * ldb(gr, d);
            }
            p = attn_prob(s, attn_masked(a, b, i, key), lse[i], uniform);
            float pf, sf;
            attn_drop_factors(a, bh, i, key, &pf, &sf);
            ds = sf * p * (dp - dsm[i]) * a.scale;
            p *= pf;
        }
        const int cnt = min(64, a.Tq - qb);
        for (int ii = 0; ii < cnt; ii++) {
            const float pi = __shfl(p, ii, 64), di = __shfl(ds, ii, 64);
            if (pi == 0.f && di == 0.f) continue;   // wavefront-uniform: masked or underflowed entries add nothing
            const T* qr = q + (size_t)(qb + ii) * a.hs;
            const T* gr = g + (size_t)(qb + ii) * a.hs;
            for (int t = 0; t < DPL; t++) {
                const int d = lane + t * 64;
                if (d < a.hs) {
                    accV[t] += pi * ldb(gr, d);
                    accK[t] += di * ldb(qr, d);
                }
            }
        }
    }
    for (int t = 0; t < DPL; t++) {
        const int d = lane + t * 64;
        if (d < a.hs) {
            stb((T*)a.dk + ko, d, accK[t]);
            stb((T*)a.dv + ko, d, accV[t]);
        }
    }
}

bool attn_bwd_mfma_usable(DType dt, const AttnBwdArgs& a);
hipError_t attn_bwd_mfma_launch(hipStream_t s, DType dt, const AttnBwdArgs& a);

size_t attn_backward_workspace_bytes(int B, int H, int Tq) { return (size_t)B * H * Tq * 2 * sizeof(float); }

hipError_t k_attn_backward(hipStream_t s, DType dt, const void* q, const void* k, const void* v, const void* y, const void* dy,
                           void* dq, void* dk, void* dv, int B, int H, int Tq, int Tk, int hs, float scale, const float* mask,
                           MaskKind kind, const float* lse2, void* workspace, size_t workspaceBytes, const AttnDropout* dropout)
{
    if (B <= 0 || H <= 0 || Tq <= 0 || Tk <= 0 || hs <= 0) return hipSuccess;
    if (B > 65535 || H > 65535 || hs > 256) return hipErrorInvalidValue;
    if (kind != MASK_NONE && kind != MASK_CAUSAL && mask == nullptr) return hipErrorInvalidValue;
    if (workspaceBytes < attn_backward_workspace_bytes(B, H, Tq)) return hipErrorInvalidValue;
    AttnBwdArgs a;
    a.q = q; a.k = k; a.v = v; a.y = y; a.dy = dy; a.dq = dq; a.dk = dk; a.dv = dv; a.mask = mask;
    a.dsum = (float*)workspace;
    a.lse2 = lse2 ? const_cast<float*>(lse2) : a.dsum + (size_t)B * H * Tq;
    a.B = B; a.H = H; a.Tq = Tq; a.Tk = Tk; a.hs = hs; a.kind = (int)kind; a.scale = scale;
    a.computeLse = lse2 ? 0 : 1;
    dim3 gq((Tq + 3) / 4, H, B), gk((Tk + 3) / 4, H, B);
    a.useDropout = dropout ? 1 : 0;
    if (dropout) a.drop = *dropout;
    const bool mfma = !dropout && attn_bwd_mfma_usable(dt, a);
    // the statistics kernel is needed for lse2 when the forward pass left none, and for D whenever the row kernels run
    a.computeD = (mfma && lse2) ? 1 : 0;
    if (!a.computeD) {
        if (dt == F32) hipLaunchKernelGGL(attn_bwd_stats_kernel<float>, gq, 256, 0, s, a);
        else hipLaunchKernelGGL(attn_bwd_stats_kernel<bf16_t>, gq, 256, 0, s, a);
    }
    if (mfma) return attn_bwd_mfma_launch(s, dt, a);
    if (dt == F32) {
        hipLaunchKernelGGL(attn_bwd_dq_rows_kernel<float>, gq, 256, 0, s, a);
        hipLaunchKernelGGL(attn_bwd_dkv_rows_kernel<float>, gk, 256, 0, s, a);
    } else {
        hipLaunchKernelGGL(attn_bwd_dq_rows_kernel<bf16_t>, gq, 256, 0, s, a);
        hipLaunchKernelGGL(attn_bwd_dkv_rows_kernel<bf16_t>, gk, 256, 0, s, a);
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// MFMA tiles for head sizes 64 and 128, bf16 and fp32 storage (fragment conventions: flash_traits.h).
//
// A 32x32 accumulator keeps its column in the lane and its rows in the registers, and it can feed the next MFMA only
// as an operand whose contraction runs over those rows.  So each gradient is computed in the orientation whose
// contraction index is the one the probabilities have in registers:
//
//   dK, dV (attn_bwd_dkv_mfma_kernel): a wavefront owns 32 keys (lane = key) and walks the queries.
//       S  = Q K^T        A = Q rows from LDS,  B = K fragments held in registers
//       dP = dY V^T       A = dY rows from LDS, B = V fragments held in registers
//       P  = exp2(S c - lse2[query]),  dS = P (dP - D[query])       query = register row: lse2, D come from LDS
//       dV^T += dY^T P    A = dY^T from LDS (transposed while staged), B = P from registers
//       dK^T += Q^T dS    A = Q^T  from LDS (transposed while staged), B = dS from registers
//   dQ (attn_bwd_dq_mfma_kernel): a wavefront owns 32 queries (lane = query) and walks the keys.
//       S^T  = K Q^T      A = K rows from LDS,  B = Q fragments held in registers
//       dP^T = V dY^T     A = V rows from LDS,  B = dY fragments held in registers
//       P^T, dS^T as above with lse2, D per lane
//       dQ^T += K^T dS^T  A = K^T from LDS (transposed while staged), B = dS^T from registers
//
// The softmax scale is applied once to the dQ / dK accumulators at the end.  Every output row has exactly one owner
// and the order of accumulation is fixed, so results are reproducible run to run.  Causal launches skip the tiles above
// the diagonal and are ordered heaviest workgroup first.
template <typename T, int HS, int BS> struct BwdTile {
    typedef FlashTraits<T> TR;
    static constexpr int NT = 256;
    static constexpr int EPC = TR::EPC, CPF = TR::CPF;
    static constexpr int KF = HS / CPF;          // fragments along the head dimension
    static constexpr int PF = 32 / CPF;          // fragments along a 32-row step
    static constexpr int DT = HS / 32;
    static constexpr int PAD = 16 / (int)sizeof(T);
    // row-major LDS stride; rows of 256 bytes take two pads with TRR (the transposing read wants rows 32 bytes apart
    // modulo the banks: 288 bytes, where 272 halves its rate)
    static constexpr int LDR = (sizeof(T) == 2 && HS == 128) ? HS + 2 * PAD : HS + PAD;
    static constexpr int LDT = BS + PAD;         // transposed LDS stride
    // 16-bit storage, head sizes 64 and 128: the transposed operands are read from the ROW-MAJOR tiles with the transposing
    // LDS read (row stride 144 bytes suits it) instead of being scattered into transposed tiles two bytes at a time
    static constexpr bool TRR = sizeof(T) == 2 && (HS == 64 || HS == 128);
    static constexpr int CHR = HS / EPC;         // 16-byte chunks per row
    static constexpr int TPR = NT / BS;          // threads per staged row
    static constexpr int CPT = CHR / TPR;        // chunks per thread per staged array
    static_assert(CHR % TPR == 0 && CPT >= 1 && BS % 32 == 0, "stage / thread mismatch");
};

template <int KIND> __device__ inline bool bwd_masked(const AttnBwdArgs& a, int b, int mb, int qrow, int key, bool keyMasked)
{
    if (KIND == 1) return key > qrow;
    if (KIND == 2) return keyMasked;
    if (KIND == 3) return qrow < a.Tq && key < a.Tk && a.mask[((size_t)b * mb * a.Tq + qrow) * a.Tk + key] == 0.f;
    return false;
}

// KIND: 0 none, 1 causal, 2 key mask (B,Tk), 3 mask (B,Tq,Tk) or, with mb = 0, one (Tq,Tk) mask for all sequences
template <typename T, int HS, int KIND, int BQ, int OCC>
__global__ __launch_bounds__(256, OCC) void attn_bwd_dkv_mfma_kernel(AttnBwdArgs a, int mb)
{
    typedef BwdTile<T, HS, BQ> TL;
    typedef FlashTraits<T> TR;
    constexpr int NW = 4, BK = NW * 32;
    constexpr int EPC = TL::EPC, CPF = TL::CPF, KF = TL::KF, PF = TL::PF, DT = TL::DT, LDR = TL::LDR, LDT = TL::LDT;
    constexpr int TPR = TL::TPR, CPT = TL::CPT;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    T* Qs = (T*)bwd_smem;
    T* Gs = Qs + BQ * LDR;
    T* Qt = Gs + BQ * LDR;                       // the transposed tiles are not there with TRR
    T* Gt = Qt + HS * LDT;
    float* Ls = TL::TRR ? (float*)Qt : (float*)(Gt + HS * LDT);
    float* Ds = Ls + BQ;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int nbh = a.B * a.H;
    const int rank = KIND == 1 ? flash_causal_rank(OCC) : (int)blockIdx.x;
    const int kblock = rank / nbh;                  // causal: low key blocks see the most queries and start first
    const int ibh = rank % nbh;
    const int b = ibh / a.H, h = ibh % a.H;
    const size_t bh = (size_t)b * a.H + h;
    const int kw = kblock * BK + wave * 32;          // first key of this wavefront
    const int key = kw + l32;
    const bool waveActive = kw < a.Tk;
    const T* qp = (const T*)a.q + bh * a.Tq * HS;
    const T* gp = (const T*)a.dy + bh * a.Tq * HS;
    const T* kp = (const T*)a.k + bh * a.Tk * HS;
    const T* vp = (const T*)a.v + bh * a.Tk * HS;
    const float* lse = a.lse2 + bh * a.Tq;
    const float* dsm = a.dsum + bh * a.Tq;

    u32x4 kf[KF], vf[KF];
    {
        const size_t r = (size_t)min(key, a.Tk - 1) * HS;
#pragma unroll
        for (int f = 0; f < KF; f++) {
            kf[f] = *(const u32x4*)(kp + r + f * CPF + half * (CPF / 2));
            vf[f] = *(const u32x4*)(vp + r + f * CPF + half * (CPF / 2));
        }
    }
    bool keyMasked = false;
    if (KIND == 2) keyMasked = a.mask[(size_t)b * a.Tk + min(key, a.Tk - 1)] == 0.f;
    floatx16 ak[DT], av[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) { ak[dt][v] = 0.f; av[dt][v] = 0.f; }

    const int srow = tid % BQ, cg = tid / BQ;
    u32x4 qreg[CPT], greg[CPT];
    float lreg = 0.f, dreg = 0.f;
    auto gload = [&](int q0) {
        const size_t r = (size_t)min(q0 + srow, a.Tq - 1) * HS;
#pragma unroll
        for (int i = 0; i < CPT; i++) {
            qreg[i] = *(const u32x4*)(qp + r + (cg + TPR * i) * EPC);
            greg[i] = *(const u32x4*)(gp + r + (cg + TPR * i) * EPC);
        }
        if (tid < BQ) {
            const int qq = q0 + tid;
            // rows past the end get lse2 = +inf: their probabilities come out as exactly 0
            lreg = qq < a.Tq ? lse[qq] : INFINITY;
            dreg = qq < a.Tq ? dsm[qq] : 0.f;
        }
    };
    auto sstore = [&]() {
#pragma unroll
        for (int i = 0; i < CPT; i++) {
            const int c = cg + TPR * i;
            *(u32x4*)(&Qs[srow * LDR + c * EPC]) = qreg[i];
            *(u32x4*)(&Gs[srow * LDR + c * EPC]) = greg[i];
            if (!TL::TRR) {
                TR::scatter_chunk(&Qt[c * EPC * LDT + srow], LDT, qreg[i]);
                TR::scatter_chunk(&Gt[c * EPC * LDT + srow], LDT, greg[i]);
            }
        }
        if (tid < BQ) { Ls[tid] = lreg; Ds[tid] = dreg; }
    };

    const float c = a.scale * LOG2E;
    const float uniform = 1.0f / a.Tk;
    const int qbegin = (KIND == 1) ? (kblock * BK / BQ) * BQ : 0;   // causal: earlier queries see none of these keys
    if (qbegin < a.Tq) {
        gload(qbegin);
        sstore();
    }
#pragma unroll
    for (int f = 0; f < KF; f++) { asm volatile("" : "+v"(kf[f])); asm volatile("" : "+v"(vf[f])); }
    __syncthreads();
    for (int q0 = qbegin; q0 < a.Tq; q0 += BQ) {
        const bool more = q0 + BQ < a.Tq;
        if (more) gload(q0 + BQ);
        if (waveActive) {
#pragma unroll
            for (int sub = 0; sub < BQ / 32; sub++) {
                const int qs0 = q0 + 32 * sub;
                if (qs0 >= a.Tq) continue;
                if (KIND == 1 && qs0 + 31 < kw) continue;     // every (query, key) pair of the tile is masked
                floatx16 s, dp;
#pragma unroll
                for (int v = 0; v < 16; v++) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
                for (int f = 0; f < KF; f++) {
                    const u32x4 qa = *(const u32x4*)(&Qs[(sub * 32 + l32) * LDR + f * CPF + half * (CPF / 2)]);
                    s = TR::mma(qa, kf[f], s);
                    const u32x4 ga = *(const u32x4*)(&Gs[(sub * 32 + l32) * LDR + f * CPF + half * (CPF / 2)]);
                    dp = TR::mma(ga, vf[f], dp);
                }
                // register v: query qs0 + 8*(v/4) + 4*half + v%4, key = this lane's
                const bool maskedTile = (KIND >= 2) || (KIND == 1 && qs0 < kw + 31);   // wavefront-uniform
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4 l4 = *(const float4*)(&Ls[sub * 32 + 8 * g + 4 * half]);
                    const float4 d4 = *(const float4*)(&Ds[sub * 32 + 8 * g + 4 * half]);
                    const float lv[4] = {l4.x, l4.y, l4.z, l4.w}, dv4[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int v = 4 * g + j;
                        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -lv[j]));
                        if (maskedTile) {
                            const int qrow = qs0 + 8 * g + 4 * half + j;
                            if (bwd_masked<KIND>(a, b, mb, qrow, key, keyMasked)) p = 0.f;
                            if (KIND >= 2 && lv[j] == -INFINITY) p = uniform;   // fully masked row: uniform over all keys
                        }
                        s[v] = p;
                        dp[v] = p * (dp[v] - dv4[j]);
                    }
                }
#pragma unroll
                for (int t = 0; t < PF; t++) {
                    const u32x4 pp = TR::pack_p(s, t), dd = TR::pack_p(dp, t);
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        const u32x4 gt = TL::TRR ? TR::load_vt_rowmajor(&Gs[32 * sub * LDR + dt * 32], LDR, t, lane)
                                                 : TR::load_vt(&Gt[(dt * 32 + l32) * LDT + 32 * sub], t, half);
                        av[dt] = TR::mma(gt, pp, av[dt]);
                        const u32x4 qt = TL::TRR ? TR::load_vt_rowmajor(&Qs[32 * sub * LDR + dt * 32], LDR, t, lane)
                                                 : TR::load_vt(&Qt[(dt * 32 + l32) * LDT + 32 * sub], t, half);
                        ak[dt] = TR::mma(qt, dd, ak[dt]);
                    }
                }
            }
        }
        __syncthreads();
        if (more) sstore();
        __syncthreads();
    }
    // dk[key, d] = scale * dK^T[d, key]; register v of tile dt is d = 32*dt + 8*(v/4) + 4*half + v%4
    if (waveActive && key < a.Tk) {
        T* dkr = (T*)a.dk + (bh * a.Tk + key) * HS;
        T* dvr = (T*)a.dv + (bh * a.Tk + key) * HS;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = 32 * dt + 8 * g + 4 * half;
                TR::store4(dkr + d, ak[dt][4 * g] * a.scale, ak[dt][4 * g + 1] * a.scale, ak[dt][4 * g + 2] * a.scale,
                           ak[dt][4 * g + 3] * a.scale);
                TR::store4(dvr + d, av[dt][4 * g], av[dt][4 * g + 1], av[dt][4 * g + 2], av[dt][4 * g + 3]);
            }
    }
}

template <typename T, int HS, int KIND, int BKS, int OCC>
__global__ __launch_bounds__(256, OCC) void attn_bwd_dq_mfma_kernel(AttnBwdArgs a, int mb)
{
    typedef BwdTile<T, HS, BKS> TL;
    typedef FlashTraits<T> TR;
    constexpr int NW = 4, BM = NW * 32;
    constexpr int EPC = TL::EPC, CPF = TL::CPF, KF = TL::KF, PF = TL::PF, DT = TL::DT, LDR = TL::LDR, LDT = TL::LDT;
    constexpr int TPR = TL::TPR, CPT = TL::CPT;
    extern __shared__ __attribute__((aligned(16))) unsigned char bwd_smem[];
    T* Ks = (T*)bwd_smem;
    T* Vs = Ks + BKS * LDR;
    T* Kt = Vs + BKS * LDR;                      // not there with TRR
    float* Ms = TL::TRR ? (float*)Kt : (float*)(Kt + HS * LDT);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, half = lane >> 5;
    const int nbh = a.B * a.H;
    const int nqb = (a.Tq + BM - 1) / BM;
    const int rank = KIND == 1 ? flash_causal_rank(OCC) : (int)blockIdx.x;
    const int qblock = (KIND == 1) ? nqb - 1 - rank / nbh : rank / nbh;   // causal: heaviest first
    const int ibh = rank % nbh;
    const int b = ibh / a.H, h = ibh % a.H;
    const size_t bh = (size_t)b * a.H + h;
    const int q0w = qblock * BM + wave * 32;
    const int qrow = q0w + l32;
    const bool waveActive = q0w < a.Tq;
    const T* qp = (const T*)a.q + bh * a.Tq * HS;
    const T* gp = (const T*)a.dy + bh * a.Tq * HS;
    const T* kp = (const T*)a.k + bh * a.Tk * HS;
    const T* vp = (const T*)a.v + bh * a.Tk * HS;

    u32x4 qf[KF], gf[KF];
    {
        const size_t r = (size_t)min(qrow, a.Tq - 1) * HS;
#pragma unroll
        for (int f = 0; f < KF; f++) {
            qf[f] = *(const u32x4*)(qp + r + f * CPF + half * (CPF / 2));
            gf[f] = *(const u32x4*)(gp + r + f * CPF + half * (CPF / 2));
        }
    }
    const float lrow = qrow < a.Tq ? a.lse2[bh * a.Tq + qrow] : INFINITY;
    // D[row] = sum_d dY * Y.  When the statistics kernel did not run (the forward pass left lse2), it is computed here from
    // the dY fragments already in registers and stored for the dK/dV kernel, which is launched after this one.
    float drow = 0.f;
    if (a.computeD) {
        const T* yp = (const T*)a.y + bh * a.Tq * HS + (size_t)min(qrow, a.Tq - 1) * HS;
#pragma unroll
        for (int f = 0; f < KF; f++) drow += TR::dot(*(const u32x4*)(yp + f * CPF + half * (CPF / 2)), gf[f]);
        drow += __shfl_xor(drow, 32, 64);
        if (qrow < a.Tq && half == 0) a.dsum[bh * a.Tq + qrow] = drow;
        if (qrow >= a.Tq) drow = 0.f;
    } else if (qrow < a.Tq) {
        drow = a.dsum[bh * a.Tq + qrow];
    }
    floatx16 aq[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int v = 0; v < 16; v++) aq[dt][v] = 0.f;

    const int srow = tid % BKS, cg = tid / BKS;
    u32x4 kreg[CPT], vreg[CPT];
    float mreg = 1.f;
    auto gload = [&](int k0) {
        const size_t r = (size_t)min(k0 + srow, a.Tk - 1) * HS;
#pragma unroll
        for (int i = 0; i < CPT; i++) {
            kreg[i] = *(const u32x4*)(kp + r + (cg + TPR * i) * EPC);
            vreg[i] = *(const u32x4*)(vp + r + (cg + TPR * i) * EPC);
        }
        if (KIND == 2 && tid < BKS) mreg = (k0 + tid < a.Tk) ? a.mask[(size_t)b * a.Tk + k0 + tid] : 1.f;
    };
    auto sstore = [&]() {
#pragma unroll
        for (int i = 0; i < CPT; i++) {
            const int c = cg + TPR * i;
            *(u32x4*)(&Ks[srow * LDR + c * EPC]) = kreg[i];
            *(u32x4*)(&Vs[srow * LDR + c * EPC]) = vreg[i];
            if (!TL::TRR) TR::scatter_chunk(&Kt[c * EPC * LDT + srow], LDT, kreg[i]);
        }
        if (KIND == 2 && tid < BKS) Ms[tid] = mreg;
    };

    const float c = a.scale * LOG2E;
    const float uniform = 1.0f / a.Tk;
    int kend = a.Tk;
    if (KIND == 1) kend = min(a.Tk, qblock * BM + BM);
    gload(0);
    sstore();
#pragma unroll
    for (int f = 0; f < KF; f++) { asm volatile("" : "+v"(qf[f])); asm volatile("" : "+v"(gf[f])); }
    __syncthreads();
    for (int kb = 0; kb < kend; kb += BKS) {
        const bool more = kb + BKS < kend;
        if (more) gload(kb + BKS);
        if (waveActive) {
#pragma unroll
            for (int sub = 0; sub < BKS / 32; sub++) {
                const int k0 = kb + 32 * sub;
                if (k0 >= a.Tk) continue;
                if (KIND == 1 && k0 > q0w + 31) continue;     // keys past this wavefront's last row
                floatx16 s, dp;
#pragma unroll
                for (int v = 0; v < 16; v++) { s[v] = 0.f; dp[v] = 0.f; }
#pragma unroll
                for (int f = 0; f < KF; f++) {
                    const u32x4 ka = *(const u32x4*)(&Ks[(sub * 32 + l32) * LDR + f * CPF + half * (CPF / 2)]);
                    s = TR::mma(ka, qf[f], s);
                    const u32x4 va = *(const u32x4*)(&Vs[(sub * 32 + l32) * LDR + f * CPF + half * (CPF / 2)]);
                    dp = TR::mma(va, gf[f], dp);
                }
                // register v: key k0 + 8*(v/4) + 4*half + v%4, query = this lane's
                const bool maskedTile = (KIND >= 2) || (KIND == 1 && k0 + 31 > q0w) || (k0 + 32 > a.Tk);   // wavefront-uniform
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[v], c, -lrow));
                    if (maskedTile) {
                        const int kl = 8 * (v >> 2) + 4 * half + (v & 3);
                        const int key = k0 + kl;
                        if (bwd_masked<KIND>(a, b, mb, qrow, key, KIND == 2 && Ms[32 * sub + kl] == 0.f)) p = 0.f;
                        if (KIND >= 2 && lrow == -INFINITY) p = uniform;
                        if (key >= a.Tk) p = 0.f;
                    }
                    dp[v] = p * (dp[v] - drow);
                }
#pragma unroll
                for (int t = 0; t < PF; t++) {
                    const u32x4 dd = TR::pack_p(dp, t);
#pragma unroll
                    for (int dt = 0; dt < DT; dt++) {
                        const u32x4 kt = TL::TRR ? TR::load_vt_rowmajor(&Ks[32 * sub * LDR + dt * 32], LDR, t, lane)
                                                 : TR::load_vt(&Kt[(dt * 32 + l32) * LDT + 32 * sub], t, half);
                        aq[dt] = TR::mma(kt, dd, aq[dt]);
                    }
                }
            }
        }
        __syncthreads();
        if (more) sstore();
        __syncthreads();
    }
    if (waveActive && qrow < a.Tq) {
        T* dqr = (T*)a.dq + (bh * a.Tq + qrow) * HS;
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                TR::store4(dqr + 32 * dt + 8 * g + 4 * half, aq[dt][4 * g] * a.scale, aq[dt][4 * g + 1] * a.scale,
                           aq[dt][4 * g + 2] * a.scale, aq[dt][4 * g + 3] * a.scale);
    }
}

template <typename T, int HS, int BS, int OCC, int KIND>
static hipError_t bwd_launch_kind(hipStream_t s, const AttnBwdArgs& a, int mb)
{
    typedef BwdTile<T, HS, BS> TL;
    const size_t nT = TL::TRR ? 0 : 1;   // transposed tiles
    const size_t kvBytes = ((size_t)2 * BS * TL::LDR + nT * 2 * HS * TL::LDT) * sizeof(T) + 2 * BS * sizeof(float);
    const size_t qBytes = ((size_t)2 * BS * TL::LDR + nT * HS * TL::LDT) * sizeof(T) + BS * sizeof(float);
    auto kkv = attn_bwd_dkv_mfma_kernel<T, HS, KIND, BS, OCC>;
    auto kq = attn_bwd_dq_mfma_kernel<T, HS, KIND, BS, OCC>;
    static bool configured = false;   // per instantiation; the attribute is idempotent, so a race only repeats the call
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)kkv, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kvBytes);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void*)kq, hipFuncAttributeMaxDynamicSharedMemorySize, (int)qBytes);
        if (e != hipSuccess) return e;
        configured = true;
    }
    const int nbh = a.B * a.H;
    const long long gkv = (long long)((a.Tk + 127) / 128) * nbh, gq = (long long)((a.Tq + 127) / 128) * nbh;
    if (gkv > 0x7fffffffll || gq > 0x7fffffffll) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kq, dim3((unsigned)gq), 256, qBytes, s, a, mb);      // first: it may produce D for the other kernel
    hipLaunchKernelGGL(kkv, dim3((unsigned)gkv), 256, kvBytes, s, a, mb);
    return hipGetLastError();
}

template <typename T, int HS, int BS, int OCC> static hipError_t bwd_launch_cfg(hipStream_t s, const AttnBwdArgs& a, int kind, int mb)
{
    switch (kind) {
    case 0: return bwd_launch_kind<T, HS, BS, OCC, 0>(s, a, mb);
    case 1: return bwd_launch_kind<T, HS, BS, OCC, 1>(s, a, mb);
    case 2: return bwd_launch_kind<T, HS, BS, OCC, 2>(s, a, mb);
    default: return bwd_launch_kind<T, HS, BS, OCC, 3>(s, a, mb);
    }
}

bool attn_bwd_mfma_usable(DType, const AttnBwdArgs& a)
{
    if (a.hs != 64 && a.hs != 128) return false;
    return (((uintptr_t)a.q | (uintptr_t)a.k | (uintptr_t)a.v | (uintptr_t)a.y | (uintptr_t)a.dy | (uintptr_t)a.dq | (uintptr_t)a.dk |
             (uintptr_t)a.dv) & 15) == 0;
}

hipError_t attn_bwd_mfma_launch(hipStream_t s, DType dt, const AttnBwdArgs& a)
{
    int kind = 0, mb = 1;
    switch (a.kind) {
    case MASK_NONE: kind = 0; break;
    case MASK_CAUSAL: kind = 1; break;
    case MASK_KEY: kind = 2; break;
    case MASK_BQK: kind = 3; break;
    default: kind = 3; mb = 0; break;          // MASK_QK: one (Tq,Tk) mask for every sequence
    }
    if (dt == BF16) {
        if (a.hs == 64) return bwd_launch_cfg<bf16_t, 64, 64, 2>(s, a, kind, mb);
        return bwd_launch_cfg<bf16_t, 128, 32, 1>(s, a, kind, mb);
    }
    if (a.hs == 64) return bwd_launch_cfg<float, 64, 32, 2>(s, a, kind, mb);
    return bwd_launch_cfg<float, 128, 32, 1>(s, a, kind, mb);
}

}  // namespace mch
