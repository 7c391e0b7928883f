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
//  * attn_bwd_stats_kernel: D for every row and, when the forward pass left no lse2, lse2 as well (one wavefront a row).
//  * attn_bwd_dq_rows_kernel / attn_bwd_dkv_rows_kernel: any head size up to 256, any mask kind, Tq != Tk: one wavefront
//    per query row (per key row), lanes over the other sequence axis.  No atomics: every output row has one owner, so
//    results do not depend on scheduling.
//  * MFMA tiles for head sizes 64 and 128 (further down).
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
};

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
            ds = p * (dp - dsum) * a.scale;
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
            ds = p * (dp - dsm[i]) * a.scale;
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

hipError_t attn_bwd_mfma_launch(hipStream_t s, DType dt, const AttnBwdArgs& a, bool* handled);

size_t attn_backward_workspace_bytes(int B, int H, int Tq) { return (size_t)B * H * Tq * 2 * sizeof(float); }

hipError_t k_attn_backward(hipStream_t s, DType dt, const void* q, const void* k, const void* v, const void* y, const void* dy,
                           void* dq, void* dk, void* dv, int B, int H, int Tq, int Tk, int hs, float scale, const float* mask,
                           MaskKind kind, const float* lse2, void* workspace, size_t workspaceBytes)
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
    if (dt == F32) hipLaunchKernelGGL(attn_bwd_stats_kernel<float>, gq, 256, 0, s, a);
    else hipLaunchKernelGGL(attn_bwd_stats_kernel<bf16_t>, gq, 256, 0, s, a);
    bool handled = false;
    hipError_t e = attn_bwd_mfma_launch(s, dt, a, &handled);
    if (e != hipSuccess || handled) return e;
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
// MFMA path (placeholder dispatch until the tiles below are enabled per shape)
hipError_t attn_bwd_mfma_launch(hipStream_t, DType, const AttnBwdArgs&, bool* handled)
{
    *handled = false;
    return hipSuccess;
}

}  // namespace mch
