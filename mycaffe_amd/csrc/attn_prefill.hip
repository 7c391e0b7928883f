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

// MFMA flash kernels are added below this line -------------------------------------
hipError_t attn_flash_launch(hipStream_t, DType, const AttnArgs&, bool* handled)
{
    *handled = false;
    return hipSuccess;
}

}  // namespace mch
