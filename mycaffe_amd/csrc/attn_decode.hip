// Decode attention for gfx950: one query token per (batch, head) against a KV
// cache, HBM-bound.  The cache is streamed exactly once with 128-bit loads;
// the key axis is split across workgroups (split-K) so that even batch 1 fills
// 256 CUs, and a second small kernel merges the per-split (max, sum, acc)
// triples with the usual log-sum-exp algebra.
//
// Work layout inside a workgroup (4 wavefronts): a cache row of hs elements is
// covered by LPR = hs / (16 B / sizeof(T)) lanes (rounded up to a power of two),
// so one wavefront load instruction fetches 64/LPR consecutive rows, and four
// such loads per operand are kept in flight.  Each lane group keeps its own
// running max / sum / output slice; groups are merged through LDS at the end.
#include "kernels.h"

namespace mch {

template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int W = 4;
    __device__ static inline void load(const float* p, float* out)
    {
        float4 v = *(const float4*)p;
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    }
};
template <> struct Vec16<bf16_t> {
    static constexpr int W = 8;
    __device__ static inline void load(const bf16_t* p, float* out)
    {
        uint4 v = *(const uint4*)p;
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            out[2 * i] = __uint_as_float(u[i] << 16);
            out[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
        }
    }
};

template <typename T> __device__ inline float ld1(const T* p);
template <> __device__ inline float ld1<float>(const float* p) { return *p; }
template <> __device__ inline float ld1<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }
template <typename T> __device__ inline void st1(T* p, float v);
template <> __device__ inline void st1<float>(float* p, float v) { *p = v; }
template <> __device__ inline void st1<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

struct DecodeArgs {
    const void* q; const void* kc; const void* vc; void* y; float* part;
    int B, H, kvMul, hs, len, splits, chunk;
    long long strideB, strideH, strideT;
    float scale;
    // when dlen is set the number of cached positions is read on the device (so one
    // captured launch serves every decode step) and the per-split chunk is derived from it
    const int* dlen;
    int rowsPerIter;
};

__device__ inline void decode_range(const DecodeArgs& a, int split, int* t0, int* t1)
{
    int len = a.len, chunk = a.chunk;
    if (a.dlen) {
        len = *a.dlen;
        chunk = (len + a.splits - 1) / a.splits;
        chunk = ((chunk + a.rowsPerIter - 1) / a.rowsPerIter) * a.rowsPerIter;
    }
    *t0 = split * chunk;
    *t1 = min(len, *t0 + chunk);
}

// partial layout: part[((b*H + h)*splits + s) * (hs + 2)] = {m, l, acc[hs]}
template <typename T, int LPR>
__global__ __launch_bounds__(256) void attn_decode_kernel(DecodeArgs a)
{
    constexpr int W = Vec16<T>::W;
    constexpr int RPW = 64 / LPR;  // rows per wavefront load
    constexpr int U = 4;           // row groups in flight per operand
    constexpr int NW = 4;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane / LPR, gl = lane % LPR;
    const int d0 = gl * W;
    const bool active = d0 < a.hs;  // lanes beyond hs idle when hs/W is not a power of two

    const T* q = (const T*)a.q + ((size_t)b * a.H + h) * a.hs;
    const size_t base = (size_t)b * a.strideB + (size_t)(h / a.kvMul) * a.strideH;
    const T* kc = (const T*)a.kc + base;
    const T* vc = (const T*)a.vc + base;

    float qv[W];
#pragma unroll
    for (int i = 0; i < W; i++) qv[i] = 0.f;
    if (active) {
        Vec16<T>::load(q + d0, qv);
#pragma unroll
        for (int i = 0; i < W; i++) qv[i] *= a.scale;
    }

    int t0, t1;
    decode_range(a, split, &t0, &t1);

    float m = -INFINITY, l = 0.f, acc[W];
#pragma unroll
    for (int i = 0; i < W; i++) acc[i] = 0.f;

    for (int tb = t0 + wave * RPW * U; tb < t1; tb += NW * RPW * U) {
        float kv[U][W], vv[U][W];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            int t = tb + u * RPW + grp;
            ok[u] = t < t1;
#pragma unroll
            for (int i = 0; i < W; i++) { kv[u][i] = 0.f; vv[u][i] = 0.f; }
            if (ok[u] && active) Vec16<T>::load(kc + (size_t)t * a.strideT + d0, kv[u]);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            int t = tb + u * RPW + grp;
            if (ok[u] && active) Vec16<T>::load(vc + (size_t)t * a.strideT + d0, vv[u]);
        }
        float s[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            float d = 0.f;
#pragma unroll
            for (int i = 0; i < W; i++) d += qv[i] * kv[u][i];
#pragma unroll
            for (int o = LPR / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
            s[u] = ok[u] ? d : -INFINITY;
        }
        float mn = m;
#pragma unroll
        for (int u = 0; u < U; u++) mn = fmaxf(mn, s[u]);
        if (mn > -INFINITY) {
            float corr = __expf(m - mn);  // m == -inf gives 0
            l *= corr;
#pragma unroll
            for (int i = 0; i < W; i++) acc[i] *= corr;
#pragma unroll
            for (int u = 0; u < U; u++) {
                float p = __expf(s[u] - mn);  // masked rows: exp(-inf) = 0
                l += p;
#pragma unroll
                for (int i = 0; i < W; i++) acc[i] += p * vv[u][i];
            }
            m = mn;
        }
    }

    // merge the NW * RPW lane groups through LDS
    __shared__ float sm[NW * RPW];
    __shared__ float sl[NW * RPW];
    __shared__ float sacc[NW * RPW][LPR * W + 1];
    const int g = wave * RPW + grp;
    if (gl == 0) { sm[g] = m; sl[g] = l; }
    if (active) {
#pragma unroll
        for (int i = 0; i < W; i++) sacc[g][d0 + i] = acc[i];
    }
    __syncthreads();
    float M = -INFINITY;
    for (int i = 0; i < NW * RPW; i++) M = fmaxf(M, sm[i]);
    float* out = a.part + (((size_t)b * a.H + h) * a.splits + split) * (a.hs + 2);
    if (threadIdx.x == 0) {
        float L = 0.f;
        for (int i = 0; i < NW * RPW; i++) L += (sm[i] > -INFINITY) ? sl[i] * __expf(sm[i] - M) : 0.f;
        out[0] = M;
        out[1] = L;
    }
    for (int d = threadIdx.x; d < a.hs; d += 256) {
        float v = 0.f;
        for (int i = 0; i < NW * RPW; i++)
            if (sm[i] > -INFINITY) v += sacc[i][d] * __expf(sm[i] - M);
        out[2 + d] = v;
    }
}

// any head size / alignment: scalar loads, one wavefront per (b, h, split)
template <typename T> __global__ __launch_bounds__(64) void attn_decode_scalar_kernel(DecodeArgs a)
{
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x;
    const T* q = (const T*)a.q + ((size_t)b * a.H + h) * a.hs;
    const size_t base = (size_t)b * a.strideB + (size_t)(h / a.kvMul) * a.strideH;
    const T* kc = (const T*)a.kc + base;
    const T* vc = (const T*)a.vc + base;
    int t0, t1;
    decode_range(a, split, &t0, &t1);
    constexpr int DPL = 8;  // output dims per lane: hs <= 512
    float m = -INFINITY, l = 0.f, acc[DPL];
    for (int i = 0; i < DPL; i++) acc[i] = 0.f;
    for (int tb = t0; tb < t1; tb += 64) {
        int t = tb + lane;
        float s = -INFINITY;
        if (t < t1) {
            float d = 0.f;
            for (int i = 0; i < a.hs; i++) d += ld1(q + i) * ld1(kc + (size_t)t * a.strideT + i);
            s = d * a.scale;
        }
        float mx = s;
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        float mn = fmaxf(m, mx);
        float corr = __expf(m - mn);
        float p = __expf(s - mn);
        float ps = p;
        for (int o = 32; o > 0; o >>= 1) ps += __shfl_xor(ps, o, 64);
        l = l * corr + ps;
        for (int i = 0; i < DPL; i++) acc[i] *= corr;
        int cnt = min(64, t1 - tb);
        for (int j = 0; j < cnt; j++) {
            float pj = __shfl(p, j, 64);
            for (int i = 0; i < DPL; i++) {
                int d = lane + i * 64;
                if (d < a.hs) acc[i] += pj * ld1(vc + (size_t)(tb + j) * a.strideT + d);
            }
        }
        m = mn;
    }
    float* out = a.part + (((size_t)b * a.H + h) * a.splits + split) * (a.hs + 2);
    if (lane == 0) { out[0] = m; out[1] = l; }
    for (int i = 0; i < DPL; i++) {
        int d = lane + i * 64;
        if (d < a.hs) out[2 + d] = acc[i];
    }
}

template <typename T>
__global__ void attn_decode_merge_kernel(const float* __restrict__ part, T* __restrict__ y, int hs, int splits)
{
    const size_t bh = blockIdx.x;
    const float* p = part + bh * splits * (size_t)(hs + 2);
    float M = -INFINITY;
    for (int s = 0; s < splits; s++) M = fmaxf(M, p[(size_t)s * (hs + 2)]);
    float L = 0.f;
    for (int s = 0; s < splits; s++) {
        float ms = p[(size_t)s * (hs + 2)];
        if (ms > -INFINITY) L += p[(size_t)s * (hs + 2) + 1] * __expf(ms - M);
    }
    for (int d = threadIdx.x; d < hs; d += blockDim.x) {
        float v = 0.f;
        for (int s = 0; s < splits; s++) {
            float ms = p[(size_t)s * (hs + 2)];
            if (ms > -INFINITY) v += p[(size_t)s * (hs + 2) + 2 + d] * __expf(ms - M);
        }
        st1(y + bh * hs + d, v / L);
    }
}

static void pick_splits(int B, int H, int len, int rows_per_iter, int* splits, int* chunk)
{
    // aim for >= 4 workgroups per CU; never less than one full iteration per split
    long long bh = (long long)B * H;
    int want = (int)((1024 + bh - 1) / bh);
    int maxs = (len + rows_per_iter - 1) / rows_per_iter;
    int s = want < 1 ? 1 : want;
    if (s > maxs) s = maxs;
    if (s < 1) s = 1;
    if (s > 256) s = 256;
    int c = (len + s - 1) / s;
    c = ((c + rows_per_iter - 1) / rows_per_iter) * rows_per_iter;
    s = (len + c - 1) / c;
    *splits = s;
    *chunk = c;
}

size_t attn_decode_workspace_bytes(int B, int H, int hs, int len)
{
    // pick_splits never asks for more than ceil(1024 / (B*H)) splits (256 at most)
    (void)len;
    long long bh = (long long)B * H;
    long long want = (1024 + bh - 1) / bh;
    if (want > 256) want = 256;
    if (want < 1) want = 1;
    return (size_t)(bh * want) * (size_t)(hs + 2) * sizeof(float);
}

template <typename T>
static hipError_t launch_decode(hipStream_t s, DecodeArgs a, int kvH)
{
    constexpr int W = Vec16<T>::W;
    (void)kvH;
    int lpr = (a.hs + W - 1) / W;
    int lprp = 1;
    while (lprp < lpr) lprp <<= 1;
    bool fast = (a.hs % W == 0) && lprp <= 64 && (a.strideT % W == 0) && (a.strideH % W == 0) && (a.strideB % W == 0) &&
                (((uintptr_t)a.q | (uintptr_t)a.kc | (uintptr_t)a.vc) % 16 == 0);
    if (fast) {
        int rpi = 4 * (64 / lprp) * 4;
        a.rowsPerIter = rpi;
        pick_splits(a.B, a.H, a.len, rpi, &a.splits, &a.chunk);
        dim3 grid(a.splits, a.H, a.B);
        switch (lprp) {
#define CASE(L) case L: hipLaunchKernelGGL((attn_decode_kernel<T, L>), grid, 256, 0, s, a); break;
            CASE(1) CASE(2) CASE(4) CASE(8) CASE(16) CASE(32) CASE(64)
#undef CASE
        }
    } else {
        if (a.hs > 512) return hipErrorInvalidValue;
        a.rowsPerIter = 64;
        pick_splits(a.B, a.H, a.len, 64, &a.splits, &a.chunk);
        dim3 grid(a.splits, a.H, a.B);
        hipLaunchKernelGGL(attn_decode_scalar_kernel<T>, grid, 64, 0, s, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    int mt = a.hs <= 64 ? 64 : (a.hs <= 128 ? 128 : 256);
    hipLaunchKernelGGL(attn_decode_merge_kernel<T>, a.B * a.H, mt, 0, s, a.part, (T*)a.y, a.hs, a.splits);
    return hipGetLastError();
}

hipError_t k_attn_decode(hipStream_t s, DType dt, const void* q, const void* kc, const void* vc, void* y, int B, int H,
                         int kvH, int hs, int len, long long strideB, long long strideH, long long strideT, float scale,
                         void* workspace, size_t workspaceBytes, const int* dlen)
{
    if (B <= 0 || H <= 0 || hs <= 0 || len <= 0) return hipSuccess;
    if (kvH <= 0 || H % kvH != 0) return hipErrorInvalidValue;
    if (B > 65535 || H > 65535) return hipErrorInvalidValue;
    if (workspaceBytes < attn_decode_workspace_bytes(B, H, hs, len)) return hipErrorInvalidValue;
    DecodeArgs a;
    a.q = q; a.kc = kc; a.vc = vc; a.y = y; a.part = (float*)workspace;
    a.B = B; a.H = H; a.kvMul = H / kvH; a.hs = hs; a.len = len; a.splits = 1; a.chunk = len;
    a.strideB = strideB; a.strideH = strideH; a.strideT = strideT; a.scale = scale;
    a.dlen = dlen; a.rowsPerIter = 64;
    if (dt == F32) return launch_decode<float>(s, a, kvH);
    return launch_decode<bf16_t>(s, a, kvH);
}

// rotate q and the new key at `pos` (adjacent-pair convention) and store the new
// key / value rows into the caches; one thread per pair / per value element
template <typename T>
__global__ void rope_append_kernel(T* q, T* knew, const T* vnew, T* kc, T* vc, int B, int H, int kvH, int hs, int pos,
                                   long long strideB, long long strideH, long long strideT, const float* fcos,
                                   const float* fsin)
{
    const int half = hs / 2;
    size_t nq = (size_t)B * H * half, nk = (size_t)B * kvH * half, nv = (size_t)B * kvH * hs;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < nq + nk + nv; i += (size_t)blockDim.x * gridDim.x) {
        if (i < nq) {
            int j = (int)(i % half);
            float c = fcos ? fcos[(size_t)pos * half + j] : 1.f, sn = fsin ? fsin[(size_t)pos * half + j] : 0.f;
            float re = ld1(q + 2 * i), im = ld1(q + 2 * i + 1);
            st1(q + 2 * i, re * c - im * sn);
            st1(q + 2 * i + 1, re * sn + im * c);
        } else if (i < nq + nk) {
            size_t p = i - nq;
            int j = (int)(p % half);
            size_t bh = p / half;
            int hh = (int)(bh % kvH);
            size_t bb = bh / kvH;
            float c = fcos ? fcos[(size_t)pos * half + j] : 1.f, sn = fsin ? fsin[(size_t)pos * half + j] : 0.f;
            float re = ld1(knew + 2 * p), im = ld1(knew + 2 * p + 1);
            float r0 = re * c - im * sn, r1 = re * sn + im * c;
            st1(knew + 2 * p, r0);
            st1(knew + 2 * p + 1, r1);
            size_t dst = bb * strideB + (size_t)hh * strideH + (size_t)pos * strideT + 2 * j;
            st1(kc + dst, r0);
            st1(kc + dst + 1, r1);
        } else {
            size_t p = i - nq - nk;
            int d = (int)(p % hs);
            size_t bh = p / hs;
            int hh = (int)(bh % kvH);
            size_t bb = bh / kvH;
            vc[bb * strideB + (size_t)hh * strideH + (size_t)pos * strideT + d] = vnew[p];
        }
    }
}

hipError_t k_rope_append(hipStream_t s, DType dt, void* q, void* knew, const void* vnew, void* kc, void* vc, int B, int H,
                         int kvH, int hs, int pos, long long strideB, long long strideH, long long strideT,
                         const float* fcos, const float* fsin)
{
    size_t n = (size_t)B * H * (hs / 2) + (size_t)B * kvH * (hs / 2) + (size_t)B * kvH * hs;
    if (n == 0) return hipSuccess;
    int grid = (int)((n + 255) / 256);
    if (grid > 4096) grid = 4096;
    if (dt == F32)
        hipLaunchKernelGGL(rope_append_kernel<float>, grid, 256, 0, s, (float*)q, (float*)knew, (const float*)vnew, (float*)kc,
                           (float*)vc, B, H, kvH, hs, pos, strideB, strideH, strideT, fcos, fsin);
    else
        hipLaunchKernelGGL(rope_append_kernel<bf16_t>, grid, 256, 0, s, (bf16_t*)q, (bf16_t*)knew, (const bf16_t*)vnew,
                           (bf16_t*)kc, (bf16_t*)vc, B, H, kvH, hs, pos, strideB, strideH, strideT, fcos, fsin);
    return hipGetLastError();
}

}  // namespace mch
