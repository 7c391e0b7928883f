// Elementwise, layout, softmax, RoPE and RMSNorm kernels for gfx950.
// All are HBM-bound: one pass over the data, 64-wide wavefronts, 128-bit
// accesses where the layout allows, grid sized to a few waves per CU.
#include "kernels.h"
#include "lane_ops.h"

namespace mch {

static constexpr int TPB = 256;

static inline int grid_for(size_t n, int per_thread = 1)
{
    size_t blocks = (n + (size_t)TPB * per_thread - 1) / ((size_t)TPB * per_thread);
    if (blocks < 1) blocks = 1;
    if (blocks > 256 * 16) blocks = 256 * 16;  // 256 CUs x 16 resident workgroups
    return (int)blocks;
}

template <typename T> __device__ inline float ld(const T* p, size_t i);
template <> __device__ inline float ld<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ inline float ld<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ inline void st(T* p, size_t i, float v);
template <> __device__ inline void st<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ inline void st<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

#define GRID_STRIDE(i, n) \
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < (n); i += (size_t)blockDim.x * gridDim.x)

#define DISPATCH_DT(dt, CALL)            \
    do {                                 \
        if ((dt) == F32) { typedef float T; CALL; } else { typedef bf16_t T; CALL; } \
    } while (0)

// ---------------------------------------------------------------------------
// Elementwise maps y = f(a, b): eight elements per thread and trip (one 16-byte access for bf16, two for fp32) when all
// operands are 16-byte aligned, one element per thread otherwise and for the tail.
typedef __bf16 ew_bf16x2 __attribute__((ext_vector_type(2)));
typedef float ew_floatx2 __attribute__((ext_vector_type(2)));
// two fp32 -> packed bf16 pair with the hardware conversion (round to nearest even)
__device__ inline uint32_t pack2_bf16_hw(float a, float b)
{
    ew_floatx2 f = {a, b};
    ew_bf16x2 r = __builtin_convertvector(f, ew_bf16x2);
    return *reinterpret_cast<uint32_t*>(&r);
}

template <typename T> struct Vec8;
template <> struct Vec8<float> {
    __device__ static inline void load(const float* p, float (&v)[8])
    {
        const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
    __device__ static inline void store(float* p, const float (&v)[8])
    {
        *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
        *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
};
template <> struct Vec8<bf16_t> {
    __device__ static inline void load(const bf16_t* p, float (&v)[8])
    {
        const uint4 a = *(const uint4*)p;
        const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ static inline void store(bf16_t* p, const float (&v)[8])
    {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = pack2_bf16_hw(v[2 * i], v[2 * i + 1]);
        *(uint4*)p = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

template <typename T, bool TWO, typename F> __global__ void map_kernel(size_t n, size_t chunks, const T* a, const T* b, T* y, F f)
{
    const size_t gid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (size_t)blockDim.x * gridDim.x;
    for (size_t c = gid; c < chunks; c += stride) {
        float va[8], vb[8], r[8];
        Vec8<T>::load(a + c * 8, va);
        if (TWO) Vec8<T>::load(b + c * 8, vb);
#pragma unroll
        for (int j = 0; j < 8; j++) r[j] = f(va[j], TWO ? vb[j] : 0.f);
        Vec8<T>::store(y + c * 8, r);
    }
    for (size_t i = chunks * 8 + gid; i < n; i += stride) st(y, i, f(ld(a, i), TWO ? ld(b, i) : 0.f));
}

// y = f(a) (b == nullptr) or y = f(a, b)
template <typename F> static hipError_t launch_map(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y, F f)
{
    if (n == 0) return hipSuccess;
    const bool aligned = ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) & 15) == 0);
    const size_t chunks = aligned ? n / 8 : 0;
    const int g = grid_for(chunks ? chunks : n);
    if (b) DISPATCH_DT(dt, hipLaunchKernelGGL((map_kernel<T, true, F>), g, TPB, 0, s, n, chunks, (const T*)a, (const T*)b, (T*)y, f));
    else DISPATCH_DT(dt, hipLaunchKernelGGL((map_kernel<T, false, F>), g, TPB, 0, s, n, chunks, (const T*)a, (const T*)a, (T*)y, f));
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
template <typename T> __global__ void set_kernel(T* y, size_t n, float v) { GRID_STRIDE(i, n) st(y, i, v); }

hipError_t k_set(hipStream_t s, DType dt, void* y, size_t n, float v)
{
    if (n == 0) return hipSuccess;
    DISPATCH_DT(dt, hipLaunchKernelGGL(set_kernel<T>, grid_for(n), TPB, 0, s, (T*)y, n, v));
    return hipGetLastError();
}

template <typename S, typename D> __global__ void convert_kernel(const S* x, D* y, size_t n)
{
    GRID_STRIDE(i, n) st(y, i, ld(x, i));
}

hipError_t k_convert(hipStream_t s, DType sdt, const void* src, DType ddt, void* dst, size_t n)
{
    if (n == 0) return hipSuccess;
    int g = grid_for(n);
    if (sdt == F32 && ddt == F32)
        return hipMemcpyAsync(dst, src, n * sizeof(float), hipMemcpyDeviceToDevice, s);
    if (sdt == BF16 && ddt == BF16)
        return hipMemcpyAsync(dst, src, n * sizeof(bf16_t), hipMemcpyDeviceToDevice, s);
    if (sdt == F32)
        hipLaunchKernelGGL((convert_kernel<float, bf16_t>), g, TPB, 0, s, (const float*)src, (bf16_t*)dst, n);
    else
        hipLaunchKernelGGL((convert_kernel<bf16_t, float>), g, TPB, 0, s, (const bf16_t*)src, (float*)dst, n);
    return hipGetLastError();
}

struct AxpyF { float a; __device__ float operator()(float x, float y) const { return a * x + y; } };
struct ScaleF { float a; __device__ float operator()(float x, float) const { return a * x; } };
struct AddF { float alpha; __device__ float operator()(float a, float b) const { return a + b * alpha; } };
struct MulF { __device__ float operator()(float a, float b) const { return a * b; } };
__device__ inline float silu_f(float x) { return x * (1.0f / (1.0f + expf(-x))); }
struct SiluF { __device__ float operator()(float x, float) const { return silu_f(x); } };
struct SwigluF { __device__ float operator()(float a, float b) const { return silu_f(a) * b; } };

hipError_t k_axpy(hipStream_t s, DType dt, size_t n, float alpha, const void* x, void* y) { return launch_map(s, dt, n, x, y, y, AxpyF{alpha}); }
hipError_t k_scale(hipStream_t s, DType dt, size_t n, float alpha, const void* x, void* y) { return launch_map(s, dt, n, x, nullptr, y, ScaleF{alpha}); }
hipError_t k_add(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y, float alpha) { return launch_map(s, dt, n, a, b, y, AddF{alpha}); }
hipError_t k_mul(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y) { return launch_map(s, dt, n, a, b, y, MulF{}); }
hipError_t k_silu(hipStream_t s, DType dt, size_t n, const void* x, void* y) { return launch_map(s, dt, n, x, nullptr, y, SiluF{}); }
hipError_t k_swiglu(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y) { return launch_map(s, dt, n, a, b, y, SwigluF{}); }

// y[i] = mask[i % maskDim] == search ? replace : xscale * x[i]   (xscale: a scaling of x that the caller had deferred; 1 otherwise)
template <typename T>
__global__ void mask_kernel(size_t n, int maskDim, const T* x, const T* mask, T* y, float search, float replace, float xscale)
{
    GRID_STRIDE(i, n) st(y, i, ld(mask, i % (size_t)maskDim) == search ? replace : xscale * ld(x, i));
}
// mask index = i % md1 + (i / dd1) * md1 (md1 = maskDim / batch, dd1 = n / batch); the plain mask is the case dd1 = n
template <typename T>
__global__ void mask_batch_kernel(size_t n, int md1, size_t dd1, const T* x, const T* mask, T* y, float search,
                                  float replace, float xscale)
{
    GRID_STRIDE(i, n)
    {
        size_t mi = i % (size_t)md1 + (i / dd1) * (size_t)md1;
        st(y, i, ld(mask, mi) == search ? replace : xscale * ld(x, i));
    }
}
// eight elements per thread: needs md1 and dd1 to be multiples of 8 (a chunk never wraps) and 16-byte aligned operands
template <typename T>
__global__ void mask_vec_kernel(size_t chunks, size_t md8, size_t dd8, const T* x, const T* mask, T* y, float search, float replace,
                                float xscale)
{
    GRID_STRIDE(c, chunks)
    {
        const size_t mc = c % md8 + (c / dd8) * md8;
        float vx[8], vm[8];
        Vec8<T>::load(x + c * 8, vx);
        Vec8<T>::load(mask + mc * 8, vm);
#pragma unroll
        for (int k = 0; k < 8; k++) vx[k] = vm[k] == search ? replace : xscale * vx[k];
        Vec8<T>::store(y + c * 8, vx);
    }
}
static hipError_t launch_mask(hipStream_t s, DType dt, size_t n, int md1, size_t dd1, float search, float replace, const void* x,
                              const void* mask, void* y, float xscale)
{
    const bool vec = md1 % 8 == 0 && dd1 % 8 == 0 && n % 8 == 0 && ((((uintptr_t)x | (uintptr_t)mask | (uintptr_t)y) & 15) == 0);
    if (vec) {
        DISPATCH_DT(dt, hipLaunchKernelGGL(mask_vec_kernel<T>, grid_for(n / 8), TPB, 0, s, n / 8, (size_t)md1 / 8, dd1 / 8, (const T*)x,
                                           (const T*)mask, (T*)y, search, replace, xscale));
    } else {
        DISPATCH_DT(dt, hipLaunchKernelGGL(mask_batch_kernel<T>, grid_for(n), TPB, 0, s, n, md1, dd1, (const T*)x, (const T*)mask,
                                           (T*)y, search, replace, xscale));
    }
    return hipGetLastError();
}
hipError_t k_mask(hipStream_t s, DType dt, size_t n, int maskDim, float search, float replace, const void* x,
                  const void* mask, void* y, float xscale)
{
    if (n == 0) return hipSuccess;
    if (maskDim % 8 == 0 && n % (size_t)maskDim == 0)
        return launch_mask(s, dt, n, maskDim, n, search, replace, x, mask, y, xscale);   // i % maskDim with dd1 = n: one "batch"
    DISPATCH_DT(dt, hipLaunchKernelGGL(mask_kernel<T>, grid_for(n), TPB, 0, s, n, maskDim, (const T*)x, (const T*)mask,
                                       (T*)y, search, replace, xscale));
    return hipGetLastError();
}
hipError_t k_mask_batch(hipStream_t s, DType dt, size_t n, int batch, int maskDim, float search, float replace,
                        const void* x, const void* mask, void* y, float xscale)
{
    if (n == 0) return hipSuccess;
    return launch_mask(s, dt, n, maskDim / batch, n / (size_t)batch, search, replace, x, mask, y, xscale);
}

// Generic permute: xc / yc hold the element strides of the source / destination
// axes as floats, map[i] the source axis feeding destination axis i.  The
// per-element index scratch of the reference kernel is replaced by registers.

template <typename T> __global__ void transpose_kernel(size_t n, const T* x, T* y, PermuteArgs a)
{
    GRID_STRIDE(i, n)
    {
        int from[8];
        size_t rem = i;
        for (int d = 0; d < a.axes; d++) {
            from[d] = (int)(rem / (size_t)a.xs[d]);
            rem = rem % (size_t)a.xs[d];
        }
        size_t to = 0;
        for (int d = 0; d < a.axes; d++) to += (size_t)from[a.map[d]] * (size_t)a.ys[d];
        y[to] = x[i];
    }
}

// (B, d1, d2, inner) -> (B, d2, d1, inner): the head split / merge of the attention layers
template <typename T>
__global__ void transpose12_kernel(const T* __restrict__ x, T* __restrict__ y, int d1, int d2, int inner, size_t n)
{
    GRID_STRIDE(o, n)
    {
        int in = (int)(o % inner);
        size_t r = o / inner;
        int a1 = (int)(r % d1);
        r /= d1;
        int a2 = (int)(r % d2);
        size_t b = r / d2;
        y[o] = x[((b * d1 + a1) * d2 + a2) * (size_t)inner + in];
    }
}

// the same with 16-byte chunks along the inner axis (inner counts chunks)
__global__ void transpose12_vec_kernel(const uint4* __restrict__ x, uint4* __restrict__ y, int d1, int d2, int inner, size_t n)
{
    GRID_STRIDE(o, n)
    {
        int in = (int)(o % inner);
        size_t r = o / inner;
        int a1 = (int)(r % d1);
        r /= d1;
        int a2 = (int)(r % d2);
        size_t b = r / d2;
        y[o] = x[((b * d1 + a1) * d2 + a2) * (size_t)inner + in];
    }
}

hipError_t k_transpose_hw(hipStream_t s, DType dt, int nc, int h, int w, const void* x, void* y);

// reads the three small float blobs (source strides, destination strides, axis map) from the device: one round trip
hipError_t k_transpose_fetch(hipStream_t s, const float* xc, const float* yc, const float* map, int axes, PermuteArgs* out)
{
    if (axes < 1 || axes > 8) return hipErrorInvalidValue;
    float hx[8], hy[8], hm[8];
    hipError_t e;
    if ((e = hipMemcpyAsync(hx, xc, axes * sizeof(float), hipMemcpyDeviceToHost, s)) != hipSuccess) return e;
    if ((e = hipMemcpyAsync(hy, yc, axes * sizeof(float), hipMemcpyDeviceToHost, s)) != hipSuccess) return e;
    if ((e = hipMemcpyAsync(hm, map, axes * sizeof(float), hipMemcpyDeviceToHost, s)) != hipSuccess) return e;
    if ((e = hipStreamSynchronize(s)) != hipSuccess) return e;
    out->axes = axes;
    for (int i = 0; i < axes; i++) {
        out->xs[i] = (int)hx[i];
        out->ys[i] = (int)hy[i];
        out->map[i] = (int)hm[i];
        if (out->xs[i] < 1 || out->ys[i] < 1 || out->map[i] < 0 || out->map[i] >= axes) return hipErrorInvalidValue;
    }
    return hipSuccess;
}

hipError_t k_transpose_run(hipStream_t s, DType dt, size_t n, const void* x, void* y, const PermuteArgs& a)
{
    if (n == 0) return hipSuccess;
    const int axes = a.axes;
    const size_t es = dt == F32 ? 4 : 2;
    // fast path: 4 axes, axes 1 and 2 swapped, coalesced along the untouched inner axis
    if (axes == 4 && a.map[0] == 0 && a.map[1] == 2 && a.map[2] == 1 && a.map[3] == 3 && a.xs[3] == 1 && a.ys[3] == 1) {
        int inner = a.xs[2];
        int d2 = a.xs[1] / a.xs[2];
        int d1 = a.xs[0] / a.xs[1];
        if (a.ys[2] == inner && a.ys[1] == inner * d1 && a.ys[0] == inner * d1 * d2) {
            const int vec = (int)(16 / es);
            if (inner % vec == 0 && ((((uintptr_t)x | (uintptr_t)y) & 15) == 0)) {
                hipLaunchKernelGGL(transpose12_vec_kernel, grid_for(n / vec), TPB, 0, s, (const uint4*)x, (uint4*)y, d1, d2, inner / vec,
                                   n / vec);
                return hipGetLastError();
            }
            DISPATCH_DT(dt, hipLaunchKernelGGL(transpose12_kernel<T>, grid_for(n), TPB, 0, s, (const T*)x, (T*)y, d1, d2,
                                               inner, n));
            return hipGetLastError();
        }
    }
    // fast path: the last two axes swapped, everything in front untouched: tiled transpose through LDS
    if (axes >= 2 && a.xs[axes - 1] == 1 && a.ys[axes - 1] == 1) {
        bool lead = a.map[axes - 1] == axes - 2 && a.map[axes - 2] == axes - 1;
        for (int i = 0; i + 2 < axes; i++) lead = lead && a.map[i] == i && a.xs[i] == a.ys[i];
        const int w = a.xs[axes - 2], h = a.ys[axes - 2];   // source rows have w elements, destination rows h
        if (lead && w > 0 && h > 0 && n % ((size_t)w * h) == 0 && (axes < 3 || a.xs[axes - 3] == w * h) && n / ((size_t)w * h) <= 65535)
            return k_transpose_hw(s, dt, (int)(n / ((size_t)w * h)), h, w, x, y);
    }
    DISPATCH_DT(dt, hipLaunchKernelGGL(transpose_kernel<T>, grid_for(n), TPB, 0, s, n, (const T*)x, (T*)y, a));
    return hipGetLastError();
}

hipError_t k_transpose(hipStream_t s, DType dt, size_t n, const void* x, void* y, const float* xc, const float* yc,
                       const float* map, int axes)
{
    if (n == 0) return hipSuccess;
    PermuteArgs a;
    hipError_t e = k_transpose_fetch(s, xc, yc, map, axes, &a);
    if (e != hipSuccess) return e;
    return k_transpose_run(s, dt, n, x, y, a);
}

// (nc, h, w) -> (nc, w, h) through a padded LDS tile so both sides are coalesced
template <typename T> __global__ void transpose_hw_kernel(const T* __restrict__ x, T* __restrict__ y, int h, int w)
{
    __shared__ T tile[32][33];
    size_t base = (size_t)blockIdx.z * h * w;
    int x0 = blockIdx.x * 32, y0 = blockIdx.y * 32;
    int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int j = ty; j < 32; j += 8)
        if (y0 + j < h && x0 + tx < w) tile[j][tx] = x[base + (size_t)(y0 + j) * w + x0 + tx];
    __syncthreads();
    for (int j = ty; j < 32; j += 8)
        if (x0 + j < w && y0 + tx < h) y[base + (size_t)(x0 + j) * h + y0 + tx] = tile[tx][j];
}

hipError_t k_transpose_hw(hipStream_t s, DType dt, int nc, int h, int w, const void* x, void* y)
{
    if (nc <= 0 || h <= 0 || w <= 0) return hipSuccess;
    dim3 grid((w + 31) / 32, (h + 31) / 32, nc);
    if (grid.z > 65535 || grid.y > 65535) return hipErrorInvalidValue;
    DISPATCH_DT(dt, hipLaunchKernelGGL(transpose_hw_kernel<T>, grid, TPB, 0, s, (const T*)x, (T*)y, h, w));
    return hipGetLastError();
}

// X viewed as (num, channels, blocks, inner), Y as (num, channels, inner);
// dir 0: Y = X[:, :, offset, :], else X[:, :, offset, :] = Y
template <typename T>
__global__ void channel_copy_kernel(size_t n, int channels, int blocks, int inner, int offset, T* x, T* y, int dir)
{
    GRID_STRIDE(i, n)
    {
        size_t nn = i / ((size_t)channels * inner);
        size_t c = (i % ((size_t)channels * inner)) / inner;
        size_t b = i % inner;
        size_t xi = (nn * channels + c) * (size_t)blocks * inner + (size_t)offset * inner + b;
        if (dir == 0) y[i] = x[xi];
        else x[xi] = y[i];
    }
}
// the same on 16-byte chunks (inner counts chunks)
__global__ void channel_copy_vec_kernel(size_t n, int channels, int blocks, int inner, int offset, uint4* x, uint4* y, int dir)
{
    GRID_STRIDE(i, n)
    {
        size_t nn = i / ((size_t)channels * inner);
        size_t c = (i % ((size_t)channels * inner)) / inner;
        size_t b = i % inner;
        size_t xi = (nn * channels + c) * (size_t)blocks * inner + (size_t)offset * inner + b;
        if (dir == 0) y[i] = x[xi];
        else x[xi] = y[i];
    }
}
hipError_t k_channel_copy(hipStream_t s, DType dt, size_t n, int channels, int blocks, int inner, int offset, void* x,
                          void* y, int dir)
{
    if (n == 0) return hipSuccess;
    const int vec = dt == F32 ? 4 : 8;
    if (inner % vec == 0 && n % vec == 0 && ((((uintptr_t)x | (uintptr_t)y) & 15) == 0)) {
        hipLaunchKernelGGL(channel_copy_vec_kernel, grid_for(n / vec), TPB, 0, s, n / vec, channels, blocks, inner / vec, offset,
                           (uint4*)x, (uint4*)y, dir);
        return hipGetLastError();
    }
    DISPATCH_DT(dt, hipLaunchKernelGGL(channel_copy_kernel<T>, grid_for(n), TPB, 0, s, n, channels, blocks, inner, offset,
                                       (T*)x, (T*)y, dir));
    return hipGetLastError();
}

template <typename T> __global__ void embed_kernel(size_t count, const float* ids, const T* w, int N, T* top)
{
    GRID_STRIDE(i, count)
    {
        size_t nn = i / N;
        int d = (int)(i % N);
        long long idx = (long long)ids[nn];
        long long wi = idx * N + d;
        if (wi < 0) wi = -wi;
        top[i] = w[wi];
    }
}
hipError_t k_embed(hipStream_t s, DType wdt, size_t count, const float* ids, const void* w, int N, void* top)
{
    if (count == 0) return hipSuccess;
    DISPATCH_DT(wdt, hipLaunchKernelGGL(embed_kernel<T>, grid_for(count), TPB, 0, s, count, ids, (const T*)w, N, (T*)top));
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// reductions
// (DPP and row-swap permutes: the same butterfly as `v += __shfl_xor(v, o)` for o = 32 .. 1, without the LDS crossbar)
__device__ inline float wave_max(float v) { return group_max<64>(v); }
__device__ inline float wave_sum(float v) { return group_sum<64>(v); }

template <int NW> __device__ inline float block_max(float v, float* red)
{
    v = wave_max(v);
    int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < NW; i++) r = fmaxf(r, red[i]);
    return r;
}
template <int NW> __device__ inline float block_sum(float v, float* red)
{
    v = wave_sum(v);
    int w = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < NW; i++) r += red[i];
    return r;
}

// one workgroup per row (inner == 1); the row is read once into registers when it
// fits (len <= 256*8) and re-read from L2 otherwise
template <typename T> __global__ void softmax_rows_kernel(const T* x, T* y, int len, bool logsm)
{
    __shared__ float red[4];
    const T* xr = x + (size_t)blockIdx.x * len;
    T* yr = y + (size_t)blockIdx.x * len;
    constexpr int R = 8;
    float v[R];
    bool cached = len <= TPB * R;
    float mx = -INFINITY;
    if (cached) {
        for (int j = 0; j < R; j++) {
            int i = threadIdx.x + j * TPB;
            v[j] = i < len ? ld(xr, i) : -INFINITY;
            mx = fmaxf(mx, v[j]);
        }
    } else {
        for (int i = threadIdx.x; i < len; i += TPB) mx = fmaxf(mx, ld(xr, i));
    }
    mx = block_max<4>(mx, red);
    float sum = 0.f;
    if (cached) {
        for (int j = 0; j < R; j++) {
            int i = threadIdx.x + j * TPB;
            if (i < len) {
                v[j] = expf(v[j] - mx);
                sum += v[j];
            }
        }
    } else {
        for (int i = threadIdx.x; i < len; i += TPB) sum += expf(ld(xr, i) - mx);
    }
    sum = block_sum<4>(sum, red);
    if (logsm) {
        float ls = logf(sum);
        for (int i = threadIdx.x; i < len; i += TPB) st(yr, i, ld(xr, i) - mx - ls);
        return;
    }
    if (cached) {
        for (int j = 0; j < R; j++) {
            int i = threadIdx.x + j * TPB;
            if (i < len) st(yr, i, v[j] / sum);
        }
    } else {
        for (int i = threadIdx.x; i < len; i += TPB) st(yr, i, expf(ld(xr, i) - mx) / sum);
    }
}

// general (outer, len, inner): one thread per series
template <typename T> __global__ void softmax_strided_kernel(const T* x, T* y, size_t series, int len, int inner, bool logsm)
{
    GRID_STRIDE(sidx, series)
    {
        size_t o = sidx / inner, in = sidx % inner;
        size_t base = o * (size_t)len * inner + in;
        float mx = -INFINITY;
        for (int l = 0; l < len; l++) mx = fmaxf(mx, ld(x, base + (size_t)l * inner));
        float sum = 0.f;
        for (int l = 0; l < len; l++) sum += expf(ld(x, base + (size_t)l * inner) - mx);
        float ls = logf(sum);
        for (int l = 0; l < len; l++) {
            float d = ld(x, base + (size_t)l * inner) - mx;
            st(y, base + (size_t)l * inner, logsm ? d - ls : expf(d) / sum);
        }
    }
}

static bool softmax_fwd_wave_launch(hipStream_t s, DType dt, const void* x, void* y, size_t rows, int len, bool logsm);

hipError_t k_softmax(hipStream_t s, DType dt, const void* x, void* y, size_t outer, int len, int inner, bool logsm)
{
    if (outer == 0 || len <= 0 || inner <= 0) return hipSuccess;
    if (inner == 1 && softmax_fwd_wave_launch(s, dt, x, y, outer, len, logsm)) return hipGetLastError();
    if (inner == 1) {
        if (outer > 0x7fffffffu) return hipErrorInvalidValue;
        DISPATCH_DT(dt, hipLaunchKernelGGL(softmax_rows_kernel<T>, (int)outer, TPB, 0, s, (const T*)x, (T*)y, len, logsm));
    } else {
        size_t series = outer * (size_t)inner;
        DISPATCH_DT(dt, hipLaunchKernelGGL(softmax_strided_kernel<T>, grid_for(series), TPB, 0, s, (const T*)x, (T*)y, series,
                                           len, inner, logsm));
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// RoPE: pair p = (x[2p], x[2p+1]); table row = (p % (seqLen*heads*half)) / (heads*half),
// column = p % half; one fused pass replaces the reference's three kernels.  sinSign = -1 gives the gradient
// (rotation by the opposite angle, rope.cu:754-770).
template <typename T>
__global__ void rope_kernel(size_t pairs, const T* x, T* y, const float* __restrict__ fcos, const float* __restrict__ fsin,
                            int seqLen, int heads, int half, int tableOff, float sinSign)
{
    size_t full = (size_t)heads * half;
    size_t wrap = (size_t)seqLen * full;
    GRID_STRIDE(p, pairs)
    {
        size_t base = p % wrap;
        size_t t = (base / full) * half + base % half + tableOff;
        float c = fcos[t], sn = sinSign * fsin[t];
        float re = ld(x, 2 * p), im = ld(x, 2 * p + 1);
        st(y, 2 * p, re * c - im * sn);
        st(y, 2 * p + 1, re * sn + im * c);
    }
}

hipError_t k_rope(hipStream_t s, DType dt, size_t n, const void* x, void* y, const float* fcos, const float* fsin,
                  int seqLen, int heads, int hs, int tableOff, bool grad)
{
    size_t pairs = n / 2;
    if (pairs == 0) return hipSuccess;
    DISPATCH_DT(dt, hipLaunchKernelGGL(rope_kernel<T>, grid_for(pairs), TPB, 0, s, pairs, (const T*)x, (T*)y, fcos, fsin,
                                       seqLen, heads, hs / 2, tableOff, grad ? -1.0f : 1.0f));
    return hipGetLastError();
}

// y = w * (x / sqrt(mean(x^2) + eps)); one workgroup per row
template <typename T> __global__ void rmsnorm_kernel(int dim, const T* x, const T* w, T* y, float eps)
{
    __shared__ float red[4];
    const T* xr = x + (size_t)blockIdx.x * dim;
    T* yr = y + (size_t)blockIdx.x * dim;
    float ss = 0.f;
    for (int i = threadIdx.x; i < dim; i += TPB) {
        float v = ld(xr, i);
        ss += v * v;
    }
    ss = block_sum<4>(ss, red);
    float inv = 1.0f / sqrtf(ss / dim + eps);
    for (int i = threadIdx.x; i < dim; i += TPB) {
        float v = inv * ld(xr, i);
        st(yr, i, w ? ld(w, i) * v : v);
    }
}

hipError_t k_rmsnorm(hipStream_t s, DType dt, int outer, int dim, const void* x, const void* w, void* y, float eps)
{
    if (outer <= 0 || dim <= 0) return hipSuccess;
    DISPATCH_DT(dt, hipLaunchKernelGGL(rmsnorm_kernel<T>, outer, TPB, 0, s, dim, (const T*)x, (const T*)w, (T*)y, eps));
    return hipGetLastError();
}


// ---------------------------------------------------------------------------
// LayerNorm (no affine part; the reference chain of layernorm.cu:219-262 in one pass): per row of `inner` values
// y = (x - mean) / sqrt(var + eps); the row's sqrt(var + eps) is kept for the backward pass.  One workgroup per
// row; the row stays in L2 between the three sweeps, so HBM sees one read and one write.
template <typename T> __global__ void layernorm_fwd_kernel(int inner, const T* x, T* y, float* stdev, float eps)
{
    __shared__ float red[4];
    const T* xr = x + (size_t)blockIdx.x * inner;
    T* yr = y + (size_t)blockIdx.x * inner;
    float sum = 0.f;
    for (int i = threadIdx.x; i < inner; i += TPB) sum += ld(xr, i);
    const float mean = block_sum<4>(sum, red) / inner;
    float sq = 0.f;
    for (int i = threadIdx.x; i < inner; i += TPB) {
        float d = ld(xr, i) - mean;
        sq += d * d;
    }
    const float sd = sqrtf(block_sum<4>(sq, red) / inner + eps);
    if (threadIdx.x == 0) stdev[blockIdx.x] = sd;
    for (int i = threadIdx.x; i < inner; i += TPB) st(yr, i, (ld(xr, i) - mean) / sd);
}

// Rows of up to 2048 values, a multiple of 4: one wavefront per row, the row lives in registers (chunks of four values,
// lane l takes chunks l, l + 64, ...), reductions stay inside the wavefront.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    __device__ static inline void load(const float* p, float (&v)[4]) { const float4 a = *(const float4*)p; v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; }
    __device__ static inline void store(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4<bf16_t> {
    __device__ static inline void load(const bf16_t* p, float (&v)[4])
    {
        const uint2 a = *(const uint2*)p;
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
    }
    __device__ static inline void store(bf16_t* p, const float (&v)[4])
    {
        *(uint2*)p = make_uint2(pack2_bf16_hw(v[0], v[1]), pack2_bf16_hw(v[2], v[3]));
    }
};

template <typename T, int R> __global__ __launch_bounds__(256) void layernorm_fwd_wave_kernel(int rows, int inner, const T* x, T* y, float* stdev, float eps)
{
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int chunks = inner >> 2;
    const T* xr = x + (size_t)row * inner;
    T* yr = y + (size_t)row * inner;
    float v[R][4];
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + 64 * r;
        if (c < chunks) {
            Vec4<T>::load(xr + 4 * c, v[r]);
            sum += (v[r][0] + v[r][1]) + (v[r][2] + v[r][3]);
        }
    }
    const float mean = wave_sum(sum) / inner;
    float sq = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++)
        if (lane + 64 * r < chunks) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[r][j] -= mean;
                sq += v[r][j] * v[r][j];
            }
        }
    const float sd = sqrtf(wave_sum(sq) / inner + eps);
    if (lane == 0) stdev[row] = sd;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + 64 * r;
        if (c < chunks) {
#pragma unroll
            for (int j = 0; j < 4; j++) v[r][j] /= sd;
            Vec4<T>::store(yr + 4 * c, v[r]);
        }
    }
}

template <typename T, int R>
__global__ __launch_bounds__(256) void layernorm_bwd_wave_kernel(int rows, int inner, const T* y, const T* dy, T* dx, const float* stdev, float bump)
{
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int chunks = inner >> 2;
    const size_t base = (size_t)row * inner;
    float vy[R][4], vg[R][4];
    float a = 0.f, b = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + 64 * r;
        if (c < chunks) {
            Vec4<T>::load(y + base + 4 * c, vy[r]);
            Vec4<T>::load(dy + base + 4 * c, vg[r]);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                a += vy[r][j] * vg[r][j];
                b += vg[r][j];
            }
        }
    }
    const float m1 = wave_sum(a) / inner, m2 = wave_sum(b) / inner;
    const float sd = stdev[row];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + 64 * r;
        if (c < chunks) {
            float o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float div = base + 4 * c + j < (size_t)rows ? sd + bump : sd;
                o[j] = (vg[r][j] - (vy[r][j] * m1 + m2)) / div;
            }
            Vec4<T>::store(dx + base + 4 * c, o);
        }
    }
}

// register budget per lane: R chunks of four values
static inline int layernorm_wave_chunks(int inner, const void* a, const void* b, const void* c, size_t esize)
{
    if (inner % 4 != 0 || inner > 2048) return 0;
    if ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & (4 * esize - 1)) != 0) return 0;
    const int r = (inner / 4 + 63) / 64;
    return r <= 1 ? 1 : (r <= 2 ? 2 : (r <= 4 ? 4 : 8));
}

hipError_t k_layernorm_fwd(hipStream_t s, DType dt, int rows, int inner, const void* x, void* y, float* stdev, float eps)
{
    if (rows <= 0 || inner <= 0) return hipSuccess;
    const int R = layernorm_wave_chunks(inner, x, y, y, dt == F32 ? 4 : 2);
    const int g = (rows + 3) / 4;
#define LN_FWD(RR) DISPATCH_DT(dt, hipLaunchKernelGGL((layernorm_fwd_wave_kernel<T, RR>), g, 256, 0, s, rows, inner, (const T*)x, (T*)y, stdev, eps))
    if (R == 1) LN_FWD(1);
    else if (R == 2) LN_FWD(2);
    else if (R == 4) LN_FWD(4);
    else if (R == 8) LN_FWD(8);
    else DISPATCH_DT(dt, hipLaunchKernelGGL(layernorm_fwd_kernel<T>, rows, TPB, 0, s, inner, (const T*)x, (T*)y, stdev, eps));
#undef LN_FWD
    return hipGetLastError();
}

// dx = (dy - (y * mean(y*dy) + mean(dy))) / divisor (layernorm.cu:268-312).  The divisor is the row's stdev; the
// reference adds eps to the first `rows` entries of its row-expanded stdev array on every backward call, which is
// reproduced through `bump` = eps x (backward calls since the last forward), applied to flat indices < rows.
template <typename T>
__global__ void layernorm_bwd_kernel(int rows, int inner, const T* y, const T* dy, T* dx, const float* stdev, float bump)
{
    __shared__ float red[4];
    const size_t base = (size_t)blockIdx.x * inner;
    float a = 0.f, b = 0.f;
    for (int i = threadIdx.x; i < inner; i += TPB) {
        float g = ld(dy, base + i);
        a += ld(y, base + i) * g;
        b += g;
    }
    const float m1 = block_sum<4>(a, red) / inner;
    const float m2 = block_sum<4>(b, red) / inner;
    const float sd = stdev[blockIdx.x];
    for (int i = threadIdx.x; i < inner; i += TPB) {
        float w = ld(y, base + i) * m1 + m2;
        float div = base + i < (size_t)rows ? sd + bump : sd;
        st(dx, base + i, (ld(dy, base + i) - w) / div);
    }
}

hipError_t k_layernorm_bwd(hipStream_t s, DType dt, int rows, int inner, const void* y, const void* dy, void* dx,
                           const float* stdev, float bump)
{
    if (rows <= 0 || inner <= 0) return hipSuccess;
    const int R = layernorm_wave_chunks(inner, y, dy, dx, dt == F32 ? 4 : 2);
    const int g = (rows + 3) / 4;
#define LN_BWD(RR) DISPATCH_DT(dt, hipLaunchKernelGGL((layernorm_bwd_wave_kernel<T, RR>), g, 256, 0, s, rows, inner, (const T*)y, (const T*)dy, (T*)dx, stdev, bump))
    if (R == 1) LN_BWD(1);
    else if (R == 2) LN_BWD(2);
    else if (R == 4) LN_BWD(4);
    else if (R == 8) LN_BWD(8);
    else DISPATCH_DT(dt, hipLaunchKernelGGL(layernorm_bwd_kernel<T>, rows, TPB, 0, s, rows, inner, (const T*)y, (const T*)dy, (T*)dx,
                                            stdev, bump));
#undef LN_BWD
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Softmax gradient (cudnnSoftmaxBackward as called from SoftmaxLayer.cs:359-367): per series of `len` values
//   accurate / fast : dx = (dy - sum(dy * y)) * y
//   log             : dx = dy - exp(y) * sum(dy)
// inner == 1 and len % 4 == 0, len <= 2048: one wavefront per row, the row kept in registers between the two passes.
// Forward pass of the same shape class: one wavefront per row, max, exp and sum on the registers that hold the row.
// MASKED: the row is first put through a mask call that was held back for this purpose,
//   x = mask[mi] == search ? replace : xscale * x,   mi = i % md1 + (i / dd1) * md1   (i = flat index; md1 and dd1 are
// multiples of the row length, so a row maps to one run of mask values).
// causalT != 0: the mask is known to keep exactly the lower triangle of a (causalT, causalT) square and rows are causalT
// long, so it is not read, and neither are the chunks of x that lie wholly above the diagonal.
struct SoftmaxMask { const void* mask; size_t md1, dd1; float search, replace, xscale; int causalT; int* zeroFlag; int epoch; };

template <typename T, int R, bool MASKED>
__global__ __launch_bounds__(256) void softmax_fwd_wave_kernel(size_t rows, int len, const T* x, T* y, bool logsm, SoftmaxMask mk)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int chunks = len >> 2;
    const T* xr = x + row * len;
    T* yr = y + row * len;
    const T* mr = nullptr;
    int qrow = 0;
    if (MASKED) {
        if (mk.causalT) {
            qrow = (int)(row % (size_t)mk.causalT);
        } else {
            const size_t i0 = row * (size_t)len;
            mr = (const T*)mk.mask + i0 % mk.md1 + (i0 / mk.dd1) * mk.md1;
        }
    }
    float v[R][4];
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + r * 64;
        if (c < chunks) {
            if (MASKED && mk.causalT) {
                if (4 * c > qrow) {
#pragma unroll
                    for (int i = 0; i < 4; i++) v[r][i] = mk.replace;
                } else {
                    Vec4<T>::load(xr + 4 * c, v[r]);
#pragma unroll
                    for (int i = 0; i < 4; i++) v[r][i] = 4 * c + i > qrow ? mk.replace : mk.xscale * v[r][i];
                }
            } else {
                Vec4<T>::load(xr + 4 * c, v[r]);
            }
            if (MASKED && !mk.causalT) {
                float mv[4];
                Vec4<T>::load(mr + 4 * c, mv);
#pragma unroll
                for (int i = 0; i < 4; i++) v[r][i] = mv[i] == mk.search ? mk.replace : mk.xscale * v[r][i];
            }
#pragma unroll
            for (int i = 0; i < 4; i++) mx = fmaxf(mx, v[r][i]);
        }
    }
    mx = wave_max(mx);
    // a later product over this row may skip the masked entries if every one of them comes out as an exact zero
    if (MASKED && mk.causalT && mk.zeroFlag && lane == 0 && qrow + 1 < len && (logsm || expf(mk.replace - mx) != 0.f))
        *mk.zeroFlag = mk.epoch;
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (lane + r * 64 < chunks) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float d = v[r][i] - mx;
                const float e = expf(d);
                sum += e;
                v[r][i] = logsm ? d : e;
            }
        }
    }
    sum = wave_sum(sum);
    const float ls = logf(sum);
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + r * 64;
        if (c < chunks) {
            float o[4];
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = logsm ? v[r][i] - ls : v[r][i] / sum;
            Vec4<T>::store(yr + 4 * c, o);
        }
    }
}

template <bool MASKED>
static bool softmax_fwd_wave_launch_t(hipStream_t s, DType dt, const void* x, void* y, size_t rows, int len, bool logsm, SoftmaxMask mk)
{
    const int R = layernorm_wave_chunks(len, x, y, MASKED ? mk.mask : y, dt == F32 ? 4 : 2);
    if (R == 0 || (rows + 3) / 4 > 0x7fffffffu) return false;
    const int g = (int)((rows + 3) / 4);
#define SM_FWD(RR) DISPATCH_DT(dt, hipLaunchKernelGGL((softmax_fwd_wave_kernel<T, RR, MASKED>), g, 256, 0, s, rows, len, (const T*)x, (T*)y, logsm, mk))
    if (R == 1) SM_FWD(1);
    else if (R == 2) SM_FWD(2);
    else if (R == 4) SM_FWD(4);
    else SM_FWD(8);
#undef SM_FWD
    return true;
}
static bool softmax_fwd_wave_launch(hipStream_t s, DType dt, const void* x, void* y, size_t rows, int len, bool logsm)
{
    return softmax_fwd_wave_launch_t<false>(s, dt, x, y, rows, len, logsm, SoftmaxMask{});
}

// Softmax over rows of `len` of a tensor whose mask call (with its folded-in scaling) has been held back: one pass
// instead of two.  Returns hipErrorNotSupported when the shape does not fit the one-wavefront-per-row kernel or a row
// would straddle a wrap of the mask; the caller then runs the mask call first.
hipError_t k_softmax_masked(hipStream_t s, DType dt, const void* x, void* y, size_t rows, int len, bool logsm, const void* mask,
                            size_t md1, size_t dd1, float search, float replace, float xscale, bool causal, int* zeroFlag, int epoch)
{
    if (rows == 0 || len <= 0) return hipSuccess;
    if (md1 == 0 || dd1 == 0 || md1 % (size_t)len != 0 || dd1 % (size_t)len != 0) return hipErrorNotSupported;
    if (causal && (md1 != (size_t)len * len || dd1 % md1 != 0)) return hipErrorInvalidValue;
    SoftmaxMask mk{mask, md1, dd1, search, replace, xscale, causal ? len : 0, causal ? zeroFlag : nullptr, epoch};
    if (!softmax_fwd_wave_launch_t<true>(s, dt, x, y, rows, len, logsm, mk)) return hipErrorNotSupported;
    return hipGetLastError();
}

template <typename T, int R>
__global__ __launch_bounds__(256) void softmax_bwd_wave_kernel(size_t rows, int len, const T* y, const T* dy, T* dx, bool logsm)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int chunks = len >> 2;
    const T* yr = y + row * len;
    const T* gr = dy + row * len;
    T* xr = dx + row * len;
    float yv[R][4], gv[R][4];
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + r * 64;
        if (c < chunks) {
            Vec4<T>::load(yr + 4 * c, yv[r]);
            Vec4<T>::load(gr + 4 * c, gv[r]);
#pragma unroll
            for (int i = 0; i < 4; i++) sum += logsm ? gv[r][i] : gv[r][i] * yv[r][i];
        }
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int c = lane + r * 64;
        if (c < chunks) {
            float o[4];
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = logsm ? gv[r][i] - __expf(yv[r][i]) * sum : (gv[r][i] - sum) * yv[r][i];
            Vec4<T>::store(xr + 4 * c, o);
        }
    }
}

// any (outer, len, inner): one workgroup per series, two passes over global memory
template <typename T>
__global__ void softmax_bwd_kernel(int len, int inner, const T* y, const T* dy, T* dx, bool logsm)
{
    __shared__ float red[4];
    const size_t o = blockIdx.x / inner, in = blockIdx.x % inner;
    const size_t base = o * (size_t)len * inner + in;
    float sum = 0.f;
    for (int l = threadIdx.x; l < len; l += TPB) {
        const float g = ld(dy, base + (size_t)l * inner);
        sum += logsm ? g : g * ld(y, base + (size_t)l * inner);
    }
    sum = block_sum<4>(sum, red);
    for (int l = threadIdx.x; l < len; l += TPB) {
        const size_t i = base + (size_t)l * inner;
        const float g = ld(dy, i), v = ld(y, i);
        st(dx, i, logsm ? g - expf(v) * sum : (g - sum) * v);
    }
}

hipError_t k_softmax_bwd(hipStream_t s, DType dt, const void* y, const void* dy, void* dx, size_t outer, int len, int inner, bool logsm)
{
    if (outer == 0 || len <= 0 || inner <= 0) return hipSuccess;
    const int R = inner == 1 ? layernorm_wave_chunks(len, y, dy, dx, dt == F32 ? 4 : 2) : 0;
    const size_t series = outer * (size_t)inner;
    if (series > 0x7fffffffu) return hipErrorInvalidValue;
    const int g = (int)((outer + 3) / 4);
#define SM_BWD(RR) DISPATCH_DT(dt, hipLaunchKernelGGL((softmax_bwd_wave_kernel<T, RR>), g, 256, 0, s, outer, len, (const T*)y, (const T*)dy, (T*)dx, logsm))
    if (R == 1) SM_BWD(1);
    else if (R == 2) SM_BWD(2);
    else if (R == 4) SM_BWD(4);
    else if (R == 8) SM_BWD(8);
    else DISPATCH_DT(dt, hipLaunchKernelGGL(softmax_bwd_kernel<T>, (int)series, TPB, 0, s, len, inner, (const T*)y, (const T*)dy, (T*)dx, logsm));
#undef SM_BWD
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// GELU (math.cu:11348-11376) and its gradient (math.cu:11412-11448).  The reference evaluates the tanh ("bert") forward
// in double and rounds to T; here everything is single precision with tanh through one exp (difference: a few 1e-7 of |x|).
// tanh through one v_exp_f32: 1 - 2 / (e^{2u} + 1); exact limits at +-inf, absolute error about one float ulp of 1
__device__ inline float tanh_fast(float u) { return 1.0f - 2.0f * __builtin_amdgcn_rcpf(__expf(2.0f * u) + 1.0f); }

struct GeluF {
    bool bert;
    __device__ float operator()(float x, float) const
    {
        if (bert) {
            const float k = 0.7978845608028654f;   // sqrt(2 / pi)
            // 0.5 x (1 + tanh u) = x (1 - 1 / (e^{2u} + 1))
            return x * (1.0f - __builtin_amdgcn_rcpf(__expf(2.0f * k * (x + 0.044715f * (x * x * x))) + 1.0f));
        }
        return x * (0.5f * (1.0f + erff(x * 0.7071067811865475f)));
    }
};
struct GeluGradF {   // f(dy, x)
    bool bert;
    __device__ float operator()(float dy, float x) const
    {
        float grad;
        if (bert) {
            const float x3 = x * x * x;
            const float t = tanh_fast(0.797885f * (x + 0.044715f * x3));      // the reference's rounded constants
            grad = 0.5f * t + (0.0535161f * x3 + 0.398942f * x) * (1.0f - t * t) + 0.5f;   // 1 / cosh^2 = 1 - tanh^2
        } else {
            const float cdf = 0.5f * (1.0f + erff(x * 0.7071067811865475f));
            const float pdf = 0.3989422804014327f * __expf(-0.5f * (x * x));   // 1 / sqrt(2 pi)
            grad = cdf + x * pdf;
        }
        return dy * grad;
    }
};
struct SiluGradF {   // f(dy, x) = dy * s (1 + x (1 - s)) (math.cu:11740-11749)
    __device__ float operator()(float dy, float x) const
    {
        const float sg = 1.0f / (1.0f + expf(-x));
        return dy * (sg * (1.0f + x * (1.0f - sg)));
    }
};
// ReLU with negative slope (math.cu:12038-12044) and its gradient, which looks at the TOP data (math.cu:12072-12078)
struct ReluF { float slope; __device__ float operator()(float x, float) const { return x > 0.f ? x : x * slope; } };
struct ReluGradF {   // f(dy, y)
    float slope;
    __device__ float operator()(float dy, float y) const { return dy * ((y > 0.f ? 1.f : 0.f) + (y <= 0.f ? 1.f : 0.f) * slope); }
};

hipError_t k_gelu_fwd(hipStream_t s, DType dt, size_t n, const void* x, void* y, bool bert) { return launch_map(s, dt, n, x, nullptr, y, GeluF{bert}); }
hipError_t k_gelu_bwd(hipStream_t s, DType dt, size_t n, const void* dy, const void* x, void* dx, bool bert)
{
    return launch_map(s, dt, n, dy, x, dx, GeluGradF{bert});
}
hipError_t k_silu_bwd(hipStream_t s, DType dt, size_t n, const void* dy, const void* x, void* dx) { return launch_map(s, dt, n, dy, x, dx, SiluGradF{}); }
hipError_t k_relu_fwd(hipStream_t s, DType dt, size_t n, const void* x, void* y, float slope) { return launch_map(s, dt, n, x, nullptr, y, ReluF{slope}); }
hipError_t k_relu_bwd(hipStream_t s, DType dt, size_t n, const void* dy, const void* y, void* dx, float slope)
{
    return launch_map(s, dt, n, dy, y, dx, ReluGradF{slope});
}

// ---------------------------------------------------------------------------
// The elementwise / per-row primitives that the C# RMSNormLayer and LayerNormLayer chains are made of
// (RMSNormLayer.cs:156-180, LayerNormLayer.cs:223-264).
struct PowxF {   // powx_kernel (math.cu:5955-5961); the square, the only exponent those layers use, is exact
    float alpha;
    __device__ float operator()(float a, float) const { return alpha == 2.0f ? a * a : powf(a, alpha); }
};
struct SqrtF { float eps; __device__ float operator()(float x, float) const { return sqrtf(x + eps); } };   // math.cu:6211-6217
struct InvertF {   // invert_kernel and its _n / _d / _nd forms (math.cu:6018-6082): 0 stays 0; factors 0 and 1 are ignored
    float num, den;
    __device__ float operator()(float x, float) const { return x == 0.f ? 0.f : num / (x * den); }
};
struct SubF { __device__ float operator()(float a, float b) const { return a - b; } };
struct AddScalarF { float alpha; __device__ float operator()(float y, float) const { return y + alpha; } };
struct DivF { __device__ float operator()(float a, float b) const { return b == 0.f ? 0.f : a / b; } };   // math.cu:5681-5687

hipError_t k_powx(hipStream_t s, DType dt, size_t n, const void* a, float alpha, void* y) { return launch_map(s, dt, n, a, nullptr, y, PowxF{alpha}); }
hipError_t k_sqrt(hipStream_t s, DType dt, size_t n, const void* x, void* y, float eps) { return launch_map(s, dt, n, x, nullptr, y, SqrtF{eps}); }
hipError_t k_invert(hipStream_t s, DType dt, size_t n, const void* x, void* y, float num, float den)
{
    const bool un = num != 0.f && num != 1.f, ud = den != 0.f && den != 1.f;
    return launch_map(s, dt, n, x, nullptr, y, InvertF{un ? num : 1.0f, ud ? den : 1.0f});
}
hipError_t k_add_scalar(hipStream_t s, DType dt, size_t n, float alpha, void* y) { return launch_map(s, dt, n, y, nullptr, y, AddScalarF{alpha}); }
hipError_t k_div(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y) { return launch_map(s, dt, n, a, b, y, DivF{}); }

// y[i] = a[i] - b[i % nB] (sub_kernel, math.cu:5064-5090); nB == 0: plain difference
template <typename T> __global__ void sub_mod_kernel(size_t n, const T* a, const T* b, T* y, size_t nB)
{
    GRID_STRIDE(i, n) st(y, i, ld(a, i) - ld(b, i % nB));
}
hipError_t k_sub(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y, size_t nB)
{
    if (n == 0) return hipSuccess;
    if (nB == 0) return launch_map(s, dt, n, a, b, y, SubF{});
    DISPATCH_DT(dt, hipLaunchKernelGGL(sub_mod_kernel<T>, grid_for(n), TPB, 0, s, n, (const T*)a, (const T*)b, (T*)y, nB));
    return hipGetLastError();
}

// sum (scale 1) or mean (scale 1 / inner) of every row of `inner` values (channel_mean_kernel, math.cu:6817-6831;
// channel_sum_kernel_withinchannel, math.cu:6983-6997): four rows per workgroup, one wavefront each
template <typename T> __global__ __launch_bounds__(256) void channel_rowsum_kernel(size_t rows, int inner, const T* x, T* y, float scale)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * inner;
    float acc = 0.f;
    if (sizeof(T) == 4 && inner % 4 == 0 && ((uintptr_t)x & 15) == 0) {
        float a1 = 0.f;
        for (int i = lane * 4; i < inner; i += 256) {
            const float4 v = *(const float4*)((const float*)xr + i);
            acc += v.x + v.y;
            a1 += v.z + v.w;
        }
        acc += a1;
    } else {
        for (int i = lane; i < inner; i += 64) acc += ld(xr, i);
    }
    acc = wave_sum(acc);
    if (lane == 0) st(y, row, acc * scale);
}
hipError_t k_channel_rowsum(hipStream_t s, DType dt, size_t rows, int inner, const void* x, void* y, float scale)
{
    if (rows == 0 || inner <= 0) return hipSuccess;
    const size_t g = (rows + 3) / 4;
    if (g > 0x7fffffffu) return hipErrorInvalidValue;
    DISPATCH_DT(dt, hipLaunchKernelGGL(channel_rowsum_kernel<T>, (int)g, 256, 0, s, rows, inner, (const T*)x, (T*)y, scale));
    return hipGetLastError();
}
hipError_t k_channel_mean(hipStream_t s, DType dt, size_t rows, int inner, const void* x, void* y)
{
    return k_channel_rowsum(s, dt, rows, inner, x, y, inner > 0 ? 1.0f / inner : 0.f);
}

// y[n, s] = sum over c of x[n, c, s] (channel_sum_kernel_acrosschannels, math.cu:6945-6980; the reference accumulates in
// double, here four fp32 partial sums per column meet in LDS).  A workgroup owns 64 columns s of one n: lane = column,
// wavefront w takes channels w, w + 4, ..., so every load instruction reads 64 consecutive values.
template <typename T> __global__ __launch_bounds__(256) void channel_colsum_kernel(int channels, int spatial, const T* x, T* y)
{
    __shared__ float part[4][64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int sIdx = blockIdx.x * 64 + lane;
    const size_t n = blockIdx.y;
    float a0 = 0.f, a1 = 0.f;
    if (sIdx < spatial) {
        const T* xc = x + n * channels * (size_t)spatial + sIdx;
        int c = w;
        for (; c + 4 < channels; c += 8) {
            a0 += ld(xc, (size_t)c * spatial);
            a1 += ld(xc, (size_t)(c + 4) * spatial);
        }
        if (c < channels) a0 += ld(xc, (size_t)c * spatial);
    }
    part[w][lane] = a0 + a1;
    __syncthreads();
    if (w == 0 && sIdx < spatial) st(y, n * spatial + sIdx, (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]));
}
hipError_t k_channel_colsum(hipStream_t s, DType dt, size_t outer, int channels, int spatial, const void* x, void* y)
{
    if (outer == 0 || channels <= 0 || spatial <= 0) return hipSuccess;
    if (spatial == 1) return k_channel_rowsum(s, dt, outer, channels, x, y, 1.0f);
    if (outer > 65535) return hipErrorInvalidValue;
    dim3 grid((spatial + 63) / 64, (unsigned)outer);
    DISPATCH_DT(dt, hipLaunchKernelGGL(channel_colsum_kernel<T>, grid, 256, 0, s, channels, spatial, (const T*)x, (T*)y));
    return hipGetLastError();
}

// MODE 0: y[i] = x[i / spatial]                               (channel_fillfrom forward, math.cu:7465-7472)
// MODE 1: x[i] = y[i * spatial], i < rows                     (channel_fillfrom backward, math.cu:7474-7481)
// MODE 2: y[i] = x[i % period]                                (channel_copyall, math.cu:7630-7639)
// MODE 3: y[i] = x[(i / period) * channels + i % channels]    (channel_duplicate, math.cu:7667-7676)
template <typename T, int MODE> __global__ void channel_spread_kernel(size_t n, size_t spatial, size_t period, size_t channels, T* x, T* y)
{
    GRID_STRIDE(i, n)
    {
        if (MODE == 0) y[i] = x[i / spatial];
        else if (MODE == 1) x[i] = y[i * spatial];
        else if (MODE == 2) y[i] = x[i % period];
        else y[i] = x[(i / period) * channels + i % channels];
    }
}
hipError_t k_channel_spread(hipStream_t s, DType dt, int mode, size_t n, size_t spatial, size_t period, size_t channels, void* x, void* y)
{
    if (n == 0) return hipSuccess;
#define SPREAD(M) DISPATCH_DT(dt, hipLaunchKernelGGL((channel_spread_kernel<T, M>), grid_for(n), TPB, 0, s, n, spatial, period, channels, (T*)x, (T*)y))
    if (mode == 0) SPREAD(0);
    else if (mode == 1) SPREAD(1);
    else if (mode == 2) SPREAD(2);
    else SPREAD(3);
#undef SPREAD
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Primitives of the CAFFE-engine softmax chain (SoftmaxLayer.cs:230-330): exp, log, and the per-(n, s) channel
// reductions and broadcasts.  x is (num, channels, spatial); the reduced tensors are (num, spatial).
struct ExpF { float beta; __device__ float operator()(float a, float) const { return expf(beta * a); } };                    // math.cu:5859-5865
struct LogF { float beta, alpha; __device__ float operator()(float a, float) const { return logf(beta * (a + alpha)); } };   // math.cu:5923-5929
hipError_t k_exp(hipStream_t s, DType dt, size_t n, const void* a, void* y, float beta) { return launch_map(s, dt, n, a, nullptr, y, ExpF{beta}); }
hipError_t k_log(hipStream_t s, DType dt, size_t n, const void* a, void* y, float beta, float alpha) { return launch_map(s, dt, n, a, nullptr, y, LogF{beta, alpha}); }

// across channels (math.cu:6697-6713, 6733-6754): y[n, s] = max over c of x[n, c, s], or its first index; within a
// channel (math.cu:6716-6730, 6757-6778, whose loop runs over num * spatial rows of `spatial` values): y[i] = max of
// row i.  Lane = s (across) so that a wavefront reads consecutive values; starts from -FLT_MAX as the reference does.
template <typename T, bool IDX, bool ACROSS>
__global__ void channel_max_kernel(size_t rows, int channels, int spatial, const T* __restrict__ x, T* __restrict__ y)
{
    GRID_STRIDE(i, rows) {
        float val = -3.402823466e+38f;
        int idx = 0;
        if (ACROSS) {
            const size_t n = i / spatial, sp = i % spatial;
            const T* xp = x + n * channels * (size_t)spatial + sp;
            for (int c = 0; c < channels; c++) {
                const float v = ld(xp, (size_t)c * spatial);
                if (v > val) { val = v; idx = c; }
            }
        } else {
            const T* xp = x + i * spatial;
            for (int j = 0; j < spatial; j++) {
                const float v = ld(xp, j);
                if (v > val) { val = v; idx = j; }
            }
        }
        st(y, i, IDX ? (float)idx : val);
    }
}
// the same over a softmax axis that is the last one (spatial = 1, rows of `channels` consecutive values): one wavefront
// a row, four rows per workgroup; among equal maxima the first index, as the loop above finds it
template <typename T, bool IDX>
__global__ __launch_bounds__(256) void channel_rowmax_kernel(size_t rows, int channels, const T* __restrict__ x, T* __restrict__ y)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * channels;
    float val = -3.402823466e+38f;
    int idx = 0;
    if (!IDX && sizeof(T) == 4 && channels % 4 == 0 && ((uintptr_t)x & 15) == 0) {
        for (int c = lane * 4; c < channels; c += 256) {
            const float4 v = *(const float4*)((const float*)xr + c);
            // (a NaN never replaces the running maximum, as in the one-value loop)
            if (v.x > val) val = v.x;
            if (v.y > val) val = v.y;
            if (v.z > val) val = v.z;
            if (v.w > val) val = v.w;
        }
    } else {
        for (int c = lane; c < channels; c += 64) {
            const float v = ld(xr, c);
            if (v > val) { val = v; idx = c; }
        }
    }
    if (IDX) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(val, o, 64);
            const int oi = __shfl_xor(idx, o, 64);
            if (ov > val || (ov == val && oi < idx)) { val = ov; idx = oi; }
        }
    } else {
        val = wave_max(val);
    }
    if (lane == 0) st(y, row, IDX ? (float)idx : val);
}

hipError_t k_channel_max(hipStream_t s, DType dt, size_t num, int channels, int spatial, const void* x, void* y, bool idx, bool across)
{
    const size_t rows = num * spatial;
    if (rows == 0) return hipSuccess;
    if (across && spatial == 1 && channels >= 64 && (rows + 3) / 4 <= 0x7fffffffu) {
        const int g = (int)((rows + 3) / 4);
        if (idx) DISPATCH_DT(dt, hipLaunchKernelGGL((channel_rowmax_kernel<T, true>), g, 256, 0, s, rows, channels, (const T*)x, (T*)y));
        else DISPATCH_DT(dt, hipLaunchKernelGGL((channel_rowmax_kernel<T, false>), g, 256, 0, s, rows, channels, (const T*)x, (T*)y));
        return hipGetLastError();
    }
#define CMAX(I, A) DISPATCH_DT(dt, hipLaunchKernelGGL((channel_max_kernel<T, I, A>), grid_for(rows), TPB, 0, s, rows, channels, spatial, (const T*)x, (T*)y))
    if (idx) { if (across) CMAX(true, true); else CMAX(true, false); }
    else { if (across) CMAX(false, true); else CMAX(false, false); }
#undef CMAX
    return hipGetLastError();
}

// MODE 0: y[i] = a[i] - x[n, s] (channel_sub_kernel, math.cu:6908-6916); MODE 1: y[i] /= x[n, s] (channel_div_kernel,
// math.cu:7160-7168); i = (n, c, s)
template <typename T, int MODE>
__global__ void channel_bcast_kernel(size_t count, int channels, int spatial, const T* __restrict__ a, const T* __restrict__ x, T* y)
{
    GRID_STRIDE(i, count) {
        const size_t n = i / channels / spatial, sp = i % spatial;
        const float r = ld(x, n * spatial + sp);
        st(y, i, MODE == 0 ? ld(a, i) - r : ld(y, i) / r);
    }
}
// whole rows of `channels` consecutive values (spatial = 1): one wavefront a row, no division per element
template <typename T, int MODE>
__global__ __launch_bounds__(256) void channel_rowbcast_kernel(size_t rows, int channels, const T* __restrict__ a, const T* __restrict__ x, T* y)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float r = ld(x, row);
    const T* ar = MODE == 0 ? a + row * channels : nullptr;
    T* yr = y + row * channels;
    if (sizeof(T) == 4 && channels % 4 == 0 && (((uintptr_t)y | (MODE == 0 ? (uintptr_t)a : 0)) & 15) == 0) {
        for (int c = lane * 4; c < channels; c += 256) {
            float4 v = *(const float4*)(MODE == 0 ? (const float*)ar + c : (const float*)yr + c);
            if (MODE == 0) { v.x -= r; v.y -= r; v.z -= r; v.w -= r; }
            else { v.x /= r; v.y /= r; v.z /= r; v.w /= r; }
            *(float4*)((float*)yr + c) = v;
        }
        return;
    }
    for (int c = lane; c < channels; c += 64) st(yr, c, MODE == 0 ? ld(ar, c) - r : ld(yr, c) / r);
}
static inline bool channel_rows_whole(size_t count, int channels, int spatial)
{
    return spatial == 1 && channels >= 64 && count % channels == 0 && (count / channels + 3) / 4 <= 0x7fffffffu;
}
hipError_t k_channel_sub(hipStream_t s, DType dt, size_t count, int channels, int spatial, const void* a, const void* x, void* y)
{
    if (count == 0) return hipSuccess;
    if (channel_rows_whole(count, channels, spatial)) {
        const size_t rows = count / channels;
        DISPATCH_DT(dt, hipLaunchKernelGGL((channel_rowbcast_kernel<T, 0>), (int)((rows + 3) / 4), 256, 0, s, rows, channels, (const T*)a, (const T*)x, (T*)y));
        return hipGetLastError();
    }
    DISPATCH_DT(dt, hipLaunchKernelGGL((channel_bcast_kernel<T, 0>), grid_for(count), TPB, 0, s, count, channels, spatial, (const T*)a, (const T*)x, (T*)y));
    return hipGetLastError();
}
hipError_t k_channel_div(hipStream_t s, DType dt, size_t count, int channels, int spatial, const void* x, void* y)
{
    if (count == 0) return hipSuccess;
    if (channel_rows_whole(count, channels, spatial)) {
        const size_t rows = count / channels;
        DISPATCH_DT(dt, hipLaunchKernelGGL((channel_rowbcast_kernel<T, 1>), (int)((rows + 3) / 4), 256, 0, s, rows, channels, (const T*)nullptr, (const T*)x, (T*)y));
        return hipGetLastError();
    }
    DISPATCH_DT(dt, hipLaunchKernelGGL((channel_bcast_kernel<T, 1>), grid_for(count), TPB, 0, s, count, channels, spatial, (const T*)nullptr, (const T*)x, (T*)y));
    return hipGetLastError();
}

// y[n, s] = sum over c of x[n, c, s] * a[n, c, s] (channel_dot_kernel, math.cu:7335-7351, double accumulation there;
// fp32 here, channel counts of a softmax axis are short)
template <typename T>
__global__ void channel_dot_kernel(size_t rows, int channels, int spatial, const T* __restrict__ x, const T* __restrict__ a, T* __restrict__ y)
{
    GRID_STRIDE(i, rows) {
        const size_t n = i / spatial, sp = i % spatial;
        const size_t base = n * channels * (size_t)spatial + sp;
        float v0 = 0.f, v1 = 0.f;
        int c = 0;
        for (; c + 1 < channels; c += 2) {
            v0 += ld(x, base + (size_t)c * spatial) * ld(a, base + (size_t)c * spatial);
            v1 += ld(x, base + (size_t)(c + 1) * spatial) * ld(a, base + (size_t)(c + 1) * spatial);
        }
        if (c < channels) v0 += ld(x, base + (size_t)c * spatial) * ld(a, base + (size_t)c * spatial);
        st(y, i, v0 + v1);
    }
}
// rows of `channels` consecutive values (spatial = 1): one wavefront a row
template <typename T>
__global__ __launch_bounds__(256) void channel_rowdot_kernel(size_t rows, int channels, const T* __restrict__ x, const T* __restrict__ a, T* __restrict__ y)
{
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * channels;
    const T* ar = a + row * channels;
    float acc = 0.f;
    for (int c = lane; c < channels; c += 64) acc += ld(xr, c) * ld(ar, c);
    acc = wave_sum(acc);
    if (lane == 0) st(y, row, acc);
}
hipError_t k_channel_dot(hipStream_t s, DType dt, size_t num, int channels, int spatial, const void* x, const void* a, void* y)
{
    const size_t rows = num * spatial;
    if (rows == 0) return hipSuccess;
    if (spatial == 1 && channels >= 64 && (rows + 3) / 4 <= 0x7fffffffu) {
        DISPATCH_DT(dt, hipLaunchKernelGGL(channel_rowdot_kernel<T>, (int)((rows + 3) / 4), 256, 0, s, rows, channels, (const T*)x, (const T*)a, (T*)y));
        return hipGetLastError();
    }
    DISPATCH_DT(dt, hipLaunchKernelGGL(channel_dot_kernel<T>, grid_for(rows), TPB, 0, s, rows, channels, spatial, (const T*)x, (const T*)a, (T*)y));
    return hipGetLastError();
}

}  // namespace mch
