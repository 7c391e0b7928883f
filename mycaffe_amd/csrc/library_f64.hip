// The double base type of the C ABI (DLL_InvokeDouble, DLL_InvokeDoubleEx2; CudaDnnDLL.cpp:494-853): a second kernel
// table whose device memory holds doubles and whose arithmetic is double, as the reference's Kernel<double> instances
// are (dllmain.cpp:6-14; the reference test base runs every test once per base type, TestBase.cs:107-115).
//
// It covers the function ids of the attention path and of the layers around it - memory, GEMM / GEMM2 / GEMV and the
// vector updates, mask, the transposes, channel copy and the channel reductions / broadcasts, softmax, the attention
// handle, rotary embedding, layer norm handle, RMS norm, the activations, each forward and backward, embedding lookup -
// with plain kernels: one output element per thread, reductions by one workgroup per row, nothing tiled for the matrix
// cores.  This is the precision twin of the fp32 path, for hosts that instantiate their layers in
// double; the fast kernels are the fp32 / bf16 ones.  Every other id returns MCH_ERROR_NOT_IMPLEMENTED with its number
// in the message.  ALLOCMEM_HALF allocates doubles (no 16-bit storage under this base type).
#include <hip/hip_runtime.h>

#include <climits>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "runtime.h"

namespace mch {

#define HIPCHK(x) do { hipError_t _e = (x); if (_e != hipSuccess) return (long)_e; } while (0)
#define ERRCHK(x) do { long _e = (x); if (_e) return _e; } while (0)
#define GRID_STRIDE(i, n) for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < (n); i += (size_t)blockDim.x * gridDim.x)

static inline int grid_of(size_t n)
{
    const size_t g = (n + 255) / 256;
    return (int)(g < 1 ? 1 : g > 65535 ? 65535 : g);
}

// ---- kernels ----------------------------------------------------------------------------------------------------
__global__ void d_set_kernel(size_t n, double* y, double v) { GRID_STRIDE(i, n) y[i] = v; }
__global__ void d_axpy_kernel(size_t n, double a, const double* x, double* y) { GRID_STRIDE(i, n) y[i] = a * x[i] + y[i]; }
__global__ void d_scale_kernel(size_t n, double a, const double* x, double* y) { GRID_STRIDE(i, n) y[i] = a * x[i]; }
__global__ void d_add_kernel(size_t n, const double* a, const double* b, double* y, double alpha) { GRID_STRIDE(i, n) y[i] = a[i] + b[i] * alpha; }
__global__ void d_mul_kernel(size_t n, const double* a, const double* b, double* y) { GRID_STRIDE(i, n) y[i] = a[i] * b[i]; }
__global__ void d_silu_kernel(size_t n, const double* x, double* y) { GRID_STRIDE(i, n) y[i] = x[i] * (1.0 / (1.0 + exp(-x[i]))); }

__global__ void d_swiglu_kernel(size_t n, const double* a, const double* b, double* y) { GRID_STRIDE(i, n) y[i] = a[i] * (1.0 / (1.0 + exp(-a[i]))) * b[i]; }
// f(dy, x) = dy s (1 + x (1 - s)) (math.cu:11740-11749)
__global__ void d_silu_bwd_kernel(size_t n, const double* dy, const double* x, double* dx)
{
    GRID_STRIDE(i, n) { const double sg = 1.0 / (1.0 + exp(-x[i])); dx[i] = dy[i] * (sg * (1.0 + x[i] * (1.0 - sg))); }
}
// GELU (math.cu:11348-11376) and its gradient with the reference's rounded constants (math.cu:11412-11448)
__global__ void d_gelu_kernel(size_t n, const double* x, double* y, bool bert)
{
    GRID_STRIDE(i, n)
    {
        const double v = x[i];
        y[i] = bert ? 0.5 * v * (1.0 + tanh(0.7978845608028654 * (v + 0.044715 * v * v * v))) : v * (0.5 * (1.0 + erf(v * 0.7071067811865475)));
    }
}
__global__ void d_gelu_bwd_kernel(size_t n, const double* dy, const double* x, double* dx, bool bert)
{
    GRID_STRIDE(i, n)
    {
        const double v = x[i];
        double grad;
        if (bert) {
            const double x3 = v * v * v, t = tanh(0.797885 * (v + 0.044715 * x3));
            grad = 0.5 * t + (0.0535161 * x3 + 0.398942 * v) * (1.0 - t * t) + 0.5;
        } else {
            grad = 0.5 * (1.0 + erf(v * 0.7071067811865475)) + v * (0.3989422804014327 * exp(-0.5 * v * v));
        }
        dx[i] = dy[i] * grad;
    }
}
// ReLU with negative slope (math.cu:12038-12044); its gradient looks at the top data (math.cu:12072-12078)
__global__ void d_relu_kernel(size_t n, const double* x, double* y, double slope) { GRID_STRIDE(i, n) y[i] = x[i] > 0.0 ? x[i] : x[i] * slope; }
__global__ void d_relu_bwd_kernel(size_t n, const double* dy, const double* y, double* dx, double slope)
{
    GRID_STRIDE(i, n) dx[i] = dy[i] * ((y[i] > 0.0 ? 1.0 : 0.0) + (y[i] <= 0.0 ? 1.0 : 0.0) * slope);
}
// the elementwise primitives of the norm chains and of the CAFFE-engine softmax (math.cu:5064-5090, 5681-5687, 5859-5865,
// 5923-5929, 5955-5961, 6018-6082, 6211-6217)
__global__ void d_sub_kernel(size_t n, const double* a, const double* b, double* y, size_t nB) { GRID_STRIDE(i, n) y[i] = a[i] - b[nB ? i % nB : i]; }
__global__ void d_div_kernel(size_t n, const double* a, const double* b, double* y) { GRID_STRIDE(i, n) y[i] = b[i] == 0.0 ? 0.0 : a[i] / b[i]; }
__global__ void d_add_scalar_kernel(size_t n, double alpha, double* y) { GRID_STRIDE(i, n) y[i] += alpha; }
__global__ void d_powx_kernel(size_t n, const double* a, double alpha, double* y) { GRID_STRIDE(i, n) y[i] = alpha == 2.0 ? a[i] * a[i] : pow(a[i], alpha); }
__global__ void d_sqrt_kernel(size_t n, const double* x, double* y, double eps) { GRID_STRIDE(i, n) y[i] = sqrt(x[i] + eps); }
__global__ void d_invert_kernel(size_t n, const double* x, double* y, double num, double den) { GRID_STRIDE(i, n) y[i] = x[i] == 0.0 ? 0.0 : num / (x[i] * den); }
__global__ void d_exp_kernel(size_t n, const double* a, double* y, double beta) { GRID_STRIDE(i, n) y[i] = exp(beta * a[i]); }
__global__ void d_log_kernel(size_t n, const double* a, double* y, double beta, double alpha) { GRID_STRIDE(i, n) y[i] = log(beta * (a[i] + alpha)); }

// mask index = i % md1 + (i / dd1) * md1 (math.cu:2995-3002, 3046-3056; the plain mask is the case dd1 = n)
__global__ void d_mask_kernel(size_t n, size_t md1, size_t dd1, const double* x, const double* mask, double* y, double search, double replace)
{
    GRID_STRIDE(i, n) y[i] = mask[i % md1 + (i / dd1) * md1] == search ? replace : x[i];
}

// C(i,j) = alpha sum_k A(i,k) B(k,j) + beta C(i,j) for any element strides (row-major GEMM and column-major GEMM2 alike),
// batched over blockIdx.z.  16 x 16 outputs per workgroup, K in slices of 16 through LDS.
__global__ __launch_bounds__(256) void d_gemm_kernel(int m, int n, int k, double alpha, const double* A, long long ars, long long acs,
                                                     const double* B, long long brs, long long bcs, double beta, double* C,
                                                     long long crs, long long ccs, long long sA, long long sB, long long sC)
{
    __shared__ double as[16][17], bs[16][17];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int i = blockIdx.y * 16 + ty, j = blockIdx.x * 16 + tx;
    A += (size_t)blockIdx.z * sA;
    B += (size_t)blockIdx.z * sB;
    C += (size_t)blockIdx.z * sC;
    double acc = 0.0;
    for (int k0 = 0; k0 < k; k0 += 16) {
        as[ty][tx] = (i < m && k0 + tx < k) ? A[(long long)i * ars + (long long)(k0 + tx) * acs] : 0.0;
        bs[ty][tx] = (k0 + ty < k && j < n) ? B[(long long)(k0 + ty) * brs + (long long)j * bcs] : 0.0;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; kk++) acc += as[ty][kk] * bs[kk][tx];
        __syncthreads();
    }
    if (i < m && j < n) {
        double* c = C + (long long)i * crs + (long long)j * ccs;
        *c = beta == 0.0 ? alpha * acc : alpha * acc + beta * *c;
    }
}

struct PermuteD { int axes; long long xs[8], ys[8]; int map[8]; };
__global__ void d_permute_kernel(size_t n, const double* x, double* y, PermuteD a)
{
    GRID_STRIDE(i, n)
    {
        long long from[8];
        size_t rem = i;
        for (int d = 0; d < a.axes; d++) {
            from[d] = (long long)(rem / (size_t)a.xs[d]);
            rem = rem % (size_t)a.xs[d];
        }
        size_t to = 0;
        for (int d = 0; d < a.axes; d++) to += (size_t)from[a.map[d]] * (size_t)a.ys[d];
        y[to] = x[i];
    }
}
// (nc, h, w) -> (nc, w, h)
__global__ void d_transpose_hw_kernel(size_t n, int h, int w, const double* x, double* y)
{
    GRID_STRIDE(o, n)
    {
        const size_t hw = (size_t)h * w, c = o / hw, r = o % hw;
        const size_t ww = r / h, hh = r % h;
        y[o] = x[c * hw + hh * w + ww];
    }
}
__global__ void d_channel_copy_kernel(size_t n, int channels, int blocks, int inner, int offset, double* x, double* y, int dir)
{
    GRID_STRIDE(i, n)
    {
        const size_t nn = i / ((size_t)channels * inner), c = (i % ((size_t)channels * inner)) / inner, b = i % inner;
        const size_t xi = (nn * channels + c) * (size_t)blocks * inner + (size_t)offset * inner + b;
        if (dir == 0) y[i] = x[xi];
        else x[xi] = y[i];
    }
}
__global__ void d_embed_kernel(size_t count, const double* ids, const double* w, int N, double* top)
{
    GRID_STRIDE(i, count)
    {
        long long wi = (long long)ids[i / N] * N + (long long)(i % N);
        if (wi < 0) wi = -wi;
        top[i] = w[wi];
    }
}
// pairs (2p, 2p+1) rotated by the angle of table entry ((p % wrap) / full) * half + p % half + off (rope.cu:725-825)
__global__ void d_rope_kernel(size_t pairs, const double* x, double* y, const double* fcos, const double* fsin, size_t full,
                              size_t wrap, int half, int off, double sinSign)
{
    GRID_STRIDE(p, pairs)
    {
        const size_t base = p % wrap, t = (base / full) * half + base % half + off;
        const double c = fcos[t], sn = sinSign * fsin[t], re = x[2 * p], im = x[2 * p + 1];
        y[2 * p] = re * c - im * sn;
        y[2 * p + 1] = re * sn + im * c;
    }
}

// MODE 0: y[i] = x[i / spatial]; 1: x[i] = y[i * spatial]; 2: y[i] = x[i % period]; 3: y[i] = x[(i / period) * channels + i % channels]
// (channel_fillfrom forward / backward, channel_copyall, channel_duplicate: math.cu:7465-7481, 7630-7639, 7667-7676)
__global__ void d_spread_kernel(int mode, size_t n, size_t spatial, size_t period, size_t channels, double* x, double* y)
{
    GRID_STRIDE(i, n)
    {
        if (mode == 0) y[i] = x[i / spatial];
        else if (mode == 1) x[i] = y[i * spatial];
        else if (mode == 2) y[i] = x[i % period];
        else y[i] = x[(i / period) * channels + i % channels];
    }
}
// y[row] = scale * sum of the row's `inner` values, one thread per row (channel_mean, channel_sum within a channel)
__global__ void d_rowsum_kernel(size_t rows, int inner, const double* x, double* y, double scale)
{
    GRID_STRIDE(r, rows)
    {
        double acc = 0.0;
        for (int i = 0; i < inner; i++) acc += x[r * inner + i];
        y[r] = acc * scale;
    }
}
// y[n, s] = sum over c of x[n, c, s] (math.cu:6945-6980), or of x a (channel_dot, math.cu:7335-7351)
__global__ void d_colsum_kernel(size_t rows, int channels, int spatial, const double* x, const double* a, double* y)
{
    GRID_STRIDE(i, rows)
    {
        const size_t n = i / spatial, sp = i % spatial, base = n * channels * (size_t)spatial + sp;
        double acc = 0.0;
        for (int c = 0; c < channels; c++) acc += a ? x[base + (size_t)c * spatial] * a[base + (size_t)c * spatial] : x[base + (size_t)c * spatial];
        y[i] = acc;
    }
}
// channel_max across channels or within one, value or first index (math.cu:6697-6810); starts from -DBL_MAX
__global__ void d_channel_max_kernel(size_t rows, int channels, int spatial, const double* x, double* y, bool idx, bool across)
{
    GRID_STRIDE(i, rows)
    {
        double val = -1.7976931348623157e308;
        int at = 0;
        if (across) {
            const size_t n = i / spatial, sp = i % spatial;
            for (int c = 0; c < channels; c++) {
                const double v = x[n * channels * (size_t)spatial + (size_t)c * spatial + sp];
                if (v > val) { val = v; at = c; }
            }
        } else {
            for (int j = 0; j < spatial; j++) {
                const double v = x[i * spatial + j];
                if (v > val) { val = v; at = j; }
            }
        }
        y[i] = idx ? (double)at : val;
    }
}
// sub: y[i] = a[i] - x[n, s]; div: y[i] /= x[n, s]; i = (n, c, s) (math.cu:6908-6916, 7160-7168)
__global__ void d_channel_bcast_kernel(size_t count, int channels, int spatial, const double* a, const double* x, double* y, bool sub)
{
    GRID_STRIDE(i, count)
    {
        const double r = x[(i / channels / spatial) * spatial + i % spatial];
        y[i] = sub ? a[i] - r : y[i] / r;
    }
}

__device__ inline double d_block_reduce(double v, double* red, bool isMax)
{
    for (int o = 32; o > 0; o >>= 1) {
        const double u = __shfl_xor(v, o, 64);
        v = isMax ? fmax(v, u) : v + u;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    double r = red[0];
    for (int w = 1; w < 4; w++) r = isMax ? fmax(r, red[w]) : r + red[w];
    return r;
}
// softmax over `len` values `inner` apart, one workgroup per (outer, inner) pair; logsm: x - max - log(sum)
__global__ __launch_bounds__(256) void d_softmax_kernel(const double* x, double* y, int len, int inner, bool logsm)
{
    __shared__ double red[4];
    const size_t o = blockIdx.x / inner, in = blockIdx.x % inner, base = o * (size_t)len * inner + in;
    double mx = -INFINITY;
    for (int i = threadIdx.x; i < len; i += 256) mx = fmax(mx, x[base + (size_t)i * inner]);
    mx = d_block_reduce(mx, red, true);
    double sum = 0.0;
    for (int i = threadIdx.x; i < len; i += 256) sum += exp(x[base + (size_t)i * inner] - mx);
    sum = d_block_reduce(sum, red, false);
    for (int i = threadIdx.x; i < len; i += 256) {
        const double v = x[base + (size_t)i * inner] - mx;
        y[base + (size_t)i * inner] = logsm ? v - log(sum) : exp(v) / sum;
    }
}

// dx = (dy - sum) y, sum = sum_l dy y over the series (log form: dx = dy - exp(y) sum dy); one workgroup per series
__global__ __launch_bounds__(256) void d_softmax_bwd_kernel(const double* y, const double* dy, double* dx, int len, int inner, bool logsm)
{
    __shared__ double red[4];
    const size_t o = blockIdx.x / inner, in = blockIdx.x % inner, base = o * (size_t)len * inner + in;
    double sum = 0.0;
    for (int l = threadIdx.x; l < len; l += 256) {
        const size_t i = base + (size_t)l * inner;
        sum += logsm ? dy[i] : dy[i] * y[i];
    }
    sum = d_block_reduce(sum, red, false);
    for (int l = threadIdx.x; l < len; l += 256) {
        const size_t i = base + (size_t)l * inner;
        dx[i] = logsm ? dy[i] - exp(y[i]) * sum : (dy[i] - sum) * y[i];
    }
}
// y = (x - mean) / sqrt(var + eps) per row, the row's sqrt(var + eps) kept (layernorm.cu:219-262)
__global__ __launch_bounds__(256) void d_layernorm_fwd_kernel(int inner, const double* x, double* y, double* stdev, double eps)
{
    __shared__ double red[4];
    const double* xr = x + (size_t)blockIdx.x * inner;
    double* yr = y + (size_t)blockIdx.x * inner;
    double sum = 0.0;
    for (int i = threadIdx.x; i < inner; i += 256) sum += xr[i];
    const double mean = d_block_reduce(sum, red, false) / inner;
    double sq = 0.0;
    for (int i = threadIdx.x; i < inner; i += 256) sq += (xr[i] - mean) * (xr[i] - mean);
    const double sd = sqrt(d_block_reduce(sq, red, false) / inner + eps);
    if (threadIdx.x == 0) stdev[blockIdx.x] = sd;
    for (int i = threadIdx.x; i < inner; i += 256) yr[i] = (xr[i] - mean) / sd;
}
// dx = (dy - (y mean(y dy) + mean(dy))) / divisor (layernorm.cu:268-312); the reference adds eps to the first `rows`
// entries of its row-expanded stdev array on every backward call: `bump` = eps x (backward calls since the forward)
__global__ __launch_bounds__(256) void d_layernorm_bwd_kernel(int rows, int inner, const double* y, const double* dy, double* dx,
                                                              const double* stdev, double bump)
{
    __shared__ double red[4];
    const size_t base = (size_t)blockIdx.x * inner;
    double a = 0.0, b = 0.0;
    for (int i = threadIdx.x; i < inner; i += 256) { a += y[base + i] * dy[base + i]; b += dy[base + i]; }
    const double m1 = d_block_reduce(a, red, false) / inner;
    const double m2 = d_block_reduce(b, red, false) / inner;
    const double sd = stdev[blockIdx.x];
    for (int i = threadIdx.x; i < inner; i += 256) {
        const double div = base + i < (size_t)rows ? sd + bump : sd;
        dx[base + i] = (dy[base + i] - (y[base + i] * m1 + m2)) / div;
    }
}
// y = w (x / sqrt(mean(x^2) + eps)), one workgroup per row
__global__ __launch_bounds__(256) void d_rmsnorm_kernel(int dim, const double* x, const double* w, double* y, double eps)
{
    __shared__ double red[4];
    const double* xr = x + (size_t)blockIdx.x * dim;
    double* yr = y + (size_t)blockIdx.x * dim;
    double ss = 0.0;
    for (int i = threadIdx.x; i < dim; i += 256) ss += xr[i] * xr[i];
    const double inv = 1.0 / sqrt(d_block_reduce(ss, red, false) / dim + eps);
    for (int i = threadIdx.x; i < dim; i += 256) yr[i] = w ? w[i] * (inv * xr[i]) : inv * xr[i];
}
// dS = P (dP - sum_k P dP) per row, in place in dp (the softmax gradient of attn.cu:608-661)
__global__ __launch_bounds__(256) void d_attn_ds_kernel(const double* p, double* dp, int Tk)
{
    __shared__ double red[4];
    const size_t base = (size_t)blockIdx.x * Tk;
    double sum = 0.0;
    for (int j = threadIdx.x; j < Tk; j += 256) sum += p[base + j] * dp[base + j];
    sum = d_block_reduce(sum, red, false);
    for (int j = threadIdx.x; j < Tk; j += 256) dp[base + j] = p[base + j] * (dp[base + j] - sum);
}

// Attention forward as the reference's chain computes it (attn.cu:518-602): scores = scale q . k, masked ones -1e29,
// softmax over the keys, y = p V.  One workgroup per (sequence, head, query row); the row of probabilities stays in LDS.
// kind 0: no mask, 1: mask (Tq,Tk), 2: mask (B,Tk), 3: mask (B,Tq,Tk); merged: y written (B,Tq,H,hs)
// probs != nullptr: the row's probabilities are written there as well (B, H, Tq, Tk) and y may be null (the backward pass)
__global__ __launch_bounds__(256) void d_attn_row_kernel(const double* q, const double* k, const double* v, double* y, int H, int Tq,
                                                         int Tk, int hs, double scale, const double* mask, int kind, bool merged,
                                                         double* probs)
{
    extern __shared__ double d_smem[];
    double* p = d_smem;        // Tk
    double* qs = p + Tk;       // hs
    __shared__ double red[4];
    const size_t row = blockIdx.x;
    const int t = (int)(row % Tq);
    const size_t bh = row / Tq;
    const int h = (int)(bh % H);
    const size_t b = bh / H;
    const double* qr = q + row * hs;
    const double* kb = k + bh * Tk * hs;
    const double* vb = v + bh * Tk * hs;
    for (int d = threadIdx.x; d < hs; d += 256) qs[d] = qr[d];
    __syncthreads();
    double mx = -INFINITY;
    for (int j = threadIdx.x; j < Tk; j += 256) {
        double s = 0.0;
        for (int d = 0; d < hs; d++) s += qs[d] * kb[(size_t)j * hs + d];
        s *= scale;
        bool masked = false;
        if (kind == 1) masked = mask[(size_t)t * Tk + j] == 0.0;
        else if (kind == 2) masked = mask[b * Tk + j] == 0.0;
        else if (kind == 3) masked = mask[(b * Tq + t) * Tk + j] == 0.0;
        if (masked) s = -1e29;
        p[j] = s;
        mx = fmax(mx, s);
    }
    mx = d_block_reduce(mx, red, true);
    double sum = 0.0;
    for (int j = threadIdx.x; j < Tk; j += 256) {
        const double e = exp(p[j] - mx);
        p[j] = e;
        sum += e;
    }
    sum = d_block_reduce(sum, red, false);
    if (probs)
        for (int j = threadIdx.x; j < Tk; j += 256) probs[row * Tk + j] = p[j] / sum;
    if (!y) return;
    double* yr = merged ? y + ((b * Tq + t) * H + h) * (size_t)hs : y + row * hs;
    for (int d = threadIdx.x; d < hs; d += 256) {
        double acc = 0.0;
        for (int j = 0; j < Tk; j++) acc += p[j] * vb[(size_t)j * hs + d];
        yr[d] = acc / sum;
    }
}

// One query row per (sequence, head) against that head's rows of a key / value cache with any strides (id 2001; the loop
// it replaces: MultiheadAttentionLayer.cs:713-730).  The row of probabilities stays in LDS.
__global__ __launch_bounds__(256) void d_attn_decode_kernel(const double* q, const double* kc, const double* vc, double* y, int H,
                                                            int kvMul, int hs, int len, long long sB, long long sH, long long sT,
                                                            double scale)
{
    extern __shared__ double d_smem[];
    double* p = d_smem;        // len
    double* qs = p + len;      // hs
    __shared__ double red[4];
    const size_t bh = blockIdx.x;
    const int h = (int)(bh % H);
    const size_t b = bh / H;
    const double* kb = kc + b * sB + (size_t)(h / kvMul) * sH;
    const double* vb = vc + b * sB + (size_t)(h / kvMul) * sH;
    for (int d = threadIdx.x; d < hs; d += 256) qs[d] = q[bh * hs + d];
    __syncthreads();
    double mx = -INFINITY;
    for (int j = threadIdx.x; j < len; j += 256) {
        double sc = 0.0;
        for (int d = 0; d < hs; d++) sc += qs[d] * kb[(size_t)j * sT + d];
        sc *= scale;
        p[j] = sc;
        mx = fmax(mx, sc);
    }
    mx = d_block_reduce(mx, red, true);
    double sum = 0.0;
    for (int j = threadIdx.x; j < len; j += 256) {
        const double e = exp(p[j] - mx);
        p[j] = e;
        sum += e;
    }
    sum = d_block_reduce(sum, red, false);
    for (int d = threadIdx.x; d < hs; d += 256) {
        double acc = 0.0;
        for (int j = 0; j < len; j++) acc += p[j] * vb[(size_t)j * sT + d];
        y[bh * hs + d] = acc / sum;
    }
}

// The step before it when a rope handle and the new key / value come with the call: q and the new key rotated in place
// at position `pos` (adjacent pairs), the new key and value stored into the caches at that position.
__global__ void d_rope_append_kernel(double* q, double* knew, const double* vnew, double* kc, double* vc, int B, int H, int kvH, int hs,
                                     int pos, long long sB, long long sH, long long sT, const double* fcos, const double* fsin)
{
    const int half = hs / 2;
    const size_t nq = (size_t)B * H * half, nk = (size_t)B * kvH * half, nv = (size_t)B * kvH * hs;
    GRID_STRIDE(i, nq + nk + nv)
    {
        if (i < nq + nk) {
            const bool isq = i < nq;
            const size_t pr = isq ? i : i - nq;
            const int j = (int)(pr % half);
            const double c = fcos ? fcos[(size_t)pos * half + j] : 1.0, sn = fsin ? fsin[(size_t)pos * half + j] : 0.0;
            double* x = isq ? q : knew;
            const double re = x[2 * pr], im = x[2 * pr + 1];
            const double r0 = re * c - im * sn, r1 = re * sn + im * c;
            x[2 * pr] = r0;
            x[2 * pr + 1] = r1;
            if (!isq) {
                const size_t bh = pr / half;
                const size_t dst = (bh / kvH) * sB + (bh % kvH) * sH + (size_t)pos * sT + 2 * j;
                kc[dst] = r0;
                kc[dst + 1] = r1;
            }
        } else {
            const size_t pv = i - nq - nk;
            const size_t bh = pv / hs;
            vc[(bh / kvH) * sB + (bh % kvH) * sH + (size_t)pos * sT + pv % hs] = vnew[pv];
        }
    }
}

// Epilogue of the fused QKV projection (id 2004): the plain product `tmp` (B*T, 3C) gets its bias and goes, head by head,
// to q, k, v as (B,H,T,hs); q and k are rotated on the way when the tables are given (position = row % seq).
__global__ void d_qkv_split_kernel(size_t pairs, const double* tmp, const double* bias, double* q, double* k, double* v, int T, int H,
                                   int hs, const double* fcos, const double* fsin, int seq)
{
    const int C = H * hs;
    GRID_STRIDE(pi, pairs)
    {
        const size_t i = 2 * pi;
        const size_t r = i / (3 * C);
        const int c = (int)(i - r * 3 * C);
        double o0 = tmp[i], o1 = tmp[i + 1];
        if (bias) { o0 += bias[c]; o1 += bias[c + 1]; }
        const int which = c / C, w = c - which * C, h = w / hs, d = w - h * hs;
        if (fcos && which < 2) {
            const size_t ti = (size_t)(r % seq) * (hs >> 1) + (d >> 1);
            const double cs = fcos[ti], sn = fsin[ti], re = o0, im = o1;
            o0 = re * cs - im * sn;
            o1 = re * sn + im * cs;
        }
        double* dst = (which == 0 ? q : which == 1 ? k : v) + (((r / T) * H + h) * T + r % T) * hs + d;
        dst[0] = o0;
        dst[1] = o1;
    }
}
__global__ void d_add_bias_rows_kernel(size_t n, int N, const double* bias, double* y) { GRID_STRIDE(i, n) y[i] += bias[i % N]; }

// ---- the kernel object --------------------------------------------------------------------------------------------
struct MemD { double* ptr = nullptr; size_t count = 0; bool used = false; long base = 0; };   // base != 0: a view into that handle's allocation
struct AttnD { bool set = false; int batch = 0, block = 0, heads = 0, hs = 0; double scale = 1.0;
               int lastTq = 0, lastTk = 0; long long lastBatchMask = 0; long lastMask = 0; };   // of the last forward call
struct LayerNormD { bool set = false; int count = 0, outer = 0, channels = 0, inner = 0, backwards = 0; double eps = 1e-10; double* stdev = nullptr;
                    ~LayerNormD() { if (stdev) (void)hipFree(stdev); } };
struct RopeD { bool set = false; int seq = 0, heads = 0, hs = 0; double* dcos = nullptr; double* dsin = nullptr;
               ~RopeD() { if (dcos) (void)hipFree(dcos); if (dsin) (void)hipFree(dsin); } };

class KernelD {
public:
    ~KernelD()
    {
        if (m_stream) (void)hipStreamSynchronize(m_stream);
        m_rope.clear();
        m_layernorm.clear();
        if (m_ws) (void)hipFree(m_ws);
        for (MemD& m : m_mem)
            if (m.used && m.ptr && !m.base) (void)hipFree(m.ptr);
        for (double* p : m_host) (void)hipHostFree(p);
        if (m_stream) (void)hipStreamDestroy(m_stream);
    }
    long initialize(const double* pf, long n)
    {
        // SetDevice: f{deviceId, flags[, seed]} (device.cu:772-795)
        if (n < 2 || n > 3) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (!pf) return MCH_ERROR_PARAM_NULL;
        int count = 0;
        HIPCHK(hipGetDeviceCount(&count));
        const int dev = (int)pf[0];
        if (dev < 0 || dev >= count) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        m_device = dev;
        HIPCHK(hipSetDevice(dev));
        if (!m_stream) HIPCHK(hipStreamCreateWithFlags(&m_stream, hipStreamNonBlocking));
        return 0;
    }
    long free_host(double* p)
    {
        for (size_t i = 0; i < m_host.size(); i++)
            if (m_host[i] == p) {
                m_host.erase(m_host.begin() + i);
                HIPCHK(hipHostFree(p));
                return 0;
            }
        return MCH_ERROR_MEMORY_NOT_FOUND;
    }
    long get_pointer(long h, void** pp)
    {
        MemD* it;
        ERRCHK(mem(h, &it));
        *pp = it->ptr;
        return 0;
    }
    long run(long fn, const double* pf, long lf, const MCH_LONGLONG* pl, long ll, double** ppOut, MCH_LONG* plOut);
    std::string last_detail;

private:
    long mem(long h, MemD** it)
    {
        if (h <= 0 || (size_t)h >= m_mem.size() || !m_mem[h].used) return MCH_ERROR_MEMORY_NOT_FOUND;
        *it = &m_mem[h];
        return 0;
    }
    long alloc(size_t count, long* h)
    {
        double* p = nullptr;
        HIPCHK(hipMalloc((void**)&p, (count ? count : 1) * sizeof(double)));
        hipError_t e = hipMemsetAsync(p, 0, (count ? count : 1) * sizeof(double), m_stream);
        if (e != hipSuccess) { (void)hipFree(p); return (long)e; }
        const size_t slot = new_slot();
        m_mem[slot] = MemD();
        m_mem[slot].ptr = p; m_mem[slot].count = count; m_mem[slot].used = true;
        *h = (long)slot;
        return 0;
    }
    size_t new_slot()
    {
        for (size_t i = 1; i < m_mem.size(); i++)
            if (!m_mem[i].used) return i;
        m_mem.emplace_back();
        return m_mem.size() - 1;
    }
    // an allocation takes its views with it (device.h:1000-1020: a memory pointer aliases the handle it was made from)
    long release(long h)
    {
        MemD* it;
        ERRCHK(mem(h, &it));
        if (!it->base) {
            HIPCHK(hipStreamSynchronize(m_stream));
            for (MemD& m : m_mem)
                if (m.used && m.base == h) m = MemD();
            HIPCHK(hipFree(it->ptr));
        }
        *it = MemD();
        return 0;
    }
    int m_device = 0;
    hipStream_t m_stream = nullptr;
    std::vector<MemD> m_mem{1};
    std::vector<double*> m_host;
    HandleTable<CudnnState> m_cudnn;
    HandleTable<TensorDesc> m_tdesc;
    HandleTable<AttnD> m_attn;
    HandleTable<RopeD> m_rope;
    HandleTable<LayerNormD> m_layernorm;
    double* m_ws = nullptr; size_t m_wsCount = 0;   // scratch of the attention backward call
    long workspace(size_t count, double** p)
    {
        if (count > m_wsCount) {
            if (m_ws) { HIPCHK(hipStreamSynchronize(m_stream)); HIPCHK(hipFree(m_ws)); m_ws = nullptr; m_wsCount = 0; }
            HIPCHK(hipMalloc((void**)&m_ws, count * sizeof(double)));
            m_wsCount = count;
        }
        *p = m_ws;
        return 0;
    }
    long attn_mask_kind(AttnD* st, MemD* M, long long batchMask, int T, int Tk, int* kind)
    {
        *kind = 0;
        if (!M) return 0;
        const long long need = batchMask == 2 ? (long long)st->batch * T * Tk : batchMask == 1 ? (long long)st->batch * Tk : (long long)T * Tk;
        if ((long long)M->count < need) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
        *kind = batchMask == 2 ? 3 : batchMask == 1 ? 2 : 1;
        return 0;
    }
};

static inline long verify_d(long n, const void* p, long lo, long hi)
{
    if (n < lo || n > hi) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    if (lo == 0 && hi == 0) return 0;
    if (!p) return MCH_ERROR_PARAM_NULL;
    return 0;
}
static inline long set_out_d(double v, double** ppOut, MCH_LONG* plOut)
{
    if (!plOut || !ppOut || !*ppOut) return MCH_ERROR_PARAM_NULL;
    if (*plOut < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    *plOut = 1;
    (*ppOut)[0] = v;
    return 0;
}

#define NEED_L(lo, hi) ERRCHK(verify_d(ll, pl, lo, hi))
#define NEED_F(lo, hi) ERRCHK(verify_d(lf, pf, lo, hi))
#define RANGE(item, off, n) do { if ((long long)(off) < 0 || (long long)(n) < 0 || (size_t)(off) + (size_t)(n) > (item)->count) { \
        last_detail = "range exceeds the allocation behind the memory handle"; return MCH_ERROR_MEMORY_RANGE_EXCEEDED; } } while (0)
#define LAUNCHED() HIPCHK(hipGetLastError())

long KernelD::run(long fn, const double* pf, long lf, const MCH_LONGLONG* pl, long ll, double** ppOut, MCH_LONG* plOut)
{
    last_detail.clear();
    hipStream_t s = m_stream;
    if (!s) return MCH_ERROR_DEVICE_NOT_INITIALIZED;
    HIPCHK(hipSetDevice(m_device));
    switch (fn) {
    case MCH_FN_SETDEVICE:
        return initialize(pf, lf);
    case MCH_FN_GETDEVICE:
        return set_out_d((double)m_device, ppOut, plOut);
    case MCH_FN_SYNCHRONIZEDEVICE:
        HIPCHK(hipStreamSynchronize(s));
        return 0;

    // ---- memory (device.cu:854-1091) ----------------------------------------------------------------------------
    case MCH_FN_ALLOCMEM:
    case MCH_FN_ALLOCMEM_HALF: {
        // l{count[,stream]}; optional f{count,[stream,] data...}
        NEED_L(1, 2);
        if (pl[0] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const size_t count = (size_t)pl[0];
        const double* src = nullptr;
        if (lf > 1) {
            if (!pf) return MCH_ERROR_PARAM_NULL;
            if ((size_t)lf == count + 1) src = pf + 1;
            else if ((size_t)lf == count + 2) src = pf + 2;
            else return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        long h = 0;
        ERRCHK(alloc(count, &h));
        if (src && count) {
            hipError_t e = hipMemcpyAsync(m_mem[h].ptr, src, count * 8, hipMemcpyHostToDevice, s);
            if (e == hipSuccess) e = hipStreamSynchronize(s);
            if (e != hipSuccess) { (void)hipFree(m_mem[h].ptr); m_mem[h] = MemD(); return (long)e; }
        }
        return set_out_d((double)h, ppOut, plOut);
    }
    case MCH_FN_FREEMEM:
    case MCH_FN_FREE_MEMORYPOINTER:
        NEED_L(1, 1);
        return release((long)pl[0]);
    case MCH_FN_CREATE_MEMORYPOINTER: {
        // l{hData, offset, count} (device.h:1000-1020)
        NEED_L(3, 3);
        if (pl[1] < 0 || pl[2] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD* b;
        ERRCHK(mem((long)pl[0], &b));
        RANGE(b, pl[1], pl[2]);
        double* ptr = b->ptr + pl[1];
        const long root = b->base ? b->base : (long)pl[0];
        const size_t slot = new_slot();   // b may dangle from here on
        m_mem[slot] = MemD();
        m_mem[slot].ptr = ptr; m_mem[slot].count = (size_t)pl[2]; m_mem[slot].used = true; m_mem[slot].base = root;
        return set_out_d((double)slot, ppOut, plOut);
    }
    case MCH_FN_GETMEM: {
        // l{h, count(-1 = all)}
        NEED_L(1, 2);
        if (!plOut || !ppOut) return MCH_ERROR_PARAM_NULL;
        MemD* it;
        ERRCHK(mem((long)pl[0], &it));
        long long count = ll > 1 ? pl[1] : 0;
        if (count < 0) count = (long long)it->count;
        else if ((size_t)count > it->count) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (count > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        double* dst = *ppOut;
        if (!(count <= *plOut && dst)) {
            HIPCHK(hipHostMalloc((void**)&dst, (size_t)(count > 0 ? count : 1) * 8, hipHostMallocDefault));
            m_host.push_back(dst);
            *ppOut = dst;   // handed back with DLL_FREEMEM
        }
        if (count) HIPCHK(hipMemcpyAsync(dst, it->ptr, (size_t)count * 8, hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        *plOut = (MCH_LONG)count;
        return 0;
    }
    case MCH_FN_SETMEM: {
        // f{h, count, [stream,] data...}, l{h, count}
        NEED_F(2, INT_MAX);
        NEED_L(2, 2);
        if (pl[1] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const size_t count = (size_t)pl[1];
        const double* data;
        if (count == (size_t)lf - 2) data = pf + 2;
        else if (count == (size_t)lf - 3) data = pf + 3;
        else return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD* it;
        ERRCHK(mem((long)pl[0], &it));
        RANGE(it, 0, count);
        if (count) HIPCHK(hipMemcpyAsync(it->ptr, data, count * 8, hipMemcpyHostToDevice, s));
        HIPCHK(hipStreamSynchronize(s));
        return 0;
    }
    case MCH_FN_SET: {
        // f{val}, l{n, h, 0, idx, xOff} (device.h:6038-6061)
        NEED_F(1, 1);
        NEED_L(3, 5);
        const long long n = pl[0], idx = ll > 3 ? pl[3] : -1;
        long long off = ll > 4 ? pl[4] : 0;
        MemD* it;
        ERRCHK(mem((long)pl[1], &it));
        if (off < 0) off = 0;
        if (idx >= 0) {
            RANGE(it, off + idx, 1);
            hipLaunchKernelGGL(d_set_kernel, 1, 256, 0, s, (size_t)1, it->ptr + off + idx, pf[0]);
        } else {
            RANGE(it, off, n);
            if (n) hipLaunchKernelGGL(d_set_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, it->ptr + off, pf[0]);
        }
        LAUNCHED();
        return 0;
    }
    case MCH_FN_COPY: {
        // l{n, hSrc, hDst, srcOff, dstOff, ...} (device.h:6063-6095)
        NEED_L(3, 8);
        const long long n = pl[0];
        long long so = ll > 3 ? pl[3] : 0, dofs = ll > 4 ? pl[4] : 0;
        MemD *src, *dst;
        ERRCHK(mem((long)pl[1], &src));
        ERRCHK(mem((long)pl[2], &dst));
        if (so < 0) so = 0;
        if (dofs < 0) dofs = 0;
        RANGE(src, so, n);
        RANGE(dst, dofs, n);
        if (n) HIPCHK(hipMemcpyAsync(dst->ptr + dofs, src->ptr + so, (size_t)n * 8, hipMemcpyDeviceToDevice, s));
        return 0;
    }

    // ---- BLAS-like (device.cu:1636-2051) ----------------------------------------------------------------------------
    case MCH_FN_GEMM: {
        // f{alpha,beta}, l{tA,tB,m,n,k,0,hA,hB,0,hC,aOff,bOff,cOff,groups,gA,gB,gC}: row-major C = alpha op(A) op(B) + beta C
        NEED_F(2, 2);
        NEED_L(10, 17);
        const bool tA = pl[0] != 0, tB = pl[1] != 0;
        const int m = (int)pl[2], n = (int)pl[3], k = (int)pl[4];
        long long aOff = ll > 10 ? pl[10] : 0, bOff = ll > 11 ? pl[11] : 0, cOff = ll > 12 ? pl[12] : 0;
        const int groups = ll > 13 ? (int)pl[13] : 1;
        const long long gA = ll > 14 ? pl[14] : 0, gB = ll > 15 ? pl[15] : 0, gC = ll > 16 ? pl[16] : 0;
        if (m < 0 || n < 0 || k < 0 || groups < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *A, *B, *C;
        ERRCHK(mem((long)pl[6], &A));
        ERRCHK(mem((long)pl[7], &B));
        ERRCHK(mem((long)pl[9], &C));
        if (aOff < 0) aOff = 0;
        if (bOff < 0) bOff = 0;
        if (cOff < 0) cOff = 0;
        for (int g = 0; g < groups; g++) {
            const long long ao = aOff + gA * g, bo = bOff + gB * g, co = cOff + gC * g;
            RANGE(A, ao, (long long)m * k);
            RANGE(B, bo, (long long)k * n);
            RANGE(C, co, (long long)m * n);
            if (m == 0 || n == 0) continue;
            hipLaunchKernelGGL(d_gemm_kernel, dim3((n + 15) / 16, (m + 15) / 16, 1), 256, 0, s, m, n, k, pf[0], A->ptr + ao,
                               tA ? 1ll : (long long)k, tA ? (long long)m : 1ll, B->ptr + bo, tB ? 1ll : (long long)n,
                               tB ? (long long)k : 1ll, pf[1], C->ptr + co, (long long)n, 1ll, 0ll, 0ll, 0ll);
            LAUNCHED();
        }
        return 0;
    }
    case MCH_FN_GEMM2: {
        // f{alpha,beta}, l{tA,tB,m,n,k,0,hA,hB,0,hC,lda,ldb,ldc[,sA,sB,sC,batch]}: BLAS column-major (device.cu:1691-1726)
        NEED_F(2, 2);
        NEED_L(13, 17);
        if (ll != 13 && ll != 17) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const bool tA = pl[0] != 0, tB = pl[1] != 0;
        const int m = (int)pl[2], n = (int)pl[3], k = (int)pl[4];
        const long long lda = pl[10], ldb = pl[11], ldc = pl[12];
        long long sA = 0, sB = 0, sC = 0;
        int batch = 1;
        if (ll == 17) { sA = pl[13]; sB = pl[14]; sC = pl[15]; batch = (int)pl[16]; }
        if (m < 0 || n < 0 || k < 0 || batch < 1 || batch > 65535 || lda < 1 || ldb < 1 || ldc < 1 || sA < 0 || sB < 0 || sC < 0)
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *A, *B, *C;
        ERRCHK(mem((long)pl[6], &A));
        ERRCHK(mem((long)pl[7], &B));
        ERRCHK(mem((long)pl[9], &C));
        if (m == 0 || n == 0) return 0;
        const long long ac = tA ? m : k, bc = tB ? k : n, ar = tA ? k : m, br = tB ? n : k;   // stored columns / rows
        RANGE(A, 0, (batch - 1) * sA + (ac - 1) * lda + ar);
        RANGE(B, 0, (batch - 1) * sB + (bc - 1) * ldb + br);
        RANGE(C, 0, (batch - 1) * sC + (long long)(n - 1) * ldc + m);
        // column-major: element (i, kk) of op(A) is A[i + kk lda], or A[kk + i lda] when transposed
        hipLaunchKernelGGL(d_gemm_kernel, dim3((n + 15) / 16, (m + 15) / 16, batch), 256, 0, s, m, n, k, pf[0], A->ptr,
                           tA ? lda : 1ll, tA ? 1ll : lda, B->ptr, tB ? ldb : 1ll, tB ? 1ll : ldb, pf[1], C->ptr, 1ll, ldc, sA, sB, sC);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_GEMV: {
        // f{alpha,beta}, l{tA,m,n,0,hA,hX,0,hY,aOff,xOff,yOff}: A row-major (m, n); y = alpha op(A) x + beta y
        NEED_F(2, 2);
        NEED_L(8, 11);
        const bool tA = pl[0] != 0;
        const int m = (int)pl[1], n = (int)pl[2];
        long long aOff = ll > 8 ? pl[8] : 0, xOff = ll > 9 ? pl[9] : 0, yOff = ll > 10 ? pl[10] : 0;
        if (m < 0 || n < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *A, *X, *Y;
        ERRCHK(mem((long)pl[4], &A));
        ERRCHK(mem((long)pl[5], &X));
        ERRCHK(mem((long)pl[7], &Y));
        if (aOff < 0) aOff = 0;
        if (xOff < 0) xOff = 0;
        if (yOff < 0) yOff = 0;
        RANGE(A, aOff, (long long)m * n);
        RANGE(X, xOff, tA ? m : n);
        RANGE(Y, yOff, tA ? n : m);
        const int rows = tA ? n : m, inner = tA ? m : n;   // y (rows) = op(A) (rows x inner) x (inner)
        if (rows == 0) return 0;
        hipLaunchKernelGGL(d_gemm_kernel, dim3(1, (rows + 15) / 16, 1), 256, 0, s, rows, 1, inner, pf[0], A->ptr + aOff,
                           tA ? 1ll : (long long)n, tA ? (long long)n : 1ll, X->ptr + xOff, 1ll, 1ll, pf[1], Y->ptr + yOff, 1ll, 1ll,
                           0ll, 0ll, 0ll);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_AXPY: {
        // f{alpha}, l{n,0,hX,hY,xOff,yOff}
        NEED_F(1, 1);
        NEED_L(4, 6);
        const long long n = pl[0], xo = ll > 4 ? pl[4] : 0, yo = ll > 5 ? pl[5] : 0;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[2], &X));
        ERRCHK(mem((long)pl[3], &Y));
        RANGE(X, xo, n);
        RANGE(Y, yo, n);
        if (n) hipLaunchKernelGGL(d_axpy_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, pf[0], X->ptr + xo, Y->ptr + yo);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_SCAL:
    case MCH_FN_SCALE: {
        // SCAL f{alpha}, l{n,0,hX,xOff}; SCALE f{alpha}, l{n,0,hX,hY,xOff,yOff}
        NEED_F(1, 1);
        const bool inplace = fn == MCH_FN_SCAL;
        if (inplace) NEED_L(3, 4); else NEED_L(4, 6);
        const long long n = pl[0];
        const long long xo = inplace ? (ll > 3 ? pl[3] : 0) : (ll > 4 ? pl[4] : 0), yo = inplace ? xo : (ll > 5 ? pl[5] : 0);
        MemD *X, *Y;
        ERRCHK(mem((long)pl[2], &X));
        ERRCHK(mem((long)pl[inplace ? 2 : 3], &Y));
        RANGE(X, xo, n);
        RANGE(Y, yo, n);
        if (n) hipLaunchKernelGGL(d_scale_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, pf[0], X->ptr + xo, Y->ptr + yo);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_ADD: {
        // [f{alpha}], l{n,hA,hB,hY}: y = a + alpha b (math.cu:3363-3369)
        if (lf > 0 && pf) NEED_F(1, 1);
        NEED_L(4, 5);
        const long long n = pl[0];
        const double alpha = (lf > 0 && pf) ? pf[0] : 1.0;
        MemD *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        RANGE(A, 0, n);
        RANGE(B, 0, n);
        RANGE(Y, 0, n);
        if (n) hipLaunchKernelGGL(d_add_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, A->ptr, B->ptr, Y->ptr, alpha);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_MUL: {
        // l{n,hA,hB,hY,aOff,bOff,yOff}
        NEED_L(4, 7);
        const long long n = pl[0], ao = ll > 4 ? pl[4] : 0, bo = ll > 5 ? pl[5] : 0, yo = ll > 6 ? pl[6] : 0;
        MemD *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        RANGE(A, ao, n);
        RANGE(B, bo, n);
        RANGE(Y, yo, n);
        if (n) hipLaunchKernelGGL(d_mul_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, A->ptr + ao, B->ptr + bo, Y->ptr + yo);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_SILU_FWD: {
        // l{count,hBtm,hTop}
        NEED_L(3, 3);
        const long long n = pl[0];
        MemD *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        if (n) hipLaunchKernelGGL(d_silu_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, X->ptr, Y->ptr);
        LAUNCHED();
        return 0;
    }

    // ---- mask, layout (device.cu:2101-2145, 3088-3127, 3730-3748) --------------------------------------------------------
    case MCH_FN_MASK:
    case MCH_FN_MASK_BATCH: {
        // MASK f{search,replace}, l{n,maskDim,0,0,hX,hMask,hY}; MASK_BATCH l{n,batch,maskDim,0,0,hX,hMask,hY}
        NEED_F(2, 2);
        const bool batched = fn == MCH_FN_MASK_BATCH;
        if (batched) NEED_L(8, 8); else NEED_L(7, 7);
        const long long n = pl[0];
        const long long batch = batched ? pl[1] : 1, md = batched ? pl[2] : pl[1];
        if (md < 1 || batch < 1 || md < batch || (batched && n < batch)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const int o = batched ? 5 : 4;
        MemD *X, *M, *Y;
        ERRCHK(mem((long)pl[o], &X));
        ERRCHK(mem((long)pl[o + 1], &M));
        ERRCHK(mem((long)pl[o + 2], &Y));
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        if (n == 0) return 0;
        const long long md1 = batched ? md / batch : md, dd1 = batched ? n / batch : n;
        RANGE(M, 0, batched ? (md1 - 1) + ((n - 1) / dd1) * md1 + 1 : md);
        hipLaunchKernelGGL(d_mask_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (size_t)md1, (size_t)dd1, X->ptr, M->ptr, Y->ptr,
                           pf[0], pf[1]);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_TRANSPOSE: {
        // l{n,hX,hY,hXCounts,hYCounts,hMapping,numAxes,hBuffer}: the three small blobs hold element strides and the axis map
        NEED_L(8, 8);
        const long long n = pl[0];
        const int axes = (int)pl[6];
        MemD *X, *Y, *XC, *YC, *MP;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        ERRCHK(mem((long)pl[3], &XC));
        ERRCHK(mem((long)pl[4], &YC));
        ERRCHK(mem((long)pl[5], &MP));
        if (axes < 1 || axes > 8) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        RANGE(XC, 0, axes);
        RANGE(YC, 0, axes);
        RANGE(MP, 0, axes);
        double hx[8], hy[8], hm[8];
        HIPCHK(hipMemcpyAsync(hx, XC->ptr, axes * 8, hipMemcpyDeviceToHost, s));
        HIPCHK(hipMemcpyAsync(hy, YC->ptr, axes * 8, hipMemcpyDeviceToHost, s));
        HIPCHK(hipMemcpyAsync(hm, MP->ptr, axes * 8, hipMemcpyDeviceToHost, s));
        HIPCHK(hipStreamSynchronize(s));
        PermuteD a;
        a.axes = axes;
        for (int i = 0; i < axes; i++) {
            a.xs[i] = (long long)hx[i]; a.ys[i] = (long long)hy[i]; a.map[i] = (int)hm[i];
            if (a.xs[i] < 1 || a.ys[i] < 1 || a.map[i] < 0 || a.map[i] >= axes) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        if (n) hipLaunchKernelGGL(d_permute_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, X->ptr, Y->ptr, a);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_TRANSPOSE_HW: {
        // l{n,c,h,w,hSrc,hDst}
        NEED_L(6, 6);
        const long long nn = pl[0], c = pl[1], h = pl[2], w = pl[3];
        if (nn < 0 || c < 0 || h < 0 || w < 0 || h > INT_MAX || w > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        const long long total = nn * c * h * w;
        RANGE(X, 0, total);
        RANGE(Y, 0, total);
        if (total) hipLaunchKernelGGL(d_transpose_hw_kernel, grid_of((size_t)total), 256, 0, s, (size_t)total, (int)h, (int)w, X->ptr, Y->ptr);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_COPY: {
        // l{count,outer,channels,blocks,inner,offset,hX,hY,dir}
        NEED_L(9, 9);
        const long long n = pl[0], chn = pl[2], blocks = pl[3], inner = pl[4], off = pl[5];
        const int dir = (int)pl[8];
        if (n < 0 || chn < 1 || blocks < 1 || inner < 1 || off < 0 || off >= blocks) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[6], &X));
        ERRCHK(mem((long)pl[7], &Y));
        RANGE(Y, 0, n);
        if (n == 0) return 0;
        const long long last = n - 1;
        const long long xi = ((last / (chn * inner)) * chn + (last % (chn * inner)) / inner) * blocks * inner + off * inner + last % inner;
        RANGE(X, 0, xi + (inner - 1 - last % inner) + 1);
        hipLaunchKernelGGL(d_channel_copy_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (int)chn, (int)blocks, (int)inner, (int)off,
                           X->ptr, Y->ptr, dir);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_EMBED_FWD: {
        // l{count,hBtm,hWeight,M,N,K,hTop} (math.cu:9314-9330)
        NEED_L(7, 7);
        const long long n = pl[0], N = pl[4], K = pl[5];
        if (n < 0 || N < 1 || K < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *I, *W, *T;
        ERRCHK(mem((long)pl[1], &I));
        ERRCHK(mem((long)pl[2], &W));
        ERRCHK(mem((long)pl[6], &T));
        RANGE(T, 0, n);
        RANGE(I, 0, (n + N - 1) / N);
        RANGE(W, 0, K * N);
        if (n) hipLaunchKernelGGL(d_embed_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, I->ptr, W->ptr, (int)N, T->ptr);
        LAUNCHED();
        return 0;
    }

    // ---- descriptors, softmax (device.h:1201-1262, 4778-4798) -----------------------------------------------------------
    case MCH_FN_CREATE_CUDNN: {
        ERRCHK(verify_d(lf, pf, 0, 1));
        long h;
        ERRCHK(m_cudnn.create(&h));
        return set_out_d((double)h, ppOut, plOut);
    }
    case MCH_FN_FREE_CUDNN:
        NEED_F(1, 1);
        return m_cudnn.free((long)pf[0]);
    case MCH_FN_CREATE_TENSORDESC: {
        long h;
        ERRCHK(m_tdesc.create(&h));
        return set_out_d((double)h, ppOut, plOut);
    }
    case MCH_FN_FREE_TENSORDESC:
        NEED_F(1, 1);
        return m_tdesc.free((long)pf[0]);
    case MCH_FN_SET_TENSORDESC: {
        // l{h,half,n,c,h,w[,sn,sc,sh,sw]}
        NEED_L(6, 10);
        if (ll != 6 && ll != 10) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        TensorDesc* d = m_tdesc.get((long)pl[0]);
        if (!d) return MCH_ERROR_PARAM_NULL;
        d->half = false;
        d->n = (int)pl[2]; d->c = (int)pl[3]; d->h = (int)pl[4]; d->w = (int)pl[5];
        if (ll == 6) { d->sw = 1; d->sh = d->w; d->sc = d->h * d->sh; d->sn = d->c * d->sc; }
        else { d->sn = (int)pl[6]; d->sc = (int)pl[7]; d->sh = (int)pl[8]; d->sw = (int)pl[9]; }
        return 0;
    }
    case MCH_FN_SOFTMAX_FWD: {
        // f{alpha,beta}, l{hCudnn,0,hBtmDesc,hBtm,0,hTopDesc,hTop,alg,mode}
        NEED_F(2, 2);
        NEED_L(9, 9);
        if (!m_cudnn.get((long)pl[0])) return MCH_ERROR_PARAM_NULL;
        TensorDesc* bd = m_tdesc.get((long)pl[2]);
        TensorDesc* td = m_tdesc.get((long)pl[5]);
        if (!bd || !td) return MCH_ERROR_PARAM_NULL;
        if (pf[0] != 1.0 || pf[1] != 0.0) { last_detail = "softmax supports alpha=1, beta=0 only"; return MCH_ERROR_NOT_IMPLEMENTED; }
        const int alg = (int)pl[7], mode = (int)pl[8];   // alg 0 fast, 1 accurate, 2 log; mode 0 instance, 1 channel
        if (alg < 0 || alg > 2 || mode < 0 || mode > 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (bd->n != td->n || bd->c != td->c || bd->h != td->h || bd->w != td->w) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const bool packed = bd->sw == 1 && bd->sh == bd->w && bd->sc == bd->h * bd->w && bd->sn == bd->c * bd->h * bd->w &&
                            td->sw == 1 && td->sh == td->w && td->sc == td->h * td->w && td->sn == td->c * td->h * td->w;
        if (!packed) { last_detail = "softmax needs fully packed NCHW descriptors"; return MCH_ERROR_NOT_IMPLEMENTED; }
        const long long total = (long long)bd->n * bd->c * bd->h * bd->w;
        const int len = mode == 0 ? bd->c * bd->h * bd->w : bd->c, inner = mode == 0 ? 1 : bd->h * bd->w;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[3], &X));
        ERRCHK(mem((long)pl[6], &Y));
        RANGE(X, 0, total);
        RANGE(Y, 0, total);
        const long long rows = (long long)bd->n * inner;
        if (total == 0) return 0;
        if (rows > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        hipLaunchKernelGGL(d_softmax_kernel, (int)rows, 256, 0, s, (const double*)X->ptr, Y->ptr, len, inner, alg == 2);
        LAUNCHED();
        return 0;
    }

    case MCH_FN_SOFTMAX_BWD: {
        // f{alpha,beta}, l{hCudnn,0,hTopDataDesc,hTopData,hTopDiffDesc,hTopDiff,0,hBtmDiffDesc,hBtmDiff,alg,mode} (device.h:4801-4823)
        NEED_F(2, 2);
        NEED_L(11, 11);
        if (!m_cudnn.get((long)pl[0])) return MCH_ERROR_PARAM_NULL;
        TensorDesc* yd = m_tdesc.get((long)pl[2]);
        TensorDesc* gd = m_tdesc.get((long)pl[4]);
        TensorDesc* bd = m_tdesc.get((long)pl[7]);
        if (!yd || !gd || !bd) return MCH_ERROR_PARAM_NULL;
        if (pf[0] != 1.0 || pf[1] != 0.0) { last_detail = "softmax supports alpha=1, beta=0 only"; return MCH_ERROR_NOT_IMPLEMENTED; }
        const int alg = (int)pl[9], mode = (int)pl[10];
        if (alg < 0 || alg > 2 || mode < 0 || mode > 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        for (TensorDesc* d : {gd, bd})
            if (d->n != yd->n || d->c != yd->c || d->h != yd->h || d->w != yd->w) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        for (TensorDesc* d : {yd, gd, bd})
            if (!(d->sw == 1 && d->sh == d->w && d->sc == d->h * d->w && d->sn == d->c * d->h * d->w)) {
                last_detail = "softmax needs fully packed NCHW descriptors";
                return MCH_ERROR_NOT_IMPLEMENTED;
            }
        MemD *Y, *G, *X;
        ERRCHK(mem((long)pl[3], &Y));
        ERRCHK(mem((long)pl[5], &G));
        ERRCHK(mem((long)pl[8], &X));
        const long long total = (long long)yd->n * yd->c * yd->h * yd->w;
        RANGE(Y, 0, total);
        RANGE(G, 0, total);
        RANGE(X, 0, total);
        const int len = mode == 0 ? yd->c * yd->h * yd->w : yd->c, inner = mode == 0 ? 1 : yd->h * yd->w;
        const long long series = (long long)yd->n * inner;
        if (total == 0) return 0;
        if (series > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        hipLaunchKernelGGL(d_softmax_bwd_kernel, (int)series, 256, 0, s, (const double*)Y->ptr, (const double*)G->ptr, X->ptr, len, inner, alg == 2);
        LAUNCHED();
        return 0;
    }

    // ---- the layers around the attention: activations, norms, the primitives of their chains --------------------------------
    case MCH_FN_SWIGLU_FWD: {
        // l{n,hA,hB,hY}: y = silu(a) b
        NEED_L(4, 4);
        const long long n = pl[0];
        MemD *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        RANGE(A, 0, n);
        RANGE(B, 0, n);
        RANGE(Y, 0, n);
        if (n) hipLaunchKernelGGL(d_swiglu_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)A->ptr, (const double*)B->ptr, Y->ptr);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_SILU_BWD:
    case MCH_FN_GELU_BWD: {
        // l{count,hTopDiff,hTopData,hBtmDiff,hBtmData[,bert]} (device.h:3269-3316)
        const bool gelu = fn == MCH_FN_GELU_BWD;
        NEED_L(gelu ? 6 : 5, gelu ? 6 : 5);
        const long long n = pl[0];
        MemD *dY, *dX, *X;
        ERRCHK(mem((long)pl[1], &dY));
        ERRCHK(mem((long)pl[3], &dX));
        ERRCHK(mem((long)pl[4], &X));
        RANGE(dY, 0, n);
        RANGE(dX, 0, n);
        RANGE(X, 0, n);
        if (n && gelu) hipLaunchKernelGGL(d_gelu_bwd_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)dY->ptr, (const double*)X->ptr, dX->ptr, pl[5] != 0);
        else if (n) hipLaunchKernelGGL(d_silu_bwd_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)dY->ptr, (const double*)X->ptr, dX->ptr);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_GELU_FWD:
    case MCH_FN_RELU_FWD: {
        // GELU l{count,hBtm,hTop,bert}; ReLU f{negativeSlope}, l{count,hBtm,hTop,0} (device.h:3253-3266, 4925-4940)
        const bool gelu = fn == MCH_FN_GELU_FWD;
        if (!gelu) NEED_F(1, 1);
        NEED_L(4, 4);
        const long long n = pl[0];
        MemD *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        if (n && gelu) hipLaunchKernelGGL(d_gelu_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)X->ptr, Y->ptr, pl[3] != 0);
        else if (n) hipLaunchKernelGGL(d_relu_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)X->ptr, Y->ptr, pf[0]);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_RELU_BWD: {
        // f{negativeSlope}, l{count,hTopDiff,hTopData,hBtmDiff,0} (device.h:4943-4959)
        NEED_F(1, 1);
        NEED_L(5, 5);
        const long long n = pl[0];
        MemD *dY, *Y, *dX;
        ERRCHK(mem((long)pl[1], &dY));
        ERRCHK(mem((long)pl[2], &Y));
        ERRCHK(mem((long)pl[3], &dX));
        RANGE(dY, 0, n);
        RANGE(Y, 0, n);
        RANGE(dX, 0, n);
        if (n) hipLaunchKernelGGL(d_relu_bwd_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)dY->ptr, (const double*)Y->ptr, dX->ptr, pf[0]);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CREATE_LAYERNORM: {
        // f{eps}, l{gpuId,count,outer,channels,inner} (device.h:4123-4147)
        NEED_F(1, 1);
        NEED_L(5, 5);
        const long long count = pl[1], outer = pl[2], channels = pl[3], inner = pl[4];
        if (outer < 1 || channels < 1 || inner < 1 || count > INT_MAX || outer * channels > INT_MAX || count != outer * channels * inner)
            return MCH_ERROR_PARAM_OUT_OF_RANGE;   // layernorm.cu:141-142
        long h;
        ERRCHK(m_layernorm.create(&h));
        LayerNormD* ln = m_layernorm.get(h);
        ln->count = (int)count; ln->outer = (int)outer; ln->channels = (int)channels; ln->inner = (int)inner;
        ln->eps = pf[0];
        hipError_t e = hipMalloc((void**)&ln->stdev, (size_t)(outer * channels) * sizeof(double));
        if (e != hipSuccess) { ln->stdev = nullptr; m_layernorm.free(h); return (long)e; }
        ln->set = true;
        return set_out_d((double)h, ppOut, plOut);
    }
    case MCH_FN_FREE_LAYERNORM:
        NEED_F(1, 1);
        HIPCHK(hipStreamSynchronize(s));
        return m_layernorm.free((long)pf[0]);
    case MCH_FN_LAYERNORM_FWD: {
        // l{hLayerNorm,hX,hY} (layernorm.cu:219-262)
        NEED_L(3, 3);
        LayerNormD* ln = m_layernorm.get((long)pl[0]);
        if (!ln || !ln->set) return MCH_ERROR_LAYERNORM_NOT_INITIALIZED;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(X, 0, ln->count);
        RANGE(Y, 0, ln->count);
        hipLaunchKernelGGL(d_layernorm_fwd_kernel, ln->outer * ln->channels, 256, 0, s, ln->inner, (const double*)X->ptr, Y->ptr, ln->stdev, ln->eps);
        LAUNCHED();
        ln->backwards = 0;
        return 0;
    }
    case MCH_FN_LAYERNORM_BWD: {
        // l{hLayerNorm,hYdata,hYdiff,hXdiff} (layernorm.cu:268-312)
        NEED_L(4, 4);
        LayerNormD* ln = m_layernorm.get((long)pl[0]);
        if (!ln || !ln->set) return MCH_ERROR_LAYERNORM_NOT_INITIALIZED;
        MemD *Y, *dY, *dX;
        ERRCHK(mem((long)pl[1], &Y));
        ERRCHK(mem((long)pl[2], &dY));
        ERRCHK(mem((long)pl[3], &dX));
        RANGE(Y, 0, ln->count);
        RANGE(dY, 0, ln->count);
        RANGE(dX, 0, ln->count);
        ln->backwards++;
        const int rows = ln->outer * ln->channels;
        hipLaunchKernelGGL(d_layernorm_bwd_kernel, rows, 256, 0, s, rows, ln->inner, (const double*)Y->ptr, (const double*)dY->ptr, dX->ptr,
                           (const double*)ln->stdev, ln->eps * (double)ln->backwards);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_RMSNORM_FWD: {
        // f{eps}, l{outer,dim,hX,hWeight(0 = none),hY}
        NEED_F(1, 1);
        NEED_L(5, 5);
        const long long outer = pl[0], dim = pl[1];
        if (outer < 0 || dim < 1 || outer > INT_MAX || dim > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *W = nullptr, *Y;
        ERRCHK(mem((long)pl[2], &X));
        if (pl[3]) ERRCHK(mem((long)pl[3], &W));
        ERRCHK(mem((long)pl[4], &Y));
        RANGE(X, 0, outer * dim);
        RANGE(Y, 0, outer * dim);
        if (W) RANGE(W, 0, dim);
        if (outer) hipLaunchKernelGGL(d_rmsnorm_kernel, (int)outer, 256, 0, s, (int)dim, (const double*)X->ptr, W ? (const double*)W->ptr : nullptr, Y->ptr, pf[0]);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_SUB: {
        // l{n,hA,hB,hY[,aOff,bOff,yOff,nB]}: y = a - b[i % nB] when nB > 0 (device.cu:2294-2331)
        NEED_L(4, 8);
        const long long n = pl[0], ao = ll > 4 ? pl[4] : 0, bo = ll > 5 ? pl[5] : 0, yo = ll > 6 ? pl[6] : 0, nB = ll > 7 ? pl[7] : 0;
        MemD *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        if (nB < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(A, ao, n);
        RANGE(B, bo, nB > 0 ? (nB < n ? nB : n) : n);
        RANGE(Y, yo, n);
        if (n) hipLaunchKernelGGL(d_sub_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)A->ptr + ao, (const double*)B->ptr + bo, Y->ptr + yo, (size_t)nB);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_DIV: {
        // l{n,hA,hB,hY}: y = b == 0 ? 0 : a / b (device.cu:2492-2505)
        NEED_L(4, 4);
        const long long n = pl[0];
        MemD *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        RANGE(A, 0, n);
        RANGE(B, 0, n);
        RANGE(Y, 0, n);
        if (n) hipLaunchKernelGGL(d_div_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)A->ptr, (const double*)B->ptr, Y->ptr);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_ADD_SCALAR: {
        // f{alpha}, l{n,0,hY[,yOff]} (device.cu:2183-2201)
        NEED_F(1, 1);
        NEED_L(3, 4);
        const long long n = pl[0], yo = ll > 3 ? pl[3] : 0;
        MemD* Y;
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(Y, yo, n);
        if (n) hipLaunchKernelGGL(d_add_scalar_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, pf[0], Y->ptr + yo);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_POWX: {
        // f{alpha}, l{n,hA,0,hY[,aOff,yOff]} (device.cu:2595-2618)
        NEED_F(1, 1);
        NEED_L(4, 6);
        const long long n = pl[0], ao = ll > 4 ? pl[4] : 0, yo = ll > 5 ? pl[5] : 0;
        MemD *A, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[3], &Y));
        RANGE(A, ao, n);
        RANGE(Y, yo, n);
        if (n) hipLaunchKernelGGL(d_powx_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)A->ptr + ao, pf[0], Y->ptr + yo);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_SQRT: {
        // [f{epsilon}], l{n,hX,hY}: y = sqrt(x + epsilon) (device.cu:2712-2728)
        NEED_L(3, 3);
        const long long n = pl[0];
        MemD *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        if (n) hipLaunchKernelGGL(d_sqrt_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)X->ptr, Y->ptr, (lf > 0 && pf) ? pf[0] : 0.0);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_INVERT: {
        // [f{numerator, denominator}], l{n,hX,hY[,xOff,yOff]}: 0 stays 0; factors 0 and 1 are ignored (device.cu:2624-2655)
        NEED_L(3, 5);
        const long long n = pl[0], xo = ll > 3 ? pl[3] : 0, yo = ll > 4 ? pl[4] : 0;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(X, xo, n);
        RANGE(Y, yo, n);
        const double num = (lf > 0 && pf) ? pf[0] : 1.0, den = (lf > 1 && pf) ? pf[1] : 1.0;
        if (n) hipLaunchKernelGGL(d_invert_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)X->ptr + xo, Y->ptr + yo,
                                  (num != 0.0 && num != 1.0) ? num : 1.0, (den != 0.0 && den != 1.0) ? den : 1.0);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_EXP:
    case MCH_FN_LOG: {
        // 235 [f{beta}] l{n,hA,hY[,aOff,yOff,0]}: y = exp(beta a); 236 [f{beta[,alpha]}] l{n,hA,hY[,0,0]}: y = log(beta (a + alpha))
        const bool isExp = fn == MCH_FN_EXP;
        ERRCHK(verify_d(lf, pf, 0, isExp ? 1 : 2));
        if (isExp) NEED_L(3, 6); else NEED_L(3, 5);
        const long long n = pl[0];
        long long aOff = isExp && ll > 3 ? pl[3] : 0, yOff = isExp && ll > 4 ? pl[4] : 0;
        if (n < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (aOff < 0) aOff = 0;
        if (yOff < 0) yOff = 0;
        const double beta = lf > 0 ? pf[0] : 1.0, alpha = !isExp && lf > 1 ? pf[1] : 0.0;
        MemD *A, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(A, aOff, n);
        RANGE(Y, yOff, n);
        if (n && isExp) hipLaunchKernelGGL(d_exp_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)A->ptr + aOff, Y->ptr + yOff, beta);
        else if (n) hipLaunchKernelGGL(d_log_kernel, grid_of((size_t)n), 256, 0, s, (size_t)n, (const double*)A->ptr, Y->ptr, beta, alpha);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_MEAN: {
        // l{count,outer,channels,inner,hX,hY[,xOff]}: y[outer*channels] = row means (device.cu:3386-3405)
        NEED_L(6, 7);
        const long long outer = pl[1], ch = pl[2], inner = pl[3], xo = ll > 6 ? pl[6] : 0;
        if (outer < 0 || ch < 0 || inner < 1 || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        RANGE(X, xo, outer * ch * inner);
        RANGE(Y, 0, outer * ch);
        if (outer * ch) hipLaunchKernelGGL(d_rowsum_kernel, grid_of((size_t)(outer * ch)), 256, 0, s, (size_t)(outer * ch), (int)inner,
                                           (const double*)X->ptr + xo, Y->ptr, 1.0 / (double)inner);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_MAX: {
        // l{count,outer,channels,inner,hX,hY,returnIdx[,acrossChannels]} (device.cu:3359-3380)
        NEED_L(7, 8);
        const long long outer = pl[1], ch = pl[2], inner = pl[3];
        const bool idx = pl[6] != 0, across = ll > 7 ? pl[7] != 0 : true;
        if (outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (X->ptr == Y->ptr) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, across ? outer * ch * inner : outer * inner * inner);
        RANGE(Y, 0, outer * inner);
        if (outer * inner) hipLaunchKernelGGL(d_channel_max_kernel, grid_of((size_t)(outer * inner)), 256, 0, s, (size_t)(outer * inner), (int)ch, (int)inner,
                                              (const double*)X->ptr, Y->ptr, idx, across);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_SUB:
    case MCH_FN_CHANNEL_DIV: {
        // 291 l{count,outer,channels,inner,hX,hY[,hA]}: y[n,c,s] = a[n,c,s] - x[n,s], a = y when absent (device.cu:3438-3457)
        // 293 l{count,outer,channels,inner,hX,hY[,method]}: y[n,c,s] /= x[n,s]; method 2 with count = outer * inner (device.cu:3541-3560)
        NEED_L(6, 7);
        const bool sub = fn == MCH_FN_CHANNEL_SUB;
        long long count = pl[0];
        const long long outer = pl[1], ch = pl[2], inner = pl[3];
        if (count < 0 || outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (!sub && ll > 6 && pl[6] == 2) {
            if (count != outer * inner) { last_detail = "channel_div method 2 takes count = outer * inner only"; return MCH_ERROR_PARAM_OUT_OF_RANGE; }
            count *= ch;
        }
        if (count > outer * ch * inner) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y, *A = nullptr;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (sub && ll > 6) ERRCHK(mem((long)pl[6], &A));
        RANGE(X, 0, outer * inner);
        RANGE(Y, 0, count);
        if (A) RANGE(A, 0, count);
        if (count) hipLaunchKernelGGL(d_channel_bcast_kernel, grid_of((size_t)count), 256, 0, s, (size_t)count, (int)ch, (int)inner,
                                      (const double*)(A ? A->ptr : Y->ptr), (const double*)X->ptr, Y->ptr, sub);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_DOT: {
        // l{count,outer,channels,inner,hX,hA,hY}: y[n,s] = sum_c x[n,c,s] a[n,c,s] (device.cu:3638-3654)
        NEED_L(7, 7);
        const long long outer = pl[1], ch = pl[2], inner = pl[3];
        if (outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *A, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &A));
        ERRCHK(mem((long)pl[6], &Y));
        if (Y->ptr == X->ptr || Y->ptr == A->ptr) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, outer * ch * inner);
        RANGE(A, 0, outer * ch * inner);
        RANGE(Y, 0, outer * inner);
        if (outer * inner) hipLaunchKernelGGL(d_colsum_kernel, grid_of((size_t)(outer * inner)), 256, 0, s, (size_t)(outer * inner), (int)ch, (int)inner,
                                              (const double*)X->ptr, (const double*)A->ptr, Y->ptr);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_SUM:
    case MCH_FN_CHANNEL_SUM2: {
        // 292 l{count,outer,channels,inner,hX,hY}: y[outer,inner] = sum over the channels (device.cu:3488-3503)
        // 309 l{count,outer,channels,inner,hX,hY,acrossChannels[,dir,channelsY]} (device.cu:3510-3534): forward sums across the
        //     channels or within every channel; backward writes X from Y, every Y value spread over what it was summed from
        const bool two = fn == MCH_FN_CHANNEL_SUM2;
        if (two) NEED_L(7, 9); else NEED_L(6, 6);
        long long outer = pl[1];
        const long long ch = pl[2], inner = pl[3];
        const bool across = two ? pl[6] != 0 : true;
        const int dir = two && ll > 7 ? (int)pl[7] : 0;
        const long long chY = two && ll > 8 ? pl[8] : -1;
        if (outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        // RMSNormLayer.cs:198-199 passes its weight gradient (inner values) as Y with outer = batch: only what Y holds is computed
        if (!two && outer > 1 && (long long)Y->count < outer * inner && (long long)Y->count >= inner) outer = (long long)Y->count / inner;
        const long long full = outer * ch * inner, reduced = across ? outer * inner : outer * ch;
        RANGE(X, 0, full);
        RANGE(Y, 0, reduced);
        if (dir == 0) {
            if (X->ptr == Y->ptr) return MCH_ERROR_PARAM_OUT_OF_RANGE;
            if (reduced == 0) return 0;
            if (across) hipLaunchKernelGGL(d_colsum_kernel, grid_of((size_t)reduced), 256, 0, s, (size_t)reduced, (int)ch, (int)inner, (const double*)X->ptr,
                                           (const double*)nullptr, Y->ptr);
            else hipLaunchKernelGGL(d_rowsum_kernel, grid_of((size_t)reduced), 256, 0, s, (size_t)reduced, (int)inner, (const double*)X->ptr, Y->ptr, 1.0);
            LAUNCHED();
            return 0;
        }
        if (chY == 1 && chY != ch) { last_detail = "channel_sum backward with channelsY = 1 is not supported"; return MCH_ERROR_NOT_IMPLEMENTED; }
        if (full == 0) return 0;
        if (across) hipLaunchKernelGGL(d_spread_kernel, grid_of((size_t)full), 256, 0, s, 3, (size_t)full, (size_t)1, (size_t)(ch * inner), (size_t)inner, Y->ptr, X->ptr);
        else hipLaunchKernelGGL(d_spread_kernel, grid_of((size_t)full), 256, 0, s, 0, (size_t)full, (size_t)inner, (size_t)1, (size_t)1, Y->ptr, X->ptr);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_CHANNEL_FILLFROM:
    case MCH_FN_CHANNEL_COPYALL:
    case MCH_FN_CHANNEL_DUP: {
        // l{count,outer,channels,inner,hX,hY[,dir]} (math.cu:7465-7481, 7630-7639, 7667-7676)
        const bool fill = fn == MCH_FN_CHANNEL_FILLFROM;
        NEED_L(fill ? 7 : 6, fill ? 7 : 6);
        const long long n = pl[0], outer = pl[1], ch = pl[2], inner = pl[3];
        if (n < 0 || outer < 1 || ch < 1 || inner < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (fill && pl[6] != 0) {
            // backward: x[i] = y[i * inner], i < outer * channels
            RANGE(X, 0, outer * ch);
            RANGE(Y, 0, (outer * ch - 1) * inner + 1);
            hipLaunchKernelGGL(d_spread_kernel, grid_of((size_t)(outer * ch)), 256, 0, s, 1, (size_t)(outer * ch), (size_t)inner, (size_t)1, (size_t)1, X->ptr, Y->ptr);
            LAUNCHED();
            return 0;
        }
        RANGE(Y, 0, n);
        if (n == 0) return 0;
        if (fill) {
            RANGE(X, 0, (n - 1) / inner + 1);
            hipLaunchKernelGGL(d_spread_kernel, grid_of((size_t)n), 256, 0, s, 0, (size_t)n, (size_t)inner, (size_t)1, (size_t)1, X->ptr, Y->ptr);
        } else if (fn == MCH_FN_CHANNEL_COPYALL) {
            RANGE(X, 0, n < ch * inner ? n : ch * inner);
            hipLaunchKernelGGL(d_spread_kernel, grid_of((size_t)n), 256, 0, s, 2, (size_t)n, (size_t)1, (size_t)(ch * inner), (size_t)1, X->ptr, Y->ptr);
        } else {
            RANGE(X, 0, ((n - 1) / (ch * inner)) * ch + ch);
            hipLaunchKernelGGL(d_spread_kernel, grid_of((size_t)n), 256, 0, s, 3, (size_t)n, (size_t)1, (size_t)(ch * inner), (size_t)ch, X->ptr, Y->ptr);
        }
        LAUNCHED();
        return 0;
    }

    // ---- attention handle (device.h:2435-2506, attn.cu:408-602) ------------------------------------------------------------
    case MCH_FN_ATTN_CREATE: {
        long h;
        ERRCHK(m_attn.create(&h));
        return set_out_d((double)h, ppOut, plOut);
    }
    case MCH_FN_ATTN_FREE:
        NEED_F(1, 1);
        return m_attn.free((long)pf[0]);
    case MCH_FN_ATTN_SET: {
        // f{dropout}, l{hCudnn,hAttn,gpuId,training,batch,blockSize,heads,hs,seed}
        NEED_L(9, 9);
        NEED_F(1, 1);
        AttnD* st = m_attn.get((long)pl[1]);
        if (!st) return MCH_ERROR_ATTN_NOT_INITIALIZED;
        if (pl[4] < 1 || pl[5] < 1 || pl[6] < 1 || pl[7] < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (pl[3] != 0 && pf[0] != 0.0) {
            last_detail = "the double base type runs the attention handle without dropout";
            return MCH_ERROR_NOT_IMPLEMENTED;
        }
        st->batch = (int)pl[4]; st->block = (int)pl[5]; st->heads = (int)pl[6]; st->hs = (int)pl[7];
        st->scale = 1.0 / sqrt((double)st->hs);   // attn.cu:427
        st->set = true;
        return 0;
    }
    case MCH_FN_ATTN_FWD: {
        // l{hCudnn,hAttn,blockSize,hQ,hK,hV,hMask,hY,batchMask[,blockSizeK[,mergedY]]}; the tenth and eleventh values as in the
        // fp32 library (key length when it differs, Y written head-merged)
        NEED_L(9, 11);
        AttnD* st = m_attn.get((long)pl[1]);
        if (!st || !st->set) return MCH_ERROR_ATTN_NOT_INITIALIZED;
        const int T = (int)pl[2], Tk = ll > 9 ? (int)pl[9] : T;
        const bool merged = ll > 10 && pl[10] != 0;
        if (T > st->block || Tk > st->block) return MCH_ERROR_ATTN_INVALID_BLOCK_SIZE;
        if (T < 1 || Tk < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *Q, *K, *V, *Y, *M = nullptr;
        ERRCHK(mem((long)pl[3], &Q));
        ERRCHK(mem((long)pl[4], &K));
        ERRCHK(mem((long)pl[5], &V));
        ERRCHK(mem((long)pl[7], &Y));
        const long long batchMask = pl[8];   // 0: (1,1,T,T); 1: (B,T,1,1); 2: (B,T,T)
        if (batchMask < 0 || batchMask > 2) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (pl[6]) ERRCHK(mem((long)pl[6], &M));
        const long long qn = (long long)st->batch * st->heads * T * st->hs, kn = (long long)st->batch * st->heads * Tk * st->hs;
        if ((long long)Q->count < qn || (long long)Y->count < qn || (long long)K->count < kn || (long long)V->count < kn)
            return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
        int kind = 0;
        ERRCHK(attn_mask_kind(st, M, batchMask, T, Tk, &kind));
        const size_t lds = ((size_t)Tk + st->hs) * sizeof(double);
        if (lds > 60000) { last_detail = "the double attention call keeps a row of scores in LDS: up to about 7000 keys"; return MCH_ERROR_NOT_IMPLEMENTED; }
        const long long rows = (long long)st->batch * st->heads * T;
        if (rows > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        hipLaunchKernelGGL(d_attn_row_kernel, (int)rows, 256, lds, s, (const double*)Q->ptr, (const double*)K->ptr, (const double*)V->ptr,
                           Y->ptr, st->heads, T, Tk, st->hs, st->scale, M ? (const double*)M->ptr : nullptr, kind, merged, (double*)nullptr);
        LAUNCHED();
        st->lastTq = T; st->lastTk = Tk; st->lastBatchMask = batchMask; st->lastMask = (long)pl[6];
        return 0;
    }
    case MCH_FN_ATTN_BWD: {
        // l{hCudnn,hAttn,hQ,hdQ,hK,hdK,hV,hdV,hMask,hY,hdY} (attn.cu:608-661): dV = P^T dY, dP = dY V^T, dS = P (dP - sum P dP),
        // dQ = scale dS K, dK = scale dS^T Q, with the probabilities recomputed under the last forward call's lengths and
        // mask (the reference reads the ones that call left behind); without a forward call: block size and hMask
        NEED_L(11, 11);
        AttnD* st = m_attn.get((long)pl[1]);
        if (!st || !st->set) return MCH_ERROR_ATTN_NOT_INITIALIZED;
        const int T = st->lastTq > 0 ? st->lastTq : st->block, Tk = st->lastTq > 0 ? st->lastTk : st->block;
        const long long batchMask = st->lastTq > 0 ? st->lastBatchMask : 0;
        MemD *Q, *dQ, *K, *dK, *V, *dV, *dY, *M = nullptr;
        ERRCHK(mem((long)pl[2], &Q));
        ERRCHK(mem((long)pl[3], &dQ));
        ERRCHK(mem((long)pl[4], &K));
        ERRCHK(mem((long)pl[5], &dK));
        ERRCHK(mem((long)pl[6], &V));
        ERRCHK(mem((long)pl[7], &dV));
        ERRCHK(mem((long)pl[10], &dY));
        const long hMask = st->lastTq > 0 ? st->lastMask : (long)pl[8];
        if (hMask) ERRCHK(mem(hMask, &M));
        const int H = st->heads, hs = st->hs;
        const long long bh = (long long)st->batch * H, qn = bh * T * hs, kn = bh * Tk * hs;
        if ((long long)Q->count < qn || (long long)dQ->count < qn || (long long)dY->count < qn || (long long)K->count < kn ||
            (long long)dK->count < kn || (long long)V->count < kn || (long long)dV->count < kn)
            return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
        int kind = 0;
        ERRCHK(attn_mask_kind(st, M, batchMask, T, Tk, &kind));
        const size_t lds = ((size_t)Tk + hs) * sizeof(double);
        const long long rows = bh * T, pn = rows * Tk;
        if (lds > 60000 || rows > INT_MAX || bh > 65535 || pn > (1ll << 28)) {
            last_detail = "the double attention gradient keeps the probabilities of all rows: up to 2^28 of them, about 7000 keys a row";
            return MCH_ERROR_NOT_IMPLEMENTED;
        }
        double* P;
        ERRCHK(workspace((size_t)pn * 2, &P));
        double* dP = P + pn;
        hipLaunchKernelGGL(d_attn_row_kernel, (int)rows, 256, lds, s, (const double*)Q->ptr, (const double*)K->ptr, (const double*)V->ptr,
                           (double*)nullptr, H, T, Tk, hs, st->scale, M ? (const double*)M->ptr : nullptr, kind, false, P);
        LAUNCHED();
        const long long sq = (long long)T * hs, sk = (long long)Tk * hs, sp = (long long)T * Tk;
        // dV (Tk x hs) = P^T dY
        hipLaunchKernelGGL(d_gemm_kernel, dim3((hs + 15) / 16, (Tk + 15) / 16, (int)bh), 256, 0, s, Tk, hs, T, 1.0, (const double*)P, 1ll, (long long)Tk,
                           (const double*)dY->ptr, (long long)hs, 1ll, 0.0, dV->ptr, (long long)hs, 1ll, sp, sq, sk);
        // dP (T x Tk) = dY V^T
        hipLaunchKernelGGL(d_gemm_kernel, dim3((Tk + 15) / 16, (T + 15) / 16, (int)bh), 256, 0, s, T, Tk, hs, 1.0, (const double*)dY->ptr, (long long)hs, 1ll,
                           (const double*)V->ptr, 1ll, (long long)hs, 0.0, dP, (long long)Tk, 1ll, sq, sk, sp);
        hipLaunchKernelGGL(d_attn_ds_kernel, (int)rows, 256, 0, s, (const double*)P, dP, Tk);
        // dQ (T x hs) = scale dS K;  dK (Tk x hs) = scale dS^T Q
        hipLaunchKernelGGL(d_gemm_kernel, dim3((hs + 15) / 16, (T + 15) / 16, (int)bh), 256, 0, s, T, hs, Tk, st->scale, (const double*)dP, (long long)Tk, 1ll,
                           (const double*)K->ptr, (long long)hs, 1ll, 0.0, dQ->ptr, (long long)hs, 1ll, sp, sk, sq);
        hipLaunchKernelGGL(d_gemm_kernel, dim3((hs + 15) / 16, (Tk + 15) / 16, (int)bh), 256, 0, s, Tk, hs, T, st->scale, (const double*)dP, 1ll, (long long)Tk,
                           (const double*)Q->ptr, (long long)hs, 1ll, 0.0, dK->ptr, (long long)hs, 1ll, sp, sq, sk);
        LAUNCHED();
        return 0;
    }

    // ---- rotary embedding (device.h:4201-4263, rope.cu:502-607, 785-825) ----------------------------------------------------
    case MCH_FN_CREATE_ROPE: {
        // f{theta}, l{sharedIdx,gpuId,count,batch,seqLen,heads,hs}
        NEED_F(1, 1);
        NEED_L(7, 7);
        const long long seq = pl[4], heads = pl[5], hs = pl[6];
        if (seq < 1 || heads < 1 || hs < 2 || (hs & 1) || seq * hs > (1ll << 30)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        long h;
        ERRCHK(m_rope.create(&h));
        RopeD* r = m_rope.get(h);
        r->seq = (int)seq; r->heads = (int)heads; r->hs = (int)hs;
        const int half = (int)hs / 2;
        // the reference's host tables for T = double (rope.cu:535-553): the power and the cosines are single-precision
        // library calls on values held in double
        std::vector<double> freq(half), hc((size_t)seq * half), hsn((size_t)seq * half);
        for (int i = 0, j = 0; i < (int)hs; i += 2, j++) {
            double power = (double)(i / (double)hs);
            power = (double)powf((float)pf[0], (float)power);
            freq[j] = 1.0 / power;
        }
        for (long long pos = 0; pos < seq; pos++)
            for (int i = 0; i < half; i++) {
                const double fpos = freq[i] * (double)pos;
                hc[(size_t)pos * half + i] = (double)cosf((float)fpos);
                hsn[(size_t)pos * half + i] = (double)sinf((float)fpos);
            }
        long e = 0;
        hipError_t he = hipMalloc((void**)&r->dcos, hc.size() * 8);
        if (he == hipSuccess) he = hipMalloc((void**)&r->dsin, hsn.size() * 8);
        if (he == hipSuccess) he = hipMemcpyAsync(r->dcos, hc.data(), hc.size() * 8, hipMemcpyHostToDevice, s);
        if (he == hipSuccess) he = hipMemcpyAsync(r->dsin, hsn.data(), hsn.size() * 8, hipMemcpyHostToDevice, s);
        if (he == hipSuccess) he = hipStreamSynchronize(s);
        if (he != hipSuccess) e = (long)he;
        if (e) { m_rope.free(h); return e; }
        r->set = true;
        return set_out_d((double)h, ppOut, plOut);
    }
    case MCH_FN_FREE_ROPE:
        NEED_F(1, 1);
        HIPCHK(hipStreamSynchronize(s));
        return m_rope.free((long)pf[0]);
    case MCH_FN_ROPE_FWD: {
        // l{hRope,n,hX,hY[,freqOffset]}
        NEED_L(4, 5);
        RopeD* r = m_rope.get((long)pl[0]);
        if (!r || !r->set) return MCH_ERROR_ROPE_NOT_INITIALIZED;
        const long long n = pl[1];
        long long off = ll > 4 ? pl[4] : -1;
        if (off < 0) off = 0;   // offsets <= 0 mean "no shift" (rope.cu:808-814)
        MemD *X, *Y;
        ERRCHK(mem((long)pl[2], &X));
        ERRCHK(mem((long)pl[3], &Y));
        if (n < 0 || (n & 1)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        const long long half = r->hs / 2, full = half * r->heads, wrap = (long long)r->seq * full, pairs = n / 2;
        const long long maxbase = (pairs < wrap ? pairs : wrap) - 1;
        if (pairs > 0 && (maxbase / full) * half + (half - 1) + off >= (long long)r->seq * half) {
            last_detail = "rope table offset reaches past the last position of the table";
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        if (pairs) hipLaunchKernelGGL(d_rope_kernel, grid_of((size_t)pairs), 256, 0, s, (size_t)pairs, (const double*)X->ptr, Y->ptr,
                                      (const double*)r->dcos, (const double*)r->dsin, (size_t)full, (size_t)wrap, (int)half, (int)off, 1.0);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_ROPE_BWD: {
        // l{hRope,n,hXdata,hYdiff,hXdiff}: the rotation by the opposite angle, never shifted (rope.cu:832-864)
        NEED_L(5, 5);
        RopeD* r = m_rope.get((long)pl[0]);
        if (!r || !r->set) return MCH_ERROR_ROPE_NOT_INITIALIZED;
        const long long n = pl[1];
        MemD *dY, *dX;
        ERRCHK(mem((long)pl[3], &dY));
        ERRCHK(mem((long)pl[4], &dX));
        if (n < 0 || (n & 1)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(dY, 0, n);
        RANGE(dX, 0, n);
        const long long half = r->hs / 2, full = half * r->heads, wrap = (long long)r->seq * full, pairs = n / 2;
        if (pairs) hipLaunchKernelGGL(d_rope_kernel, grid_of((size_t)pairs), 256, 0, s, (size_t)pairs, (const double*)dY->ptr, dX->ptr,
                                      (const double*)r->dcos, (const double*)r->dsin, (size_t)full, (size_t)wrap, (int)half, 0, -1.0);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_LINEAR_FWD: {
        // l{M, N, K, hX, hW, hBias(0 = none), hY}: Y = X W^T + bias
        NEED_L(7, 7);
        const long long M = pl[0], N = pl[1], K = pl[2];
        if (M < 1 || N < 1 || K < 1 || M > INT_MAX || N > INT_MAX || K > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *X, *W, *Bi = nullptr, *Y;
        ERRCHK(mem((long)pl[3], &X));
        ERRCHK(mem((long)pl[4], &W));
        if (pl[5]) ERRCHK(mem((long)pl[5], &Bi));
        ERRCHK(mem((long)pl[6], &Y));
        RANGE(X, 0, M * K);
        RANGE(W, 0, N * K);
        if (Bi) RANGE(Bi, 0, N);
        RANGE(Y, 0, M * N);
        hipLaunchKernelGGL(d_gemm_kernel, dim3((unsigned)((N + 15) / 16), (unsigned)((M + 15) / 16), 1), 256, 0, s, (int)M, (int)N, (int)K, 1.0,
                           (const double*)X->ptr, K, 1ll, (const double*)W->ptr, 1ll, K, 0.0, Y->ptr, N, 1ll, 0ll, 0ll, 0ll);
        LAUNCHED();
        if (Bi) {
            hipLaunchKernelGGL(d_add_bias_rows_kernel, grid_of((size_t)(M * N)), 256, 0, s, (size_t)(M * N), (int)N, (const double*)Bi->ptr, Y->ptr);
            LAUNCHED();
        }
        return 0;
    }
    case MCH_FN_QKV_PROJ_HEADS: {
        // l{batch, T, heads, hs, hX, hW, hBias(0 = none), hQ, hK, hV [, hRope]}
        NEED_L(10, 11);
        const long long B = pl[0], T = pl[1], H = pl[2], hs = pl[3];
        if (B < 1 || T < 1 || H < 1 || hs < 1 || B * T > INT_MAX || 3 * H * hs > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const long long C = H * hs, M = B * T;
        MemD *X, *W, *Bi = nullptr, *Q, *K, *V;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &W));
        if (pl[6]) ERRCHK(mem((long)pl[6], &Bi));
        ERRCHK(mem((long)pl[7], &Q));
        ERRCHK(mem((long)pl[8], &K));
        ERRCHK(mem((long)pl[9], &V));
        RANGE(X, 0, M * C);
        RANGE(W, 0, 3 * C * C);
        if (Bi) RANGE(Bi, 0, 3 * C);
        RANGE(Q, 0, M * C);
        RANGE(K, 0, M * C);
        RANGE(V, 0, M * C);
        RopeD* r = nullptr;
        if (ll > 10 && pl[10]) {
            r = m_rope.get((long)pl[10]);
            if (!r || !r->set) return MCH_ERROR_ROPE_NOT_INITIALIZED;
            if (r->heads != H || r->hs != hs) {
                last_detail = "the rope handle was created for other heads or another head size";
                return MCH_ERROR_PARAM_OUT_OF_RANGE;
            }
        }
        if (hs & 1) {
            last_detail = "the double form of the fused QKV projection takes even head sizes";
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        double* tmp;
        ERRCHK(workspace((size_t)(M * 3 * C), &tmp));
        hipLaunchKernelGGL(d_gemm_kernel, dim3((unsigned)((3 * C + 15) / 16), (unsigned)((M + 15) / 16), 1), 256, 0, s, (int)M, (int)(3 * C), (int)C,
                           1.0, (const double*)X->ptr, C, 1ll, (const double*)W->ptr, 1ll, C, 0.0, tmp, 3 * C, 1ll, 0ll, 0ll, 0ll);
        LAUNCHED();
        const size_t pairs = (size_t)(M * 3 * C) / 2;
        hipLaunchKernelGGL(d_qkv_split_kernel, grid_of(pairs), 256, 0, s, pairs, (const double*)tmp, Bi ? (const double*)Bi->ptr : nullptr,
                           Q->ptr, K->ptr, V->ptr, (int)T, (int)H, (int)hs, r ? (const double*)r->dcos : nullptr,
                           r ? (const double*)r->dsin : nullptr, r ? r->seq : 1);
        LAUNCHED();
        return 0;
    }
    case MCH_FN_ATTN_DECODE_FWD: {
        // f{scale (0 = 1/sqrt(hs))}, l{batch, heads, kvHeads, hs, len, hQ, hKcache, hVcache, hY, strideKvBatch, strideKvHead,
        //   strideKvPos [, hRope, hKnew, hVnew]}
        NEED_F(1, 1);
        NEED_L(12, 15);
        if (ll != 12 && ll != 15) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const long long B = pl[0], H = pl[1], KVH = pl[2], hs = pl[3], len = pl[4];
        const long long sB = pl[9], sH = pl[10], sT = pl[11];
        if (B < 1 || H < 1 || KVH < 1 || hs < 1 || len < 1 || H % KVH || sB < 0 || sH < 0 || sT < 1 || (hs & 1) || B * H > INT_MAX)
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemD *Q, *KC, *VC, *Y;
        ERRCHK(mem((long)pl[5], &Q));
        ERRCHK(mem((long)pl[6], &KC));
        ERRCHK(mem((long)pl[7], &VC));
        ERRCHK(mem((long)pl[8], &Y));
        RANGE(Q, 0, B * H * hs);
        RANGE(Y, 0, B * H * hs);
        const long long need = (B - 1) * sB + (KVH - 1) * sH + (len - 1) * sT + hs;
        RANGE(KC, 0, need);
        RANGE(VC, 0, need);
        const double scale = pf[0] != 0.0 ? pf[0] : 1.0 / sqrt((double)hs);
        const size_t lds = (size_t)(len + hs) * sizeof(double);
        if (lds > 60000) {
            last_detail = "the double form of the decode attention keeps a row of probabilities in LDS: up to about 7000 positions";
            return MCH_ERROR_NOT_IMPLEMENTED;
        }
        if (ll == 15 && (pl[12] || pl[13] || pl[14])) {
            RopeD* rp = pl[12] ? m_rope.get((long)pl[12]) : nullptr;
            if (pl[12] && (!rp || !rp->set)) return MCH_ERROR_ROPE_NOT_INITIALIZED;
            if (rp && (rp->hs != hs || len > rp->seq)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
            MemD *KN, *VN;
            ERRCHK(mem((long)pl[13], &KN));
            ERRCHK(mem((long)pl[14], &VN));
            RANGE(KN, 0, B * KVH * hs);
            RANGE(VN, 0, B * KVH * hs);
            const size_t items = (size_t)(B * H * (hs / 2) + B * KVH * (hs / 2) + B * KVH * hs);
            hipLaunchKernelGGL(d_rope_append_kernel, grid_of(items), 256, 0, s, Q->ptr, KN->ptr, (const double*)VN->ptr, KC->ptr, VC->ptr, (int)B,
                               (int)H, (int)KVH, (int)hs, (int)len - 1, sB, sH, sT, rp ? (const double*)rp->dcos : nullptr,
                               rp ? (const double*)rp->dsin : nullptr);
            LAUNCHED();
        }
        hipLaunchKernelGGL(d_attn_decode_kernel, (unsigned)(B * H), 256, lds, s, (const double*)Q->ptr, (const double*)KC->ptr,
                           (const double*)VC->ptr, Y->ptr, (int)H, (int)(H / KVH), (int)hs, (int)len, sB, sH, sT, scale);
        LAUNCHED();
        return 0;
    }
    default:
        break;
    }
    char buf[160];
    snprintf(buf, sizeof(buf), "function id %ld is not built for the double base type (the attention path's ids are)", fn);
    last_detail = buf;
    return MCH_ERROR_NOT_IMPLEMENTED;
}

// ---- kernel table and entry points ----------------------------------------------------------------------------------
static const int MAX_KERNELS_D = 2048;   // CudaDnnDLL/main.h:21
static KernelD* g_kernelsD[MAX_KERNELS_D];
static std::mutex g_tableLockD;

static KernelD* kernel_d(long idx)
{
    if (idx <= 0 || idx >= MAX_KERNELS_D) return nullptr;
    std::lock_guard<std::mutex> g(g_tableLockD);
    return g_kernelsD[idx];
}
static void put_error_d(KernelD* k, long e, MCH_TCHAR* szErr, long max)
{
    if (!szErr || max <= 0) return;
    char buf[512];
    if (k && !k->last_detail.empty()) snprintf(buf, sizeof(buf), "%s (%ld)", k->last_detail.c_str(), e);
    else if (e > 0 && e < 2000) snprintf(buf, sizeof(buf), "HIP runtime error: %s (%ld)", hipGetErrorString((hipError_t)e), e);
    else snprintf(buf, sizeof(buf), "error %ld in the double base type's call", e);
    utf8_to_utf16(buf, szErr, max);
}

static long invoke_d(long kIdx, long fn, double* pf, long lf, MCH_LONGLONG* pl, long ll, double** ppOut, MCH_LONG* plOut, MCH_TCHAR* szErr,
                     long errMax)
{
    if (szErr && errMax > 0) szErr[0] = 0;
    if (kIdx < 0 || kIdx >= MAX_KERNELS_D) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    long e = 0;
    KernelD* k = nullptr;
    switch (fn) {
    case MCH_DLL_INITIALIZE: {
        // creates a kernel, returns its index in (*ppOutput)[0] (CudaDnnDLL.cpp:154-176)
        if (!ppOut || !*ppOut || !plOut) return MCH_ERROR_PARAM_NULL;
        k = new KernelD();
        e = k->initialize(pf, lf);
        if (e) { put_error_d(k, e, szErr, errMax); delete k; return e; }
        long slot = -1;
        {
            std::lock_guard<std::mutex> g(g_tableLockD);
            for (int i = 1; i < MAX_KERNELS_D; i++)
                if (!g_kernelsD[i]) { g_kernelsD[i] = k; slot = i; break; }
        }
        if (slot < 0) { delete k; e = MCH_ERROR_MEMORY_OUT; put_error_d(nullptr, e, szErr, errMax); return e; }
        (*ppOut)[0] = (double)slot;
        *plOut = 1;
        return 0;
    }
    case MCH_DLL_CLEANUP: {
        std::lock_guard<std::mutex> g(g_tableLockD);
        k = g_kernelsD[kIdx];
        g_kernelsD[kIdx] = nullptr;
        delete k;
        return 0;
    }
    case MCH_DLL_FREEMEM:
        if (!(k = kernel_d(kIdx))) { e = MCH_ERROR_PARAM_NULL; put_error_d(nullptr, e, szErr, errMax); return e; }
        e = k->free_host(pf);
        if (e) put_error_d(k, e, szErr, errMax);
        return e;
    default:
        break;
    }
    if (!(k = kernel_d(kIdx))) { e = MCH_ERROR_PARAM_NULL; put_error_d(nullptr, e, szErr, errMax); return e; }
    e = k->run(fn, pf, lf, pl, ll, ppOut, plOut);
    if (e) put_error_d(k, e, szErr, errMax);
    return e;
}

}  // namespace mch

using namespace mch;

extern "C" {

MCH_LONG DLL_InvokeDouble(MCH_LONG k, MCH_LONG fn, double* pIn, MCH_LONG lIn, double** ppOut, MCH_LONG* plOut, MCH_TCHAR* szErr,
                          MCH_LONG errMax)
{
    // the legacy entry point forwards no integer array (CudaDnnDLL.cpp:303)
    return (MCH_LONG)invoke_d(k, fn, pIn, lIn, nullptr, 0, ppOut, plOut, szErr, errMax);
}

MCH_LONG DLL_InvokeDoubleEx2(MCH_LONG k, MCH_LONG fn, double* pIn, MCH_LONG lIn, MCH_LONGLONG* plIn, MCH_LONG llIn, double** ppOut,
                             MCH_LONG* plOut, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return (MCH_LONG)invoke_d(k, fn, pIn, lIn, plIn, llIn, ppOut, plOut, szErr, errMax);
}

MCH_LONG Internal_GetPointerDouble(int32_t ht, MCH_LONG kIdx, MCH_LONG h, void** pp)
{
    if (ht != 0 || !pp) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    KernelD* k = kernel_d(kIdx);
    if (!k) return MCH_ERROR_PARAM_NULL;
    return (MCH_LONG)k->get_pointer(h, pp);
}

}  // extern "C"
