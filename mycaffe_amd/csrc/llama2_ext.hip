// libmycaffe_hip_llama2.so: the llama2 inference extension for gfx950.
//
// Drop-in for the reference's CudaExtension.llm32.llama2 DLL: same three exports
// and function ids (CudaExtension.llm32.cpp:20-26, 67-268), loaded by the parent
// library through CREATE_EXTENSION.  The forward pass computes what
// TransformerGpu::forward / TransformerCpu::forward compute
// (llama2_gpu.cpp:32-111, llama2_cpu.cpp:264-386) but is organised for MI355X:
//
//  * weights are repacked once at load (wq|wk|wv and w1|w3 row-concatenated per
//    layer, optionally stored as bf16) so one token needs 7 launches per layer;
//  * RMSNorm is fused into the prologue of the QKV and W1/W3 mat-vecs, SwiGLU and
//    the residual adds into their epilogues;
//  * position, current token and sampled token live in device memory, so a whole
//    greedy generation runs without any host round trip, and one decode step is
//    captured into a HIP graph that is replayed per token;
//  * attention over the KV cache is the split-K decode kernel of the parent.
//
// KV cache layout: [layer][batch][seq_len][kv_dim] fp32, position-major inside a
// sequence as in the reference (llama2_gpu.cpp:67-71).
#include <dlfcn.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <algorithm>
#include <type_traits>
#include <vector>

#include "../../include/mycaffe_hip_abi.h"
#include "bpe_tokenizer.h"
#include "kernels.h"
#include "lane_ops.h"

namespace mch {

#define HIPCHK(x) do { hipError_t _e = (x); if (_e != hipSuccess) return (long)_e; } while (0)

struct Config { int dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len; };

// ---- device-side generation state ---------------------------------------------------
struct GenState {
    int pos;        // position of the token being processed
    int n_prompt;   // prompt length (same for all sequences of a batch)
    int len;        // pos + 1, read by the attention kernel
    int pad;
};

template <typename T> __device__ inline float wld(const T* p, size_t i);
template <> __device__ inline float wld<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ inline float wld<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }

// sum over the 64 lanes of a wavefront, the result in every lane
__device__ inline float wsum(float v) { return group_sum<64>(v); }

// x[b,:] = emb[token,:] where token is the forced prompt id while pos < n_prompt and
// the previously sampled id afterwards (generate loop, llm.cpp:208-228)
template <typename T>
__global__ void embed_step_kernel(const GenState* st, const int* prompt, int promptStride, const int* next, const T* emb,
                                  float* x, int dim, int* cur)
{
    const int b = blockIdx.x;
    const int pos = st->pos;
    const int tok = pos < st->n_prompt ? prompt[(size_t)b * promptStride + pos] : next[b];
    if (threadIdx.x == 0) cur[b] = tok;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) x[(size_t)b * dim + i] = wld(emb, (size_t)tok * dim + i);
}

// 4 weight values of one row against 4 activations
template <typename T> struct Row4;
template <> struct Row4<float> {
    __device__ static inline float4 load(const float* p) { return *(const float4*)p; }
};
template <> struct Row4<bf16_t> {
    __device__ static inline float4 load(const bf16_t* p)
    {
        uint2 u = *(const uint2*)p;
        return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                           __uint_as_float(u.y & 0xffff0000u));
    }
};

template <typename T> struct Row8;
template <> struct Row8<float> {
    __device__ static inline void load(const float* p, float* w)
    {
        const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
        w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
    }
};
template <> struct Row8<bf16_t> {
    __device__ static inline void load(const bf16_t* p, float* w)
    {
        const uint4 u = *(const uint4*)p;
        const uint32_t v[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[2 * i] = __uint_as_float(v[i] << 16);
            w[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
        }
    }
};

// The 8 of a 32-column slab's values that lane group kk (0..3) of the matrix-core mat-vec contracts.  Which columns a
// group takes is free as long as both operands agree, so it is chosen for the loads: with fp32 weights a group takes
// columns 4 kk .. 4 kk + 3 and 16 + 4 kk .. + 3, so that the four groups of a row read 64 contiguous bytes per load
// instruction; with bf16 weights a group's 16-byte load holds columns 8 kk .. 8 kk + 7 and x follows that.
template <typename T> struct Slab8;
template <> struct Slab8<float> {
    __device__ static inline void w(const float* slab, int kk, float* o) { x(slab, kk, o); }
    __device__ static inline void x(const float* slab, int kk, float* o)
    {
        const float4 a = *(const float4*)(slab + 4 * kk), b = *(const float4*)(slab + 16 + 4 * kk);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
};
template <> struct Slab8<bf16_t> {
    __device__ static inline void w(const bf16_t* slab, int kk, float* o) { Row8<bf16_t>::load(slab + 8 * kk, o); }
    __device__ static inline void x(const float* slab, int kk, float* o) { Row8<float>::load(slab + 8 * kk, o); }
};

// Mat-vec family for one token per sequence.  One wavefront owns ROWS output rows
// of W (n columns, n % 4 == 0) and walks them with 128-bit (fp32) / 64-bit (bf16)
// loads; the activation chunk a lane needs is the same for every row, so it is
// loaded (and, when NORM, RMS-normalised) once per batch entry.
//   MODE 0: y[b,r]  = W[r,:] . xn[b,:]
//   MODE 1: y[b,r] += W[r,:] . x[b,:]                      (residual epilogue)
//   MODE 2: y[b,r]  = silu(W[r,:] . xn) * (W[r+half,:] . xn)   (SwiGLU epilogue, half = rows)
// NORM: xn = g * x / sqrt(mean(x^2) + 1e-5), recomputed per wavefront from the
// chunks it already holds (x is L2 resident; it saves a launch and a barrier).
// WIDE (bf16 weights, n % 8 == 0): a lane takes 8 consecutive weights per load (16 bytes, two of the CH float4 slots),
// so 16-bit weights move in as few load instructions per byte as fp32 ones.
template <bool WIDE> __device__ __forceinline__ int matvec_col(int c, int lane)
{
    return WIDE ? ((c >> 1) * 64 + lane) * 8 + (c & 1) * 4 : (c * 64 + lane) * 4;
}

template <typename T, int MODE, bool NORM, int CH, int ROWS, bool WIDE = false>
__global__ __launch_bounds__(256) void matvec_kernel(const T* __restrict__ W, const float* __restrict__ x,
                                                     const float* __restrict__ g, float* __restrict__ y, int rows, int n,
                                                     int B, int ldy)
{
    static_assert(!WIDE || (sizeof(T) == 2 && CH % 2 == 0), "wide loads are for 16-bit weights, two slots per load");
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int r0 = wave * ROWS;
    if (r0 >= rows) return;
    // Every load below is unconditional (columns past the end come from a clamped address and meet a zeroed activation):
    // loads under a branch would make the compiler wait for ALL outstanding loads at the first use of any of them.
    // The first sequence's activations (and the norm weights) are requested before the weights: loads return in order,
    // so the sum of squares, its reduction and the square root run while the weights are still on their way.
    constexpr int LW = WIDE ? 8 : 4;   // columns per load
    float4 xv[CH], gq[NORM ? CH : 1];
    float prev[ROWS];
    auto request_x = [&](int b) {
        const float* xb = x + (size_t)b * n;
        // the residual epilogue's old values are requested now, not once the row sums are known
#pragma unroll
        for (int rr = 0; rr < ROWS; rr++) prev[rr] = (MODE == 1 && lane == 0) ? y[(size_t)b * ldy + min(r0 + rr, rows - 1)] : 0.f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int jc = min(matvec_col<WIDE>(c, lane), n - 4);
            xv[c] = *(const float4*)(xb + jc);
            if (NORM) gq[c] = *(const float4*)(g + jc);
        }
    };
    request_x(0);
    // weight chunks of this wavefront's rows stay in registers across the batch loop
    float4 w[(MODE == 2 ? 2 : 1) * ROWS][CH];
#pragma unroll
    for (int rr = 0; rr < ROWS; rr++) {
        const int r = min(r0 + rr, rows - 1);
        if (WIDE) {
#pragma unroll
            for (int c = 0; c < CH; c += 2) {
                const int jc = min(matvec_col<WIDE>(c, lane), n - LW);
                float lo[8], hi[8];
                Row8<T>::load(W + (size_t)r * n + jc, lo);
                w[rr][c] = make_float4(lo[0], lo[1], lo[2], lo[3]);
                w[rr][c + 1] = make_float4(lo[4], lo[5], lo[6], lo[7]);
                if (MODE == 2) {
                    Row8<T>::load(W + (size_t)(r + rows) * n + jc, hi);
                    w[ROWS + rr][c] = make_float4(hi[0], hi[1], hi[2], hi[3]);
                    w[ROWS + rr][c + 1] = make_float4(hi[4], hi[5], hi[6], hi[7]);
                }
            }
        } else {
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int jc = min(matvec_col<WIDE>(c, lane), n - 4);
                w[rr][c] = Row4<T>::load(W + (size_t)r * n + jc);
                if (MODE == 2) w[ROWS + rr][c] = Row4<T>::load(W + (size_t)(r + rows) * n + jc);
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);   // every request above is issued before any arithmetic below
    auto sequence = [&](int b, auto first) {
        if (!decltype(first)::value) request_x(b);
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const float keep = matvec_col<WIDE>(c, lane) < n ? 1.f : 0.f;
            xv[c].x *= keep; xv[c].y *= keep; xv[c].z *= keep; xv[c].w *= keep;
        }
        if (NORM) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < CH; c++) ss += xv[c].x * xv[c].x + xv[c].y * xv[c].y + xv[c].z * xv[c].z + xv[c].w * xv[c].w;
            ss = wsum(ss);
            const float inv = 1.0f / sqrtf(ss / n + 1e-5f);
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const float4 gv = gq[c];
                xv[c].x = gv.x * (inv * xv[c].x);
                xv[c].y = gv.y * (inv * xv[c].y);
                xv[c].z = gv.z * (inv * xv[c].z);
                xv[c].w = gv.w * (inv * xv[c].w);
            }
        }
#pragma unroll
        for (int rr = 0; rr < ROWS; rr++) {
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int c = 0; c < CH; c++) {
                a0 += w[rr][c].x * xv[c].x + w[rr][c].y * xv[c].y + w[rr][c].z * xv[c].z + w[rr][c].w * xv[c].w;
                if (MODE == 2)
                    a1 += w[ROWS + rr][c].x * xv[c].x + w[ROWS + rr][c].y * xv[c].y + w[ROWS + rr][c].z * xv[c].z +
                          w[ROWS + rr][c].w * xv[c].w;
            }
            a0 = wsum(a0);
            if (MODE == 2) a1 = wsum(a1);
            const int r = r0 + rr;
            if (lane == 0 && r < rows) {
                float* out = y + (size_t)b * ldy + r;
                if (MODE == 0) *out = a0;
                else if (MODE == 1) *out = prev[rr] + a0;
                else *out = a0 * (1.0f / (1.0f + expf(-a0))) * a1;
            }
        }
    };
    // the first sequence in straight-line code, so that the wait before the norm counts only the loads it needs
    sequence(0, std::true_type());
    for (int b = 1; b < B; b++) sequence(b, std::false_type());
}

// Output projection of a decode step whose attention left its split partials unmerged (batch 1):
//   y[r] += W[r,:] . att,   att[h*hs + d] = sum_s acc[s][h][d] e^(m[s][h] - M[h]) / sum_s l[s][h] e^(m[s][h] - M[h])
// over the nAct = ceil(*dlen / rowsPerSplit) splits that hold rows.  Thread t of a workgroup merges columns 4t .. 4t + 3
// (one head: hs % 4 == 0) with all NS splits' loads in flight, the merged vector meets the wavefronts in LDS, and each
// wavefront then finishes its row of W as matvec_kernel does.  This replaces the attention kernel's own merge - partial
// stores acknowledged, a ticket, the partials read back: three trips to memory in a row - by loads that travel together
// with the weights.  Splits beyond nAct hold stale partials: they are masked, not multiplied away.
template <typename T, int CH, bool WIDE, int NS>
__global__ __launch_bounds__(256) void matvec_merge_kernel(const T* __restrict__ W, const float* __restrict__ partAcc,
                                                           const float* __restrict__ partML, const int* __restrict__ dlen,
                                                           int splits, int rowsPerSplit, int H, int hs, float* __restrict__ y, int rows,
                                                           int n)
{
    __shared__ float4 xs[256];
    const int tid = threadIdx.x, lane = tid & 63;
    const int r = min(blockIdx.x * 4 + (tid >> 6), rows - 1);   // a wavefront past the end repeats the last row and stores nothing
    const bool store = blockIdx.x * 4 + (tid >> 6) < rows && lane == 0;
    constexpr int LW = WIDE ? 8 : 4;
    // partials first: the longer chain (merge, LDS, barrier) hangs on them
    const int col = min(tid * 4, n - 4);
    const int h = col / hs;
    float4 pa[NS];
    float2 pm[NS];
#pragma unroll
    for (int k = 0; k < NS; k++) {
        const int kc = min(k, splits - 1);
        pa[k] = *(const float4*)(partAcc + (size_t)kc * n + col);
        pm[k] = *(const float2*)(partML + ((size_t)kc * H + h) * 2);
    }
    const float prev = y[r];
    float4 w[CH];
    if (WIDE) {
#pragma unroll
        for (int c = 0; c < CH; c += 2) {
            float lo[8];
            Row8<T>::load(W + (size_t)r * n + min(matvec_col<WIDE>(c, lane), n - LW), lo);
            w[c] = make_float4(lo[0], lo[1], lo[2], lo[3]);
            w[c + 1] = make_float4(lo[4], lo[5], lo[6], lo[7]);
        }
    } else {
#pragma unroll
        for (int c = 0; c < CH; c++) w[c] = Row4<T>::load(W + (size_t)r * n + min(matvec_col<WIDE>(c, lane), n - 4));
    }
    __builtin_amdgcn_sched_barrier(0);   // every request above is issued before the length is asked for
    const int len = *dlen;
    const int nAct = (len + rowsPerSplit - 1) / rowsPerSplit;
    float M = -INFINITY;
#pragma unroll
    for (int k = 0; k < NS; k++) {
        if (k >= nAct) pm[k].x = -INFINITY;
        M = fmaxf(M, pm[k].x);
    }
    float L = 0.f;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int k = 0; k < NS; k++) {
        const bool on = k < nAct;
        const float e = on ? __expf(pm[k].x - M) : 0.f;
        L += on ? pm[k].y * e : 0.f;
        a.x += on ? pa[k].x * e : 0.f;
        a.y += on ? pa[k].y * e : 0.f;
        a.z += on ? pa[k].z * e : 0.f;
        a.w += on ? pa[k].w * e : 0.f;
    }
    const float inv = 1.0f / L;
    xs[tid] = make_float4(a.x * inv, a.y * inv, a.z * inv, a.w * inv);
    __syncthreads();
    float a0 = 0.f;
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int j = matvec_col<WIDE>(c, lane);
        float4 xv = xs[min(j, n - 4) >> 2];
        const float keep = j < n ? 1.f : 0.f;
        a0 += keep * (w[c].x * xv.x + w[c].y * xv.y + w[c].z * xv.z + w[c].w * xv.w);
    }
    a0 = wsum(a0);
    if (store) y[r] = prev + a0;
}

// The same family for rows too long to hold in registers (n > 4096): one wavefront per row walks K in slabs of
// 64 x 4 columns, four slabs in flight.  With NORM the sum of squares of x (L2 resident) is taken in a first walk.
template <typename T, int MODE, bool NORM>
__global__ __launch_bounds__(256) void matvec_loop_kernel(const T* __restrict__ W, const float* __restrict__ x,
                                                          const float* __restrict__ g, float* __restrict__ y, int rows, int n,
                                                          int B, int ldy)
{
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const T* w0 = W + (size_t)r * n;
    const T* w1 = W + (size_t)(r + rows) * n;   // only read when MODE == 2
    constexpr int U = 4;
    for (int b = 0; b < B; b++) {
        const float* xb = x + (size_t)b * n;
        const float prev = (MODE == 1 && lane == 0) ? y[(size_t)b * ldy + r] : 0.f;
        float inv = 1.f;
        if (NORM) {
            float ss = 0.f;
            for (int j = lane * 4; j < n; j += 256) {
                const float4 v = *(const float4*)(xb + j);
                ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
            }
            ss = wsum(ss);
            inv = 1.0f / sqrtf(ss / n + 1e-5f);
        }
        float a0 = 0.f, a1 = 0.f;
        for (int j0 = lane * 4; j0 < n; j0 += 256 * U) {
            float4 wv[U], w2v[MODE == 2 ? U : 1], xv[U], gv[NORM ? U : 1];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int j = j0 + u * 256;
                const bool in = j < n;
                wv[u] = in ? Row4<T>::load(w0 + j) : make_float4(0.f, 0.f, 0.f, 0.f);
                if (MODE == 2) w2v[MODE == 2 ? u : 0] = in ? Row4<T>::load(w1 + j) : make_float4(0.f, 0.f, 0.f, 0.f);
                xv[u] = in ? *(const float4*)(xb + j) : make_float4(0.f, 0.f, 0.f, 0.f);
                if (NORM) gv[NORM ? u : 0] = in ? *(const float4*)(g + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                float4 v = xv[u];
                if (NORM) {
                    const float4 gq = gv[NORM ? u : 0];
                    v.x = gq.x * (inv * v.x); v.y = gq.y * (inv * v.y); v.z = gq.z * (inv * v.z); v.w = gq.w * (inv * v.w);
                }
                a0 += wv[u].x * v.x + wv[u].y * v.y + wv[u].z * v.z + wv[u].w * v.w;
                if (MODE == 2) {
                    const float4 q = w2v[MODE == 2 ? u : 0];
                    a1 += q.x * v.x + q.y * v.y + q.z * v.z + q.w * v.w;
                }
            }
        }
        a0 = wsum(a0);
        if (MODE == 2) a1 = wsum(a1);
        if (lane == 0) {
            float* out = y + (size_t)b * ldy + r;
            if (MODE == 0) *out = a0;
            else if (MODE == 1) *out = prev + a0;
            else *out = a0 * (1.0f / (1.0f + expf(-a0))) * a1;
        }
    }
}

// Tile-packed copy of a weight matrix for matvec_mfma_kernel.  In the row-major matrix one load instruction of that kernel
// touches 16 rows (64 bytes of each): sixteen half-used cache lines.  The packed copy stores, for every tile of 16 rows
// and every slab of 32 columns, the 2 KB (fp32) or 1 KB (bf16) of the slab in the order the lanes read it, so that an
// instruction reads 1 KB of consecutive bytes: fp32 [tile][slab][half][lane][4], lane (i = row, kk) holding columns
// 16 half + 4 kk .. + 3; bf16 [tile][slab][lane][8], columns 8 kk .. 8 kk + 7.  Rows past the end are zero.
template <typename T> struct PackedSlab;
template <> struct PackedSlab<float> {
    __device__ static inline void w(const float* slab, int lane, float* o)
    {
        const float4 a = *(const float4*)(slab + lane * 4), b = *(const float4*)(slab + 256 + lane * 4);
        o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
    }
};
template <> struct PackedSlab<bf16_t> {
    __device__ static inline void w(const bf16_t* slab, int lane, float* o) { Row8<bf16_t>::load(slab + lane * 8, o); }
};
template <typename T>
__global__ void pack_tiles_kernel(const T* __restrict__ W, T* __restrict__ P, int rows, int n)
{
    constexpr int E = 16 / sizeof(T);                 // elements per 16-byte piece
    constexpr int PPS = 512 / E;                      // pieces per slab
    const int nit = n >> 5, tiles = (rows + 15) >> 4;
    const size_t total = (size_t)tiles * nit * PPS;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const int piece = (int)(idx % PPS);
        const size_t ts = idx / PPS;
        const int slab = (int)(ts % nit), tile = (int)(ts / nit);
        const int lane = piece & 63, half = piece >> 6;       // bf16: one piece per lane, half stays 0
        const int i = lane & 15, kk = lane >> 4;
        const int r = tile * 16 + i;
        const int c = slab * 32 + (sizeof(T) == 4 ? 16 * half + 4 * kk : 8 * kk);
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (r < rows) v = *(const uint4*)(W + (size_t)r * n + c);
        *(uint4*)(P + idx * E) = v;
    }
}

// Batched form of the mat-vec family (2 or more sequences): the same three epilogues, computed on the matrix
// cores so that a decode step stays bound by the weight stream instead of by vector ALU work.  A workgroup owns
// 16 rows of W; its wavefronts take the 32-column slabs of K round robin.  Per slab a lane (row i = lane % 16,
// group kk = lane / 16) loads W[i][k0 + 8 kk .. + 7] and, as the other operand, x[j = lane % 16][k0 + 8 kk .. + 7],
// and issues eight v_mfma_f32_16x16x4_f32, step e contracting column k0 + 8 kk + e of the four groups: the slot to
// column assignment only has to agree between the two operands.  Weights stored as bf16 are widened in
// registers; activations and accumulation stay fp32.  NORM: the RMS factor of every sequence is a per-column
// scale of the result, so the sum of squares is gathered from the x values that pass through anyway and g is
// folded into x.  Partial tiles of the wavefronts meet in LDS; wavefront 0 finishes.
typedef float floatx4v __attribute__((ext_vector_type(4)));

template <typename T, int MODE, bool NORM, int G = 1, int NS = 8, bool PACKED = false>
__global__ __launch_bounds__(NS * 64) void matvec_mfma_kernel(const T* __restrict__ W, const float* __restrict__ x,
                                                          const float* __restrict__ g, float* __restrict__ y, int rows, int n,
                                                          int B, int ldy, int nGroups)
{
    // Workgroups go to the chip's 8 dies round robin by their index, and each die has its own L2: the nGroups
    // workgroups that walk the same 16 rows of W (one per group of 16 G sequences or prompt rows) are given indices
    // that are equal modulo 8, so a slab of weights is fetched into one L2 instead of all eight.
    const int die = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int r0 = ((slot / nGroups) * 8 + die) * 16;
    const int b0 = (slot % nGroups) * 16 * G;
    if (r0 >= rows) return;   // the grid is padded to a multiple of 8 row tiles
    // G groups of 16 sequences (or prompt rows) per pass: a slab of weights is loaded once and multiplied into all of
    // them, so up to 128 rows of x share one walk over W (the batched prompt pass of a single sequence)
    __shared__ __attribute__((aligned(16))) float part[NS][(MODE == 2 ? 2 : 1) * 256];
    __shared__ float sspart[NS][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;   // NS wavefronts: a compile-time count keeps the final sums unrolled
    const int i = lane & 15, kk = lane >> 4;
    const int nit = n >> 5;
    // PACKED: W is the tile-packed copy (pack_tiles_kernel); the second matrix of MODE 2 follows the first one's tiles
    const T* wr = PACKED ? W + (size_t)(r0 >> 4) * nit * 512 : W + (size_t)min(r0 + i, rows - 1) * n;
    const T* wr2 = PACKED ? wr + (size_t)((rows + 15) >> 4) * nit * 512 : wr + (size_t)rows * n;
    bool jv[G];                                 // this lane's batch column exists
    const float* xr[G];
#pragma unroll
    for (int q = 0; q < G; q++) {
        jv[q] = b0 + 16 * q + i < B;
        xr[q] = x + (size_t)min(b0 + 16 * q + i, B - 1) * n;
    }
    floatx4v acc[G], acc2[MODE == 2 ? G : 1];
    float ss[G];
#pragma unroll
    for (int q = 0; q < G; q++) {
        acc[q] = floatx4v{0.f, 0.f, 0.f, 0.f};
        if (MODE == 2) acc2[MODE == 2 ? q : 0] = floatx4v{0.f, 0.f, 0.f, 0.f};
        ss[q] = 0.f;
    }
    // the residual epilogue's old values (wavefront 0 finishes the tile) are requested with the first weights
    float prev[G][4];
#pragma unroll
    for (int q = 0; q < G; q++)
#pragma unroll
        for (int v = 0; v < 4; v++)
            prev[q][v] = (MODE == 1 && wave == 0 && jv[q] && r0 + 4 * kk + v < rows) ? y[(size_t)(b0 + 16 * q + i) * ldy + r0 + 4 * kk + v] : 0.f;
    constexpr int U = G == 1 ? 4 : 2;   // slabs whose loads are in flight together
    for (int base = wave; base < nit; base += NS * U) {
        float w[U][8], w2[MODE == 2 ? U : 1][8], gv[NORM ? U : 1][8];
#pragma unroll
        for (int t = 0; t < U; t++) {
            const int k0 = min(base + t * NS, nit - 1) << 5;   // past the end: re-read the last slab, not used
            if (PACKED) {
                PackedSlab<T>::w(wr + (size_t)(k0 >> 5) * 512, lane, w[t]);
                if (MODE == 2) PackedSlab<T>::w(wr2 + (size_t)(k0 >> 5) * 512, lane, w2[MODE == 2 ? t : 0]);
            } else {
                Slab8<T>::w(wr + k0, kk, w[t]);
                if (MODE == 2) Slab8<T>::w(wr2 + k0, kk, w2[MODE == 2 ? t : 0]);
            }
            if (NORM) Slab8<T>::x(g + k0, kk, gv[NORM ? t : 0]);
        }
#pragma unroll
        for (int q = 0; q < G; q++) {
            float xv[U][8];
#pragma unroll
            for (int t = 0; t < U; t++) Slab8<T>::x(xr[q] + (min(base + t * NS, nit - 1) << 5), kk, xv[t]);
#pragma unroll
            for (int t = 0; t < U; t++) {
                if (base + t * NS >= nit) break;
                if (NORM) {
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        ss[q] += xv[t][e] * xv[t][e];
                        xv[t][e] *= gv[NORM ? t : 0][e];
                    }
                }
                if (!jv[q]) {
#pragma unroll
                    for (int e = 0; e < 8; e++) xv[t][e] = 0.f;
                }
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    acc[q] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[t][e], xv[t][e], acc[q], 0, 0, 0);
                    if (MODE == 2)
                        acc2[MODE == 2 ? q : 0] = __builtin_amdgcn_mfma_f32_16x16x4f32(w2[MODE == 2 ? t : 0][e], xv[t][e], acc2[MODE == 2 ? q : 0], 0, 0, 0);
                }
            }
        }
    }
    // the wavefronts' partial tiles meet in LDS one group at a time; wavefront 0 finishes each
#pragma unroll
    for (int q = 0; q < G; q++) {
        if (q > 0) __syncthreads();   // wavefront 0 has read the previous group's partials
        if (NORM) {
            float t = ss[q];
            t += __shfl_xor(t, 16, 64);
            t += __shfl_xor(t, 32, 64);
            if (kk == 0) sspart[wave][i] = t;
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            part[wave][lane * 4 + v] = acc[q][v];
            if (MODE == 2) part[wave][256 + lane * 4 + v] = acc2[MODE == 2 ? q : 0][v];
        }
        __syncthreads();
        if (wave != 0) continue;
        // accumulator register v of lane l is row 4 * (l / 16) + v, batch column l % 16
        float d[4], d2[4];
#pragma unroll
        for (int v = 0; v < 4; v++) {
            d[v] = 0.f;
            d2[v] = 0.f;
        }
#pragma unroll
        for (int w_ = 0; w_ < NS; w_++) {
            const float4 p = *(const float4*)&part[w_][lane * 4];
            d[0] += p.x; d[1] += p.y; d[2] += p.z; d[3] += p.w;
            if (MODE == 2) {
                const float4 p2 = *(const float4*)&part[w_][256 + lane * 4];
                d2[0] += p2.x; d2[1] += p2.y; d2[2] += p2.z; d2[3] += p2.w;
            }
        }
        if (!jv[q]) continue;
        float inv = 1.f;
        if (NORM) {
            float t = 0.f;
#pragma unroll
            for (int w_ = 0; w_ < NS; w_++) t += sspart[w_][i];
            inv = 1.0f / sqrtf(t / n + 1e-5f);
        }
        float* out = y + (size_t)(b0 + 16 * q + i) * ldy + r0 + 4 * kk;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            if (r0 + 4 * kk + v >= rows) break;
            const float a0 = d[v] * inv;
            if (MODE == 0) out[v] = a0;
            else if (MODE == 1) out[v] = prev[q][v] + a0;
            else out[v] = a0 * (1.0f / (1.0f + expf(-a0))) * (d2[v] * inv);
        }
    }
}

// End of a decode step, one workgroup per sequence: first-max argmax over the logits
// (sample_argmax, llama2_sampler.cpp:25-36: strict '>' so the lowest index wins ties), record
// the id, embed the token of the next position (forced prompt id while pos + 1 < n_prompt,
// generate loop llm.cpp:208-228) and, in the workgroup that takes the last ticket, advance the
// position.  Every workgroup reads the position before it takes its ticket.
// With `given` the id of every sequence comes from the host sampler instead of the scan.
template <typename T>
__global__ __launch_bounds__(1024) void sample_advance_kernel(const float* __restrict__ logits, int V, GenState* st, int* ticket,
                                                               const int* __restrict__ prompt, int promptStride, int* next,
                                                               int* out_ids, const T* __restrict__ emb, float* __restrict__ x,
                                                               int dim, int* cur, const int* __restrict__ given,
                                                               unsigned long long* rng = nullptr)
{
    __shared__ float sv[16];
    __shared__ int si[16];
    __shared__ int stok;
    const int b = blockIdx.x;
    const int pos = st->pos, nPrompt = st->n_prompt;
    const float* lg = logits + (size_t)b * V;
    // the forced id of the next position, if there is one, is requested before the scan instead of after it
    const bool forced = pos + 1 < nPrompt && pos + 1 < promptStride;
    const int forcedTok = (threadIdx.x == 0 && forced) ? prompt[(size_t)b * promptStride + pos + 1] : 0;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    if (given) V = 0;   // the host sampler chose the id: nothing to scan
    auto take = [&](float v, int i) {
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
    };
    if ((V & 3) == 0) {
        const int n4 = V >> 2;
        constexpr int U = 8;
        for (int i0 = threadIdx.x; i0 < n4; i0 += 1024 * U) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = i0 + u * 1024;
                v[u] = i < n4 ? *(const float4*)(lg + (size_t)i * 4) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = (i0 + u * 1024) * 4;
                take(v[u].x, i); take(v[u].y, i + 1); take(v[u].z, i + 2); take(v[u].w, i + 3);
            }
        }
    } else {
        for (int i = threadIdx.x; i < V; i += 1024) take(lg[i], i);
    }
    wave_argmax_first(bv, bi);
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) { sv[w] = bv; si[w] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 16; i++)
            if (sv[i] > bv || (sv[i] == bv && si[i] < bi)) { bv = sv[i]; bi = si[i]; }
        if (bi == 0x7fffffff) bi = 0;  // all NaN: index 0, as a scan that never finds a larger value would give
        if (given) bi = given[b];
        next[b] = bi;
        out_ids[(size_t)b * promptStride + pos] = bi;
        const int tok = forced ? forcedTok : bi;
        cur[b] = tok;
        stok = tok;
    }
    __syncthreads();
    const int tok = stok;
    for (int i = threadIdx.x; i < dim; i += 1024) x[(size_t)b * dim + i] = wld(emb, (size_t)tok * dim + i);
    if (threadIdx.x == 0) {
        // the last sequence to finish advances the position; a single sequence has no one to wait for (and no atomic
        // whose answer the kernel would have to wait for before it can end)
        if (gridDim.x == 1 || atomicAdd(ticket, 1) == (int)gridDim.x - 1) {
            if (gridDim.x > 1) *ticket = 0;
            st->pos = pos + 1;
            st->len = pos + 2;
            if (rng) {
                // the device sampler drew one coin per sequence from this step's state (sample_device_kernel)
                unsigned long long r = *rng;
                for (unsigned int d = 0; d < gridDim.x; d++) {
                    r ^= r >> 12;
                    r ^= r << 25;
                    r ^= r >> 27;
                }
                *rng = r;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Temperature / top-p sampling on the device (sample, llama2_sampler.cpp:126-151, with sample_mult :38-49 and
// sample_topp :59-100), one workgroup of 1024 threads per sequence, so that a sampled generation needs no copy of the
// logits to the host.  The reference's arithmetic is sequential - the softmax denominator and the cumulative sums are
// running fp32 sums in index order and in sorted order - and with a flat distribution the rounding of those sums moves
// the chosen id as often as one time in five, so it is kept: what can run in parallel does (maximum, exponentials,
// division, the sort), and the running sums come out bit for bit as the reference's loops leave them
// (wg_running_sum_until).
//   * The coin is the reference's: xorshift64* (:115-124) on a state kept in device memory; sequence b of a step takes
//     draw b + 1 from the step's state (the reference flips one coin per forward call, forced positions included), and
//     the step's tail kernel moves the state on by one draw per sequence.
//   * exp is taken in double and rounded to float: the host library's expf is correctly rounded for all but a handful of
//     arguments, the device's single-precision one is not.
//   * The logits are overwritten by the probabilities, as in the reference.
//   * Top-p: the candidates (probability >= (1 - topp) / (n - 1)) are gathered in LDS and sorted by value (bitonic,
//     descending, 32 values per thread in registers); the order among equal values does not change a sum, only which
//     index a position stands for, and that is settled afterwards: the m-th of the equal values in the sorted list is
//     the m-th of them by index.
// Up to 32768 logits (128 KB of LDS); the engine samples longer vocabularies on the host.
__device__ __forceinline__ unsigned long long xorshift64_next(unsigned long long st)
{
    st ^= st >> 12;
    st ^= st << 25;
    st ^= st >> 27;
    return st;
}
struct WgScratch { float f[16]; int i[16]; };
__device__ __forceinline__ float wg_max_1024(float v, WgScratch& sc)
{
    v = group_max<64>(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sc.f[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = sc.f[0];
#pragma unroll
    for (int w = 1; w < 16; w++) t = fmaxf(t, sc.f[w]);
    return t;
}
__device__ __forceinline__ int wg_exclusive_scan_int_1024(int v, WgScratch& sc)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int inc = v;
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(inc, o, 64);
        if (lane >= o) inc += up;
    }
    __syncthreads();
    if (lane == 63) sc.i[wave] = inc;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; w++) base += sc.i[w];
    return base + inc - v;
}
constexpr int SAMPLE_MAX_VOCAB = 32768;
// The running sum acc += buf[0], acc += buf[1], ... in fp32, every addition rounded, as the reference's loops do it: the
// sum after the last value, or the first index at which a threshold on the sum holds.  One lane adding 32000 numbers
// one after the other is 150000 cycles of dependent additions; this does the same additions, bit for bit, in a
// fraction of that.  While the sum stays in one binade it is an integer m < 2^24 times u = ulp(sum), and adding
// x >= 0 gives m + round(x / u) - round to nearest, a tie (x / u = k + 1/2) to the even neighbour, which depends on
// nothing but the parity of m.  So a run of values is, for a known exponent of the sum, a function of that parity alone:
// it adds an integer and leaves a parity, and a tie forces the parity to even whatever it was.  Every thread works
// that function out for its own chunk of 33 consecutive values (stride 33: its LDS reads hit 64 different banks),
// taking the exponent from an approximate prefix sum; then one lane goes over the chunks in order with a few integer
// operations each.  A chunk whose guess was wrong (the exact sum has another exponent than the approximate one), in
// which the sum reaches the next binade, whose prefix is zero, or the one in which the threshold is crossed is added
// up value by value - a handful of the thousand chunks.  All 1024 threads call it; values must not be negative.
struct SumChunk { int e, sum0, sum1, meta; };   // meta: bit 0 / 1 parity left for incoming parity 0 / 1, bit 2 usable
constexpr int SUM_CHUNK = 33;
static_assert(SAMPLE_MAX_VOCAB <= 1024 * SUM_CHUNK, "one chunk per thread");
template <typename F>
__device__ __forceinline__ int wg_running_sum_until(const float* buf, int n, float& acc, F exceeds, SumChunk* tab, WgScratch& sc,
                                                    int* result)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i0 = tid * SUM_CHUNK;
    const int cnt = min(max(n - i0, 0), SUM_CHUNK);
    float x[SUM_CHUNK];
    float part = 0.f;
#pragma unroll
    for (int i = 0; i < SUM_CHUNK; i++) {
        x[i] = i < cnt ? buf[i0 + i] : 0.f;
        part += x[i];
    }
    // approximate sum in front of this chunk: scan over the lanes, then over the wavefronts
    float inc = part;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float up = __shfl_up(inc, o, 64);
        if (lane >= o) inc += up;
    }
    __syncthreads();
    if (lane == 63) sc.f[wave] = inc;
    __syncthreads();
    float before = acc;
    for (int w = 0; w < wave; w++) before += sc.f[w];
    before += inc - part;
    {
        const unsigned int bb = __float_as_uint(before), be = (bb >> 23) & 0xffu;
        SumChunk t;
        t.e = (int)be;                                        // biased exponent the sum is expected to have
        bool ok = cnt == SUM_CHUNK && be >= 1u && be <= 254u;
        int sum[2] = {0, 0}, par[2] = {0, 1};
        const int shift = 150 - (int)be;                       // x / u = x * 2^(23 - (be - 127))
#pragma unroll
        for (int i = 0; i < SUM_CHUNK; i++) {
            const float y = __builtin_ldexpf(x[i], shift);
            ok = ok && y < 16777216.f;
            const float fl = floorf(y), fr = y - fl;
            const int k = (int)fminf(fl, 16777216.f);
            const int up = fr > 0.5f ? 1 : 0;
            const bool tie = fr == 0.5f;
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const int q = k + (tie ? ((par[p] ^ k) & 1) : up);
                par[p] ^= q & 1;
                sum[p] += q;
            }
        }
        ok = ok && sum[0] < 16777216 && sum[1] < 16777216;
        t.sum0 = sum[0];
        t.sum1 = sum[1];
        t.meta = par[0] | (par[1] << 1) | (ok ? 4 : 0);
        tab[tid] = t;
    }
    __syncthreads();
    if (wave == 0) {
        // Wavefront 0 goes over the chunks 64 at a time.  The chunks' functions compose (parity in -> integer added,
        // parity out), so an inclusive scan over the lanes gives every lane the sum after its chunk, all at once; the
        // first lane whose chunk cannot be taken that way (or behind which the threshold holds) is where the value-by-value
        // additions take over for one chunk, and the scan resumes behind it.
        const int nch = (n + SUM_CHUNK - 1) / SUM_CHUNK;
        unsigned int sb = __float_as_uint(acc);
        int hit = n, c = 0;
        while (c < nch) {
            const int cc = c + lane;
            const SumChunk t = tab[min(cc, 1023)];
            unsigned int s0 = (unsigned int)t.sum0, s1 = (unsigned int)t.sum1;
            int p0 = t.meta & 1, p1 = (t.meta >> 1) & 1;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const unsigned int us0 = __shfl_up(s0, o, 64), us1 = __shfl_up(s1, o, 64);
                const int up0 = __shfl_up(p0, o, 64), up1 = __shfl_up(p1, o, 64);
                if (lane >= o) {
                    // the lanes before, then mine
                    const unsigned int n0 = us0 + (up0 ? s1 : s0), n1 = us1 + (up1 ? s1 : s0);
                    const int q0 = up0 ? p1 : p0, q1 = up1 ? p1 : p0;
                    s0 = n0; s1 = n1; p0 = q0; p1 = q1;
                }
            }
            const unsigned int m = (sb & 0x7fffffu) | 0x800000u;
            // behind a chunk that cannot be taken the scan's sums mean nothing (and may have wrapped): 64 bits for the compare
            const unsigned long long tot = (unsigned long long)m + (unsigned long long)((m & 1u) ? s1 : s0);
            const unsigned int nb = (sb & 0xff800000u) | ((unsigned int)tot & 0x7fffffu);
            const bool fail = cc >= nch || !(t.meta & 4) || (int)(sb >> 23) != t.e || tot >= 0x1000000ull || exceeds(__uint_as_float(nb));
            const unsigned long long mask = __ballot(fail);
            const int f = mask ? __builtin_ctzll(mask) : 64;
            if (f > 0) sb = (unsigned int)__builtin_amdgcn_readlane((int)nb, f - 1);
            c += f;
            if (f < 64 && c < nch) {
                // value by value (every lane the same additions: the result stays uniform)
                float a = __uint_as_float(sb);
                const int j0 = c * SUM_CHUNK, j1 = min(j0 + SUM_CHUNK, n);
                int j = j0;
                for (; j < j1; j++) {
                    a += buf[j];
                    if (exceeds(a)) break;
                }
                sb = __float_as_uint(a);
                if (j < j1) { hit = j; break; }
                c++;
            }
        }
        if (lane == 0) {
            result[0] = hit;
            result[1] = (int)sb;
        }
    }
    __syncthreads();
    acc = __uint_as_float((unsigned int)result[1]);
    const int hit = result[0];
    __syncthreads();   // result[] may be written again by the next call
    return hit;
}
// Rows of a batched prompt pass (P > 0): row row0 + blockIdx.x = (sequence b, position p) of B sequences takes draw
// p B + b + 1 - the coin the one-position-at-a-time loop would have flipped for it - and its id goes to
// out_ids[b][p] (and to next[b] after the last position) instead of given[].
__global__ __launch_bounds__(1024) void sample_device_kernel(float* __restrict__ logits, int V, float temperature, float topp,
                                                             const unsigned long long* __restrict__ rng, int* __restrict__ given,
                                                             int row0 = 0, int P = 0, int B = 0, int promptStride = 0,
                                                             int* __restrict__ out_ids = nullptr, int* __restrict__ next = nullptr)
{
    extern __shared__ __attribute__((aligned(16))) float sbuf[];   // V values in index order, later the sorted candidates
    __shared__ WgScratch sc;
    __shared__ SumChunk tab[1024];
    __shared__ int sres[2];
    __shared__ float sval[2];
    __shared__ int sint[4];
    const int tid = threadIdx.x, b = blockIdx.x;
    float* p = logits + (size_t)b * V;
    const int rowSeq = P > 0 ? (row0 + b) / P : b, rowPos = P > 0 ? (row0 + b) - rowSeq * P : 0;
    auto emit = [&](int id) {
        if (P > 0) {
            out_ids[(size_t)rowSeq * promptStride + rowPos] = id;
            if (rowPos == P - 1) next[rowSeq] = id;
        } else given[b] = id;
    };
    // the coin: draw b + 1 of the step's state (:115-124)
    unsigned long long st = *rng;
    const int draws = P > 0 ? rowPos * B + rowSeq : b;
    for (int d = 0; d <= draws; d++) st = xorshift64_next(st);
    const float coin = (float)((unsigned int)((st * 0x2545F4914F6CDD1Dull) >> 32) >> 8) / 16777216.0f;
    // probabilities (:131-135; softmax, llama2_cpu.cpp): maximum, exponentials, their sum in index order, division
    float mx = -INFINITY;
    for (int i = tid; i < V; i += 1024) {
        const float v = p[i] / temperature;
        sbuf[i] = v;
        mx = fmaxf(mx, v);
    }
    mx = wg_max_1024(mx, sc);
    for (int i = tid; i < V; i += 1024) sbuf[i] = (float)exp((double)(sbuf[i] - mx));
    __syncthreads();
    float sum = 0.f;
    wg_running_sum_until(sbuf, V, sum, [](float) { return false; }, tab, sc, sres);
    for (int i = tid; i < V; i += 1024) {
        const float q = sbuf[i] / sum;
        sbuf[i] = q;
        p[i] = q;
    }
    __syncthreads();
    if (topp <= 0.f || topp >= 1.f) {
        // sample_mult: the first index whose running sum exceeds the coin, else the last one
        float cdf = 0.f;
        const int hit = wg_running_sum_until(sbuf, V, cdf, [coin](float c) { return coin < c; }, tab, sc, sres);
        if (tid == 0) emit(hit < V ? hit : V - 1);
        return;
    }
    // candidates into LDS, in any order (this thread's values are in registers of a sort: re-read from memory)
    const float cutoff = (1.0f - topp) / (float)(V - 1);
    float mine[SAMPLE_MAX_VOCAB / 1024];
#pragma unroll
    for (int j = 0; j < SAMPLE_MAX_VOCAB / 1024; j++) {
        const int i = j * 1024 + tid;
        mine[j] = i < V ? sbuf[i] : 0.f;
    }
    int keep = 0;
#pragma unroll
    for (int j = 0; j < SAMPLE_MAX_VOCAB / 1024; j++) keep += (mine[j] >= cutoff && j * 1024 + tid < V) ? 1 : 0;
    int at = wg_exclusive_scan_int_1024(keep, sc);   // its barriers also separate the reads above from the writes below
    if (tid == 1023) sint[0] = at + keep;
#pragma unroll
    for (int j = 0; j < SAMPLE_MAX_VOCAB / 1024; j++)
        if (mine[j] >= cutoff && j * 1024 + tid < V) sbuf[at++] = mine[j];
    __syncthreads();
    const int n0 = sint[0];
    if (n0 == 0) {
        // the reference would index in front of its list; the largest probability (lowest index) is the sane answer
        float best = 0.f;
        for (int i = tid; i < V; i += 1024) best = fmaxf(best, p[i]);
        best = wg_max_1024(best, sc);
        if (tid == 0) sint[1] = 0x7fffffff;
        __syncthreads();
        for (int i = tid; i < V; i += 1024)
            if (p[i] == best) atomicMin(&sint[1], i);
        __syncthreads();
        if (tid == 0) emit(sint[1]);
        return;
    }
    // Bitonic sort, descending, 32 values per thread in registers: position 32 t + r of the sequence is register r of
    // thread t.  Exchanges 1 .. 16 apart stay inside a thread, those 32 .. 1024 apart are lane exchanges inside a wavefront,
    // only the ones 2048 and more apart go through LDS (ten of the 120 steps at 32768 values).  Padding zeros sort behind
    // every candidate (a candidate is at least the cutoff, which is positive).
    constexpr int EPT = 32;
    int n2 = EPT;
    while (n2 < n0) n2 <<= 1;
    const int nthr = n2 / EPT;
    float el[EPT];
#pragma unroll
    for (int r = 0; r < EPT; r++) {
        const int i = r * nthr + tid;
        el[r] = (tid < nthr && i < n0) ? sbuf[i] : 0.f;
    }
    __syncthreads();   // the values are in registers: the buffer is free for the exchanges
    auto inside = [&](int j, bool desc) {   // compare-exchange of the registers j apart, larger first where desc
#pragma unroll
        for (int r = 0; r < EPT; r++)
            if ((r & j) == 0) {
                const float mx = fmaxf(el[r], el[r | j]), mn = fminf(el[r], el[r | j]);
                el[r] = desc ? mx : mn;
                el[r | j] = desc ? mn : mx;
            }
    };
    // runs of 32 inside each thread, alternating direction from thread to thread as a run of 64 wants them
#pragma unroll
    for (int k = 2; k <= EPT; k <<= 1)
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
#pragma unroll
            for (int r = 0; r < EPT; r++)
                if ((r & j) == 0) {
                    const bool desc = k == EPT ? (tid & 1) == 0 : (r & k) == 0;
                    const float mx = fmaxf(el[r], el[r | j]), mn = fminf(el[r], el[r | j]);
                    el[r] = desc ? mx : mn;
                    el[r | j] = desc ? mn : mx;
                }
        }
    for (int k = 2 * EPT; k <= n2; k <<= 1) {
        const bool desc = ((tid * EPT) & k) == 0;
        for (int j = k >> 1; j >= EPT; j >>= 1) {
            const int jm = j / EPT;
            const bool keepmax = ((tid & jm) == 0) == desc;
            if (jm < 64) {
#pragma unroll
                for (int r = 0; r < EPT; r++) {
                    const float other = __shfl_xor(el[r], jm, 64);
                    el[r] = keepmax ? fmaxf(el[r], other) : fminf(el[r], other);
                }
            } else {
#pragma unroll
                for (int r = 0; r < EPT; r++) sbuf[r * 1024 + tid] = el[r];
                __syncthreads();
#pragma unroll
                for (int r = 0; r < EPT; r++) {
                    const float other = sbuf[r * 1024 + (tid ^ jm)];
                    el[r] = keepmax ? fmaxf(el[r], other) : fminf(el[r], other);
                }
                __syncthreads();
            }
        }
#pragma unroll
        for (int j = EPT >> 1; j > 0; j >>= 1) inside(j, desc);
    }
    if (tid < nthr) {
#pragma unroll
        for (int r = 0; r < EPT; r += 4) *(float4*)(sbuf + tid * EPT + r) = make_float4(el[r], el[r + 1], el[r + 2], el[r + 3]);
    }
    __syncthreads();
    // end of the nucleus (:78-87) and the sampled position (:89-99), running sums in sorted order
    float cum = 0.f;
    int last = wg_running_sum_until(sbuf, n0, cum, [topp](float c) { return c > topp; }, tab, sc, sres);
    if (last == n0) last = n0 - 1;
    const float r = coin * cum;
    float cdf = 0.f;
    int pos = wg_running_sum_until(sbuf, last + 1, cdf, [r](float c) { return r < c; }, tab, sc, sres);
    if (pos > last) pos = last;
    if (tid == 0) {
        // the position stands for the m-th (by index) of the candidates that share its value
        const float v = sbuf[pos];
        int first = pos;
        while (first > 0 && sbuf[first - 1] == v) first--;
        sval[1] = v;
        sint[2] = pos - first + 1;
        sint[3] = -1;
    }
    __syncthreads();
    const float v = sval[1];
    const int m = sint[2];
    const int chunk = (V + 1023) / 1024, i0 = min(tid * chunk, V), i1 = min(i0 + chunk, V);
    int cnt = 0;
    for (int i = i0; i < i1; i++) cnt += p[i] == v ? 1 : 0;
    const int before = wg_exclusive_scan_int_1024(cnt, sc);
    if (before < m && m <= before + cnt) {
        int k = before;
        for (int i = i0; i < i1; i++)
            if (p[i] == v && ++k == m) sint[3] = i;
    }
    __syncthreads();
    if (tid == 0) emit(sint[3]);
}

// The sampler's running sum by itself (the RUNNING_SUM entry, for checking it against a plain loop): out[0] = first index
// at which the sum exceeds `threshold` (n if none), out[1] = bits of the sum reached.
__global__ __launch_bounds__(1024) void running_sum_kernel(const float* __restrict__ values, int n, float threshold, int* out)
{
    extern __shared__ __attribute__((aligned(16))) float sbuf[];
    __shared__ WgScratch sc;
    __shared__ SumChunk tab[1024];
    __shared__ int sres[2];
    for (int i = threadIdx.x; i < n; i += 1024) sbuf[i] = values[i];
    __syncthreads();
    float acc = 0.f;
    const int hit = wg_running_sum_until(sbuf, n, acc, [threshold](float c) { return c > threshold; }, tab, sc, sres);
    if (threadIdx.x == 0) { out[0] = hit; out[1] = (int)__float_as_uint(acc); }
}

// the random stream moved on by n draws (what a batched prompt pass of n rows used up)
__global__ void rng_advance_kernel(unsigned long long* rng, int n)
{
    unsigned long long st = *rng;
    for (int d = 0; d < n; d++) st = xorshift64_next(st);
    *rng = st;
}

// the sampling kernel keeps a whole vocabulary in LDS: 128 KB of dynamic LDS, allowed once per process
static hipError_t sample_attr()
{
    static bool done = false;
    if (done) return hipSuccess;
    hipError_t e = hipFuncSetAttribute((const void*)sample_device_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SAMPLE_MAX_VOCAB * 4);
    done = e == hipSuccess;
    return e;
}

// ---------------------------------------------------------------------------
// Batched prompt prefill: the P forced prompt positions of every sequence go through the layers as one (B*P)-row
// matrix (row m = b*P + p) instead of P single-token steps (the reference's loop, llm.cpp:208-231, forward() per
// token).  The projections run on the MFMA GEMM, attention on the fused causal kernel; the kernels below are the
// glue between their layouts.

// x[m,:] = emb[prompt[b][p],:]
template <typename T>
__global__ void prefill_embed_kernel(const int* __restrict__ prompt, int promptStride, int P, const T* __restrict__ emb,
                                     float* __restrict__ x, int dim)
{
    const int m = blockIdx.x, b = m / P, p = m - b * P;
    const int tok = prompt[(size_t)b * promptStride + p];
    for (int i = threadIdx.x; i < dim; i += blockDim.x) x[(size_t)m * dim + i] = wld(emb, (size_t)tok * dim + i);
}

__device__ inline void store_pair(float* p, float2 v) { *(float2*)p = v; }
__device__ inline void store_pair(bf16_t* p, float2 v) { *(uint32_t*)p = (uint32_t)f32_to_bf16(v.x) | ((uint32_t)f32_to_bf16(v.y) << 16); }
// what a later decode step reads back from a cache of type TC
template <typename TC> __device__ inline float2 as_stored(float2 v) { return v; }
template <> __device__ inline float2 as_stored<bf16_t>(float2 v) { return make_float2(bf16_to_f32(f32_to_bf16(v.x)), bf16_to_f32(f32_to_bf16(v.y))); }

// One row [q | k | v] of raw projections per (b, p): rotate q and k at position p (adjacent pairs, the arithmetic of
// the decode kernel), write q as (B,H,P,hs), k and v as (B,H,P,hs) with every key / value head repeated for the query
// heads that share it, and append the rotated key and the value to the caches [b][pos][kvd].
template <typename TC, typename TQ>
__global__ void prefill_rope_scatter_kernel(const float* __restrict__ qkv, TQ* __restrict__ qh, TQ* __restrict__ kh,
                                            TQ* __restrict__ vh, TC* __restrict__ kc, TC* __restrict__ vc,
                                            const float* __restrict__ fcos, const float* __restrict__ fsin, int B, int P, int H,
                                            int kvH, int hs, int seqLen)
{
    const int dim = H * hs, kvd = kvH * hs, ldq = dim + 2 * kvd, half = hs / 2, kvMul = H / kvH;
    const size_t pairsPerRow = (size_t)ldq / 2;
    const size_t total = (size_t)B * P * pairsPerRow;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)blockDim.x * gridDim.x) {
        const size_t m = i / pairsPerRow;
        const int col = (int)(i - m * pairsPerRow) * 2;
        const int b = (int)(m / P), p = (int)(m - (size_t)b * P);
        const float2 r = *(const float2*)(qkv + m * ldq + col);
        if (col < dim + kvd) {
            const int c = col < dim ? col : col - dim;
            const int h = c / hs, d = c - h * hs;
            const float cs = fcos[(size_t)p * half + d / 2], sn = fsin[(size_t)p * half + d / 2];
            float2 o;
            o.x = r.x * cs - r.y * sn;
            o.y = r.x * sn + r.y * cs;
            if (col < dim) {
                store_pair(qh + (((size_t)b * H + h) * P + p) * hs + d, o);
            } else {
                o = as_stored<TC>(o);   // the pass attends over the values the cache holds, as the decode steps will
                store_pair(kc + ((size_t)b * seqLen + p) * kvd + c, o);
                for (int g = 0; g < kvMul; g++) store_pair(kh + (((size_t)b * H + h * kvMul + g) * P + p) * hs + d, o);
            }
        } else {
            const int c = col - dim - kvd;
            const int h = c / hs, d = c - h * hs;
            const float2 rs = as_stored<TC>(r);
            store_pair(vc + ((size_t)b * seqLen + p) * kvd + c, rs);
            for (int g = 0; g < kvMul; g++) store_pair(vh + (((size_t)b * H + h * kvMul + g) * P + p) * hs + d, rs);
        }
    }
}

// hb[m, j] = silu(h2[m, j]) * h2[m, hid + j], the epilogue of the decode path's W1|W3 mat-vec
__global__ void prefill_swiglu_kernel(const float* __restrict__ h2, float* __restrict__ hb, size_t rows, int hid)
{
    const size_t total = rows * hid;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)blockDim.x * gridDim.x) {
        const size_t m = i / hid;
        const int j = (int)(i - m * hid);
        const float a0 = h2[m * 2 * hid + j], a1 = h2[m * 2 * hid + hid + j];
        hb[i] = a0 * (1.0f / (1.0f + expf(-a0))) * a1;
    }
}

// The prompt pass over 16-bit weights multiplies its fp32 activations on the bf16 matrix cores.  LO = true: as two bf16
// numbers each - hi, the bf16 nearest to the value, and lo, the bf16 nearest to what hi leaves over; both products with
// a bf16 weight are exact and the sums are fp32, so the activations keep sixteen leading bits.  A row of n values then
// becomes 2 n bf16 values, the n his first.  LO = false: hi alone (activations rounded to bf16), rows of n.
template <bool LO> __device__ inline void split_store4(bf16_t* row, int n, int i, float4 v)
{
    const float f[4] = {v.x, v.y, v.z, v.w};
    bf16_t hi[4], lo[4];
#pragma unroll
    for (int q = 0; q < 4; q++) {
        hi[q] = f32_to_bf16(f[q]);
        lo[q] = f32_to_bf16(f[q] - bf16_to_f32(hi[q]));
    }
    *(uint2*)(row + i) = make_uint2((uint32_t)hi[0] | ((uint32_t)hi[1] << 16), (uint32_t)hi[2] | ((uint32_t)hi[3] << 16));
    if (LO) *(uint2*)(row + n + i) = make_uint2((uint32_t)lo[0] | ((uint32_t)lo[1] << 16), (uint32_t)lo[2] | ((uint32_t)lo[3] << 16));
}
// out[m] = split(g * x[m] / sqrt(mean(x[m]^2) + eps)) (g null: split(x[m])); one workgroup per row, n a multiple of 4
template <bool LO>
__global__ __launch_bounds__(256) void prefill_norm_split_kernel(const float* __restrict__ x, const float* __restrict__ g,
                                                                 bf16_t* __restrict__ out, int n, float eps)
{
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * n;
    bf16_t* orow = out + (size_t)blockIdx.x * (LO ? 2 : 1) * n;
    float inv = 1.0f;
    if (g) {
        float ss = 0.f;
        for (int i = threadIdx.x * 4; i < n; i += 1024) {
            const float4 v = *(const float4*)(xr + i);
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
        ss = group_sum<64>(ss);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
        __syncthreads();
        ss = red[0] + red[1] + red[2] + red[3];
        inv = 1.0f / sqrtf(ss / n + eps);
    }
    for (int i = threadIdx.x * 4; i < n; i += 1024) {
        float4 v = *(const float4*)(xr + i);
        if (g) {
            const float4 w = *(const float4*)(g + i);
            v = make_float4(w.x * (inv * v.x), w.y * (inv * v.y), w.z * (inv * v.z), w.w * (inv * v.w));
        }
        split_store4<LO>(orow, n, i, v);
    }
}
// First-max argmax of every logits row (sample_argmax, llama2_sampler.cpp:25-36), one workgroup per row: the id
// chosen after prompt position p of sequence b goes to out_ids[b][p]; the one after the last prefilled position is
// also the token the first decode step starts from (next[b]).
__global__ __launch_bounds__(256) void prefill_argmax_kernel(const float* __restrict__ logits, int V, int row0, int P,
                                                             int promptStride, int* __restrict__ out_ids, int* __restrict__ next)
{
    __shared__ float sv[4];
    __shared__ int si[4];
    const int m = row0 + blockIdx.x, b = m / P, p = m - b * P;
    const float* lg = logits + (size_t)blockIdx.x * V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    auto take = [&](float v, int i) {
        if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
    };
    if ((V & 3) == 0 && (((uintptr_t)lg) & 15) == 0) {
        // 16 bytes per lane, eight loads in flight
        const int n4 = V >> 2;
        constexpr int U = 8;
        for (int i0 = threadIdx.x; i0 < n4; i0 += 256 * U) {
            float4 v[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = i0 + u * 256;
                v[u] = i < n4 ? *(const float4*)(lg + (size_t)i * 4) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int i = (i0 + u * 256) * 4;
                take(v[u].x, i); take(v[u].y, i + 1); take(v[u].z, i + 2); take(v[u].w, i + 3);
            }
        }
    } else {
        for (int i = threadIdx.x; i < V; i += 256) take(lg[i], i);
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oi = __shfl_xor(bi, o, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < 4; i++)
            if (sv[i] > bv || (sv[i] == bv && si[i] < bi)) { bv = sv[i]; bi = si[i]; }
        if (bi == 0x7fffffff) bi = 0;
        out_ids[(size_t)b * promptStride + p] = bi;
        if (p == P - 1) next[b] = bi;
    }
}

__global__ void save_logits_kernel(const float* logits, float* all, const GenState* st, int V, int nSteps)
{
    const int b = blockIdx.y;
    float* dst = all + ((size_t)b * nSteps + st->pos) * V;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < V; i += blockDim.x * gridDim.x) dst[i] = logits[(size_t)b * V + i];
}

// ---------------------------------------------------------------------------
// per-kernel-class timing of one decode step: a HIP event pair around every launch
enum StepClass { SC_MATVEC_QKV = 0, SC_ROPE_STORE, SC_ATTN_DECODE, SC_MATVEC_WO, SC_MATVEC_W13, SC_MATVEC_W2, SC_MATVEC_CLS,
                 SC_SAMPLE, SC_COUNT };
struct StepProfile {
    std::vector<std::pair<int, std::pair<hipEvent_t, hipEvent_t>>> spans;
    hipError_t begin(int cls, hipStream_t s)
    {
        hipEvent_t a, b;
        hipError_t e = hipEventCreate(&a);
        if (e == hipSuccess) e = hipEventCreate(&b);
        if (e != hipSuccess) return e;
        spans.push_back({cls, {a, b}});
        return hipEventRecord(a, s);
    }
    hipError_t end(hipStream_t s) { return hipEventRecord(spans.back().second.second, s); }
};

template <typename T> struct LayerW { T *wqkv, *wo, *w13, *w2; float *rms_att, *rms_ffn; };

// The sampler of the reference engine (CudaExtension.llm32.llama2/Files/llama2_sampler.cpp), on the host as there:
// temperature, softmax (llama2_cpu.cpp:204-222), one 24-bit coin from xorshift64* per call, then the inverse CDF over
// all tokens or over the top-p nucleus.  Sums run sequentially in fp32, in the reference's order.
struct HostSampler {
    float temperature = 1.0f, topp = 0.9f;
    unsigned long long state = 0;
    std::vector<std::pair<float, int>> probindex;

    void build(float temp, float p, unsigned long long seed) { temperature = temp; topp = p; state = seed; }   // :102-109
    bool greedy() const { return temperature == 0.0f; }
    unsigned int random_u32()                                     // :115-121
    {
        state ^= state >> 12;
        state ^= state << 25;
        state ^= state >> 27;
        return (unsigned int)((state * 0x2545F4914F6CDD1Dull) >> 32);
    }
    float random_f32() { return (random_u32() >> 8) / 16777216.0f; }   // :122-124
    static int argmax(const float* p, int n)                     // :25-36
    {
        int best = 0;
        for (int i = 1; i < n; i++)
            if (p[i] > p[best]) best = i;
        return best;
    }
    static int sample_mult(const float* p, int n, float coin)    // :38-49
    {
        float cdf = 0.0f;
        for (int i = 0; i < n; i++) {
            cdf += p[i];
            if (coin < cdf) return i;
        }
        return n - 1;
    }
    int sample_topp(const float* p, int n, float coin)           // :59-100
    {
        probindex.clear();
        const float cutoff = (1.0f - topp) / (n - 1);
        for (int i = 0; i < n; i++)
            if (p[i] >= cutoff) probindex.push_back({p[i], i});
        // descending by probability; the reference's qsort leaves the order of equal probabilities to the C library,
        // here the lower index comes first
        std::sort(probindex.begin(), probindex.end(), [](const std::pair<float, int>& a, const std::pair<float, int>& b) {
            return a.first > b.first || (a.first == b.first && a.second < b.second);
        });
        const int n0 = (int)probindex.size();
        float cum = 0.0f;
        int last = n0 - 1;
        for (int i = 0; i < n0; i++) {
            cum += probindex[i].first;
            if (cum > topp) { last = i; break; }
        }
        const float r = coin * cum;
        float cdf = 0.0f;
        for (int i = 0; i <= last; i++) {
            cdf += probindex[i].first;
            if (r < cdf) return probindex[i].second;
        }
        return probindex[last].second;
    }
    // overwrites the logits with the probabilities unless greedy (:126-151)
    int sample(float* logits, int n)
    {
        if (greedy()) return argmax(logits, n);
        for (int q = 0; q < n; q++) logits[q] /= temperature;
        float mx = logits[0];
        for (int i = 1; i < n; i++)
            if (logits[i] > mx) mx = logits[i];
        float sum = 0.0f;
        for (int i = 0; i < n; i++) {
            logits[i] = expf(logits[i] - mx);
            sum += logits[i];
        }
        for (int i = 0; i < n; i++) logits[i] /= sum;
        const float coin = random_f32();
        if (topp <= 0 || topp >= 1) return sample_mult(logits, n, coin);
        return sample_topp(logits, n, coin);
    }
};

class Engine {
public:
    Config cfg{};
    bool loaded = false;
    bool bf16_weights = false;   // storage the NEXT load uploads the weights in
    bool stored_bf16 = false;    // storage of the weights that are on the device now: every launch dispatches on this
    bool use_graph = true;
    bool lastUsedGraph = false;  // whether the last generate replayed a captured graph (false: eager launches)
    bool use_prefill = true;     // prompt positions as one batched pass (false: one decode step per position)
    bool prefill_act16 = false;  // 16-bit weights, many prompt rows: activations of the pass rounded to bf16 (false: kept to sixteen bits)
    bool device_sampling = true; // temperature / top-p on the device (false: logits to the host every step)
    bool kv_bf16 = false;        // caches stored as bf16 (option 8; takes effect when the run state is next allocated)
    bool state_kv_bf16 = false;  // what the allocated caches hold
    void set_kv_bf16(bool on) { kv_bf16 = on; if (on != state_kv_bf16) { stateB = -1; graphB = -1; } }
    float lastPrefillMs = 0.f;   // HIP-event duration of the batched prompt pass of the last generate (0: none ran)
    int lastPrefillRows = 0;     // sequences x prompt positions it covered
    int mvRows = 0;              // weight rows per wavefront in the mat-vec kernels (0: chosen per shape)
    void set_mv_rows(int r) { mvRows = r; graphB = -1; }   // the captured step is rebuilt at the next generation
    bool defer_merge = true;     // batch 1: the output projection merges the attention's splits (when the shapes allow)
    void set_defer_merge(bool on) { defer_merge = on; graphB = -1; }
    int shared_classifier = 0;
    int timedFrom = -1;          // first step of the timed span (-1: first step after the prompt)
    std::string lastError;       // detail of the last failed load, handed to the caller's error text
    float lastTimedMs = 0.f;     // HIP-event duration of the timed span of the last generate
    int lastTimedSteps = 0;

    ~Engine() { release(); }
    long load(const char* path);
    long sample_device(float* lg, int n, HostSampler* sampler, int* id);
    long running_sum_device(const float* values, int n, float threshold, int* out2);
    long generate(const int* prompts, int batch, int nPrompt, int nSteps, bool wantLogits, std::vector<int>* ids,
                  std::vector<float>* logits, std::atomic<bool>* cancel, int chunk = 0,
                  const std::function<bool(const int*, int, int)>& onChunk = nullptr, HostSampler* sampler = nullptr);
    void release();
    long profile_step(int pos, int reps, int B, std::vector<float>* out);

private:
    template <typename T> long upload(const float* blob);
    // tail: 1 = first-max argmax on the device, 0 = stop at the logits (the host samples), 2 = temperature / top-p on the device
    template <typename T> long step(hipStream_t s, int B, int nSteps, float* allLogits, StepProfile* prof = nullptr, int tail = 1);
    template <typename T> long advance_given(hipStream_t s, int B);
    long ensure_state(int B, int nSteps);
    long ensure_prefill(size_t rows);
    template <typename T> long prefill(hipStream_t s, int B, int P, int nSteps, float* allLogits, int tail = 1);
    hipError_t embed_first(hipStream_t s, int B);

    hipStream_t stream = nullptr;
    std::vector<void*> allocs;
    void* dalloc(size_t bytes)
    {
        void* p = nullptr;
        if (hipMalloc(&p, bytes ? bytes : 4) != hipSuccess) return nullptr;
        allocs.push_back(p);
        return p;
    }
    // weights
    void* emb = nullptr; void* wcls = nullptr; float* rms_final = nullptr;
    // tile-packed copies of the matrices for the matrix-core mat-vec (batched steps, skinny prompt passes); null pointers
    // where a matrix cannot be packed (columns not a multiple of 32) or the memory was not to be had
    std::vector<LayerW<void>> packed;
    void* wclsP = nullptr;
    template <typename T> void* pack_matrix(const void* W, size_t rows, size_t n, size_t second = 0);
    template <typename T> void pack_all();
    std::vector<LayerW<void>> layers;
    float *fcos = nullptr, *fsin = nullptr;
    // run state (sized for stateB sequences)
    int stateB = 0, stateSteps = 0;
    std::vector<void*> stateAllocs;
    float *x = nullptr, *xb = nullptr, *qkv = nullptr, *qc = nullptr, *hb = nullptr, *logits = nullptr;
    void *kc = nullptr, *vc = nullptr;             // caches [layer][batch][seq][kv_dim], fp32 or bf16 (state_kv_bf16)
    void* ws = nullptr; size_t wsBytes = 0;
    GenState* dstate = nullptr;
    int *dprompt = nullptr, *dnext = nullptr, *dcur = nullptr, *dout = nullptr;
    int *dcount = nullptr, *dticket = nullptr;   // attention merge tickets (B * heads) and the step ticket; zero between launches
    hipGraphExec_t graphExec = nullptr;
    int graphB = 0;
    int graphTail = 1;                           // the tail the captured step ends with (see step), and the sampler
    float graphTemperature = 0.f, graphTopp = 0.f;   // parameters captured with tail 2
    float sampleTemperature = 1.f, sampleTopp = 0.9f;
    unsigned long long* drng = nullptr;          // state of the device sampler's random stream
    int* dgiven = nullptr;                       // ids chosen by the host sampler (one per sequence)
    int hostNPrompt = 0;                         // prompt length of the running generation
    float* hLogits = nullptr; int* hGiven = nullptr; size_t hLogitsCount = 0;   // pinned staging of the sampled path
    // batched prompt pass: activations of rows = sequences x prompt positions, sized for pfRows
    size_t pfRows = 0, pfLogitRows = 0;
    std::vector<void*> prefillAllocs;
    float *pfX = nullptr, *pfXn = nullptr, *pfQkv = nullptr, *pfQ = nullptr, *pfK = nullptr, *pfV = nullptr,
          *pfH2 = nullptr, *pfHb = nullptr, *pfLogits = nullptr, *pfW = nullptr;
    bool pfSplit = false;
};

void Engine::release()
{
    if (stream) (void)hipStreamSynchronize(stream);
    if (graphExec) { (void)hipGraphExecDestroy(graphExec); graphExec = nullptr; }
    if (hLogits) { (void)hipHostFree(hLogits); hLogits = nullptr; hLogitsCount = 0; }
    if (hGiven) { (void)hipHostFree(hGiven); hGiven = nullptr; }
    for (void* p : stateAllocs) (void)hipFree(p);
    stateAllocs.clear();
    for (void* p : prefillAllocs) (void)hipFree(p);
    prefillAllocs.clear();
    pfRows = 0;
    for (void* p : allocs) (void)hipFree(p);
    allocs.clear();
    layers.clear();
    packed.clear();
    wclsP = nullptr;
    if (stream) { (void)hipStreamDestroy(stream); stream = nullptr; }
    loaded = false;
    stateB = 0;
}

// host fp32 -> device T
template <typename T> static long put(void* dst, const float* src, size_t n, hipStream_t s, std::vector<bf16_t>& tmp);
template <> long put<float>(void* dst, const float* src, size_t n, hipStream_t s, std::vector<bf16_t>&)
{
    HIPCHK(hipMemcpyAsync(dst, src, n * 4, hipMemcpyHostToDevice, s));
    HIPCHK(hipStreamSynchronize(s));
    return 0;
}
template <> long put<bf16_t>(void* dst, const float* src, size_t n, hipStream_t s, std::vector<bf16_t>& tmp)
{
    tmp.resize(n);
    for (size_t i = 0; i < n; i++) tmp[i] = f32_to_bf16(src[i]);
    HIPCHK(hipMemcpyAsync(dst, tmp.data(), n * 2, hipMemcpyHostToDevice, s));
    HIPCHK(hipStreamSynchronize(s));
    return 0;
}

template <typename T> long Engine::upload(const float* p)
{
    // file order (llama2_cpu.cpp:74-106): rms_att, rms_ffn, rms_final, tok_emb, wq, wk, wv, wo, w1, w2, w3[, wcls]
    const size_t L = cfg.n_layers, dim = cfg.dim, hid = cfg.hidden_dim;
    const size_t hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads, V = cfg.vocab_size;
    const float* rms_att = p;   p += L * dim;
    const float* rms_ffn = p;   p += L * dim;
    const float* rmsf = p;      p += dim;
    const float* tok = p;       p += V * dim;
    const float* wq = p;        p += L * dim * dim;
    const float* wk = p;        p += L * dim * kvd;
    const float* wv = p;        p += L * dim * kvd;
    const float* wo = p;        p += L * dim * dim;
    const float* w1 = p;        p += L * dim * hid;
    const float* w2 = p;        p += L * hid * dim;
    const float* w3 = p;        p += L * dim * hid;
    const float* wc = shared_classifier ? tok : p;
    std::vector<bf16_t> tmp;
    const size_t es = sizeof(T);
    long e;
    if (!(emb = dalloc(V * dim * es))) return MCH_ERROR_MEMORY_OUT;
    if ((e = put<T>(emb, tok, V * dim, stream, tmp))) return e;
    if (shared_classifier) wcls = emb;
    else {
        if (!(wcls = dalloc(V * dim * es))) return MCH_ERROR_MEMORY_OUT;
        if ((e = put<T>(wcls, wc, V * dim, stream, tmp))) return e;
    }
    if (!(rms_final = (float*)dalloc(dim * 4))) return MCH_ERROR_MEMORY_OUT;
    HIPCHK(hipMemcpy(rms_final, rmsf, dim * 4, hipMemcpyHostToDevice));
    layers.resize(L);
    for (size_t l = 0; l < L; l++) {
        LayerW<void>& w = layers[l];
        const size_t qkvRows = dim + 2 * kvd;
        if (!(w.wqkv = dalloc(qkvRows * dim * es)) || !(w.wo = dalloc(dim * dim * es)) || !(w.w13 = dalloc(2 * hid * dim * es)) ||
            !(w.w2 = dalloc(dim * hid * es)) || !(w.rms_att = (float*)dalloc(dim * 4)) || !(w.rms_ffn = (float*)dalloc(dim * 4)))
            return MCH_ERROR_MEMORY_OUT;
        char* q = (char*)w.wqkv;
        if ((e = put<T>(q, wq + l * dim * dim, dim * dim, stream, tmp))) return e;
        if ((e = put<T>(q + dim * dim * es, wk + l * dim * kvd, kvd * dim, stream, tmp))) return e;
        if ((e = put<T>(q + (dim + kvd) * dim * es, wv + l * dim * kvd, kvd * dim, stream, tmp))) return e;
        if ((e = put<T>(w.wo, wo + l * dim * dim, dim * dim, stream, tmp))) return e;
        if ((e = put<T>(w.w13, w1 + l * dim * hid, hid * dim, stream, tmp))) return e;
        if ((e = put<T>((char*)w.w13 + hid * dim * es, w3 + l * dim * hid, hid * dim, stream, tmp))) return e;
        if ((e = put<T>(w.w2, w2 + l * hid * dim, dim * hid, stream, tmp))) return e;
        HIPCHK(hipMemcpy(w.rms_att, rms_att + l * dim, dim * 4, hipMemcpyHostToDevice));
        HIPCHK(hipMemcpy(w.rms_ffn, rms_ffn + l * dim, dim * 4, hipMemcpyHostToDevice));
    }
    return 0;
}

// tile-packed copy of a rows x n matrix (of two stacked ones of `rows` rows each when second != 0: the second one's tiles
// follow the first one's); nullptr when n is not a multiple of 32 or there is no memory for it
template <typename T> void* Engine::pack_matrix(const void* W, size_t rows, size_t n, size_t second)
{
    if (n % 32 != 0 || rows == 0) return nullptr;
    const size_t tiles = (rows + 15) / 16, per = tiles * 16 * n;
    void* P = dalloc((second ? 2 : 1) * per * sizeof(T));
    if (!P) { (void)hipGetLastError(); return nullptr; }
    for (int m = 0; m < (second ? 2 : 1); m++) {
        const size_t pieces = per * sizeof(T) / 16;
        const int grid = (int)std::min<size_t>((pieces + 255) / 256, 65535);
        hipLaunchKernelGGL(pack_tiles_kernel<T>, grid, 256, 0, stream, (const T*)W + m * second * n, (T*)P + m * per, (int)rows, (int)n);
    }
    return P;
}

template <typename T> void Engine::pack_all()
{
    const size_t dim = cfg.dim, hid = cfg.hidden_dim, hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads;
    packed.assign(layers.size(), LayerW<void>{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr});
    for (size_t l = 0; l < layers.size(); l++) {
        packed[l].wqkv = pack_matrix<T>(layers[l].wqkv, dim + 2 * kvd, dim);
        packed[l].wo = pack_matrix<T>(layers[l].wo, dim, dim);
        packed[l].w13 = pack_matrix<T>(layers[l].w13, hid, dim, hid);
        packed[l].w2 = pack_matrix<T>(layers[l].w2, dim, hid);
    }
    wclsP = pack_matrix<T>(wcls, cfg.vocab_size, dim);
    (void)hipStreamSynchronize(stream);
}

long Engine::load(const char* path)
{
    release();
    lastError.clear();
    FILE* f = fopen(path, "rb");
    if (!f) { lastError = "The model file could not be opened."; return MCH_ERROR_LLM_MISSING_MODEL_FILE; }
    // header (llama2_cpu.cpp:108-147): magic "ak42", version 1, Config, shared-classifier byte, 256 bytes in all
    uint32_t magic = 0;
    int version = 0;
    uint8_t shared = 0;
    bool ok = fread(&magic, 4, 1, f) == 1 && magic == 0x616b3432 && fread(&version, 4, 1, f) == 1 && version == 1 &&
              fread(&cfg, sizeof(Config), 1, f) == 1 && fread(&shared, 1, 1, f) == 1;
    if (!ok) {
        fclose(f);
        lastError = "Not a llama2.c version 1 checkpoint (magic 'ak42', version 1, seven-integer configuration).";
        return MCH_ERROR_LLM_LOAD_MODEL;
    }
    shared_classifier = shared;
    if (cfg.seq_len > 20480) cfg.seq_len = 20480;   // the reference clamps the context the same way (llama2_cpu.cpp:145)
    if (cfg.dim <= 0 || cfg.n_heads <= 0 || cfg.n_kv_heads <= 0 || cfg.n_layers <= 0 || cfg.vocab_size <= 0 || cfg.seq_len <= 0 ||
        cfg.hidden_dim <= 0 || cfg.dim % cfg.n_heads || cfg.n_heads % cfg.n_kv_heads || (cfg.dim / cfg.n_heads) % 4 ||
        cfg.dim / cfg.n_heads > 256 ||
        cfg.dim % 4 || cfg.hidden_dim % 4) {
        fclose(f);
        char msg[256];
        snprintf(msg, sizeof(msg), "Unsupported model shape: dim %d, hidden %d, layers %d, heads %d, kv heads %d, vocabulary %d, "
                 "context %d (dim and hidden must be multiples of 4, dim a multiple of heads, heads of kv heads, head size a multiple of 4 up to 256).",
                 cfg.dim, cfg.hidden_dim, cfg.n_layers, cfg.n_heads, cfg.n_kv_heads, cfg.vocab_size, cfg.seq_len);
        lastError = msg;
        return MCH_ERROR_LLM_LOAD_MODEL;
    }
    const size_t L = cfg.n_layers, dim = cfg.dim, hid = cfg.hidden_dim, hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads;
    size_t need = 2 * L * dim + dim + (size_t)cfg.vocab_size * dim + 2 * L * dim * dim + 2 * L * dim * kvd + 3 * L * dim * hid;
    if (!shared) need += (size_t)cfg.vocab_size * dim;
    fseek(f, 0, SEEK_END);
    long fsize = ftell(f);
    if (fsize < 0 || (size_t)fsize < 256 + need * 4) {
        fclose(f);
        lastError = "The model file is shorter than its configuration requires.";
        return MCH_ERROR_LLM_LOAD_MODEL;
    }
    fseek(f, 256, SEEK_SET);
    std::vector<float> blob(need);
    size_t got = fread(blob.data(), 4, need, f);
    fclose(f);
    if (got != need) { lastError = "The model file could not be read."; return MCH_ERROR_LLM_LOAD_MODEL; }

    HIPCHK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    stored_bf16 = bf16_weights;
    long e = stored_bf16 ? upload<bf16_t>(blob.data()) : upload<float>(blob.data());
    if (e) { release(); return e; }
    if (stored_bf16) pack_all<bf16_t>(); else pack_all<float>();
    // rotary tables as precompute_freqs_cis builds them (llama2_cpu.cpp:388-414)
    const int half = (int)hs / 2;
    std::vector<float> fr(half), hc((size_t)cfg.seq_len * half), hsn((size_t)cfg.seq_len * half);
    for (int i = 0; i < (int)hs; i += 2) {
        float v = i / (float)hs;
        float d = powf(10000.0f, v);
        fr[i / 2] = (d == 0.0) ? 0 : 1.0f / d;
    }
    for (size_t i = 0; i < (size_t)cfg.seq_len; i++)
        for (int j = 0; j < half; j++) {
            hc[i * half + j] = cosf(i * fr[j]);
            hsn[i * half + j] = sinf(i * fr[j]);
        }
    if (!(fcos = (float*)dalloc(hc.size() * 4)) || !(fsin = (float*)dalloc(hc.size() * 4))) { release(); return MCH_ERROR_MEMORY_OUT; }
    HIPCHK(hipMemcpy(fcos, hc.data(), hc.size() * 4, hipMemcpyHostToDevice));
    HIPCHK(hipMemcpy(fsin, hsn.data(), hc.size() * 4, hipMemcpyHostToDevice));
    loaded = true;
    return 0;
}

long Engine::ensure_state(int B, int nSteps)
{
    if (B == stateB && nSteps <= stateSteps) return 0;
    HIPCHK(hipStreamSynchronize(stream));
    if (graphExec) { (void)hipGraphExecDestroy(graphExec); graphExec = nullptr; }
    if (hLogits) { (void)hipHostFree(hLogits); hLogits = nullptr; hLogitsCount = 0; }
    if (hGiven) { (void)hipHostFree(hGiven); hGiven = nullptr; }
    for (void* p : stateAllocs) (void)hipFree(p);
    stateAllocs.clear();
    stateB = 0;
    const size_t dim = cfg.dim, hid = cfg.hidden_dim, hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads;
    auto sa = [&](size_t bytes) -> void* {
        void* p = nullptr;
        if (hipMalloc(&p, bytes ? bytes : 4) != hipSuccess) return nullptr;
        stateAllocs.push_back(p);
        return p;
    };
    const size_t cacheN = (size_t)cfg.n_layers * B * cfg.seq_len * kvd;
    wsBytes = attn_decode_workspace_bytes(B, cfg.n_heads, (int)hs, cfg.seq_len);
    x = (float*)sa(B * dim * 4);
    xb = (float*)sa(B * dim * 4);
    qkv = (float*)sa(B * (dim + 2 * kvd) * 4);
    qc = (float*)sa(B * dim * 4);
    hb = (float*)sa(B * hid * 4);
    logits = (float*)sa((size_t)B * cfg.vocab_size * 4);
    state_kv_bf16 = kv_bf16 && hs % 8 == 0;       // a 16-byte chunk of a bf16 row is 8 dims of one head
    kc = sa(cacheN * (state_kv_bf16 ? 2 : 4));
    vc = sa(cacheN * (state_kv_bf16 ? 2 : 4));
    ws = sa(wsBytes);
    dstate = (GenState*)sa(sizeof(GenState));
    dprompt = (int*)sa((size_t)B * cfg.seq_len * 4);
    dnext = (int*)sa(B * 4);
    dcur = (int*)sa(B * 4);
    dgiven = (int*)sa(B * 4);
    drng = (unsigned long long*)sa(8);
    dout = (int*)sa((size_t)B * cfg.seq_len * 4);
    dcount = (int*)sa(((size_t)B * cfg.n_heads + 1) * 4);
    if (!x || !xb || !qkv || !qc || !hb || !logits || !kc || !vc || !ws || !dstate || !dprompt || !dnext || !dcur || !dout || !dcount)
        return MCH_ERROR_MEMORY_OUT;
    dticket = dcount + (size_t)B * cfg.n_heads;
    HIPCHK(hipMemset(dcount, 0, ((size_t)B * cfg.n_heads + 1) * 4));
    stateB = B;
    stateSteps = cfg.seq_len;
    return 0;
}

template <int MODE, bool NORM, typename T>
static hipError_t launch_matvec_rows(hipStream_t s, const void* W, const float* x, const float* g, float* y, int rows, int n, int M, int ldy,
                                     const void* Wp = nullptr);

long Engine::ensure_prefill(size_t rows)
{
    if (rows <= pfRows) return 0;
    HIPCHK(hipStreamSynchronize(stream));
    for (void* p : prefillAllocs) (void)hipFree(p);
    prefillAllocs.clear();
    pfRows = 0;
    const size_t dim = cfg.dim, hid = cfg.hidden_dim, hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads, V = cfg.vocab_size;
    auto pa = [&](size_t floats) -> float* {
        void* p = nullptr;
        if (hipMalloc(&p, floats ? floats * 4 : 4) != hipSuccess) return nullptr;
        prefillAllocs.push_back(p);
        return (float*)p;
    };
    // the classifier runs over at most 512 MB of logits at a time
    pfLogitRows = std::max<size_t>(1, std::min(rows, ((size_t)128 << 20) / V));
    pfX = pa(rows * dim); pfXn = pa(rows * dim); pfQkv = pa(rows * (dim + 2 * kvd));
    pfQ = pa(rows * dim); pfK = pa(rows * dim); pfV = pa(rows * dim);
    pfH2 = pa(rows * 2 * hid); pfHb = pa(rows * hid); pfLogits = pa(pfLogitRows * V);
    // 16-bit weights: the GEMMs read their activations as pairs of bf16 rows (prefill_norm_split_kernel), 2 x 2 bytes a
    // value; widths that are no multiple of 64 widen one matrix at a time to fp32 instead and need room for the largest
    pfSplit = dim % 64 == 0 && hid % 64 == 0;
    pfW = !stored_bf16 ? pfX : pfSplit ? pa(rows * std::max(dim, hid)) : pa(std::max({(dim + 2 * kvd) * dim, 2 * hid * dim, V * dim}));
    if (!pfX || !pfXn || !pfQkv || !pfQ || !pfK || !pfV || !pfH2 || !pfHb || !pfLogits || !pfW) return MCH_ERROR_MEMORY_OUT;
    pfRows = rows;
    return 0;
}

// Positions 0 .. P-1 of all B sequences in one pass.  Leaves what P single-token steps leave: the caches of every
// layer filled up to P - 1, the id chosen after every position in dout, the id after the last one in dnext, and the
// generation state at position P.
template <typename T> long Engine::prefill(hipStream_t s, int B, int P, int nSteps, float* allLogits, int tail)
{
    const int dim = cfg.dim, hid = cfg.hidden_dim, H = cfg.n_heads, kvH = cfg.n_kv_heads, hs = dim / H, kvd = hs * kvH, V = cfg.vocab_size;
    const int ldq = dim + 2 * kvd;
    const size_t M = (size_t)B * P;
    long e = ensure_prefill(M);
    if (e) return e;
    const float scale = 1.0f / sqrtf((float)hs);
    auto grid_for = [](size_t items) { return (int)std::min<size_t>((items + 255) / 256, 8192); };
    hipLaunchKernelGGL(prefill_embed_kernel<T>, (int)M, 256, 0, s, dprompt, cfg.seq_len, P, (const T*)emb, pfX, dim);
    HIPCHK(hipGetLastError());
    // Few rows (one or two sequences' prompts): the fused mat-vec family on the matrix cores, all rows sharing one walk
    // over each matrix, norms / SwiGLU / residuals in its epilogues.  Many rows: 128 x 128-tile GEMMs.
    const bool skinny = M <= 256 && dim % 32 == 0 && hid % 32 == 0;
    enum { PF_F32, PF_WIDEN, PF_SPLIT, PF_ACT16 };
    const int mode = sizeof(T) == 4 ? PF_F32 : !pfSplit ? PF_WIDEN : (prefill_act16 && (hs == 64 || hs == 128)) ? PF_ACT16 : PF_SPLIT;
    for (int l = 0; l < cfg.n_layers; l++) {
        const LayerW<void>& w = layers[l];
        const LayerW<void>& wp = packed[l];
        const size_t cacheOfs = (size_t)l * B * cfg.seq_len * kvd * (state_kv_bf16 ? 2 : 4);
        void* kcl = (char*)kc + cacheOfs;
        void* vcl = (char*)vc + cacheOfs;
        // act16: the q / k / v head tensors (and with them the attention) in bf16
        auto rope_scatter = [&](bool act16) {
            const int g = grid_for(M * ldq / 2);
#define ROPE_SCATTER(TC, TQ) hipLaunchKernelGGL((prefill_rope_scatter_kernel<TC, TQ>), g, 256, 0, s, pfQkv, (TQ*)pfQ, (TQ*)pfK, (TQ*)pfV, (TC*)kcl, \
                                                (TC*)vcl, fcos, fsin, B, P, H, kvH, hs, cfg.seq_len)
            if (state_kv_bf16) { if (act16) ROPE_SCATTER(bf16_t, bf16_t); else ROPE_SCATTER(bf16_t, float); }
            else { if (act16) ROPE_SCATTER(float, bf16_t); else ROPE_SCATTER(float, float); }
#undef ROPE_SCATTER
            return hipGetLastError();
        };
        if (skinny) {
            HIPCHK((launch_matvec_rows<0, true, T>(s, w.wqkv, pfX, w.rms_att, pfQkv, ldq, dim, (int)M, ldq, wp.wqkv)));
            HIPCHK(rope_scatter(false));
            HIPCHK(k_attn_prefill(s, F32, pfQ, pfK, pfV, pfXn, B, H, P, P, hs, scale, nullptr, MASK_CAUSAL, nullptr, true));
            HIPCHK((launch_matvec_rows<1, false, T>(s, w.wo, pfXn, nullptr, pfX, dim, dim, (int)M, dim, wp.wo)));          // x += Wo att
            HIPCHK((launch_matvec_rows<2, true, T>(s, w.w13, pfX, w.rms_ffn, pfHb, hid, dim, (int)M, hid, wp.w13)));
            HIPCHK((launch_matvec_rows<1, false, T>(s, w.w2, pfHb, nullptr, pfX, dim, hid, (int)M, dim, wp.w2)));           // x += W2 hb
            continue;
        }
        if (mode == PF_F32 || mode == PF_WIDEN) {
            // fp32 weights - or 16-bit ones of a width the bf16 GEMM does not take, widened one matrix at a time - on
            // the fp32 MFMA GEMM
            auto wf = [&](const void* W, size_t n) -> const float* {
                if (mode == PF_F32) return (const float*)W;
                const hipError_t ce = k_convert(s, BF16, W, F32, pfW, n);
                if (ce != hipSuccess) e = (long)ce;
                return pfW;
            };
            HIPCHK(k_rmsnorm(s, F32, (int)M, dim, pfX, w.rms_att, pfXn, 1e-5f));
            HIPCHK(k_gemm(s, F32, false, true, (int)M, ldq, dim, 1.f, pfXn, wf(w.wqkv, (size_t)ldq * dim), 0.f, pfQkv));
            HIPCHK(rope_scatter(false));
            HIPCHK(k_attn_prefill(s, F32, pfQ, pfK, pfV, pfXn, B, H, P, P, hs, scale, nullptr, MASK_CAUSAL, nullptr, true));   // head-merged output
            HIPCHK(k_gemm(s, F32, false, true, (int)M, dim, dim, 1.f, pfXn, wf(w.wo, (size_t)dim * dim), 1.f, pfX));          // x += Wo att
            HIPCHK(k_rmsnorm(s, F32, (int)M, dim, pfX, w.rms_ffn, pfXn, 1e-5f));
            HIPCHK(k_gemm(s, F32, false, true, (int)M, 2 * hid, dim, 1.f, pfXn, wf(w.w13, (size_t)2 * hid * dim), 0.f, pfH2));
            hipLaunchKernelGGL(prefill_swiglu_kernel, grid_for(M * hid), 256, 0, s, pfH2, pfHb, M, hid);
            HIPCHK(hipGetLastError());
            HIPCHK(k_gemm(s, F32, false, true, (int)M, dim, hid, 1.f, pfHb, wf(w.w2, (size_t)dim * hid), 1.f, pfX));          // x += W2 hb
            if (e) return e;
            continue;
        }
        // 16-bit weights on the bf16 MFMA GEMM, fp32 results and residual stream.  PF_SPLIT: every activation goes in
        // as two bf16 numbers (k_gemm_bf16_f32, split), attention in fp32.  PF_ACT16: activations rounded to bf16, q / k /
        // v and the attention in bf16, whose head-merged output is the next GEMM's operand as it is.
        const bool split = mode == PF_SPLIT;
        bf16_t* a16 = (bf16_t*)pfW;
        auto norm16 = [&](const float* x, const float* g, int k) {
            if (split) hipLaunchKernelGGL(prefill_norm_split_kernel<true>, (int)M, 256, 0, s, x, g, a16, k, 1e-5f);
            else hipLaunchKernelGGL(prefill_norm_split_kernel<false>, (int)M, 256, 0, s, x, g, a16, k, 1e-5f);
            return hipGetLastError();
        };
        HIPCHK(norm16(pfX, w.rms_att, dim));
        // rotation, head tensors and cache rows leave the QKV product's epilogue
        HIPCHK(k_gemm_bf16_qkv_rope(s, B, P, H, kvH, hs, dim, a16, split, w.wqkv, pfQ, pfK, pfV, !split, kcl, vcl, state_kv_bf16, cfg.seq_len,
                                    fcos, fsin));
        if (split) {
            HIPCHK(k_attn_prefill(s, F32, pfQ, pfK, pfV, pfXn, B, H, P, P, hs, scale, nullptr, MASK_CAUSAL, nullptr, true));
            HIPCHK(norm16(pfXn, nullptr, dim));
        } else {
            HIPCHK(k_attn_prefill(s, BF16, pfQ, pfK, pfV, a16, B, H, P, P, hs, scale, nullptr, MASK_CAUSAL, nullptr, true));
        }
        HIPCHK(k_gemm_bf16_f32(s, (int)M, dim, dim, 1.f, a16, split, w.wo, 1.f, pfX));                               // x += Wo att
        HIPCHK(norm16(pfX, w.rms_ffn, dim));
        // silu(w1 x) (w3 x) leaves the W1 | W3 product's epilogue in the operand form of the next product
        HIPCHK(k_gemm_bf16_swiglu(s, (int)M, hid, dim, a16, split, w.w13, pfH2, split));
        HIPCHK(k_gemm_bf16_f32(s, (int)M, dim, hid, 1.f, pfH2, split, w.w2, 1.f, pfX));                              // x += W2 hb
    }
    // The classifier has 250 tiles of 128 x 128 per 128 rows, enough for the tiled GEMM even where the layers' matrices
    // are not: the mat-vec family keeps it only for a handful of rows.
    const bool clsGemm = !skinny || M >= 64;
    const bool cls16 = mode == PF_SPLIT || mode == PF_ACT16;
    const int a16Row = mode == PF_SPLIT ? 2 * dim : dim;
    if (clsGemm) {
        if (!cls16) {
            HIPCHK(k_rmsnorm(s, F32, (int)M, dim, pfX, rms_final, pfXn, 1e-5f));
            if (mode == PF_WIDEN) HIPCHK(k_convert(s, BF16, wcls, F32, pfW, (size_t)V * dim));
        } else {
            if (mode == PF_SPLIT) hipLaunchKernelGGL(prefill_norm_split_kernel<true>, (int)M, 256, 0, s, pfX, rms_final, (bf16_t*)pfW, dim, 1e-5f);
            else hipLaunchKernelGGL(prefill_norm_split_kernel<false>, (int)M, 256, 0, s, pfX, rms_final, (bf16_t*)pfW, dim, 1e-5f);
            HIPCHK(hipGetLastError());
        }
    }
    for (size_t r0 = 0; r0 < M; r0 += pfLogitRows) {
        const int rows = (int)std::min(pfLogitRows, M - r0);
        if (!clsGemm) HIPCHK((launch_matvec_rows<0, true, T>(s, wcls, pfX + r0 * dim, rms_final, pfLogits, V, dim, rows, V, wclsP)));
        else if (!cls16) HIPCHK(k_gemm(s, F32, false, true, rows, V, dim, 1.f, pfXn + r0 * dim, mode == PF_F32 ? wcls : (const void*)pfW, 0.f, pfLogits));
        else HIPCHK(k_gemm_bf16_f32(s, rows, V, dim, 1.f, (bf16_t*)pfW + r0 * a16Row, mode == PF_SPLIT, wcls, 0.f, pfLogits));
        if (tail != 2) {
            hipLaunchKernelGGL(prefill_argmax_kernel, rows, 256, 0, s, pfLogits, V, (int)r0, P, cfg.seq_len, dout, dnext);
            HIPCHK(hipGetLastError());
        }
        if (allLogits) {
            // rows of one sequence are contiguous on both sides: [b][nSteps][V] <- [b*P + p][V]
            for (size_t m = r0; m < r0 + rows;) {
                const size_t b = m / P, p = m - b * P;
                const size_t n = std::min<size_t>(P - p, r0 + rows - m);
                HIPCHK(hipMemcpyAsync(allLogits + ((size_t)b * nSteps + p) * V, pfLogits + (m - r0) * V, n * V * sizeof(float),
                                      hipMemcpyDeviceToDevice, s));
                m += n;
            }
        }
        if (tail == 2) {
            // the ids of a sampled generation: every row's own draw of the random stream (the logits become probabilities)
            HIPCHK(sample_attr());
            hipLaunchKernelGGL(sample_device_kernel, rows, 1024, SAMPLE_MAX_VOCAB * 4, s, pfLogits, V, sampleTemperature, sampleTopp,
                               (const unsigned long long*)drng, (int*)nullptr, (int)r0, P, B, cfg.seq_len, dout, dnext);
            HIPCHK(hipGetLastError());
        }
    }
    if (tail == 2) {
        hipLaunchKernelGGL(rng_advance_kernel, 1, 1, 0, s, drng, B * P);
        HIPCHK(hipGetLastError());
    }
    GenState st = {P, 0, P + 1, 0};
    st.n_prompt = hostNPrompt;
    HIPCHK(hipMemcpyAsync(dstate, &st, sizeof(st), hipMemcpyHostToDevice, s));
    HIPCHK(hipStreamSynchronize(s));   // `st` lives on this stack frame
    return 0;
}

template <int MODE, bool NORM, typename T>
static hipError_t launch_matvec(hipStream_t s, const void* W, const float* x, const float* g, float* y, int rows, int n, int B,
                                int ldy, int rowsPerWave, const void* Wp = nullptr)
{
    if (B >= 2 && n % 32 == 0) {
        // batched: matrix-core kernel, 16 sequences per pass over the weights
        const int ns = rows >= 8192 ? 4 : 8;   // fewer, longer wavefronts once the rows alone fill the chip
        // every group of 16 sequences walks the weights in the same launch
        const int nGroups = (B + 15) / 16, tiles8 = ((rows + 15) / 16 + 7) / 8;
        // Wp: the tile-packed copy of W, when the engine holds one
        if (Wp) {
            if (ns == 4) hipLaunchKernelGGL((matvec_mfma_kernel<T, MODE, NORM, 1, 4, true>), tiles8 * 8 * nGroups, 256, 0, s, (const T*)Wp, x, g, y, rows, n, B, ldy, nGroups);
            else hipLaunchKernelGGL((matvec_mfma_kernel<T, MODE, NORM, 1, 8, true>), tiles8 * 8 * nGroups, 512, 0, s, (const T*)Wp, x, g, y, rows, n, B, ldy, nGroups);
        } else if (ns == 4) hipLaunchKernelGGL((matvec_mfma_kernel<T, MODE, NORM, 1, 4>), tiles8 * 8 * nGroups, 256, 0, s, (const T*)W, x, g, y, rows, n, B, ldy, nGroups);
        else hipLaunchKernelGGL((matvec_mfma_kernel<T, MODE, NORM, 1, 8>), tiles8 * 8 * nGroups, 512, 0, s, (const T*)W, x, g, y, rows, n, B, ldy, nGroups);
        return hipGetLastError();
    }
    // one row per wavefront fills the chip for the layer matrices; the classifier has rows to spare
    const bool two = rowsPerWave ? rowsPerWave == 2 : rows >= 16384;
    const int waves = two ? (rows + 1) / 2 : rows;
    const int grid = (waves + 3) / 4;
    const bool wide = sizeof(T) == 2 && n % 8 == 0 && (((uintptr_t)W) & 15) == 0;
    const int ch = wide ? 2 * ((n / 8 + 63) / 64) : (n / 4 + 63) / 64;
#define MV1(C, WIDE_)                                                                                                      \
    do {                                                                                                                   \
        if (two) hipLaunchKernelGGL((matvec_kernel<T, MODE, NORM, C, 2, WIDE_>), grid, 256, 0, s, (const T*)W, x, g, y, rows, n, B, ldy); \
        else hipLaunchKernelGGL((matvec_kernel<T, MODE, NORM, C, 1, WIDE_>), grid, 256, 0, s, (const T*)W, x, g, y, rows, n, B, ldy);     \
    } while (0)
#define MV(C)                                                                                                              \
    do {                                                                                                                   \
        if constexpr (sizeof(T) == 2 && (C) % 2 == 0) {                                                                    \
            if (wide) { MV1(C, true); break; }                                                                             \
        }                                                                                                                  \
        MV1(C, false);                                                                                                     \
    } while (0)
    if (ch <= 2) MV(2);
    else if (ch <= 3 && !wide) MV(3);
    else if (ch <= 4) MV(4);
    else if (ch <= 8) MV(8);
    else if (ch <= 16) MV(16);
    else hipLaunchKernelGGL((matvec_loop_kernel<T, MODE, NORM>), (rows + 3) / 4, 256, 0, s, (const T*)W, x, g, y, rows, n, B, ldy);
#undef MV1
#undef MV
    return hipGetLastError();
}

constexpr int kMergeSplits = 16;   // split partials a thread of matvec_merge_kernel holds in flight
// whether the output projection can merge the attention's splits itself: one float4 of the merged vector per thread
static bool matvec_merge_usable(int n, int hs, int splits)
{
    return n % 4 == 0 && n <= 1024 && hs % 4 == 0 && splits >= 1 && splits <= kMergeSplits;
}
template <typename T>
static hipError_t launch_matvec_merge(hipStream_t s, const void* W, const float* part, int splits, int rowsPerSplit, const int* dlen,
                                      int H, int hs, float* y, int rows, int n)
{
    if (!matvec_merge_usable(n, hs, splits)) return hipErrorInvalidValue;
    const float* partML = part + (size_t)splits * n;
    const int grid = (rows + 3) / 4;
    const bool wide = sizeof(T) == 2 && n % 8 == 0 && (((uintptr_t)W) & 15) == 0;
    const int ch = wide ? 2 * ((n / 8 + 63) / 64) : (n / 4 + 63) / 64;
#define MVM(C, WIDE_) hipLaunchKernelGGL((matvec_merge_kernel<T, C, WIDE_, kMergeSplits>), grid, 256, 0, s, (const T*)W, part, partML, dlen, splits, rowsPerSplit, H, hs, y, rows, n)
    if constexpr (sizeof(T) == 2) {
        if (wide) {
            if (ch <= 2) MVM(2, true); else MVM(4, true);
            return hipGetLastError();
        }
    }
    if (ch <= 2) MVM(2, false);
    else if (ch <= 3) MVM(3, false);
    else MVM(4, false);
#undef MVM
    return hipGetLastError();
}

// The same kernels over the M rows of a prompt pass (row = one position of one sequence): up to 128 rows share one walk
// over the weights, so a single sequence's prompt streams every matrix once (or a few times) instead of going through
// 128 x 128 GEMM tiles that would leave most of the chip idle at this height.
template <int MODE, bool NORM, typename T>
static hipError_t launch_matvec_rows(hipStream_t s, const void* W, const float* x, const float* g, float* y, int rows, int n, int M, int ldy,
                                     const void* Wp)
{
    const int tiles8 = ((rows + 15) / 16 + 7) / 8;
    // two groups of 16 rows per workgroup: half the weight traffic from L2 of one group, and still more workgroups than CUs
#define MVG(G_, PK_, W_) hipLaunchKernelGGL((matvec_mfma_kernel<T, MODE, NORM, G_, 8, PK_>), tiles8 * 8 * ((M + 16 * G_ - 1) / (16 * G_)), 512, 0, s, (const T*)(W_), x, g, y, rows, n, M, ldy, (M + 16 * G_ - 1) / (16 * G_))
    if (Wp) { if (M > 16) MVG(2, true, Wp); else MVG(1, true, Wp); }
    else if (M > 16) MVG(2, false, W); else MVG(1, false, W);
#undef MVG
    return hipGetLastError();
}

// x = embedding of the token at the starting position; later steps get theirs from the previous step's tail kernel
hipError_t Engine::embed_first(hipStream_t s, int B)
{
    if (stored_bf16)
        hipLaunchKernelGGL(embed_step_kernel<bf16_t>, B, 256, 0, s, dstate, dprompt, cfg.seq_len, dnext, (const bf16_t*)emb, x, cfg.dim, dcur);
    else
        hipLaunchKernelGGL(embed_step_kernel<float>, B, 256, 0, s, dstate, dprompt, cfg.seq_len, dnext, (const float*)emb, x, cfg.dim, dcur);
    return hipGetLastError();
}

// enqueue one decode step for B sequences at the device-side position
template <typename T> long Engine::step(hipStream_t s, int B, int nSteps, float* allLogits, StepProfile* prof, int tail)
{
    const int dim = cfg.dim, hid = cfg.hidden_dim, hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads, V = cfg.vocab_size;
    const int ldq = dim + 2 * kvd;
#define SPAN_BEGIN(cls) do { if (prof) HIPCHK(prof->begin(cls, s)); } while (0)
#define SPAN_END() do { if (prof) HIPCHK(prof->end(s)); } while (0)
    const float scale = 1.0f / sqrtf((float)hs);
    // batch 1 with the cache in one iteration of rows per split: the attention leaves its splits to the output projection
    int deferRows = 0;
    int deferSplits = defer_merge ? attn_decode_fused_deferred_splits(B, cfg.n_heads, hs, cfg.seq_len, state_kv_bf16 ? BF16 : F32, &deferRows) : 0;
    if (!matvec_merge_usable(dim, hs, deferSplits)) deferSplits = 0;
    for (int l = 0; l < cfg.n_layers; l++) {
        const LayerW<void>& w = layers[l];
        const LayerW<void>& wp = packed[l];
        const size_t cacheOfs = (size_t)l * B * cfg.seq_len * kvd * (state_kv_bf16 ? 2 : 4);
        void* kcl = (char*)kc + cacheOfs;
        void* vcl = (char*)vc + cacheOfs;
        // qkv = [Wq;Wk;Wv] rmsnorm(x)
        SPAN_BEGIN(SC_MATVEC_QKV);
        HIPCHK((launch_matvec<0, true, T>(s, w.wqkv, x, w.rms_att, qkv, ldq, dim, B, ldq, mvRows, wp.wqkv)));
        SPAN_END();
        // xb = attention(rope(q), cache[0..pos] with rope(k), v appended)
        SPAN_BEGIN(SC_ATTN_DECODE);
        HIPCHK(k_attn_decode_fused(s, qkv, kcl, vcl, state_kv_bf16 ? BF16 : F32, xb, B, cfg.n_heads, cfg.n_kv_heads, hs, cfg.seq_len, scale, fcos, fsin,
                                   &dstate->len, ws, wsBytes, dcount, deferSplits > 0));
        SPAN_END();
        // x += Wo xb (with the merge of the attention's splits in front when it was left to this kernel)
        SPAN_BEGIN(SC_MATVEC_WO);
        if (deferSplits > 0) HIPCHK((launch_matvec_merge<T>(s, w.wo, (const float*)ws, deferSplits, deferRows, &dstate->len, cfg.n_heads, hs, x, dim, dim)));
        else HIPCHK((launch_matvec<1, false, T>(s, w.wo, xb, nullptr, x, dim, dim, B, dim, mvRows, wp.wo)));
        SPAN_END();
        // hb = silu(W1 rmsnorm(x)) * (W3 rmsnorm(x))
        SPAN_BEGIN(SC_MATVEC_W13);
        HIPCHK((launch_matvec<2, true, T>(s, w.w13, x, w.rms_ffn, hb, hid, dim, B, hid, mvRows, wp.w13)));
        SPAN_END();
        // x += W2 hb
        SPAN_BEGIN(SC_MATVEC_W2);
        HIPCHK((launch_matvec<1, false, T>(s, w.w2, hb, nullptr, x, dim, hid, B, dim, mvRows, wp.w2)));
        SPAN_END();
    }
    // logits = Wcls rmsnorm(x)
    SPAN_BEGIN(SC_MATVEC_CLS);
    HIPCHK((launch_matvec<0, true, T>(s, wcls, x, rms_final, logits, V, dim, B, V, mvRows, wclsP)));
    SPAN_END();
    if (allLogits) {
        hipLaunchKernelGGL(save_logits_kernel, dim3((V + 255) / 256 > 64 ? 64 : (V + 255) / 256, B), 256, 0, s, logits, allLogits,
                           dstate, V, nSteps);
        HIPCHK(hipGetLastError());
    }
    if (tail == 1) {
        SPAN_BEGIN(SC_SAMPLE);
        hipLaunchKernelGGL(sample_advance_kernel<T>, B, 1024, 0, s, logits, V, dstate, dticket, dprompt, cfg.seq_len, dnext, dout,
                           (const T*)emb, x, dim, dcur, (const int*)nullptr, (unsigned long long*)nullptr);
        HIPCHK(hipGetLastError());
        SPAN_END();
    } else if (tail == 2) {
        SPAN_BEGIN(SC_SAMPLE);
        HIPCHK(sample_attr());
        hipLaunchKernelGGL(sample_device_kernel, B, 1024, SAMPLE_MAX_VOCAB * 4, s, logits, V, sampleTemperature, sampleTopp,
                           (const unsigned long long*)drng, dgiven, 0, 0, 0, 0, (int*)nullptr, (int*)nullptr);
        HIPCHK(hipGetLastError());
        hipLaunchKernelGGL(sample_advance_kernel<T>, B, 1024, 0, s, logits, V, dstate, dticket, dprompt, cfg.seq_len, dnext, dout,
                           (const T*)emb, x, dim, dcur, (const int*)dgiven, drng);
        HIPCHK(hipGetLastError());
        SPAN_END();
    }
#undef SPAN_BEGIN
#undef SPAN_END
    return 0;
}

// One call of the sampler on the device over n logits given on the host (the SAMPLE entry): the kernel of the decode
// steps, the handle's random stream, one draw.  The logits come back as probabilities, as the host sampler leaves them.
long Engine::sample_device(float* lg, int n, HostSampler* sampler, int* id)
{
    if (n < 1 || n > SAMPLE_MAX_VOCAB) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    struct Dev {
        void* p = nullptr;
        ~Dev() { if (p) (void)hipFree(p); }
    } d;
    HIPCHK(hipMalloc(&d.p, (size_t)n * 4 + 16));
    float* dl = (float*)d.p;
    unsigned long long* dr = (unsigned long long*)(dl + n + (n & 1));
    int* dg = (int*)(dr + 1);
    hipStream_t s = stream;
    HIPCHK(hipMemcpyAsync(dl, lg, (size_t)n * 4, hipMemcpyHostToDevice, s));
    HIPCHK(hipMemcpyAsync(dr, &sampler->state, 8, hipMemcpyHostToDevice, s));
    HIPCHK(sample_attr());
    hipLaunchKernelGGL(sample_device_kernel, 1, 1024, SAMPLE_MAX_VOCAB * 4, s, dl, n, sampler->temperature, sampler->topp,
                       (const unsigned long long*)dr, dg, 0, 0, 0, 0, (int*)nullptr, (int*)nullptr);
    HIPCHK(hipGetLastError());
    HIPCHK(hipMemcpyAsync(lg, dl, (size_t)n * 4, hipMemcpyDeviceToHost, s));
    HIPCHK(hipMemcpyAsync(id, dg, 4, hipMemcpyDeviceToHost, s));
    HIPCHK(hipStreamSynchronize(s));
    (void)sampler->random_u32();   // the draw the kernel took
    return 0;
}

long Engine::running_sum_device(const float* values, int n, float threshold, int* out2)
{
    if (n < 1 || n > SAMPLE_MAX_VOCAB) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    struct Dev {
        void* p = nullptr;
        ~Dev() { if (p) (void)hipFree(p); }
    } d;
    HIPCHK(hipMalloc(&d.p, (size_t)n * 4 + 8));
    float* dv = (float*)d.p;
    int* dout2 = (int*)(dv + n);
    hipStream_t s = stream;
    HIPCHK(hipMemcpyAsync(dv, values, (size_t)n * 4, hipMemcpyHostToDevice, s));
    static bool attr = false;
    if (!attr) {
        HIPCHK(hipFuncSetAttribute((const void*)running_sum_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SAMPLE_MAX_VOCAB * 4));
        attr = true;
    }
    hipLaunchKernelGGL(running_sum_kernel, 1, 1024, SAMPLE_MAX_VOCAB * 4, s, (const float*)dv, n, threshold, dout2);
    HIPCHK(hipGetLastError());
    HIPCHK(hipMemcpyAsync(out2, dout2, 8, hipMemcpyDeviceToHost, s));
    HIPCHK(hipStreamSynchronize(s));
    return 0;
}

// tail of a step whose ids were chosen on the host (dgiven): record, embed the next token, advance the position
template <typename T> long Engine::advance_given(hipStream_t s, int B)
{
    hipLaunchKernelGGL(sample_advance_kernel<T>, B, 1024, 0, s, logits, cfg.vocab_size, dstate, dticket, dprompt, cfg.seq_len, dnext,
                       dout, (const T*)emb, x, cfg.dim, dcur, (const int*)dgiven, (unsigned long long*)nullptr);
    HIPCHK(hipGetLastError());
    return 0;
}

__global__ void noop_kernel() {}

// Runs `reps` eager decode steps of one sequence starting at position `pos` (the cache
// content before `pos` is whatever earlier generations left; only timing matters here) and
// returns, per kernel class: {milliseconds per step, launches per step, algorithmic bytes per step}, followed by one
// more value: the median milliseconds an event pair measures around an empty kernel (dispatch + event cost that
// every pair above includes).
long Engine::profile_step(int pos, int reps, int B, std::vector<float>* out)
{
    if (!loaded) return MCH_ERROR_LLM_GENERATE;
    if (reps < 1 || pos < 0 || pos + reps > cfg.seq_len || B < 1 || B > 64) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    long e = ensure_state(B, cfg.seq_len);
    if (e) return e;
    hipStream_t s = stream;
    std::vector<int> hp((size_t)B * cfg.seq_len, 1);
    HIPCHK(hipMemcpyAsync(dprompt, hp.data(), hp.size() * 4, hipMemcpyHostToDevice, s));
    GenState st0 = {pos, cfg.seq_len, pos + 1, 0};
    HIPCHK(hipMemcpyAsync(dstate, &st0, sizeof(st0), hipMemcpyHostToDevice, s));
    HIPCHK(hipStreamSynchronize(s));
    HIPCHK(embed_first(s, B));
    std::vector<float> empty;
    {
        StepProfile cal;
        for (int i = 0; i < 33; i++) {
            HIPCHK(cal.begin(0, s));
            hipLaunchKernelGGL(noop_kernel, 1, 64, 0, s);
            HIPCHK(cal.end(s));
        }
        HIPCHK(hipStreamSynchronize(s));
        for (auto& sp : cal.spans) {
            float t = 0.f;
            if (hipEventElapsedTime(&t, sp.second.first, sp.second.second) == hipSuccess) empty.push_back(t);
            (void)hipEventDestroy(sp.second.first);
            (void)hipEventDestroy(sp.second.second);
        }
        std::sort(empty.begin(), empty.end());
    }
    StepProfile prof;
    for (int i = 0; i < reps && !e; i++) e = stored_bf16 ? step<bf16_t>(s, B, cfg.seq_len, nullptr, &prof) : step<float>(s, B, cfg.seq_len, nullptr, &prof);
    hipError_t he = hipStreamSynchronize(s);
    if (!e && he != hipSuccess) e = (long)he;
    std::vector<double> ms(SC_COUNT, 0.0), cnt(SC_COUNT, 0.0);
    for (auto& sp : prof.spans) {
        float t = 0.f;
        if (!e && hipEventElapsedTime(&t, sp.second.first, sp.second.second) == hipSuccess) { ms[sp.first] += t; cnt[sp.first] += 1; }
        (void)hipEventDestroy(sp.second.first);
        (void)hipEventDestroy(sp.second.second);
    }
    if (e) return e;
    const double es = stored_bf16 ? 2.0 : 4.0;
    const double L = cfg.n_layers, dim = cfg.dim, hid = cfg.hidden_dim, hs = dim / cfg.n_heads, kvd = hs * cfg.n_kv_heads;
    const double meanLen = pos + 1 + (reps - 1) / 2.0;
    double bytes[SC_COUNT] = {0};
    bytes[SC_MATVEC_QKV] = L * (dim + 2 * kvd) * dim * es;
    bytes[SC_MATVEC_WO] = L * dim * dim * es;
    bytes[SC_MATVEC_W13] = L * 2 * hid * dim * es;
    bytes[SC_MATVEC_W2] = L * dim * hid * es;
    bytes[SC_MATVEC_CLS] = (double)cfg.vocab_size * dim * es;
    bytes[SC_ATTN_DECODE] = B * L * 2 * meanLen * kvd * 4.0;
    out->clear();
    for (int c = 0; c < SC_COUNT; c++) {
        out->push_back((float)(ms[c] / reps));
        out->push_back((float)(cnt[c] / reps));
        out->push_back((float)bytes[c]);
    }
    out->push_back(empty.empty() ? 0.f : empty[empty.size() / 2]);
    return 0;
}

long Engine::generate(const int* prompts, int B, int nPrompt, int nSteps, bool wantLogits, std::vector<int>* ids,
                      std::vector<float>* outLogits, std::atomic<bool>* cancel, int chunk,
                      const std::function<bool(const int*, int, int)>& onChunk, HostSampler* sampler)
{
    if (!loaded) return MCH_ERROR_LLM_GENERATE;
    if (B < 1 || B > 64 || nSteps < 1 || nSteps > cfg.seq_len || nPrompt < 1 || nPrompt > cfg.seq_len) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    for (int i = 0; i < B * nPrompt; i++)
        if (prompts[i] < 0 || prompts[i] >= cfg.vocab_size) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    long e = ensure_state(B, nSteps);
    if (e) return e;
    hostNPrompt = nPrompt;
    hipStream_t s = stream;
    std::vector<int> hp((size_t)B * cfg.seq_len, 0);
    for (int b = 0; b < B; b++) memcpy(&hp[(size_t)b * cfg.seq_len], prompts + (size_t)b * nPrompt, nPrompt * sizeof(int));
    HIPCHK(hipMemcpyAsync(dprompt, hp.data(), hp.size() * 4, hipMemcpyHostToDevice, s));
    GenState st0 = {0, nPrompt, 1, 0};
    HIPCHK(hipMemcpyAsync(dstate, &st0, sizeof(st0), hipMemcpyHostToDevice, s));
    HIPCHK(hipStreamSynchronize(s));
    // owned here so that every early return below releases them
    struct Scratch {
        float* allLogits = nullptr;
        hipEvent_t evA = nullptr, evB = nullptr, evP0 = nullptr, evP1 = nullptr;
        ~Scratch()
        {
            if (allLogits) (void)hipFree(allLogits);
            for (hipEvent_t ev : {evA, evB, evP0, evP1})
                if (ev) (void)hipEventDestroy(ev);
        }
    } sc;
    if (wantLogits) {
        HIPCHK(hipMalloc((void**)&sc.allLogits, (size_t)B * nSteps * cfg.vocab_size * 4));
    }
    float* const allLogits = sc.allLogits;
    // With a sampler whose temperature is not 0 the id of every step is chosen on the host, as in the reference: the
    // step's kernels stop at the logits, which are copied out, sampled, and the chosen id goes back for the step's tail.
    const bool sampled = sampler && !sampler->greedy();
    const bool devSample = sampled && device_sampling && cfg.vocab_size <= SAMPLE_MAX_VOCAB, hostSample = sampled && !devSample;
    const int tail = hostSample ? 0 : devSample ? 2 : 1;
    if (devSample) {
        sampleTemperature = sampler->temperature;
        sampleTopp = sampler->topp;
        HIPCHK(hipMemcpyAsync(drng, &sampler->state, 8, hipMemcpyHostToDevice, stream));
        HIPCHK(hipStreamSynchronize(stream));
    }
    const size_t V = (size_t)cfg.vocab_size;
    if (hostSample) {
        if (hLogitsCount < (size_t)B * V) {
            if (hLogits) (void)hipHostFree(hLogits);
            hLogits = nullptr;
            HIPCHK(hipHostMalloc((void**)&hLogits, (size_t)B * V * sizeof(float), hipHostMallocDefault));
            hLogitsCount = (size_t)B * V;
        }
        if (!hGiven) HIPCHK(hipHostMalloc((void**)&hGiven, 64 * sizeof(int), hipHostMallocDefault));
    }
    auto enqueue = [&]() -> long {
        return stored_bf16 ? step<bf16_t>(s, B, nSteps, allLogits, nullptr, tail)
                            : step<float>(s, B, nSteps, allLogits, nullptr, tail);
    };
    HIPCHK(hipEventCreate(&sc.evA));
    HIPCHK(hipEventCreate(&sc.evB));
    const hipEvent_t evA = sc.evA, evB = sc.evB;
    const int t0 = timedFrom < 0 ? nPrompt : timedFrom;
    bool graph = use_graph && !wantLogits;
    if (graph && (!graphExec || graphB != B || graphTail != tail || (tail == 2 && (graphTemperature != sampleTemperature || graphTopp != sampleTopp)))) {
        // one decode step, captured once; position / tokens are device-side so the graph is replayed as is
        if (graphExec) { (void)hipGraphExecDestroy(graphExec); graphExec = nullptr; }
        hipGraph_t g = nullptr;
        hipError_t he = hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal);
        if (he == hipSuccess) {
            e = enqueue();
            he = hipStreamEndCapture(s, &g);
            if (e == 0 && he == hipSuccess) he = hipGraphInstantiate(&graphExec, g, nullptr, nullptr, 0);
            if (g) (void)hipGraphDestroy(g);
        }
        if (e || he != hipSuccess || !graphExec) { graphExec = nullptr; graph = false; e = 0; }
        graphB = B;
        graphTail = tail;
        graphTemperature = sampleTemperature;
        graphTopp = sampleTopp;
    }
    lastUsedGraph = graph;
    // The forced prompt positions in one batched pass.  The reference flips a coin at every position, forced ones
    // included: the device sampler gives every row of the pass the draw its position would have had.  Ids chosen on
    // the host need every position's logits in turn, so that kind of generation keeps the one-step-per-position loop.
    const int nPre = std::min(nPrompt, nSteps);
    const bool batched = use_prefill && !hostSample && nPre >= 2;
    const int start = batched ? nPre : 0;
    lastPrefillMs = 0.f;
    lastPrefillRows = 0;
    bool timing = false;
    if (t0 < start) { (void)hipEventRecord(evA, s); timing = true; }
    if (batched) {
        e = ensure_prefill((size_t)B * nPre);      // allocations stay out of the timed pass
        if (e) return e;
        HIPCHK(hipEventCreate(&sc.evP0));
        HIPCHK(hipEventCreate(&sc.evP1));
        HIPCHK(hipEventRecord(sc.evP0, s));
        e = stored_bf16 ? prefill<bf16_t>(s, B, nPre, nSteps, allLogits, tail) : prefill<float>(s, B, nPre, nSteps, allLogits, tail);
        if (e) return e;
        HIPCHK(hipEventRecord(sc.evP1, s));
        HIPCHK(hipEventSynchronize(sc.evP1));
        (void)hipEventElapsedTime(&lastPrefillMs, sc.evP0, sc.evP1);
        lastPrefillRows = B * nPre;
    }
    HIPCHK(embed_first(s, B));
    int done = start, reported = 0;
    // hands the ids of sequence 0 chosen at positions [reported, done) to the caller, who may stop the generation
    auto report = [&]() -> int {
        std::vector<int> part((size_t)done);
        hipError_t hc = hipStreamSynchronize(s);
        if (hc == hipSuccess) hc = hipMemcpy(part.data(), dout, part.size() * 4, hipMemcpyDeviceToHost);
        if (hc != hipSuccess) { e = (long)hc; return -1; }
        const bool go = onChunk(part.data(), reported, done);
        reported = done;
        return go ? 1 : 0;
    };
    bool stop = false;
    if (onChunk && chunk > 0 && done > 0) stop = report() != 1;
    for (int i = start; i < nSteps && !e && !stop; i++) {
        if (i == t0 && !timing) { (void)hipEventRecord(evA, s); timing = true; }
        if (graph) {
            hipError_t he = hipGraphLaunch(graphExec, s);
            if (he != hipSuccess) e = (long)he;
        } else e = enqueue();
        if (hostSample && !e) {
            hipError_t hc = hipMemcpyAsync(hLogits, logits, (size_t)B * V * sizeof(float), hipMemcpyDeviceToHost, s);
            if (hc == hipSuccess) hc = hipStreamSynchronize(s);
            if (hc != hipSuccess) { e = (long)hc; break; }
            for (int b = 0; b < B; b++) hGiven[b] = sampler->sample(hLogits + (size_t)b * V, (int)V);
            hc = hipMemcpyAsync(dgiven, hGiven, (size_t)B * sizeof(int), hipMemcpyHostToDevice, s);
            if (hc != hipSuccess) { e = (long)hc; break; }
            e = stored_bf16 ? advance_given<bf16_t>(s, B) : advance_given<float>(s, B);
            if (e) break;
        }
        done++;
        if (cancel && (i & 15) == 15 && cancel->load()) break;
        if (onChunk && chunk > 0 && (done - reported >= chunk || done == nSteps)) stop = report() != 1;
    }
    (void)hipEventRecord(evB, s);
    hipError_t he = hipStreamSynchronize(s);
    if (!e && he != hipSuccess) e = (long)he;
    if (!e && devSample) {
        // the host sampler carries the random stream from one generation to the next
        he = hipMemcpy(&sampler->state, drng, 8, hipMemcpyDeviceToHost);
        if (he != hipSuccess) e = (long)he;
    }
    lastTimedMs = 0.f;
    lastTimedSteps = 0;
    if (!e && done > t0 && t0 >= 0 && timing) {
        (void)hipEventElapsedTime(&lastTimedMs, evA, evB);
        lastTimedSteps = done - t0;
    }
    if (!e) {
        ids->assign((size_t)B * nSteps, 0);
        std::vector<int> tmp((size_t)B * cfg.seq_len);
        he = hipMemcpy(tmp.data(), dout, tmp.size() * 4, hipMemcpyDeviceToHost);
        if (he != hipSuccess) e = (long)he;
        for (int b = 0; b < B && !e; b++) memcpy(&(*ids)[(size_t)b * nSteps], &tmp[(size_t)b * cfg.seq_len], done * sizeof(int));
        if (!e && wantLogits && outLogits) {
            outLogits->resize((size_t)B * nSteps * cfg.vocab_size);
            he = hipMemcpy(outLogits->data(), allLogits, outLogits->size() * 4, hipMemcpyDeviceToHost);
            if (he != hipSuccess) e = (long)he;
        }
    }
    return e;
}

// ---------------------------------------------------------------------------
// one LLM object per CREATE (CudaExtension.llm32.cpp:100-130, llm.cpp:20-60)
struct Llm {
    float temperature = 1.0f, topp = 0.9f;
    long seed = 0;
    Engine engine;
    BpeTokenizer tokenizer;
    HostSampler sampler;         // built at LOAD from the CREATE arguments, state kept across generations (llm.cpp:140)
    bool sampleIds = false;      // GENERATE_IDS / GENERATE_BATCH draw from the sampler instead of the device argmax
    bool batchLogits = false;    // GENERATE_BATCH also returns the logits of every step (eager launches)
    std::atomic<bool> cancel{false};
    std::atomic<bool> busy{false};
    std::atomic<bool> loaded{false};
    std::atomic<bool> end{false};
    std::string response;
    std::mutex responseLock;
    std::mutex runLock;
};

typedef MCH_LONG (*FnInvoke)(MCH_LONG, MCH_LONG, float*, MCH_LONG, float**, MCH_LONG*, MCH_TCHAR*, MCH_LONG);
typedef MCH_LONG (*FnAllocHost)(MCH_LONG, MCH_LONG, float**, float*, bool);

static FnInvoke g_parentInvoke = nullptr;
static FnAllocHost g_parentAllocHost = nullptr;
static MCH_LONG g_kernelIdx = 0;
static std::map<long, std::shared_ptr<Llm>> g_llms;   // calls in flight hold a reference of their own
static std::mutex g_mapLock;

static std::shared_ptr<Llm> find_llm(long h)
{
    std::lock_guard<std::mutex> g(g_mapLock);
    auto it = g_llms.find(h);
    return it == g_llms.end() ? nullptr : it->second;
}

// UTF-8 -> UTF-16 into a caller buffer (malformed bytes become U+FFFD).  The reference converts through the ANSI
// code page (A2T / T2A); UTF-8 keeps every prompt and response byte intact instead.
static void put_text(MCH_TCHAR* out, long max, const char* s)
{
    if (!out || max <= 0) return;
    long o = 0;
    const unsigned char* p = (const unsigned char*)s;
    while (*p && o < max - 1) {
        // one code point, or U+FFFD for the longest prefix of an ill-formed sequence (the usual decoder practice)
        uint32_t cp = 0xFFFD;
        int n = 1;
        const unsigned char b0 = *p;
        int need = 0;
        unsigned char lo = 0x80, hi = 0xBF;
        if (b0 < 0x80) cp = b0;
        else if (b0 >= 0xC2 && b0 <= 0xDF) need = 1;
        else if (b0 >= 0xE0 && b0 <= 0xEF) { need = 2; if (b0 == 0xE0) lo = 0xA0; if (b0 == 0xED) hi = 0x9F; }
        else if (b0 >= 0xF0 && b0 <= 0xF4) { need = 3; if (b0 == 0xF0) lo = 0x90; if (b0 == 0xF4) hi = 0x8F; }
        if (need) {
            uint32_t v = b0 & (need == 1 ? 0x1Fu : need == 2 ? 0x0Fu : 0x07u);
            int k = 1;
            for (; k <= need; k++) {
                const unsigned char bk = p[k];
                const unsigned char l = k == 1 ? lo : 0x80, h = k == 1 ? hi : 0xBF;
                if (bk < l || bk > h) break;
                v = (v << 6) | (bk & 0x3Fu);
            }
            if (k > need) { cp = v; n = need + 1; }
            else n = k;      // the bytes before the offending one form the ill-formed prefix
        }
        if (cp >= 0x10000) {
            if (o >= max - 2) break;
            cp -= 0x10000;
            out[o++] = (MCH_TCHAR)(0xD800 + (cp >> 10));
            out[o++] = (MCH_TCHAR)(0xDC00 + (cp & 0x3FF));
        } else out[o++] = (MCH_TCHAR)cp;
        p += n;
    }
    out[o] = 0;
}

// UTF-16 -> UTF-8
static std::string narrow(const MCH_TCHAR* s)
{
    std::string o;
    if (!s) return o;
    for (; *s; s++) {
        uint32_t cp = *s;
        if (cp >= 0xD800 && cp < 0xDC00 && s[1] >= 0xDC00 && s[1] < 0xE000) { cp = 0x10000 + ((cp - 0xD800) << 10) + (s[1] - 0xDC00); s++; }
        if (cp < 0x80) o += (char)cp;
        else if (cp < 0x800) { o += (char)(0xC0 | (cp >> 6)); o += (char)(0x80 | (cp & 0x3F)); }
        else if (cp < 0x10000) { o += (char)(0xE0 | (cp >> 12)); o += (char)(0x80 | ((cp >> 6) & 0x3F)); o += (char)(0x80 | (cp & 0x3F)); }
        else { o += (char)(0xF0 | (cp >> 18)); o += (char)(0x80 | ((cp >> 12) & 0x3F)); o += (char)(0x80 | ((cp >> 6) & 0x3F)); o += (char)(0x80 | (cp & 0x3F)); }
    }
    return o;
}

// number of leading bytes of s that end on a code-point boundary (a trailing incomplete sequence is left out)
static size_t utf8_complete_prefix(const std::string& s)
{
    size_t n = s.size(), i = n;
    int back = 0;
    while (i > 0 && back < 4 && ((unsigned char)s[i - 1] & 0xC0) == 0x80) { i--; back++; }
    if (i == 0) return n;
    const unsigned char lead = (unsigned char)s[i - 1];
    int need = lead < 0x80 ? 1 : (lead & 0xE0) == 0xC0 ? 2 : (lead & 0xF0) == 0xE0 ? 3 : (lead & 0xF8) == 0xF0 ? 4 : 1;
    return (int)(n - (i - 1)) < need ? i - 1 : n;
}

static long give(const std::vector<float>& v, float** ppOut, MCH_LONG* plOut)
{
    // results are handed over in memory owned by the parent (CudaExtension.llm32.cpp:123)
    long e = g_parentAllocHost(g_kernelIdx, (MCH_LONG)v.size(), ppOut, const_cast<float*>(v.data()), false);
    if (e) return e;
    *plOut = (MCH_LONG)v.size();
    return 0;
}

}  // namespace mch

using namespace mch;

extern "C" {

MCH_LONG DLL_InitFloatCustomExtension(void* hParent, MCH_LONG lKernelIdx)
{
    if (!hParent) return MCH_ERROR_PARAM_NULL;
    g_parentInvoke = (FnInvoke)dlsym(hParent, "DLL_InvokeFloat");
    g_parentAllocHost = (FnAllocHost)dlsym(hParent, "Internal_AllocHostFloat");
    if (!g_parentInvoke || !g_parentAllocHost) return MCH_ERROR_PARAM;
    g_kernelIdx = lKernelIdx;
    return 0;
}

MCH_LONG DLL_InvokeFloatCustomExtension(MCH_LONG fn, float* pIn, MCH_LONG lIn, float** ppOut, MCH_LONG* plOut, MCH_TCHAR* szErr,
                                        MCH_LONG errMax)
{
    if (!g_parentInvoke) return MCH_ERROR_EXTENSION_NOT_INITIALIZED;
    switch (fn) {
    case MCH_LLM_CREATE: {
        std::shared_ptr<Llm> m = std::make_shared<Llm>();
        if (lIn > 0) m->temperature = pIn[0];
        if (lIn > 1) m->topp = pIn[1];
        if (lIn > 2) m->seed = (long)pIn[2];
        long h;
        {
            std::lock_guard<std::mutex> g(g_mapLock);
            h = g_llms.empty() ? 1 : g_llms.rbegin()->first + 1;
            g_llms[h] = m;
        }
        long e = give({(float)h}, ppOut, plOut);
        if (e) {
            std::lock_guard<std::mutex> g(g_mapLock);
            g_llms.erase(h);
        }
        return (MCH_LONG)e;
    }
    case MCH_LLM_DESTROY: {
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m;
        {
            std::lock_guard<std::mutex> g(g_mapLock);
            auto it = g_llms.find((long)pIn[0]);
            if (it != g_llms.end()) { m = it->second; g_llms.erase(it); }
        }
        if (m) {
            m->cancel.store(true);
            // wait for a running generate to notice the flag; the lock is released before the object can go away, and
            // a call that looked the handle up before the erase keeps the object alive until it returns
            { std::lock_guard<std::mutex> run(m->runLock); }
            m.reset();
        }
        return 0;
    }
    case MCH_LLM_ABORT: {
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (m) m->cancel.store(true);
        return 0;
    }
    case MCH_LLM_QUERYSTATUS: {
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        float v = m->loaded.load() ? 1.f : 0.f;
        return (MCH_LONG)give({v, v}, ppOut, plOut);
    }
    case MCH_LLM_SET_OPTION: {
        if (lIn < 3) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        std::lock_guard<std::mutex> run(m->runLock);
        int opt = (int)pIn[1];
        if (opt == 1) m->engine.bf16_weights = pIn[2] != 0.f;
        else if (opt == 2) m->engine.timedFrom = (int)pIn[2];
        else if (opt == 3) m->engine.use_graph = pIn[2] != 0.f;
        else if (opt == 4) m->engine.set_mv_rows(pIn[2] == 1.f ? 1 : (pIn[2] == 2.f ? 2 : 0));
        else if (opt == 5) m->sampleIds = pIn[2] != 0.f;
        else if (opt == 6) m->batchLogits = pIn[2] != 0.f;
        else if (opt == 7) m->engine.use_prefill = pIn[2] != 0.f;
        else if (opt == 8) m->engine.set_kv_bf16(pIn[2] != 0.f);
        else if (opt == 9) m->engine.set_defer_merge(pIn[2] != 0.f);
        else if (opt == 10) m->engine.prefill_act16 = pIn[2] != 0.f;
        else if (opt == 11) m->engine.device_sampling = pIn[2] != 0.f;
        else return MCH_ERROR_PARAM_OUT_OF_RANGE;
        return 0;
    }
    case MCH_LLM_QUERY_TIMING: {
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        return (MCH_LONG)give({m->engine.lastTimedMs, (float)m->engine.lastTimedSteps, m->engine.lastUsedGraph ? 1.f : 0.f,
                                m->engine.lastPrefillMs, (float)m->engine.lastPrefillRows}, ppOut, plOut);
    }
    case MCH_LLM_PROFILE_STEP: {
        if (lIn < 3) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        std::lock_guard<std::mutex> run(m->runLock);
        std::vector<float> out;
        long e = m->engine.profile_step((int)pIn[1], (int)pIn[2], lIn > 3 ? (int)pIn[3] : 1, &out);
        if (e) return (MCH_LONG)e;
        return (MCH_LONG)give(out, ppOut, plOut);
    }
    case MCH_LLM_SAMPLE: {
        // f{hLlm, logits...} -> f{id}: one call of the handle's sampler (advances its random state unless greedy)
        if (lIn < 2) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        if (!m->loaded.load()) return MCH_ERROR_LLM_GENERATE;
        std::lock_guard<std::mutex> run(m->runLock);
        std::vector<float> lg(pIn + 1, pIn + lIn);
        if (!m->sampler.greedy() && m->engine.device_sampling && (int)lg.size() <= SAMPLE_MAX_VOCAB) {
            // where the generations sample: on the device (option 11)
            int id = 0;
            const long e = m->engine.sample_device(lg.data(), (int)lg.size(), &m->sampler, &id);
            if (e) return (MCH_LONG)e;
            return (MCH_LONG)give({(float)id}, ppOut, plOut);
        }
        return (MCH_LONG)give({(float)m->sampler.sample(lg.data(), (int)lg.size())}, ppOut, plOut);
    }
    case MCH_LLM_RUNNING_SUM: {
        // f{hLlm, threshold, values...} -> f{index, sum}: the device sampler's rounded running sum over the values, stopped at
        // the first index where it exceeds the threshold (index = count when it never does)
        if (lIn < 3) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        if (!m->loaded.load()) return MCH_ERROR_LLM_GENERATE;
        std::lock_guard<std::mutex> run(m->runLock);
        int out2[2] = {0, 0};
        const long e = m->engine.running_sum_device(pIn + 2, (int)(lIn - 2), pIn[1], out2);
        if (e) return (MCH_LONG)e;
        float sum;
        memcpy(&sum, &out2[1], 4);
        return (MCH_LONG)give({(float)out2[0], sum}, ppOut, plOut);
    }
    case MCH_LLM_GENERATE_IDS:
    case MCH_LLM_GENERATE_BATCH: {
        // GENERATE_IDS   f{hLlm, nSteps, wantLogits, ids...}
        // GENERATE_BATCH f{hLlm, nSteps, batch, nPrompt, ids of sequence 0 .., sequence 1 ..}
        //                -> f{batch x nSteps ids [, batch x nSteps x vocabulary logits with option 6]}
        const bool batch = fn == MCH_LLM_GENERATE_BATCH;
        const int head = batch ? 4 : 3;
        if (lIn < head + 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        std::lock_guard<std::mutex> run(m->runLock);
        const int nSteps = (int)pIn[1];
        const int B = batch ? (int)pIn[2] : 1;
        const int nPrompt = batch ? (int)pIn[3] : lIn - head;
        const bool wantLogits = batch ? m->batchLogits : pIn[2] != 0.f;
        if (B < 1 || nPrompt < 1 || (long long)B * nPrompt != lIn - head) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::vector<int> prompts((size_t)B * nPrompt);
        for (size_t i = 0; i < prompts.size(); i++) prompts[i] = (int)pIn[head + i];
        std::vector<int> ids;
        std::vector<float> logits;
        m->cancel.store(false);
        m->busy.store(true);
        long e = m->engine.generate(prompts.data(), B, nPrompt, nSteps, wantLogits, &ids, &logits, &m->cancel, 0, nullptr,
                                    m->sampleIds ? &m->sampler : nullptr);
        m->busy.store(false);
        if (e) {
            if (e == MCH_ERROR_LLM_GENERATE) put_text(szErr, errMax, "The model is not loaded.");
            return (MCH_LONG)e;
        }
        std::vector<float> out(ids.size() + logits.size());
        for (size_t i = 0; i < ids.size(); i++) out[i] = (float)ids[i];
        if (!logits.empty()) memcpy(out.data() + ids.size(), logits.data(), logits.size() * 4);
        return (MCH_LONG)give(out, ppOut, plOut);
    }
    default:
        put_text(szErr, errMax, "The function specified is not supported.");
        return MCH_ERROR_NOT_IMPLEMENTED;
    }
}

MCH_LONG DLL_InvokeFloatCustomExtensionEx(MCH_LONG fn, float* pIn, MCH_LONG lIn, float** ppOut, MCH_LONG* plOut, MCH_TCHAR* szIn,
                                          MCH_TCHAR* szOut, MCH_LONG outMax, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    if (!g_parentInvoke) return MCH_ERROR_EXTENSION_NOT_INITIALIZED;
    switch (fn) {
    case MCH_LLM_LOAD: {
        // "model.bin;tokenizer.bin" (llm.cpp:78-98).  An empty tokenizer part selects the token-id front door.
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return 0;
        std::string in = narrow(szIn), model = in, tok;
        size_t p = in.find(';');
        if (p != std::string::npos) { model = in.substr(0, p); tok = in.substr(p + 1); }
        FILE* f = fopen(model.c_str(), "rb");
        if (!f) return MCH_ERROR_LLM_MISSING_MODEL_FILE;
        fclose(f);
        if (!tok.empty()) {
            f = fopen(tok.c_str(), "rb");
            if (!f) return MCH_ERROR_LLM_MISSING_TOKENIZER_FILE;
            fclose(f);
        }
        std::lock_guard<std::mutex> run(m->runLock);
        m->busy.store(true);
        long e = m->engine.load(model.c_str());
        if (!e && !tok.empty() && !m->tokenizer.load(tok.c_str(), m->engine.cfg.vocab_size)) e = MCH_ERROR_LLM_LOAD_MODEL;
        m->busy.store(false);
        if (!e) m->sampler.build(m->temperature, m->topp, (unsigned long long)m->seed);
        m->loaded.store(e == 0);
        if (e && !m->engine.lastError.empty()) put_text(szErr, errMax, m->engine.lastError.c_str());
        return (MCH_LONG)e;
    }
    case MCH_LLM_GENERATE: {
        // LLMData::Generate (llm.cpp:193-263): encode the rendered prompt with BOS, force its tokens, then feed
        // back the sampled token; from the last prompt position on every sampled token that is not EOS (2)
        // appends its piece to the response; stop at EOS, at the step limit or on ABORT.  The device loop runs
        // in chunks of 32 positions, so the response grows while the caller polls QUERY_RESPONSE.
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        if (!m->loaded.load()) return MCH_ERROR_LLM_GENERATE;
        if (!m->tokenizer.loaded()) {
            put_text(szErr, errMax, "No tokenizer file was given at LOAD; use the token-id entry.");
            return MCH_ERROR_LLM_MISSING_TOKENIZER_FILE;
        }
        const std::string prompt = narrow(szIn);
        if (prompt.size() > 4096) return MCH_ERROR_LLM_RENDERED_PROMPT_TO_LONG;
        std::lock_guard<std::mutex> run(m->runLock);
        m->end.store(false);
        m->cancel.store(false);
        m->busy.store(true);
        const std::vector<int> toks = m->tokenizer.encode(prompt, true, false);
        const int nP = (int)toks.size();
        const int steps = std::min(2048, m->engine.cfg.seq_len);
        long e = 0;
        if (nP > steps) e = MCH_ERROR_LLM_RENDERED_PROMPT_TO_LONG;
        for (int t : toks)
            if (t < 0 || t >= m->engine.cfg.vocab_size) e = MCH_ERROR_LLM_GENERATE;   // e.g. a vocabulary without the " " entry
        if (!e) {
            std::vector<int> ids;
            int endPos = -1;   // the position whose token or sampled id ended the generation
            const unsigned long long rng0 = m->sampler.state;
            auto onChunk = [&](const int* out, int from, int to) -> bool {
                for (int pos = from; pos < to; pos++) {
                    const int token = pos < nP ? toks[pos] : out[pos - 1];
                    const int next = out[pos];
                    if (pos + 1 >= nP && next != 2) {
                        const std::string piece = m->tokenizer.decode(token, next);
                        std::lock_guard<std::mutex> g(m->responseLock);
                        m->response += piece;
                    }
                    if (token == 2 || next == 2) { endPos = pos; return false; }
                }
                return !m->cancel.load();
            };
            // greedy: ids are looked at every 32 steps; sampled: after every step, so that the generation stops on the very
            // step that draws the end-of-text id and the random stream stays where the reference's would be
            e = m->engine.generate(toks.data(), 1, nP, steps, false, &ids, nullptr, &m->cancel, m->sampler.greedy() ? 32 : 1, onChunk,
                                   &m->sampler);
            if (!e && !m->sampler.greedy() && endPos >= 0) {
                // The reference stops on the very position that draws the end-of-text id, one coin per position up to
                // it.  The batched prompt pass flips the coins of all prompt positions at once: the stream is put
                // where the reference's would be.
                m->sampler.state = rng0;
                for (int d = 0; d <= endPos; d++) (void)m->sampler.random_u32();
            }
            if (m->cancel.load()) {
                std::lock_guard<std::mutex> g(m->responseLock);
                m->response.clear();
            }
        }
        m->busy.store(false);
        m->end.store(true);
        return (MCH_LONG)e;
    }
    case MCH_LLM_TOKENIZE: {
        // f{hLlm, bos, eos} + text -> token ids; f{hLlm, -1, prev, token} -> the piece in szOutput
        if (lIn < 3) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        if (!m) return MCH_ERROR_PARAM;
        if (!m->tokenizer.loaded()) return MCH_ERROR_LLM_MISSING_TOKENIZER_FILE;
        if (pIn[1] < 0.f) {
            if (lIn < 4) return MCH_ERROR_PARAM_OUT_OF_RANGE;
            put_text(szOut, outMax, m->tokenizer.decode((int)pIn[2], (int)pIn[3]).c_str());
            return 0;
        }
        const std::vector<int> toks = m->tokenizer.encode(narrow(szIn), pIn[1] != 0.f, pIn[2] != 0.f);
        return (MCH_LONG)give(std::vector<float>(toks.begin(), toks.end()), ppOut, plOut);
    }
    case MCH_LLM_QUERYRESPONSE: {
        if (lIn < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        std::shared_ptr<Llm> m = find_llm((long)pIn[0]);
        long end = 1;
        if (m) {
            std::lock_guard<std::mutex> g(m->responseLock);
            end = m->end.load() ? 1 : 0;
            // hand out whole code points only while the generation is still running (byte tokens arrive one at a time),
            // and no more than fits the caller's buffer (llm.cpp:272-283)
            size_t n = end ? m->response.size() : utf8_complete_prefix(m->response);
            if (outMax > 0 && n > (size_t)(outMax - 1)) { n = utf8_complete_prefix(m->response.substr(0, (size_t)(outMax - 1))); end = 0; }
            put_text(szOut, outMax, m->response.substr(0, n).c_str());
            m->response.erase(0, n);
            if (end) m->end.store(false);
        }
        if (ppOut) *ppOut = (float*)end;  // the end flag travels through the pointer (CudaExtension.llm32.cpp:257-258)
        return 0;
    }
    default:
        put_text(szErr, errMax, "The function specified is not supported.");
        return MCH_ERROR_NOT_IMPLEMENTED;
    }
}

// Double twins of the three exports (CudaExtension.llm32.11.8.def:8-11): the engine computes in fp32 only.
static MCH_LONG ext_double_unsupported(MCH_TCHAR* szErr, MCH_LONG errMax)
{
    put_text(szErr, errMax, "The double base type is not built: the llama2 engine runs in fp32 and 16-bit storage. (90009)");
    return MCH_ERROR_NOT_IMPLEMENTED;
}
MCH_LONG DLL_InitDoubleCustomExtension(void*, MCH_LONG) { return MCH_ERROR_NOT_IMPLEMENTED; }
MCH_LONG DLL_InvokeDoubleCustomExtension(MCH_LONG, double*, MCH_LONG, double**, MCH_LONG*, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return ext_double_unsupported(szErr, errMax);
}
MCH_LONG DLL_InvokeDoubleCustomExtensionEx(MCH_LONG, double*, MCH_LONG, double**, MCH_LONG*, MCH_TCHAR*, MCH_TCHAR*, MCH_LONG,
                                           MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return ext_double_unsupported(szErr, errMax);
}

}  // extern "C"
