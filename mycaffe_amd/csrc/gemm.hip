// GEMM / GEMV kernels for gfx950.
//
//  * gemm_nt_f32_mfma  : C = alpha*A[M,K]*B[N,K]^T + beta*C, fp32 in, fp32 MFMA
//                        (v_mfma_f32_32x32x2_f32), 128x128x16 LDS-staged tiles.
//                        This is the InnerProduct shape (weights stored [N,K]).
//  * gemm_nt_bf16_mfma : same contraction on bf16 storage with
//                        v_mfma_f32_32x32x16_bf16, fp32 accumulate, 128x128x32 tiles.
//  * gemm_generic      : any transpose / stride combination (row-major gemm with
//                        transposed operands, column-major strided-batched gemm2),
//                        64x64x16 LDS tiles, fp32 FMA.
//  * gemv              : HBM-bound y = A x, one wavefront per row, 128-bit loads.
#include <algorithm>

#include <type_traits>

#include "kernels.h"

namespace mch {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef float floatx2v __attribute__((ext_vector_type(2)));

__device__ inline uint32_t pack2_bf16(float a, float b)
{
    floatx2v f = {a, b};
    bf16x2v r = __builtin_convertvector(f, bf16x2v);
    return *reinterpret_cast<uint32_t*>(&r);
}

template <typename T> __device__ inline float ldf(const T* p, size_t i);
template <> __device__ inline float ldf<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ inline float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
template <typename T> __device__ inline void stf(T* p, size_t i, float v);
template <> __device__ inline void stf<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ inline void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// ---------------------------------------------------------------------------
// generic strided GEMM: C(i,j) = alpha * sum_k A(i,k) B(k,j) + beta * C(i,j)
// element addresses: A[i*ai + k*ak], B[k*bk + j*bj], C[i*ci + j*cj]; blockIdx.z = batch
struct GemmStrides { long long ai, ak, bk, bj, ci, cj, sA, sB, sC; };

template <typename T>
__global__ __launch_bounds__(256) void gemm_generic_kernel(int M, int N, int K, float alpha, const T* __restrict__ A,
                                                           const T* __restrict__ B, float beta, T* __restrict__ C,
                                                           GemmStrides st)
{
    constexpr int BM = 64, BN = 64, BK = 16;
    __shared__ float As[BK][BM + 4];
    __shared__ float Bs[BK][BN + 4];
    A += (size_t)blockIdx.z * st.sA;
    B += (size_t)blockIdx.z * st.sB;
    C += (size_t)blockIdx.z * st.sC;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int tid = threadIdx.x;
    const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
    // pick the load order that walks the unit-stride axis with consecutive threads
    const bool a_k_fast = st.ak == 1;
    const bool b_k_fast = st.bk == 1;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
        for (int e = tid; e < BM * BK; e += 256) {
            int i, k;
            if (a_k_fast) { i = e / BK; k = e % BK; } else { k = e / BM; i = e % BM; }
            float v = 0.f;
            if (m0 + i < M && k0 + k < K) v = ldf(A, (size_t)((long long)(m0 + i) * st.ai + (long long)(k0 + k) * st.ak));
            As[k][i] = v;
        }
        for (int e = tid; e < BN * BK; e += 256) {
            int j, k;
            if (b_k_fast) { j = e / BK; k = e % BK; } else { k = e / BN; j = e % BN; }
            float v = 0.f;
            if (n0 + j < N && k0 + k < K) v = ldf(B, (size_t)((long long)(k0 + k) * st.bk + (long long)(n0 + j) * st.bj));
            Bs[k][j] = v;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; k++) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = As[k][tm + i];
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = Bs[k][tn + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++) {
            int r = m0 + tm + i, c = n0 + tn + j;
            if (r < M && c < N) {
                size_t ci = (size_t)((long long)r * st.ci + (long long)c * st.cj);
                float v = alpha * acc[i][j];
                if (beta != 0.f) v += beta * ldf(C, ci);
                stf(C, ci, v);
            }
        }
}

template <typename T>
static hipError_t launch_generic(hipStream_t s, int M, int N, int K, float alpha, const T* A, const T* B, float beta, T* C,
                                 GemmStrides st, int batch)
{
    if (M <= 0 || N <= 0 || batch <= 0) return hipSuccess;
    dim3 grid((N + 63) / 64, (M + 63) / 64, batch);
    if (grid.y > 65535 || grid.z > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gemm_generic_kernel<T>, grid, 256, 0, s, M, N, K, alpha, A, B, beta, C, st);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// fp32 MFMA, NT.  4 wavefronts in a 2x2 arrangement, each owning 64x64 of the
// 128x128 tile as 2x2 MFMA 32x32 blocks.  One 128-bit LDS read feeds four
// MFMA steps: lane group g (= lane/32) holds k = kk+4g .. kk+4g+3, and MFMA step
// j contracts the two slots {kk+j, kk+4+j}; the slot-to-k assignment is free as
// long as A and B use the same one.
__global__ __launch_bounds__(256) void gemm_nt_f32_mfma_kernel(int M, int N, int K, float alpha,
                                                               const float* __restrict__ A,
                                                               const float* __restrict__ B, float beta,
                                                               float* __restrict__ C)
{
    constexpr int BM = 128, BN = 128, BK = 16, LDK = BK + 4;
    __shared__ __attribute__((aligned(16))) float As[2][BM * LDK];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN * LDK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int lr = tid >> 2, lc = (tid & 3) * 4;  // 64 rows x 4 float4 per pass, 2 passes

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    float4 ra[2], rb[2];
    auto gload = [&](int k0) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            int r = lr + p * 64;
            ra[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            rb[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m0 + r < M && k0 + lc < K) ra[p] = *(const float4*)(A + (size_t)(m0 + r) * K + k0 + lc);
            if (n0 + r < N && k0 + lc < K) rb[p] = *(const float4*)(B + (size_t)(n0 + r) * K + k0 + lc);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            int r = lr + p * 64;
            *(float4*)(&As[buf][r * LDK + lc]) = ra[p];
            *(float4*)(&Bs[buf][r * LDK + lc]) = rb[p];
        }
    };

    const int nk = (K + BK - 1) / BK;
    gload(0);
    sstore(0);
    __syncthreads();
    const int fr = lane & 31, fg = (lane >> 5) * 4;
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) gload((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 8) {
            float4 a[2], b[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                a[t] = *(const float4*)(&As[buf][(wm + t * 32 + fr) * LDK + kk + fg]);
                b[t] = *(const float4*)(&Bs[buf][(wn + t * 32 + fr) * LDK + kk + fg]);
            }
            const float* af0 = (const float*)&a[0];
            const float* af1 = (const float*)&a[1];
            const float* bf0 = (const float*)&b[0];
            const float* bf1 = (const float*)&b[1];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af0[j], bf0[j], acc[0][0], 0, 0, 0);
                acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(af0[j], bf1[j], acc[0][1], 0, 0, 0);
                acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af1[j], bf0[j], acc[1][0], 0, 0, 0);
                acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(af1[j], bf1[j], acc[1][1], 0, 0, 0);
            }
        }
        if (kt + 1 < nk) sstore(buf ^ 1);
        __syncthreads();
    }
    // accumulator register v of a 32x32 block: row = 8*(v/4) + 4*(lane/32) + v%4, col = lane%32
    const int col_l = lane & 31, row_l = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            int c = n0 + wn + j * 32 + col_l;
            if (c >= N) continue;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int r = m0 + wm + i * 32 + (v >> 2) * 8 + row_l + (v & 3);
                if (r < M) {
                    size_t ci = (size_t)r * N + c;
                    float o = alpha * acc[i][j][v];
                    if (beta != 0.f) o += beta * C[ci];
                    C[ci] = o;
                }
            }
        }
}

// ---------------------------------------------------------------------------
// bf16 MFMA, NT, 128x128x32 tiles, 4 wavefronts each 64x64 (2x2 MFMA 32x32x16).
// Lane l feeds row l%32 with the eight k values 8*(l/32) .. 8*(l/32)+7 of a
// 16-wide MFMA step: one 128-bit LDS read per operand block and step.
__global__ __launch_bounds__(256) void gemm_nt_bf16_mfma_kernel(int M, int N, int K, float alpha,
                                                                const bf16_t* __restrict__ A,
                                                                const bf16_t* __restrict__ B, float beta,
                                                                bf16_t* __restrict__ C)
{
    constexpr int BM = 128, BN = 128, BK = 32, LDK = BK + 8;  // row stride 80 B
    __shared__ __attribute__((aligned(16))) bf16_t As[2][BM * LDK];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[2][BN * LDK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int lr = tid >> 2, lc = (tid & 3) * 8;  // 64 rows x 4 x (8 bf16) per pass, 2 passes

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    uint4 ra[2], rb[2];
    auto gload = [&](int k0) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            int r = lr + p * 64;
            ra[p] = make_uint4(0, 0, 0, 0);
            rb[p] = make_uint4(0, 0, 0, 0);
            if (m0 + r < M && k0 + lc < K) ra[p] = *(const uint4*)(A + (size_t)(m0 + r) * K + k0 + lc);
            if (n0 + r < N && k0 + lc < K) rb[p] = *(const uint4*)(B + (size_t)(n0 + r) * K + k0 + lc);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            int r = lr + p * 64;
            *(uint4*)(&As[buf][r * LDK + lc]) = ra[p];
            *(uint4*)(&Bs[buf][r * LDK + lc]) = rb[p];
        }
    };

    const int nk = (K + BK - 1) / BK;
    gload(0);
    sstore(0);
    __syncthreads();
    const int fr = lane & 31, fg = (lane >> 5) * 8;
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) gload((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            bf16x8 a[2], b[2];
#pragma unroll
            for (int t = 0; t < 2; t++) {
                a[t] = *(const bf16x8*)(&As[buf][(wm + t * 32 + fr) * LDK + kk + fg]);
                b[t] = *(const bf16x8*)(&Bs[buf][(wn + t * 32 + fr) * LDK + kk + fg]);
            }
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[1], acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[0], acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], acc[1][1], 0, 0, 0);
        }
        if (kt + 1 < nk) sstore(buf ^ 1);
        __syncthreads();
    }
    const int col_l = lane & 31, row_l = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            int c = n0 + wn + j * 32 + col_l;
            if (c >= N) continue;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                int r = m0 + wm + i * 32 + (v >> 2) * 8 + row_l + (v & 3);
                if (r < M) {
                    size_t ci = (size_t)r * N + c;
                    float o = alpha * acc[i][j][v];
                    if (beta != 0.f) o += beta * bf16_to_f32(C[ci]);
                    C[ci] = f32_to_bf16(o);
                }
            }
        }
}

// ---------------------------------------------------------------------------
// MFMA, NT, large tiles, bf16 and fp32: 2 x 2 wavefronts, each owning WM x WN MFMA 32x32 tiles, so a workgroup
// covers (64 WM) x (64 WN) of C.  A 128 x 128 wavefront tile (WM = WN = 4) reads 8 LDS fragments per 16 tile
// products, a quarter of the LDS traffic per flop of the 64 x 64 wavefront tile, which is what keeps the matrix
// cores fed; its 256 accumulators live in the accumulation registers.  K is walked in stages of 128 bytes per
// row through a double-buffered LDS stage (one barrier per stage).  A k-step is one 16-byte fragment per lane
// and operand: one v_mfma_f32_32x32x16_bf16, or four v_mfma_f32_32x32x2_f32 (lane half h holds k = 4h .. 4h+3 of
// a group of eight and step e contracts {e, 4 + e}; the slot assignment only has to agree between A and B).
// Tiles are numbered so that each XCD (workgroup index mod 8) works on a contiguous band of tile rows and
// re-uses its A rows out of its own L2.
template <typename T> struct BigTraits;
template <> struct BigTraits<bf16_t> {
    static constexpr int E = 8;   // elements per 16-byte chunk
    __device__ static inline floatx16 mma(u32x4 a, u32x4 b, floatx16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8*>(&a), *reinterpret_cast<bf16x8*>(&b), c, 0, 0, 0);
    }
    __device__ static inline float ld(const bf16_t* p) { return bf16_to_f32(*p); }
    __device__ static inline void st(bf16_t* p, float v) { *p = f32_to_bf16(v); }
    __device__ static inline void st4(bf16_t* p, float a, float b, float c, float d)
    {
        uint2 w;
        w.x = pack2_bf16(a, b);
        w.y = pack2_bf16(c, d);
        *(uint2*)p = w;
    }
};
template <> struct BigTraits<float> {
    static constexpr int E = 4;
    __device__ static inline floatx16 mma(u32x4 a, u32x4 b, floatx16 c)
    {
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
        return c;
    }
    __device__ static inline float ld(const float* p) { return *p; }
    __device__ static inline void st(float* p, float v) { *p = v; }
    __device__ static inline void st4(float* p, float a, float b, float c, float d) { *(float4*)p = make_float4(a, b, c, d); }
};

// Epilogue of the fused QKV projection (HEADS): row r = (b, t) of the M = B*T rows, column c = (which, h, d) of the
// N = 3*H*hs columns goes, bias added, to element (b, h, t, d) of tensor `which` (q, k, v), i.e. the layout the
// attention kernels read, instead of to C[r][c].  Replaces the bias GEMM, the three channel copies and the three head
// transposes that follow the fused InnerProduct in CausalSelfAttentionLayer.forward (CausalSelfAttentionLayer.cs:526-557).
// With fcos / fsin set (tables [seq][hs/2]) the q and k thirds are also rotated, after their rounding to the storage type:
// adjacent pairs (2i, 2i+1) of row r by the angle of table row r % seq, column i - the rotary embedding that the layer
// applies to q and k in (B,T,H,hs) layout before the head transposes (CausalSelfAttentionLayer.cs:538-545, rope.cu:785-825).
struct HeadsEpilogue { const void* bias; void* dst[3]; int T, H, hs; const float* fcos; const float* fsin; int seq; };

template <typename T>
__device__ __forceinline__ T* heads_dst(const HeadsEpilogue& he, int row, int col)
{
    const int Cd = he.H * he.hs;
    const int which = col / Cd, w = col - which * Cd, h = w / he.hs, d = w - h * he.hs;
    const int b = row / he.T, t = row - b * he.T;
    return (T*)he.dst[which] + (((size_t)b * he.H + h) * he.T + t) * he.hs + d;
}

// (re, im) of one pair of q or k, rotated; the expressions of rope_kernel (ew_kernels.hip)
__device__ __forceinline__ void heads_rope_pair(float c, float sn, float& re, float& im)
{
    const float a = re * c - im * sn, b = re * sn + im * c;
    re = a; im = b;
}

// the rotation applied to one 16-byte piece (columns col .. col + 16 / sizeof(T) - 1 of row `row`; whole pairs of one head)
template <typename T>
__device__ __forceinline__ u32x4 heads_rope_piece(const HeadsEpilogue& he, int row, int col, u32x4 v)
{
    if (!he.fcos || col >= 2 * he.H * he.hs) return v;
    constexpr int NP = 8 / (int)sizeof(T);
    const size_t ti = (size_t)(row % he.seq) * (he.hs >> 1) + ((col % he.hs) >> 1);
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const float c = he.fcos[ti + i], sn = he.fsin[ti + i];
        if constexpr (sizeof(T) == 4) {
            float re = __uint_as_float(w[2 * i]), im = __uint_as_float(w[2 * i + 1]);
            heads_rope_pair(c, sn, re, im);
            w[2 * i] = __float_as_uint(re); w[2 * i + 1] = __float_as_uint(im);
        } else {
            float re = __uint_as_float(w[i] << 16), im = __uint_as_float(w[i] & 0xffff0000u);
            heads_rope_pair(c, sn, re, im);
            w[i] = (uint32_t)f32_to_bf16(re) | ((uint32_t)f32_to_bf16(im) << 16);
        }
    }
    u32x4 o; o.x = w[0]; o.y = w[1]; o.z = w[2]; o.w = w[3];
    return o;
}

// Epilogues of the prompt pass of the Llama engine (fp32 results of 16-bit operands; llama2_ext.hip), which save the
// round trip of the product through memory and the kernel that would read it back:
//   EPI 1, SwiGLU of the stacked W1 | W3 product.  Tile column c multiplies weight row (c & 1) hid + c / 2, so that a
//     lane's register quad holds (w1 x, w3 x) of two consecutive hidden units j: out[j] = silu(w1 x) (w3 x), stored as
//     bf16 (rows of hid), or as the bf16 nearest to it followed, hid further on, by the bf16 nearest to the remainder
//     (rows of 2 hid: the operand form of k_gemm_bf16_f32's split product).
//   EPI 2, rotation and scatter of the stacked Wq | Wk | Wv product (row = sequence b, position p): q and k rotated at p
//     (adjacent pairs, the decode kernel's arithmetic), q / k / v written as (B, H, P, hs) head tensors - fp32 or bf16,
//     every key / value head repeated for the query heads that share it - and the rotated key and the value appended to
//     the caches [b][p][kvd] (fp32 or bf16; the head tensors then carry the values the cache holds).
struct PromptEpilogue {
    void* out; int hid; int split;                                   // EPI 1
    void* q; void* k; void* v; void* kc; void* vc;                   // EPI 2
    const float* fcos; const float* fsin;
    int P, H, kvH, hs, seqLen, heads16, cache16, kvMul;
    float invP, invHs;
};
__device__ __forceinline__ uint32_t pe_pack(float a, float b) { return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16); }
__device__ __forceinline__ float pe_round(float a) { return bf16_to_f32(f32_to_bf16(a)); }
// four consecutive values to a tensor of fp32 or bf16
__device__ __forceinline__ void pe_store4(void* base, size_t idx, int is16, const float (&v)[4])
{
    if (is16) *(uint2*)((bf16_t*)base + idx) = make_uint2(pe_pack(v[0], v[1]), pe_pack(v[2], v[3]));
    else *(float4*)((float*)base + idx) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void prompt_epilogue_swiglu(const PromptEpilogue& pe, int r, int c, const float (&a)[4])
{
    const int j = c >> 1;   // c is a multiple of 4: hidden units j, j + 1
    float o[2];
#pragma unroll
    for (int q = 0; q < 2; q++) o[q] = a[2 * q] * (1.0f / (1.0f + expf(-a[2 * q]))) * a[2 * q + 1];
    bf16_t* row = (bf16_t*)pe.out + (size_t)r * (pe.split ? 2 : 1) * pe.hid;
    *(uint32_t*)(row + j) = pe_pack(o[0], o[1]);
    if (pe.split) *(uint32_t*)(row + pe.hid + j) = pe_pack(o[0] - pe_round(o[0]), o[1] - pe_round(o[1]));
}
// x / d for 0 <= x < 2^24, d > 0, through the reciprocal (an integer division is some forty instructions)
__device__ __forceinline__ int pe_div(int x, int d, float inv)
{
    int q = (int)((float)x * inv);
    if ((q + 1) * d <= x) q++;
    if (q * d > x) q--;
    return q;
}
__device__ __forceinline__ void prompt_epilogue_rope(const PromptEpilogue& pe, int r, int c, const float (&a)[4])
{
    const int dim = pe.H * pe.hs, kvd = pe.kvH * pe.hs, kvMul = pe.kvMul, half = pe.hs >> 1;
    const int b = pe_div(r, pe.P, pe.invP), p = r - b * pe.P;
    float o[4] = {a[0], a[1], a[2], a[3]};
    const int which = c < dim ? 0 : c < dim + kvd ? 1 : 2;
    const int cc = which == 0 ? c : which == 1 ? c - dim : c - dim - kvd;
    const int h = pe_div(cc, pe.hs, pe.invHs), d = cc - h * pe.hs;
    if (which < 2) {
        const float2 cs = *(const float2*)(pe.fcos + (size_t)p * half + (d >> 1)), sn = *(const float2*)(pe.fsin + (size_t)p * half + (d >> 1));
        o[0] = a[0] * cs.x - a[1] * sn.x; o[1] = a[0] * sn.x + a[1] * cs.x;
        o[2] = a[2] * cs.y - a[3] * sn.y; o[3] = a[2] * sn.y + a[3] * cs.y;
    }
    if (which == 0) {
        pe_store4(pe.q, (((size_t)b * pe.H + h) * pe.P + p) * pe.hs + d, pe.heads16, o);
        return;
    }
    if (pe.cache16) {
#pragma unroll
        for (int q = 0; q < 4; q++) o[q] = pe_round(o[q]);   // the pass attends over the values the cache holds
    }
    pe_store4(which == 1 ? pe.kc : pe.vc, ((size_t)b * pe.seqLen + p) * kvd + cc, pe.cache16, o);
    for (int g = 0; g < kvMul; g++)
        pe_store4(which == 1 ? pe.k : pe.v, (((size_t)b * pe.H + h * kvMul + g) * pe.P + p) * pe.hs + d, pe.heads16, o);
}

// SPLIT (16-bit operands, fp32 C): a row of A is 2 K long, the upper halves of K fp32 values followed by what the upper
// halves leave over (see k_gemm_bf16_split), and B is walked twice: C = alpha (A_hi + A_lo) B^T + beta C.
template <typename T, int WM, int WN, int OCC, bool HEADS = false, typename TC = T, bool SPLIT = false, int EPI = 0>
__global__ __launch_bounds__(256, OCC) void gemm_nt_big_kernel(int M, int N, int K, float alpha, const T* __restrict__ A,
                                                               const T* __restrict__ B, float beta, TC* __restrict__ C, int tilesN,
                                                               int tilesTotal, int bandRows, int colBlock, HeadsEpilogue he,
                                                               PromptEpilogue pe, int ld)
{
    // K: the contraction length of this launch's products, ld: the distance between rows of A and of B.  With a second
    // grid dimension, workgroup row y multiplies columns y K .. y K + K - 1 of the operands into the y-th M x N matrix
    // behind C (partial products of a long contraction, added up by splitk_reduce_kernel).
    A += (size_t)blockIdx.y * K;
    B += (size_t)blockIdx.y * K;
    C += (size_t)blockIdx.y * M * N;
    static_assert(EPI == 0 || !std::is_same<T, TC>::value, "the prompt epilogues take the fp32 results of 16-bit operands");
    static_assert(std::is_same<T, TC>::value || (!HEADS && std::is_same<TC, float>::value), "C is of the operands' type, or fp32");
    static_assert(!SPLIT || !std::is_same<T, TC>::value, "the split product writes fp32");
    typedef BigTraits<T> TR;
    constexpr int E = TR::E;
    constexpr int BK = 8 * E;                                 // elements per stage and row (128 bytes)
    constexpr int BM = 64 * WM, BN = 64 * WN, LDK = BK + E;   // row stride 16 B past a power of two: conflict-free 128-bit reads
    constexpr int CPR = 8;                                    // 16-byte chunks per tile row
    constexpr int RPP = 256 / CPR;                            // rows covered by one pass of the 256 threads
    constexpr int PA = BM / RPP, PB = BN / RPP;               // passes (16-byte chunks per thread) per operand
    constexpr int KS = 4;                                     // k-steps (fragments of 2 E elements) per stage
    constexpr int NMF = WM * WN;                              // tile products per k-step
    // Memory instructions ride along with the tile products (below): RF fragment reads and SC staging instructions per
    // product.  One of each where a k-step has at least as many products as fragments (every tile of 128 x 128 and up);
    // two with the 64-row tiles, whose wavefronts own one or two MFMA tiles.
    constexpr int RF = (WM + WN + NMF - 1) / NMF;
    constexpr int SC = ((PA + PB + KS / 2 - 1) / (KS / 2) + NMF - 1) / NMF;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    T* As = smem;                        // [2][BM * LDK]
    T* Bs = smem + 2 * BM * LDK;         // [2][BN * LDK]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per = (tilesTotal + 7) / 8;
    int tile = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
    if (colBlock > 0) {
        // The XCD's band of bandRows tile rows is walked in blocks of colBlock tile columns, so that the tiles in
        // flight on the XCD at one time share few enough A and B rows for its L2 to hold them.
        const int i = (int)(blockIdx.x / 8), nb = (tilesN + colBlock - 1) / colBlock;
        const int blk = min(i / (bandRows * colBlock), nb - 1);
        const int rem = i - blk * bandRows * colBlock;
        const int width = blk == nb - 1 ? tilesN - blk * colBlock : colBlock;
        tile = ((int)(blockIdx.x % 8) * bandRows + rem / width) * tilesN + blk * colBlock + rem % width;
    }
    if (tile >= tilesTotal) return;
    const int m0 = (tile / tilesN) * BM, n0 = (tile % tilesN) * BN;
    const int wm = (wave >> 1) * (32 * WM), wn = (wave & 1) * (32 * WN);
    const int lr = tid / CPR, lc = (tid % CPR) * E;

    floatx16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // rows past the matrix edge are clamped: they are loaded (valid memory) and never stored
    const T* ga[PA];
    const T* gb[PB];
#pragma unroll
    for (int p = 0; p < PA; p++) ga[p] = A + (size_t)min(m0 + lr + p * RPP, M - 1) * (SPLIT ? 2 * K : ld) + lc;
#pragma unroll
    for (int p = 0; p < PB; p++) {
        const int c = min(n0 + lr + p * RPP, N - 1);
        gb[p] = B + (size_t)(EPI == 1 ? (c & 1) * pe.hid + (c >> 1) : c) * ld + lc;
    }
    T* sa = As + lr * LDK + lc;
    T* sb = Bs + lr * LDK + lc;
    u32x4 ra[PA], rb[PB];

    const int nkB = K / BK, nk = SPLIT ? 2 * nkB : nkB;   // stage kt of A goes with stage kt % nkB of B
    // stage 0 -> LDS buffer 0, stage 1 -> registers
#pragma unroll
    for (int p = 0; p < PA; p++) ra[p] = *(const u32x4*)(ga[p]);
#pragma unroll
    for (int p = 0; p < PB; p++) rb[p] = *(const u32x4*)(gb[p]);
#pragma unroll
    for (int p = 0; p < PA; p++) *(u32x4*)(sa + p * RPP * LDK) = ra[p];
#pragma unroll
    for (int p = 0; p < PB; p++) *(u32x4*)(sb + p * RPP * LDK) = rb[p];
    {
        const int s1 = min(1, nk - 1), k1 = s1 * BK, k1b = (SPLIT ? s1 % nkB : s1) * BK;
#pragma unroll
        for (int p = 0; p < PA; p++) ra[p] = *(const u32x4*)(ga[p] + k1);
#pragma unroll
        for (int p = 0; p < PB; p++) rb[p] = *(const u32x4*)(gb[p] + k1b);
    }
    __syncthreads();
    const int fr = lane & 31, fg = (lane >> 5) * E;
    const T* fa = As + (wm + fr) * LDK + fg;
    const T* fb = Bs + (wn + fr) * LDK + fg;
    u32x4 a[2][WM], b[2][WN];
    // One stage: KS k-steps of NMF tile products on LDS buffer kt & 1.  Riding along between them (the wavefront
    // is alone on its SIMD, so whatever it issues between two MFMAs is hidden behind the first one's passes, and
    // whatever it issues in a block of its own is not):
    //   first half of the k-steps : the registers holding stage kt + 1 go to the other LDS buffer
    //   second half               : stage kt + 2 is fetched from global memory into those registers
    //   every k-step but the last : the fragments of the next k-step are read from LDS
    // Past the end of K the extra fetches re-read the last stage (valid memory, never consumed).
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        const T* pa = fa + buf * BM * LDK;
        const T* pb = fb + buf * BN * LDK;
        T* wa = sa + (buf ^ 1) * BM * LDK;
        T* wb = sb + (buf ^ 1) * BN * LDK;
        const int s2 = min(kt + 2, nk - 1), k2 = s2 * BK, k2b = (SPLIT ? (s2 >= nkB ? s2 - nkB : s2) : s2) * BK;
#pragma unroll
        for (int t = 0; t < WM; t++) a[0][t] = *(const u32x4*)(pa + t * 32 * LDK);
#pragma unroll
        for (int t = 0; t < WN; t++) b[0][t] = *(const u32x4*)(pb + t * 32 * LDK);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int cur = ks & 1, nxt = cur ^ 1;
            // this k-step's share of the staging traffic: chunks [c0, c1) of the PA + PB chunks per thread
            constexpr int HALF = KS / 2;
            const int part = ks % HALF;
            const int c0 = (PA + PB) * part / HALF, c1 = (PA + PB) * (part + 1) / HALF;
            // written in issue order, one small scheduling region per tile product so that the order stays as
            // written: product q, then the q-th fragment read of the next k-step, then the q-th staging instruction
#pragma unroll
            for (int q = 0; q < NMF; q++) {
                const int i = q / WN, j = q % WN;
                acc[i][j] = TR::mma(b[cur][j], a[cur][i], acc[i][j]);
                if (ks + 1 < KS) {
#pragma unroll
                    for (int r = q * RF; r < (q + 1) * RF; r++) {
                        if (r < WM) a[nxt][r] = *(const u32x4*)(pa + r * 32 * LDK + (ks + 1) * 2 * E);
                        else if (r < WM + WN) b[nxt][r - WM] = *(const u32x4*)(pb + (r - WM) * 32 * LDK + (ks + 1) * 2 * E);
                    }
                }
#pragma unroll
                for (int c = c0 + q * SC; c < c0 + (q + 1) * SC; c++) {
                    if (c >= c1) break;
                    if (ks < HALF) {
                        if (c < PA) *(u32x4*)(wa + c * RPP * LDK) = ra[c];
                        else *(u32x4*)(wb + (c - PA) * RPP * LDK) = rb[c - PA];
                    } else {
                        if (c < PA) ra[c] = *(const u32x4*)(ga[c] + k2);
                        else rb[c - PA] = *(const u32x4*)(gb[c - PA] + k2b);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();
    }
    // The tile products above are the TRANSPOSED 32x32 tiles (B fragment as the row operand), so a lane owns one
    // row of C (lane%32) and register v is column 8*(v/4) + 4*(lane/32) + v%4: four consecutive columns per
    // register quad.
    const int row_l = lane & 31, col_l = (lane >> 5) * 4;
    if constexpr (!std::is_same<T, TC>::value) {
        // fp32 results of 16-bit operands.  A lane owns a row of the tile, so its own stores would be 16 bytes each in 32
        // different rows; each wavefront passes its tile, 32 rows at a time, through its own slice of LDS (free after
        // the last barrier) and the lanes then walk the rows: consecutive lanes take consecutive quads of columns, and
        // whatever the epilogue stores is contiguous along the row.
        constexpr int CW = 32 * WN, LDC = CW + 4;
        constexpr int LPR = CW / 4, RPI = 64 / LPR;             // lanes per row, rows per pass
        constexpr int NIT = (32 + RPI - 1) / RPI;
        float* cs = reinterpret_cast<float*>(smem_raw) + wave * 32 * LDC;
        const int rr = lane / LPR, cc = (lane % LPR) * 4;
        const bool vec4 = (N & 3) == 0 && (((uintptr_t)C) & 15) == 0;
#pragma unroll
        for (int i = 0; i < WM; i++) {
#pragma unroll
            for (int j = 0; j < WN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    *(float4*)(cs + row_l * LDC + j * 32 + 8 * g + col_l) =
                        make_float4(alpha * acc[i][j][4 * g], alpha * acc[i][j][4 * g + 1], alpha * acc[i][j][4 * g + 2], alpha * acc[i][j][4 * g + 3]);
            // same wavefront wrote and reads: LDS operations of one wavefront complete in order
#pragma unroll 4
            for (int it = 0; it < NIT; it++) {
                const int row = it * RPI + rr, r = m0 + wm + i * 32 + row, c = n0 + wn + cc;
                if (rr >= RPI || row >= 32 || r >= M || c >= N) continue;
                const float4 v = *(const float4*)(cs + row * LDC + cc);
                if (EPI != 0) {
                    // N is a multiple of 4 here: a quad is inside the matrix or outside it
                    const float a4[4] = {v.x, v.y, v.z, v.w};
                    if (EPI == 1) prompt_epilogue_swiglu(pe, r, c, a4);
                    else prompt_epilogue_rope(pe, r, c, a4);
                    continue;
                }
                float* cp = C + (size_t)r * N + c;
                if (vec4 && c + 3 < N) {
                    float4 o = v;
                    if (beta != 0.f) {
                        const float4 old = *(const float4*)cp;
                        o.x += beta * old.x; o.y += beta * old.y; o.z += beta * old.z; o.w += beta * old.w;
                    }
                    *(float4*)cp = o;
                } else {
                    const float a4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        if (c + q < N) cp[q] = a4[q] + (beta != 0.f ? beta * cp[q] : 0.f);
                }
            }
        }
        return;
    } else
    if (m0 + BM <= M && n0 + BN <= N && (HEADS || (beta == 0.f && (((uintptr_t)C) & 15) == 0)) && (N % E) == 0) {
        // interior tile: each wavefront passes its tile, 32 rows at a time, through its own slice of LDS (free
        // after the last barrier) and writes whole 16-byte pieces of rows, the lanes covering full cache lines
        constexpr int CW = 32 * WN, LDC = CW + E;
        constexpr int LPR = CW / E, RPI = 64 / LPR;            // lanes per row, rows per store instruction
        constexpr int NIT = (32 + RPI - 1) / RPI;
        T* cs = smem + wave * 32 * LDC;
        const int rr = lane / LPR, cc = (lane % LPR) * E;
#pragma unroll
        for (int i = 0; i < WM; i++) {
#pragma unroll
            for (int j = 0; j < WN; j++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
                    if (HEADS && he.bias) {
                        const T* bp = (const T*)he.bias + n0 + wn + j * 32 + 8 * g + col_l;
                        b0 = TR::ld(bp); b1 = TR::ld(bp + 1); b2 = TR::ld(bp + 2); b3 = TR::ld(bp + 3);
                    }
                    TR::st4(cs + row_l * LDC + j * 32 + 8 * g + col_l, alpha * acc[i][j][4 * g] + b0, alpha * acc[i][j][4 * g + 1] + b1,
                            alpha * acc[i][j][4 * g + 2] + b2, alpha * acc[i][j][4 * g + 3] + b3);
                }
            // same wavefront wrote and reads: LDS operations of one wavefront complete in order
            T* cg = C + (size_t)(m0 + wm + i * 32 + rr) * N + n0 + wn + cc;
#pragma unroll
            for (int it = 0; it < NIT; it++) {
                // lanes past RPI * LPR (row widths that do not divide 64) and rows past the block stay idle
                if (rr < RPI && it * RPI + rr < 32) {
                    const u32x4 v = *(const u32x4*)(cs + (it * RPI + rr) * LDC + cc);
                    if (HEADS) {
                        const int hr = m0 + wm + i * 32 + it * RPI + rr, hc = n0 + wn + cc;
                        *(u32x4*)heads_dst<T>(he, hr, hc) = heads_rope_piece<T>(he, hr, hc, v);
                    }
                    else *(u32x4*)(cg + (size_t)it * RPI * N) = v;
                }
            }
        }
        return;
    }
    // edge tiles, beta != 0: element-wise (unrolled, so the accumulators are never indexed dynamically)
    if constexpr (std::is_same<T, TC>::value) {
#pragma unroll
    for (int i = 0; i < WM; i++)
#pragma unroll
        for (int j = 0; j < WN; j++) {
            const int r = m0 + wm + i * 32 + row_l;
            if (r >= M) continue;
            if constexpr (HEADS) {
                // pairs of adjacent columns (N = 3 H hs with hs even: a pair is inside the matrix or outside it)
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    const int c = n0 + wn + j * 32 + (v >> 2) * 8 + col_l + (v & 3);
                    if (c >= N) continue;
                    float o0 = alpha * acc[i][j][v], o1 = alpha * acc[i][j][v + 1];
                    if (he.bias) { o0 += TR::ld((const T*)he.bias + c); o1 += TR::ld((const T*)he.bias + c + 1); }
                    T* dp = heads_dst<T>(he, r, c);
                    if (he.fcos && c < 2 * he.H * he.hs) {
                        TR::st(dp, o0); TR::st(dp + 1, o1);
                        o0 = TR::ld(dp); o1 = TR::ld(dp + 1);      // the values as the storage type holds them
                        const size_t ti = (size_t)(r % he.seq) * (he.hs >> 1) + ((c % he.hs) >> 1);
                        heads_rope_pair(he.fcos[ti], he.fsin[ti], o0, o1);
                    }
                    TR::st(dp, o0); TR::st(dp + 1, o1);
                }
                continue;
            }
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int c = n0 + wn + j * 32 + (v >> 2) * 8 + col_l + (v & 3);
                if (c < N) {
                    const size_t ci = (size_t)r * N + c;
                    float o = alpha * acc[i][j][v];
                    if (HEADS) {
                        if (he.bias) o += TR::ld((const T*)he.bias + c);
                        TR::st(heads_dst<T>(he, r, c), o);
                    } else {
                        if (beta != 0.f) o += beta * TR::ld(C + ci);
                        TR::st(C + ci, o);
                    }
                }
            }
        }
    }
}

template <typename T, int WM, int WN, int OCC, bool HEADS = false, typename TC = T, bool SPLIT = false, int EPI = 0>
static hipError_t launch_big(hipStream_t s, int m, int n, int k, float alpha, const void* A, const void* B, float beta, void* C,
                             const HeadsEpilogue* heads = nullptr, const PromptEpilogue* prompt = nullptr, int ksplits = 1)
{
    // ksplits > 1: the contraction in ksplits equal parts, part y into the y-th m x n matrix behind C
    const int ld = k;
    k /= ksplits;
    PromptEpilogue pe = {};
    if (prompt) pe = *prompt;
    HeadsEpilogue he = {};
    if (heads) he = *heads;
    constexpr int E = BigTraits<T>::E;
    const int tm = (m + 64 * WM - 1) / (64 * WM), tn = (n + 64 * WN - 1) / (64 * WN);
    const long long total = (long long)tm * tn;
    if (total > (1ll << 30)) return hipErrorInvalidValue;
    const int per = (int)((total + 7) / 8);
    size_t lds = (size_t)2 * (64 * WM + 64 * WN) * (9 * E) * sizeof(T);
    const size_t ldsEpilogue = std::is_same<T, TC>::value ? (size_t)4 * 32 * (32 * WN + E) * sizeof(T) : (size_t)4 * 32 * (32 * WN + 4) * sizeof(float);
    if (ldsEpilogue > lds) lds = ldsEpilogue;
    static bool attr = false;   // per instantiation: allow more than the default 64 KB of dynamic LDS
    if (!attr) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_nt_big_kernel<T, WM, WN, OCC, HEADS, TC, SPLIT, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr = true;
    }
    // Bands of whole tile rows per XCD (tm divisible by 8): pick the column block so that the rows of A and B behind
    // one block of tiles stay under 3 MB of the XCD's 4 MB L2; 0 keeps the plain row-major walk of the band.
    int bandRows = 0, colBlock = 0;
    if (tm % 8 == 0 && tn > 1) {
        bandRows = tm / 8;
        const double rowBytes = 64.0 * WM * k * sizeof(T), colBytes = 64.0 * WN * k * sizeof(T), budget = 3.0 * 1024 * 1024;
        const int fit = (int)((budget - bandRows * rowBytes) / colBytes);
        if (fit >= 1 && fit < tn) {
            const int nb = (tn + fit - 1) / fit;
            colBlock = (tn + nb - 1) / nb;   // equal-width blocks
        }
    }
    hipLaunchKernelGGL((gemm_nt_big_kernel<T, WM, WN, OCC, HEADS, TC, SPLIT, EPI>), dim3(per * 8, ksplits), 256, lds, s, m, n, k, alpha, (const T*)A, (const T*)B, beta,
                       (TC*)C, tn, (int)total, bandRows, colBlock, he, pe, ld);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// NT, one 256 x 288 (WN = 9) or 256 x 192 (WN = 6) tile per workgroup and one workgroup per CU: 8192 x 2304 (the fused
// QKV projection of a 768-wide layer over 8192 tokens) is exactly 256 tiles of 256 x 288, one round of the chip, and a
// stage of K moves half the bytes per flop of the 128 x 128 tile from L2 to LDS.  Eight wavefronts stacked along M,
// 32 rows x 32 WN columns each (WN MFMA tiles, 144 accumulation registers at WN = 9), two per SIMD.
//   * Staging goes from global memory straight into LDS (global_load_lds_dwordx4: lane i of a wavefront lands 16 i bytes
//     past a wavefront-uniform address, so one instruction fills eight 128-byte rows): no staging registers and no
//     ds_write_b128, whose issue nothing covers when a SIMD holds one or two wavefronts.  Rows therefore lie 128 bytes
//     apart without padding, and the 16-byte piece c of row r is kept at position c ^ ((r >> 1) & 7) of its row (the
//     lane that fills position s of row r fetches piece s ^ ((r >> 1) & 7)): a 128-bit read serves sixteen lanes per
//     cycle out of 64 banks, and sixteen consecutive rows (two per 256 bytes of bank space) then fall on sixteen
//     different bank groups.
//   * A k-step is one A fragment and WN B fragments for WN tile products; only RB B fragments are held: fragment
//     f + RB - 1 of the (k-step, column) sequence is read while fragment f is multiplied.
// No edge handling: launched only where the tiles divide the matrix (wide_tile_fits).
template <typename T, int WN, bool HEADS>
__global__ __launch_bounds__(512, 1) void gemm_nt_wide_kernel(int M, int N, int K, float alpha, const T* __restrict__ A,
                                                               const T* __restrict__ B, T* __restrict__ C, int tilesN,
                                                               int tilesTotal, HeadsEpilogue he)
{
    typedef BigTraits<T> TR;
    constexpr int E = TR::E, BK = 8 * E, BM = 256, BN = 32 * WN, KS = 4;   // a stage is 128 bytes of every row
    constexpr int ROWS = BM + BN;                 // rows of one stage: A's 256, then B's 32 WN
    constexpr int STAGE = ROWS * BK;              // elements of one stage buffer
    constexpr int NP = (ROWS + 63) / 64;          // fetch instructions per thread and stage (a wavefront fills 8 rows with each)
    constexpr int RB = 5;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per = (tilesTotal + 7) / 8;         // each XCD (workgroup index mod 8) takes a contiguous run of tiles
    const int tile = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
    if (tile >= tilesTotal) return;
    const int m0 = (tile / tilesN) * BM, n0 = (tile % tilesN) * BN;
    const int wm = wave * 32;

    floatx16 acc[WN];
#pragma unroll
    for (int j = 0; j < WN; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[j][v] = 0.f;

    // fetch p of a stage: rows 64 p + 8 wave .. + 7 of the stage; this lane fills position tid & 7 of row 64 p + tid / 8.
    // The last fetch covers the 32 rows past a multiple of 64 only: wavefronts 0 .. 3.
    const int lr = tid >> 3;
    const int piece = ((tid & 7) ^ ((lr >> 1) & 7)) * E;
    const T* srcA = A + (size_t)(m0 + lr) * K + piece;
    const T* srcB = B + (size_t)(n0 + lr) * K + piece;
    const size_t passStride = (size_t)64 * K;
    auto fetch = [&](int p, int k0, T* stage) {
        if (p * 64 + wave * 8 >= ROWS) return;   // wavefront-uniform
        const T* src = p < BM / 64 ? srcA + p * passStride + k0 : srcB + (p - BM / 64) * passStride + k0;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(stage + (p * 64 + wave * 8) * BK), 16, 0, 0);
    };
    const int nk = K / BK;
#pragma unroll
    for (int p = 0; p < NP; p++) fetch(p, 0, smem);
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): the fetches have landed in LDS
    __syncthreads();

    // fragment of rows base + lane % 32, k-step ks: piece 2 ks + lane / 32, kept at position piece ^ ((row >> 1) & 7)
    const int fr = lane & 31, half = lane >> 5;
    int koff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) koff[ks] = ((2 * ks + half) ^ ((fr >> 1) & 7)) * E;
    const T* fa = smem + (wm + fr) * BK;
    const T* fb = smem + (BM + fr) * BK;
    u32x4 a[2], b[RB];
    for (int kt = 0; kt < nk; kt++) {
        const T* pa = fa + (kt & 1) * STAGE;
        const T* pb = fb + (kt & 1) * STAGE;
        T* next = smem + ((kt & 1) ^ 1) * STAGE;   // read during stage kt - 1; free since the barrier that ended it
        const int k1 = min(kt + 1, nk - 1) * BK;   // past the end the last stage is fetched again (valid memory, never read)
        a[0] = *(const u32x4*)(pa + koff[0]);
#pragma unroll
        for (int f = 0; f < RB - 1; f++) b[f] = *(const u32x4*)(pb + (f % WN) * 32 * BK + koff[f / WN]);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            // written in issue order, one scheduling region per tile product: the product, a fragment read, and with
            // each of the stage's first products one fetch of the next stage
#pragma unroll
            for (int j = 0; j < WN; j++) {
                acc[j] = TR::mma(b[(ks * WN + j) % RB], a[ks & 1], acc[j]);
                const int f = ks * WN + j + RB - 1, fks = f / WN, fj = f % WN;
                if (fks < KS) b[f % RB] = *(const u32x4*)(pb + fj * 32 * BK + koff[fks]);
                if (j == WN / 2 && ks + 1 < KS) a[(ks + 1) & 1] = *(const u32x4*)(pa + koff[ks + 1]);
                const int n = ks * WN + j;
                if (n < NP) fetch(n, k1, next);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
    }

    // Epilogue as in gemm_nt_big_kernel: the products are the transposed 32x32 tiles, a lane owns row lane % 32 and
    // register v is column 8 (v / 4) + 4 (lane / 32) + v % 4.  Each wavefront passes its 32 rows, CH tiles of columns at a
    // time (all of them in 16-bit storage, three in fp32: eight slices have to fit the LDS), through its own slice of LDS
    // (free after the last barrier) and stores 16-byte pieces, dealt to the lanes in row-major order.
    constexpr int CH = sizeof(T) == 2 ? WN : 3;
    static_assert(WN % CH == 0, "whole column chunks");
    constexpr int CW = 32 * CH, LDC = CW + E, LPR = CW / E, NIT = (32 * LPR) / 64;
    static_assert((32 * LPR) % 64 == 0, "the pieces of a 32-row block fill whole store instructions");
    const int row_l = lane & 31, col_l = (lane >> 5) * 4;
    T* cs = smem + wave * 32 * LDC;
#pragma unroll
    for (int c = 0; c < WN / CH; c++) {
#pragma unroll
        for (int jj = 0; jj < CH; jj++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int j = c * CH + jj;
                float b0 = 0.f, b1 = 0.f, b2 = 0.f, b3 = 0.f;
                if (HEADS && he.bias) {
                    const T* bp = (const T*)he.bias + n0 + j * 32 + 8 * g + col_l;
                    b0 = TR::ld(bp); b1 = TR::ld(bp + 1); b2 = TR::ld(bp + 2); b3 = TR::ld(bp + 3);
                }
                TR::st4(cs + row_l * LDC + jj * 32 + 8 * g + col_l, alpha * acc[j][4 * g] + b0, alpha * acc[j][4 * g + 1] + b1,
                        alpha * acc[j][4 * g + 2] + b2, alpha * acc[j][4 * g + 3] + b3);
            }
        // same wavefront wrote and reads, and writes the next chunk after it has read this one: LDS operations of one
        // wavefront complete in order
#pragma unroll 6
        for (int it = 0; it < NIT; it++) {
            const int id = it * 64 + lane, r = id / LPR, cc = (id - r * LPR) * E;
            const u32x4 v = *(const u32x4*)(cs + r * LDC + cc);
            if (HEADS) *(u32x4*)heads_dst<T>(he, m0 + wm + r, n0 + c * CW + cc) = heads_rope_piece<T>(he, m0 + wm + r, n0 + c * CW + cc, v);
            else *(u32x4*)(C + (size_t)(m0 + wm + r) * N + n0 + c * CW + cc) = v;
        }
    }
}

// The wide tiles have no edge handling and one workgroup per CU: they are used where they divide the matrix, fill whole
// rounds of the 256 CUs to at least 85 % and K is long enough to pay for the larger prologue and epilogue.  Returns the
// tile width in MFMA tiles (9: 256 x 288, 6: 256 x 192) or 0.
static int wide_tile_fits(int m, int n, int k, int stageElems, const void* A, const void* B, const void* C)
{
    if (m % 256 != 0 || k % stageElems != 0 || k < 8 * stageElems) return 0;
    if ((((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) != 0) return 0;
    for (int wn : {9, 6}) {
        if (n % (32 * wn) != 0) continue;
        const long long tiles = (long long)(m / 256) * (n / (32 * wn)), rounds = (tiles + 255) / 256;
        if (tiles <= (1ll << 30) && tiles * 100 >= rounds * 256 * 85) return wn;
    }
    return 0;
}

template <typename T, int WN, bool HEADS>
static hipError_t launch_wide(hipStream_t s, int m, int n, int k, float alpha, const void* A, const void* B, void* C,
                              const HeadsEpilogue* heads = nullptr)
{
    HeadsEpilogue he = {};
    if (heads) he = *heads;
    constexpr int BN = 32 * WN, E = BigTraits<T>::E, CH = sizeof(T) == 2 ? WN : 3;
    const int tm = m / 256, tn = n / BN, total = tm * tn, per = (total + 7) / 8;
    // two stages of (256 + BN) rows x 128 bytes, or the epilogue's eight slices of 32 x (32 CH + E) elements, whichever is larger
    const size_t lds = std::max((size_t)2 * (256 + BN) * 128, (size_t)8 * 32 * (32 * CH + E) * sizeof(T));
    static bool attr = false;   // per instantiation: allow more than the default 64 KB of dynamic LDS
    if (!attr) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_nt_wide_kernel<T, WN, HEADS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
        attr = true;
    }
    hipLaunchKernelGGL((gemm_nt_wide_kernel<T, WN, HEADS>), dim3(per * 8), 512, lds, s, m, n, k, alpha, (const T*)A, (const T*)B,
                       (T*)C, tn, total, he);
    return hipGetLastError();
}

// Fewer 128 x 128 tiles than CUs: 64 x 128 tiles if they give every CU one, 64 x 64 otherwise (three or four of these
// small workgroups fit a CU, so more tiles than CUs is welcome).
template <typename T, bool HEADS>
static bool launch_small_if_few(hipError_t* e, hipStream_t s, int m, int n, int k, float alpha, const void* A, const void* B, float beta, void* C,
                                const HeadsEpilogue* heads = nullptr)
{
    const long long t128 = (long long)((m + 127) / 128) * ((n + 127) / 128);
    if (t128 >= 200) return false;
    const long long t64x128 = (long long)((m + 63) / 64) * ((n + 127) / 128);
    if (t64x128 >= 200) *e = launch_big<T, 1, 2, 3, HEADS>(s, m, n, k, alpha, A, B, beta, C, heads);
    else *e = launch_big<T, 1, 1, 3, HEADS>(s, m, n, k, alpha, A, B, beta, C, heads);
    return true;
}

// fp32 keeps the matrix cores busy with 128 x 128 tiles as well (512 of them fill the chip at two workgroups per CU) and
// measures 3 % faster with them when their rounds are full or half full; the wide tile wins (8192 x 2304 x 768: 232 ->
// 214 us) where the last round of 128 x 128 tiles would be mostly empty.
static bool short_last_round(long long t128)
{
    const long long rem = t128 % 512;
    return rem != 0 && rem * 10 < 512 * 4;
}

// one stage of K is 128 bytes of a row: 64 elements in 16-bit storage, 32 in fp32
template <typename T, bool HEADS>
static bool launch_wide_if_fits(hipError_t* e, hipStream_t s, int m, int n, int k, float alpha, const void* A, const void* B, void* C,
                                const HeadsEpilogue* heads = nullptr)
{
    switch (wide_tile_fits(m, n, k, 8 * BigTraits<T>::E, A, B, C)) {
    case 9: *e = launch_wide<T, 9, HEADS>(s, m, n, k, alpha, A, B, C, heads); return true;
    case 6: *e = launch_wide<T, 6, HEADS>(s, m, n, k, alpha, A, B, C, heads); return true;
    }
    return false;
}

// K = 1: the rank-1 update C[i,j] = alpha a[i] b[j] + beta C[i,j] that InnerProductLayer uses to add its bias
// (ones (M,1) x bias (1,N), InnerProductLayer.cs:405-414): one streaming pass over C, four columns per thread
template <typename T> struct Quad;
template <> struct Quad<float> {
    __device__ static inline void load(const float* p, float (&v)[4]) { const float4 a = *(const float4*)p; v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; }
    __device__ static inline void store(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Quad<bf16_t> {
    __device__ static inline void load(const bf16_t* p, float (&v)[4])
    {
        const uint2 a = *(const uint2*)p;
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
    }
    __device__ static inline void store(bf16_t* p, const float (&v)[4]) { *(uint2*)p = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3])); }
};
template <typename T, bool VEC>
__global__ void gemm_rank1_kernel(int m, int n, float alpha, const T* __restrict__ a, const T* __restrict__ b, float beta, T* C)
{
    const size_t total = (size_t)m * n;
    const size_t items = VEC ? total / 4 : total;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < items; e += (size_t)blockDim.x * gridDim.x) {
        if (VEC) {
            const size_t idx = e * 4;
            const int i = (int)(idx / n), j = (int)(idx % n);
            const float ai = alpha * ldf(a, i);
            float bv[4], cv[4];
            Quad<T>::load(b + j, bv);
            if (beta != 0.f) Quad<T>::load(C + idx, cv);
#pragma unroll
            for (int q = 0; q < 4; q++) cv[q] = beta != 0.f ? ai * bv[q] + beta * cv[q] : ai * bv[q];
            Quad<T>::store(C + idx, cv);
        } else {
            const int i = (int)(e / n), j = (int)(e % n);
            float v = alpha * ldf(a, i) * ldf(b, j);
            if (beta != 0.f) v += beta * ldf(C, e);
            stf(C, e, v);
        }
    }
}

// Fallback of the fused QKV projection: the plain product in `tmp` (M x 3C) is split, bias added, into the three
// (B,H,T,hs) tensors in one pass.
template <typename T>
__global__ void qkv_split_heads_kernel(const T* __restrict__ tmp, size_t total, int N, HeadsEpilogue he)
{
    // one pair of adjacent columns per step (hs is even when the rotation is asked for; otherwise N may be odd)
    const bool pairs = he.fcos != nullptr;
    const size_t steps = pairs ? total / 2 : total;
    for (size_t s = (size_t)blockIdx.x * blockDim.x + threadIdx.x; s < steps; s += (size_t)blockDim.x * gridDim.x) {
        const size_t i = pairs ? 2 * s : s;
        const int r = (int)(i / N), c = (int)(i - (size_t)r * N);
        float o = ldf(tmp, i);
        if (he.bias) o += ldf((const T*)he.bias, c);
        T* dp = heads_dst<T>(he, r, c);
        if (!pairs) { stf(dp, 0, o); continue; }
        float o1 = ldf(tmp, i + 1);
        if (he.bias) o1 += ldf((const T*)he.bias, c + 1);
        if (c < 2 * he.H * he.hs) {
            stf(dp, 0, o); stf(dp, 1, o1);
            o = ldf(dp, 0); o1 = ldf(dp, 1);                       // the values as the storage type holds them
            const size_t ti = (size_t)(r % he.seq) * (he.hs >> 1) + ((c % he.hs) >> 1);
            heads_rope_pair(he.fcos[ti], he.fsin[ti], o, o1);
        }
        stf(dp, 0, o); stf(dp, 1, o1);
    }
}

// X (m x kk) W^T (n x kk) through the tile kernels' HEADS epilogue `he`, or through `tmp` (m x n) and the splitting pass
// whether a product with these operands goes through the scratch matrix (shapes and addresses the tile kernels do not take)
static bool gemm_heads_through_tmp(DType dt, int kk, int rowUnit, const void* X, const void* W, const void* d0, const void* d1, const void* d2)
{
    const int vec = dt == F32 ? 4 : 8;
    const bool aligned = (((uintptr_t)X | (uintptr_t)W | (uintptr_t)d0 | (uintptr_t)d1 | (uintptr_t)d2) % 16 == 0) && rowUnit % vec == 0;
    return !(aligned && kk % (dt == F32 ? 32 : 64) == 0);
}
bool k_gemm_bias_needs_tmp(DType dt, int n, int k, const void* X, const void* W, const void* Y)
{
    return gemm_heads_through_tmp(dt, k, n, X, W, Y, Y, Y);
}
bool k_gemm_qkv_heads_needs_tmp(DType dt, int H, int hs, const void* X, const void* W, const void* q, const void* k, const void* v)
{
    return gemm_heads_through_tmp(dt, H * hs, hs, X, W, q, k, v);
}

// (tiles256: the 256 x 256 tiles may be chosen as k_gemm chooses them)
static hipError_t gemm_heads_dispatch(hipStream_t s, DType dt, int m, int n, int kk, const void* X, const void* W, const HeadsEpilogue& he,
                                      int rowUnit, void* tmp, bool tiles256)
{
    const long long t256 = (long long)((m + 255) / 256) * ((n + 255) / 256);
    const bool full256 = tiles256 && (double)t256 / (double)(((t256 + 255) / 256) * 256) >= 0.85;
    const bool aligned = !gemm_heads_through_tmp(dt, kk, rowUnit, X, W, he.dst[0], he.dst[1], he.dst[2]);   // and K in whole stages
    const long long t128 = (long long)((m + 127) / 128) * ((n + 127) / 128);
    if (aligned && dt == F32) {
        hipError_t e;
        if (full256 && kk >= 1024) return launch_big<float, 4, 4, 1, true>(s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he);
        if (launch_small_if_few<float, true>(&e, s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he)) return e;
        if (n % 192 == 0 && t128 <= 512) return launch_big<float, 2, 3, 2, true>(s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he);
        if (short_last_round(t128) && launch_wide_if_fits<float, true>(&e, s, m, n, kk, 1.f, X, W, nullptr, &he)) return e;
        return launch_big<float, 2, 2, 2, true>(s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he);
    }
    if (aligned && dt == BF16) {
        hipError_t e;
        if (full256 && kk >= 2048) return launch_big<bf16_t, 4, 4, 1, true>(s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he);
        if (launch_wide_if_fits<bf16_t, true>(&e, s, m, n, kk, 1.f, X, W, nullptr, &he)) return e;
        if (launch_small_if_few<bf16_t, true>(&e, s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he)) return e;
        if (n % 192 == 0 && t128 <= 512) return launch_big<bf16_t, 2, 3, 2, true>(s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he);
        return launch_big<bf16_t, 2, 2, 2, true>(s, m, n, kk, 1.f, X, W, 0.f, nullptr, &he);
    }
    // any other shape: plain product into the caller's scratch matrix, then one splitting pass
    if (!tmp) return hipErrorInvalidValue;
    hipError_t e = k_gemm(s, dt, false, true, m, n, kk, 1.f, X, W, 0.f, tmp);
    if (e != hipSuccess) return e;
    const size_t total = (size_t)m * n;
    const int grid = (int)std::min<size_t>((total + 255) / 256, 8192);
    if (dt == F32) hipLaunchKernelGGL(qkv_split_heads_kernel<float>, grid, 256, 0, s, (const float*)tmp, total, n, he);
    else hipLaunchKernelGGL(qkv_split_heads_kernel<bf16_t>, grid, 256, 0, s, (const bf16_t*)tmp, total, n, he);
    return hipGetLastError();
}

hipError_t k_gemm_qkv_heads(hipStream_t s, DType dt, int B, int T, int H, int hs, const void* X, const void* W, const void* bias,
                            void* q, void* k, void* v, void* tmp, const float* fcos, const float* fsin, int ropeSeq)
{
    if (fcos && (!fsin || ropeSeq < 1 || (hs & 1))) return hipErrorInvalidValue;
    const int m = B * T, C = H * hs, n = 3 * C, kk = C;
    if (m <= 0 || C <= 0) return hipSuccess;
    HeadsEpilogue he;
    he.bias = bias; he.dst[0] = q; he.dst[1] = k; he.dst[2] = v; he.T = T; he.H = H; he.hs = hs;
    he.fcos = fcos; he.fsin = fcos ? fsin : nullptr; he.seq = fcos ? ropeSeq : 1;
    return gemm_heads_dispatch(s, dt, m, n, kk, X, W, he, hs, tmp, false);
}

// Y (m x n) = X (m x k) W^T (n x k) + bias (n): the inner product layer's forward in one launch (InnerProductLayer.cs:
// 372-417 issues the product and a rank-1 update with a vector of ones).  The HEADS epilogue with one head of n values
// over m positions is the plain row-major layout, so the same kernels serve.
hipError_t k_gemm_bias(hipStream_t s, DType dt, int m, int n, int k, const void* X, const void* W, const void* bias, void* Y, void* tmp)
{
    if (m <= 0 || n <= 0) return hipSuccess;
    HeadsEpilogue he;
    he.bias = bias; he.dst[0] = he.dst[1] = he.dst[2] = Y; he.T = m; he.H = 1; he.hs = n;
    he.fcos = nullptr; he.fsin = nullptr; he.seq = 1;
    return gemm_heads_dispatch(s, dt, m, n, k, X, W, he, n, tmp, true);
}

// C (m x n, fp32) = alpha X W^T + beta C for a 16-bit weight matrix W (n x k), on the bf16 matrix cores, C in fp32.
// split = false: A is X rounded to bf16, m rows of k.  split = true keeps the activations' precision: A holds every row of
// an fp32 X as two bf16 rows back to back, the bf16 nearest to each of its k values and then the bf16 nearest to what
// those leave over, and the kernel walks W once for each.  The products are exact and accumulate in fp32, so what is lost
// is the part of X below its leading sixteen bits: 2^-17 relative, against 2^-9 for activations rounded to bf16.
// k a multiple of 64, 16-byte aligned operands.
template <bool SPLIT, int EPI>
static hipError_t gemm_bf16_f32_tiles(hipStream_t s, int m, int n, int k, float alpha, const void* A, const void* W, float beta, float* C,
                                      const PromptEpilogue* pe)
{
    // Tile shapes as k_gemm picks them for bf16: below 200 tiles of 128 x 128, 64 x 128 tiles where they give every CU
    // one, else 64 x 64 (2048 x 768: 384 tiles of 64 x 64 measure 27.8 us a product, 192 of 64 x 128 30.1 us).
    const long long t128 = (long long)((m + 127) / 128) * ((n + 127) / 128);
    if (t128 < 200) {
        const long long t64x128 = (long long)((m + 63) / 64) * ((n + 127) / 128);
        if (t64x128 >= 200) return launch_big<bf16_t, 1, 2, 3, false, float, SPLIT, EPI>(s, m, n, k, alpha, A, W, beta, C, nullptr, pe);
        return launch_big<bf16_t, 1, 1, 3, false, float, SPLIT, EPI>(s, m, n, k, alpha, A, W, beta, C, nullptr, pe);
    }
    if (n % 192 == 0 && t128 <= 512) return launch_big<bf16_t, 2, 3, 2, false, float, SPLIT, EPI>(s, m, n, k, alpha, A, W, beta, C, nullptr, pe);
    return launch_big<bf16_t, 2, 2, 2, false, float, SPLIT, EPI>(s, m, n, k, alpha, A, W, beta, C, nullptr, pe);
}
static bool bf16_f32_operands_ok(int k, const void* A, const void* W) { return k > 0 && k % 64 == 0 && (((uintptr_t)A | (uintptr_t)W) & 15) == 0; }
hipError_t k_gemm_bf16_f32(hipStream_t s, int m, int n, int k, float alpha, const void* A, bool split, const void* W, float beta, float* C)
{
    if (m <= 0 || n <= 0) return hipSuccess;
    if (!bf16_f32_operands_ok(k, A, W)) return hipErrorInvalidValue;
    return split ? gemm_bf16_f32_tiles<true, 0>(s, m, n, k, alpha, A, W, beta, C, nullptr) : gemm_bf16_f32_tiles<false, 0>(s, m, n, k, alpha, A, W, beta, C, nullptr);
}
// out (m x hid) = silu(X W1^T) (X W3^T) for the stacked 16-bit W13 (2 hid x k), as bf16 rows (outSplit: hi | lo rows)
hipError_t k_gemm_bf16_swiglu(hipStream_t s, int m, int hid, int k, const void* A, bool split, const void* W13, void* out, bool outSplit)
{
    if (m <= 0 || hid <= 0) return hipSuccess;
    if (!bf16_f32_operands_ok(k, A, W13) || (hid & 1) || (((uintptr_t)out) & 3)) return hipErrorInvalidValue;
    PromptEpilogue pe = {};
    pe.out = out; pe.hid = hid; pe.split = outSplit ? 1 : 0;
    return split ? gemm_bf16_f32_tiles<true, 1>(s, m, 2 * hid, k, 1.f, A, W13, 0.f, nullptr, &pe) : gemm_bf16_f32_tiles<false, 1>(s, m, 2 * hid, k, 1.f, A, W13, 0.f, nullptr, &pe);
}
// the stacked 16-bit Wqkv ((H + 2 kvH) hs x k) product of B x P rows, rotated and scattered (PromptEpilogue, EPI 2)
hipError_t k_gemm_bf16_qkv_rope(hipStream_t s, int B, int P, int H, int kvH, int hs, int k, const void* A, bool split, const void* Wqkv,
                                void* q, void* kh, void* vh, bool heads16, void* kc, void* vc, bool cache16, int seqLen,
                                const float* fcos, const float* fsin)
{
    const int m = B * P, n = (H + 2 * kvH) * hs;
    if (m <= 0 || n <= 0) return hipSuccess;
    if (!bf16_f32_operands_ok(k, A, Wqkv) || (hs & 3) || kvH <= 0 || H % kvH != 0) return hipErrorInvalidValue;
    if ((((uintptr_t)q | (uintptr_t)kh | (uintptr_t)vh | (uintptr_t)kc | (uintptr_t)vc) & 15) != 0) return hipErrorInvalidValue;
    PromptEpilogue pe = {};
    pe.q = q; pe.k = kh; pe.v = vh; pe.kc = kc; pe.vc = vc; pe.fcos = fcos; pe.fsin = fsin;
    pe.P = P; pe.H = H; pe.kvH = kvH; pe.hs = hs; pe.seqLen = seqLen; pe.heads16 = heads16 ? 1 : 0; pe.cache16 = cache16 ? 1 : 0;
    pe.kvMul = H / kvH; pe.invP = 1.0f / (float)P; pe.invHs = 1.0f / (float)hs;
    if (m >= (1 << 24) || n >= (1 << 24)) return hipErrorInvalidValue;
    return split ? gemm_bf16_f32_tiles<true, 2>(s, m, n, k, 1.f, A, Wqkv, 0.f, nullptr, &pe) : gemm_bf16_f32_tiles<false, 2>(s, m, n, k, 1.f, A, Wqkv, 0.f, nullptr, &pe);
}

// (rows, cols) -> (cols, rows), 64 x 64 elements per workgroup: 16-byte pieces in, a padded LDS tile, 16-byte pieces out
// (rows and cols multiples of 16 bytes' worth of elements; edge tiles are clipped piece by piece)
template <typename T>
__global__ __launch_bounds__(256) void transpose2d_kernel(const T* __restrict__ x, T* __restrict__ y, int rows, int cols)
{
    constexpr int E = 16 / sizeof(T), PPR = 64 / E, NP = 64 * PPR / 256;   // elements per piece, pieces per tile row, pieces per thread
    __shared__ T tile[64][64 + (sizeof(T) == 2 ? 2 : 1)];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int p = threadIdx.x + 256 * i, r = p / PPR, c = (p % PPR) * E;
        if (r0 + r < rows && c0 + c < cols) {
            const u32x4 v = *(const u32x4*)(x + (size_t)(r0 + r) * cols + c0 + c);
            const T* e = reinterpret_cast<const T*>(&v);
#pragma unroll
            for (int j = 0; j < E; j++) tile[r][c + j] = e[j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NP; i++) {
        const int p = threadIdx.x + 256 * i, c = p / PPR, r = (p % PPR) * E;   // output row c0 + c, columns r0 + r ..
        if (c0 + c < cols && r0 + r < rows) {
            u32x4 v;
            T* e = reinterpret_cast<T*>(&v);
#pragma unroll
            for (int j = 0; j < E; j++) e[j] = tile[r + j][c];
            *(u32x4*)(y + (size_t)(c0 + c) * rows + r0 + r) = v;
        }
    }
}

static hipError_t transpose2d(hipStream_t s, DType dt, const void* x, void* y, int rows, int cols)
{
    dim3 grid((cols + 63) / 64, (rows + 63) / 64);
    if (grid.y > 65535) return hipErrorInvalidValue;
    if (dt == F32) hipLaunchKernelGGL(transpose2d_kernel<float>, grid, 256, 0, s, (const float*)x, (float*)y, rows, cols);
    else hipLaunchKernelGGL(transpose2d_kernel<bf16_t>, grid, 256, 0, s, (const bf16_t*)x, (bf16_t*)y, rows, cols);
    return hipGetLastError();
}

// The transpose combinations other than A B^T (InnerProductLayer backward: data gradient dY W, weight gradient dY^T X,
// InnerProductLayer.cs:429-494).  The tile kernels want both operands with the contracted index at unit stride; an
// operand that lies the other way is turned once into scratch memory and the product then runs on them.  In 16-bit
// storage that replaces the strided scalar kernel (8192 x 768 x 2304: 604 -> 36 us, the weight gradient 1778 -> 63 us),
// in fp32 the strided MFMA kernel where the product is large enough to pay for the pass over the operand.
static size_t round256(size_t b) { return (b + 255) & ~(size_t)255; }

// A long contraction with few tiles (weight gradients: K is the token count) is cut into 2 .. 16 equal parts, one row of
// workgroups of 128 x 128 tiles each, until the launch has some 400 workgroups; every part stays 512 long at least.
static int gemm_ksplits(DType dt, int m, int n, int k)
{
    const int bk = dt == F32 ? 32 : 64;
    const long long t128 = (long long)((m + 127) / 128) * ((n + 127) / 128);
    if (t128 >= 200 || k < 2048 || ((long long)m * n) % 4) return 1;
    int S = 1;
    while (S < 16 && t128 * S < 400 && k % (2 * S * bk) == 0 && k / (2 * S) >= 512) S *= 2;
    return S;
}
// C = sum of the S partial products (fp32, alpha already applied) + beta C
template <typename T>
__global__ void splitk_reduce_kernel(const float* __restrict__ part, int S, size_t total4, float beta, T* __restrict__ C)
{
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total4; e += (size_t)blockDim.x * gridDim.x) {
        float4 a = *(const float4*)(part + 4 * e);
        for (int z = 1; z < S; z++) {
            const float4 b = *(const float4*)(part + (size_t)z * total4 * 4 + 4 * e);
            a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        float v[4] = {a.x, a.y, a.z, a.w};
        if (beta != 0.f) {
            float c[4];
            Quad<T>::load(C + 4 * e, c);
#pragma unroll
            for (int q = 0; q < 4; q++) v[q] += beta * c[q];
        }
        Quad<T>::store(C + 4 * e, v);
    }
}
static bool gemm_turns_operands(DType dt, bool tA, bool tB, int m, int n, int k)
{
    if (!tA && tB) return false;
    const int vec = dt == F32 ? 4 : 8;
    if (k < 64 || k % vec || (tA && m % vec) || (!tB && n % vec)) return false;
    const double turned = (tA ? (double)m * k : 0.0) + (!tB ? (double)n * k : 0.0);
    if (dt == BF16) return (double)m * n >= 64.0 * 64.0;
    // fp32: 136 against 88 TFLOP/s for the product, about 3 TB/s (read + write) for the pass over an operand
    // Also where the strided kernel would split a long contraction over workgroups that add their parts with atomics
    // (few tiles, K of 2048 and more): here the parts are summed in a fixed order, so a weight gradient comes out the
    // same bits every run, at the same speed to within a few per cent.
    if ((long long)((m + 127) / 128) * ((n + 127) / 128) < 256 && k >= 2048) return true;
    return (double)m * n * k * 8.0e-15 > 1.5 * turned * 8.0 / 3.0e12;
}
static size_t gemm_turned_bytes(DType dt, bool tA, bool tB, int m, int n, int k)
{
    const size_t es = dt == F32 ? 4 : 2;
    return (tA ? round256((size_t)m * k * es) : 0) + (!tB ? round256((size_t)n * k * es) : 0);
}
size_t k_gemm_workspace_bytes(DType dt, bool tA, bool tB, int m, int n, int k)
{
    if (m <= 0 || n <= 0 || k <= 0) return 0;
    const bool nt = !tA && tB;
    if (!nt && !gemm_turns_operands(dt, tA, tB, m, n, k)) return 0;
    const int S = k % (dt == F32 ? 4 : 8) == 0 ? gemm_ksplits(dt, m, n, k) : 1;
    return (nt ? 0 : gemm_turned_bytes(dt, tA, tB, m, n, k)) + (S > 1 ? (size_t)S * m * n * sizeof(float) : 0);
}

hipError_t k_gemm(hipStream_t s, DType dt, bool tA, bool tB, int m, int n, int k, float alpha, const void* A,
                  const void* B, float beta, void* C, void* ws, size_t wsBytes)
{
    if (m <= 0 || n <= 0) return hipSuccess;
    if (ws && k > 1 && (((uintptr_t)A | (uintptr_t)B | (uintptr_t)ws) % 16 == 0) && gemm_turns_operands(dt, tA, tB, m, n, k) &&
        wsBytes >= k_gemm_workspace_bytes(dt, tA, tB, m, n, k)) {
        const size_t es = dt == F32 ? 4 : 2;
        const void *a2 = A, *b2 = B;
        char* w = (char*)ws;
        if (tA) {   // stored (k, m)
            hipError_t e = transpose2d(s, dt, A, w, k, m);
            if (e != hipSuccess) return e;
            a2 = w;
            w += round256((size_t)m * k * es);
        }
        if (!tB) {  // stored (k, n)
            hipError_t e = transpose2d(s, dt, B, w, k, n);
            if (e != hipSuccess) return e;
            b2 = w;
            w += round256((size_t)n * k * es);
        }
        return k_gemm(s, dt, false, true, m, n, k, alpha, a2, b2, beta, C, w, wsBytes - (size_t)(w - (char*)ws));
    }
    if (k == 1) {
        const size_t es = dt == F32 ? 4 : 2;
        const bool vec = n % 4 == 0 && ((((uintptr_t)B | (uintptr_t)C) & (4 * es - 1)) == 0);
        const size_t items = vec ? (size_t)m * n / 4 : (size_t)m * n;
        const int g = (int)std::min<size_t>((items + 255) / 256, 256 * 16);
#define RANK1(TT, V) hipLaunchKernelGGL((gemm_rank1_kernel<TT, V>), g, 256, 0, s, m, n, alpha, (const TT*)A, (const TT*)B, beta, (TT*)C)
        if (dt == F32) { if (vec) RANK1(float, true); else RANK1(float, false); }
        else { if (vec) RANK1(bf16_t, true); else RANK1(bf16_t, false); }
#undef RANK1
        return hipGetLastError();
    }
    if (m <= 0 || n <= 0) return hipSuccess;
    if (k <= 0) k = 0;
    // MFMA fast path: A (m,k) and B (n,k) both k-contiguous, 16-byte aligned rows
    const int vec = dt == F32 ? 4 : 8;
    bool aligned = (k % vec == 0) && (((uintptr_t)A | (uintptr_t)B) % 16 == 0) && k >= vec;
    if (!tA && tB && aligned) {
        dim3 grid((n + 127) / 128, (m + 127) / 128);
        if (grid.y > 65535) return hipErrorInvalidValue;
        // Large-tile kernels need whole 128-byte stages along K.  256 x 256 tiles (one wavefront per SIMD, 128 x 128
        // per wavefront) win once K is long enough to amortise their prologue and the tile count fills the 256 CUs
        // evenly; 128 x 128 tiles with two workgroups per CU otherwise, 128 x 192 when that gives at most one round
        // of workgroups.
        const long long t256 = (long long)((m + 255) / 256) * ((n + 255) / 256);
        const double fill = (double)t256 / (double)(((t256 + 255) / 256) * 256);
        const long long t128 = (long long)((m + 127) / 128) * ((n + 127) / 128);
        const int S = ws && (((uintptr_t)ws | (uintptr_t)C) % 16 == 0) ? gemm_ksplits(dt, m, n, k) : 1;
        if (S > 1 && wsBytes >= (size_t)S * m * n * sizeof(float)) {
            hipError_t e = dt == F32 ? launch_big<float, 2, 2, 2>(s, m, n, k, alpha, A, B, 0.f, ws, nullptr, nullptr, S)
                                     : launch_big<bf16_t, 2, 2, 2, false, float>(s, m, n, k, alpha, A, B, 0.f, ws, nullptr, nullptr, S);
            if (e != hipSuccess) return e;
            const size_t total4 = (size_t)m * n / 4;
            const int g = (int)std::min<size_t>((total4 + 255) / 256, 4096);
            if (dt == F32) hipLaunchKernelGGL(splitk_reduce_kernel<float>, g, 256, 0, s, (const float*)ws, S, total4, beta, (float*)C);
            else hipLaunchKernelGGL(splitk_reduce_kernel<bf16_t>, g, 256, 0, s, (const float*)ws, S, total4, beta, (bf16_t*)C);
            return hipGetLastError();
        }
        if (dt == F32) {
            if (k % 32 == 0) {
                if (k >= 1024 && fill >= 0.85) return launch_big<float, 4, 4, 1>(s, m, n, k, alpha, A, B, beta, C);
                hipError_t e;
                if (launch_small_if_few<float, false>(&e, s, m, n, k, alpha, A, B, beta, C)) return e;
                if (n % 192 == 0 && t128 <= 512) return launch_big<float, 2, 3, 2>(s, m, n, k, alpha, A, B, beta, C);
                if (beta == 0.f && short_last_round(t128) && launch_wide_if_fits<float, false>(&e, s, m, n, k, alpha, A, B, C)) return e;
                return launch_big<float, 2, 2, 2>(s, m, n, k, alpha, A, B, beta, C);
            }
            hipLaunchKernelGGL(gemm_nt_f32_mfma_kernel, grid, 256, 0, s, m, n, k, alpha, (const float*)A, (const float*)B,
                               beta, (float*)C);
        } else {
            if (k % 64 == 0) {
                if (k >= 2048 && fill >= 0.85) return launch_big<bf16_t, 4, 4, 1>(s, m, n, k, alpha, A, B, beta, C);
                hipError_t e;
                if (beta == 0.f && launch_wide_if_fits<bf16_t, false>(&e, s, m, n, k, alpha, A, B, C)) return e;
                if (launch_small_if_few<bf16_t, false>(&e, s, m, n, k, alpha, A, B, beta, C)) return e;
                if (n % 192 == 0 && t128 <= 512) return launch_big<bf16_t, 2, 3, 2>(s, m, n, k, alpha, A, B, beta, C);
                return launch_big<bf16_t, 2, 2, 2>(s, m, n, k, alpha, A, B, beta, C);
            }
            hipLaunchKernelGGL(gemm_nt_bf16_mfma_kernel, grid, 256, 0, s, m, n, k, alpha, (const bf16_t*)A,
                               (const bf16_t*)B, beta, (bf16_t*)C);
        }
        return hipGetLastError();
    }
    GemmStrides st;
    st.ai = tA ? 1 : k;  st.ak = tA ? m : 1;   // A stored (m,k) or (k,m)
    st.bk = tB ? 1 : n;  st.bj = tB ? k : 1;   // B stored (k,n) or (n,k)
    st.ci = n;           st.cj = 1;
    st.sA = st.sB = st.sC = 0;
    if (dt == F32 && k > 0) {
        // the other transpose combinations (InnerProductLayer backward: weight gradient dY^T X, data gradient dY W) run on
        // the strided fp32 MFMA kernel: row-major C = op(A) op(B) is column-major C^T = op(B)^T op(A)^T
        return k_gemm2(s, tB, tA, n, m, k, alpha, (const float*)B, (const float*)A, beta, (float*)C, tB ? k : n, tA ? m : k, n, 0, 0, 0, 1);
    }
    if (dt == F32)
        return launch_generic<float>(s, m, n, k, alpha, (const float*)A, (const float*)B, beta, (float*)C, st, 1);
    return launch_generic<bf16_t>(s, m, n, k, alpha, (const bf16_t*)A, (const bf16_t*)B, beta, (bf16_t*)C, st, 1);
}

// ---------------------------------------------------------------------------
// fp32 MFMA for the strided-batched gemm2 (the Blob.MatMul route of the explicit attention chain: Q K^T and P V per
// (batch, head), math.cu:1750-1788).  Column-major operands with any leading dimension: A(i,k) has either i or k at unit
// stride, B(k,j) either k or j, C(i,j) has i at unit stride.  An operand with k at unit stride is staged into LDS as
// [row][k], so that one 128-bit LDS read feeds four v_mfma_f32_32x32x2_f32 steps (slot trick as in
// gemm_nt_f32_mfma_kernel); one with the row index at unit stride is staged as it lies, [k][row], and a lane gathers its
// four k with 32-bit reads (consecutive lanes, consecutive words: no bank conflicts on either side).  The MFMA row operand is B and the column
// operand is A: the accumulator then has i in the lane and every store instruction of a wavefront writes two 128-byte
// runs of C.  TI x TJ tile (i x j), four wavefronts 2 x 2.
template <bool A_IFAST, bool B_KFAST, int TI, int TJ>
__global__ __launch_bounds__(256) void gemm2_f32_mfma_kernel(int M, int N, int K, float alpha, const float* __restrict__ A,
                                                             const float* __restrict__ B, float beta, float* __restrict__ C,
                                                             GemmStrides st, int splits, int kChunk, const int* causalFlag, int epoch)
{
    // B(k,j) known to be zero for k > j (the probabilities of a causal softmax, unless the flag carries this launch's
    // epoch): the contraction of this tile of columns stops at its last column
    // Tiles of columns then differ in length.  Consecutive workgroups go to consecutive dies, and workgroup i shares its CU
    // with i + 256, i + 512, ... (all are resident at once): the tile a workgroup takes is rotated by its batch index, so
    // that no die is left with the long ones, and every other round of 256 takes them in reverse, so that a long tile
    // meets a short one on its CU.
    int jTile = blockIdx.y;
    if (causalFlag) {
        // (decided per batch index, so that the tiles of one batch entry are still each taken once)
        const unsigned first = gridDim.x * gridDim.y * blockIdx.z;
        jTile = (int)((blockIdx.y + blockIdx.z) % gridDim.y);
        if ((first >> 8) & 1) jTile = (int)gridDim.y - 1 - jTile;
    }
    // (B given transposed, B(k,j) stored as [k][j]: the same tensor read the other way, zero for k < j - the product with the
    // transposed probabilities in the backward pass - and the contraction begins at the tile's first column instead)
    const bool causal = causalFlag && *causalFlag != epoch;
    if (causal && B_KFAST) K = min(K, (jTile + 1) * TJ);
    constexpr int BK = 16, LDK = BK + 4;
    constexpr int LDI = TI + 4, LDJ = TJ + 4;        // row strides of the [k][row] layouts
    constexpr int NI = TI / 64, NJ = TJ / 64;        // 32x32 blocks per wavefront along i and j
    __shared__ __attribute__((aligned(16))) float Is[2][A_IFAST ? BK * LDI : TI * LDK];   // A: [k][i] or [i][k]
    __shared__ __attribute__((aligned(16))) float Js[2][B_KFAST ? TJ * LDK : BK * LDJ];   // B: [j][k] or [k][j]
    // blockIdx.z = batch * splits + split; with splits > 1 every workgroup covers kChunk of the contraction and adds its
    // part to C with float atomics (C holds beta * C already)
    const int batchIdx = blockIdx.z / splits, split = blockIdx.z % splits;
    const int kBegin = (causal && !B_KFAST) ? min(K, jTile * TJ) : split * kChunk;
    if (splits > 1) K = min(K, kBegin + kChunk);
    A += (size_t)batchIdx * st.sA;
    B += (size_t)batchIdx * st.sB;
    C += (size_t)batchIdx * st.sC;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave & 1) * (TI / 2), wj = (wave >> 1) * (TJ / 2);
    const int i0 = blockIdx.x * TI, j0 = jTile * TJ;
    const long long lda = A_IFAST ? st.ak : st.ai, ldb = B_KFAST ? st.bj : st.bk;

    floatx16 acc[NJ][NI];
#pragma unroll
    for (int a = 0; a < NJ; a++)
#pragma unroll
        for (int b = 0; b < NI; b++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[a][b][v] = 0.f;

    // staging: TI*BK/4 float4 of A and TJ*BK/4 of B per stage, 256 threads
    constexpr int PA = TI * BK / 4 / 256, PB = TJ * BK / 4 / 256;
    float4 ra[PA], rb[PB];
    auto gload = [&](int k0) {
#pragma unroll
        for (int p = 0; p < PA; p++) {
            const int e = tid + p * 256;
            ra[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (A_IFAST) {   // four consecutive i at one k
                const int ig = e % (TI / 4), k = e / (TI / 4);
                if (i0 + 4 * ig < M && k0 + k < K) ra[p] = *(const float4*)(A + (size_t)(i0 + 4 * ig) + (size_t)(k0 + k) * lda);
            } else {         // four consecutive k at one i
                const int kg = e % (BK / 4), i = e / (BK / 4);
                if (i0 + i < M && k0 + 4 * kg < K) ra[p] = *(const float4*)(A + (size_t)(i0 + i) * lda + (size_t)(k0 + 4 * kg));
            }
        }
#pragma unroll
        for (int p = 0; p < PB; p++) {
            const int e = tid + p * 256;
            rb[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (B_KFAST) {
                const int kg = e % (BK / 4), j = e / (BK / 4);
                if (j0 + j < N && k0 + 4 * kg < K) rb[p] = *(const float4*)(B + (size_t)(j0 + j) * ldb + (size_t)(k0 + 4 * kg));
            } else {
                const int jg = e % (TJ / 4), k = e / (TJ / 4);
                if (j0 + 4 * jg < N && k0 + k < K) rb[p] = *(const float4*)(B + (size_t)(j0 + 4 * jg) + (size_t)(k0 + k) * ldb);
            }
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PA; p++) {
            const int e = tid + p * 256;
            if (A_IFAST) {
                const int ig = e % (TI / 4), k = e / (TI / 4);
                *(float4*)(&Is[buf][k * LDI + 4 * ig]) = ra[p];
            } else {
                const int kg = e % (BK / 4), i = e / (BK / 4);
                *(float4*)(&Is[buf][i * LDK + 4 * kg]) = ra[p];
            }
        }
#pragma unroll
        for (int p = 0; p < PB; p++) {
            const int e = tid + p * 256;
            if (B_KFAST) {
                const int kg = e % (BK / 4), j = e / (BK / 4);
                *(float4*)(&Js[buf][j * LDK + 4 * kg]) = rb[p];
            } else {
                const int jg = e % (TJ / 4), k = e / (TJ / 4);
                *(float4*)(&Js[buf][k * LDJ + 4 * jg]) = rb[p];
            }
        }
    };

    const int nk = (K - kBegin + BK - 1) / BK;
    gload(kBegin);
    sstore(0);
    __syncthreads();
    const int fr = lane & 31, fg = (lane >> 5) * 4;
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) gload(kBegin + (kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 8) {
            float4 fj[NJ], fi[NI];
#pragma unroll
            for (int t = 0; t < NJ; t++) {
                if (B_KFAST) {
                    fj[t] = *(const float4*)(&Js[buf][(wj + t * 32 + fr) * LDK + kk + fg]);
                } else {   // four k of one j: consecutive lanes read consecutive words
                    const float* q = &Js[buf][(kk + fg) * LDJ + wj + t * 32 + fr];
                    fj[t] = make_float4(q[0], q[LDJ], q[2 * LDJ], q[3 * LDJ]);
                }
            }
#pragma unroll
            for (int t = 0; t < NI; t++) {
                if (A_IFAST) {
                    const float* q = &Is[buf][(kk + fg) * LDI + wi + t * 32 + fr];
                    fi[t] = make_float4(q[0], q[LDI], q[2 * LDI], q[3 * LDI]);
                } else {
                    fi[t] = *(const float4*)(&Is[buf][(wi + t * 32 + fr) * LDK + kk + fg]);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int a = 0; a < NJ; a++)
#pragma unroll
                    for (int b = 0; b < NI; b++)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(((const float*)&fj[a])[e], ((const float*)&fi[b])[e], acc[a][b], 0, 0, 0);
        }
        if (kt + 1 < nk) sstore(buf ^ 1);
        __syncthreads();
    }
    // accumulator register v of a block: j = 8*(v/4) + 4*(lane/32) + v%4, i = lane%32
    const int il = lane & 31, jl = (lane >> 5) * 4;
#pragma unroll
    for (int a = 0; a < NJ; a++)
#pragma unroll
        for (int b = 0; b < NI; b++) {
            const int i = i0 + wi + b * 32 + il;
            if (i >= M) continue;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int j = j0 + wj + a * 32 + (v >> 2) * 8 + jl + (v & 3);
                if (j < N) {
                    const size_t ci = (size_t)i + (size_t)j * st.cj;
                    float o = alpha * acc[a][b][v];
                    if (splits > 1) {
                        unsafeAtomicAdd(&C[ci], o);
                    } else {
                        if (beta != 0.f) o += beta * C[ci];
                        C[ci] = o;
                    }
                }
            }
        }
}

// The same product for a short contraction (K = KC of at most 128: Q K^T of the explicit attention chain, K = head size)
// with A(i,k) i-fast and B(k,j) k-fast.  A tile of such a product is all prologue and epilogue for the kernel above: one
// trip to memory for the operands, a few MFMAs, 64 KB of C to write.  Here a workgroup keeps its 128 rows of B (the j
// panel) in registers as MFMA operands for its whole life and walks `tilesPerWg` tiles of 128 i: the next tile's slice of
// A is requested before the current tile is multiplied, and the stores of one pair of 32 x 32 blocks drain under the
// MFMAs of the next (the loads are older than the stores, so waiting for them does not wait for the stores).
template <int KC>
__global__ __launch_bounds__(256, 2) void gemm2_panel_f32_kernel(int M, int N, float alpha, const float* __restrict__ A,
                                                              const float* __restrict__ B, float beta, float* __restrict__ C,
                                                              GemmStrides st, int iChunks, int tilesPerWg, int causal)
{
    constexpr int LDI = 128 + 4, NP = KC * 128 / 4 / 256;       // [k][i] row stride; float4 per thread and tile of A
    extern __shared__ __attribute__((aligned(16))) float panel_smem[];   // two stages of KC x LDI
    A += (size_t)blockIdx.y * st.sA;
    B += (size_t)blockIdx.y * st.sB;
    C += (size_t)blockIdx.y * st.sC;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int jp = blockIdx.x / iChunks;
    const int ic = blockIdx.x % iChunks;
    if (causal) {
        // One workgroup per j panel (iChunks == 1), which walks the tiles up to its diagonal: 1 to gridDim.x of them.
        // Panels are rotated by the batch index and taken in reverse in every other round of 256 workgroups, so that
        // neither a die (workgroup i goes to die i mod 8) nor a CU (i and i + 256 share one) collects the long ones.
        jp = (int)((blockIdx.x + blockIdx.y) % gridDim.x);
        if (((gridDim.x * blockIdx.y) >> 8) & 1) jp = (int)gridDim.x - 1 - jp;
    }
    const int j0 = jp * 128, wj = (wave >> 1) * 64, wi = (wave & 1) * 64;
    const int fr = lane & 31, fg = (lane >> 5) * 4;
    const int t0 = ic * tilesPerWg, nT = (M + 127) / 128;
    int t1 = min(nT, t0 + tilesPerWg);
    if (causal) t1 = min(t1, jp + 1);   // tile t holds i >= 128 t, the panel j <= 128 jp + 127
    if (t0 >= t1) return;

    // B fragments: block a holds rows j0 + wj + 32 a + fr, this lane's four k of every eight
    float4 qf[2][KC / 8];
#pragma unroll
    for (int a = 0; a < 2; a++) {
        const int j = j0 + wj + a * 32 + fr;
        const float* bp = B + (size_t)min(j, N - 1) * st.bj + fg;
#pragma unroll
        for (int q = 0; q < KC / 8; q++) qf[a][q] = *(const float4*)(bp + 8 * q);
    }
    float4 ra[NP];
    // whole: the tile lies inside the matrix (wavefront-uniform), so nothing is masked
    auto gload = [&](int t, bool whole) {
        const int i0 = t * 128;
        if (whole) {
#pragma unroll
            for (int p = 0; p < NP; p++) {
                const int e = tid + p * 256, ig = e & 31, k = e >> 5;
                ra[p] = *(const float4*)(A + (size_t)(i0 + 4 * ig) + (size_t)k * st.ak);
            }
            return;
        }
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int e = tid + p * 256, ig = e & 31, k = e >> 5;
            ra[p] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i0 + 4 * ig < M) ra[p] = *(const float4*)(A + (size_t)(i0 + 4 * ig) + (size_t)k * st.ak);
        }
    };
    auto sstore = [&](int buf) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int e = tid + p * 256, ig = e & 31, k = e >> 5;
            *(float4*)(&panel_smem[buf * KC * LDI + k * LDI + 4 * ig]) = ra[p];
        }
    };
    const bool jWhole = j0 + 128 <= N;
    gload(t0, t0 * 128 + 128 <= M);
    sstore(0);
    __syncthreads();
    for (int t = t0; t < t1; t++) {
        const int buf = (t - t0) & 1;
        if (t + 1 < t1) gload(t + 1, (t + 1) * 128 + 128 <= M);
        const float* as = panel_smem + buf * KC * LDI;
        const bool plain = jWhole && t * 128 + 128 <= M && beta == 0.f;   // wavefront-uniform
#pragma unroll
        for (int b = 0; b < 2; b++) {
            floatx16 acc[2];
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[a][v] = 0.f;
#pragma unroll
            for (int q = 0; q < KC / 8; q++) {
                const float* ap = as + (8 * q + fg) * LDI + wi + b * 32 + fr;
                const float fi[4] = {ap[0], ap[LDI], ap[2 * LDI], ap[3 * LDI]};
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int a = 0; a < 2; a++)
                        acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(((const float*)&qf[a][q])[e], fi[e], acc[a], 0, 0, 0);
            }
            // accumulator register v of a block: j = 8 (v / 4) + 4 (lane / 32) + v % 4, i = lane % 32
            const int i = t * 128 + wi + b * 32 + fr;
            if (plain) {
#pragma unroll
                for (int a = 0; a < 2; a++) {
                    float* cp = C + (size_t)i + (size_t)(j0 + wj + a * 32 + fg) * st.cj;
#pragma unroll
                    for (int v = 0; v < 16; v++) cp[(size_t)((v >> 2) * 8 + (v & 3)) * st.cj] = alpha * acc[a][v];
                }
            } else if (i < M) {
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int j = j0 + wj + a * 32 + (v >> 2) * 8 + fg + (v & 3);
                        if (j < N) {
                            const size_t ci = (size_t)i + (size_t)j * st.cj;
                            float o = alpha * acc[a][v];
                            if (beta != 0.f) o += beta * C[ci];
                            C[ci] = o;
                        }
                    }
            }
        }
        if (t + 1 < t1) sstore(buf ^ 1);
        // LDS only: a full __syncthreads() would also wait for this tile's stores of C
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
}

template <int KC>
static hipError_t launch_gemm2_panel(hipStream_t s, int M, int N, float alpha, const float* A, const float* B, float beta, float* C,
                                     const GemmStrides& st, int batch, bool causal)
{
    const int jPanels = (N + 127) / 128, nT = (M + 127) / 128;
    // enough workgroups for two rounds of two per CU, as long as a workgroup keeps two tiles
    int iChunks = 1;
    while (!causal && (long long)jPanels * iChunks * batch < 1024 && nT / (2 * iChunks) >= 2) iChunks *= 2;
    const int tilesPerWg = (nT + iChunks - 1) / iChunks;
    constexpr int lds = 2 * KC * (128 + 4) * 4;
    static bool attr = false;
    if (!attr) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm2_panel_f32_kernel<KC>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr = true;
    }
    dim3 grid(jPanels * iChunks, batch);
    if (grid.y > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gemm2_panel_f32_kernel<KC>, grid, 256, lds, s, M, N, alpha, A, B, beta, C, st, iChunks, tilesPerWg, causal ? 1 : 0);
    return hipGetLastError();
}

template <typename T> __global__ void gemm_prescale_kernel(T* c, size_t n, float beta)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)blockDim.x * gridDim.x)
        c[i] = beta == 0.f ? 0.f : beta * c[i];
}

template <bool A_IFAST, bool B_KFAST>
static hipError_t launch_gemm2_mfma(hipStream_t s, int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                                    float* C, const GemmStrides& st, int batch, const int* causalFlag = nullptr, int epoch = 0)
{
    const bool si = M <= 64, sj = N <= 64;
    const int gi = (M + (si ? 63 : 127)) / (si ? 64 : 128), gj = (N + (sj ? 63 : 127)) / (sj ? 64 : 128);
    // Split the contraction when one batch of few tiles has a long K (weight gradients: K = batch x sequence): enough
    // workgroups for two per CU, at least 512 of K each.  Needs a dense C (ldc == M) for the beta pre-pass.
    int splits = 1, kChunk = K;
    const long long tiles = (long long)gi * gj;
    if (batch == 1 && tiles < 256 && K >= 2048 && st.cj == M) {
        splits = (int)std::min<long long>((512 + tiles - 1) / tiles, K / 512);
        if (splits > 1) {
            kChunk = (((K + splits - 1) / splits) + 15) / 16 * 16;
            splits = (K + kChunk - 1) / kChunk;
        }
        if (splits > 1 && beta != 1.f) {
            const size_t cn = (size_t)M * N;
            hipLaunchKernelGGL(gemm_prescale_kernel<float>, (int)std::min<size_t>((cn + 255) / 256, 4096), 256, 0, s, C, cn, beta);
        }
    }
    dim3 grid(gi, gj, batch * splits);
    if (grid.y > 65535 || grid.z > 65535) return hipErrorInvalidValue;
    if (si && sj) hipLaunchKernelGGL((gemm2_f32_mfma_kernel<A_IFAST, B_KFAST, 64, 64>), grid, 256, 0, s, M, N, K, alpha, A, B, beta, C, st, splits, kChunk, splits > 1 ? nullptr : causalFlag, epoch);
    else if (si) hipLaunchKernelGGL((gemm2_f32_mfma_kernel<A_IFAST, B_KFAST, 64, 128>), grid, 256, 0, s, M, N, K, alpha, A, B, beta, C, st, splits, kChunk, splits > 1 ? nullptr : causalFlag, epoch);
    else if (sj) hipLaunchKernelGGL((gemm2_f32_mfma_kernel<A_IFAST, B_KFAST, 128, 64>), grid, 256, 0, s, M, N, K, alpha, A, B, beta, C, st, splits, kChunk, splits > 1 ? nullptr : causalFlag, epoch);
    else hipLaunchKernelGGL((gemm2_f32_mfma_kernel<A_IFAST, B_KFAST, 128, 128>), grid, 256, 0, s, M, N, K, alpha, A, B, beta, C, st, splits, kChunk, splits > 1 ? nullptr : causalFlag, epoch);
    return hipGetLastError();
}

hipError_t k_gemm2(hipStream_t s, bool tA, bool tB, int m, int n, int k, float alpha, const float* A, const float* B,
                   float beta, float* C, int lda, int ldb, int ldc, long long sA, long long sB, long long sC, int batch,
                   const int* causalFlag, int epoch, bool skipAboveDiagonal)
{
    if (causalFlag && (tA || n != k)) return hipErrorInvalidValue;
    if (skipAboveDiagonal && (tA || tB || m != n || beta != 0.f)) return hipErrorInvalidValue;
    // column-major: op(A)(i,kk) = tA ? A[kk + i*lda] : A[i + kk*lda]
    GemmStrides st;
    st.ai = tA ? lda : 1;  st.ak = tA ? 1 : lda;
    st.bk = tB ? ldb : 1;  st.bj = tB ? 1 : ldb;
    st.ci = 1;             st.cj = ldc;
    st.sA = sA; st.sB = sB; st.sC = sC;
    if (m <= 0 || n <= 0 || batch <= 0) return hipSuccess;
    // MFMA path: every float4 the staging loads must be aligned and whole (the unit-stride extent a multiple of 4)
    const bool aligned = ((((uintptr_t)A | (uintptr_t)B) & 15) == 0) && lda % 4 == 0 && ldb % 4 == 0 && sA % 4 == 0 && sB % 4 == 0;
    const bool aOk = tA ? (k % 4 == 0) : (m % 4 == 0);
    const bool bOk = tB ? (n % 4 == 0) : (k % 4 == 0);
    if (aligned && aOk && bOk && k > 0 && (long long)m * n >= 1024) {
        if (!tA && !tB && m >= 256 && n >= 128 && (long long)m * n * batch >= (1ll << 22)) {
            // a short contraction over large matrices (Q K^T of the attention chain): the j panel stays in registers
            if (k == 32) return launch_gemm2_panel<32>(s, m, n, alpha, A, B, beta, C, st, batch, skipAboveDiagonal);
            if (k == 64) return launch_gemm2_panel<64>(s, m, n, alpha, A, B, beta, C, st, batch, skipAboveDiagonal);
            if (k == 128) return launch_gemm2_panel<128>(s, m, n, alpha, A, B, beta, C, st, batch, skipAboveDiagonal);
        }
        if (!tA && !tB) return launch_gemm2_mfma<true, true>(s, m, n, k, alpha, A, B, beta, C, st, batch, causalFlag, epoch);
        if (!tA && tB) return launch_gemm2_mfma<true, false>(s, m, n, k, alpha, A, B, beta, C, st, batch, causalFlag, epoch);
        if (tA && !tB) return launch_gemm2_mfma<false, true>(s, m, n, k, alpha, A, B, beta, C, st, batch);
        return launch_gemm2_mfma<false, false>(s, m, n, k, alpha, A, B, beta, C, st, batch);
    }
    return launch_generic<float>(s, m, n, k, alpha, A, B, beta, C, st, batch);
}

// ---------------------------------------------------------------------------
// GEMV, not transposed: one wavefront per row, 128-bit loads along the row.
template <typename T> struct VecLoad;
template <> struct VecLoad<float> {
    static constexpr int W = 4;
    __device__ static inline float dot(const float* a, const float* x)
    {
        float4 av = *(const float4*)a, xv = *(const float4*)x;
        return av.x * xv.x + av.y * xv.y + av.z * xv.z + av.w * xv.w;
    }
};
template <> struct VecLoad<bf16_t> {
    static constexpr int W = 8;
    __device__ static inline float dot(const bf16_t* a, const float* x)
    {
        uint4 av = *(const uint4*)a;
        float4 x0 = *(const float4*)x, x1 = *(const float4*)(x + 4);
        const uint32_t u[4] = {av.x, av.y, av.z, av.w};
        const float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            acc += __uint_as_float(u[i] << 16) * xs[2 * i];
            acc += __uint_as_float(u[i] & 0xffff0000u) * xs[2 * i + 1];
        }
        return acc;
    }
};

template <typename T>
__global__ __launch_bounds__(256) void gemv_n_kernel(int m, int n, float alpha, const T* __restrict__ A,
                                                     const float* __restrict__ x, float beta, float* __restrict__ y)
{
    constexpr int W = VecLoad<T>::W;
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= m) return;
    const T* a = A + (size_t)row * n;
    float acc = 0.f;
    const bool vec_ok = (n % W == 0) && (((uintptr_t)a % 16) == 0) && (((uintptr_t)x % 16) == 0);
    if (vec_ok) {
        for (int j = lane * W; j < n; j += 64 * W) acc += VecLoad<T>::dot(a + j, x + j);
    } else {
        for (int j = lane; j < n; j += 64) acc += ldf(a, j) * x[j];
    }
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (lane == 0) {
        float v = alpha * acc;
        if (beta != 0.f) v += beta * y[row];
        y[row] = v;
    }
}

// transposed: y[j] = sum_i A[i,j] x[i]; consecutive threads walk consecutive columns
template <typename T>
__global__ void gemv_t_kernel(int m, int n, float alpha, const T* __restrict__ A, const float* __restrict__ x, float beta,
                              float* __restrict__ y)
{
    int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    float acc = 0.f;
    for (int i = 0; i < m; i++) acc += ldf(A, (size_t)i * n + j) * x[i];
    float v = alpha * acc;
    if (beta != 0.f) v += beta * y[j];
    y[j] = v;
}

// The transposed product over many rows (the bias gradient of an inner product layer: A = dY (rows x outputs), x = ones):
// the rows are dealt over workgroups, each leaves one partial row of sums, and a second launch adds the partials in the
// order of their rows - the same sum on every run.  A workgroup is 16 x 16 threads: 16 V columns (V = 4: 256 bytes of a
// row), sixteen rows at a time.
template <typename T, int V>
__global__ __launch_bounds__(256) void gemv_t_part_kernel(int m, int n, int rowsPer, const T* __restrict__ A,
                                                          const float* __restrict__ x, float* __restrict__ part)
{
    __shared__ float red[16][16 * V + 1];
    const int cl = threadIdx.x & 15, rl = threadIdx.x >> 4;
    const int j = (blockIdx.x * 16 + cl) * V;
    const int r0 = blockIdx.y * rowsPer, r1 = min(m, r0 + rowsPer);
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; v++) acc[v] = 0.f;
    if (j < n) {
#pragma unroll 8
        for (int i = r0 + rl; i < r1; i += 16) {
            const float xi = x ? x[i] : 1.f;   // no vector: the plain sum of every column
            const T* a = A + (size_t)i * n + j;
            if (V == 4) {
                float av[4];
                if (sizeof(T) == 4) {
                    const float4 t = *(const float4*)a;
                    av[0] = t.x; av[1] = t.y; av[2] = t.z; av[3] = t.w;
                } else {
                    const uint2 t = *(const uint2*)a;
                    av[0] = __uint_as_float(t.x << 16); av[1] = __uint_as_float(t.x & 0xffff0000u);
                    av[2] = __uint_as_float(t.y << 16); av[3] = __uint_as_float(t.y & 0xffff0000u);
                }
#pragma unroll
                for (int v = 0; v < V; v++) acc[v] = __builtin_fmaf(av[v], xi, acc[v]);
            } else {
                acc[0] = __builtin_fmaf(ldf(a, 0), xi, acc[0]);
            }
        }
    }
#pragma unroll
    for (int v = 0; v < V; v++) red[rl][cl * V + v] = acc[v];
    __syncthreads();
    if (threadIdx.x < 16 * V) {
        const int jj = blockIdx.x * 16 * V + threadIdx.x;
        if (jj < n) {
            float t = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) t += red[r][threadIdx.x];
            part[(size_t)blockIdx.y * n + jj] = t;
        }
    }
}

__global__ void gemv_t_sum_kernel(int n, int chunks, float alpha, const float* __restrict__ part, float beta, float* __restrict__ y)
{
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    float acc = 0.f;
#pragma unroll 8
    for (int c = 0; c < chunks; c++) acc += part[(size_t)c * n + j];
    float v = alpha * acc;
    if (beta != 0.f) v += beta * y[j];
    y[j] = v;
}

// how the rows of a transposed product are dealt: (columns per thread, rows per workgroup, workgroups along the rows)
static inline int gemv_t_chunks(int m, int colBlocks)
{
    int c = std::max(1, std::min(64, 4096 / colBlocks));
    return std::min(c, (m + 31) / 32);
}
static inline void gemv_t_split(DType adt, int m, int n, const void* A, int* V, int* rowsPer, int* chunks)
{
    const size_t es = adt == F32 ? 4 : 2;
    *V = (n % 4 == 0 && ((uintptr_t)A % (4 * es)) == 0) ? 4 : 1;
    const int c = gemv_t_chunks(m, (n + 16 * *V - 1) / (16 * *V));
    *rowsPer = (m + c - 1) / c;
    *chunks = (m + *rowsPer - 1) / *rowsPer;
}

size_t k_gemv_workspace_bytes(bool tA, int m, int n)
{
    if (!tA || m < 256 || n <= 0) return 0;
    // whichever column count per thread the alignment allows
    return (size_t)std::max(gemv_t_chunks(m, (n + 63) / 64), gemv_t_chunks(m, (n + 15) / 16)) * n * sizeof(float);
}

hipError_t k_gemv(hipStream_t s, DType adt, bool tA, int m, int n, float alpha, const void* A, const float* x, float beta,
                  float* y, void* ws, size_t wsBytes)
{
    if (m <= 0 || n <= 0) return hipSuccess;
    if (!tA) {
        int grid = (m + 3) / 4;
        if (adt == F32)
            hipLaunchKernelGGL(gemv_n_kernel<float>, grid, 256, 0, s, m, n, alpha, (const float*)A, x, beta, y);
        else
            hipLaunchKernelGGL(gemv_n_kernel<bf16_t>, grid, 256, 0, s, m, n, alpha, (const bf16_t*)A, x, beta, y);
    } else if (ws && m >= 256) {
        int V, rowsPer, chunks;
        gemv_t_split(adt, m, n, A, &V, &rowsPer, &chunks);
        if (wsBytes < (size_t)chunks * n * sizeof(float)) return hipErrorInvalidValue;
        float* part = (float*)ws;
        const dim3 grid((n + 16 * V - 1) / (16 * V), chunks);
        if (adt == F32) {
            if (V == 4) hipLaunchKernelGGL((gemv_t_part_kernel<float, 4>), grid, 256, 0, s, m, n, rowsPer, (const float*)A, x, part);
            else hipLaunchKernelGGL((gemv_t_part_kernel<float, 1>), grid, 256, 0, s, m, n, rowsPer, (const float*)A, x, part);
        } else {
            if (V == 4) hipLaunchKernelGGL((gemv_t_part_kernel<bf16_t, 4>), grid, 256, 0, s, m, n, rowsPer, (const bf16_t*)A, x, part);
            else hipLaunchKernelGGL((gemv_t_part_kernel<bf16_t, 1>), grid, 256, 0, s, m, n, rowsPer, (const bf16_t*)A, x, part);
        }
        hipLaunchKernelGGL(gemv_t_sum_kernel, (n + 63) / 64, 64, 0, s, n, chunks, alpha, part, beta, y);
    } else {
        int grid = (n + 255) / 256;
        if (adt == F32)
            hipLaunchKernelGGL(gemv_t_kernel<float>, grid, 256, 0, s, m, n, alpha, (const float*)A, x, beta, y);
        else
            hipLaunchKernelGGL(gemv_t_kernel<bf16_t>, grid, 256, 0, s, m, n, alpha, (const bf16_t*)A, x, beta, y);
    }
    return hipGetLastError();
}

}  // namespace mch
