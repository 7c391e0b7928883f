// Host-side launchers of the gfx950 kernels.  Every launcher enqueues on the
// given stream and returns the launch status; none of them synchronises.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace mch {

// storage type of a device buffer: fp32 or bf16 (the library's 16-bit storage)
enum DType { F32 = 0, BF16 = 1 };

typedef uint16_t bf16_t;

__host__ __device__ inline float bf16_to_f32(bf16_t v)
{
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)v) << 16;
    return c.f;
}

// round to nearest even; NaN stays NaN
__host__ __device__ inline bf16_t f32_to_bf16(float f)
{
    union { uint32_t u; float f; } c;
    c.f = f;
    if ((c.u & 0x7fffffffu) > 0x7f800000u)
        return (bf16_t)((c.u >> 16) | 0x40);
    uint32_t r = 0x7fffu + ((c.u >> 16) & 1u);
    return (bf16_t)((c.u + r) >> 16);
}

// ---- elementwise and layout kernels (ew_kernels.hip) ----------------------
hipError_t k_set(hipStream_t s, DType dt, void* y, size_t n, float v);
hipError_t k_convert(hipStream_t s, DType sdt, const void* src, DType ddt, void* dst, size_t n);
hipError_t k_axpy(hipStream_t s, DType dt, size_t n, float alpha, const void* x, void* y);
hipError_t k_scale(hipStream_t s, DType dt, size_t n, float alpha, const void* x, void* y);
hipError_t k_add(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y, float alpha);
hipError_t k_mul(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y);
hipError_t k_silu(hipStream_t s, DType dt, size_t n, const void* x, void* y);
hipError_t k_swiglu(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y);
hipError_t k_mask(hipStream_t s, DType dt, size_t n, int maskDim, float search, float replace, const void* x,
                  const void* mask, void* y, float xscale = 1.0f);
hipError_t k_mask_batch(hipStream_t s, DType dt, size_t n, int batch, int maskDim, float search, float replace,
                        const void* x, const void* mask, void* y, float xscale = 1.0f);
hipError_t k_transpose(hipStream_t s, DType dt, size_t n, const void* x, void* y, const float* xc, const float* yc,
                       const float* map, int axes);
// the two halves of k_transpose: fetching the stride / map blobs costs a device round trip, so callers keep the result
struct PermuteArgs { int xs[8]; int ys[8]; int map[8]; int axes; };
hipError_t k_transpose_fetch(hipStream_t s, const float* xc, const float* yc, const float* map, int axes, PermuteArgs* out);
hipError_t k_transpose_run(hipStream_t s, DType dt, size_t n, const void* x, void* y, const PermuteArgs& a);
hipError_t k_transpose_hw(hipStream_t s, DType dt, int nc, int h, int w, const void* x, void* y);
hipError_t k_channel_copy(hipStream_t s, DType dt, size_t n, int channels, int blocks, int inner, int offset,
                          void* x, void* y, int dir);
hipError_t k_embed(hipStream_t s, DType wdt, size_t count, const float* ids, const void* w, int N, void* top);
// softmax over `len` for outer x inner independent series; element (o, l, i) at (o*len + l)*inner + i
hipError_t k_softmax(hipStream_t s, DType dt, const void* x, void* y, size_t outer, int len, int inner, bool logsm);
// softmax of mask(x) in one pass (mask semantics of k_mask / k_mask_batch with md1 = maskDim / batch, dd1 = n / batch);
// hipErrorNotSupported when the shape does not fit
// zeroFlag (causal only): a row whose masked entries do not all come out as exact zeros writes `epoch` there
hipError_t k_softmax_masked(hipStream_t s, DType dt, const void* x, void* y, size_t rows, int len, bool logsm, const void* mask,
                            size_t md1, size_t dd1, float search, float replace, float xscale, bool causal = false,
                            int* zeroFlag = nullptr, int epoch = 0);
// gradient with respect to the softmax input from the output y and its gradient dy (dx may alias dy)
hipError_t k_softmax_bwd(hipStream_t s, DType dt, const void* y, const void* dy, void* dx, size_t outer, int len, int inner, bool logsm);
// adjacent-pair rotary embedding with the CudaDnnDLL index rule; x == y allowed
hipError_t k_rope(hipStream_t s, DType dt, size_t n, const void* x, void* y, const float* fcos, const float* fsin,
                  int seqLen, int heads, int hs, int tableOff, bool grad = false);
// LayerNorm without affine part over rows x inner; stdev[rows] keeps sqrt(var + eps) of every row for the gradient
hipError_t k_layernorm_fwd(hipStream_t s, DType dt, int rows, int inner, const void* x, void* y, float* stdev, float eps);
hipError_t k_layernorm_bwd(hipStream_t s, DType dt, int rows, int inner, const void* y, const void* dy, void* dx,
                           const float* stdev, float bump);
hipError_t k_gelu_fwd(hipStream_t s, DType dt, size_t n, const void* x, void* y, bool bert);
hipError_t k_gelu_bwd(hipStream_t s, DType dt, size_t n, const void* dy, const void* x, void* dx, bool bert);
hipError_t k_relu_fwd(hipStream_t s, DType dt, size_t n, const void* x, void* y, float slope);
hipError_t k_relu_bwd(hipStream_t s, DType dt, size_t n, const void* dy, const void* y, void* dx, float slope);
hipError_t k_silu_bwd(hipStream_t s, DType dt, size_t n, const void* dy, const void* x, void* dx);
// primitives of the C# RMSNormLayer / LayerNormLayer chains
hipError_t k_powx(hipStream_t s, DType dt, size_t n, const void* a, float alpha, void* y);
hipError_t k_sqrt(hipStream_t s, DType dt, size_t n, const void* x, void* y, float eps);
hipError_t k_invert(hipStream_t s, DType dt, size_t n, const void* x, void* y, float num, float den);
hipError_t k_add_scalar(hipStream_t s, DType dt, size_t n, float alpha, void* y);
hipError_t k_div(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y);
hipError_t k_sub(hipStream_t s, DType dt, size_t n, const void* a, const void* b, void* y, size_t nB);
hipError_t k_channel_mean(hipStream_t s, DType dt, size_t rows, int inner, const void* x, void* y);
// y[row] = scale * sum of the row's `inner` values; y[n, s] = sum over the channels of x[n, c, s]
hipError_t k_channel_rowsum(hipStream_t s, DType dt, size_t rows, int inner, const void* x, void* y, float scale);
hipError_t k_channel_colsum(hipStream_t s, DType dt, size_t outer, int channels, int spatial, const void* x, void* y);
// mode 0 fillfrom forward, 1 fillfrom backward, 2 copyall, 3 duplicate (index rules in ew_kernels.hip)
hipError_t k_channel_spread(hipStream_t s, DType dt, int mode, size_t n, size_t spatial, size_t period, size_t channels, void* x, void* y);
hipError_t k_rmsnorm(hipStream_t s, DType dt, int outer, int dim, const void* x, const void* w, void* y, float eps);
// primitives of the CAFFE-engine softmax chain: x is (num, channels, spatial), reduced tensors (num, spatial)
hipError_t k_exp(hipStream_t s, DType dt, size_t n, const void* a, void* y, float beta);
hipError_t k_log(hipStream_t s, DType dt, size_t n, const void* a, void* y, float beta, float alpha);
hipError_t k_channel_max(hipStream_t s, DType dt, size_t num, int channels, int spatial, const void* x, void* y, bool idx, bool across);
hipError_t k_channel_sub(hipStream_t s, DType dt, size_t count, int channels, int spatial, const void* a, const void* x, void* y);
hipError_t k_channel_div(hipStream_t s, DType dt, size_t count, int channels, int spatial, const void* x, void* y);
hipError_t k_channel_dot(hipStream_t s, DType dt, size_t num, int channels, int spatial, const void* x, const void* a, void* y);

// ---- GEMM family (gemm.hip) ------------------------------------------------
// row-major C[m,n] = alpha*op(A)*op(B) + beta*C; A, B, C all of storage type dt
// ws: k_gemm_workspace_bytes(...) bytes of scratch for the transpose combinations that run as "transpose the operand that
// lies the other way, then the A B^T kernels" (without it they take the strided kernels)
hipError_t k_gemm(hipStream_t s, DType dt, bool tA, bool tB, int m, int n, int k, float alpha, const void* A,
                  const void* B, float beta, void* C, void* ws = nullptr, size_t wsBytes = 0);
size_t k_gemm_workspace_bytes(DType dt, bool tA, bool tB, int m, int n, int k);
// Fused QKV projection of CausalSelfAttentionLayer: [q|k|v] = X W^T + bias with X (B*T, C), W (3C, C), C = H*hs, written
// straight into three (B,H,T,hs) tensors.  tmp: (B*T, 3C) scratch, only used for shapes the fused kernel does not take.
hipError_t k_gemm_qkv_heads(hipStream_t s, DType dt, int B, int T, int H, int hs, const void* X, const void* W, const void* bias,
                            void* q, void* k, void* v, void* tmp, const float* fcos = nullptr, const float* fsin = nullptr,
                            int ropeSeq = 0);
// Y (m x n) = X (m x k) W^T + bias: product and bias in one launch; tmp: m x n scratch for shapes the tile kernels do not take
hipError_t k_gemm_bias(hipStream_t s, DType dt, int m, int n, int k, const void* X, const void* W, const void* bias, void* Y, void* tmp);
// whether these operands make k_gemm_bias / k_gemm_qkv_heads use their scratch matrix (tmp may be null otherwise)
bool k_gemm_bias_needs_tmp(DType dt, int n, int k, const void* X, const void* W, const void* Y);
bool k_gemm_qkv_heads_needs_tmp(DType dt, int H, int hs, const void* X, const void* W, const void* q, const void* k, const void* v);
// column-major strided batched gemm with BLAS semantics (fp32)
// C (fp32) = alpha X W^T + beta C on the bf16 matrix cores: W 16-bit (n x k), k % 64 == 0; A is X as bf16 (m x k) or,
// split, every row of X as two bf16 rows (nearest bf16, then the bf16 nearest to the remainder; m x 2k)
hipError_t k_gemm_bf16_f32(hipStream_t s, int m, int n, int k, float alpha, const void* A, bool split, const void* W, float beta, float* C);
// the same product with the epilogues of the Llama prompt pass: SwiGLU of the stacked W1 | W3 (bf16 rows of hid, or hi | lo
// rows of 2 hid), and rotation + scatter of the stacked Wq | Wk | Wv into head tensors and caches (gemm.hip, PromptEpilogue)
hipError_t k_gemm_bf16_swiglu(hipStream_t s, int m, int hid, int k, const void* A, bool split, const void* W13, void* out, bool outSplit);
hipError_t k_gemm_bf16_qkv_rope(hipStream_t s, int B, int P, int H, int kvH, int hs, int k, const void* A, bool split, const void* Wqkv,
                                void* q, void* kh, void* vh, bool heads16, void* kc, void* vc, bool cache16, int seqLen,
                                const float* fcos, const float* fsin);
// causalFlag != nullptr (no transposes, n == k): B(k,j) is known to be exactly zero for k > j unless *causalFlag == epoch,
// and the contraction of a tile of columns stops at its last column
hipError_t k_gemm2(hipStream_t s, bool tA, bool tB, int m, int n, int k, float alpha, const float* A, const float* B,
                   float beta, float* C, int lda, int ldb, int ldc, long long sA, long long sB, long long sC,
                   int batch, const int* causalFlag = nullptr, int epoch = 0, bool skipAboveDiagonal = false);
// skipAboveDiagonal (no transposes, m == n, short contraction): entries C(i,j) of tiles that lie wholly at i > j need not
// be computed (their memory is left as it is); other shapes ignore the request
// A row-major (m,n) of type adt; x, y fp32.  y = alpha*A*x + beta*y, or with tA y = alpha*A^T*x + beta*y
size_t k_gemv_workspace_bytes(bool tA, int m, int n);   // scratch for the partial sums of a transposed product over many rows
hipError_t k_gemv(hipStream_t s, DType adt, bool tA, int m, int n, float alpha, const void* A, const float* x,
                  float beta, float* y, void* ws = nullptr, size_t wsBytes = 0);

// ---- attention (attn_prefill.hip, attn_decode.hip) --------------------------
enum MaskKind { MASK_NONE = 0, MASK_QK = 1, MASK_KEY = 2, MASK_BQK = 3, MASK_CAUSAL = 4 };
// q (B,H,Tq,hs), k/v (B,H,Tk,hs), y (B,H,Tq,hs), all dt.  mask is fp32:
//   MASK_QK (Tq,Tk) shared, MASK_KEY (B,Tk), MASK_BQK (B,Tq,Tk); zero entries are filled with -1e29.
//   MASK_CAUSAL needs no mask buffer (lower triangle kept).
// Attention dropout (training mode of the handle, attn.cu:455-486, 578-583): which probabilities survive is a pure
// function of (seed, batch*heads index, query, key), so the backward pass regenerates the mask of the forward call
// instead of storing it.  keep(i) = high 32 bits of splitmix64(seed * 0x9E3779B97F4A7C15 + i) >= threshold, with
// i = ((b*H + h)*Tq + query)*Tk + key and threshold = ratio * 2^32; survivors are scaled by 1 / (1 - ratio).
struct AttnDropout {
    uint64_t seed;
    uint32_t threshold;
    float keepScale;
};
__host__ __device__ inline bool attn_dropout_keep(uint64_t seed, uint64_t index, uint32_t threshold)
{
    uint64_t z = seed * 0x9E3779B97F4A7C15ull + index + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (uint32_t)(z >> 32) >= threshold;
}
hipError_t k_attn_prefill(hipStream_t s, DType dt, const void* q, const void* k, const void* v, void* y, int B, int H,
                          int Tq, int Tk, int hs, float scale, const float* mask, MaskKind kind, float* lse2 = nullptr,
                          bool yMerged = false, const AttnDropout* dropout = nullptr);
// yMerged: y is written as (B,Tq,H,hs), the head-merged layout the output projection reads, instead of (B,H,Tq,hs).
// With lse2 ([B*H*Tq] fp32) the forward pass also stores log2 of every row's softmax denominator (scores scaled, masked
// ones at -1e29; -inf marks a row whose keys are all masked), which is all the backward pass needs of the probabilities.
//
// Gradients of the same attention: dq, dk, dv from dy (attn_backward.hip).  lse2 as stored by the forward pass, or
// nullptr to have it recomputed (slow path).  workspace: attn_backward_workspace_bytes(B, H, Tq).
size_t attn_backward_workspace_bytes(int B, int H, int Tq);
hipError_t k_attn_backward(hipStream_t s, DType dt, const void* q, const void* k, const void* v, const void* y, const void* dy,
                           void* dq, void* dk, void* dv, int B, int H, int Tq, int Tk, int hs, float scale, const float* mask,
                           MaskKind kind, const float* lse2, void* workspace, size_t workspaceBytes,
                           const AttnDropout* dropout = nullptr);
// With dropout both calls take the general one-row-per-wavefront kernels (no matrix-core path), and the backward pass
// follows the reference's sequence literally: its softmax backward reads the probabilities AFTER dropout was applied to
// them in place (attn.cu:578-583, 637-646), which gives dS = M / (1 - ratio)^2 * P * (dP - dY.Y) and dV = (P M')^T dY.
size_t attn_decode_workspace_bytes(int B, int H, int hs, int len);
// one query per (b,h): q (B,H,hs), caches addressed as
//   cache[b*strideB + (h/kvMul)*strideH + t*strideT + i], y (B,H,hs).  All dt.
// With dlen set, `len` is only the upper bound used to size the launch and the
// actual number of cached positions is read from *dlen on the device.
hipError_t k_attn_decode(hipStream_t s, DType dt, const void* q, const void* kc, const void* vc, void* y, int B, int H,
                         int kvH, int hs, int len, long long strideB, long long strideH, long long strideT,
                         float scale, void* workspace, size_t workspaceBytes, const int* dlen = nullptr,
                         int* counters = nullptr);
// `counters`: B*H zero-initialised ints that stay zero between launches; when given, the last
// workgroup of every (batch, head) merges the split partials inside the kernel (no second launch).
//
// Decode step of the llama2 engine in one launch: rotate q / k at position *dlen - 1, append k, v to the caches
// ([B][seqLen][kvH*hs], stored as cacheType: fp32, or bf16 with hs a multiple of 8), attend over positions
// 0 .. *dlen - 1.  qkv: [B][(H + 2 kvH) hs] raw fp32 projections, y: [B][H*hs] fp32.
// deferMerge (batch 1 with the whole cache in one iteration of rows per split; attn_decode_fused_deferred_splits says whether
// and how many splits): y is not written.  Split s leaves its accumulator of head h at workspace[s * H*hs + h * hs ..] and
// {running maximum, sum} at workspace[splits * H*hs + (s * H + h) * 2 ..] (fp32) for the next kernel of the stream, which
// merges the ceil(*dlen / rowsPerSplit) splits that hold rows (k_llama_matvec_merge in the engine).
hipError_t k_attn_decode_fused(hipStream_t s, const float* qkv, void* kc, void* vc, DType cacheType, float* y, int B, int H, int kvH,
                               int hs, int seqLen, float scale, const float* fcos, const float* fsin, const int* dlen, void* workspace,
                               size_t workspaceBytes, int* counters, bool deferMerge = false);
int attn_decode_fused_deferred_splits(int B, int H, int hs, int seqLen, DType cacheType, int* rowsPerSplit);
// rotate q (B,H,hs) and knew (B,kvH,hs) at position pos and append knew/vnew to the caches at pos
hipError_t k_rope_append(hipStream_t s, DType dt, void* q, void* knew, const void* vnew, void* kc, void* vc, int B,
                         int H, int kvH, int hs, int pos, long long strideB, long long strideH, long long strideT,
                         const float* fcos, const float* fsin);

}  // namespace mch
