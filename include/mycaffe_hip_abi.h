/*
 * C ABI of libmycaffe_hip.so - the gfx950 (MI355X) replacement for the
 * attention hot path of MyCaffe's CudaDnnDLL.
 *
 * The exported names, argument order and argument meaning are those of the
 * reference's native DLL (CudaDnnDLL/CudaDnnDLL.11.8.def:5-18,
 * CudaDnnDLL/CudaDnnDLL.cpp:57-1161), with the Win64 typedefs replaced by
 * fixed-width types: LONG = int32_t, LONGLONG = int64_t, LPTSTR = UTF-16 text
 * (char16_t*).  Device memory is only ever named by integer handles; no
 * pointer to device memory crosses this boundary.
 *
 * Only the function ids listed below are dispatched; every other id returns
 * MCH_ERROR_NOT_IMPLEMENTED with a message naming the id.  DLL_InvokeDouble and
 * DLL_InvokeDoubleEx2 drive a second kernel table whose memory and arithmetic are
 * double (the reference's Kernel<double>): the ids of the attention path are built
 * for it, with plain kernels - see the comment at their declarations.
 */
#ifndef MYCAFFE_HIP_ABI_H
#define MYCAFFE_HIP_ABI_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t MCH_LONG;
typedef int64_t MCH_LONGLONG;
typedef uint16_t MCH_TCHAR; /* UTF-16 code unit */

/* ---- error codes (CudaDnnDLL/Cuda Files/util.h:128-228) ------------------- */
enum {
    /* Win32 codes the reference's blob loader returns as they are (blobloader.cu:30-42, 83-99) */
    MCH_ERROR_WIN_FILE_NOT_FOUND = 2,
    MCH_ERROR_WIN_INVALID_PARAMETER = 87,
    MCH_ERROR_WIN_INSUFFICIENT_BUFFER = 122,
    MCH_ERROR_DLL_NOT_INIT = 89999,
    MCH_ERROR_PARAM = 90000,
    MCH_ERROR_PARAM_OUT_OF_RANGE = 90001,
    MCH_ERROR_PARAM_NULL = 90002,
    MCH_ERROR_FILE_READ = 90004,
    MCH_ERROR_FILE_OPEN = 90005,
    MCH_ERROR_MEMORY_OUT = 90007,
    MCH_ERROR_MEMORY_NULL = 90008,
    MCH_ERROR_NOT_IMPLEMENTED = 90009,
    MCH_ERROR_MEMORY_RANGE_EXCEEDED = 90010,
    MCH_ERROR_MEMORY_MIXED_HALF_TYPES = 90011,
    MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED = 90012,
    MCH_ERROR_MEMORY_NOT_FOUND = 90014,
    MCH_ERROR_MEMORY_TOO_SMALL = 90016,
    MCH_ERROR_DEVICE_NOT_INITIALIZED = 90017,
    MCH_ERROR_LAYERNORM_NOT_INITIALIZED = 90161,
    MCH_ERROR_ROPE_NOT_INITIALIZED = 90201,
    MCH_ERROR_ATTN_NOT_INITIALIZED = 90281,
    MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE = 90284,
    MCH_ERROR_ATTN_INVALID_BLOCK_SIZE = 90285,
    MCH_ERROR_BLOBLOADER_NOT_INITIALIZED = 90321,
    MCH_ERROR_EXTENSION_NOT_INITIALIZED = 90401,
    /* llama2 extension (CudaExtension.llm32.llama2/Files/llm.h:15-19) */
    MCH_ERROR_LLM_RENDERED_PROMPT_TO_LONG = 10000,
    MCH_ERROR_LLM_LOAD_MODEL = 10001,
    MCH_ERROR_LLM_MISSING_MODEL_FILE = 10002,
    MCH_ERROR_LLM_MISSING_TOKENIZER_FILE = 10003,
    MCH_ERROR_LLM_GENERATE = 10004
};

/* ---- function ids (CudaDnnDLL/inc/FunctionIDs.h:71-551, main.h:23-40) ------
 * f{...} = the float array of the call, l{...} = the 64-bit integer array (DLL_InvokeFloatEx2); ids that take no l{}
 * go through DLL_InvokeFloat.  [..] = optional trailing values.  Handles are integers.  Each id cites the reference's
 * unmarshalling code, whose argument order and count checks are reproduced. */
enum {
    MCH_DLL_FREEMEM = -1,
    MCH_DLL_INITIALIZE = -2,
    MCH_DLL_CLEANUP = -3,

    MCH_FN_SETDEVICE = 1,                   /* f{deviceId[, flags, seed]} (device.cu:772-795) */
    MCH_FN_GETDEVICE = 3,                   /* -> f{deviceId}  */
    MCH_FN_SYNCHRONIZEDEVICE = 5,
    MCH_FN_CREATE_MEMORYPOINTER = 16,       /* l{hData, offset, count} -> view handle (device.h:1000-1020) */
    MCH_FN_FREE_MEMORYPOINTER = 17,         /* l{hView} */
    MCH_FN_ALLOCMEM_HALF = 19,              /* as ALLOCMEM, 16-bit storage (bf16 here) */
    MCH_FN_ALLOCMEM = 20,                   /* l{count[, stream]} [f{count, [stream,] data...}] -> handle (device.cu:854-949) */
    MCH_FN_FREEMEM = 21,                    /* l{h} (device.cu:956-968) */
    MCH_FN_GETMEM = 22,                     /* l{h, count(-1 = all)} -> data (device.cu:973-1022) */
    MCH_FN_SETMEM = 23,                     /* f{h, count, [stream,] data...} l{h, count} (device.cu:1029-1091) */
    MCH_FN_CREATE_CUDNN = 47,               /* f{[stream]} -> handle (device.h:1201-1221) */
    MCH_FN_FREE_CUDNN = 48,                 /* f{h} */
    MCH_FN_CREATE_TENSORDESC = 50,          /* -> handle */
    MCH_FN_FREE_TENSORDESC = 51,            /* f{h} */
    MCH_FN_SET_TENSORDESC = 52,             /* l{h, half, n, c, h, w[, strides x4]} (device.cu:1426-1464) */
    MCH_FN_CREATE_EXTENSION = 67,           /* DLL_InvokeFloatEx: library path -> handle (device.h:4569-4588) */
    MCH_FN_FREE_EXTENSION = 68,             /* f{h} */
    MCH_FN_EXTENSION_RUN = 69,              /* f{hExt, fnIdx, args...} [+ text] (device.h:4569-4588) */
    MCH_FN_SOFTMAX_FWD = 111,               /* f{alpha, beta} l{hCudnn, 0, hBtmDesc, hBtm, 0, hTopDesc, hTop, alg, mode} (device.h:4778-4798) */
    MCH_FN_SOFTMAX_BWD = 112,               /* f{alpha, beta} l{hCudnn, 0, hTopDataDesc, hTopData, hTopDiffDesc, hTopDiff, 0, hBtmDiffDesc, hBtmDiff, alg, mode} (device.h:4801-4823) */
    MCH_FN_ATTN_CREATE = 160,               /* -> handle */
    MCH_FN_ATTN_FREE = 161,                 /* f{h} */
    MCH_FN_ATTN_SET = 162,                  /* f{dropout} l{hCudnn, hAttn, gpuId, training, batch, blockSize, heads, hs, seed} (device.h:2463-2485);
                                             * dropout in [0, 1) acts in training mode only (attn.cu:578-583): a new mask per forward call from a
                                             * counter-based generator seeded with `seed`, repeated by the backward call that follows */
    MCH_FN_ATTN_FWD = 163,                  /* l{hCudnn, hAttn, blockSize, hQ, hK, hV, hMask, hY, batchMask[, blockSizeK[, mergedY]]} (device.h:2488-2506, attn.cu:518-602) */
    MCH_FN_ATTN_BWD = 164,                  /* l{hCudnn, hAttn, hQ, hdQ, hK, hdK, hV, hdV, hMask, hY, hdY} (device.h:2509-2529, attn.cu:608-661) */
    MCH_FN_SET = 200,                       /* f{val} l{n, h, 0, idx, xOff} (device.h:6038-6061) */
    MCH_FN_COPY = 202,                      /* l{n, hSrc, hDst, srcOff, dstOff, hStream, srcHalf, dstHalf} (device.h:6063-6095) */
    MCH_FN_GEMM2 = 219,                     /* f{alpha, beta} l{tA, tB, m, n, k, 0, hA, hB, 0, hC, lda, ldb, ldc[, sA, sB, sC, batch]}, column-major (device.cu:1691-1726) */
    MCH_FN_GEMM = 220,                      /* f{alpha, beta} l{tA, tB, m, n, k, 0, hA, hB, 0, hC[, aOff, bOff, cOff, groups, gA, gB, gC]}, row-major (device.cu:1636-1685) */
    MCH_FN_GEMV = 221,                      /* f{alpha, beta} l{tA, m, n, 0, hA, hX, 0, hY[, aOff, xOff, yOff]} (device.cu:1733-1767) */
    MCH_FN_AXPY = 222,                      /* f{alpha} l{n, 0, hX, hY[, xOff, yOff]} (device.cu:1830-1857) */
    MCH_FN_SCAL = 224,                      /* f{alpha} l{n, 0, hX[, xOff]} (device.cu:1887-1905) */
    MCH_FN_SCALE = 227,                     /* f{alpha} l{n, 0, hX, hY[, xOff, yOff]} (device.cu:2028-2051) */
    MCH_FN_ADD_SCALAR = 228,                /* f{alpha} l{n, 0, hY[, yOff]} (device.cu:2183-2201) */
    MCH_FN_ADD = 229,                       /* [f{alpha}] l{n, hA, hB, hY} (device.cu:2208-2236) */
    MCH_FN_SUB = 230,                       /* l{n, hA, hB, hY[, aOff, bOff, yOff, nB]} (device.cu:2294-2331) */
    MCH_FN_MUL = 231,                       /* l{n, hA, hB, hY[, aOff, bOff, yOff]} (device.cu:2398-2423) */
    MCH_FN_DIV = 233,                       /* l{n, hA, hB, hY} (device.cu:2492-2505) */
    MCH_FN_EXP = 235,                       /* [f{beta}] l{n, hA, hY[, aOff, yOff, 0]} (device.cu:2531-2557) */
    MCH_FN_LOG = 236,                       /* [f{beta[, alpha]}] l{n, hA, hY[, 0, 0]} (device.cu:2564-2590) */
    MCH_FN_POWX = 237,                      /* f{alpha} l{n, hA, 0, hY[, aOff, yOff]} (device.cu:2595-2618) */
    MCH_FN_SQRT = 239,                      /* [f{epsilon}] l{n, hX, hY} (device.cu:2712-2728) */
    MCH_FN_TRANSPOSE = 261,                 /* l{n, hX, hY, hXCounts, hYCounts, hMapping, numAxes, hBuffer} (device.cu:3088-3107) */
    MCH_FN_MASK = 264,                      /* f{search, replace} l{n, maskDim, 0, 0, hX, hMask, hY} (device.cu:2101-2120) */
    MCH_FN_MASK_BATCH = 266,                /* f{search, replace} l{n, batch, maskDim, 0, 0, hX, hMask, hY} (device.cu:2125-2145) */
    MCH_FN_TRANSPOSE_HW = 267,              /* l{n, c, h, w, hSrc, hDst} (device.cu:3110-3127) */
    MCH_FN_INVERT = 273,                    /* [f{numerator, denominator}] l{n, hX, hY[, xOff, yOff]} (device.cu:2624-2655) */
    MCH_FN_CHANNEL_MEAN = 287,              /* l{count, outer, channels, inner, hX, hY[, xOff]} (device.cu:3386-3405) */
    MCH_FN_CHANNEL_MAX = 290,               /* l{count, outer, channels, inner, hX, hY, returnIdx[, acrossChannels]} (device.cu:3359-3380) */
    MCH_FN_CHANNEL_SUB = 291,               /* l{count, outer, channels, inner, hX, hY[, hA]}: y = a - x[n, s], a = y when absent (device.cu:3438-3457) */
    MCH_FN_CHANNEL_SUM = 292,               /* l{count, outer, channels, inner, hX, hY} (device.cu:3488-3503) */
    MCH_FN_CHANNEL_DIV = 293,               /* l{count, outer, channels, inner, hX, hY[, method]}: y /= x[n, s] (device.cu:3541-3560) */
    MCH_FN_CHANNEL_DOT = 294,               /* l{count, outer, channels, inner, hX, hA, hY} (device.cu:3638-3654) */
    MCH_FN_CHANNEL_COPY = 300,              /* l{count, outer, channels, blocks, inner, offset, hX, hY, dir} (device.cu:3730-3748) */
    MCH_FN_CHANNEL_FILLFROM = 301,          /* l{count, outer, channels, inner, hX, hY, dir} (CudaDnn.cs:9086-9092, math.cu:7465-7481) */
    MCH_FN_CHANNEL_COPYALL = 302,           /* l{count, outer, channels, inner, hX, hY} (CudaDnn.cs:9443-9449, math.cu:7630-7639) */
    MCH_FN_CHANNEL_DUP = 303,               /* l{count, outer, channels, inner, hX, hY} (CudaDnn.cs:9312-9318, math.cu:7667-7676) */
    MCH_FN_CHANNEL_SUM2 = 309,              /* l{count, outer, channels, inner, hX, hY, acrossChannels[, dir, channelsY]} (device.cu:3510-3534) */
    MCH_FN_EMBED_FWD = 390,                 /* l{count, hBtm, hWeight, M, N, K, hTop} (CudaDnn.cs:9751, math.cu:9314-9330) */
    MCH_FN_RELU_FWD = 428,                  /* f{negativeSlope} l{count, hBtm, hTop, 0} (device.h:4925-4940) */
    MCH_FN_RELU_BWD = 429,                  /* f{negativeSlope} l{count, hTopDiff, hTopData, hBtmDiff, 0} (device.h:4943-4959) */
    MCH_FN_GELU_FWD = 600,                  /* l{count, hBtm, hTop, bert} (device.h:3253-3266) */
    MCH_FN_GELU_BWD = 601,                  /* l{count, hTopDiff, hTopData, hBtmDiff, hBtmData, bert} (device.h:3269-3316) */
    MCH_FN_SILU_FWD = 605,                  /* l{count, hBtm, hTop} (CudaDnn.cs:10152) */
    MCH_FN_SILU_BWD = 606,                  /* l{count, hTopDiff, hTopData, hBtmDiff, hBtmData} (CudaDnn.cs:10132-10180, device.h:3269-3316) */
    MCH_FN_CREATE_LAYERNORM = 970,          /* f{eps} l{gpuId, count, outer, channels, inner} -> handle (device.h:4123-4147) */
    MCH_FN_FREE_LAYERNORM = 971,            /* f{h} */
    MCH_FN_LAYERNORM_FWD = 975,             /* l{h, hX, hY} (CudaDnn.cs:6339-6345, layernorm.cu:219-262) */
    MCH_FN_LAYERNORM_BWD = 976,             /* l{h, hYdata, hYdiff, hXdiff} (CudaDnn.cs:6354-6360, layernorm.cu:268-312) */
    MCH_FN_CREATE_ROPE = 980,               /* f{theta} l{sharedIdx, gpuId, count, batch, seqLen, heads, hs} -> handle (device.h:4201-4229) */
    MCH_FN_FREE_ROPE = 981,                 /* f{h} */
    MCH_FN_ROPE_FWD = 982,                  /* l{hRope, n, hX, hY[, freqOffset]} (device.h:4232-4255, rope.cu:785-825) */
    MCH_FN_ROPE_BWD = 983,                  /* l{hRope, n, hXdata, hYdiff, hXdiff} (device.h:4266-4283, rope.cu:832-864) */
    MCH_FN_CREATE_BLOBLOADER = 990,       /* DLL_InvokeFloatEx: file path -> handle */
    MCH_FN_FREE_BLOBLOADER = 991,           /* f{h} */
    MCH_FN_BLOBLOADER_LOAD = 992,           /* l{h, count, hData, localItemOffset} (device.h:4635-4648, blobloader.cu:83-126) */
    MCH_FN_BLOBLOADER_RESETOFFSET = 993,    /* l{h, offsetInBytes} (device.h:4651-4662) */
    MCH_FN_BLOBLOADER_ADDTOOFFSET = 994,    /* l{h, offsetInItems} (device.h:4665-4676) */
    MCH_QRY_DEVICE_NAME = 1000,             /* DLL_QueryString: LONG{deviceId} */
    MCH_QRY_EXTENSION_STRING = 1003,        /* DLL_QueryStringFloatEx: LONG{hExt, fnIdx, args...} (device.h:4590-4603) */

    /* Ids with no counterpart in the reference: single-call replacements for
     * host-side loops of the reference's C# layers.  A maintainer adds one
     * CudaDnn<T> wrapper per id.
     *
     * ATTN_DECODE_FWD replaces the O(pos) loop of the KV-cache branch of
     * MultiheadAttentionLayer.forward (MultiheadAttentionLayer.cs:713-730,
     * 759-777) and Primitives::attention (primitives.cu:158-202,389-403).
     *   f{scale (0 = 1/sqrt(hs))}
     *   l{batch, heads, kvHeads, hs, len, hQ, hKcache, hVcache, hY,
     *     strideKvBatch, strideKvHead, strideKvPos [, hRope, hKnew, hVnew]}
     * With hRope != 0 the call first rotates q and k_new at position len-1
     * with that rope handle's tables and stores k_new/v_new into the caches
     * at position len-1.
     *
     * RMSNORM_FWD replaces the six-call chain of RMSNormLayer.forward
     * (RMSNormLayer.cs:156-180):  f{eps}  l{outer, dim, hX, hWeight(0=none), hY}
     *
     * SWIGLU_FWD = silu(a)*b (TransformerBlockLayer.cs:860-875):  l{n, hA, hB, hY}
     *
     * QKV_PROJ_HEADS replaces the head of CausalSelfAttentionLayer.forward (CausalSelfAttentionLayer.cs:526-557):
     * the fused InnerProduct, its bias GEMM, the three channel copies and the three head transposes become one
     * GEMM whose epilogue adds the bias and writes q, k, v as (batch, heads, T, hs):
     *   l{batch, T, heads, hs, hX, hWeight (3C x C), hBias (0 = none), hQ, hK, hV [, hRope]}
     * With hRope (a CREATE_ROPE handle of the same heads and hs) the epilogue also rotates q and k, which replaces the
     * two ROPE_FWD calls the layer makes between the channel copies and the transposes (:538-545).
     * Together with the 11th value of ATTN_FWD (Y written head-merged) the layer forward is four calls:
     * QKV_PROJ_HEADS, ATTN_FWD, GEMM and bias GEMM of the output projection.
     *
     * LINEAR_FWD replaces the two GEMM calls of InnerProductLayer.forward (InnerProductLayer.cs:372-417: the product
     * with the transposed weight, then the rank-1 update with the vector of ones) by one GEMM whose epilogue adds
     * the bias:  l{M, N, K, hX (M x K), hWeight (N x K), hBias (N; 0 = none), hY (M x N)}.
     * With it the causal self attention layer's forward is three calls.
     */
    MCH_FN_ATTN_DECODE_FWD = 2001,
    MCH_FN_RMSNORM_FWD = 2002,
    MCH_FN_SWIGLU_FWD = 2003,
    MCH_FN_QKV_PROJ_HEADS = 2004,
    MCH_FN_LINEAR_FWD = 2005
};

/* DEVINIT flags (CudaDnnDLL/Cuda Files/device.h:18-22) */
enum { MCH_DEVINIT_CUBLAS = 1, MCH_DEVINIT_CURAND = 2, MCH_DEVINIT_SETSEED = 4, MCH_DEVINIT_RESETDEVICE = 8 };

/* ---- reference entry points ------------------------------------------------ */

/* CudaDnnDLL.cpp:134-312.  Legacy packing: every argument (ints and handles
 * included) travels as float in pInput. */
MCH_LONG DLL_InvokeFloat(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, float* pInput, MCH_LONG lInput,
                         float** ppOutput, MCH_LONG* plOutput, MCH_TCHAR* szErr, MCH_LONG lszErrMax);

/* CudaDnnDLL.cpp:314-492.  Scalars in pInput, integers and handles in plInput. */
MCH_LONG DLL_InvokeFloatEx2(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, float* pInput, MCH_LONG lInput,
                            MCH_LONGLONG* plInput, MCH_LONG llInput, float** ppOutput, MCH_LONG* plOutput,
                            MCH_TCHAR* szErr, MCH_LONG lszErrMax);

/* CudaDnnDLL.cpp:1017-1100.  As DLL_InvokeFloat plus one UTF-16 input string
 * (CREATE_EXTENSION: library path; EXTENSION_RUN: text handed to the extension). */
MCH_LONG DLL_InvokeFloatEx(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, float* pInput, MCH_LONG lInput,
                           MCH_TCHAR* pszInput, float** ppOutput, MCH_LONG* plOutput, MCH_TCHAR* szErr,
                           MCH_LONG lszErrMax);

/* CudaDnnDLL.cpp:494-853: the double base type.  Kernel indices of these calls are their own table (dllmain.cpp:6-14),
 * arrays cross the boundary as doubles, device memory holds doubles and every result is computed in double.  Built:
 * INITIALIZE / CLEANUP / FREEMEM(-1), SETDEVICE, GETDEVICE, SYNCHRONIZEDEVICE, ALLOCMEM (ALLOCMEM_HALF allocates doubles
 * too), FREEMEM, CREATE / FREE_MEMORYPOINTER, GETMEM, SETMEM, SET, COPY, GEMM, GEMM2, GEMV, AXPY, SCAL, SCALE, ADD, SUB, MUL, DIV, ADD_SCALAR, POWX,
 * SQRT, INVERT, EXP, LOG, MASK, MASK_BATCH, TRANSPOSE, TRANSPOSE_HW, CHANNEL_COPY / MEAN / MAX / SUB / DIV / DOT / SUM /
 * SUM2 / FILLFROM / COPYALL / DUP, EMBED_FWD, SILU / GELU / RELU forward and backward, SWIGLU_FWD, RMSNORM_FWD, CREATE /
 * FREE_LAYERNORM and LAYERNORM_FWD / BWD, CREATE / FREE_CUDNN, CREATE / FREE / SET_TENSORDESC, SOFTMAX_FWD / BWD,
 * ATTN_CREATE / FREE / SET / FWD / BWD (no dropout; the tenth and eleventh values of ATTN_FWD as on the float side),
 * CREATE_ROPE / FREE_ROPE / ROPE_FWD / BWD, and the fused ids ATTN_DECODE_FWD, QKV_PROJ_HEADS (even head sizes) and
 * LINEAR_FWD - same packing as the float ids above: what the attention, multi-head attention and transformer block layers
 * call, forward and backward.  These are one-element-per-thread kernels: the precision twin of the path, not a fast
 * one.  Any other id (blob loaders, extensions), and DLL_InvokeDoubleEx (extensions and blob loaders are float objects),
 * returns MCH_ERROR_NOT_IMPLEMENTED with the id in the message. */
MCH_LONG DLL_InvokeDouble(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, double* pInput, MCH_LONG lInput,
                          double** ppOutput, MCH_LONG* plOutput, MCH_TCHAR* szErr, MCH_LONG lszErrMax);
MCH_LONG DLL_InvokeDoubleEx2(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, double* pInput, MCH_LONG lInput,
                             MCH_LONGLONG* plInput, MCH_LONG llInput, double** ppOutput, MCH_LONG* plOutput,
                             MCH_TCHAR* szErr, MCH_LONG lszErrMax);
MCH_LONG DLL_InvokeDoubleEx(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, double* pInput, MCH_LONG lInput,
                            MCH_TCHAR* pszInput, double** ppOutput, MCH_LONG* plOutput, MCH_TCHAR* szErr,
                            MCH_LONG lszErrMax);

/* CudaDnnDLL.cpp:855-933.  *ppOutput receives a malloc'ed UTF-16 string that the
 * caller returns through DLL_QueryString(.., MCH_DLL_FREEMEM, ..). */
MCH_LONG DLL_QueryString(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, MCH_LONG* pInput, MCH_LONG lInput,
                         MCH_TCHAR** ppOutput, MCH_TCHAR* szErr, MCH_LONG lszErrMax);

/* CudaDnnDLL.cpp:935-1015.  Text is written into the caller's buffer. */
MCH_LONG DLL_QueryStringFloatEx(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, MCH_LONG* pInput, MCH_LONG lInput,
                                MCH_TCHAR* pszOutput, MCH_LONG lOutputMax, MCH_TCHAR* szErr,
                                MCH_LONG lszErrMax);
MCH_LONG DLL_QueryStringDoubleEx(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, MCH_LONG* pInput, MCH_LONG lInput,
                                 MCH_TCHAR* pszOutput, MCH_LONG lOutputMax, MCH_TCHAR* szErr,
                                 MCH_LONG lszErrMax);

/* CudaDnnDLL.cpp:57-128.  Used by extension libraries: device pointer behind a
 * memory handle, and host result buffers owned by the parent. */
MCH_LONG Internal_GetPointerFloat(int32_t ht, MCH_LONG lKernelIdx, MCH_LONG hHandle, void** ppPtr);
MCH_LONG Internal_GetPointerDouble(int32_t ht, MCH_LONG lKernelIdx, MCH_LONG hHandle, void** ppPtr);
MCH_LONG Internal_AllocHostFloat(MCH_LONG lKernelIdx, MCH_LONG lCount, float** ppfDst, float* pfSrc,
                                 bool bSrcOnDevice);
MCH_LONG Internal_AllocHostDouble(MCH_LONG lKernelIdx, MCH_LONG lCount, double** ppfDst, double* pfSrc,
                                  bool bSrcOnDevice);

/* ---- extension ABI (libmycaffe_hip_llama2.so) ------------------------------
 * CudaExtension.llm32.llama2/CudaExtension.llm32.11.8.def:5-11,
 * CudaExtension.llm32.cpp:67-268.  hParent is the dlopen handle of the parent
 * library (HMODULE in the reference). */
enum {
    MCH_LLM_CREATE = 1,         /* f{temperature, topp, seed} -> f{hLlm} */
    MCH_LLM_DESTROY = 2,        /* f{hLlm} */
    MCH_LLM_LOAD = 3,           /* Ex: f{hLlm}, "model.bin;tokenizer.bin" */
    MCH_LLM_QUERYSTATUS = 4,    /* f{hLlm} -> f{pct, status} */
    MCH_LLM_GENERATE = 5,       /* Ex: f{hLlm}, prompt text (needs a tokenizer file at LOAD) */
    MCH_LLM_QUERYRESPONSE = 6,  /* Ex: f{hLlm} -> text in szOutput, *ppOutput = end flag */
    MCH_LLM_ABORT = 7,          /* f{hLlm} */
    /* No counterpart in the reference: token-id front door used where no
     * tokenizer file exists (synthetic checkpoints).
     *   GENERATE_IDS  f{hLlm, nSteps, wantLogits(0|1), id0, id1, ...}
     *                 -> f{next id after each position [, logits of every step]}
     *   SET_OPTION    f{hLlm, option, value}; option 1 = weight storage
     *                 (0 fp32, 1 bf16), applied at the next LOAD (weights already on the
     *                 device keep the storage they were loaded in); option 2 = first
     *                 step of the timed span; option 3 = replay one captured
     *                 HIP graph per step (1, default) or launch eagerly (0);
     *                 option 4 = weight rows per wavefront of the mat-vec
     *                 kernels (1 or 2; 0 = library's choice); option 5 = GENERATE_IDS /
     *                 GENERATE_BATCH draw from the handle's sampler (temperature, top-p,
     *                 seed of CREATE) instead of the argmax (0, default); option 6 = GENERATE_BATCH
     *                 appends the logits of every step, batch x nSteps x vocabulary (0, default);
     *                 option 7 = the forced prompt positions run as one batched pass (1, default: MFMA
     *                 GEMMs + fused causal attention over sequences x positions rows) or one decode
     *                 step per position as in the reference's loop (0); option 8 = storage of the key /
     *                 value caches: fp32 (0, default) or bf16 (1: rotated keys and values are rounded to
     *                 nearest-even when they are appended, every step attends over the rounded rows;
     *                 activations stay fp32; needs a head size that is a multiple of 8, otherwise the
     *                 caches stay fp32); takes effect at the next generation; option 9 = where the
     *                 partial results of a single sequence's attention splits are merged: in front of
     *                 the output projection's mat-vec (1, default, when dim <= 1024 and the cache fits
     *                 one pass of rows per split) or inside the attention kernel (0); option 10 = the
     *                 batched prompt pass over 16-bit weights (more than 256 prompt rows, widths that are
     *                 multiples of 64) keeps its activations to sixteen leading bits - two bf16 numbers a
     *                 value on the bf16 matrix cores, attention in fp32: logits within the fp32 bar of the
     *                 step-per-position loop (0, default) - or rounds them to bf16 and runs the attention
     *                 in bf16 (1: half the matrix-core work, logits within the 16-bit bar); option 11 = where
     *                 a sampler with a temperature above 0 runs: on the device (1, default: softmax, the
     *                 xorshift64* coin and the top-p / multinomial choice in one kernel per step, so the
     *                 steps replay as a captured graph, and the prompt stays one batched pass in which
     *                 every row takes the draw of its position; the id can differ from the host's only where the
     *                 coin falls within rounding of an edge of the cumulative distribution) or on the host
     *                 after a copy of the logits, as llama2_gpu.cpp:108 and llama2_sampler.cpp do it (0)
     *   GENERATE_BATCH f{hLlm, nSteps, batch, nPrompt, ids of seq 0.., seq 1..}
     *                 -> f{batch x nSteps next ids [, logits with option 6]}
     *   QUERY_TIMING  f{hLlm} -> f{ms of the timed span (HIP events), steps in it, 1 if the steps were
     *                 replays of the captured graph / 0 if they were launched eagerly, ms of the batched
     *                 prompt pass (0 if none ran), sequences x prompt positions it covered}
     *   PROFILE_STEP  f{hLlm, pos, reps[, batch]} -> per kernel class of one decode step
     *                 f{ms per step, launches per step, algorithmic bytes per step}, classes in
     *                 the order qkv mat-vec, rope+cache store, decode attention, wo, w1|w3,
     *                 w2, classifier, embed+argmax
     *   TOKENIZE      Ex: f{hLlm, bos(0|1), eos(0|1)} + text -> f{token ids};
     *                 f{hLlm, -1, prevToken, token} -> the token's piece in szOutput
     *   SAMPLE        f{hLlm, logits...} -> f{id}: one call of the handle's sampler
     *                 (llama2_sampler.cpp:126-151); advances its random state unless greedy; runs where the
     *                 generations sample (option 11: the device kernel for up to 32768 logits, else the host)
     *   RUNNING_SUM   f{hLlm, threshold, values...} -> f{index, sum}: the device sampler's way of adding up
     *                 non-negative fp32 values one after the other, every addition rounded (the sums of
     *                 llama2_sampler.cpp:38-49, 78-99 and of the softmax), stopped at the first index where
     *                 the sum exceeds the threshold (index = count if it never does); for checking it
     *                 against a plain loop, up to 32768 values */
    MCH_LLM_GENERATE_IDS = 100,
    MCH_LLM_SET_OPTION = 101,
    MCH_LLM_GENERATE_BATCH = 102,
    MCH_LLM_QUERY_TIMING = 103,
    MCH_LLM_PROFILE_STEP = 104,
    MCH_LLM_TOKENIZE = 105,
    MCH_LLM_SAMPLE = 106,
    MCH_LLM_RUNNING_SUM = 107
};

MCH_LONG DLL_InitFloatCustomExtension(void* hParent, MCH_LONG lKernelIdx);
MCH_LONG DLL_InvokeFloatCustomExtension(MCH_LONG lfnIdx, float* pInput, MCH_LONG lInput, float** ppOutput,
                                        MCH_LONG* plOutput, MCH_TCHAR* szErr, MCH_LONG lErrMax);
MCH_LONG DLL_InvokeFloatCustomExtensionEx(MCH_LONG lfnIdx, float* pInput, MCH_LONG lInput, float** ppOutput,
                                          MCH_LONG* plOutput, MCH_TCHAR* szInput, MCH_TCHAR* szOutput,
                                          MCH_LONG lOutputMax, MCH_TCHAR* szErr, MCH_LONG lErrMax);
/* CudaExtension.llm32.cpp:85-89, 180-206, 270-330: double twins; the engine is fp32 / 16-bit storage only, so all
 * three return MCH_ERROR_NOT_IMPLEMENTED (a double-typed parent fails cleanly at CREATE_EXTENSION). */
MCH_LONG DLL_InitDoubleCustomExtension(void* hParent, MCH_LONG lKernelIdx);
MCH_LONG DLL_InvokeDoubleCustomExtension(MCH_LONG lfnIdx, double* pInput, MCH_LONG lInput, double** ppOutput,
                                         MCH_LONG* plOutput, MCH_TCHAR* szErr, MCH_LONG lErrMax);
MCH_LONG DLL_InvokeDoubleCustomExtensionEx(MCH_LONG lfnIdx, double* pInput, MCH_LONG lInput, double** ppOutput,
                                           MCH_LONG* plOutput, MCH_TCHAR* szInput, MCH_TCHAR* szOutput,
                                           MCH_LONG lOutputMax, MCH_TCHAR* szErr, MCH_LONG lErrMax);

/* ---- measurement hook (no counterpart in the reference) --------------------
 * Runs the same Ex2 dispatch `nWarmup` + `nReps` times on the kernel's stream
 * and returns the mean duration of the timed launches in milliseconds,
 * measured with HIP events recorded on that stream.  Only for calls whose
 * result does not depend on how often they run. */
MCH_LONG MCH_TimeInvokeFloatEx2(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, float* pInput, MCH_LONG lInput,
                                MCH_LONGLONG* plInput, MCH_LONG llInput, MCH_LONG nWarmup, MCH_LONG nReps,
                                float* pfMs, MCH_TCHAR* szErr, MCH_LONG lszErrMax);
/* The same with `nSets` lists of `llInput` long arguments each, one after the other in plInput: dispatch i takes list
 * i mod nSets.  With handles of different buffers in the lists, a kernel whose operands would otherwise stay in the
 * caches from one repeat to the next is timed on operands that come from memory. */
MCH_LONG MCH_TimeInvokeFloatEx2Sets(MCH_LONG lKernelIdx, MCH_LONG lFunctionIdx, float* pInput, MCH_LONG lInput,
                                    MCH_LONGLONG* plInput, MCH_LONG llInput, MCH_LONG nSets, MCH_LONG nWarmup,
                                    MCH_LONG nReps, float* pfMs, MCH_TCHAR* szErr, MCH_LONG lszErrMax);

/* ---- entry point that allocates nothing (no counterpart in the reference) ----
 * For callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  (What the entry point guarantees is that nothing is allocated and that its scratch is cleared
 * by a fill kernel, not a memset node; it still makes host-side calls - hipSetDevice, hipGetLastError - and a capture
 * of the call itself is not part of its tests.)  The call is ATTN_DECODE_FWD (id 2001) with the same f{scale} and l{...} arrays; the
 * split partials and merge tickets come from a fixed device array inside the library (4 MiB + 16 KiB per GPU,
 * held until the process ends) instead of the kernel object's growable workspace, and no hipMalloc, hipFree or
 * other allocating routine is called.  Limits: batch x heads <= 4096 and (batch x heads x splits) x (hs + 2) x 4
 * bytes <= 4 MiB, where splits = ceil(256 / (batch x heads)); larger calls return
 * MCH_ERROR_PARAM_OUT_OF_RANGE before anything is enqueued (q, the new key / value and the caches are untouched, so
 * the same call can then go through id 2001).  All calls on one GPU share the array: calls that overlap on one GPU (two kernel
 * objects, two host threads) race, so serialise them. */
MCH_LONG MCH_AttnDecodeForwardNoAlloc(MCH_LONG lKernelIdx, float* pInput, MCH_LONG lInput, MCH_LONGLONG* plInput,
                                      MCH_LONG llInput, MCH_TCHAR* szErr, MCH_LONG lszErrMax);

#ifdef __cplusplus
}
#endif
#endif /* MYCAFFE_HIP_ABI_H */
