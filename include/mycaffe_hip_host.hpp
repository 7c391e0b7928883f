// C++ host side of the attention path above the C ABI of mycaffe_hip_abi.h.
//
// The reference host is C# (MyCaffe/common/CudaDnn.cs) talking to the native DLL through the CudaControl
// marshaller.  This header is the same two layers in C++17, header-only:
//
//   Marshaller   loads the shared library by path, resolves the exported names and forwards float / long
//                arrays to DLL_InvokeFloat / DLL_InvokeFloatEx / DLL_InvokeFloatEx2 / DLL_QueryString*,
//                including the caller-owned result buffer, the library-replaced buffer handed back with
//                FREEMEM (-1), UTF-16 strings, and error codes turned into exceptions
//                (the role of CudaControlLib.ICudaKernel: CudaDnn.cs:1105-1115, 1711, 1729-1736).
//   CudaDnn      the methods of CudaDnn<float> that the attention layers and the llama2 wrapper call, with
//                the reference's names and argument order; each packs its arguments exactly as the C# method
//                cited beside it does.
//   LlmInference the wrapper of the llama2 extension (MyCaffe/common/LlmInference.cs), token-id front door
//                included.
//
// No CPU fallback exists: constructing CudaDnn throws when the library cannot be loaded.
#pragma once
#include <dlfcn.h>

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "mycaffe_hip_abi.h"

namespace mycaffe {

class CudaDnnError : public std::runtime_error {
public:
    CudaDnnError(long code, const std::string& msg) : std::runtime_error(msg + " [error " + std::to_string(code) + "]"), m_code(code) {}
    long code() const { return m_code; }

private:
    long m_code;
};

inline std::u16string to_utf16(const std::string& s)   // ASCII / Latin-1 paths and prompts
{
    std::u16string r;
    for (unsigned char ch : s) r.push_back((char16_t)ch);
    return r;
}

inline std::string from_utf16(const MCH_TCHAR* p, size_t max)
{
    std::string r;
    for (size_t i = 0; i < max && p[i]; i++) r.push_back(p[i] < 128 ? (char)p[i] : '?');
    return r;
}

// ---- the marshaller -------------------------------------------------------------------------------
class Marshaller {
public:
    explicit Marshaller(const std::string& path)
    {
        m_lib = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
        if (!m_lib) throw std::runtime_error(std::string("cannot load ") + path + ": " + dlerror());
        m_invoke = (FnInvoke)sym("DLL_InvokeFloat");
        m_invokeEx = (FnInvokeEx)sym("DLL_InvokeFloatEx");
        m_invokeEx2 = (FnInvokeEx2)sym("DLL_InvokeFloatEx2");
        m_query = (FnQuery)sym("DLL_QueryString");
        m_queryEx = (FnQueryEx)sym("DLL_QueryStringFloatEx");
        m_time = (FnTime)dlsym(m_lib, "MCH_TimeInvokeFloatEx2");
        m_decodeNoAlloc = (FnDecodeNoAlloc)dlsym(m_lib, "MCH_AttnDecodeForwardNoAlloc");
    }
    ~Marshaller()
    {
        if (m_lib) dlclose(m_lib);
    }
    Marshaller(const Marshaller&) = delete;
    Marshaller& operator=(const Marshaller&) = delete;

    std::vector<float> RunFloat(long kernel, long fn, const std::vector<float>& in, size_t capacity = 16)
    {
        Out out(capacity);
        MCH_TCHAR err[kErrMax] = {0};
        MCH_LONG rc = m_invoke((MCH_LONG)kernel, (MCH_LONG)fn, in.empty() ? nullptr : const_cast<float*>(in.data()), (MCH_LONG)in.size(),
                               &out.p, &out.n, err, kErrMax);
        check(rc, err);
        return collect(kernel, out);
    }
    std::vector<float> RunFloatEx2(long kernel, long fn, const std::vector<float>& f, const std::vector<long long>& l, size_t capacity = 16)
    {
        Out out(capacity);
        MCH_TCHAR err[kErrMax] = {0};
        static_assert(sizeof(long long) == sizeof(MCH_LONGLONG), "64-bit longs");
        MCH_LONG rc = m_invokeEx2((MCH_LONG)kernel, (MCH_LONG)fn, f.empty() ? nullptr : const_cast<float*>(f.data()), (MCH_LONG)f.size(),
                                  l.empty() ? nullptr : (MCH_LONGLONG*)const_cast<long long*>(l.data()), (MCH_LONG)l.size(), &out.p, &out.n,
                                  err, kErrMax);
        check(rc, err);
        return collect(kernel, out);
    }
    std::vector<float> RunFloatEx(long kernel, long fn, const std::vector<float>& in, const std::string& text)
    {
        Out out(16);
        MCH_TCHAR err[kErrMax] = {0};
        std::u16string w = to_utf16(text);
        MCH_LONG rc = m_invokeEx((MCH_LONG)kernel, (MCH_LONG)fn, in.empty() ? nullptr : const_cast<float*>(in.data()), (MCH_LONG)in.size(),
                                 (MCH_TCHAR*)w.c_str(), &out.p, &out.n, err, kErrMax);
        check(rc, err);
        return collect(kernel, out);
    }
    std::string QueryString(long kernel, long fn, const std::vector<int32_t>& args)
    {
        MCH_TCHAR* p = nullptr;
        MCH_TCHAR err[kErrMax] = {0};
        MCH_LONG rc = m_query((MCH_LONG)kernel, (MCH_LONG)fn, args.empty() ? nullptr : (MCH_LONG*)const_cast<int32_t*>(args.data()),
                              (MCH_LONG)args.size(), &p, err, kErrMax);
        check(rc, err);
        std::string r = p ? from_utf16(p, 1 << 20) : std::string();
        if (p) m_query((MCH_LONG)kernel, MCH_DLL_FREEMEM, nullptr, 0, &p, err, kErrMax);   // the DLL allocated the string
        return r;
    }
    std::string QueryStringFloatEx(long kernel, long fn, const std::vector<int32_t>& args, size_t max = 16384)
    {
        std::vector<MCH_TCHAR> buf(max, 0);
        MCH_TCHAR err[kErrMax] = {0};
        MCH_LONG rc = m_queryEx((MCH_LONG)kernel, (MCH_LONG)fn, (MCH_LONG*)const_cast<int32_t*>(args.data()), (MCH_LONG)args.size(), buf.data(),
                                (MCH_LONG)max, err, kErrMax);
        check(rc, err);
        return from_utf16(buf.data(), max);
    }
    // mean milliseconds of nReps back-to-back dispatches of one Ex2 call (measurement hook of this library)
    // id 2001 through the entry point that allocates no device memory (fixed scratch inside the library)
    void AttnDecodeNoAlloc(long kernel, const std::vector<float>& f, const std::vector<long long>& l)
    {
        if (!m_decodeNoAlloc) throw std::runtime_error("MCH_AttnDecodeForwardNoAlloc is not exported");
        MCH_TCHAR err[kErrMax] = {0};
        check(m_decodeNoAlloc((MCH_LONG)kernel, const_cast<float*>(f.data()), (MCH_LONG)f.size(),
                              (MCH_LONGLONG*)const_cast<long long*>(l.data()), (MCH_LONG)l.size(), err, kErrMax), err);
    }
    float TimeFloatEx2(long kernel, long fn, const std::vector<float>& f, const std::vector<long long>& l, int nWarmup, int nReps)
    {
        if (!m_time) throw std::runtime_error("MCH_TimeInvokeFloatEx2 is not exported");
        float ms = 0.f;
        MCH_TCHAR err[kErrMax] = {0};
        MCH_LONG rc = m_time((MCH_LONG)kernel, (MCH_LONG)fn, f.empty() ? nullptr : const_cast<float*>(f.data()), (MCH_LONG)f.size(),
                             l.empty() ? nullptr : (MCH_LONGLONG*)const_cast<long long*>(l.data()), (MCH_LONG)l.size(), nWarmup, nReps, &ms, err,
                             kErrMax);
        check(rc, err);
        return ms;
    }

private:
    static constexpr MCH_LONG kErrMax = 1024;
    typedef MCH_LONG (*FnInvoke)(MCH_LONG, MCH_LONG, float*, MCH_LONG, float**, MCH_LONG*, MCH_TCHAR*, MCH_LONG);
    typedef MCH_LONG (*FnInvokeEx)(MCH_LONG, MCH_LONG, float*, MCH_LONG, MCH_TCHAR*, float**, MCH_LONG*, MCH_TCHAR*, MCH_LONG);
    typedef MCH_LONG (*FnInvokeEx2)(MCH_LONG, MCH_LONG, float*, MCH_LONG, MCH_LONGLONG*, MCH_LONG, float**, MCH_LONG*, MCH_TCHAR*, MCH_LONG);
    typedef MCH_LONG (*FnQuery)(MCH_LONG, MCH_LONG, MCH_LONG*, MCH_LONG, MCH_TCHAR**, MCH_TCHAR*, MCH_LONG);
    typedef MCH_LONG (*FnQueryEx)(MCH_LONG, MCH_LONG, MCH_LONG*, MCH_LONG, MCH_TCHAR*, MCH_LONG, MCH_TCHAR*, MCH_LONG);
    typedef MCH_LONG (*FnDecodeNoAlloc)(MCH_LONG, float*, MCH_LONG, MCH_LONGLONG*, MCH_LONG, MCH_TCHAR*, MCH_LONG);
    typedef MCH_LONG (*FnTime)(MCH_LONG, MCH_LONG, float*, MCH_LONG, MCH_LONGLONG*, MCH_LONG, MCH_LONG, MCH_LONG, float*, MCH_TCHAR*, MCH_LONG);

    struct Out {   // caller-owned result buffer, as the C# marshaller passes one
        std::vector<float> own;
        float* p;
        MCH_LONG n;
        explicit Out(size_t cap) : own(cap ? cap : 1), p(own.data()), n((MCH_LONG)own.size()) {}
    };
    void* sym(const char* name)
    {
        void* p = dlsym(m_lib, name);
        if (!p) throw std::runtime_error(std::string("missing export ") + name);
        return p;
    }
    void check(MCH_LONG rc, const MCH_TCHAR* err)
    {
        if (rc != 0) throw CudaDnnError(rc, from_utf16(err, kErrMax));
    }
    std::vector<float> collect(long kernel, Out& out)
    {
        if (out.n <= 0) return {};
        if (out.p == out.own.data()) return std::vector<float>(out.own.begin(), out.own.begin() + out.n);
        // the library replaced the buffer with its own allocation (device.cu:1000-1015): copy, then FREEMEM = -1
        std::vector<float> r(out.p, out.p + out.n);
        MCH_TCHAR err[kErrMax] = {0};
        float dummy[4];
        float* dp = dummy;
        MCH_LONG dn = 4;
        m_invoke((MCH_LONG)kernel, MCH_DLL_FREEMEM, out.p, 0, &dp, &dn, err, kErrMax);
        return r;
    }
    void* m_lib = nullptr;
    FnInvoke m_invoke = nullptr;
    FnInvokeEx m_invokeEx = nullptr;
    FnInvokeEx2 m_invokeEx2 = nullptr;
    FnQuery m_query = nullptr;
    FnQueryEx m_queryEx = nullptr;
    FnTime m_time = nullptr;
    FnDecodeNoAlloc m_decodeNoAlloc = nullptr;
};

enum DIR { FWD = 0, BWD = 1 };

// ---- CudaDnn<float>: the methods of the attention path ---------------------------------------------
class CudaDnn {
public:
    // CudaDnn.cs:1679-1760: load the DLL at strPath, INITIALIZE {deviceId, flags} -> kernel index
    CudaDnn(int nDeviceID, const std::string& strPath, int flags = MCH_DEVINIT_CUBLAS | MCH_DEVINIT_CURAND) : m_cuda(strPath), m_strPath(strPath)
    {
        std::vector<float> rg = m_cuda.RunFloat(0, MCH_DLL_INITIALIZE, {(float)nDeviceID, (float)flags});
        m_hKernel = (long)rg.at(0);
    }
    ~CudaDnn()
    {
        try {
            Dispose();
        } catch (...) {
        }
    }
    void Dispose()   // CudaDnn.cs:1800-1815
    {
        if (m_hKernel > 0) {
            m_cuda.RunFloat(m_hKernel, MCH_DLL_CLEANUP, {(float)m_hKernel});
            m_hKernel = 0;
        }
    }
    const std::string& Path() const { return m_strPath; }
    Marshaller& Raw() { return m_cuda; }
    long KernelHandle() const { return m_hKernel; }

    void SynchronizeDevice() { m_cuda.RunFloat(m_hKernel, MCH_FN_SYNCHRONIZEDEVICE, {}); }                                   // :2311
    std::string GetDeviceName(int nDeviceID = 0) { return m_cuda.QueryString(m_hKernel, MCH_QRY_DEVICE_NAME, {nDeviceID}); }  // :2253

    // ---- memory (CudaDnn.cs:2584-2745, 2763-2790, 2935-2970, 3027-3095)
    long AllocMemory(const std::vector<float>& data, bool bHalfSize = false)
    {
        if (data.empty()) throw std::invalid_argument("no data");
        std::vector<float> rgf;
        rgf.reserve(data.size() + 1);
        rgf.push_back((float)data.size());
        rgf.insert(rgf.end(), data.begin(), data.end());
        return (long)ex2(bHalfSize ? MCH_FN_ALLOCMEM_HALF : MCH_FN_ALLOCMEM, rgf, {(long long)data.size()}).at(0);
    }
    long AllocMemory(long long lCapacity, bool bHalfSize = false)
    {
        if (lCapacity <= 0) throw std::invalid_argument("capacity must be positive");
        return (long)ex2(bHalfSize ? MCH_FN_ALLOCMEM_HALF : MCH_FN_ALLOCMEM, {}, {lCapacity}).at(0);
    }
    void FreeMemory(long hMem) { ex2(MCH_FN_FREEMEM, {}, {hMem}); }
    std::vector<float> GetMemoryFloat(long hMem, long long lCount = -1)
    {
        return m_cuda.RunFloatEx2(m_hKernel, MCH_FN_GETMEM, {}, {hMem, lCount}, lCount > 0 ? (size_t)lCount : 16);
    }
    void SetMemory(long hMem, const std::vector<float>& src)
    {
        if (src.empty()) throw std::invalid_argument("There are no data items to set!");
        std::vector<float> rgf;
        rgf.reserve(src.size() + 2);
        rgf.push_back((float)hMem);
        rgf.push_back((float)src.size());
        rgf.insert(rgf.end(), src.begin(), src.end());
        ex2(MCH_FN_SETMEM, rgf, {hMem, (long long)src.size()});
    }

    // ---- math
    void set(long long n, long h, float fVal, int nIdx = -1, int nXOff = 0) { ex2(MCH_FN_SET, {fVal}, {n, h, 0, nIdx, nXOff}); }   // :6739
    void copy(long long n, long hSrc, long hDst, long long nSrcOff = 0, long long nDstOff = 0)                                 // :6824
    {
        ex2(MCH_FN_COPY, {}, {n, hSrc, hDst, nSrcOff, nDstOff, -1, -1, -1});
    }
    void gemm(bool bTransA, bool bTransB, int m, int n, int k, float fAlpha, long hA, long hB, float fBeta, long hC, long long nAOff = 0,
              long long nBOff = 0, long long nCOff = 0)                                                                        // :7102
    {
        ex2(MCH_FN_GEMM, {fAlpha, fBeta}, {bTransA, bTransB, m, n, k, 0, hA, hB, 0, hC, nAOff, nBOff, nCOff, 1, 0, 0, 0});
    }
    void gemm2(bool bTransA, bool bTransB, int m, int n, int k, float fAlpha, long hA, long hB, float fBeta, long hC, int lda, int ldb, int ldc,
               long long strideA, long long strideB, long long strideC, int batch)                                            // :7129-7166
    {
        ex2(MCH_FN_GEMM2, {fAlpha, fBeta}, {bTransA, bTransB, m, n, k, 0, hA, hB, 0, hC, lda, ldb, ldc, strideA, strideB, strideC, batch});
    }
    // row-major batched matmul as a column-major gemm with swapped operands (CudaDnn.cs:7513-7524)
    void matmul(int nOuter, int m, int n, int k, long hA, long hB, long hC, float fScale = 1.f, bool bTransA = false, bool bTransB = false)
    {
        gemm2(bTransB, bTransA, n, m, k, fScale, hB, hA, 0.f, hC, bTransB ? k : n, bTransA ? m : k, n, (long long)k * n, (long long)m * k,
              (long long)m * n, nOuter);
    }
    void gemv(bool bTransA, int m, int n, float fAlpha, long hA, long hX, float fBeta, long hY)                                // :7289
    {
        ex2(MCH_FN_GEMV, {fAlpha, fBeta}, {bTransA, m, n, 0, hA, hX, 0, hY, 0, 0, 0});
    }
    void scal(long long n, float fAlpha, long hX) { ex2(MCH_FN_SCAL, {fAlpha}, {n, 0, hX, 0}); }                              // :7617
    void add(long long n, long hA, long hB, long hY) { ex2(MCH_FN_ADD, {}, {n, hA, hB, hY}); }                                // :8047
    void mul(long long n, long hA, long hB, long hY) { ex2(MCH_FN_MUL, {}, {n, hA, hB, hY, 0, 0, 0}); }                       // :8154
    void mask(long long n, long long nMaskDim, float fSearch, float fReplace, long hX, long hMask, long hY)                    // :7850
    {
        ex2(MCH_FN_MASK, {fSearch, fReplace}, {n, nMaskDim, 0, 0, hX, hMask, hY});
    }
    void mask_batch(long long n, int nBatch, long long nMaskDim, float fSearch, float fReplace, long hX, long hMask, long hY)  // :7899
    {
        ex2(MCH_FN_MASK_BATCH, {fSearch, fReplace}, {n, nBatch, nMaskDim, 0, 0, hX, hMask, hY});
    }
    void transpose(long long n, long hX, long hY, long hXCounts, long hYCounts, long hMapping, int nNumAxes, long hBuffer)     // :8773
    {
        ex2(MCH_FN_TRANSPOSE, {}, {n, hX, hY, hXCounts, hYCounts, hMapping, nNumAxes, hBuffer});
    }
    void transposeHW(int n, int c, int h, int w, long hSrc, long hDst) { ex2(MCH_FN_TRANSPOSE_HW, {}, {n, c, h, w, hSrc, hDst}); }   // :7536
    void channel_copy(long long nCount, int nOuterNum, int nChannels, int nBlocks, int nInnerNum, int nOffset, long hX, long hY, DIR dir)   // :9426
    {
        ex2(MCH_FN_CHANNEL_COPY, {}, {nCount, nOuterNum, nChannels, nBlocks, nInnerNum, nOffset, hX, hY, (long long)dir});
    }
    void embed_fwd(long long nCount, long hBottom, long hWeight, int nM, int nN, int nK, long hTop)                            // :9751
    {
        ex2(MCH_FN_EMBED_FWD, {}, {nCount, hBottom, hWeight, nM, nN, nK, hTop});
    }
    void silu_fwd(long long nCount, long hBottom, long hTop) { ex2(MCH_FN_SILU_FWD, {}, {nCount, hBottom, hTop}); }            // :10152
    void silu_bwd(long long nCount, long hTopDiff, long hTopData, long hBottomDiff, long hBottomData)                          // :10174
    {
        ex2(MCH_FN_SILU_BWD, {}, {nCount, hTopDiff, hTopData, hBottomDiff, hBottomData});
    }
    void gelu_fwd(long long nCount, long hBottom, long hTop, bool bEnableBertVersion)                                           // :10098
    {
        ex2(MCH_FN_GELU_FWD, {}, {nCount, hBottom, hTop, bEnableBertVersion ? 1 : 0});
    }
    void gelu_bwd(long long nCount, long hTopDiff, long hTopData, long hBottomDiff, long hBottomData, bool bEnableBertVersion)  // :10132
    {
        ex2(MCH_FN_GELU_BWD, {}, {nCount, hTopDiff, hTopData, hBottomDiff, hBottomData, bEnableBertVersion ? 1 : 0});
    }
    void relu_fwd(long long nCount, long hBottom, long hTop, float fNegativeSlope = 0.f)                                        // :10417
    {
        ex2(MCH_FN_RELU_FWD, {fNegativeSlope}, {nCount, hBottom, hTop, 0});
    }
    void relu_bwd(long long nCount, long hTopDiff, long hTopData, long hBottomDiff, float fNegativeSlope = 0.f)                 // :10438
    {
        ex2(MCH_FN_RELU_BWD, {fNegativeSlope}, {nCount, hTopDiff, hTopData, hBottomDiff, 0});
    }

    // ---- LayerNorm handle (CudaDnn.cs:6307-6360) ---------------------------------------------------------------------
    long CreateLayerNorm(int nGpuID, long long nCount, int nOuterNum, int nChannels, int nInnerNum, float fEps = 1e-10f)
    {
        return (long)ex2(MCH_FN_CREATE_LAYERNORM, {fEps}, {nGpuID, nCount, nOuterNum, nChannels, nInnerNum}).at(0);
    }
    void FreeLayerNorm(long h) { m_cuda.RunFloat(m_hKernel, MCH_FN_FREE_LAYERNORM, {(float)h}); }
    void LayerNormForward(long hLayerNorm, long hXdata, long hYdata) { ex2(MCH_FN_LAYERNORM_FWD, {}, {hLayerNorm, hXdata, hYdata}); }
    void LayerNormBackward(long hLayerNorm, long hYdata, long hYdiff, long hXdiff)
    {
        ex2(MCH_FN_LAYERNORM_BWD, {}, {hLayerNorm, hYdata, hYdiff, hXdiff});
    }

    // ---- blob loader (CudaDnn.cs:6438-6504) ---------------------------------------------------------------------------
    long CreateBlobLoader(const std::string& strFile) { return (long)m_cuda.RunFloatEx(m_hKernel, MCH_FN_CREATE_BLOBLOADER, {}, strFile).at(0); }
    void FreeBlobLoader(long h) { m_cuda.RunFloat(m_hKernel, MCH_FN_FREE_BLOBLOADER, {(float)h}); }
    void LoadBlob(long hBlobLoader, long long lCount, long hDst, long long lLocalOffsetInItems)
    {
        ex2(MCH_FN_BLOBLOADER_LOAD, {}, {hBlobLoader, lCount, hDst, lLocalOffsetInItems});
    }
    void BlobLoaderResetOffset(long hBlobLoader, long long lOffsetInBytes) { ex2(MCH_FN_BLOBLOADER_RESETOFFSET, {}, {hBlobLoader, lOffsetInBytes}); }
    void BlobLoaderAddToOffset(long hBlobLoader, long long lOffsetInItems) { ex2(MCH_FN_BLOBLOADER_ADDTOOFFSET, {}, {hBlobLoader, lOffsetInItems}); }

    // ---- cuDNN-shaped handles, softmax (CudaDnn.cs:3509-3527, 3819-3900, 4919)
    long CreateCuDNN(long hStream = 0) { return (long)m_cuda.RunFloat(m_hKernel, MCH_FN_CREATE_CUDNN, {(float)hStream}).at(0); }
    void FreeCuDNN(long h) { m_cuda.RunFloat(m_hKernel, MCH_FN_FREE_CUDNN, {(float)h}); }
    long CreateTensorDesc() { return (long)m_cuda.RunFloat(m_hKernel, MCH_FN_CREATE_TENSORDESC, {}).at(0); }
    void FreeTensorDesc(long h) { m_cuda.RunFloat(m_hKernel, MCH_FN_FREE_TENSORDESC, {(float)h}); }
    void SetTensorDesc(long hHandle, int n, int c, int h, int w, bool bHalf = false)
    {
        ex2(MCH_FN_SET_TENSORDESC, {}, {hHandle, bHalf, n, c, h, w});
    }
    void SoftmaxForward(long hCuDnn, long hBottomDesc, long hBottom, long hTopDesc, long hTop, int alg = 1, int mode = 1)
    {
        ex2(MCH_FN_SOFTMAX_FWD, {1.f, 0.f}, {hCuDnn, 0, hBottomDesc, hBottom, 0, hTopDesc, hTop, alg, mode});
    }

    void SoftmaxBackward(long hCuDnn, long hTopDataDesc, long hTopData, long hTopDiffDesc, long hTopDiff, long hBottomDiffDesc, long hBottomDiff,
                         int alg = 1, int mode = 1)   // :4941
    {
        ex2(MCH_FN_SOFTMAX_BWD, {1.f, 0.f}, {hCuDnn, 0, hTopDataDesc, hTopData, hTopDiffDesc, hTopDiff, 0, hBottomDiffDesc, hBottomDiff, alg, mode});
    }

    // ---- attention handle (CudaDnn.cs:5614-5701)
    long CreateAttn() { return (long)m_cuda.RunFloat(m_hKernel, MCH_FN_ATTN_CREATE, {}).at(0); }
    void FreeAttn(long h) { m_cuda.RunFloat(m_hKernel, MCH_FN_ATTN_FREE, {(float)h}); }
    void SetAttn(long hCuDnn, long hAttn, int nGpuID, bool bTraining, int nBatch, int nBlockSize, int nHeads, int nSize, float fDropout,
                 long long lSeed = 0)
    {
        ex2(MCH_FN_ATTN_SET, {fDropout}, {hCuDnn, hAttn, nGpuID, bTraining, nBatch, nBlockSize, nHeads, nSize, lSeed});
    }
    void AttnScaledDotProductForward(long hCuDnn, long hAttn, int nBlockSize, long hQ, long hK, long hV, long hMask, long hY, int nBatchMask = 1,
                                     bool bMergedY = false)
    {
        // the eleventh value (Y written head-merged, (B,T,H,hs)) has no counterpart in the reference
        if (bMergedY) ex2(MCH_FN_ATTN_FWD, {}, {hCuDnn, hAttn, nBlockSize, hQ, hK, hV, hMask, hY, nBatchMask, nBlockSize, 1});
        else ex2(MCH_FN_ATTN_FWD, {}, {hCuDnn, hAttn, nBlockSize, hQ, hK, hV, hMask, hY, nBatchMask});
    }
    // additions of this library (no counterpart in the reference)
    void AttnScaledDotProductBackward(long hCuDnn, long hAttn, long hQ, long hdQ, long hK, long hdK, long hV, long hdV, long hMask, long hY,
                                      long hdY)                                                                                // :5695
    {
        ex2(MCH_FN_ATTN_BWD, {}, {hCuDnn, hAttn, hQ, hdQ, hK, hdK, hV, hdV, hMask, hY, hdY});
    }
    void AttnDecodeForward(int nBatch, int nHeads, int nKvHeads, int nSize, int nLen, long hQ, long hKCache, long hVCache, long hY,
                           long long nStrideBatch, long long nStrideHead, long long nStridePos, float fScale = 0.f)
    {
        ex2(MCH_FN_ATTN_DECODE_FWD, {fScale}, {nBatch, nHeads, nKvHeads, nSize, nLen, hQ, hKCache, hVCache, hY, nStrideBatch, nStrideHead, nStridePos});
    }
    void AttnDecodeForwardNoAlloc(int nBatch, int nHeads, int nKvHeads, int nSize, int nLen, long hQ, long hKCache, long hVCache, long hY,
                                  long long nStrideBatch, long long nStrideHead, long long nStridePos, float fScale = 0.f)
    {
        m_cuda.AttnDecodeNoAlloc(m_hKernel, {fScale}, {nBatch, nHeads, nKvHeads, nSize, nLen, hQ, hKCache, hVCache, hY, nStrideBatch, nStrideHead, nStridePos});
    }
    // fused QKV projection: q, k, v = X W^T + bias written as (B,H,T,hs), q and k rotated when hRope is given (no
    // counterpart in the reference)
    void QkvProjHeads(int nBatch, int nT, int nHeads, int nSize, long hX, long hWeight, long hBias, long hQ, long hK, long hV,
                      long hRope = 0)
    {
        if (hRope) ex2(MCH_FN_QKV_PROJ_HEADS, {}, {nBatch, nT, nHeads, nSize, hX, hWeight, hBias, hQ, hK, hV, hRope});
        else ex2(MCH_FN_QKV_PROJ_HEADS, {}, {nBatch, nT, nHeads, nSize, hX, hWeight, hBias, hQ, hK, hV});
    }
    // y (M,N) = x (M,K) W^T (N,K) + bias (hBias 0: none) in one GEMM (no counterpart in the reference)
    void LinearForward(int nM, int nN, int nK, long hX, long hWeight, long hBias, long hY)
    {
        ex2(MCH_FN_LINEAR_FWD, {}, {nM, nN, nK, hX, hWeight, hBias, hY});
    }
    void RmsNormForward(int nOuter, int nDim, long hX, long hWeight, long hY, float fEps = 1e-5f)
    {
        ex2(MCH_FN_RMSNORM_FWD, {fEps}, {nOuter, nDim, hX, hWeight, hY});
    }

    // ---- RoPE (CudaDnn.cs:6375-6415)
    long CreateRope(int nSharedIndex, int nGpuID, long long nCount, int nBatch, int nSeqLen, int nHeads, int nDim, float fTheta = 10000.f)
    {
        return (long)ex2(MCH_FN_CREATE_ROPE, {fTheta}, {nSharedIndex, nGpuID, nCount, nBatch, nSeqLen, nHeads, nDim}).at(0);
    }
    void FreeRope(long h) { m_cuda.RunFloat(m_hKernel, MCH_FN_FREE_ROPE, {(float)h}); }
    void RopeForward(long hRope, long long n, long hX, long hY, int nFreqOffset = -1) { ex2(MCH_FN_ROPE_FWD, {}, {hRope, n, hX, hY, nFreqOffset}); }
    void RopeBackward(long hRope, long long n, long hXdata, long hYdiff, long hXdiff) { ex2(MCH_FN_ROPE_BWD, {}, {hRope, n, hXdata, hYdiff, hXdiff}); }   // :6425

    // ---- extensions (CudaDnn.cs:3703-3811)
    long CreateExtension(const std::string& strExtensionDllPath)
    {
        return (long)m_cuda.RunFloatEx(m_hKernel, MCH_FN_CREATE_EXTENSION, {}, strExtensionDllPath).at(0);
    }
    void FreeExtension(long hExtension) { m_cuda.RunFloat(m_hKernel, MCH_FN_FREE_EXTENSION, {(float)hExtension}); }
    std::vector<float> RunExtension(long hExtension, long lfnIdx, const std::vector<float>& rgParam, size_t capacity = 16)
    {
        std::vector<float> rg = {(float)hExtension, (float)lfnIdx};
        rg.insert(rg.end(), rgParam.begin(), rgParam.end());
        return m_cuda.RunFloat(m_hKernel, MCH_FN_EXTENSION_RUN, rg, capacity);
    }
    std::vector<float> RunExtensionEx(long hExtension, long lfnIdx, const std::vector<float>& rgParam, const std::string& strInput)
    {
        std::vector<float> rg = {(float)hExtension, (float)lfnIdx};
        rg.insert(rg.end(), rgParam.begin(), rgParam.end());
        return m_cuda.RunFloatEx(m_hKernel, MCH_FN_EXTENSION_RUN, rg, strInput);
    }
    std::string QueryExtensionStrings(long hExtension, long lfnIdx, const std::vector<int32_t>& rgParam)
    {
        std::vector<int32_t> rg = {(int32_t)hExtension, (int32_t)lfnIdx};
        rg.insert(rg.end(), rgParam.begin(), rgParam.end());
        return m_cuda.QueryStringFloatEx(m_hKernel, MCH_QRY_EXTENSION_STRING, rg);
    }

private:
    std::vector<float> ex2(long fn, const std::vector<float>& f, const std::vector<long long>& l) { return m_cuda.RunFloatEx2(m_hKernel, fn, f, l); }
    Marshaller m_cuda;
    std::string m_strPath;
    long m_hKernel = 0;
};

// ---- LlmInference (MyCaffe/common/LlmInference.cs), greedy decoding through token ids ----------------
class LlmInference {
public:
    LlmInference(CudaDnn& cuda, const std::string& strExtensionPath, float fTemperature = 0.f, float fTopp = 0.9f, long lSeed = 0) : m_cuda(cuda)
    {
        m_hExtension = m_cuda.CreateExtension(strExtensionPath);                                           // LlmInference.cs:110-130
        m_hLlm = (long)m_cuda.RunExtension(m_hExtension, MCH_LLM_CREATE, {fTemperature, fTopp, (float)lSeed}).at(0);
    }
    ~LlmInference()
    {
        try {
            if (m_hLlm) m_cuda.RunExtension(m_hExtension, MCH_LLM_DESTROY, {(float)m_hLlm});
            if (m_hExtension) m_cuda.FreeExtension(m_hExtension);
        } catch (...) {
        }
    }
    void Load(const std::string& strModelFile, const std::string& strTokenizerFile = "")                    // LlmInference.cs:150-190
    {
        m_cuda.RunExtensionEx(m_hExtension, MCH_LLM_LOAD, {(float)m_hLlm}, strModelFile + ";" + strTokenizerFile);
    }
    void SetOption(int option, float value) { m_cuda.RunExtension(m_hExtension, MCH_LLM_SET_OPTION, {(float)m_hLlm, (float)option, value}); }
    // ids forced for the prompt positions, then greedy; returns the id chosen after every position
    std::vector<int> GenerateIds(const std::vector<int>& prompt, int nSteps)
    {
        std::vector<float> rg = {(float)m_hLlm, (float)nSteps, 0.f};
        for (int id : prompt) rg.push_back((float)id);
        std::vector<float> out = m_cuda.RunExtension(m_hExtension, MCH_LLM_GENERATE_IDS, rg, (size_t)nSteps);
        return std::vector<int>(out.begin(), out.end());
    }
    // {milliseconds of the timed span, steps in it}
    std::vector<float> QueryTiming() { return m_cuda.RunExtension(m_hExtension, MCH_LLM_QUERY_TIMING, {(float)m_hLlm}); }

private:
    CudaDnn& m_cuda;
    long m_hExtension = 0, m_hLlm = 0;
};

}  // namespace mycaffe
