// Handle tables and per-kernel state of libmycaffe_hip.so.
//
// Mirrors the object model the reference DLL exposes through its C ABI: a table
// of "kernels" (one device context each, CudaDnnDLL/dllmain.cpp:6-14), and inside
// each kernel integer-handle tables for device memory and for the cuDNN /
// tensor-descriptor / attention / RoPE / extension objects
// (CudaDnnDLL/Cuda Files/memorycol.h:282-370, handlecol.h:21-113).
#pragma once
#include <hip/hip_runtime.h>

#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/mycaffe_hip_abi.h"
#include "kernels.h"

namespace mch {

struct MemItem {
    void* ptr = nullptr;
    size_t count = 0;     // elements
    bool half = false;    // 16-bit (bf16) storage
    bool used = false;
    bool view = false;    // aliases part of another item (memory pointer)
    long base = 0;        // owning handle when view
    uint64_t version = 0; // bumped on every write through the ABI
    int views = 0;        // memory pointers that alias this allocation
    // A whole-tensor SCAL that has not run yet: the contents are `pending` times what memory holds.  Only set on
    // allocations without views; every access through Kernel::mem() applies it first, except the mask calls, which
    // fold it into their own pass (the scale / mask pair of the explicit attention chain becomes one pass).
    float pending = 1.f;
    // The raw device address has been handed out (Internal_GetPointerFloat): its holder reads memory without passing
    // through Kernel::mem(), so nothing is ever held back on this allocation again.
    bool exposed = false;
    DType dt() const { return half ? BF16 : F32; }
    size_t esize() const { return half ? 2 : 4; }
};

// Device memory by handle.  Handles are 1-based; 0 is the null handle.
class MemTable {
public:
    long alloc(size_t count, bool half, hipStream_t s, long* h);
    long alloc_view(long hBase, size_t offset, size_t count, long* h);
    long free(long h);
    long get(long h, MemItem** it);
    void touch(long h);               // mark written
    uint64_t version(long h);
    void free_all();
private:
    long new_slot();
    std::vector<MemItem> m_items{1};  // slot 0 unused
    std::vector<long> m_free;
    uint64_t m_clock = 0;             // source of content versions
};

template <class S> class HandleTable {
public:
    long create(long* h)
    {
        for (size_t i = 1; i < m_items.size(); i++)
            if (!m_items[i]) { m_items[i].reset(new S()); *h = (long)i; return 0; }
        m_items.emplace_back(new S());
        *h = (long)m_items.size() - 1;
        return 0;
    }
    S* get(long h) { return (h > 0 && (size_t)h < m_items.size()) ? m_items[h].get() : nullptr; }
    long free(long h)
    {
        if (h <= 0 || (size_t)h >= m_items.size() || !m_items[h]) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        m_items[h].reset();
        return 0;
    }
    void clear() { m_items.clear(); m_items.emplace_back(nullptr); }
private:
    std::vector<std::unique_ptr<S>> m_items{1};
};

struct CudnnState { long stream = 0; };
struct TensorDesc { bool half = false; int n = 0, c = 0, h = 0, w = 0, sn = 0, sc = 0, sh = 0, sw = 0; };
struct AttnState {
    bool set = false, training = false;
    int batch = 0, block = 0, heads = 0, hs = 0;
    float dropout = 0.f, scale = 1.f;
    uint64_t seed = 0, fwdCalls = 0;   // dropout: seed of ATTN_SET, training-mode forward calls since
    AttnDropout drop = {0, 0, 1.f};    // mask parameters of the last training-mode forward call
    // cache of "the (T,T) mask is the lower-triangular ones matrix"
    long maskHandle = 0; uint64_t maskVersion = 0; int maskT = 0; bool maskCausal = false;
    // what the backward pass needs of the last training-mode forward: log2 of every row's softmax denominator
    float* lse = nullptr; size_t lseCap = 0; bool lseValid = false;
    void* ysave = nullptr; size_t ysaveBytes = 0;   // copy of that forward's output (the caller's Y buffer may be reused)
    int lastTq = 0, lastTk = 0; long long lastBatchMask = 0; long lastMask = 0;
    ~AttnState() { if (lse) (void)hipFree(lse); if (ysave) (void)hipFree(ysave); }
};
struct RopeState {
    bool set = false;
    int sharedIdx = 0, count = 0, batch = 0, seq = 0, heads = 0, hs = 0;
    float theta = 10000.f;
    std::shared_ptr<void> dcos, dsin;  // device tables [seq, hs/2] fp32, shared by sharedIdx
};
struct LayerNormState {
    bool set = false;
    int count = 0, outer = 0, channels = 0, inner = 0;
    float eps = 1e-10f;
    float* stdev = nullptr;   // [outer*channels] sqrt(var + eps) of the last forward
    int backwards = 0;        // backward calls since the last forward
    ~LayerNormState() { if (stdev) (void)hipFree(stdev); }
};
// read-only mapping of a weight file (CudaDnnDLL/Cuda Files/blobloader.h:25-70)
struct BlobLoaderState {
    int fd = -1;
    const unsigned char* data = nullptr;   // start of the mapping
    size_t fileSize = 0;
    size_t offsetBytes = 0;                // set by RESETOFFSET
    size_t offsetItems = 0;                // advanced by ADDTOOFFSET, cleared by RESETOFFSET
    ~BlobLoaderState();
};
// A whole-tensor, in-place mask call (ids 264 / 266) that has not run yet: X's contents are what that call would leave.
// At most one is outstanding.  A softmax forward over X takes it into its own pass; anything else that touches X or
// the mask blob runs it first (Kernel::mem), a call that overwrites all of X or frees it cancels it.
struct PendingMask {
    long hX = 0, hM = 0;
    long long n = 0;
    int md = 0, batch = 0;      // batch 0: plain mask (index i % md); else mask_batch
    float search = 0.f, replace = 0.f, xscale = 1.f;
};
// A GEMM2 call held back: the Q K^T product of the explicit attention chain, which the calls that follow scale, mask and
// put through a softmax.  If the mask turns out to be the causal one, the tiles wholly above the diagonal are never
// computed (the softmax does not read them and the mask call, whenever it is applied, overwrites them).
//
// kind 1 is a GEMM call held back the same way: the product of an inner product layer, Y = X W^T written over the whole of
// Y in fp32.  When the next call on Y is the rank-1 update that adds the bias to every row (ones (m) times bias (n), alpha =
// beta = 1), both run as one launch with the bias added where the tile is stored - the sum is rounded once either way, so
// no result changes.  lda/ldb/ldc, the strides and batch are unused then.
struct PendingProduct {
    int kind = 0;
    long hA = 0, hB = 0, hC = 0;
    int m = 0, n = 0, k = 0, lda = 0, ldb = 0, ldc = 0, batch = 0;
    long long sA = 0, sB = 0, sC = 0;
    float alpha = 1.f;
};
struct OnesCacheEntry { long handle = 0; uint64_t version = 0; int n = 0; bool ones = false; };
struct PermuteCacheEntry { uint64_t key[6]; int axes; PermuteArgs args; };
struct ExtensionState {
    void* lib = nullptr;
    void* fnInvoke = nullptr;
    void* fnInvokeEx = nullptr;
    ~ExtensionState();
};

class Kernel {
public:
    Kernel();
    ~Kernel();
    long initialize(const float* pf, long n);
    long run(long fn, float* pf, long lf, MCH_LONGLONG* pl, long ll, float** ppOut, MCH_LONG* plOut, bool timing);
    long attn_decode_no_alloc(float* pf, long lf, MCH_LONGLONG* pl, long ll);
    long run_extension(long hExt, long fn, float* pf, long lf, MCH_TCHAR* szIn, float** ppOut, MCH_LONG* plOut,
                       MCH_TCHAR* szErr, long errMax);
    long create_extension(long kernelIdx, MCH_TCHAR* path, float** ppOut, MCH_LONG* plOut);
    long create_blobloader(MCH_TCHAR* path, float** ppOut, MCH_LONG* plOut);
    long query_extension(MCH_LONG* pIn, long n, MCH_TCHAR* out, long outMax, MCH_TCHAR* err, long errMax);
    long alloc_host(long count, float** dst, const float* src, bool srcOnDevice);
    long free_host(float* p);
    long get_pointer(long h, void** pp);
    hipStream_t stream() const { return m_stream; }
    int device() const { return m_device; }
    std::string device_name();
    std::string last_detail;  // human-readable detail of the last failure

private:
    long attn_decode_fwd(float* pf, long lf, MCH_LONGLONG* pl, long ll, bool staticScratch);
    long workspace(size_t bytes, void** p);
    long staging(size_t bytes, void** p);
    long tickets(size_t count, int** p);
    long mem(long h, MemItem** it);                                            // with any deferred scaling applied
    long mem_lazy(long h, MemItem** it);                                       // as it is; the caller deals with `pending`
    // an operand of a product: a deferred scaling by a power of two stays deferred and goes into *fold (the product's alpha
    // takes it: every partial product and sum is the same number times that power, so no bit changes)
    long mem_factor(long h, MemItem** it, float* fold);
    // the target of a call that writes all `count` elements without reading any: what was held back for it is dropped
    long mem_overwritten(long h, MemItem** it, long long count);
    PendingProduct m_pendingProduct;
    long flush_pending_product(bool causal = false);
    long mask_operands(long hX, long hM, long hY, long long n, MemItem** X, MemItem** M, MemItem** Y, float* xscale);
    long flush_pending_mask();
    bool defer_mask(long hX, long hM, long hY, MemItem* X, MemItem* M, long long n, int md, int batch, float search, float replace,
                    float xscale, bool timing);
    PendingMask m_pendingMask;
    bool mask_is_causal(AttnState* st, long hMask, MemItem* mask, int T);
    bool tril_scan(MemItem* mask, int T, bool* causal);
    bool held_mask_is_causal(long hMask, MemItem* mask, int T);
    // whether the first n entries of an fp32 blob are all 1.0 (the bias multiplier of an inner product layer): one scan and
    // host read-back per (handle, content version), a few blobs remembered
    bool vector_is_ones(long h, MemItem* v, int n);
    OnesCacheEntry m_onesCache[16]; int m_onesNext = 0;
    long m_heldMaskHandle = 0; uint64_t m_heldMaskVersion = 0; int m_heldMaskT = 0; bool m_heldMaskCausal = false;
    // the last output of a softmax with a causal mask folded in: (handle, content version) of the tensor, its row length
    // and row count; m_zeroFlag (device) holds m_zeroEpoch if one of its rows has a masked entry that is not exactly zero
    int* m_zeroFlag = nullptr; int m_zeroEpoch = 0;
    long m_zeroHandle = 0; uint64_t m_zeroVersion = 0; int m_zeroLen = 0; size_t m_zeroRows = 0;

    int m_device = 0;
    hipStream_t m_stream = nullptr;
    MemTable m_mem;
    HandleTable<CudnnState> m_cudnn;
    HandleTable<TensorDesc> m_tdesc;
    HandleTable<AttnState> m_attn;
    HandleTable<RopeState> m_rope;
    HandleTable<LayerNormState> m_layernorm;
    HandleTable<ExtensionState> m_ext;
    HandleTable<BlobLoaderState> m_blobLoader;
    std::map<int, std::weak_ptr<void>> m_ropeSharedCos, m_ropeSharedSin;
    void* m_ws = nullptr; size_t m_wsBytes = 0;          // device scratch (split-K partials, conversions)
    int* m_tickets = nullptr; size_t m_ticketCount = 0;  // split-K merge tickets; zero whenever no kernel is running
    void* m_stage = nullptr; size_t m_stageBytes = 0;    // pinned host staging
    std::mutex m_stageLock;
    std::vector<PermuteCacheEntry> m_permuteCache;   // decoded TRANSPOSE arguments by (blob handles, versions)
    std::vector<float*> m_hostAllocs;
    std::mutex m_hostLock;
};

// UTF-16 helpers
std::string utf16_to_utf8(const MCH_TCHAR* s);
void utf8_to_utf16(const std::string& s, MCH_TCHAR* out, long max);

}  // namespace mch
