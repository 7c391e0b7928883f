// libmycaffe_hip.so: exported C ABI, kernel table, argument unmarshalling.
//
// Every case of Kernel::run reproduces the argument positions of the reference's
// Device<T> unmarshaller for that function id (CudaDnnDLL/Cuda Files/device.cu,
// device.h; positions are quoted per case) and then enqueues hand-written gfx950
// kernels on the kernel's own HIP stream.  Compute calls return without waiting;
// calls that hand data to the host (GETMEM, SYNCHRONIZEDEVICE, extension results)
// wait for the stream, so "returned means visible" holds for everything the host
// can observe.
#include <dlfcn.h>
#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <climits>

#include "runtime.h"

namespace mch {

#define HIPCHK(x) do { hipError_t _e = (x); if (_e != hipSuccess) return (long)_e; } while (0)
#define ERRCHK(x) do { long _e = (x); if (_e) return _e; } while (0)

// ---------------------------------------------------------------------------
std::string utf16_to_utf8(const MCH_TCHAR* s)
{
    std::string out;
    if (!s) return out;
    for (; *s; s++) {
        uint32_t c = *s;
        if (c >= 0xD800 && c <= 0xDBFF && s[1] >= 0xDC00 && s[1] <= 0xDFFF) {
            c = 0x10000 + ((c - 0xD800) << 10) + (s[1] - 0xDC00);
            s++;
        }
        if (c < 0x80) out += (char)c;
        else if (c < 0x800) { out += (char)(0xC0 | (c >> 6)); out += (char)(0x80 | (c & 0x3F)); }
        else if (c < 0x10000) { out += (char)(0xE0 | (c >> 12)); out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F)); }
        else { out += (char)(0xF0 | (c >> 18)); out += (char)(0x80 | ((c >> 12) & 0x3F)); out += (char)(0x80 | ((c >> 6) & 0x3F)); out += (char)(0x80 | (c & 0x3F)); }
    }
    return out;
}

void utf8_to_utf16(const std::string& s, MCH_TCHAR* out, long max)
{
    if (!out || max <= 0) return;
    long o = 0;
    for (size_t i = 0; i < s.size() && o < max - 1;) {
        uint32_t c = (unsigned char)s[i];
        int n = c < 0x80 ? 1 : (c >> 5) == 6 ? 2 : (c >> 4) == 14 ? 3 : 4;
        if (n == 2) c &= 0x1F; else if (n == 3) c &= 0x0F; else if (n == 4) c &= 0x07;
        for (int j = 1; j < n && i + j < s.size(); j++) c = (c << 6) | ((unsigned char)s[i + j] & 0x3F);
        i += n;
        if (c >= 0x10000) {
            if (o >= max - 2) break;
            c -= 0x10000;
            out[o++] = (MCH_TCHAR)(0xD800 + (c >> 10));
            out[o++] = (MCH_TCHAR)(0xDC00 + (c & 0x3FF));
        } else out[o++] = (MCH_TCHAR)c;
    }
    out[o] = 0;
}

// ---------------------------------------------------------------------------
long MemTable::new_slot()
{
    if (!m_free.empty()) { long h = m_free.back(); m_free.pop_back(); return h; }
    m_items.emplace_back();
    return (long)m_items.size() - 1;
}

long MemTable::alloc(size_t count, bool half, hipStream_t s, long* h)
{
    void* p = nullptr;
    size_t bytes = count * (half ? 2 : 4);
    if (bytes == 0) bytes = 4;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return e == hipErrorOutOfMemory ? (long)MCH_ERROR_MEMORY_OUT : (long)e;
    // every device allocation starts zero-filled (memorycol.h:75-107); callers rely on it
    e = hipMemsetAsync(p, 0, bytes, s);
    if (e != hipSuccess) { (void)hipFree(p); return (long)e; }
    long slot = new_slot();
    MemItem& it = m_items[slot];
    it = MemItem();
    it.ptr = p; it.count = count; it.half = half; it.used = true;
    it.version = ++m_clock;
    *h = slot;
    return 0;
}

long MemTable::alloc_view(long hBase, size_t offset, size_t count, long* h)
{
    MemItem* b;
    ERRCHK(get(hBase, &b));
    if (offset + count > b->count) return MCH_ERROR_MEMORY_RANGE_EXCEEDED;
    long root = b->view ? b->base : hBase;
    char* p = (char*)b->ptr + offset * b->esize();
    bool half = b->half;
    long slot = new_slot();
    MemItem& it = m_items[slot];  // b may dangle after new_slot(); not used below
    it = MemItem();
    it.ptr = p; it.count = count; it.half = half; it.used = true; it.view = true; it.base = root;
    it.version = ++m_clock;
    m_items[root].views++;
    *h = slot;
    return 0;
}

long MemTable::get(long h, MemItem** it)
{
    if (h <= 0 || (size_t)h >= m_items.size() || !m_items[h].used) return MCH_ERROR_MEMORY_NOT_FOUND;
    *it = &m_items[h];
    return 0;
}

long MemTable::free(long h)
{
    MemItem* it;
    ERRCHK(get(h, &it));
    if (!it->view) {
        // views of this allocation die with it
        for (size_t i = 1; i < m_items.size(); i++)
            if (m_items[i].used && m_items[i].view && m_items[i].base == h) { m_items[i] = MemItem(); m_free.push_back((long)i); }
        hipError_t e = hipFree(it->ptr);
        if (e != hipSuccess) return (long)e;
    } else if (it->base > 0 && (size_t)it->base < m_items.size() && m_items[it->base].used) {
        m_items[it->base].views--;
    }
    *it = MemItem();
    m_free.push_back(h);
    return 0;
}

void MemTable::touch(long h)
{
    MemItem* it;
    if (get(h, &it)) return;
    // one clock for the whole table: a (handle, version) pair never repeats, also after the handle is freed and reused
    it->version = ++m_clock;
    if (it->view && !get(it->base, &it)) it->version = m_clock;
}

uint64_t MemTable::version(long h)
{
    MemItem* it;
    if (get(h, &it)) return 0;
    uint64_t v = it->version;
    if (it->view && !get(it->base, &it) && it->version > v) v = it->version;   // a write through the base changes the view
    return v;
}

void MemTable::free_all()
{
    for (size_t i = 1; i < m_items.size(); i++)
        if (m_items[i].used && !m_items[i].view) (void)hipFree(m_items[i].ptr);
    m_items.assign(1, MemItem());
    m_free.clear();
}

BlobLoaderState::~BlobLoaderState()
{
    if (data) munmap((void*)data, fileSize);
    if (fd >= 0) close(fd);
}

ExtensionState::~ExtensionState()
{
    if (lib) dlclose(lib);
}

// ---------------------------------------------------------------------------
// Scratch of the entry point that allocates nothing (MCH_AttnDecodeForwardNoAlloc): merge tickets followed by the
// split-K partials of the decode attention.  Every GPU this library runs on holds its own copy of the array until the
// process ends; g_scratch below is only the host-side stand-in of the symbol, the device address is looked up once per
// device and that pointer is what kernels, fills and copies get.
enum : long long { MCH_NOALLOC_MAX_TICKETS = 4096, MCH_NOALLOC_PARTIAL_BYTES = 4ll << 20 };
static __device__ __align__(256) unsigned char g_scratch[MCH_NOALLOC_MAX_TICKETS * sizeof(int) + MCH_NOALLOC_PARTIAL_BYTES];
static char* g_scratchPtr[64];
static std::mutex g_scratchLock;

// looks the array's address up on `device`, which must be the current device; called when a kernel object is
// initialised on it
static long static_scratch_init(int device)
{
    if (device < 0 || device >= 64) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    std::lock_guard<std::mutex> g(g_scratchLock);
    if (g_scratchPtr[device]) return 0;
    void* p = nullptr;
    HIPCHK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_scratch)));
    if (!p) return MCH_ERROR_MEMORY_NULL;
    g_scratchPtr[device] = (char*)p;
    return 0;
}

static long static_scratch(int device, char** p)
{
    if (device < 0 || device >= 64) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    std::lock_guard<std::mutex> g(g_scratchLock);
    if (!g_scratchPtr[device]) return MCH_ERROR_DEVICE_NOT_INITIALIZED;
    *p = g_scratchPtr[device];
    return 0;
}

// ---------------------------------------------------------------------------
Kernel::Kernel() {}

Kernel::~Kernel()
{
    if (m_stream) (void)hipStreamSynchronize(m_stream);
    m_ext.clear();
    m_blobLoader.clear();
    m_rope.clear();
    m_layernorm.clear();
    m_mem.free_all();
    if (m_ws) (void)hipFree(m_ws);
    if (m_zeroFlag) (void)hipFree(m_zeroFlag);
    if (m_tickets) (void)hipFree(m_tickets);
    if (m_stage) (void)hipHostFree(m_stage);
    for (float* p : m_hostAllocs) (void)hipHostFree(p);
    if (m_stream) (void)hipStreamDestroy(m_stream);
}

long Kernel::initialize(const float* pf, long n)
{
    // SetDevice: f{deviceId, flags[, seed]} (device.cu:772-795)
    if (n < 2 || n > 3) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    if (!pf) return MCH_ERROR_PARAM_NULL;
    int count = 0;
    HIPCHK(hipGetDeviceCount(&count));
    int dev = (int)pf[0];
    if (dev < 0 || dev >= count) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    m_device = dev;
    HIPCHK(hipSetDevice(dev));
    if (!m_stream) HIPCHK(hipStreamCreateWithFlags(&m_stream, hipStreamNonBlocking));
    ERRCHK(static_scratch_init(dev));
    return 0;
}

std::string Kernel::device_name()
{
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, m_device) != hipSuccess) return "unknown";
    char buf[512];
    // some driver stacks report no marketing name
    snprintf(buf, sizeof(buf), "%s (%s, %d CUs, %.1f GB)", p.name[0] ? p.name : "AMD GPU", p.gcnArchName, p.multiProcessorCount,
             (double)p.totalGlobalMem / (1024.0 * 1024.0 * 1024.0));
    return buf;
}

long Kernel::workspace(size_t bytes, void** p)
{
    if (bytes > m_wsBytes) {
        if (m_ws) { HIPCHK(hipStreamSynchronize(m_stream)); HIPCHK(hipFree(m_ws)); m_ws = nullptr; m_wsBytes = 0; }
        size_t want = bytes < (size_t)(8u << 20) ? (size_t)(8u << 20) : bytes + bytes / 4;
        HIPCHK(hipMalloc(&m_ws, want));
        m_wsBytes = want;
    }
    *p = m_ws;
    return 0;
}

long Kernel::tickets(size_t count, int** p)
{
    if (count > m_ticketCount) {
        if (m_tickets) { HIPCHK(hipStreamSynchronize(m_stream)); HIPCHK(hipFree(m_tickets)); m_tickets = nullptr; m_ticketCount = 0; }
        size_t want = count < 4096 ? 4096 : count * 2;
        HIPCHK(hipMalloc((void**)&m_tickets, want * sizeof(int)));
        HIPCHK(hipMemsetAsync(m_tickets, 0, want * sizeof(int), m_stream));
        m_ticketCount = want;
    }
    *p = m_tickets;
    return 0;
}

long Kernel::staging(size_t bytes, void** p)
{
    if (bytes > m_stageBytes) {
        if (m_stage) { HIPCHK(hipStreamSynchronize(m_stream)); HIPCHK(hipHostFree(m_stage)); m_stage = nullptr; m_stageBytes = 0; }
        size_t want = bytes < (size_t)(4u << 20) ? (size_t)(4u << 20) : bytes + bytes / 4;
        HIPCHK(hipHostMalloc(&m_stage, want, hipHostMallocDefault));
        m_stageBytes = want;
    }
    *p = m_stage;
    return 0;
}

long Kernel::alloc_host(long count, float** dst, const float* src, bool srcOnDevice)
{
    if (count < 0 || !dst) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    float* p = nullptr;
    HIPCHK(hipHostMalloc((void**)&p, (size_t)(count > 0 ? count : 1) * sizeof(float), hipHostMallocDefault));
    if (src && count > 0) {
        if (srcOnDevice) {
            hipError_t e = hipMemcpyAsync(p, src, (size_t)count * 4, hipMemcpyDeviceToHost, m_stream);
            if (e == hipSuccess) e = hipStreamSynchronize(m_stream);
            if (e != hipSuccess) { (void)hipHostFree(p); return (long)e; }
        } else memcpy(p, src, (size_t)count * 4);
    }
    std::lock_guard<std::mutex> g(m_hostLock);
    m_hostAllocs.push_back(p);
    *dst = p;
    return 0;
}

long Kernel::free_host(float* p)
{
    std::lock_guard<std::mutex> g(m_hostLock);
    for (size_t i = 0; i < m_hostAllocs.size(); i++)
        if (m_hostAllocs[i] == p) {
            m_hostAllocs.erase(m_hostAllocs.begin() + i);
            HIPCHK(hipHostFree(p));
            return 0;
        }
    return MCH_ERROR_MEMORY_NOT_FOUND;
}

// The held-back product, in full or (causal) up to the diagonal tiles.  Its operands were resolved when the call was
// recorded; every later call that names one of them runs it first (mem / mem_lazy), so they still hold what the call saw.
long Kernel::flush_pending_product(bool causal)
{
    const PendingProduct p = m_pendingProduct;
    m_pendingProduct = PendingProduct();
    if (!p.hC) return 0;
    MemItem *A, *B, *C;
    if (m_mem.get(p.hA, &A) || m_mem.get(p.hB, &B) || m_mem.get(p.hC, &C)) return 0;   // an operand is gone
    if (p.kind == 1) {
        HIPCHK(k_gemm(m_stream, F32, false, true, p.m, p.n, p.k, p.alpha, A->ptr, B->ptr, 0.f, C->ptr));
        return 0;
    }
    HIPCHK(k_gemm2(m_stream, false, false, p.m, p.n, p.k, p.alpha, (const float*)A->ptr, (const float*)B->ptr, 0.f, (float*)C->ptr,
                   p.lda, p.ldb, p.ldc, p.sA, p.sB, p.sC, p.batch, nullptr, 0, causal));
    return 0;
}

long Kernel::mem_lazy(long h, MemItem** it)
{
    ERRCHK(m_mem.get(h, it));
    if (m_pendingProduct.hC) {
        const long hr = (*it)->view ? (*it)->base : h;
        if (hr == m_pendingProduct.hA || hr == m_pendingProduct.hB) ERRCHK(flush_pending_product());
    }
    return 0;
}

long Kernel::flush_pending_mask()
{
    if (m_pendingProduct.hC && m_pendingProduct.hC == m_pendingMask.hX) ERRCHK(flush_pending_product());
    const PendingMask p = m_pendingMask;
    m_pendingMask = PendingMask();
    if (!p.hX) return 0;
    MemItem *X, *M;
    if (m_mem.get(p.hX, &X) || m_mem.get(p.hM, &M)) return 0;   // an operand is gone: nothing left to apply it to
    if (p.batch == 0) HIPCHK(k_mask(m_stream, X->dt(), (size_t)p.n, p.md, p.search, p.replace, X->ptr, M->ptr, X->ptr, p.xscale));
    else HIPCHK(k_mask_batch(m_stream, X->dt(), (size_t)p.n, p.batch, p.md, p.search, p.replace, X->ptr, M->ptr, X->ptr, p.xscale));
    return 0;
}

// Holds a mask call back when it masks a large whole allocation in place (the attention chain's score tensor), so that
// the softmax that follows can do both in one pass.  The folded-in scaling of X moves into the record.
bool Kernel::defer_mask(long hX, long hM, long hY, MemItem* X, MemItem* M, long long n, int md, int batch, float search,
                        float replace, float xscale, bool timing)
{
    if (timing || hX != hY || hX == hM || X->view || X->views != 0 || X->exposed || M->view || M->exposed || (size_t)n != X->count || n < (1 << 20)) return false;
    m_pendingMask.hX = hX; m_pendingMask.hM = hM; m_pendingMask.n = n; m_pendingMask.md = md; m_pendingMask.batch = batch;
    m_pendingMask.search = search; m_pendingMask.replace = replace; m_pendingMask.xscale = xscale;
    X->pending = 1.f;
    return true;
}

long Kernel::mem(long h, MemItem** it)
{
    ERRCHK(m_mem.get(h, it));
    MemItem* root = *it;
    if (m_pendingProduct.hC) {
        const long hr = root->view ? root->base : h;
        if (hr == m_pendingProduct.hA || hr == m_pendingProduct.hB || hr == m_pendingProduct.hC) ERRCHK(flush_pending_product());
    }
    if (m_pendingMask.hX) {
        const long hr = root->view ? root->base : h;
        if (hr == m_pendingMask.hX || hr == m_pendingMask.hM) ERRCHK(flush_pending_mask());
    }
    if (root->view && m_mem.get(root->base, &root)) return 0;
    if (root->pending != 1.f) {
        const float a = root->pending;
        root->pending = 1.f;
        HIPCHK(k_scale(m_stream, root->dt(), root->count, a, root->ptr, root->ptr));
    }
    return 0;
}

static inline bool power_of_two(float f)
{
    int e;
    return f > 0.f && std::isfinite(f) && frexpf(f, &e) == 0.5f && e > -100 && e < 100;
}

long Kernel::mem_factor(long h, MemItem** it, float* fold)
{
    ERRCHK(m_mem.get(h, it));
    MemItem* r = *it;
    if (r->view || r->pending == 1.f || !power_of_two(r->pending) || m_pendingMask.hX == h || m_pendingMask.hM == h ||
        m_pendingProduct.hC == h)
        return mem(h, it);
    if (m_pendingProduct.hC && (h == m_pendingProduct.hA || h == m_pendingProduct.hB)) ERRCHK(flush_pending_product());
    *fold *= r->pending;
    return 0;
}

long Kernel::mem_overwritten(long h, MemItem** it, long long count)
{
    ERRCHK(m_mem.get(h, it));
    MemItem* r = *it;
    if (r->view || count < 0 || (size_t)count != r->count || m_pendingMask.hM == h) return mem(h, it);
    if (m_pendingProduct.hC == h) m_pendingProduct = PendingProduct();
    else if (m_pendingProduct.hA == h || m_pendingProduct.hB == h) ERRCHK(flush_pending_product());
    if (m_pendingMask.hX == h) m_pendingMask = PendingMask();
    r->pending = 1.f;
    return 0;
}

// Operands of a mask call.  When X carries a deferred scaling and the call masks the whole tensor in place, the factor
// is handed to the mask kernel (*xscale) instead of being applied in a pass of its own.
long Kernel::mask_operands(long hX, long hM, long hY, long long n, MemItem** X, MemItem** M, MemItem** Y, float* xscale)
{
    *xscale = 1.f;
    if (m_pendingMask.hX) ERRCHK(flush_pending_mask());   // one outstanding mask call at a time
    ERRCHK(mem(hM, M));
    MemItem* x;
    ERRCHK(mem_lazy(hX, &x));
    if (m_pendingProduct.hC == hX && m_pendingProduct.kind == 0 && hX == hY && n > 0 && (size_t)n == x->count) {
        // the result of a held-back product, masked in place as a whole: the caller either holds the mask back as well
        // or runs the product first
        *X = *Y = x;
        return 0;
    }
    if (!x->view && x->pending != 1.f && hX == hY && n > 0 && (size_t)n == x->count) {
        *xscale = x->pending;   // the caller clears `pending` once its kernel is launched
        *X = *Y = x;
        return 0;
    }
    ERRCHK(mem(hX, X));
    ERRCHK(mem(hY, Y));
    return 0;
}

long Kernel::get_pointer(long h, void** pp)
{
    MemItem* it;
    ERRCHK(mem(h, &it));
    it->exposed = true;
    MemItem* root;
    if (it->view && !m_mem.get(it->base, &root)) root->exposed = true;
    *pp = it->ptr;
    return 0;
}

static inline long verify(long n, const void* p, long lo, long hi)
{
    // verifyInput (device.h:712-745)
    if (n < lo || n > hi) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    if (lo == 0 && hi == 0) return 0;
    if (!p) return MCH_ERROR_PARAM_NULL;
    return 0;
}

static inline long set_out(float v, float** ppOut, MCH_LONG* plOut)
{
    if (!plOut || !ppOut || !*ppOut) return MCH_ERROR_PARAM_NULL;
    if (*plOut < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    *plOut = 1;
    (*ppOut)[0] = v;
    return 0;
}

__global__ void check_tril_kernel(const float* m, int T, int* bad)
{
    size_t n = (size_t)T * T;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)blockDim.x * gridDim.x) {
        int r = (int)(i / T), c = (int)(i % T);
        float want = c <= r ? 1.f : 0.f;
        // any non-zero on/below the diagonal keeps the entry, so only zero-ness matters
        if ((m[i] == 0.f) != (want == 0.f)) *bad = 1;
    }
}

// true when the (T,T) mask keeps exactly the lower triangle; result cached per
// (handle, content version, T) so the scan and its host read-back happen once
bool Kernel::mask_is_causal(AttnState* st, long hMask, MemItem* mask, int T)
{
    // a blob whose device address was handed out can change without its version moving: it is read every time
    MemItem* root = mask;
    if (mask->exposed || (mask->view && !m_mem.get(mask->base, &root) && root->exposed)) return false;
    uint64_t ver = m_mem.version(hMask);
    if (st->maskHandle == hMask && st->maskVersion == ver && st->maskT == T) return st->maskCausal;
    bool causal;
    if (!tril_scan(mask, T, &causal)) return false;
    st->maskHandle = hMask; st->maskVersion = ver; st->maskT = T; st->maskCausal = causal;
    return st->maskCausal;
}

// one scan of a (T,T) fp32 mask and its host read-back; false when the scan could not be run
bool Kernel::tril_scan(MemItem* mask, int T, bool* causal)
{
    void* ws;
    if (workspace(256, &ws)) return false;
    int* flag = (int*)ws;
    if (hipMemsetAsync(flag, 0, sizeof(int), m_stream) != hipSuccess) return false;
    size_t n = (size_t)T * T;
    int grid = (int)((n + 255) / 256);
    if (grid > 2048) grid = 2048;
    hipLaunchKernelGGL(check_tril_kernel, grid, 256, 0, m_stream, (const float*)mask->ptr, T, flag);
    int bad = 1;
    if (hipMemcpyAsync(&bad, flag, sizeof(int), hipMemcpyDeviceToHost, m_stream) != hipSuccess) return false;
    if (hipStreamSynchronize(m_stream) != hipSuccess) return false;
    *causal = (bad == 0);
    return true;
}

__global__ void check_ones_kernel(const float* v, int n, int* bad)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += blockDim.x * gridDim.x)
        if (v[i] != 1.f) *bad = 1;
}

bool Kernel::vector_is_ones(long h, MemItem* v, int n)
{
    if (v->half || v->view || v->exposed || v->count < (size_t)n) return false;
    const uint64_t ver = m_mem.version(h);
    for (const OnesCacheEntry& e : m_onesCache)
        if (e.handle == h && e.version == ver && e.n >= n && e.ones) return true;
        else if (e.handle == h && e.version == ver && e.n <= n && !e.ones) return false;
    void* ws;
    if (workspace(256, &ws)) return false;
    int* flag = (int*)ws;
    if (hipMemsetAsync(flag, 0, sizeof(int), m_stream) != hipSuccess) return false;
    int grid = (n + 255) / 256;
    if (grid > 1024) grid = 1024;
    hipLaunchKernelGGL(check_ones_kernel, grid, 256, 0, m_stream, (const float*)v->ptr, n, flag);
    int bad = 1;
    if (hipMemcpyAsync(&bad, flag, sizeof(int), hipMemcpyDeviceToHost, m_stream) != hipSuccess) return false;
    if (hipStreamSynchronize(m_stream) != hipSuccess) return false;
    OnesCacheEntry& e = m_onesCache[m_onesNext];
    m_onesNext = (m_onesNext + 1) % 16;
    e.handle = h; e.version = ver; e.n = n; e.ones = (bad == 0);
    return e.ones;
}

// the same question for the mask blob of a held-back mask call (no attention handle to keep the answer on): cached per
// (handle, content version, T) on the kernel
bool Kernel::held_mask_is_causal(long hMask, MemItem* mask, int T)
{
    if (mask->half || mask->view || mask->exposed || mask->count < (size_t)T * T) return false;
    const uint64_t ver = m_mem.version(hMask);
    if (m_heldMaskHandle == hMask && m_heldMaskVersion == ver && m_heldMaskT == T) return m_heldMaskCausal;
    bool causal;
    if (!tril_scan(mask, T, &causal)) return false;
    m_heldMaskHandle = hMask; m_heldMaskVersion = ver; m_heldMaskT = T; m_heldMaskCausal = causal;
    return causal;
}

#define NEED_L(lo, hi) ERRCHK(verify(ll, pl, lo, hi))
#define NEED_F(lo, hi) ERRCHK(verify(lf, pf, lo, hi))
#define RANGE(item, off, n) do { if ((long long)(off) < 0 || (long long)(n) < 0 || (size_t)(off) + (size_t)(n) > (item)->count) { \
        last_detail = "range exceeds the allocation behind the memory handle"; return MCH_ERROR_MEMORY_RANGE_EXCEEDED; } } while (0)
#define PTR(item, off) ((char*)(item)->ptr + (size_t)(off) * (item)->esize())

long Kernel::run(long fn, float* pf, long lf, MCH_LONGLONG* pl, long ll, float** ppOut, MCH_LONG* plOut, bool timing)
{
    (void)timing;
    last_detail.clear();
    hipStream_t s = m_stream;
    if (!s) return MCH_ERROR_DEVICE_NOT_INITIALIZED;
    HIPCHK(hipSetDevice(m_device));

    switch (fn) {
    case MCH_FN_SETDEVICE:
        return initialize(pf, lf);

    case MCH_FN_GETDEVICE:
        return set_out((float)m_device, ppOut, plOut);

    case MCH_FN_SYNCHRONIZEDEVICE:
        // a held-back product runs now, so that a host that times a section between two of these calls sees all of its work
        // (a held-back mask stays: after the softmax pass that applied it on the fly it may never be needed in memory)
        if (m_pendingProduct.hC) ERRCHK(flush_pending_product());
        HIPCHK(hipStreamSynchronize(s));
        return 0;

    // ---- memory ------------------------------------------------------------
    case MCH_FN_ALLOCMEM:
    case MCH_FN_ALLOCMEM_HALF: {
        // l{count[,stream]}; optional f{count,[stream,] data...} (device.cu:854-949)
        NEED_L(1, 2);
        if (pl[0] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        size_t count = (size_t)pl[0];
        const float* src = nullptr;
        if (lf > 1) {
            if (!pf) return MCH_ERROR_PARAM_NULL;
            if ((size_t)lf == count + 1) src = pf + 1;
            else if ((size_t)lf == count + 2) src = pf + 2;
            else return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        bool half = fn == MCH_FN_ALLOCMEM_HALF;
        long h = 0;
        ERRCHK(m_mem.alloc(count, half, s, &h));
        if (src && count) {
            MemItem* it;
            ERRCHK(mem(h, &it));
            long e = 0;
            if (!half) {
                hipError_t he = hipMemcpyAsync(it->ptr, src, count * 4, hipMemcpyHostToDevice, s);
                if (he == hipSuccess) he = hipStreamSynchronize(s);
                e = (long)he;
            } else {
                void* ws;
                e = workspace(count * 4, &ws);
                if (!e) {
                    hipError_t he = hipMemcpyAsync(ws, src, count * 4, hipMemcpyHostToDevice, s);
                    if (he == hipSuccess) he = k_convert(s, F32, ws, BF16, it->ptr, count);
                    if (he == hipSuccess) he = hipStreamSynchronize(s);
                    e = (long)he;
                }
            }
            if (e) { m_mem.free(h); return e; }
        }
        return set_out((float)h, ppOut, plOut);
    }

    case MCH_FN_FREEMEM:
        NEED_L(1, 1);
        if (m_pendingProduct.hC == (long)pl[0]) m_pendingProduct = PendingProduct();   // the result goes: nothing to compute
        else if (m_pendingProduct.hA == (long)pl[0] || m_pendingProduct.hB == (long)pl[0]) ERRCHK(flush_pending_product());
        if (m_pendingMask.hX == (long)pl[0]) m_pendingMask = PendingMask();       // the tensor goes: nothing to apply
        else if (m_pendingMask.hM == (long)pl[0]) ERRCHK(flush_pending_mask());   // the mask blob goes: apply it now
        HIPCHK(hipStreamSynchronize(s));
        return m_mem.free((long)pl[0]);

    case MCH_FN_CREATE_MEMORYPOINTER: {
        // l{hData, offset, count} (device.h:1000-1020)
        NEED_L(3, 3);
        if (pl[1] < 0 || pl[2] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        long h = 0;
        MemItem* base;
        ERRCHK(mem((long)pl[0], &base));   // applies a deferred scaling before the allocation gets an alias
        ERRCHK(m_mem.alloc_view((long)pl[0], (size_t)pl[1], (size_t)pl[2], &h));
        return set_out((float)h, ppOut, plOut);
    }
    case MCH_FN_FREE_MEMORYPOINTER:
        NEED_L(1, 1);
        return m_mem.free((long)pl[0]);

    case MCH_FN_GETMEM: {
        // l{h, count(-1 = all)} (device.cu:973-1022)
        NEED_L(1, 2);
        if (!plOut || !ppOut) return MCH_ERROR_PARAM_NULL;
        MemItem* it;
        ERRCHK(mem((long)pl[0], &it));
        long long count = ll > 1 ? pl[1] : 0;
        if (count < 0) count = (long long)it->count;
        else if ((size_t)count > it->count) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (count > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const void* dsrc = it->ptr;
        if (it->half && count) {
            void* ws;
            ERRCHK(workspace((size_t)count * 4, &ws));
            HIPCHK(k_convert(s, BF16, it->ptr, F32, ws, (size_t)count));
            dsrc = ws;
        }
        if (count <= *plOut && *ppOut) {
            if (count) HIPCHK(hipMemcpyAsync(*ppOut, dsrc, (size_t)count * 4, hipMemcpyDeviceToHost, s));
            HIPCHK(hipStreamSynchronize(s));
        } else {
            float* host = nullptr;
            ERRCHK(alloc_host((long)count, &host, (const float*)dsrc, true));
            *ppOut = host;
        }
        *plOut = (MCH_LONG)count;
        return 0;
    }

    case MCH_FN_SETMEM: {
        // f{h, count, [stream,] data...}, l{h, count} (device.cu:1029-1091)
        NEED_F(2, INT_MAX);
        NEED_L(2, 2);
        if (pl[1] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        size_t count = (size_t)pl[1];
        const float* data;
        if (count == (size_t)lf - 2) data = pf + 2;
        else if (count == (size_t)lf - 3) data = pf + 3;
        else return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem* it;
        ERRCHK(mem((long)pl[0], &it));
        RANGE(it, 0, count);
        if (count == 0) return 0;
        if (!it->half) {
            HIPCHK(hipMemcpyAsync(it->ptr, data, count * 4, hipMemcpyHostToDevice, s));
        } else {
            void* ws;
            ERRCHK(workspace(count * 4, &ws));
            HIPCHK(hipMemcpyAsync(ws, data, count * 4, hipMemcpyHostToDevice, s));
            HIPCHK(k_convert(s, F32, ws, BF16, it->ptr, count));
        }
        HIPCHK(hipStreamSynchronize(s));  // the caller may reuse its buffer immediately
        m_mem.touch((long)pl[0]);
        return 0;
    }

    case MCH_FN_SET: {
        // f{val}, l{n, h, 0, idx, xOff} (device.h:6038-6061, math.cu:431-495)
        NEED_F(1, 1);
        NEED_L(3, 5);
        long long n = pl[0];
        long long idx = ll > 3 ? pl[3] : -1;
        long long off = ll > 4 ? pl[4] : 0;
        MemItem* it;
        ERRCHK(mem((long)pl[1], &it));
        m_mem.touch((long)pl[1]);
        if (pf[0] == 0.f && idx == -1 && off == 0) {
            HIPCHK(hipMemsetAsync(it->ptr, 0, it->count * it->esize(), s));
            return 0;
        }
        if (off < 0) off = 0;
        if (idx >= 0) {
            RANGE(it, off + idx, 1);
            HIPCHK(k_set(s, it->dt(), PTR(it, off + idx), 1, pf[0]));
        } else {
            RANGE(it, off, n);
            HIPCHK(k_set(s, it->dt(), PTR(it, off), (size_t)n, pf[0]));
        }
        return 0;
    }

    case MCH_FN_COPY: {
        // l{n, hSrc, hDst, srcOff, dstOff, hStream, srcHalfOverride, dstHalfOverride} (device.h:6063-6095)
        NEED_L(3, 8);
        long long n = pl[0];
        long long so = ll > 3 ? pl[3] : 0, dofs = ll > 4 ? pl[4] : 0;
        MemItem *src, *dst;
        ERRCHK(mem((long)pl[1], &src));
        ERRCHK(mem((long)pl[2], &dst));
        if (so < 0) so = 0;
        if (dofs < 0) dofs = 0;
        RANGE(src, so, n);
        RANGE(dst, dofs, n);
        HIPCHK(k_convert(s, src->dt(), PTR(src, so), dst->dt(), PTR(dst, dofs), (size_t)n));
        m_mem.touch((long)pl[2]);
        return 0;
    }

    // ---- BLAS-like -----------------------------------------------------------
    case MCH_FN_GEMM: {
        // f{alpha,beta}, l{tA,tB,m,n,k,0,hA,hB,0,hC,aOff,bOff,cOff,groups,gA,gB,gC} (device.cu:1636-1685)
        NEED_F(2, 2);
        NEED_L(10, 17);
        bool tA = pl[0] != 0, tB = pl[1] != 0;
        int m = (int)pl[2], n = (int)pl[3], k = (int)pl[4];
        long long aOff = ll > 10 ? pl[10] : 0, bOff = ll > 11 ? pl[11] : 0, cOff = ll > 12 ? pl[12] : 0;
        int groups = ll > 13 ? (int)pl[13] : 1;
        long long gA = ll > 14 ? pl[14] : 0, gB = ll > 15 ? pl[15] : 0, gC = ll > 16 ? pl[16] : 0;
        if (m < 0 || n < 0 || k < 0 || groups < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (aOff < 0) aOff = 0;
        if (bOff < 0) bOff = 0;
        if (cOff < 0) cOff = 0;
        MemItem *A, *B, *C;
        const long hA = (long)pl[6], hB = (long)pl[7], hC = (long)pl[9];
        // The bias of an inner product layer: ones (m) times bias (n) added to the held-back product X W^T.  Both run as one
        // launch that adds the bias where the tile is stored.
        if (m_pendingProduct.kind == 1 && m_pendingProduct.hC == hC && !tA && !tB && k == 1 && m == m_pendingProduct.m &&
            n == m_pendingProduct.n && pf[0] == 1.f && pf[1] == 1.f && groups == 1 && aOff == 0 && bOff == 0 && cOff == 0 &&
            hA != hC && hB != hC && hA != m_pendingProduct.hA && hA != m_pendingProduct.hB && hB != m_pendingProduct.hA &&
            hB != m_pendingProduct.hB) {
            ERRCHK(mem(hA, &A));
            ERRCHK(mem(hB, &B));
            if (m_pendingProduct.kind == 1 && m_pendingProduct.hC == hC && !A->half && !B->half && !B->view && B->count >= (size_t)n &&
                vector_is_ones(hA, A, m)) {
                const PendingProduct p = m_pendingProduct;
                MemItem *X, *W;
                if (!m_mem.get(p.hA, &X) && !m_mem.get(p.hB, &W) && !m_mem.get(p.hC, &C)) {
                    m_pendingProduct = PendingProduct();
                    void* ws = nullptr;
                    if (k_gemm_bias_needs_tmp(F32, p.n, p.k, X->ptr, W->ptr, C->ptr)) ERRCHK(workspace((size_t)p.m * p.n * 4, &ws));
                    HIPCHK(k_gemm_bias(s, F32, p.m, p.n, p.k, X->ptr, W->ptr, B->ptr, C->ptr, ws));
                    m_mem.touch(hC);
                    return 0;
                }
            }
        }
        ERRCHK(mem(hA, &A));
        ERRCHK(mem(hB, &B));
        // a product written over the whole of C leaves nothing of a held-back product into C to compute
        bool whole = false;
        if (hC != hA && hC != hB && pf[1] == 0.f && groups == 1 && cOff == 0 && !mem_lazy(hC, &C) && !C->view && C->views == 0 &&
            (size_t)m * n == C->count && C->pending == 1.f && m_pendingMask.hX != hC && m_pendingMask.hM != hC)
            whole = true;
        else
            ERRCHK(mem(hC, &C));
        if (A->half != B->half || A->half != C->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (whole) {
            RANGE(A, aOff, (long long)m * k);
            RANGE(B, bOff, (long long)k * n);
            if (m_pendingProduct.hC == hC) m_pendingProduct = PendingProduct();
            // Y = X W^T of an inner product layer, large enough for the saved pass to matter and not one whose contraction
            // the library would split over workgroups (that sum has another order than the fused launch's)
            if (!timing && !tA && tB && !A->half && pf[0] == 1.f && aOff == 0 && bOff == 0 && m >= 256 && n >= 64 && k >= 32 &&
                (long long)m * n >= (1ll << 20) && !A->view && !B->view && !A->exposed && !B->exposed && !C->exposed &&
                k_gemm_workspace_bytes(F32, false, true, m, n, k) == 0) {
                if (m_pendingProduct.hC) ERRCHK(flush_pending_product());   // one at a time
                PendingProduct& pp = m_pendingProduct;
                pp.kind = 1; pp.hA = hA; pp.hB = hB; pp.hC = hC; pp.m = m; pp.n = n; pp.k = k; pp.alpha = 1.f;
                m_mem.touch(hC);
                return 0;
            }
        }
        for (int g = 0; g < groups; g++) {
            long long ao = aOff + gA * g, bo = bOff + gB * g, co = cOff + gC * g;
            RANGE(A, ao, (long long)m * k);
            RANGE(B, bo, (long long)k * n);
            RANGE(C, co, (long long)m * n);
            // the transpose combinations of the layers' backward passes turn an operand in scratch memory
            void* ws = nullptr;
            const size_t wsb = k_gemm_workspace_bytes(A->dt(), tA, tB, m, n, k);
            if (wsb) ERRCHK(workspace(wsb, &ws));
            HIPCHK(k_gemm(s, A->dt(), tA, tB, m, n, k, pf[0], PTR(A, ao), PTR(B, bo), pf[1], PTR(C, co), ws, wsb));
        }
        m_mem.touch((long)pl[9]);
        return 0;
    }

    case MCH_FN_GEMM2: {
        // f{alpha,beta}, l{tA,tB,m,n,k,0,hA,hB,0,hC,lda,ldb,ldc[,sA,sB,sC,batch]}: BLAS column-major (device.cu:1691-1726)
        NEED_F(2, 2);
        NEED_L(13, 17);
        if (ll != 13 && ll != 17) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        bool tA = pl[0] != 0, tB = pl[1] != 0;
        int m = (int)pl[2], n = (int)pl[3], k = (int)pl[4];
        int lda = (int)pl[10], ldb = (int)pl[11], ldc = (int)pl[12];
        long long sA = 0, sB = 0, sC = 0;
        int batch = 1;
        if (ll == 17) { sA = pl[13]; sB = pl[14]; sC = pl[15]; batch = (int)pl[16]; }
        if (m < 0 || n < 0 || k < 0 || batch < 1 || lda < 1 || ldb < 1 || ldc < 1 || sA < 0 || sB < 0 || sC < 0)
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *A, *B, *C;
        float fold = 1.f;   // deferred power-of-two scalings of the operands (MatMulGrad scales a gradient, then multiplies by it twice)
        if (timing || (long)pl[9] == (long)pl[6] || (long)pl[9] == (long)pl[7]) {
            ERRCHK(mem((long)pl[6], &A));
            ERRCHK(mem((long)pl[7], &B));
        } else {
            ERRCHK(mem_factor((long)pl[6], &A, &fold));
            ERRCHK(mem_factor((long)pl[7], &B, &fold));
        }
        const float alpha2 = pf[0] * fold;
        // When every element of C is overwritten, a held-back scaling or mask call on C has nothing left to act on and is
        // cancelled (once the arguments have passed their checks) instead of being run first.
        bool overwrite = false;
        if ((long)pl[9] != (long)pl[6] && (long)pl[9] != (long)pl[7] && (long)pl[9] != m_pendingMask.hM && pf[1] == 0.f &&
            !mem_lazy((long)pl[9], &C) && !C->view && ldc == m && (batch == 1 || sC == (long long)m * n) &&
            (long long)batch * m * n == (long long)C->count)
            overwrite = true;
        else
            ERRCHK(mem((long)pl[9], &C));
        if (A->half || B->half || C->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;  // math.cu:1777-1778
        if (m == 0 || n == 0) return 0;
        long long ac = tA ? m : k, bc = tB ? k : n;  // stored column counts
        long long ar = tA ? k : m, br = tB ? n : k;
        RANGE(A, 0, (batch - 1) * sA + (ac - 1) * lda + ar);
        RANGE(B, 0, (batch - 1) * sB + (bc - 1) * ldb + br);
        RANGE(C, 0, (batch - 1) * sC + (long long)(n - 1) * ldc + m);
        if (overwrite) {
            C->pending = 1.f;
            if (m_pendingMask.hX == (long)pl[9]) m_pendingMask = PendingMask();
            if (m_pendingProduct.hC == (long)pl[9]) m_pendingProduct = PendingProduct();
            // Q K^T of the explicit attention chain (square result per batch entry, contraction = head size, everything
            // contiguous): held back until the calls that follow show what is needed of it
            if (!timing && !tA && !tB && m == n && m >= 256 && (k == 32 || k == 64 || k == 128) && lda == m && ldb == k &&
                (batch == 1 || (sA == (long long)m * k && sB == (long long)n * k)) && (long long)m * n * batch >= (1ll << 22) &&
                !A->view && !B->view && !A->exposed && !B->exposed && !C->exposed && C->views == 0 && (long)pl[6] != (long)pl[7] &&
                (((uintptr_t)A->ptr | (uintptr_t)B->ptr) & 15) == 0) {
                if (m_pendingProduct.hC) ERRCHK(flush_pending_product());   // one at a time
                PendingProduct& pp = m_pendingProduct;
                pp.hA = (long)pl[6]; pp.hB = (long)pl[7]; pp.hC = (long)pl[9];
                pp.m = m; pp.n = n; pp.k = k; pp.lda = lda; pp.ldb = ldb; pp.ldc = ldc; pp.batch = batch;
                pp.sA = sA; pp.sB = sB; pp.sC = sC; pp.alpha = alpha2;
                m_mem.touch((long)pl[9]);
                return 0;
            }
        }
        // The second operand is the output of a softmax with a causal mask folded in (the P V product of the explicit
        // attention chain): its entries above the diagonal are exact zeros - the softmax kernel raises a flag on the
        // device if a row's are not - and the contraction stops at the diagonal.
        const int* zeroFlag = nullptr;
        // (given transposed - the product P^T dY of the backward pass - the same zeros let it begin at the diagonal)
        if (m_zeroHandle && (long)pl[7] == m_zeroHandle && (long)pl[9] != m_zeroHandle && !tA && n == k && k == m_zeroLen &&
            ldb == k && (batch == 1 || sB == (long long)k * n) && (unsigned long long)batch * n <= m_zeroRows &&
            m_mem.version(m_zeroHandle) == m_zeroVersion && !B->view && !B->exposed)
            zeroFlag = m_zeroFlag;
        HIPCHK(k_gemm2(s, tA, tB, m, n, k, alpha2, (const float*)A->ptr, (const float*)B->ptr, pf[1], (float*)C->ptr, lda,
                       ldb, ldc, sA, sB, sC, batch, zeroFlag, m_zeroEpoch));
        m_mem.touch((long)pl[9]);
        return 0;
    }

    case MCH_FN_GEMV: {
        // f{alpha,beta}, l{tA,m,n,0,hA,hX,0,hY,aOff,xOff,yOff} (device.cu:1733-1767)
        NEED_F(2, 2);
        NEED_L(8, 11);
        bool tA = pl[0] != 0;
        int m = (int)pl[1], n = (int)pl[2];
        long long aOff = ll > 8 ? pl[8] : 0, xOff = ll > 9 ? pl[9] : 0, yOff = ll > 10 ? pl[10] : 0;
        if (m < 0 || n < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *A, *X, *Y;
        ERRCHK(mem((long)pl[4], &A));
        ERRCHK(mem((long)pl[5], &X));
        ERRCHK(mem((long)pl[7], &Y));
        // vectors in 16-bit storage are taken with a 16-bit matrix only (the bias gradient of an inner product kept in 16-bit
        // storage): they are widened into scratch memory below; the reference reads such memory as floats (math.cu:2155-2185)
        const bool all16 = A->half && X->half && Y->half;
        if ((X->half || Y->half) && !all16) return MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED;
        if (aOff < 0) aOff = 0;
        if (xOff < 0) xOff = 0;
        if (yOff < 0) yOff = 0;
        RANGE(A, aOff, (long long)m * n);
        RANGE(X, xOff, tA ? m : n);
        RANGE(Y, yOff, tA ? n : m);
        void* ws = nullptr;
        const size_t wsb = (k_gemv_workspace_bytes(tA, m, n) + 255) / 256 * 256;
        if (all16) {
            // the vectors widened into scratch memory (a few KB), the matrix read as it is stored, the result rounded once
            if (m == 0 || n == 0) return 0;
            const size_t nx = tA ? m : n, ny = tA ? n : m;
            const size_t xb = (nx * 4 + 255) / 256 * 256;
            ERRCHK(workspace(wsb + xb + ny * 4, &ws));
            float* xf = (float*)((char*)ws + wsb);
            float* yf = (float*)((char*)ws + wsb + xb);
            HIPCHK(k_convert(s, BF16, PTR(X, xOff), F32, xf, nx));
            if (pf[1] != 0.f) HIPCHK(k_convert(s, BF16, PTR(Y, yOff), F32, yf, ny));
            HIPCHK(k_gemv(s, BF16, tA, m, n, pf[0], PTR(A, aOff), xf, pf[1], yf, wsb ? ws : nullptr, wsb));
            HIPCHK(k_convert(s, F32, yf, BF16, PTR(Y, yOff), ny));
            m_mem.touch((long)pl[7]);
            return 0;
        }
        if (wsb) ERRCHK(workspace(wsb, &ws));
        HIPCHK(k_gemv(s, A->dt(), tA, m, n, pf[0], PTR(A, aOff), (const float*)PTR(X, xOff), pf[1], (float*)PTR(Y, yOff), ws, wsb));
        m_mem.touch((long)pl[7]);
        return 0;
    }

    case MCH_FN_AXPY: {
        // f{alpha}, l{n,0,hX,hY,xOff,yOff} (device.cu:1830-1857)
        NEED_F(1, 1);
        NEED_L(4, 6);
        long long n = pl[0], xo = ll > 4 ? pl[4] : 0, yo = ll > 5 ? pl[5] : 0;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[2], &X));
        ERRCHK(mem((long)pl[3], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, xo, n);
        RANGE(Y, yo, n);
        HIPCHK(k_axpy(s, X->dt(), (size_t)n, pf[0], PTR(X, xo), PTR(Y, yo)));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_SCAL: {
        // f{alpha}, l{n,0,hX,xOff} (device.cu:1887-1905)
        NEED_F(1, 1);
        NEED_L(3, 4);
        long long n = pl[0], xo = ll > 3 ? pl[3] : 0;
        MemItem* X;
        if (m_pendingProduct.hC == (long)pl[2] && m_pendingProduct.kind == 0 && m_pendingProduct.alpha == 1.f && !timing && xo == 0 &&
            !m_mem.get((long)pl[2], &X) && (size_t)n == X->count) {
            // the scaling of a held-back product's whole result becomes its alpha (one rounding either way, alpha being 1)
            m_pendingProduct.alpha = pf[0];
            m_mem.touch((long)pl[2]);
            return 0;
        }
        ERRCHK(mem((long)pl[2], &X));
        RANGE(X, xo, n);
        if (!timing && !X->view && X->views == 0 && !X->exposed && xo == 0 && (size_t)n == X->count && n >= (1 << 20)) {
            // a large whole tensor: the multiplication waits for the next call that touches the tensor; the mask calls
            // of the attention chain (scale, then mask in place) do it in their own pass
            X->pending = pf[0];
            m_mem.touch((long)pl[2]);
            return 0;
        }
        HIPCHK(k_scale(s, X->dt(), (size_t)n, pf[0], PTR(X, xo), PTR(X, xo)));
        m_mem.touch((long)pl[2]);
        return 0;
    }

    case MCH_FN_SCALE: {
        // f{alpha}, l{n,0,hX,hY,xOff,yOff} (device.cu:2028-2051)
        NEED_F(1, 1);
        NEED_L(4, 6);
        long long n = pl[0], xo = ll > 4 ? pl[4] : 0, yo = ll > 5 ? pl[5] : 0;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[2], &X));
        ERRCHK(mem((long)pl[3], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, xo, n);
        RANGE(Y, yo, n);
        HIPCHK(k_scale(s, X->dt(), (size_t)n, pf[0], PTR(X, xo), PTR(Y, yo)));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_ADD: {
        // [f{alpha}], l{n,hA,hB,hY}: y = a + alpha*b (device.cu:2208-2236, math.cu:3363-3369)
        if (lf > 0 && pf) NEED_F(1, 1);
        NEED_L(4, 5);
        long long n = pl[0];
        float alpha = (lf > 0 && pf) ? pf[0] : 1.f;
        MemItem *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        if (A->half != B->half || A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(A, 0, n);
        RANGE(B, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_add(s, A->dt(), (size_t)n, A->ptr, B->ptr, Y->ptr, alpha));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_MUL: {
        // l{n,hA,hB,hY,aOff,bOff,yOff} (device.cu:2398-2423)
        NEED_L(4, 7);
        long long n = pl[0], ao = ll > 4 ? pl[4] : 0, bo = ll > 5 ? pl[5] : 0, yo = ll > 6 ? pl[6] : 0;
        MemItem *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        if (A->half != B->half || A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(A, ao, n);
        RANGE(B, bo, n);
        RANGE(Y, yo, n);
        HIPCHK(k_mul(s, A->dt(), (size_t)n, PTR(A, ao), PTR(B, bo), PTR(Y, yo)));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_SUB: {
        // l{n,hA,hB,hY[,aOff,bOff,yOff,nB]}: y = a - b[i % nB] when nB > 0 (CudaDnn.cs:8132-8138, device.cu:2294-2331)
        NEED_L(4, 8);
        long long n = pl[0], ao = ll > 4 ? pl[4] : 0, bo = ll > 5 ? pl[5] : 0, yo = ll > 6 ? pl[6] : 0, nB = ll > 7 ? pl[7] : 0;
        MemItem *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        if (A->half != B->half || A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (nB < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(A, ao, n);
        RANGE(B, bo, nB > 0 ? (nB < n ? nB : n) : n);
        RANGE(Y, yo, n);
        HIPCHK(k_sub(s, A->dt(), (size_t)n, PTR(A, ao), PTR(B, bo), PTR(Y, yo), (size_t)nB));
        m_mem.touch((long)pl[3]);
        return 0;
    }
    case MCH_FN_DIV: {
        // l{n,hA,hB,hY}: y = b == 0 ? 0 : a / b (CudaDnn.cs:8281-8287, device.cu:2492-2505)
        NEED_L(4, 4);
        long long n = pl[0];
        MemItem *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        if (A->half != B->half || A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(A, 0, n);
        RANGE(B, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_div(s, A->dt(), (size_t)n, A->ptr, B->ptr, Y->ptr));
        m_mem.touch((long)pl[3]);
        return 0;
    }
    case MCH_FN_ADD_SCALAR: {
        // f{alpha}, l{n,0,hY[,yOff]} (CudaDnn.cs:8010-8016, device.cu:2183-2201)
        NEED_F(1, 1);
        NEED_L(3, 4);
        long long n = pl[0], yo = ll > 3 ? pl[3] : 0;
        MemItem* Y;
        ERRCHK(mem((long)pl[2], &Y));
        RANGE(Y, yo, n);
        HIPCHK(k_add_scalar(s, Y->dt(), (size_t)n, pf[0], PTR(Y, yo)));
        m_mem.touch((long)pl[2]);
        return 0;
    }
    case MCH_FN_POWX: {
        // f{alpha}, l{n,hA,0,hY[,aOff,yOff]} (CudaDnn.cs:8419-8425, device.cu:2595-2618)
        NEED_F(1, 1);
        NEED_L(4, 6);
        long long n = pl[0], ao = ll > 4 ? pl[4] : 0, yo = ll > 5 ? pl[5] : 0;
        MemItem *A, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[3], &Y));
        if (A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(A, ao, n);
        RANGE(Y, yo, n);
        HIPCHK(k_powx(s, A->dt(), (size_t)n, PTR(A, ao), pf[0], PTR(Y, yo)));
        m_mem.touch((long)pl[3]);
        return 0;
    }
    case MCH_FN_SQRT: {
        // [f{epsilon}], l{n,hX,hY}: y = sqrt(x + epsilon) (CudaDnn.cs:8520-8526, device.cu:2712-2728)
        NEED_L(3, 3);
        long long n = pl[0];
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_sqrt(s, X->dt(), (size_t)n, X->ptr, Y->ptr, (lf > 0 && pf) ? pf[0] : 0.f));
        m_mem.touch((long)pl[2]);
        return 0;
    }
    case MCH_FN_INVERT: {
        // [f{numerator, denominator}], l{n,hX,hY[,xOff,yOff]} (CudaDnn.cs:8453-8459, device.cu:2624-2655)
        NEED_L(3, 5);
        long long n = pl[0], xo = ll > 3 ? pl[3] : 0, yo = ll > 4 ? pl[4] : 0;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, xo, n);
        RANGE(Y, yo, n);
        HIPCHK(k_invert(s, X->dt(), (size_t)n, PTR(X, xo), PTR(Y, yo), (lf > 0 && pf) ? pf[0] : 1.f, (lf > 1 && pf) ? pf[1] : 1.f));
        m_mem.touch((long)pl[2]);
        return 0;
    }
    case MCH_FN_CHANNEL_MEAN: {
        // l{count,outer,channels,inner,hX,hY[,xOff]}: y[outer*channels] = row means (CudaDnn.cs:9030-9036, device.cu:3386-3405)
        NEED_L(6, 7);
        long long outer = pl[1], ch = pl[2], inner = pl[3], xo = ll > 6 ? pl[6] : 0;
        if (outer < 0 || ch < 0 || inner < 1 || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, xo, outer * ch * inner);
        RANGE(Y, 0, outer * ch);
        HIPCHK(k_channel_mean(s, X->dt(), (size_t)(outer * ch), (int)inner, PTR(X, xo), Y->ptr));
        m_mem.touch((long)pl[5]);
        return 0;
    }
    case MCH_FN_EXP:
    case MCH_FN_LOG: {
        // 235 [f{beta}] l{n,hA,hY[,aOff,yOff,0]}: y = exp(beta a) (device.cu:2531-2557, math.cu:5859-5865)
        // 236 [f{beta[,alpha]}] l{n,hA,hY[,0,0]}: y = log(beta (a + alpha)) (device.cu:2564-2590, math.cu:5923-5929)
        const bool isExp = fn == MCH_FN_EXP;
        ERRCHK(verify(lf, pf, 0, isExp ? 1 : 2));
        if (isExp) NEED_L(3, 6); else NEED_L(3, 5);
        const long long n = pl[0];
        long long aOff = isExp && ll > 3 ? pl[3] : 0, yOff = isExp && ll > 4 ? pl[4] : 0;
        if (n < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (aOff < 0) aOff = 0;
        if (yOff < 0) yOff = 0;
        const float beta = lf > 0 ? pf[0] : 1.f, alpha = !isExp && lf > 1 ? pf[1] : 0.f;
        MemItem *A, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &Y));
        if (A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(A, aOff, n);
        RANGE(Y, yOff, n);
        if (isExp) HIPCHK(k_exp(s, A->dt(), (size_t)n, PTR(A, aOff), PTR(Y, yOff), beta));
        else HIPCHK(k_log(s, A->dt(), (size_t)n, A->ptr, Y->ptr, beta, alpha));
        m_mem.touch((long)pl[2]);
        return 0;
    }
    case MCH_FN_CHANNEL_MAX: {
        // l{count,outer,channels,inner,hX,hY,returnIdx[,acrossChannels]} (device.cu:3359-3380, math.cu:6697-6810)
        NEED_L(7, 8);
        const long long outer = pl[1], ch = pl[2], inner = pl[3];
        const bool idx = pl[6] != 0, across = ll > 7 ? pl[7] != 0 : true;
        if (outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (X->ptr == Y->ptr) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        // within a channel the reference's kernel walks outer * inner rows of `inner` values
        RANGE(X, 0, across ? outer * ch * inner : outer * inner * inner);
        RANGE(Y, 0, outer * inner);
        HIPCHK(k_channel_max(s, X->dt(), (size_t)outer, (int)ch, (int)inner, X->ptr, Y->ptr, idx, across));
        m_mem.touch((long)pl[5]);
        return 0;
    }
    case MCH_FN_CHANNEL_SUB:
    case MCH_FN_CHANNEL_DIV: {
        // 291 l{count,outer,channels,inner,hX,hY[,hA]}: y[n,c,s] = a[n,c,s] - x[n,s], a = y when absent (device.cu:3438-3457)
        // 293 l{count,outer,channels,inner,hX,hY[,method]}: y[n,c,s] /= x[n,s]; method 2 is the same division walked
        //     from the (n, s) side with count = outer * inner (device.cu:3541-3560, math.cu:7160-7204)
        NEED_L(6, 7);
        const bool sub = fn == MCH_FN_CHANNEL_SUB;
        long long count = pl[0];
        const long long outer = pl[1], ch = pl[2], inner = pl[3];
        if (count < 0 || outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (!sub && ll > 6 && pl[6] == 2) {
            // the reference's second kernel divides all channels of the first `count` (n, s) pairs; that is the first
            // kernel's element set only for the full count, the one the layers pass - a partial count is refused
            if (count != outer * inner) {
                last_detail = "channel_div method 2 takes count = outer * inner only";
                return MCH_ERROR_PARAM_OUT_OF_RANGE;
            }
            count *= ch;
        }
        if (count > outer * ch * inner) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y, *A = nullptr;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (sub && ll > 6) ERRCHK(mem((long)pl[6], &A));
        if (X->half != Y->half || (A && A->half != Y->half)) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, outer * inner);
        RANGE(Y, 0, count);
        if (A) RANGE(A, 0, count);
        if (sub) HIPCHK(k_channel_sub(s, Y->dt(), (size_t)count, (int)ch, (int)inner, A ? A->ptr : Y->ptr, X->ptr, Y->ptr));
        else HIPCHK(k_channel_div(s, Y->dt(), (size_t)count, (int)ch, (int)inner, X->ptr, Y->ptr));
        m_mem.touch((long)pl[5]);
        return 0;
    }
    case MCH_FN_CHANNEL_DOT: {
        // l{count,outer,channels,inner,hX,hA,hY}: y[n,s] = sum_c x[n,c,s] a[n,c,s] (device.cu:3638-3654, math.cu:7335-7351)
        NEED_L(7, 7);
        const long long outer = pl[1], ch = pl[2], inner = pl[3];
        if (outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *A, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &A));
        ERRCHK(mem((long)pl[6], &Y));
        if (X->half != A->half || X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (Y->ptr == X->ptr || Y->ptr == A->ptr) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, outer * ch * inner);
        RANGE(A, 0, outer * ch * inner);
        RANGE(Y, 0, outer * inner);
        HIPCHK(k_channel_dot(s, X->dt(), (size_t)outer, (int)ch, (int)inner, X->ptr, A->ptr, Y->ptr));
        m_mem.touch((long)pl[6]);
        return 0;
    }
    case MCH_FN_CHANNEL_SUM:
    case MCH_FN_CHANNEL_SUM2: {
        // 292 l{count,outer,channels,inner,hX,hY}: y[outer,inner] = sum over the channels (CudaDnn.cs:9182-9188,
        //     device.cu:3488-3503, math.cu:6945-6961)
        // 309 l{count,outer,channels,inner,hX,hY,acrossChannels[,dir,channelsY]} (CudaDnn.cs:9205-9211, device.cu:3510-3534,
        //     math.cu:7076-7114): forward sums across the channels (as 292) or within every channel (y[outer,channels] = row
        //     sums); backward writes X from Y, every Y value spread over what it was summed from.
        const bool two = fn == MCH_FN_CHANNEL_SUM2;
        if (two) NEED_L(7, 9); else NEED_L(6, 6);
        long long outer = pl[1], ch = pl[2], inner = pl[3];
        const bool across = two ? pl[6] != 0 : true;
        const int dir = two && ll > 7 ? (int)pl[7] : 0;
        const long long chY = two && ll > 8 ? pl[8] : -1;
        if (outer < 0 || ch < 1 || inner < 1 || ch > INT_MAX || inner > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (!two && outer > 1 && (long long)Y->count < outer * inner && (long long)Y->count >= inner) {
            // RMSNormLayer.cs:198-199 passes its weight gradient (inner values) as Y with outer = batch: the reference
            // writes the sums of every batch entry, the later ones past the end of Y.  Only what Y holds is computed.
            outer = (long long)Y->count / inner;
        }
        const long long full = outer * ch * inner, reduced = across ? outer * inner : outer * ch;
        RANGE(X, 0, full);
        RANGE(Y, 0, reduced);
        if (dir == 0) {
            if (X->ptr == Y->ptr) return MCH_ERROR_PARAM_OUT_OF_RANGE;
            // one tensor of many channels and few columns (a norm layer's weight gradient: 8192 rows of 768): the rows are
            // dealt over workgroups as for a transposed mat-vec, partial sums added in a fixed order
            const size_t wsb = (!X->half && outer == 1 && (inner + 63) / 64 < 256) ? k_gemv_workspace_bytes(true, (int)ch, (int)inner) : 0;
            if (across && wsb) {
                void* ws;
                ERRCHK(workspace(wsb, &ws));
                HIPCHK(k_gemv(s, F32, true, (int)ch, (int)inner, 1.f, X->ptr, nullptr, 0.f, (float*)Y->ptr, ws, wsb));
            } else if (across) HIPCHK(k_channel_colsum(s, X->dt(), (size_t)outer, (int)ch, (int)inner, X->ptr, Y->ptr));
            else HIPCHK(k_channel_rowsum(s, X->dt(), (size_t)(outer * ch), (int)inner, X->ptr, Y->ptr, 1.0f));
            m_mem.touch((long)pl[5]);
            return 0;
        }
        if (chY == 1 && chY != ch) {
            // the reference's second pair of backward kernels (math.cu:7017-7052) reads Y with an index that runs past
            // outer * inner for the within-channel form; neither is used by the layers of this path
            last_detail = "channel_sum backward with channelsY = 1 is not supported";
            return MCH_ERROR_NOT_IMPLEMENTED;
        }
        if (across) HIPCHK(k_channel_spread(s, X->dt(), 3, (size_t)full, 1, (size_t)(ch * inner), (size_t)inner, Y->ptr, X->ptr));
        else HIPCHK(k_channel_spread(s, X->dt(), 0, (size_t)full, (size_t)inner, 1, 1, Y->ptr, X->ptr));
        m_mem.touch((long)pl[4]);
        return 0;
    }
    case MCH_FN_CHANNEL_FILLFROM:
    case MCH_FN_CHANNEL_COPYALL:
    case MCH_FN_CHANNEL_DUP: {
        // l{count,outer,channels,inner,hX,hY[,dir]} (CudaDnn.cs:9086-9092, 9443-9449, 9312-9318; math.cu:7465-7481, 7630-7639, 7667-7676)
        const bool fill = fn == MCH_FN_CHANNEL_FILLFROM;
        NEED_L(fill ? 7 : 6, fill ? 7 : 6);
        long long n = pl[0], outer = pl[1], ch = pl[2], inner = pl[3];
        if (n < 0 || outer < 1 || ch < 1 || inner < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (fill && pl[6] != 0) {
            // backward: x[i] = y[i * inner], i < outer * channels
            RANGE(X, 0, outer * ch);
            RANGE(Y, 0, (outer * ch - 1) * inner + 1);
            HIPCHK(k_channel_spread(s, X->dt(), 1, (size_t)(outer * ch), (size_t)inner, 1, 1, X->ptr, Y->ptr));
            m_mem.touch((long)pl[4]);
            return 0;
        }
        RANGE(Y, 0, n);
        if (fill) {
            RANGE(X, 0, n > 0 ? (n - 1) / inner + 1 : 0);
            HIPCHK(k_channel_spread(s, X->dt(), 0, (size_t)n, (size_t)inner, 1, 1, X->ptr, Y->ptr));
        } else if (fn == MCH_FN_CHANNEL_COPYALL) {
            RANGE(X, 0, n < ch * inner ? n : ch * inner);
            HIPCHK(k_channel_spread(s, X->dt(), 2, (size_t)n, 1, (size_t)(ch * inner), 1, X->ptr, Y->ptr));
        } else {
            RANGE(X, 0, n > 0 ? ((n - 1) / (ch * inner)) * ch + ch : 0);
            HIPCHK(k_channel_spread(s, X->dt(), 3, (size_t)n, 1, (size_t)(ch * inner), (size_t)ch, X->ptr, Y->ptr));
        }
        m_mem.touch((long)pl[5]);
        return 0;
    }

    case MCH_FN_MASK: {
        // f{search,replace}, l{n,maskDim,0,0,hX,hMask,hY} (device.cu:2101-2120)
        NEED_F(2, 2);
        NEED_L(7, 7);
        long long n = pl[0];
        int md = (int)pl[1];
        if (md < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *M, *Y;
        float xscale = 1.f;
        ERRCHK(mask_operands((long)pl[4], (long)pl[5], (long)pl[6], n, &X, &M, &Y, &xscale));
        if (X->half != M->half || X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        RANGE(M, 0, md);
        if (defer_mask((long)pl[4], (long)pl[5], (long)pl[6], X, M, n, md, 0, pf[0], pf[1], xscale, timing)) {
            m_mem.touch((long)pl[6]);
            return 0;
        }
        if (m_pendingProduct.hC == (long)pl[4]) ERRCHK(flush_pending_product());
        HIPCHK(k_mask(s, X->dt(), (size_t)n, md, pf[0], pf[1], X->ptr, M->ptr, Y->ptr, xscale));
        if (xscale != 1.f) X->pending = 1.f;
        m_mem.touch((long)pl[6]);
        return 0;
    }

    case MCH_FN_MASK_BATCH: {
        // f{search,replace}, l{n,batch,maskDim,0,0,hX,hMask,hY} (device.cu:2125-2145)
        NEED_F(2, 2);
        NEED_L(8, 8);
        long long n = pl[0];
        int batch = (int)pl[1], md = (int)pl[2];
        if (batch < 1 || md < batch || n < batch) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *M, *Y;
        float xscale = 1.f;
        ERRCHK(mask_operands((long)pl[5], (long)pl[6], (long)pl[7], n, &X, &M, &Y, &xscale));
        if (X->half != M->half || X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        // largest mask index = (md/batch - 1) + ((n-1)/(n/batch)) * (md/batch)
        {
            long long md1 = md / batch, dd1 = n / batch;
            RANGE(M, 0, (md1 - 1) + ((n - 1) / dd1) * md1 + 1);
        }
        if (n % batch == 0 && md % batch == 0 &&
            defer_mask((long)pl[5], (long)pl[6], (long)pl[7], X, M, n, md, batch, pf[0], pf[1], xscale, timing)) {
            m_mem.touch((long)pl[7]);
            return 0;
        }
        if (m_pendingProduct.hC == (long)pl[5]) ERRCHK(flush_pending_product());
        HIPCHK(k_mask_batch(s, X->dt(), (size_t)n, batch, md, pf[0], pf[1], X->ptr, M->ptr, Y->ptr, xscale));
        if (xscale != 1.f) X->pending = 1.f;
        m_mem.touch((long)pl[7]);
        return 0;
    }

    case MCH_FN_TRANSPOSE: {
        // l{n,hX,hY,hXCounts,hYCounts,hMapping,numAxes,hBuffer} (device.cu:3088-3107)
        NEED_L(8, 8);
        long long n = pl[0];
        int axes = (int)pl[6];
        MemItem *X, *Y, *XC, *YC, *MP;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        ERRCHK(mem((long)pl[3], &XC));
        ERRCHK(mem((long)pl[4], &YC));
        ERRCHK(mem((long)pl[5], &MP));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (XC->half || YC->half || MP->half) return MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED;
        if (axes < 1 || axes > 8) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        RANGE(XC, 0, axes);
        RANGE(YC, 0, axes);
        RANGE(MP, 0, axes);
        {
            // the stride / map blobs sit on the device; reading them costs a round trip, so the decoded form is kept per
            // (handles, content versions) - a layer passes the same three blobs on every call
            const uint64_t key[6] = {(uint64_t)pl[3], (uint64_t)pl[4], (uint64_t)pl[5], m_mem.version((long)pl[3]),
                                     m_mem.version((long)pl[4]), m_mem.version((long)pl[5])};
            const PermuteArgs* pa = nullptr;
            for (const PermuteCacheEntry& e : m_permuteCache)
                if (e.axes == axes && memcmp(e.key, key, sizeof(key)) == 0) { pa = &e.args; break; }
            if (!pa) {
                PermuteCacheEntry e;
                memcpy(e.key, key, sizeof(key));
                e.axes = axes;
                HIPCHK(k_transpose_fetch(s, (const float*)XC->ptr, (const float*)YC->ptr, (const float*)MP->ptr, axes, &e.args));
                if (m_permuteCache.size() >= 64) m_permuteCache.erase(m_permuteCache.begin());
                m_permuteCache.push_back(e);
                pa = &m_permuteCache.back().args;
            }
            HIPCHK(k_transpose_run(s, X->dt(), (size_t)n, X->ptr, Y->ptr, *pa));
        }
        m_mem.touch((long)pl[2]);
        return 0;
    }

    case MCH_FN_TRANSPOSE_HW: {
        // l{n,c,h,w,hSrc,hDst} (device.cu:3110-3127)
        NEED_L(6, 6);
        long long nn = pl[0], c = pl[1], h = pl[2], w = pl[3];
        if (nn < 0 || c < 0 || h < 0 || w < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, nn * c * h * w);
        RANGE(Y, 0, nn * c * h * w);
        HIPCHK(k_transpose_hw(s, X->dt(), (int)(nn * c), (int)h, (int)w, X->ptr, Y->ptr));
        m_mem.touch((long)pl[5]);
        return 0;
    }

    case MCH_FN_CHANNEL_COPY: {
        // l{count,outer,channels,blocks,inner,offset,hX,hY,dir} (device.cu:3730-3748)
        NEED_L(9, 9);
        long long n = pl[0], chn = pl[2], blocks = pl[3], inner = pl[4], off = pl[5];
        int dir = (int)pl[8];
        if (n < 0 || chn < 1 || blocks < 1 || inner < 1 || off < 0 || off >= blocks) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[6], &X));
        ERRCHK(mem((long)pl[7], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(Y, 0, n);
        if (n > 0) {
            long long last = n - 1;
            long long xi = ((last / (chn * inner)) * chn + (last % (chn * inner)) / inner) * blocks * inner + off * inner + last % inner;
            // the last element has the largest n and c, so together with inner-1 this bounds every index
            RANGE(X, 0, xi + (inner - 1 - last % inner) + 1);
        }
        HIPCHK(k_channel_copy(s, X->dt(), (size_t)n, (int)chn, (int)blocks, (int)inner, (int)off, X->ptr, Y->ptr, dir));
        m_mem.touch(dir == 0 ? (long)pl[7] : (long)pl[6]);
        return 0;
    }

    case MCH_FN_EMBED_FWD: {
        // l{count,hBtm,hWeight,M,N,K,hTop} (CudaDnn.cs:9751; math.cu:9314-9330)
        NEED_L(7, 7);
        long long n = pl[0], N = pl[4], K = pl[5];
        if (n < 0 || N < 1 || K < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *I, *W, *T;
        ERRCHK(mem((long)pl[1], &I));
        ERRCHK(mem((long)pl[2], &W));
        ERRCHK(mem((long)pl[6], &T));
        if (I->half) return MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED;
        if (W->half != T->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(T, 0, n);
        RANGE(I, 0, (n + N - 1) / N);
        RANGE(W, 0, K * N);
        HIPCHK(k_embed(s, W->dt(), (size_t)n, (const float*)I->ptr, W->ptr, (int)N, T->ptr));
        m_mem.touch((long)pl[6]);
        return 0;
    }

    case MCH_FN_SILU_FWD: {
        // l{count,hBtm,hTop} (CudaDnn.cs:10152)
        NEED_L(3, 3);
        long long n = pl[0];
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_silu(s, X->dt(), (size_t)n, X->ptr, Y->ptr));
        m_mem.touch((long)pl[2]);
        return 0;
    }

    case MCH_FN_SILU_BWD:
    case MCH_FN_GELU_BWD: {
        // l{count,hTopDiff,hTopData,hBtmDiff,hBtmData[,bert]} (CudaDnn.cs:10132-10180, device.h:3269-3316)
        const bool gelu = fn == MCH_FN_GELU_BWD;
        NEED_L(gelu ? 6 : 5, gelu ? 6 : 5);
        long long n = pl[0];
        MemItem *dY, *dX, *X;
        ERRCHK(mem((long)pl[1], &dY));
        ERRCHK(mem((long)pl[3], &dX));
        ERRCHK(mem((long)pl[4], &X));
        if (dY->half != dX->half || X->half != dX->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(dY, 0, n);
        RANGE(dX, 0, n);
        RANGE(X, 0, n);
        if (gelu) HIPCHK(k_gelu_bwd(s, X->dt(), (size_t)n, dY->ptr, X->ptr, dX->ptr, pl[5] != 0));
        else HIPCHK(k_silu_bwd(s, X->dt(), (size_t)n, dY->ptr, X->ptr, dX->ptr));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_RELU_FWD: {
        // f{negativeSlope}, l{count,hBtm,hTop,0} (CudaDnn.cs:10417-10423, device.h:4925-4940)
        NEED_F(1, 1);
        NEED_L(4, 4);
        long long n = pl[0];
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_relu_fwd(s, X->dt(), (size_t)n, X->ptr, Y->ptr, pf[0]));
        m_mem.touch((long)pl[2]);
        return 0;
    }
    case MCH_FN_RELU_BWD: {
        // f{negativeSlope}, l{count,hTopDiff,hTopData,hBtmDiff,0} (CudaDnn.cs:10438-10444, device.h:4943-4959)
        NEED_F(1, 1);
        NEED_L(5, 5);
        long long n = pl[0];
        MemItem *dY, *Y, *dX;
        ERRCHK(mem((long)pl[1], &dY));
        ERRCHK(mem((long)pl[2], &Y));
        ERRCHK(mem((long)pl[3], &dX));
        if (dY->half != Y->half || dX->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(dY, 0, n);
        RANGE(Y, 0, n);
        RANGE(dX, 0, n);
        HIPCHK(k_relu_bwd(s, Y->dt(), (size_t)n, dY->ptr, Y->ptr, dX->ptr, pf[0]));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_GELU_FWD: {
        // l{count,hBtm,hTop,bert} (CudaDnn.cs:10098-10104, device.h:3253-3266)
        NEED_L(4, 4);
        long long n = pl[0];
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_gelu_fwd(s, X->dt(), (size_t)n, X->ptr, Y->ptr, pl[3] != 0));
        m_mem.touch((long)pl[2]);
        return 0;
    }

    case MCH_FN_CREATE_LAYERNORM: {
        // f{eps}, l{gpuId,count,outer,channels,inner} (CudaDnn.cs:6307-6319, device.h:4123-4147)
        NEED_F(1, 1);
        NEED_L(5, 5);
        long long count = pl[1], outer = pl[2], channels = pl[3], inner = pl[4];
        if (outer < 1 || channels < 1 || inner < 1 || count > INT_MAX || outer * channels > INT_MAX ||
            count != outer * channels * inner)
            return MCH_ERROR_PARAM_OUT_OF_RANGE;   // layernorm.cu:141-142
        long h;
        ERRCHK(m_layernorm.create(&h));
        LayerNormState* ln = m_layernorm.get(h);
        ln->count = (int)count; ln->outer = (int)outer; ln->channels = (int)channels; ln->inner = (int)inner;
        ln->eps = pf[0];
        hipError_t e = hipMalloc((void**)&ln->stdev, (size_t)(outer * channels) * sizeof(float));
        if (e != hipSuccess) {
            ln->stdev = nullptr;
            m_layernorm.free(h);
            return (long)e;
        }
        ln->set = true;
        return set_out((float)h, ppOut, plOut);
    }
    case MCH_FN_FREE_LAYERNORM:
        NEED_F(1, 1);
        HIPCHK(hipStreamSynchronize(s));
        return m_layernorm.free((long)pf[0]);
    case MCH_FN_LAYERNORM_FWD: {
        // l{hLayerNorm,hX,hY} (CudaDnn.cs:6339-6345, layernorm.cu:219-262)
        NEED_L(3, 3);
        LayerNormState* ln = m_layernorm.get((long)pl[0]);
        if (!ln || !ln->set) return MCH_ERROR_LAYERNORM_NOT_INITIALIZED;
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[1], &X));
        ERRCHK(mem((long)pl[2], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, ln->count);
        RANGE(Y, 0, ln->count);
        HIPCHK(k_layernorm_fwd(s, X->dt(), ln->outer * ln->channels, ln->inner, X->ptr, Y->ptr, ln->stdev, ln->eps));
        ln->backwards = 0;
        m_mem.touch((long)pl[2]);
        return 0;
    }
    case MCH_FN_LAYERNORM_BWD: {
        // l{hLayerNorm,hYdata,hYdiff,hXdiff} (CudaDnn.cs:6354-6360, layernorm.cu:268-312)
        NEED_L(4, 4);
        LayerNormState* ln = m_layernorm.get((long)pl[0]);
        if (!ln || !ln->set) return MCH_ERROR_LAYERNORM_NOT_INITIALIZED;
        MemItem *Y, *dY, *dX;
        ERRCHK(mem((long)pl[1], &Y));
        ERRCHK(mem((long)pl[2], &dY));
        ERRCHK(mem((long)pl[3], &dX));
        if (Y->half != dY->half || Y->half != dX->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(Y, 0, ln->count);
        RANGE(dY, 0, ln->count);
        RANGE(dX, 0, ln->count);
        ln->backwards++;
        HIPCHK(k_layernorm_bwd(s, Y->dt(), ln->outer * ln->channels, ln->inner, Y->ptr, dY->ptr, dX->ptr, ln->stdev,
                               ln->eps * (float)ln->backwards));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_SWIGLU_FWD: {
        NEED_L(4, 4);
        long long n = pl[0];
        MemItem *A, *B, *Y;
        ERRCHK(mem((long)pl[1], &A));
        ERRCHK(mem((long)pl[2], &B));
        ERRCHK(mem((long)pl[3], &Y));
        if (A->half != B->half || A->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(A, 0, n);
        RANGE(B, 0, n);
        RANGE(Y, 0, n);
        HIPCHK(k_swiglu(s, A->dt(), (size_t)n, A->ptr, B->ptr, Y->ptr));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_RMSNORM_FWD: {
        NEED_F(1, 1);
        NEED_L(5, 5);
        long long outer = pl[0], dim = pl[1];
        if (outer < 0 || dim < 1 || outer > INT_MAX || dim > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *W = nullptr, *Y;
        ERRCHK(mem((long)pl[2], &X));
        if (pl[3]) ERRCHK(mem((long)pl[3], &W));
        ERRCHK(mem((long)pl[4], &Y));
        if (X->half != Y->half || (W && W->half != X->half)) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, outer * dim);
        RANGE(Y, 0, outer * dim);
        if (W) RANGE(W, 0, dim);
        HIPCHK(k_rmsnorm(s, X->dt(), (int)outer, (int)dim, X->ptr, W ? W->ptr : nullptr, Y->ptr, pf[0]));
        m_mem.touch((long)pl[4]);
        return 0;
    }

    // ---- cuDNN-shaped handles: opaque records here ---------------------------
    case MCH_FN_CREATE_CUDNN: {
        // f{[stream]} (device.h:1201-1221)
        ERRCHK(verify(lf, pf, 0, 1));
        long h;
        ERRCHK(m_cudnn.create(&h));
        return set_out((float)h, ppOut, plOut);
    }
    case MCH_FN_FREE_CUDNN:
        NEED_F(1, 1);
        return m_cudnn.free((long)pf[0]);
    case MCH_FN_CREATE_TENSORDESC: {
        long h;
        ERRCHK(m_tdesc.create(&h));
        return set_out((float)h, ppOut, plOut);
    }
    case MCH_FN_FREE_TENSORDESC:
        NEED_F(1, 1);
        return m_tdesc.free((long)pf[0]);
    case MCH_FN_SET_TENSORDESC: {
        // l{h,half,n,c,h,w[,sn,sc,sh,sw]} (device.cu:1426-1464)
        NEED_L(6, 10);
        if (ll != 6 && ll != 10) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        TensorDesc* d = m_tdesc.get((long)pl[0]);
        if (!d) return MCH_ERROR_PARAM_NULL;
        d->half = pl[1] == 1;
        d->n = (int)pl[2]; d->c = (int)pl[3]; d->h = (int)pl[4]; d->w = (int)pl[5];
        if (ll == 6) { d->sw = 1; d->sh = d->w; d->sc = d->h * d->sh; d->sn = d->c * d->sc; }
        else { d->sn = (int)pl[6]; d->sc = (int)pl[7]; d->sh = (int)pl[8]; d->sw = (int)pl[9]; }
        return 0;
    }

    case MCH_FN_SOFTMAX_FWD: {
        // f{alpha,beta}, l{hCudnn,0,hBtmDesc,hBtm,0,hTopDesc,hTop,alg,mode} (device.h:4778-4798)
        NEED_F(2, 2);
        NEED_L(9, 9);
        if (!m_cudnn.get((long)pl[0])) return MCH_ERROR_PARAM_NULL;
        TensorDesc* bd = m_tdesc.get((long)pl[2]);
        TensorDesc* td = m_tdesc.get((long)pl[5]);
        if (!bd || !td) return MCH_ERROR_PARAM_NULL;
        if (pf[0] != 1.f || pf[1] != 0.f) { last_detail = "softmax supports alpha=1, beta=0 only"; return MCH_ERROR_NOT_IMPLEMENTED; }
        int alg = (int)pl[7], mode = (int)pl[8];  // alg 0 fast, 1 accurate, 2 log; mode 0 instance, 1 channel
        if (alg < 0 || alg > 2 || mode < 0 || mode > 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (bd->n != td->n || bd->c != td->c || bd->h != td->h || bd->w != td->w) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        bool packed = bd->sw == 1 && bd->sh == bd->w && bd->sc == bd->h * bd->w && bd->sn == bd->c * bd->h * bd->w &&
                      td->sw == 1 && td->sh == td->w && td->sc == td->h * td->w && td->sn == td->c * td->h * td->w;
        if (!packed) { last_detail = "softmax needs fully packed NCHW descriptors"; return MCH_ERROR_NOT_IMPLEMENTED; }
        MemItem *X, *Y;
        long long total = (long long)bd->n * bd->c * bd->h * bd->w;
        size_t outer = bd->n;
        int len = mode == 0 ? bd->c * bd->h * bd->w : bd->c;
        int inner = mode == 0 ? 1 : bd->h * bd->w;
        if (m_pendingMask.hX == (long)pl[3] && (long)pl[6] != (long)pl[3] && (long)pl[6] != m_pendingMask.hM && inner == 1 &&
            total == m_pendingMask.n) {
            // the bottom's mask call is still outstanding: mask, scale and softmax in one pass; the bottom stays as it is
            // (masked only on record) until something else needs it
            MemItem* M;
            ERRCHK(mem((long)pl[6], &Y));
            if (m_pendingMask.hX == (long)pl[3] && !mem_lazy((long)pl[3], &X) && !mem_lazy(m_pendingMask.hM, &M) && X->half == Y->half &&
                (size_t)total <= Y->count) {
                const PendingMask& p = m_pendingMask;
                const size_t md1 = p.batch ? (size_t)(p.md / p.batch) : (size_t)p.md, dd1 = p.batch ? (size_t)(p.n / p.batch) : (size_t)p.n;
                // a (len,len) lower-triangle mask with search == 0 is not read at all, and neither are the scores above the diagonal
                const bool causal = p.batch == 0 && !X->half && p.search == 0.f && md1 == (size_t)len * len && dd1 % md1 == 0 &&
                                    held_mask_is_causal(p.hM, M, len);
                // the scores themselves may still be a held-back product: under the causal mask only the tiles that touch
                // the lower triangle are computed (the pass below reads nothing else, and the mask call, whenever it is
                // applied to the tensor, overwrites the rest)
                if (m_pendingProduct.hC == (long)pl[3])
                    ERRCHK(flush_pending_product(causal && m_pendingProduct.kind == 0 && m_pendingProduct.m == len && (long long)m_pendingProduct.batch * len == (long long)outer));
                // a causal pass over fp32 probabilities leaves word of whether every masked entry came out as an exact zero
                const bool tag = causal && alg != 2 && !Y->view && !Y->exposed;
                if (tag && !m_zeroFlag) {
                    HIPCHK(hipMalloc((void**)&m_zeroFlag, sizeof(int)));
                    HIPCHK(hipMemsetAsync(m_zeroFlag, 0, sizeof(int), s));
                }
                m_zeroHandle = 0;
                if (tag) m_zeroEpoch = m_zeroEpoch == INT_MAX ? 1 : m_zeroEpoch + 1;
                hipError_t e = k_softmax_masked(s, X->dt(), X->ptr, Y->ptr, outer, len, alg == 2, M->ptr, md1, dd1, p.search, p.replace, p.xscale, causal,
                                                tag ? m_zeroFlag : nullptr, m_zeroEpoch);
                if (e == hipSuccess) {
                    m_mem.touch((long)pl[6]);
                    if (tag) { m_zeroHandle = (long)pl[6]; m_zeroVersion = m_mem.version((long)pl[6]); m_zeroLen = len; m_zeroRows = outer; }
                    return 0;
                }
                if (e != hipErrorNotSupported) return (long)e;
            }
        }
        ERRCHK(mem((long)pl[3], &X));
        ERRCHK(mem((long)pl[6], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, total);
        RANGE(Y, 0, total);
        HIPCHK(k_softmax(s, X->dt(), X->ptr, Y->ptr, outer, len, inner, alg == 2));
        m_mem.touch((long)pl[6]);
        return 0;
    }

    case MCH_FN_SOFTMAX_BWD: {
        // f{alpha,beta}, l{hCudnn,0,hTopDataDesc,hTopData,hTopDiffDesc,hTopDiff,0,hBtmDiffDesc,hBtmDiff,alg,mode}
        // (CudaDnn.cs:4941-4947, device.h:4801-4823)
        NEED_F(2, 2);
        NEED_L(11, 11);
        if (!m_cudnn.get((long)pl[0])) return MCH_ERROR_PARAM_NULL;
        TensorDesc* yd = m_tdesc.get((long)pl[2]);
        TensorDesc* gd = m_tdesc.get((long)pl[4]);
        TensorDesc* bd = m_tdesc.get((long)pl[7]);
        if (!yd || !gd || !bd) return MCH_ERROR_PARAM_NULL;
        if (pf[0] != 1.f || pf[1] != 0.f) { last_detail = "softmax supports alpha=1, beta=0 only"; return MCH_ERROR_NOT_IMPLEMENTED; }
        int alg = (int)pl[9], mode = (int)pl[10];
        if (alg < 0 || alg > 2 || mode < 0 || mode > 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        for (TensorDesc* d : {gd, bd}) {
            if (d->n != yd->n || d->c != yd->c || d->h != yd->h || d->w != yd->w) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        for (TensorDesc* d : {yd, gd, bd}) {
            if (!(d->sw == 1 && d->sh == d->w && d->sc == d->h * d->w && d->sn == d->c * d->h * d->w)) {
                last_detail = "softmax needs fully packed NCHW descriptors";
                return MCH_ERROR_NOT_IMPLEMENTED;
            }
        }
        MemItem *Y, *G, *X;
        long long total = (long long)yd->n * yd->c * yd->h * yd->w;
        ERRCHK(mem((long)pl[3], &Y));
        ERRCHK(mem((long)pl[5], &G));
        if (pl[8] != pl[3] && pl[8] != pl[5]) ERRCHK(mem_overwritten((long)pl[8], &X, total));
        else ERRCHK(mem((long)pl[8], &X));
        if (Y->half != G->half || Y->half != X->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(Y, 0, total);
        RANGE(G, 0, total);
        RANGE(X, 0, total);
        size_t outer = yd->n;
        int len = mode == 0 ? yd->c * yd->h * yd->w : yd->c;
        int inner = mode == 0 ? 1 : yd->h * yd->w;
        HIPCHK(k_softmax_bwd(s, Y->dt(), Y->ptr, G->ptr, X->ptr, outer, len, inner, alg == 2));
        m_mem.touch((long)pl[8]);
        return 0;
    }

    // ---- attention -------------------------------------------------------------
    case MCH_FN_ATTN_CREATE: {
        long h;
        ERRCHK(m_attn.create(&h));
        return set_out((float)h, ppOut, plOut);
    }
    case MCH_FN_ATTN_FREE:
        NEED_F(1, 1);
        return m_attn.free((long)pf[0]);
    case MCH_FN_ATTN_SET: {
        // f{dropout}, l{hCudnn,hAttn,gpuId,training,batch,blockSize,heads,hs,seed} (device.h:2463-2485)
        NEED_L(9, 9);
        NEED_F(1, 1);
        AttnState* st = m_attn.get((long)pl[1]);
        if (!st) return MCH_ERROR_ATTN_NOT_INITIALIZED;
        if (pl[4] < 1 || pl[5] < 1 || pl[6] < 1 || pl[7] < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        st->training = pl[3] != 0;
        st->batch = (int)pl[4]; st->block = (int)pl[5]; st->heads = (int)pl[6]; st->hs = (int)pl[7];
        st->dropout = pf[0];
        if (!(st->dropout >= 0.f) || st->dropout >= 1.f) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        st->seed = (uint64_t)pl[8];
        st->fwdCalls = 0;
        st->scale = (float)(1.0 / sqrt((double)st->hs));  // attn.cu:427
        st->set = true;
        st->maskHandle = 0;
        st->lseValid = false;
        st->lastTq = st->lastTk = 0;
        st->lastMask = 0;
        return 0;
    }
    case MCH_FN_ATTN_FWD: {
        // l{hCudnn,hAttn,blockSize,hQ,hK,hV,hMask,hY,batchMask[,blockSizeK[,mergedY]]} (device.h:2488-2506, attn.cu:518-602)
        // The optional 10th value (key length when it differs from the query length) and 11th (1: Y is written
        // head-merged, (B,T,H,hs), ready for the output projection) have no counterpart in the reference, whose
        // handle needs T_q == T_k and always writes (B,H,T,hs).
        NEED_L(9, 11);
        const bool mergedY = ll > 10 && pl[10] != 0;
        AttnState* st = m_attn.get((long)pl[1]);
        if (!st || !st->set) return MCH_ERROR_ATTN_NOT_INITIALIZED;
        int T = (int)pl[2];
        int Tk = ll > 9 ? (int)pl[9] : T;
        if (T > st->block || Tk > st->block) return MCH_ERROR_ATTN_INVALID_BLOCK_SIZE;
        if (T < 1 || Tk < 1) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *Q, *K, *V, *Y, *M = nullptr;
        ERRCHK(mem((long)pl[3], &Q));
        ERRCHK(mem((long)pl[4], &K));
        ERRCHK(mem((long)pl[5], &V));
        ERRCHK(mem((long)pl[7], &Y));
        long hMask = (long)pl[6];
        // batchMask: 0 = (1,1,T,T), 1 = (B,T,1,1) as in the reference; 2 = (B,T,T) per-sequence mask (an
        // extension that lets MultiheadAttentionLayer keep its decoder mask on the fused route)
        const long long batchMask = pl[8];
        if (batchMask < 0 || batchMask > 2) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        if (hMask) ERRCHK(mem(hMask, &M));
        if (Q->half != K->half || Q->half != V->half || Q->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        long long qn = (long long)st->batch * st->heads * T * st->hs, kn = (long long)st->batch * st->heads * Tk * st->hs;
        if ((long long)Q->count < qn || (long long)Y->count < qn || (long long)K->count < kn || (long long)V->count < kn)
            return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
        MaskKind kind = MASK_NONE;
        if (M) {
            if (M->half) return MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED;
            if (batchMask == 2) {
                if ((long long)M->count < (long long)st->batch * T * Tk) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
                kind = MASK_BQK;
            } else if (batchMask == 1) {
                if ((long long)M->count < (long long)st->batch * Tk) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
                kind = MASK_KEY;
            } else {
                if ((long long)M->count < (long long)T * Tk) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
                kind = (T == Tk && mask_is_causal(st, hMask, M, T)) ? MASK_CAUSAL : MASK_QK;
            }
        }
        float* lse = nullptr;
        st->lseValid = false;
        if (st->training && mergedY) {
            last_detail = "the head-merged output layout is for inference: the backward pass reads Y as (B,H,T,hs)";
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        if (st->training) {
            // training mode: keep one number per query row for ATTN_BWD (the reference keeps the T x T probabilities)
            const size_t rows = (size_t)st->batch * st->heads * T;
            if (st->lseCap < rows) {
                if (st->lse) { HIPCHK(hipStreamSynchronize(s)); (void)hipFree(st->lse); st->lse = nullptr; st->lseCap = 0; }
                HIPCHK(hipMalloc((void**)&st->lse, rows * sizeof(float)));
                st->lseCap = rows;
            }
            lse = st->lse;
            const size_t ybytes = (size_t)qn * Y->esize();
            if (st->ysaveBytes < ybytes) {
                if (st->ysave) { HIPCHK(hipStreamSynchronize(s)); (void)hipFree(st->ysave); st->ysave = nullptr; st->ysaveBytes = 0; }
                HIPCHK(hipMalloc(&st->ysave, ybytes));
                st->ysaveBytes = ybytes;
            }
        }
        // training with a dropout ratio: a fresh mask per forward call (the reference's generator state advances with
        // every call), remembered for the backward call that follows
        const bool drop = st->training && st->dropout > 0.f;
        if (drop) {
            st->drop.seed = st->seed + 0xD1B54A32D192ED03ull * (uint64_t)(++st->fwdCalls);
            st->drop.threshold = (uint32_t)fmin((double)st->dropout * 4294967296.0, 4294967295.0);
            st->drop.keepScale = 1.0f / (1.0f - st->dropout);
        }
        HIPCHK(k_attn_prefill(s, Q->dt(), Q->ptr, K->ptr, V->ptr, Y->ptr, st->batch, st->heads, T, Tk, st->hs, st->scale,
                              M ? (const float*)M->ptr : nullptr, kind, lse, mergedY, drop ? &st->drop : nullptr));
        // the backward pass needs this output (dY . Y per row); the C# layer hands ATTN_BWD a Y buffer that holds the
        // head-merged layout by then (CausalSelfAttentionLayer.cs:668-672), so a copy stays with the handle
        if (lse) HIPCHK(hipMemcpyAsync(st->ysave, Y->ptr, (size_t)qn * Y->esize(), hipMemcpyDeviceToDevice, s));
        st->lseValid = lse != nullptr;
        st->lastTq = T; st->lastTk = Tk; st->lastBatchMask = batchMask; st->lastMask = hMask;
        m_mem.touch((long)pl[7]);
        return 0;
    }
    case MCH_FN_ATTN_BWD: {
        // l{hCudnn,hAttn,hQ,hdQ,hK,hdK,hV,hdV,hMask,hY,hdY} (CudaDnn.cs:5695-5701, device.h:2509-2529, attn.cu:608-661).
        // Sequence lengths, the mask and its layout are those of the handle's last forward call: the reference reads
        // the probabilities that call left behind and never looks at hMask here (CausalSelfAttentionLayer.cs:672 passes
        // 0), so the probabilities are recomputed under the forward call's mask.  Without a forward call the block
        // size given to ATTN_SET and the hMask argument are used.
        NEED_L(11, 11);
        AttnState* st = m_attn.get((long)pl[1]);
        if (!st || !st->set) return MCH_ERROR_ATTN_NOT_INITIALIZED;
        const bool drop = st->training && st->dropout > 0.f;
        if (drop && !st->lseValid) { last_detail = "ATTN_BWD with dropout needs the training-mode forward call whose mask it repeats"; return MCH_ERROR_ATTN_NOT_INITIALIZED; }
        const int T = st->lastTq > 0 ? st->lastTq : st->block, Tk = st->lastTq > 0 ? st->lastTk : st->block;
        const long long batchMask = st->lastTq > 0 ? st->lastBatchMask : 0;
        MemItem *Q, *dQ, *K, *dK, *V, *dV, *Y, *dY, *M = nullptr;
        ERRCHK(mem((long)pl[2], &Q));
        ERRCHK(mem((long)pl[3], &dQ));
        ERRCHK(mem((long)pl[4], &K));
        ERRCHK(mem((long)pl[5], &dK));
        ERRCHK(mem((long)pl[6], &V));
        ERRCHK(mem((long)pl[7], &dV));
        ERRCHK(mem((long)pl[9], &Y));
        ERRCHK(mem((long)pl[10], &dY));
        long hMask = st->lastTq > 0 ? st->lastMask : (long)pl[8];
        if (hMask) ERRCHK(mem(hMask, &M));
        for (MemItem* it : {dQ, K, dK, V, dV, Y, dY})
            if (it->half != Q->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        long long qn = (long long)st->batch * st->heads * T * st->hs, kn = (long long)st->batch * st->heads * Tk * st->hs;
        if ((long long)Q->count < qn || (long long)dQ->count < qn || (long long)Y->count < qn || (long long)dY->count < qn ||
            (long long)K->count < kn || (long long)dK->count < kn || (long long)V->count < kn || (long long)dV->count < kn)
            return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
        MaskKind kind = MASK_NONE;
        if (M) {
            if (M->half) return MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED;
            if (batchMask == 2) {
                if ((long long)M->count < (long long)st->batch * T * Tk) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
                kind = MASK_BQK;
            } else if (batchMask == 1) {
                if ((long long)M->count < (long long)st->batch * Tk) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
                kind = MASK_KEY;
            } else {
                if ((long long)M->count < (long long)T * Tk) return MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE;
                kind = (T == Tk && mask_is_causal(st, hMask, M, T)) ? MASK_CAUSAL : MASK_QK;
            }
        }
        void* ws;
        const size_t wsBytes = attn_backward_workspace_bytes(st->batch, st->heads, T);
        ERRCHK(workspace(wsBytes, &ws));
        const bool haveLse = st->lseValid && st->lseCap >= (size_t)st->batch * st->heads * T;
        const bool haveY = haveLse && st->ysave && st->ysaveBytes >= (size_t)qn * Y->esize();
        HIPCHK(k_attn_backward(s, Q->dt(), Q->ptr, K->ptr, V->ptr, haveY ? st->ysave : Y->ptr, dY->ptr, dQ->ptr, dK->ptr, dV->ptr, st->batch, st->heads,
                               T, Tk, st->hs, st->scale, M ? (const float*)M->ptr : nullptr, kind, haveLse ? st->lse : nullptr,
                               ws, wsBytes, drop ? &st->drop : nullptr));
        m_mem.touch((long)pl[3]);
        m_mem.touch((long)pl[5]);
        m_mem.touch((long)pl[7]);
        return 0;
    }

    case MCH_FN_ATTN_DECODE_FWD:
        return attn_decode_fwd(pf, lf, pl, ll, false);

    case MCH_FN_QKV_PROJ_HEADS: {
        // l{batch, T, heads, hs, hX, hW, hBias(0 = none), hQ, hK, hV}: [q|k|v] = X W^T + bias, X (batch*T, C), W (3C, C),
        // C = heads*hs, each third written as (batch, heads, T, hs).  An eleventh value, hRope != 0, also applies that
        // handle's rotation to q and k, as ROPE_FWD without an offset does to their (batch, T, heads, hs) form.
        NEED_L(10, 11);
        const long long B = pl[0], T = pl[1], H = pl[2], hs = pl[3];
        if (B < 1 || T < 1 || H < 1 || hs < 1 || B * T > INT_MAX || 3 * H * hs > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        const long long C = H * hs, M = B * T;
        MemItem *X, *W, *Bi = nullptr, *Q, *K, *V;
        ERRCHK(mem((long)pl[4], &X));
        ERRCHK(mem((long)pl[5], &W));
        if (pl[6]) ERRCHK(mem((long)pl[6], &Bi));
        ERRCHK(mem((long)pl[7], &Q));
        ERRCHK(mem((long)pl[8], &K));
        ERRCHK(mem((long)pl[9], &V));
        if (X->half != W->half || X->half != Q->half || X->half != K->half || X->half != V->half || (Bi && Bi->half != X->half))
            return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, M * C);
        RANGE(W, 0, 3 * C * C);
        if (Bi) RANGE(Bi, 0, 3 * C);
        RANGE(Q, 0, M * C);
        RANGE(K, 0, M * C);
        RANGE(V, 0, M * C);
        RopeState* r = nullptr;
        if (ll > 10 && pl[10]) {
            r = m_rope.get((long)pl[10]);
            if (!r || !r->set) return MCH_ERROR_ROPE_NOT_INITIALIZED;
            if (r->heads != H || r->hs != hs) {
                last_detail = "the rope handle was created for other heads or another head size";
                return MCH_ERROR_PARAM_OUT_OF_RANGE;
            }
        }
        void* ws = nullptr;
        if (k_gemm_qkv_heads_needs_tmp(X->dt(), (int)H, (int)hs, X->ptr, W->ptr, Q->ptr, K->ptr, V->ptr))
            ERRCHK(workspace((size_t)(M * 3 * C) * X->esize(), &ws));
        HIPCHK(k_gemm_qkv_heads(s, X->dt(), (int)B, (int)T, (int)H, (int)hs, X->ptr, W->ptr, Bi ? Bi->ptr : nullptr, Q->ptr, K->ptr,
                                V->ptr, ws, r ? (const float*)r->dcos.get() : nullptr, r ? (const float*)r->dsin.get() : nullptr,
                                r ? r->seq : 0));
        m_mem.touch((long)pl[7]);
        m_mem.touch((long)pl[8]);
        m_mem.touch((long)pl[9]);
        return 0;
    }

    case MCH_FN_LINEAR_FWD: {
        // l{M, N, K, hX, hW, hBias(0 = none), hY}: Y (M x N) = X (M x K) W^T (N x K) + bias (N), one launch
        NEED_L(7, 7);
        const long long M = pl[0], N = pl[1], K = pl[2];
        if (M < 1 || N < 1 || K < 1 || M > INT_MAX || N > INT_MAX || K > INT_MAX) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem *X, *W, *Bi = nullptr, *Y;
        ERRCHK(mem((long)pl[3], &X));
        ERRCHK(mem((long)pl[4], &W));
        if (pl[5]) ERRCHK(mem((long)pl[5], &Bi));
        ERRCHK(mem((long)pl[6], &Y));
        if (X->half != W->half || X->half != Y->half || (Bi && Bi->half != X->half)) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(X, 0, M * K);
        RANGE(W, 0, N * K);
        if (Bi) RANGE(Bi, 0, N);
        RANGE(Y, 0, M * N);
        void* ws = nullptr;
        if (k_gemm_bias_needs_tmp(X->dt(), (int)N, (int)K, X->ptr, W->ptr, Y->ptr)) ERRCHK(workspace((size_t)(M * N) * X->esize(), &ws));
        HIPCHK(k_gemm_bias(s, X->dt(), (int)M, (int)N, (int)K, X->ptr, W->ptr, Bi ? Bi->ptr : nullptr, Y->ptr, ws));
        m_mem.touch((long)pl[6]);
        return 0;
    }

    // ---- RoPE ------------------------------------------------------------------
    case MCH_FN_CREATE_ROPE: {
        // f{theta}, l{sharedIdx,gpuId,count,batch,seqLen,heads,hs} (device.h:4201-4229, rope.cu:502-607)
        NEED_F(1, 1);
        NEED_L(7, 7);
        long long seq = pl[4], heads = pl[5], hs = pl[6];
        if (seq < 1 || heads < 1 || hs < 2 || (hs & 1) || seq * hs > (1ll << 30)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        long h;
        ERRCHK(m_rope.create(&h));
        RopeState* r = m_rope.get(h);
        r->sharedIdx = (int)pl[0]; r->count = (int)pl[2]; r->batch = (int)pl[3];
        r->seq = (int)seq; r->heads = (int)heads; r->hs = (int)hs; r->theta = pf[0];
        int half = (int)hs / 2;
        // host tables exactly as the reference builds them: powf, then fp32 product, then cosf/sinf
        std::vector<float> freq(half), hc((size_t)seq * half), hsn((size_t)seq * half);
        int idx = 0;
        for (int i = 0; i < hs; i += 2) {
            float power = (float)(i / (float)hs);
            power = powf(r->theta, power);
            freq[idx++] = 1.0f / power;
        }
        for (int pos = 0; pos < seq; pos++)
            for (int i = 0; i < half; i++) {
                float fp = freq[i] * pos;
                hc[(size_t)pos * half + i] = cosf(fp);
                hsn[(size_t)pos * half + i] = sinf(fp);
            }
        size_t bytes = (size_t)seq * half * sizeof(float);
        void *dc = nullptr, *ds = nullptr;
        hipError_t e = hipMalloc(&dc, bytes);
        if (e == hipSuccess) e = hipMalloc(&ds, bytes);
        if (e == hipSuccess) e = hipMemcpyAsync(dc, hc.data(), bytes, hipMemcpyHostToDevice, s);
        if (e == hipSuccess) e = hipMemcpyAsync(ds, hsn.data(), bytes, hipMemcpyHostToDevice, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
        if (e != hipSuccess) {
            if (dc) (void)hipFree(dc);
            if (ds) (void)hipFree(ds);
            m_rope.free(h);
            return (long)e;
        }
        r->dcos = std::shared_ptr<void>(dc, [](void* p) { (void)hipFree(p); });
        r->dsin = std::shared_ptr<void>(ds, [](void* p) { (void)hipFree(p); });
        r->set = true;
        return set_out((float)h, ppOut, plOut);
    }
    case MCH_FN_FREE_ROPE:
        NEED_F(1, 1);
        HIPCHK(hipStreamSynchronize(s));
        return m_rope.free((long)pf[0]);
    case MCH_FN_ROPE_FWD: {
        // l{hRope,n,hX,hY[,freqOffset]} (device.h:4232-4255, rope.cu:785-825)
        NEED_L(4, 5);
        RopeState* r = m_rope.get((long)pl[0]);
        if (!r || !r->set) return MCH_ERROR_ROPE_NOT_INITIALIZED;
        long long n = pl[1];
        long long off = ll > 4 ? pl[4] : -1;
        if (off < 0) off = 0;  // offsets <= 0 mean "no shift" (rope.cu:808-814)
        MemItem *X, *Y;
        ERRCHK(mem((long)pl[2], &X));
        ERRCHK(mem((long)pl[3], &Y));
        if (X->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (n < 0 || (n & 1)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(X, 0, n);
        RANGE(Y, 0, n);
        {
            // largest table index any pair can reach must stay inside the [seq, hs/2] tables
            long long half = r->hs / 2, full = half * r->heads, wrap = (long long)r->seq * full;
            long long pairs = n / 2;
            long long maxbase = (pairs < wrap ? pairs : wrap) - 1;
            if (pairs > 0 && (maxbase / full) * half + (half - 1) + off >= (long long)r->seq * half) {
                last_detail = "rope table offset reaches past the last position of the table";
                return MCH_ERROR_PARAM_OUT_OF_RANGE;
            }
        }
        HIPCHK(k_rope(s, X->dt(), (size_t)n, X->ptr, Y->ptr, (const float*)r->dcos.get(), (const float*)r->dsin.get(), r->seq,
                      r->heads, r->hs, (int)off));
        m_mem.touch((long)pl[3]);
        return 0;
    }

    case MCH_FN_ROPE_BWD: {
        // l{hRope,n,hXdata,hYdiff,hXdiff}: the rotation by the opposite angle, never shifted (device.h:4266-4283, rope.cu:832-864)
        NEED_L(5, 5);
        RopeState* r = m_rope.get((long)pl[0]);
        if (!r || !r->set) return MCH_ERROR_ROPE_NOT_INITIALIZED;
        long long n = pl[1];
        MemItem *dY, *dX;
        ERRCHK(mem((long)pl[3], &dY));
        ERRCHK(mem((long)pl[4], &dX));
        if (dY->half != dX->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        if (n < 0 || (n & 1)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        RANGE(dY, 0, n);
        RANGE(dX, 0, n);
        HIPCHK(k_rope(s, dY->dt(), (size_t)n, dY->ptr, dX->ptr, (const float*)r->dcos.get(), (const float*)r->dsin.get(), r->seq,
                      r->heads, r->hs, 0, true));
        m_mem.touch((long)pl[4]);
        return 0;
    }

    case MCH_FN_FREE_BLOBLOADER:
        NEED_F(1, 1);
        return m_blobLoader.free((long)pf[0]);
    case MCH_FN_BLOBLOADER_RESETOFFSET: {
        // l{hBlobLoader, offsetInBytes} (device.h:4651-4662, blobloader.h:56-61)
        NEED_L(2, 2);
        BlobLoaderState* bl = m_blobLoader.get((long)pl[0]);
        if (!bl) return MCH_ERROR_BLOBLOADER_NOT_INITIALIZED;
        if (pl[1] < 0) return MCH_ERROR_WIN_INVALID_PARAMETER;
        bl->offsetBytes = (size_t)pl[1];
        bl->offsetItems = 0;
        return 0;
    }
    case MCH_FN_BLOBLOADER_ADDTOOFFSET: {
        // l{hBlobLoader, offsetInItems} (device.h:4665-4676, blobloader.h:63-67)
        NEED_L(2, 2);
        BlobLoaderState* bl = m_blobLoader.get((long)pl[0]);
        if (!bl) return MCH_ERROR_BLOBLOADER_NOT_INITIALIZED;
        if (pl[1] < 0) return MCH_ERROR_WIN_INVALID_PARAMETER;
        bl->offsetItems += (size_t)pl[1];
        return 0;
    }
    case MCH_FN_BLOBLOADER_LOAD: {
        // l{hBlobLoader, count, hData, localItemOffset} (device.h:4635-4648, blobloader.cu:83-126): copy `count` fp32
        // items starting at byte offsetBytes + 4 * (offsetItems + localItemOffset) of the file into the blob.  The
        // reference does not look at the file size; reading past the end is refused here instead of faulting.
        NEED_L(4, 4);
        BlobLoaderState* bl = m_blobLoader.get((long)pl[0]);
        if (!bl || !bl->data) return MCH_ERROR_BLOBLOADER_NOT_INITIALIZED;
        if (pl[3] < 0) return MCH_ERROR_WIN_INVALID_PARAMETER;
        if (pl[1] < 0) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        MemItem* D;
        ERRCHK(mem((long)pl[2], &D));
        const size_t count = (size_t)pl[1];
        if (count > D->count) return MCH_ERROR_WIN_INSUFFICIENT_BUFFER;
        const size_t start = bl->offsetBytes + (bl->offsetItems + (size_t)pl[3]) * sizeof(float);
        if (start > bl->fileSize || count * sizeof(float) > bl->fileSize - start) {
            last_detail = "the requested items lie past the end of the weight file";
            return MCH_ERROR_MEMORY_RANGE_EXCEEDED;
        }
        const unsigned char* src = bl->data + start;
        // through pinned staging in slices, so that one blob of any size needs a bounded host buffer
        const size_t slice = (size_t)16 << 20;   // items per slice (64 MiB)
        void* ws = nullptr;
        if (D->half) ERRCHK(workspace(std::min(count, slice) * sizeof(float), &ws));
        std::lock_guard<std::mutex> g(m_stageLock);
        for (size_t done = 0; done < count; done += slice) {
            const size_t n = std::min(slice, count - done);
            void* st;
            ERRCHK(staging(n * sizeof(float), &st));
            memcpy(st, src + done * sizeof(float), n * sizeof(float));
            if (!D->half) {
                HIPCHK(hipMemcpyAsync((float*)D->ptr + done, st, n * sizeof(float), hipMemcpyHostToDevice, s));
            } else {
                HIPCHK(hipMemcpyAsync(ws, st, n * sizeof(float), hipMemcpyHostToDevice, s));
                HIPCHK(k_convert(s, F32, ws, BF16, (bf16_t*)D->ptr + done, n));
            }
            HIPCHK(hipStreamSynchronize(s));   // the staging buffer is reused by the next slice
        }
        m_mem.touch((long)pl[2]);
        return 0;
    }

    case MCH_FN_FREE_EXTENSION:
        NEED_F(1, 1);
        return m_ext.free((long)pf[0]);

    default:
        break;
    }
    char buf[96];
    snprintf(buf, sizeof(buf), "function id %ld is outside the attention hot path and is not dispatched", fn);
    last_detail = buf;
    return MCH_ERROR_NOT_IMPLEMENTED;
}

// ---- extensions (extension.cu:17-179) ---------------------------------------------
typedef MCH_LONG (*FnExtInit)(void*, MCH_LONG);
typedef MCH_LONG (*FnExtInvoke)(MCH_LONG, float*, MCH_LONG, float**, MCH_LONG*, MCH_TCHAR*, MCH_LONG);
typedef MCH_LONG (*FnExtInvokeEx)(MCH_LONG, float*, MCH_LONG, float**, MCH_LONG*, MCH_TCHAR*, MCH_TCHAR*, MCH_LONG, MCH_TCHAR*,
                                  MCH_LONG);

static void* self_handle()
{
    Dl_info info;
    if (!dladdr((void*)&self_handle, &info) || !info.dli_fname) return nullptr;
    return dlopen(info.dli_fname, RTLD_NOW | RTLD_NOLOAD);
}

long Kernel::create_extension(long kernelIdx, MCH_TCHAR* path, float** ppOut, MCH_LONG* plOut)
{
    if (!path) return MCH_ERROR_PARAM_NULL;
    std::string p = utf16_to_utf8(path);
    void* lib = dlopen(p.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (!lib) { last_detail = std::string("cannot load extension: ") + dlerror(); return MCH_ERROR_FILE_OPEN; }
    FnExtInit init = (FnExtInit)dlsym(lib, "DLL_InitFloatCustomExtension");
    void* inv = dlsym(lib, "DLL_InvokeFloatCustomExtension");
    if (!init || !inv) { dlclose(lib); last_detail = "extension lacks DLL_InitFloatCustomExtension / DLL_InvokeFloatCustomExtension"; return MCH_ERROR_NOT_IMPLEMENTED; }
    long e = init(self_handle(), (MCH_LONG)kernelIdx);
    if (e) { dlclose(lib); return e; }
    long h;
    if ((e = m_ext.create(&h))) { dlclose(lib); return e; }
    ExtensionState* st = m_ext.get(h);
    st->lib = lib;
    st->fnInvoke = inv;
    st->fnInvokeEx = dlsym(lib, "DLL_InvokeFloatCustomExtensionEx");
    return set_out((float)h, ppOut, plOut);
}

// CUDA_FN_CREATE_BLOBLOADER (CudaDnn.cs:6438-6450, device.h:4606-4618, blobloader.cu:24-52): map the file read-only
long Kernel::create_blobloader(MCH_TCHAR* path, float** ppOut, MCH_LONG* plOut)
{
    if (!path) return MCH_ERROR_PARAM_NULL;
    if (!plOut || !ppOut || !*ppOut) return MCH_ERROR_PARAM_NULL;
    const std::string p = utf16_to_utf8(path);
    const int fd = open(p.c_str(), O_RDONLY);
    if (fd < 0) { last_detail = "cannot open " + p; return MCH_ERROR_WIN_FILE_NOT_FOUND; }
    struct stat sb;
    if (fstat(fd, &sb) != 0 || sb.st_size <= 0) { close(fd); last_detail = "cannot size " + p; return MCH_ERROR_WIN_FILE_NOT_FOUND; }
    void* m = mmap(nullptr, (size_t)sb.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (m == MAP_FAILED) { close(fd); last_detail = "cannot map " + p; return MCH_ERROR_WIN_FILE_NOT_FOUND; }
    long h;
    if (long e = m_blobLoader.create(&h)) { munmap(m, (size_t)sb.st_size); close(fd); return e; }
    BlobLoaderState* st = m_blobLoader.get(h);
    st->fd = fd; st->data = (const unsigned char*)m; st->fileSize = (size_t)sb.st_size;
    return set_out((float)h, ppOut, plOut);
}

// ATTN_DECODE_FWD: f{scale}, l{batch,heads,kvHeads,hs,len,hQ,hKc,hVc,hY,strideB,strideH,strideT[,hRope,hKnew,hVnew]}.
// With staticScratch the split partials and merge tickets come from the file-scope device array instead of the
// kernel object's allocations.
long Kernel::attn_decode_fwd(float* pf, long lf, MCH_LONGLONG* pl, long ll, bool staticScratch)
{
    hipStream_t s = m_stream;
    NEED_F(1, 1);
    NEED_L(12, 15);
    if (ll != 12 && ll != 15) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    long long B = pl[0], H = pl[1], KVH = pl[2], hs = pl[3], len = pl[4];
    long long sB = pl[9], sH = pl[10], sT = pl[11];
    if (B < 1 || H < 1 || KVH < 1 || hs < 1 || len < 1 || H % KVH || sB < 0 || sH < 0 || sT < 1 || (hs & 1))
        return MCH_ERROR_PARAM_OUT_OF_RANGE;
    MemItem *Q, *KC, *VC, *Y;
    ERRCHK(mem((long)pl[5], &Q));
    ERRCHK(mem((long)pl[6], &KC));
    ERRCHK(mem((long)pl[7], &VC));
    ERRCHK(mem((long)pl[8], &Y));
    if (Q->half != KC->half || Q->half != VC->half || Q->half != Y->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
    RANGE(Q, 0, B * H * hs);
    RANGE(Y, 0, B * H * hs);
    long long need = (B - 1) * sB + (KVH - 1) * sH + (len - 1) * sT + hs;
    RANGE(KC, 0, need);
    RANGE(VC, 0, need);
    float scale = pf[0] != 0.f ? pf[0] : (float)(1.0 / sqrt((double)hs));
    // Everything that can refuse the call comes before the first kernel: a refused call leaves q, the new key / value and
    // the caches untouched, so that the caller can repeat it through the other entry point.
    RopeState* rp = nullptr;
    MemItem *KN = nullptr, *VN = nullptr;
    const bool append = ll == 15 && (pl[12] || pl[13] || pl[14]);
    if (append) {
        rp = pl[12] ? m_rope.get((long)pl[12]) : nullptr;
        if (pl[12] && (!rp || !rp->set)) return MCH_ERROR_ROPE_NOT_INITIALIZED;
        if (rp && (rp->hs != hs || len > rp->seq)) return MCH_ERROR_PARAM_OUT_OF_RANGE;
        ERRCHK(mem((long)pl[13], &KN));
        ERRCHK(mem((long)pl[14], &VN));
        if (KN->half != Q->half || VN->half != Q->half) return MCH_ERROR_MEMORY_MIXED_HALF_TYPES;
        RANGE(KN, 0, B * KVH * hs);
        RANGE(VN, 0, B * KVH * hs);
    }
    size_t wsb = attn_decode_workspace_bytes((int)B, (int)H, (int)hs, (int)len);
    void* ws;
    size_t wsHave;
    int* tk;
    if (staticScratch) {
        // partials and tickets live in this device's copy of the file-scope array: nothing is allocated
        char* base = nullptr;
        ERRCHK(static_scratch(m_device, &base));
        if (B * H > MCH_NOALLOC_MAX_TICKETS || wsb > MCH_NOALLOC_PARTIAL_BYTES) {
            last_detail = "the no-allocation decode attention holds at most 4096 (batch x head) pairs and 4 MiB of split partials";
            return MCH_ERROR_PARAM_OUT_OF_RANGE;
        }
        tk = (int*)base;
        ws = base + MCH_NOALLOC_MAX_TICKETS * sizeof(int);
        wsHave = MCH_NOALLOC_PARTIAL_BYTES;
    } else {
        ERRCHK(workspace(wsb, &ws));
        wsHave = m_wsBytes;
        ERRCHK(tickets((size_t)(B * H), &tk));
    }
    if (append) {
        HIPCHK(k_rope_append(s, Q->dt(), Q->ptr, KN->ptr, VN->ptr, KC->ptr, VC->ptr, (int)B, (int)H, (int)KVH, (int)hs,
                             (int)len - 1, sB, sH, sT, rp ? (const float*)rp->dcos.get() : nullptr,
                             rp ? (const float*)rp->dsin.get() : nullptr));
        m_mem.touch((long)pl[5]);
        m_mem.touch((long)pl[6]);
        m_mem.touch((long)pl[7]);
        m_mem.touch((long)pl[13]);
    }
    // the static array keeps what the last call left: the tickets must start at zero (a fill kernel, not a memset node)
    if (staticScratch) HIPCHK(k_set(s, F32, tk, (size_t)(B * H), 0.f));
    HIPCHK(k_attn_decode(s, Q->dt(), Q->ptr, KC->ptr, VC->ptr, Y->ptr, (int)B, (int)H, (int)KVH, (int)hs, (int)len, sB, sH,
                         sT, scale, ws, wsHave, nullptr, tk));
    m_mem.touch((long)pl[8]);
    return 0;
}

// the same call through the entry point that allocates nothing
long Kernel::attn_decode_no_alloc(float* pf, long lf, MCH_LONGLONG* pl, long ll)
{
    last_detail.clear();
    if (!m_stream) return MCH_ERROR_DEVICE_NOT_INITIALIZED;
    HIPCHK(hipSetDevice(m_device));
    return attn_decode_fwd(pf, lf, pl, ll, true);
}

long Kernel::run_extension(long hExt, long fn, float* pf, long lf, MCH_TCHAR* szIn, float** ppOut, MCH_LONG* plOut,
                           MCH_TCHAR* szErr, long errMax)
{
    ExtensionState* st = m_ext.get(hExt);
    if (!st) return MCH_ERROR_EXTENSION_NOT_INITIALIZED;
    if (lf == 0) pf = nullptr;
    if (szIn == nullptr)
        return ((FnExtInvoke)st->fnInvoke)((MCH_LONG)fn, pf, (MCH_LONG)lf, ppOut, plOut, szErr, (MCH_LONG)errMax);
    if (!st->fnInvokeEx) return MCH_ERROR_NOT_IMPLEMENTED;
    return ((FnExtInvokeEx)st->fnInvokeEx)((MCH_LONG)fn, pf, (MCH_LONG)lf, ppOut, plOut, szIn, nullptr, 0, szErr, (MCH_LONG)errMax);
}

long Kernel::query_extension(MCH_LONG* pIn, long n, MCH_TCHAR* out, long outMax, MCH_TCHAR* err, long errMax)
{
    // LONG{hExt, fnIdx, args...} (device.h:4590-4603); at most 5 args are forwarded as floats (extension.cu:153-179)
    if (n < 2) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    if (!pIn) return MCH_ERROR_PARAM_NULL;
    ExtensionState* st = m_ext.get(pIn[0]);
    if (!st) return MCH_ERROR_EXTENSION_NOT_INITIALIZED;
    if (!st->fnInvokeEx) return MCH_ERROR_NOT_IMPLEMENTED;
    long cnt = n - 2;
    if (cnt > 5) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    float args[5];
    for (long i = 0; i < cnt; i++) args[i] = (float)pIn[2 + i];
    float* o = nullptr;
    MCH_LONG lo = 0;
    if (out && outMax > 0) out[0] = 0;
    long e = ((FnExtInvokeEx)st->fnInvokeEx)(pIn[1], args, (MCH_LONG)cnt, &o, &lo, nullptr, out, (MCH_LONG)outMax, err, (MCH_LONG)errMax);
    if (e) return e;
    if (o != nullptr && out) {
        // the extension passes its "finished" flag through the output pointer; the parent appends the end marker
        std::string cur = utf16_to_utf8(out) + "\n[END]";
        utf8_to_utf16(cur, out, outMax);
    }
    return 0;
}

// ---------------------------------------------------------------------------
// kernel table (dllmain.cpp:6-14, CudaDnnDLL.cpp:1747-1805): 2048 slots, slot 0 reserved
static const int MAX_KERNELS = 2048;
static Kernel* g_kernels[MAX_KERNELS];
static std::mutex g_tableLock;

static const char* error_text(long e)
{
    switch (e) {
    case MCH_ERROR_DLL_NOT_INIT: return "The library is not initialized.";
    case MCH_ERROR_PARAM: return "General parameter error.";
    case MCH_ERROR_PARAM_OUT_OF_RANGE: return "A parameter is out of range.";
    case MCH_ERROR_PARAM_NULL: return "A parameter is NULL (or the kernel/handle does not exist).";
    case MCH_ERROR_FILE_OPEN: return "Failed to open the file.";
    case MCH_ERROR_MEMORY_OUT: return "Out of device memory.";
    case MCH_ERROR_MEMORY_NULL: return "The memory is NULL.";
    case MCH_ERROR_NOT_IMPLEMENTED: return "The function is not implemented.";
    case MCH_ERROR_MEMORY_RANGE_EXCEEDED: return "The memory range was exceeded.";
    case MCH_ERROR_MEMORY_MIXED_HALF_TYPES: return "Half and full size memory types were mixed.";
    case MCH_ERROR_MEMORY_HALF_TYPE_NOT_SUPPORTED: return "Half size memory is not supported by this function.";
    case MCH_ERROR_MEMORY_NOT_FOUND: return "The memory handle was not found.";
    case MCH_ERROR_DEVICE_NOT_INITIALIZED: return "The device is not initialized.";
    case MCH_ERROR_ROPE_NOT_INITIALIZED: return "The RoPE handle is not initialized.";
    case MCH_ERROR_ATTN_NOT_INITIALIZED: return "The attention handle is not initialized.";
    case MCH_ERROR_ATTN_INCOMPATIBLE_BLOB_SIZE: return "A blob passed to the attention handle has an incompatible size.";
    case MCH_ERROR_ATTN_INVALID_BLOCK_SIZE: return "The block size exceeds the one the attention handle was set for.";
    case MCH_ERROR_EXTENSION_NOT_INITIALIZED: return "The extension is not initialized.";
    default: return nullptr;
    }
}

static void put_error(Kernel* k, long e, MCH_TCHAR* szErr, long max)
{
    if (!szErr || max <= 0) return;
    std::string msg;
    const char* t = error_text(e);
    if (t) msg = t;
    else if (e > 0 && e < 2000) msg = std::string("HIP runtime error: ") + hipGetErrorString((hipError_t)e);
    else msg = "Unknown error.";
    if (k && !k->last_detail.empty()) msg += " " + k->last_detail;
    char code[32];
    snprintf(code, sizeof(code), " (%ld)", e);
    msg += code;
    utf8_to_utf16(msg, szErr, max);
}

static Kernel* kernel_at(long idx)
{
    if (idx < 0 || idx >= MAX_KERNELS) return nullptr;
    std::lock_guard<std::mutex> g(g_tableLock);
    return g_kernels[idx];
}

// ---------------------------------------------------------------------------
// Call trace, the counterpart of the reference's _TRACEAPI build (CudaDnnDLL/Cuda Files/main.cu:44-55): with the
// environment variable MYCAFFE_HIP_TRACE set, every dispatched call appends one line
//   FLOAT calling CudaDnnDLL FunctionID (220) CUDA_FN_GEMM kernel 1 floats 2 longs 10 -> 0
// to stderr (value "1" or "stderr") or to the file the variable names.  Off (one pointer test per call) otherwise.
static const char* api_name(long fn)
{
#define N(x) {MCH_FN_##x, "CUDA_FN_" #x}
    static const struct { long id; const char* name; } table[] = {
        {MCH_DLL_FREEMEM, "CUDA_DLL_FREEMEM"}, {MCH_DLL_INITIALIZE, "CUDA_DLL_INITIALIZE"}, {MCH_DLL_CLEANUP, "CUDA_DLL_CLEANUP"},
        N(SETDEVICE), N(GETDEVICE), N(SYNCHRONIZEDEVICE), N(CREATE_MEMORYPOINTER), N(FREE_MEMORYPOINTER), N(ALLOCMEM_HALF), N(ALLOCMEM), N(FREEMEM), N(GETMEM), N(SETMEM), N(CREATE_CUDNN), N(FREE_CUDNN), N(CREATE_TENSORDESC), N(FREE_TENSORDESC), N(SET_TENSORDESC), N(CREATE_EXTENSION), N(FREE_EXTENSION), N(EXTENSION_RUN), N(SOFTMAX_FWD), N(SOFTMAX_BWD), N(ATTN_CREATE), N(ATTN_FREE), N(ATTN_SET), N(ATTN_FWD), N(ATTN_BWD), N(SET), N(COPY), N(GEMM2), N(GEMM), N(GEMV), N(AXPY), N(SCAL), N(SCALE), N(ADD_SCALAR), N(ADD), N(SUB), N(MUL), N(DIV), N(EXP), N(LOG), N(POWX), N(SQRT), N(TRANSPOSE), N(MASK), N(MASK_BATCH), N(TRANSPOSE_HW), N(INVERT), N(CHANNEL_MEAN), N(CHANNEL_MAX), N(CHANNEL_SUB), N(CHANNEL_SUM), N(CHANNEL_DIV), N(CHANNEL_DOT), N(CHANNEL_COPY), N(CHANNEL_FILLFROM), N(CHANNEL_COPYALL), N(CHANNEL_DUP), N(CHANNEL_SUM2), N(EMBED_FWD), N(RELU_FWD), N(RELU_BWD), N(GELU_FWD), N(GELU_BWD), N(SILU_FWD), N(SILU_BWD), N(CREATE_LAYERNORM), N(FREE_LAYERNORM), N(LAYERNORM_FWD), N(LAYERNORM_BWD), N(CREATE_ROPE), N(FREE_ROPE), N(ROPE_FWD), N(ROPE_BWD), N(CREATE_BLOBLOADER), N(FREE_BLOBLOADER), N(BLOBLOADER_LOAD), N(BLOBLOADER_RESETOFFSET), N(BLOBLOADER_ADDTOOFFSET), N(ATTN_DECODE_FWD), N(RMSNORM_FWD), N(SWIGLU_FWD), N(QKV_PROJ_HEADS), N(LINEAR_FWD)};
#undef N
    for (const auto& t : table)
        if (t.id == fn) return t.name;
    return "(not dispatched)";
}

static FILE* trace_file()
{
    static FILE* f = []() -> FILE* {
        const char* v = getenv("MYCAFFE_HIP_TRACE");
        if (!v || !*v || !strcmp(v, "0")) return nullptr;
        if (!strcmp(v, "1") || !strcmp(v, "stderr")) return stderr;
        return fopen(v, "a");
    }();
    return f;
}

static void trace_call(long kIdx, long fn, long lf, long ll, long rc)
{
    FILE* f = trace_file();
    if (!f) return;
    static std::mutex lock;
    std::lock_guard<std::mutex> g(lock);
    fprintf(f, "FLOAT calling CudaDnnDLL FunctionID (%ld) %s kernel %ld floats %ld longs %ld -> %ld\n", fn, api_name(fn), kIdx, lf, ll, rc);
    fflush(f);
}

static long invoke_untraced(long kIdx, long fn, float* pf, long lf, MCH_LONGLONG* pl, long ll, MCH_TCHAR* szIn, float** ppOut,
                   MCH_LONG* plOut, MCH_TCHAR* szErr, long errMax, bool ex)
{
    if (szErr && errMax > 0) szErr[0] = 0;
    if (kIdx < 0 || kIdx >= MAX_KERNELS) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    long e = 0;
    Kernel* k = nullptr;
    switch (fn) {
    case MCH_DLL_INITIALIZE: {
        // creates a kernel, returns its index in (*ppOutput)[0] (CudaDnnDLL.cpp:154-176)
        if (!ppOut || !*ppOut || !plOut) return MCH_ERROR_PARAM_NULL;
        k = new Kernel();
        e = k->initialize(pf, lf);
        if (e) { put_error(k, e, szErr, errMax); delete k; return e; }
        long slot = -1;
        {
            std::lock_guard<std::mutex> g(g_tableLock);
            for (int i = 1; i < MAX_KERNELS; i++)
                if (!g_kernels[i]) { g_kernels[i] = k; slot = i; break; }
        }
        if (slot < 0) { delete k; e = MCH_ERROR_MEMORY_OUT; put_error(nullptr, e, szErr, errMax); return e; }
        (*ppOut)[0] = (float)slot;
        *plOut = 1;
        return 0;
    }
    case MCH_DLL_CLEANUP: {
        std::lock_guard<std::mutex> g(g_tableLock);
        k = g_kernels[kIdx];
        g_kernels[kIdx] = nullptr;
        delete k;
        return 0;
    }
    case MCH_DLL_FREEMEM:
        if (!(k = kernel_at(kIdx))) { e = MCH_ERROR_PARAM_NULL; put_error(nullptr, e, szErr, errMax); return e; }
        e = k->free_host(pf);
        if (e) put_error(k, e, szErr, errMax);
        return e;
    default:
        break;
    }
    if (!(k = kernel_at(kIdx))) { e = MCH_ERROR_PARAM_NULL; put_error(nullptr, e, szErr, errMax); return e; }
    if (ex && fn == MCH_FN_CREATE_EXTENSION) {
        e = k->create_extension(kIdx, szIn, ppOut, plOut);
    } else if (ex && fn == MCH_FN_CREATE_BLOBLOADER) {
        e = k->create_blobloader(szIn, ppOut, plOut);
    } else if (fn == MCH_FN_EXTENSION_RUN) {
        // f{hExt, fnIdx, args...} (device.h:4569-4588)
        if (lf < 2) e = MCH_ERROR_PARAM_OUT_OF_RANGE;
        else if (!pf) e = MCH_ERROR_PARAM_NULL;
        else {
            e = k->run_extension((long)pf[0], (long)pf[1], pf + 2, lf - 2, ex ? szIn : nullptr, ppOut, plOut, szErr, errMax);
            if (e && szErr && szErr[0]) return e;  // the extension wrote its own message
        }
    } else if (ex) {
        e = MCH_ERROR_PARAM_OUT_OF_RANGE;
    } else {
        e = k->run(fn, pf, lf, pl, ll, ppOut, plOut, false);
    }
    if (e) put_error(k, e, szErr, errMax);
    return e;
}

static long invoke(long kIdx, long fn, float* pf, long lf, MCH_LONGLONG* pl, long ll, MCH_TCHAR* szIn, float** ppOut,
                   MCH_LONG* plOut, MCH_TCHAR* szErr, long errMax, bool ex)
{
    const long rc = invoke_untraced(kIdx, fn, pf, lf, pl, ll, szIn, ppOut, plOut, szErr, errMax, ex);
    if (trace_file()) trace_call(kIdx, fn, lf, ll, rc);
    return rc;
}

}  // namespace mch

using namespace mch;

extern "C" {

MCH_LONG DLL_InvokeFloat(MCH_LONG k, MCH_LONG fn, float* pIn, MCH_LONG lIn, float** ppOut, MCH_LONG* plOut, MCH_TCHAR* szErr,
                         MCH_LONG errMax)
{
    // the legacy entry point forwards no integer array (CudaDnnDLL.cpp:303)
    return (MCH_LONG)invoke(k, fn, pIn, lIn, nullptr, 0, nullptr, ppOut, plOut, szErr, errMax, false);
}

MCH_LONG DLL_InvokeFloatEx2(MCH_LONG k, MCH_LONG fn, float* pIn, MCH_LONG lIn, MCH_LONGLONG* plIn, MCH_LONG llIn, float** ppOut,
                            MCH_LONG* plOut, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return (MCH_LONG)invoke(k, fn, pIn, lIn, plIn, llIn, nullptr, ppOut, plOut, szErr, errMax, false);
}

MCH_LONG DLL_InvokeFloatEx(MCH_LONG k, MCH_LONG fn, float* pIn, MCH_LONG lIn, MCH_TCHAR* pszIn, float** ppOut, MCH_LONG* plOut,
                           MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return (MCH_LONG)invoke(k, fn, pIn, lIn, nullptr, 0, pszIn, ppOut, plOut, szErr, errMax, true);
}

// The double base type's own entry points (DLL_InvokeDouble, DLL_InvokeDoubleEx2, Internal_GetPointerDouble) are in
// library_f64.hip.  What stays unbuilt for it: the string-carrying calls, which only create extensions and blob loaders -
// the llama2 extension is a float library (a double-typed parent fails cleanly at CREATE_EXTENSION).
static MCH_LONG double_unsupported(MCH_TCHAR* szErr, MCH_LONG errMax)
{
    utf8_to_utf16("This call is not built for the double base type: extensions and blob loaders are float objects. (90009)", szErr, errMax);
    return MCH_ERROR_NOT_IMPLEMENTED;
}

MCH_LONG DLL_InvokeDoubleEx(MCH_LONG, MCH_LONG, double*, MCH_LONG, MCH_TCHAR*, double**, MCH_LONG*, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return double_unsupported(szErr, errMax);
}

MCH_LONG DLL_QueryString(MCH_LONG kIdx, MCH_LONG fn, MCH_LONG* pIn, MCH_LONG lIn, MCH_TCHAR** ppOut, MCH_TCHAR* szErr,
                         MCH_LONG errMax)
{
    if (szErr && errMax > 0) szErr[0] = 0;
    if (kIdx < 0 || kIdx >= MAX_KERNELS) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    Kernel* k = kernel_at(kIdx);
    if (!k) { put_error(nullptr, MCH_ERROR_PARAM_OUT_OF_RANGE, szErr, errMax); return MCH_ERROR_PARAM_OUT_OF_RANGE; }
    if (fn == MCH_DLL_FREEMEM) {
        if (ppOut && *ppOut) { free(*ppOut); *ppOut = nullptr; }
        return 0;
    }
    if (ppOut) *ppOut = nullptr;
    if (fn == MCH_QRY_DEVICE_NAME) {
        (void)pIn; (void)lIn;
        if (!ppOut) return MCH_ERROR_PARAM_NULL;
        std::string name = k->device_name();
        long cap = (long)name.size() + 1;
        MCH_TCHAR* buf = (MCH_TCHAR*)malloc(cap * sizeof(MCH_TCHAR));
        if (!buf) return MCH_ERROR_MEMORY_OUT;
        utf8_to_utf16(name, buf, cap);
        *ppOut = buf;
        return 0;
    }
    put_error(nullptr, MCH_ERROR_NOT_IMPLEMENTED, szErr, errMax);
    return MCH_ERROR_NOT_IMPLEMENTED;
}

MCH_LONG DLL_QueryStringFloatEx(MCH_LONG kIdx, MCH_LONG fn, MCH_LONG* pIn, MCH_LONG lIn, MCH_TCHAR* pszOut, MCH_LONG outMax,
                                MCH_TCHAR* szErr, MCH_LONG errMax)
{
    if (szErr && errMax > 0) szErr[0] = 0;
    if (kIdx < 0 || kIdx >= MAX_KERNELS) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    Kernel* k = kernel_at(kIdx);
    if (!k) { put_error(nullptr, MCH_ERROR_PARAM_OUT_OF_RANGE, szErr, errMax); return MCH_ERROR_PARAM_OUT_OF_RANGE; }
    long e = fn == MCH_QRY_EXTENSION_STRING ? k->query_extension(pIn, lIn, pszOut, outMax, szErr, errMax)
                                            : (long)MCH_ERROR_PARAM_OUT_OF_RANGE;
    if (e && szErr && szErr[0] == 0) put_error(k, e, szErr, errMax);
    return (MCH_LONG)e;
}

MCH_LONG DLL_QueryStringDoubleEx(MCH_LONG, MCH_LONG, MCH_LONG*, MCH_LONG, MCH_TCHAR*, MCH_LONG, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return double_unsupported(szErr, errMax);
}

MCH_LONG Internal_GetPointerFloat(int32_t ht, MCH_LONG kIdx, MCH_LONG h, void** pp)
{
    if (ht != 0 || !pp) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    Kernel* k = kernel_at(kIdx);
    if (!k) return MCH_ERROR_PARAM_NULL;
    return (MCH_LONG)k->get_pointer(h, pp);
}

MCH_LONG Internal_AllocHostFloat(MCH_LONG kIdx, MCH_LONG count, float** dst, float* src, bool srcOnDevice)
{
    if (kIdx < 0 || kIdx >= MAX_KERNELS) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    Kernel* k = kernel_at(kIdx);
    if (!k) return MCH_ERROR_PARAM_NULL;
    return (MCH_LONG)k->alloc_host(count, dst, src, srcOnDevice);
}
MCH_LONG Internal_AllocHostDouble(MCH_LONG, MCH_LONG, double**, double*, bool) { return MCH_ERROR_NOT_IMPLEMENTED; }

MCH_LONG MCH_AttnDecodeForwardNoAlloc(MCH_LONG kIdx, float* pIn, MCH_LONG lIn, MCH_LONGLONG* plIn, MCH_LONG llIn, MCH_TCHAR* szErr,
                                      MCH_LONG errMax)
{
    if (szErr && errMax > 0) szErr[0] = 0;
    if (kIdx < 0 || kIdx >= MAX_KERNELS) return MCH_ERROR_PARAM_OUT_OF_RANGE;
    Kernel* k = kernel_at(kIdx);
    if (!k) { put_error(nullptr, MCH_ERROR_PARAM_NULL, szErr, errMax); return MCH_ERROR_PARAM_NULL; }
    long e = k->attn_decode_no_alloc(pIn, lIn, plIn, llIn);
    if (e) put_error(k, e, szErr, errMax);
    return (MCH_LONG)e;
}

MCH_LONG MCH_TimeInvokeFloatEx2(MCH_LONG kIdx, MCH_LONG fn, float* pIn, MCH_LONG lIn, MCH_LONGLONG* plIn, MCH_LONG llIn,
                                MCH_LONG nWarmup, MCH_LONG nReps, float* pfMs, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    return MCH_TimeInvokeFloatEx2Sets(kIdx, fn, pIn, lIn, plIn, llIn, 1, nWarmup, nReps, pfMs, szErr, errMax);
}

MCH_LONG MCH_TimeInvokeFloatEx2Sets(MCH_LONG kIdx, MCH_LONG fn, float* pIn, MCH_LONG lIn, MCH_LONGLONG* plIn, MCH_LONG llIn,
                                    MCH_LONG nSets, MCH_LONG nWarmup, MCH_LONG nReps, float* pfMs, MCH_TCHAR* szErr, MCH_LONG errMax)
{
    if (szErr && errMax > 0) szErr[0] = 0;
    Kernel* k = kernel_at(kIdx);
    if (!k || !pfMs || nReps < 1 || nWarmup < 0 || nSets < 1 || (nSets > 1 && (!plIn || llIn < 1))) return MCH_ERROR_PARAM_NULL;
    float dummy[4];
    float* po = dummy;
    MCH_LONG lo = 4;
    long e = 0;
    // dispatch i takes the i-th list of long arguments, round robin over the nSets lists that lie one after the other
    auto longs = [&](int i) { return plIn ? plIn + (size_t)(i % nSets) * llIn : plIn; };
    for (int i = 0; i < nWarmup && !e; i++) { po = dummy; lo = 4; e = k->run(fn, pIn, lIn, longs(i), llIn, &po, &lo, true); }
    hipEvent_t a = nullptr, b = nullptr;
    if (!e) e = (long)hipEventCreate(&a);
    if (!e) e = (long)hipEventCreate(&b);
    if (!e) e = (long)hipEventRecord(a, k->stream());
    for (int i = 0; i < nReps && !e; i++) { po = dummy; lo = 4; e = k->run(fn, pIn, lIn, longs(nWarmup + i), llIn, &po, &lo, true); }
    if (!e) e = (long)hipEventRecord(b, k->stream());
    if (!e) e = (long)hipEventSynchronize(b);
    float ms = 0.f;
    if (!e) e = (long)hipEventElapsedTime(&ms, a, b);
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
    if (e) { put_error(k, e, szErr, errMax); return (MCH_LONG)e; }
    *pfMs = ms / (float)nReps;
    return 0;
}

}  // extern "C"
