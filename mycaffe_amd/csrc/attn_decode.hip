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
#include "lane_ops.h"

namespace mch {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 16 bytes of a cache row: W elements
template <typename T> struct Vec16;
template <> struct Vec16<float> {
    static constexpr int W = 4;
    __device__ static inline void load(const float* p, float* out)
    {
        float4 v = *(const float4*)p;
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    }
    __device__ static inline void unpack(u32x4 r, float* out)
    {
#pragma unroll
        for (int i = 0; i < 4; i++) out[i] = __uint_as_float(r[i]);
    }
    __device__ static inline u32x4 pack(const float* in)
    {
        return u32x4{__float_as_uint(in[0]), __float_as_uint(in[1]), __float_as_uint(in[2]), __float_as_uint(in[3])};
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
    __device__ static inline void unpack(u32x4 r, float* out)
    {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            out[2 * i] = __uint_as_float(r[i] << 16);
            out[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
        }
    }
    __device__ static inline u32x4 pack(const float* in)
    {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; i++) r[i] = (uint32_t)f32_to_bf16(in[2 * i]) | ((uint32_t)f32_to_bf16(in[2 * i + 1]) << 16);
        return r;
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
    int* counters;   // one zero-initialised ticket per (batch, head): enables the in-kernel merge
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

// Streams cache rows [t0, t1) for one (batch, head): every lane group of LPR lanes keeps its own
// running max m, sum l and output slice acc[W] (dims gl*W ..).  qv holds the query slice, pre-scaled.
// A stage is U row groups of K and of V per wavefront, kept as loaded (16 bytes per lane and row);
// the loads of the next stage are issued before the current one is consumed.
template <int U> struct DecodeStage { u32x4 k[U], v[U]; };

template <typename T, int LPR, int U>
__device__ __forceinline__ void decode_issue(DecodeStage<U>& st, const T* __restrict__ kc, const T* __restrict__ vc, long long strideT,
                                             int tb, int t1, int grp, int d0, bool active)
{
    constexpr int RPW = 64 / LPR;
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int t = tb + u * RPW + grp;
        u32x4 z = {0u, 0u, 0u, 0u};
        st.k[u] = z;
        if (t < t1 && active) st.k[u] = *(const u32x4*)(kc + (size_t)t * strideT + d0);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int t = tb + u * RPW + grp;
        u32x4 z = {0u, 0u, 0u, 0u};
        st.v[u] = z;
        if (t < t1 && active) st.v[u] = *(const u32x4*)(vc + (size_t)t * strideT + d0);
    }
}

template <typename T, int LPR, int U>
__device__ __forceinline__ void decode_consume(const DecodeStage<U>& st, int tb, int t1, int grp, const float (&qv)[Vec16<T>::W],
                                               float& m, float& l, float (&acc)[Vec16<T>::W])
{
    constexpr int W = Vec16<T>::W;
    constexpr int RPW = 64 / LPR;
    float s[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        float kv[W];
        Vec16<T>::unpack(st.k[u], kv);
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < W; i++) d += qv[i] * kv[i];
        d = group_sum<LPR>(d);
        s[u] = (tb + u * RPW + grp) < t1 ? d : -INFINITY;
    }
    float mn = m;
#pragma unroll
    for (int u = 0; u < U; u++) mn = fmaxf(mn, s[u]);
    if (mn > -INFINITY) {
        const float corr = __expf(m - mn);  // m == -inf gives 0
        l *= corr;
#pragma unroll
        for (int i = 0; i < W; i++) acc[i] *= corr;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const float p = __expf(s[u] - mn);  // masked rows: exp(-inf) = 0
            l += p;
            float vv[W];
            Vec16<T>::unpack(st.v[u], vv);
#pragma unroll
            for (int i = 0; i < W; i++) acc[i] += p * vv[i];
        }
        m = mn;
    }
}

template <typename T, int LPR>
__device__ __forceinline__ void decode_stream(const T* __restrict__ kc, const T* __restrict__ vc, long long strideT, int t0, int t1,
                                              unsigned rot, int wave, int grp, int d0, bool active,
                                              const float (&qv)[Vec16<T>::W], float& m, float& l, float (&acc)[Vec16<T>::W])
{
    constexpr int RPW = 64 / LPR;  // rows per wavefront load
    constexpr int U = 4;           // row groups per stage and operand
    constexpr int NW = 4;
    constexpr int STEP = NW * RPW * U;
    // The online softmax does not care about row order, so every workgroup starts at its own rotation of the
    // range instead of all of them walking their caches in lockstep.
    const int nIt = (t1 - t0 + STEP - 1) / STEP;
    if (nIt <= 0) return;
    int j = (int)(rot % (unsigned)nIt);
    auto next = [&](int x) { return x + 1 == nIt ? 0 : x + 1; };
    const int w0 = t0 + wave * RPW * U;
    DecodeStage<U> A, B;
    decode_issue<T, LPR, U>(A, kc, vc, strideT, w0 + j * STEP, t1, grp, d0, active);
    for (int it = 0; it < nIt; it += 2) {
        const int j1 = next(j), j2 = next(j1);
        const bool has1 = it + 1 < nIt, has2 = it + 2 < nIt;
        if (has1) decode_issue<T, LPR, U>(B, kc, vc, strideT, w0 + j1 * STEP, t1, grp, d0, active);
        decode_consume<T, LPR, U>(A, w0 + j * STEP, t1, grp, qv, m, l, acc);
        if (has1) {
            if (has2) decode_issue<T, LPR, U>(A, kc, vc, strideT, w0 + j2 * STEP, t1, grp, d0, active);
            decode_consume<T, LPR, U>(B, w0 + j1 * STEP, t1, grp, qv, m, l, acc);
        }
        j = j2;
    }
}

// Partials cross workgroups (and XCDs, whose L2 caches are not coherent with each other) inside one
// launch, so they are written and read with device-scope relaxed atomics, which go to the coherent
// level of the memory system, instead of a device-scope fence, which would write back and invalidate
// the whole L2 on every call.
__device__ __forceinline__ void part_store(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float part_load(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

// Merges the 4 * (64/LPR) lane groups of a workgroup through LDS and writes {M, L, acc[hs]} to `out`, or, when
// this workgroup saw every cached row (yfinal set), the normalised result straight to yfinal.  With plainAcc set the
// partial is meant for the NEXT kernel of the stream, which merges the splits itself: {M, L} go to `out` and acc[hs] to
// plainAcc with ordinary stores (the kernel boundary makes them visible).
template <typename T, int LPR, typename TY = T>
__device__ __forceinline__ void decode_reduce_wg(float m, float l, const float (&acc)[Vec16<T>::W], int wave, int grp, int gl,
                                                 int d0, bool active, int hs, float* __restrict__ out, TY* __restrict__ yfinal = nullptr,
                                                 float* __restrict__ plainAcc = nullptr)
{
    constexpr int W = Vec16<T>::W;
    constexpr int RPW = 64 / LPR, NW = 4;
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
    constexpr int NG = NW * RPW;
    if constexpr (NG <= 32) {
        // Every LDS read is unconditional and the group weights are computed once, side by side: with the reads under
        // `if (sm[i] > -inf)` the compiler emits one branch and one LDS round trip after the other.  An empty group has
        // weight 0 and a zero accumulator, so the sums are those of the loop form below, term for term.
        float w[NG], M = -INFINITY, L = 0.f;
#pragma unroll
        for (int i = 0; i < NG; i++) { w[i] = sm[i]; M = fmaxf(M, w[i]); }
#pragma unroll
        for (int i = 0; i < NG; i++) w[i] = w[i] > -INFINITY ? __expf(w[i] - M) : 0.f;
        if (yfinal || threadIdx.x == 0) {
#pragma unroll
            for (int i = 0; i < NG; i++) L += sl[i] * w[i];
        }
        if (!yfinal && threadIdx.x == 0) {
            if (plainAcc) { out[0] = M; out[1] = L; }
            else { part_store(out, M); part_store(out + 1, L); }
        }
        for (int d = threadIdx.x; d < hs; d += 256) {
            float v = 0.f;
#pragma unroll
            for (int i = 0; i < NG; i++) v += sacc[i][d] * w[i];
            if (yfinal) st1(yfinal + d, v / L);
            else if (plainAcc) plainAcc[d] = v;
            else part_store(out + 2 + d, v);
        }
        return;
    }
    float M = -INFINITY;
    for (int i = 0; i < NW * RPW; i++) M = fmaxf(M, sm[i]);
    if (yfinal) {
        float L = 0.f;
        for (int i = 0; i < NW * RPW; i++) L += (sm[i] > -INFINITY) ? sl[i] * __expf(sm[i] - M) : 0.f;
        for (int d = threadIdx.x; d < hs; d += 256) {
            float v = 0.f;
            for (int i = 0; i < NW * RPW; i++)
                if (sm[i] > -INFINITY) v += sacc[i][d] * __expf(sm[i] - M);
            st1(yfinal + d, v / L);
        }
        return;
    }
    if (threadIdx.x == 0) {
        float L = 0.f;
        for (int i = 0; i < NW * RPW; i++) L += (sm[i] > -INFINITY) ? sl[i] * __expf(sm[i] - M) : 0.f;
        if (plainAcc) { out[0] = M; out[1] = L; }
        else { part_store(out, M); part_store(out + 1, L); }
    }
    for (int d = threadIdx.x; d < hs; d += 256) {
        float v = 0.f;
        for (int i = 0; i < NW * RPW; i++)
            if (sm[i] > -INFINITY) v += sacc[i][d] * __expf(sm[i] - M);
        if (plainAcc) plainAcc[d] = v;
        else part_store(out + 2 + d, v);
    }
}

// The workgroup that takes the last ticket of a (batch, head) merges all split partials (splits <= 256,
// 256 threads).  Every wavefront waits for its own partial stores to be acknowledged before the barrier
// that precedes the ticket, so a workgroup that sees ticket == splits - 1 can read every partial.
template <typename T>
__device__ __forceinline__ void decode_merge_last(const float* part, int* counter, int splits, int hs, T* __restrict__ y)
{
    __shared__ int ticket;
    __shared__ float sM[256], sL[256], sA[256];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) ticket = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket != splits - 1) return;
    // One round trip: thread (g, d) merges splits g, g + G, ... for output dimension d with its own running
    // maximum, four splits' {m, l, value} loads in flight at a time; the G groups then meet in LDS.
    const int tid = threadIdx.x;
    const int stride = hs + 2;
    const int G = hs >= 256 ? 1 : 256 / hs;
    const int g = tid / hs;
    for (int dbase = 0; dbase < hs; dbase += 256) {
        const int d = dbase + tid - g * hs;
        const bool mine = g < G && d < hs;
        float M = -INFINITY, L = 0.f, A = 0.f;
        for (int s0 = g; s0 < splits && mine; s0 += 4 * G) {
            float ms[4], ls[4], vs[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int sp = s0 + k * G;
                const bool ok = sp < splits;
                const float* p = part + (size_t)(ok ? sp : s0) * stride;
                ms[k] = part_load(p);
                ls[k] = part_load(p + 1);
                vs[k] = part_load(p + 2 + d);
                if (!ok) ms[k] = -INFINITY;
            }
            float Mn = fmaxf(fmaxf(fmaxf(M, ms[0]), fmaxf(ms[1], ms[2])), ms[3]);
            if (Mn > -INFINITY) {
                const float c = __expf(M - Mn);   // M == -inf gives 0
                L *= c;
                A *= c;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float w = ms[k] > -INFINITY ? __expf(ms[k] - Mn) : 0.f;
                    L += ls[k] * w;
                    A += vs[k] * w;
                }
                M = Mn;
            }
        }
        if (G == 1) {
            if (mine) st1(y + d, A / L);
        } else {
            sM[tid] = M; sL[tid] = L; sA[tid] = A;
            __syncthreads();
            if (g == 0 && d < hs) {
                for (int k = 1; k < G; k++) {
                    const float m2 = sM[k * hs + d];
                    if (m2 > -INFINITY) {
                        const float Mn = fmaxf(M, m2), c1 = __expf(M - Mn), c2 = __expf(m2 - Mn);
                        L = L * c1 + sL[k * hs + d] * c2;
                        A = A * c1 + sA[k * hs + d] * c2;
                        M = Mn;
                    }
                }
                st1(y + d, A / L);
            }
        }
    }
    if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
}

// The same for head sizes up to 64, where the first wavefront alone wrote the workgroup's partial (decode_reduce_wg: thread
// d stores dimension d): it waits for its own stores, takes the ticket and, if it is the last one, merges with one lane
// per dimension and sixteen splits' loads in flight - no workgroup barrier and no LDS on the way.  The other wavefronts
// are done.
template <typename T>
__device__ __forceinline__ void decode_merge_last_wave(const float* part, int* counter, int splits, int hs, T* __restrict__ y)
{
    if (threadIdx.x >= 64) return;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    int ticket = 0;
    if (threadIdx.x == 0) ticket = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __builtin_amdgcn_readfirstlane(ticket);
    if (ticket != splits - 1) return;
    const int d = threadIdx.x < hs ? threadIdx.x : 0;
    const int stride = hs + 2;
    constexpr int NS = 16;
    float M = -INFINITY, L = 0.f, A = 0.f;
    for (int s0 = 0; s0 < splits; s0 += NS) {
        float ms[NS], ls[NS], vs[NS];
#pragma unroll
        for (int k = 0; k < NS; k++) {
            const bool ok = s0 + k < splits;
            const float* p = part + (size_t)(ok ? s0 + k : s0) * stride;
            ms[k] = part_load(p);
            ls[k] = part_load(p + 1);
            vs[k] = part_load(p + 2 + d);
            if (!ok) ms[k] = -INFINITY;
        }
        float Mn = M;
#pragma unroll
        for (int k = 0; k < NS; k++) Mn = fmaxf(Mn, ms[k]);
        if (Mn > -INFINITY) {
            const float c = __expf(M - Mn);   // M == -inf gives 0
            L *= c;
            A *= c;
#pragma unroll
            for (int k = 0; k < NS; k++) {
                const float w = ms[k] > -INFINITY ? __expf(ms[k] - Mn) : 0.f;
                L += ls[k] * w;
                A += vs[k] * w;
            }
            M = Mn;
        }
    }
    if ((int)threadIdx.x < hs) st1(y + threadIdx.x, A / L);
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
}

template <typename T>
__device__ __forceinline__ void decode_merge(const float* part, int* counter, int splits, int hs, T* __restrict__ y)
{
    if (hs <= 64) decode_merge_last_wave<T>(part, counter, splits, hs, y);
    else decode_merge_last<T>(part, counter, splits, hs, y);
}

// partial layout: part[((b*H + h)*splits + s) * (hs + 2)] = {m, l, acc[hs]}
template <typename T, int LPR>
__global__ __launch_bounds__(256) void attn_decode_kernel(DecodeArgs a)
{
    constexpr int W = Vec16<T>::W;
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
    // splits that hold rows: with a device-side length the launch is sized for the longest cache and the rest idle
    int nAct = a.splits;
    if (a.dlen) {
        const int len = *a.dlen;
        int chunk = (len + a.splits - 1) / a.splits;
        chunk = ((chunk + a.rowsPerIter - 1) / a.rowsPerIter) * a.rowsPerIter;
        nAct = (len + chunk - 1) / chunk;
        if (a.counters && split >= nAct) return;
    }

    float m = -INFINITY, l = 0.f, acc[W];
#pragma unroll
    for (int i = 0; i < W; i++) acc[i] = 0.f;
    decode_stream<T, LPR>(kc, vc, a.strideT, t0, t1, (unsigned)((b * a.H + h) * 37 + split * 11), wave, grp, d0, active, qv, m, l, acc);

    const size_t bh = (size_t)b * a.H + h;
    float* out = a.part + (bh * a.splits + split) * (a.hs + 2);
    if (a.counters && nAct == 1) {
        decode_reduce_wg<T, LPR>(m, l, acc, wave, grp, gl, d0, active, a.hs, out, (T*)a.y + bh * a.hs);
        return;
    }
    decode_reduce_wg<T, LPR>(m, l, acc, wave, grp, gl, d0, active, a.hs, out);
    if (a.counters)
        decode_merge<T>(a.part + bh * a.splits * (a.hs + 2), a.counters + bh, nAct, a.hs, (T*)a.y + bh * a.hs);
}

// Engine form (fp32): one launch per layer does what the reference's decode step does between the QKV
// mat-vecs and the output projection (llama2_cpu.cpp:288-341): rotate q and k at the current position,
// store k and v into the cache, attend over positions 0..pos, write the head outputs.  qkv holds one
// row [q | k | v] of dim + 2*kvd raw projections per sequence; caches are [B][seqLen][kvd].
struct FusedDecodeArgs {
    const float* qkv; void* kc; void* vc; float* y; float* part; int* counters;
    const float* fcos; const float* fsin; const int* dlen;
    int B, H, kvMul, hs, dim, kvd, seqLen, splits, rowsPerIter;
    float scale;
    bool oneIter;   // seqLen <= splits * rowsPerIter: a split never holds more than one iteration of rows
    // B == 1 and oneIter only: leave the merge of the splits to the next kernel.  Split s of head h writes its
    // accumulator to part[s * dim + h * hs ..] and {m, l} to part[splits * dim + (s * H + h) * 2 ..]; y is not written.
    bool deferMerge;
};

// TC: storage type of the caches (fp32, or bf16: the rotated key and the value are rounded when they are appended, and the
// step that appends them attends over the rounded row as well, so a position is seen the same way by every later step).
// Activations (q, the head outputs) stay fp32; a lane owns the W = 16 bytes / sizeof(TC) dimensions d0 .. d0 + W - 1.
template <int LPR, typename TC>
__global__ __launch_bounds__(256) void attn_decode_fused_kernel(FusedDecodeArgs a)
{
    constexpr int W = Vec16<TC>::W;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane / LPR, gl = lane % LPR;
    const int d0 = gl * W;
    const bool active = d0 < a.hs;
    const int len = *a.dlen, pos = len - 1;
    const int half = a.hs / 2;
    const int kvh = h / a.kvMul;
    const int ldq = a.dim + 2 * a.kvd;
    const float* row = a.qkv + (size_t)b * ldq;
    TC* kc = (TC*)a.kc + (size_t)b * a.seqLen * a.kvd + (size_t)kvh * a.hs;
    TC* vc = (TC*)a.vc + (size_t)b * a.seqLen * a.kvd + (size_t)kvh * a.hs;
    auto load_row = [&](const float* p, float* o) {
#pragma unroll
        for (int j = 0; j < W / 4; j++) {
            const float4 t = *(const float4*)(p + 4 * j);
            o[4 * j] = t.x; o[4 * j + 1] = t.y; o[4 * j + 2] = t.z; o[4 * j + 3] = t.w;
        }
    };
    // rotation factors of this lane's adjacent pairs (dims d0 + 2 j, d0 + 2 j + 1) at `pos`
    float cs[W / 2], sn[W / 2];
    auto load_factors = [&]() {
#pragma unroll
        for (int j = 0; j < W / 2; j++) { cs[j] = 1.f; sn[j] = 0.f; }
        if (active) {
            const size_t ti = (size_t)pos * half + d0 / 2;
#pragma unroll
            for (int j = 0; j < W / 2; j++) { cs[j] = a.fcos[ti + j]; sn[j] = a.fsin[ti + j]; }
        }
    };
    auto rotate = [&](const float* in, float* out, float scale) {
#pragma unroll
        for (int j = 0; j < W / 2; j++) {
            out[2 * j] = (in[2 * j] * cs[j] - in[2 * j + 1] * sn[j]) * scale;
            out[2 * j + 1] = (in[2 * j] * sn[j] + in[2 * j + 1] * cs[j]) * scale;
        }
    };
    auto rotate_key = [&](const float* in, float* out) {
#pragma unroll
        for (int j = 0; j < W / 2; j++) {
            out[2 * j] = in[2 * j] * cs[j] - in[2 * j + 1] * sn[j];
            out[2 * j + 1] = in[2 * j] * sn[j] + in[2 * j + 1] * cs[j];
        }
    };

    int chunk = (len + a.splits - 1) / a.splits;
    chunk = ((chunk + a.rowsPerIter - 1) / a.rowsPerIter) * a.rowsPerIter;
    const int t0 = split * chunk, t1 = min(len, t0 + chunk);
    const int nAct = (len + chunk - 1) / chunk;      // splits that hold rows; the rest of the launch idles
    if (split >= nAct) return;

    load_factors();
    float qv[W];
#pragma unroll
    for (int i = 0; i < W; i++) qv[i] = 0.f;
    if (active) {
        float r[W];
        load_row(row + (size_t)h * a.hs + d0, r);
        rotate(r, qv, a.scale);
    }
    // the split that owns the current position appends the rotated key and the value first
    if (t0 <= pos && pos < t1) {
        if (wave == 0 && grp == 0 && active) {
            float kr[W], vr[W], ko[W];
            load_row(row + a.dim + (size_t)kvh * a.hs + d0, kr);
            load_row(row + a.dim + a.kvd + (size_t)kvh * a.hs + d0, vr);
            rotate_key(kr, ko);
            *(u32x4*)(kc + (size_t)pos * a.kvd + d0) = Vec16<TC>::pack(ko);
            *(u32x4*)(vc + (size_t)pos * a.kvd + d0) = Vec16<TC>::pack(vr);
        }
        __syncthreads();   // the row is read back by this workgroup only (other heads of the group write their own copy)
    }
    float m = -INFINITY, l = 0.f, acc[W];
#pragma unroll
    for (int i = 0; i < W; i++) acc[i] = 0.f;
    decode_stream<TC, LPR>(kc, vc, a.kvd, t0, t1, (unsigned)((b * a.H + h) * 37 + split * 11), wave, grp, d0, active, qv, m, l, acc);
    const size_t bh = (size_t)b * a.H + h;
    float* out = a.part + (bh * a.splits + split) * (a.hs + 2);
    float* yout = a.y + (size_t)b * a.dim + (size_t)h * a.hs;
    if (nAct == 1) {
        decode_reduce_wg<TC, LPR, float>(m, l, acc, wave, grp, gl, d0, active, a.hs, out, yout);
        return;
    }
    decode_reduce_wg<TC, LPR, float>(m, l, acc, wave, grp, gl, d0, active, a.hs, out);
    decode_merge<float>(a.part + bh * a.splits * (a.hs + 2), a.counters + bh, nAct, a.hs, yout);
}

// The engine form when the whole cache fits one iteration per split (seqLen <= splits * rowsPerIter): a kernel of its
// own so that the order of its memory requests is the one written here.
template <int LPR, typename TC>
__global__ __launch_bounds__(256) void attn_decode_fused_step_kernel(FusedDecodeArgs a)
{
    constexpr int W = Vec16<TC>::W;
    const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane / LPR, gl = lane % LPR;
    const int d0 = gl * W;
    const bool active = d0 < a.hs;
    const int half = a.hs / 2;
    const int kvh = h / a.kvMul;
    const int ldq = a.dim + 2 * a.kvd;
    const float* row = a.qkv + (size_t)b * ldq;
    TC* kc = (TC*)a.kc + (size_t)b * a.seqLen * a.kvd + (size_t)kvh * a.hs;
    TC* vc = (TC*)a.vc + (size_t)b * a.seqLen * a.kvd + (size_t)kvh * a.hs;
    auto load_row = [&](const float* p, float* o) {
#pragma unroll
        for (int j = 0; j < W / 4; j++) {
            const float4 t = *(const float4*)(p + 4 * j);
            o[4 * j] = t.x; o[4 * j + 1] = t.y; o[4 * j + 2] = t.z; o[4 * j + 3] = t.w;
        }
    };
    float cs[W / 2], sn[W / 2];   // rotation factors of this lane's adjacent pairs (dims d0 + 2 j, d0 + 2 j + 1) at `pos`
    auto rotate = [&](const float* in, float* out, float scale) {
#pragma unroll
        for (int j = 0; j < W / 2; j++) {
            out[2 * j] = (in[2 * j] * cs[j] - in[2 * j + 1] * sn[j]) * scale;
            out[2 * j + 1] = (in[2 * j] * sn[j] + in[2 * j + 1] * cs[j]) * scale;
        }
    };
    auto rotate_key = [&](const float* in, float* out) {
#pragma unroll
        for (int j = 0; j < W / 2; j++) {
            out[2 * j] = in[2 * j] * cs[j] - in[2 * j + 1] * sn[j];
            out[2 * j + 1] = in[2 * j] * sn[j] + in[2 * j + 1] * cs[j];
        }
    };
    // The whole cache fits one iteration per split.  Everything that does not depend on the length is requested at
    // once, before the length is looked at: the query, the new key / value and this split's cache rows (rows past
    // the end of the cache clamped; rows past the length are masked afterwards).  All loads are unconditional -
    // lanes past the head size read column 0 - because loads under a branch make the compiler wait for every
    // outstanding load at the first use of any.  The rotation factors follow as soon as the length is known, and
    // the row at `pos` (which the cache does not hold yet) is patched in registers instead of being stored and
    // read back.  Arithmetic and its order are those of attn_decode_fused_kernel.
    constexpr int RPW = 64 / LPR, U = 4, STEP = 4 * RPW * U;
    const int t0 = split * STEP;
    const int tb = t0 + wave * RPW * U;
    const int dc = active ? d0 : 0;
    float r[W], kr[W], vr[W];
    load_row(row + (size_t)h * a.hs + dc, r);
    load_row(row + a.dim + (size_t)kvh * a.hs + dc, kr);
    load_row(row + a.dim + a.kvd + (size_t)kvh * a.hs + dc, vr);
    DecodeStage<U> A;
#pragma unroll
    for (int u = 0; u < U; u++) A.k[u] = *(const u32x4*)(kc + (size_t)min(tb + u * RPW + grp, a.seqLen - 1) * a.kvd + dc);
#pragma unroll
    for (int u = 0; u < U; u++) A.v[u] = *(const u32x4*)(vc + (size_t)min(tb + u * RPW + grp, a.seqLen - 1) * a.kvd + dc);
    __builtin_amdgcn_sched_barrier(0);   // the requests above are issued before the length is asked for
    const int len = *a.dlen, pos = len - 1;
    const int nAct = (len + STEP - 1) / STEP;
    if (split >= nAct) return;
    const int t1 = min(len, t0 + STEP);
    {
        const size_t ti = (size_t)pos * half + dc / 2;
#pragma unroll
        for (int j = 0; j < W / 2; j++) { cs[j] = a.fcos[ti + j]; sn[j] = a.fsin[ti + j]; }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!active) {
#pragma unroll
        for (int i = 0; i < W; i++) r[i] = 0.f;
    }
    float qv[W];
    rotate(r, qv, a.scale);
    // rows past the length hold whatever the cache memory holds: their scores are masked when they are consumed,
    // their values are cleared here (0 x NaN would not be 0)
#pragma unroll
    for (int u = 0; u < U; u++) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        if (tb + u * RPW + grp >= t1) A.v[u] = z;
    }
    if (t0 <= pos && pos < t1) {
        float ko[W];
        rotate_key(kr, ko);
        const u32x4 kb = Vec16<TC>::pack(ko), vb = Vec16<TC>::pack(vr);
        if (wave == 0 && grp == 0 && active) {
            *(u32x4*)(kc + (size_t)pos * a.kvd + d0) = kb;
            *(u32x4*)(vc + (size_t)pos * a.kvd + d0) = vb;
        }
#pragma unroll
        for (int u = 0; u < U; u++)
            if (tb + u * RPW + grp == pos) { A.k[u] = kb; A.v[u] = vb; }   // every lane: none keeps what the cache held
    }
    float m = -INFINITY, l = 0.f, acc[W];
#pragma unroll
    for (int i = 0; i < W; i++) acc[i] = 0.f;
    decode_consume<TC, LPR, U>(A, tb, t1, grp, qv, m, l, acc);
    if (a.deferMerge) {
        decode_reduce_wg<TC, LPR, float>(m, l, acc, wave, grp, gl, d0, active, a.hs,
                                         a.part + (size_t)a.splits * a.dim + ((size_t)split * a.H + h) * 2, (float*)nullptr,
                                         a.part + (size_t)split * a.dim + (size_t)h * a.hs);
        return;
    }
    const size_t bh = (size_t)b * a.H + h;
    float* out = a.part + (bh * a.splits + split) * (a.hs + 2);
    float* yout = a.y + (size_t)b * a.dim + (size_t)h * a.hs;
    if (nAct == 1) {
        decode_reduce_wg<TC, LPR, float>(m, l, acc, wave, grp, gl, d0, active, a.hs, out, yout);
        return;
    }
    decode_reduce_wg<TC, LPR, float>(m, l, acc, wave, grp, gl, d0, active, a.hs, out);
    decode_merge<float>(a.part + bh * a.splits * (a.hs + 2), a.counters + bh, nAct, a.hs, yout);
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

// Workgroups a launch aims for: one per CU.  More splits per (batch, head) shorten each workgroup's stream but add
// partials to store, count and merge, which costs more than it saves from 8 sequences x 32 heads down (measured: 256
// against 1024 gains up to 20 % at batch 1 and a few per cent at batch 8, and changes nothing at batch 32).
constexpr int kDecodeTargetWgs = 256;
// The engine's fused kernel is content with half the CUs once the (sequence, head) pairs alone reach that many: a single
// split per pair needs no merge at all, and at 16 sequences x 12 heads that is worth more than a second split's
// bandwidth (27.5k -> 27.9k tokens/s).  Fewer pairs keep the usual target.
static int fused_target(int B, int H) { return (long long)B * H >= 128 ? 128 : kDecodeTargetWgs; }
static void pick_splits(int B, int H, int len, int rows_per_iter, int* splits, int* chunk, int target = kDecodeTargetWgs)
{
    // never less than one full iteration per split
    long long bh = (long long)B * H;
    int want = (int)((target + bh - 1) / bh);
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
    // pick_splits never asks for more than ceil(256 / (B*H)) splits
    (void)len;
    long long bh = (long long)B * H;
    long long want = (kDecodeTargetWgs + bh - 1) / bh;   // (the fused kernel's smaller target asks for fewer)
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
    if (fast && a.counters) return hipSuccess;   // the last workgroup of every (batch, head) merged in-kernel
    int mt = a.hs <= 64 ? 64 : (a.hs <= 128 ? 128 : 256);
    hipLaunchKernelGGL(attn_decode_merge_kernel<T>, a.B * a.H, mt, 0, s, a.part, (T*)a.y, a.hs, a.splits);
    return hipGetLastError();
}

hipError_t k_attn_decode(hipStream_t s, DType dt, const void* q, const void* kc, const void* vc, void* y, int B, int H,
                         int kvH, int hs, int len, long long strideB, long long strideH, long long strideT, float scale,
                         void* workspace, size_t workspaceBytes, const int* dlen, int* counters)
{
    if (B <= 0 || H <= 0 || hs <= 0 || len <= 0) return hipSuccess;
    if (kvH <= 0 || H % kvH != 0) return hipErrorInvalidValue;
    if (B > 65535 || H > 65535) return hipErrorInvalidValue;
    if (workspaceBytes < attn_decode_workspace_bytes(B, H, hs, len)) return hipErrorInvalidValue;
    DecodeArgs a;
    a.q = q; a.kc = kc; a.vc = vc; a.y = y; a.part = (float*)workspace;
    a.B = B; a.H = H; a.kvMul = H / kvH; a.hs = hs; a.len = len; a.splits = 1; a.chunk = len;
    a.strideB = strideB; a.strideH = strideH; a.strideT = strideT; a.scale = scale;
    a.dlen = dlen; a.rowsPerIter = 64; a.counters = counters;
    if (dt == F32) return launch_decode<float>(s, a, kvH);
    return launch_decode<bf16_t>(s, a, kvH);
}

// The splits of a launch that leaves the merge to the next kernel (batch 1, the whole cache in one iteration per split), and
// the rows each of them covers; 0 when the launch cannot be of that kind.
int attn_decode_fused_deferred_splits(int B, int H, int hs, int seqLen, DType cacheType, int* rowsPerSplit)
{
    const int W = cacheType == F32 ? 4 : 8;
    if (B != 1 || H <= 0 || hs <= 0 || hs % W != 0 || seqLen <= 0) return 0;
    int lpr = hs / W, lprp = 1;
    while (lprp < lpr) lprp <<= 1;
    if (lprp > 64) return 0;
    const int rpi = 4 * (64 / lprp) * 4;
    int splits, chunk;
    pick_splits(B, H, seqLen, rpi, &splits, &chunk, fused_target(B, H));
    if (seqLen > splits * rpi) return 0;
    if (rowsPerSplit) *rowsPerSplit = rpi;
    return splits;
}

hipError_t k_attn_decode_fused(hipStream_t s, const float* qkv, void* kc, void* vc, DType cacheType, float* y, int B, int H, int kvH,
                               int hs, int seqLen, float scale, const float* fcos, const float* fsin, const int* dlen, void* workspace,
                               size_t workspaceBytes, int* counters, bool deferMerge)
{
    if (B <= 0 || H <= 0 || hs <= 0 || seqLen <= 0) return hipSuccess;
    const int W = cacheType == F32 ? 4 : 8;   // elements per 16-byte cache chunk
    if (kvH <= 0 || H % kvH != 0 || (hs % W) != 0 || B > 65535 || H > 65535 || !counters || !dlen) return hipErrorInvalidValue;
    int lpr = hs / W, lprp = 1;
    while (lprp < lpr) lprp <<= 1;
    if (lprp > 64) return hipErrorInvalidValue;
    if (workspaceBytes < attn_decode_workspace_bytes(B, H, hs, seqLen)) return hipErrorInvalidValue;
    FusedDecodeArgs a;
    a.qkv = qkv; a.kc = kc; a.vc = vc; a.y = y; a.part = (float*)workspace; a.counters = counters;
    a.fcos = fcos; a.fsin = fsin; a.dlen = dlen;
    a.B = B; a.H = H; a.kvMul = H / kvH; a.hs = hs; a.dim = H * hs; a.kvd = kvH * hs; a.seqLen = seqLen;
    a.rowsPerIter = 4 * (64 / lprp) * 4;
    int chunk;
    pick_splits(B, H, seqLen, a.rowsPerIter, &a.splits, &chunk, fused_target(B, H));
    a.scale = scale;
    a.oneIter = seqLen <= a.splits * a.rowsPerIter;
    a.deferMerge = deferMerge;
    if (deferMerge && (B != 1 || !a.oneIter)) return hipErrorInvalidValue;
    dim3 grid(a.splits, H, B);
    switch (lprp) {
#define CASE(L)                                                                                                            \
    case L:                                                                                                                \
        if (a.oneIter) {                                                                                                   \
            if (cacheType == F32) hipLaunchKernelGGL((attn_decode_fused_step_kernel<L, float>), grid, 256, 0, s, a);       \
            else hipLaunchKernelGGL((attn_decode_fused_step_kernel<L, bf16_t>), grid, 256, 0, s, a);                       \
        } else if (cacheType == F32) hipLaunchKernelGGL((attn_decode_fused_kernel<L, float>), grid, 256, 0, s, a);         \
        else hipLaunchKernelGGL((attn_decode_fused_kernel<L, bf16_t>), grid, 256, 0, s, a);                                \
        break;
        CASE(1) CASE(2) CASE(4) CASE(8) CASE(16) CASE(32) CASE(64)
#undef CASE
    }
    return hipGetLastError();
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
