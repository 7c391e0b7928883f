// Micro-benchmarks of the gfx950 properties that the kernel designs of this library rest on.  Each prints one line per
// case; none of them touches the library.  Build: mycaffe_amd/build.py; run: mycaffe_amd/host_bench/hw_probes [section]
// with section in {overlap, lds, graph, persist, stage} (default: all).
//   overlap  how much vector-ALU work a wavefront can hide behind its own MFMAs (plain fma and v_exp_f32)
//   lds      rate of the LDS fragment reads of the attention and GEMM kernels (ds_read_b128 in the K-fragment pattern,
//            the transposing ds_read_b64_tr_b16 in the row-major V pattern) alone and with one MFMA per fragment
//   graph    cost of a kernel boundary inside a replayed HIP graph and of a bare mat-vec kernel at several working sets
//   persist  the same mat-vec chain as one cooperative kernel with bounded grid barriers, with and without the next
//            phase's weights requested across the barrier
//   stage    what the GEMM kernels' operand staging can draw from the caches: where the lanes of a direct global-to-LDS
//            load (global_load_lds_dwordx4) land, and the rate at which all CUs together stream 16-byte loads out of
//            their die's L2 and out of the last-level cache, into registers and straight into LDS
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

#define CK(x)                                                                                                              \
    do {                                                                                                                   \
        hipError_t e_ = (x);                                                                                               \
        if (e_ != hipSuccess) {                                                                                            \
            printf("HIP error %d (%s) at line %d\n", (int)e_, hipGetErrorString(e_), __LINE__);                            \
            return 1;                                                                                                      \
        }                                                                                                                  \
    } while (0)

// ---- overlap: one wavefront per SIMD; per group one MFMA followed by NV vector instructions, order pinned -------------
// MODE 0: MFMAs only; 1: vector instructions only; 2: interleaved
template <int MODE, int NV, bool EXP> __global__ __launch_bounds__(256) void overlap_kernel(float* out, int iters)
{
    floatx16 acc[4];
    for (int j = 0; j < 4; j++)
        for (int i = 0; i < 16; i++) acc[j][i] = 0.f;
    uint4 u = {threadIdx.x, 1, 2, 3};
    bf16x8 a = *reinterpret_cast<bf16x8*>(&u), b = a;
    float f[16];
    for (int i = 0; i < 16; i++) f[i] = threadIdx.x * 0.001f + i * 0.01f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (MODE != 1) acc[g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[g], 0, 0, 0);
            if (MODE != 0) {
#pragma unroll
                for (int i = 0; i < NV; i++) {
                    const int q = (g * NV + i) & 15;
                    if (EXP) f[q] = __builtin_amdgcn_exp2f(f[q]);
                    else f[q] = __builtin_fmaf(f[q], 1.0001f, 0.5f);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0;
    for (int i = 0; i < 16; i++) s += f[i] + acc[0][i] + acc[1][i] + acc[2][i] + acc[3][i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <int MODE, int NV, bool EXP> static int run_overlap(const char* name, float* d)
{
    const int iters = 20000;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    hipLaunchKernelGGL((overlap_kernel<MODE, NV, EXP>), 256, 256, 0, 0, d, 10);
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((overlap_kernel<MODE, NV, EXP>), 256, 256, 0, 0, d, iters);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    printf("overlap  %-34s %7.1f ns per group of four\n", name, ms * 1e6 / iters);
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return 0;
}

// ---- lds: fragment reads of a 64 KB tile, eight per iteration and wavefront ---------------------------------------------
// MODE 0: ds_read_b128, lane reads 16 bytes of row lane % 32 (row stride LD bytes), column half lane / 32
// MODE 1: two ds_read_b64_tr_b16 in the row-major V^T pattern (four rows of 32 bytes per 16 lanes)
// MODE 2: MODE 0 with one MFMA per fragment, the fragment as its operand
template <int MODE, int LD> __global__ __launch_bounds__(512) void lds_kernel(unsigned* out, int iters)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 65536 / 4; i += blockDim.x) ((unsigned*)lds)[i] = i * 2654435761u;
    __syncthreads();
    u32x4 acc = {0, 0, 0, 0};
    floatx16 c;
    for (int i = 0; i < 16; i++) c[i] = 0.f;
    int off;
    if (MODE == 1) {
        const int i = lane & 15, half = lane >> 5;
        off = (4 * half + (i >> 2)) * LD + (16 * ((lane >> 4) & 1) + 4 * (i & 3)) * 2;
    } else {
        off = (lane & 31) * LD + (lane >> 5) * 16;
    }
    off += wave * 64;
    for (int it = 0; it < iters; it++) {
        asm volatile("" : "+v"(off));   // keeps the reads inside the loop
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int o = (off + u * 32 + (it & 1) * 2048) & 65535 & ~15;
            if (MODE == 1) {
                const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(lds + o));
                const s16x4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(lds + o + 8 * LD));
                acc.x ^= (unsigned)a[0] ^ (unsigned)b[1];
                acc.y ^= (unsigned)a[2] ^ (unsigned)b[3];
            } else {
                const u32x4 v = *(const u32x4*)(lds + o);
                if (MODE == 2) {
                    const bf16x8 a = *(const bf16x8*)&v;
                    c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, a, c, 0, 0, 0);
                } else {
                    acc ^= v;
                }
            }
        }
    }
    unsigned s = acc.x ^ acc.y ^ acc.z ^ acc.w;
    for (int i = 0; i < 16; i++) s ^= __float_as_uint(c[i]);
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <int MODE, int LD> static int run_lds(const char* name, int threads, unsigned* d)
{
    const int iters = 4000;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    hipLaunchKernelGGL((lds_kernel<MODE, LD>), 256, threads, 65536, 0, d, 10);
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((lds_kernel<MODE, LD>), 256, threads, 65536, 0, d, iters);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double frags = (double)iters * 8 * (threads / 64);   // 1 KB fragments per CU
    printf("lds      %-52s %2d wavefronts/CU  %5.2f ns per 1 KB fragment per CU  (%4.0f B/ns/CU)\n", name, threads / 64, ms * 1e6 / frags,
           frags * 1024 / (ms * 1e6));
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return 0;
}

// ---- graph: kernel boundaries and bare mat-vec kernels inside a replayed graph ------------------------------------------
__global__ void noop_kernel(float* p)
{
    if (p && threadIdx.x == 1000) p[0] = 1.f;
}
// one wavefront per row of 768 floats: three 16-byte loads per lane, a wavefront reduction, one store
__global__ __launch_bounds__(256) void matvec_probe_kernel(const float4* __restrict__ w, const float* __restrict__ x, float* y, int rows)
{
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (wave >= rows) return;
    float4 a[3];
    for (int c = 0; c < 3; c++) a[c] = w[(size_t)wave * 192 + c * 64 + lane];
    float s = x[lane];
    for (int c = 0; c < 3; c++) s += a[c].x + a[c].y + a[c].z + a[c].w;
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    if (lane == 0) y[wave] = s;
}

// touches the same bytes as matvec_probe_kernel from the same workgroup index (same die, same L2) and keeps nothing
__global__ __launch_bounds__(256) void prefetch_probe_kernel(const float4* __restrict__ w, int rows)
{
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (wave >= rows) return;
    for (int c = 0; c < 3; c++) {
        float4 a = w[(size_t)wave * 192 + c * 64 + lane];
        asm volatile("" :: "v"(a.x), "v"(a.y), "v"(a.z), "v"(a.w));
    }
}

static int run_graph()
{
    hipStream_t s;
    CK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    float *x, *y, *big;
    const size_t matBytes = (size_t)2304 * 768 * 4;
    CK(hipMalloc(&x, 1 << 20));
    CK(hipMalloc(&y, 1 << 20));
    CK(hipMalloc(&big, 64 * matBytes));
    CK(hipMemset(x, 0, 1 << 20));
    CK(hipMemset(big, 0, 64 * matBytes));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    auto timeGraph = [&](int kernels, int reps, auto launch, float* usPerKernel) -> int {
        hipGraph_t g;
        hipGraphExec_t ge;
        CK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < kernels; i++) launch(i);
        CK(hipStreamEndCapture(s, &g));
        CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
        for (int r = 0; r < 5; r++) CK(hipGraphLaunch(ge, s));
        CK(hipStreamSynchronize(s));
        CK(hipEventRecord(e0, s));
        for (int r = 0; r < reps; r++) CK(hipGraphLaunch(ge, s));
        CK(hipEventRecord(e1, s));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        *usPerKernel = ms * 1e3f / reps / kernels;
        CK(hipGraphExecDestroy(ge));
        CK(hipGraphDestroy(g));
        return 0;
    };
    float us;
    if (timeGraph(62, 50, [&](int) { hipLaunchKernelGGL(noop_kernel, 1, 64, 0, s, (float*)nullptr); }, &us)) return 1;
    printf("graph    62 empty kernels of one wavefront                 %5.2f us per kernel\n", us);
    if (timeGraph(62, 50, [&](int) { hipLaunchKernelGGL(noop_kernel, 576, 256, 0, s, (float*)nullptr); }, &us)) return 1;
    printf("graph    62 empty kernels of 576 workgroups                %5.2f us per kernel\n", us);
    if (timeGraph(62, 50, [&](int i) { hipLaunchKernelGGL(matvec_probe_kernel, 192, 256, 0, s, (const float4*)big + (size_t)(i % 8) * 768 * 192, x, (i & 1) ? x : y, 768); }, &us)) return 1;
    printf("graph    62 mat-vec kernels 768 x 768 (2.4 MB each, 8 matrices)  %5.2f us per kernel\n", us);
    for (int nmat : {4, 8, 16, 32, 64}) {
        if (timeGraph(64, 30, [&](int i) { hipLaunchKernelGGL(matvec_probe_kernel, 576, 256, 0, s, (const float4*)big + (size_t)(i % nmat) * 2304 * 192, x, (i & 1) ? x : y, 2304); }, &us)) return 1;
        printf("graph    64 mat-vec kernels 2304 x 768 (7.1 MB each) cycling through %4.0f MB  %5.2f us per kernel\n", nmat * matBytes / 1e6, us);
    }
    // the same chain through all 64 matrices with a second branch of the graph that reads matrix i + ahead while kernel i
    // runs (the branch forks after kernel i - 1 and joins at the end of the graph)
    {
        hipStream_t s2;
        CK(hipStreamCreateWithFlags(&s2, hipStreamNonBlocking));
        hipEvent_t fork[64], join;
        for (int i = 0; i < 64; i++) CK(hipEventCreateWithFlags(&fork[i], hipEventDisableTiming));
        CK(hipEventCreateWithFlags(&join, hipEventDisableTiming));
        for (int ahead : {1, 2, 3}) {
            hipGraph_t g;
            hipGraphExec_t ge;
            CK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
            for (int i = 0; i < 64; i++) {
                if (i + ahead < 64) {
                    CK(hipEventRecord(fork[i], s));
                    CK(hipStreamWaitEvent(s2, fork[i], 0));
                    hipLaunchKernelGGL(prefetch_probe_kernel, 576, 256, 0, s2, (const float4*)big + (size_t)(i + ahead) * 2304 * 192, 2304);
                }
                hipLaunchKernelGGL(matvec_probe_kernel, 576, 256, 0, s, (const float4*)big + (size_t)i * 2304 * 192, x, (i & 1) ? x : y, 2304);
            }
            CK(hipEventRecord(join, s2));
            CK(hipStreamWaitEvent(s, join, 0));
            CK(hipStreamEndCapture(s, &g));
            CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
            for (int r = 0; r < 5; r++) CK(hipGraphLaunch(ge, s));
            CK(hipStreamSynchronize(s));
            CK(hipEventRecord(e0, s));
            for (int r = 0; r < 30; r++) CK(hipGraphLaunch(ge, s));
            CK(hipEventRecord(e1, s));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf("graph    64 mat-vec kernels 2304 x 768 cycling through  453 MB, matrix i + %d read on a parallel branch  %5.2f us per kernel\n",
                   ahead, ms * 1e3f / 30 / 64);
            CK(hipGraphExecDestroy(ge));
            CK(hipGraphDestroy(g));
        }
        CK(hipStreamDestroy(s2));
    }
    CK(hipFree(x));
    CK(hipFree(y));
    CK(hipFree(big));
    return 0;
}

// ---- persist: the same 62-phase mat-vec chain as ONE kernel with grid-wide barriers -------------------------------------
// 256 workgroups (one per CU, launched cooperatively so that all are resident), four computing wavefronts each.  A wavefront owns up
// to three rows of every 2304 x 768 matrix; it requests the NEXT phase's rows before it waits at the barrier, so the trip
// to HBM overlaps the barrier.  Barrier: arrive on one of 8 counters (workgroup index mod 8, i.e. per die), the last
// arrival of a die arrives on the global counter, the last of those releases one flag per die, which the die's workgroups poll.  Every wait is bounded: after
// `spinLimit` polls a workgroup sets the error flag, and once the flag is set nobody waits any more, so the kernel ends.
struct PersistArgs {
    const float4* w;        // matrices of 2304 x 192 float4, phase p uses matrix p % nmat
    float* xy;              // two vectors of 2304 floats (ping-pong); the first 768 of one are the next phase's input
    int* counters;          // [0..7] per-die arrivals, [8] global arrivals, [9] error flag, [32 + 16 d] release flag of die d; zero at launch
    int phases, nmat, spinLimit, prefetch;
};
__global__ __launch_bounds__(320) void persist_kernel(PersistArgs a)
{
    // wavefronts 0..3 compute; wavefront 4 only runs the barrier, so that its polls are not queued behind the weight
    // requests of a computing wavefront (memory operations of a wavefront complete in order)
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const bool worker = wv < 4;
    const int wave = blockIdx.x * 4 + wv;   // 1024 computing wavefronts
    const int die = blockIdx.x & 7;
    float4 cur[3][3], nxt[3][3];
    auto request = [&](int p, float4 (&r)[3][3]) {
        const float4* m = a.w + (size_t)(p % a.nmat) * 2304 * 192;
#pragma unroll
        for (int k = 0; k < 3; k++) {
            const int row = min(wave + 1024 * k, 2303);
#pragma unroll
            for (int c = 0; c < 3; c++) r[k][c] = m[(size_t)row * 192 + c * 64 + lane];
        }
    };
    if (worker) request(0, cur);
    for (int p = 0; p < a.phases; p++) {
        if (worker) {
            const float* x = a.xy + (p & 1) * 2304;
            float* y = a.xy + ((p + 1) & 1) * 2304;
            float4 xv[3];
#pragma unroll
            for (int c = 0; c < 3; c++) {
                const float* xp = x + (c * 64 + lane) * 4;
                xv[c].x = __hip_atomic_load(xp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                xv[c].y = __hip_atomic_load(xp + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                xv[c].z = __hip_atomic_load(xp + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                xv[c].w = __hip_atomic_load(xp + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int k = 0; k < 3; k++) {
                float s = 0.f;
#pragma unroll
                for (int c = 0; c < 3; c++)
                    s += cur[k][c].x * xv[c].x + cur[k][c].y * xv[c].y + cur[k][c].z * xv[c].z + cur[k][c].w * xv[c].w;
                for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
                const int row = wave + 1024 * k;
                if (lane == 0 && row < 2304) __hip_atomic_store(y + row, s * 1e-3f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wavefront's results have been acknowledged
        }
        if (p + 1 == a.phases) break;
        __syncthreads();   // all results of the workgroup are out
        if (worker) {
            if (a.prefetch) request(p + 1, nxt);   // in flight while the barrier wavefront waits
        } else if (lane == 0) {
            // arrive on the die's counter; the die's last arrival arrives on the global counter; the last of those
            // releases the eight per-die flags (one cache line each), which is what the workgroups poll: 32 pollers per
            // address instead of 256 (same-address accesses at this scope serialise)
            if (__hip_atomic_fetch_add(a.counters + die, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (p + 1) * 32 - 1) {
                if (__hip_atomic_fetch_add(a.counters + 8, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (p + 1) * 8 - 1) {
                    for (int d = 0; d < 8; d++) __hip_atomic_store(a.counters + 32 + 16 * d, p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            int spins = 0;
            while (__hip_atomic_load(a.counters + 32 + 16 * die, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < p + 1) {
                if ((++spins & 255) == 0 && __hip_atomic_load(a.counters + 9, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
                if (spins > a.spinLimit) {
                    __hip_atomic_store(a.counters + 9, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
        __syncthreads();   // the grid barrier has been passed (or given up)
        if (worker) {
            if (a.prefetch) {
#pragma unroll
                for (int k = 0; k < 3; k++)
#pragma unroll
                    for (int c = 0; c < 3; c++) cur[k][c] = nxt[k][c];
            } else {
                request(p + 1, cur);
            }
        }
    }
}

static int run_persist()
{
    int dev = 0, coop = 0, cus = 0;
    CK(hipGetDevice(&dev));
    CK(hipDeviceGetAttribute(&coop, hipDeviceAttributeCooperativeLaunch, dev));
    CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (!coop || cus < 256) {
        printf("persist  skipped (cooperative launch %d, CUs %d)\n", coop, cus);
        return 0;
    }
    hipStream_t s;
    CK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    const size_t matBytes = (size_t)2304 * 768 * 4;
    float *big, *xy;
    int* counters;
    CK(hipMalloc(&big, 64 * matBytes));
    CK(hipMalloc(&xy, 2 * 2304 * 4));
    CK(hipMalloc(&counters, 1024));
    CK(hipMemset(big, 0, 64 * matBytes));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int prefetch = 0; prefetch < 2; prefetch++) {
        for (int nmat : {4, 64}) {
            PersistArgs a = {(const float4*)big, xy, counters, 62, nmat, 1 << 20, prefetch};
            void* args[] = {&a};
            float best = 1e30f;
            int err = 0;
            for (int rep = 0; rep < 6; rep++) {
                CK(hipMemsetAsync(counters, 0, 1024, s));
                CK(hipMemsetAsync(xy, 0, 2 * 2304 * 4, s));
                CK(hipEventRecord(e0, s));
                CK(hipLaunchCooperativeKernel((const void*)persist_kernel, dim3(256), dim3(320), args, 0, s));
                CK(hipEventRecord(e1, s));
                CK(hipEventSynchronize(e1));
                float ms;
                CK(hipEventElapsedTime(&ms, e0, e1));
                int h[16];
                CK(hipMemcpy(h, counters, 64, hipMemcpyDeviceToHost));
                err |= h[9];
                if (rep > 0 && ms < best) best = ms;
            }
            printf("persist  62 phases of a 7.1 MB mat-vec in one kernel, weights cycling through %4.0f MB, next phase's rows %s: %5.2f us per phase%s\n",
                   nmat * matBytes / 1e6, prefetch ? "requested before the barrier" : "requested after the barrier ", best * 1e3 / 62,
                   err ? "  (a barrier wait hit its spin limit)" : "");
        }
    }
    CK(hipFree(big));
    CK(hipFree(xy));
    CK(hipFree(counters));
    return 0;
}


// ---- stage: direct global-to-LDS loads ---------------------------------------------------------------------------------
// placement: every thread loads 16 bytes of a counting pattern with four direct-to-LDS instructions; the workgroup then
// reads LDS back linearly.  If lane i of a wavefront lands 16 i bytes past the wavefront's (uniform) destination, LDS
// holds the pattern in order.
__global__ __launch_bounds__(256) void dma_place_kernel(const unsigned* __restrict__ g, unsigned* out)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char dsm[];
    const int wave = threadIdx.x >> 6;
    const unsigned* src = g + (size_t)threadIdx.x * 4;
#pragma unroll
    for (int p = 0; p < 4; p++)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + p * 1024),
                                         (__attribute__((address_space(3))) void*)(dsm + p * 4096 + wave * 1024), 16, 0, 0);
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
    __syncthreads();
    for (int i = threadIdx.x; i < 4096; i += 256) out[i] = ((const unsigned*)dsm)[i];
}

// rate: every workgroup streams from a region that belongs to its die (workgroup index mod 8); a region that fits the
// die's 4 MB L2 is served from it, a larger one from the last-level cache.  UNR 16-byte loads per thread in flight.
template <int UNR, bool DIRECT>
__global__ __launch_bounds__(256) void stage_rate_kernel(const unsigned* __restrict__ g, unsigned* out, size_t regionWords, int iters)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char dsm[];
    const int die = blockIdx.x % 8, idx = blockIdx.x / 8;
    const unsigned* base = g + (size_t)die * regionWords;
    const size_t chunkWords = 256 * 4 * UNR, nChunks = regionWords / chunkWords;
    u32x4 acc = {0, 0, 0, 0};
    for (int it = 0; it < iters; it++) {
        const unsigned* p = base + (((size_t)idx * 7 + it) % nChunks) * chunkWords + threadIdx.x * 4;
        if (DIRECT) {
#pragma unroll
            for (int u = 0; u < UNR; u++)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p + u * 1024),
                                                 (__attribute__((address_space(3))) void*)(dsm + (u * 4 + (threadIdx.x >> 6)) * 1024), 16, 0, 0);
        } else {
            u32x4 v[UNR];
#pragma unroll
            for (int u = 0; u < UNR; u++) v[u] = *(const u32x4*)(p + u * 1024);
#pragma unroll
            for (int u = 0; u < UNR; u++) acc ^= v[u];
        }
    }
    if (DIRECT) {
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        acc = *(const u32x4*)(dsm + threadIdx.x * 16);
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) out[0] = 1;   // keeps the loads alive
}

template <bool DIRECT> static int run_stage_rate(const unsigned* g, unsigned* out, size_t regionWords, int wgs)
{
    constexpr int UNR = 8;
    const int iters = 400, reps = 10;
    const size_t lds = DIRECT ? UNR * 4096 : 0;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int w = 0; w < 3; w++) hipLaunchKernelGGL((stage_rate_kernel<UNR, DIRECT>), wgs, 256, lds, 0, g, out, regionWords, iters);
    CK(hipEventRecord(e0));
    for (int r = 0; r < reps; r++) hipLaunchKernelGGL((stage_rate_kernel<UNR, DIRECT>), wgs, 256, lds, 0, g, out, regionWords, iters);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms = 0;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double bytes = (double)wgs * iters * 256 * 16 * UNR * reps;
    printf("stage    %-22s %4d workgroups, %5.1f MB per die: %6.2f TB/s (%5.1f GB/s per CU)\n", DIRECT ? "straight into LDS," : "into registers,", wgs,
           regionWords * 4 / 1e6, bytes / ms / 1e9, bytes / ms / 1e6 / 256);
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return 0;
}

static int run_stage()
{
    const size_t maxRegionWords = (size_t)16 << 20;   // 64 MB per die
    unsigned *g, *out;
    CK(hipMalloc(&g, maxRegionWords * 4 * 8));
    CK(hipMalloc(&out, 4096 * 4));
    {
        unsigned* h = (unsigned*)malloc(8192 * 4);
        for (int i = 0; i < 8192; i++) h[i] = (unsigned)i;
        CK(hipMemcpy(g, h, 8192 * 4, hipMemcpyHostToDevice));
        hipLaunchKernelGGL(dma_place_kernel, 1, 256, 16384, 0, g, out);
        CK(hipMemcpy(h, out, 4096 * 4, hipMemcpyDeviceToHost));
        int bad = 0;
        for (int i = 0; i < 4096; i++) bad += h[i] != (unsigned)i;
        printf("stage    global_load_lds_dwordx4: lane i of a wavefront lands 16 i bytes past the wavefront's LDS address: %s (%d of 4096 words differ)\n",
               bad ? "NO" : "yes", bad);
        free(h);
    }
    CK(hipMemset(g, 1, maxRegionWords * 4 * 8));
    for (size_t mb : {2, 16}) {
        const size_t rw = mb * 1024 * 1024 / 4;
        for (int wgs : {256, 512}) {
            if (run_stage_rate<false>(g, out, rw, wgs)) return 1;
            if (run_stage_rate<true>(g, out, rw, wgs)) return 1;
        }
    }
    CK(hipFree(g));
    CK(hipFree(out));
    return 0;
}

int main(int argc, char** argv)
{
    const char* sec = argc > 1 ? argv[1] : "all";
    const bool all = !strcmp(sec, "all");
    void* d;
    CK(hipMalloc(&d, 256 * 512 * 4 * 8));
    if (all || !strcmp(sec, "overlap")) {
        if (run_overlap<0, 0, false>("4 MFMA", (float*)d)) return 1;
        if (run_overlap<1, 4, false>("16 fma", (float*)d)) return 1;
        if (run_overlap<2, 4, false>("4 x (MFMA + 4 fma)", (float*)d)) return 1;
        if (run_overlap<1, 8, false>("32 fma", (float*)d)) return 1;
        if (run_overlap<2, 8, false>("4 x (MFMA + 8 fma)", (float*)d)) return 1;
        if (run_overlap<1, 12, false>("48 fma", (float*)d)) return 1;
        if (run_overlap<2, 12, false>("4 x (MFMA + 12 fma)", (float*)d)) return 1;
        if (run_overlap<1, 2, true>("8 exp2", (float*)d)) return 1;
        if (run_overlap<2, 2, true>("4 x (MFMA + 2 exp2)", (float*)d)) return 1;
        if (run_overlap<1, 4, true>("16 exp2", (float*)d)) return 1;
        if (run_overlap<2, 4, true>("4 x (MFMA + 4 exp2)", (float*)d)) return 1;
    }
    if (all || !strcmp(sec, "lds")) {
        for (int threads : {256, 512}) {
            if (run_lds<0, 272>("b128, K-fragment pattern, rows 272 B apart", threads, (unsigned*)d)) return 1;
            if (run_lds<0, 288>("b128, K-fragment pattern, rows 288 B apart", threads, (unsigned*)d)) return 1;
            if (run_lds<0, 144>("b128, K-fragment pattern, rows 144 B apart", threads, (unsigned*)d)) return 1;
            if (run_lds<1, 272>("2 x tr16_b64, row-major V pattern, rows 272 B apart", threads, (unsigned*)d)) return 1;
            if (run_lds<1, 288>("2 x tr16_b64, row-major V pattern, rows 288 B apart", threads, (unsigned*)d)) return 1;
            if (run_lds<1, 144>("2 x tr16_b64, row-major V pattern, rows 144 B apart", threads, (unsigned*)d)) return 1;
            if (run_lds<2, 272>("b128 fragment + one MFMA on it", threads, (unsigned*)d)) return 1;
        }
    }
    if (all || !strcmp(sec, "graph")) {
        if (run_graph()) return 1;
    }
    if (all || !strcmp(sec, "persist")) {
        if (run_persist()) return 1;
    }
    if (all || !strcmp(sec, "stage")) {
        if (run_stage()) return 1;
    }
    CK(hipFree(d));
    return 0;
}
