// Micro-benchmarks of the gfx950 properties that the kernel designs of this library rest on.  Each prints one line per
// case; none of them touches the library.  Build: mycaffe_amd/build.py; run: mycaffe_amd/host_bench/hw_probes [section]
// with section in {overlap, lds, graph} (default: all).
//   overlap  how much vector-ALU work a wavefront can hide behind its own MFMAs (plain fma and v_exp_f32)
//   lds      rate of the LDS fragment reads of the attention and GEMM kernels (ds_read_b128 in the K-fragment pattern,
//            the transposing ds_read_b64_tr_b16 in the row-major V pattern) alone and with one MFMA per fragment
//   graph    cost of a kernel boundary inside a replayed HIP graph and of a bare mat-vec kernel at several working sets
#include <hip/hip_runtime.h>
#include <stdio.h>
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
    CK(hipFree(x));
    CK(hipFree(y));
    CK(hipFree(big));
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
    CK(hipFree(d));
    return 0;
}
