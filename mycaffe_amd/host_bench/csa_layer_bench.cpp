// Wall-clock benchmark of CausalSelfAttentionLayer.forward (CausalSelfAttentionLayer.cs:526-628) driven from a compiled
// host over the C ABI, the way the reference's C# layer drives CudaDnnDLL: the call sequence below is the layer's, issued
// through the CudaDnn method mirror of include/mycaffe_hip_host.hpp.  B = 8, T = 1024, C = 768, 12 heads (minGPT / GPT-2
// small block), N(0,1) input, N(0,0.02) weights, zero biases.
//
//   csa_layer_bench <libmycaffe_hip.so> [reps]
//
// prints one JSON object: milliseconds per forward for
//   f32_fused     fp32 storage, fused attention handle (ids 160-163)
//   f32_explicit  fp32 storage, the layer's default chain: transpose, MatMul, scale, mask, softmax, MatMul
//   bf16_fused    16-bit storage (ALLOCMEM_HALF), fused attention handle
//   *_4call       the same forward as four calls: fused QKV projection writing (B,H,T,hs) (id 2004), attention handle
//                 writing head-merged output, output projection GEMM and its bias GEMM
//   *_3call       the same with the output projection and its bias as one call (id 2005)
// Timed region: `reps` forwards between two device synchronisations (steady_clock), after 60 ms of untimed forwards.
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "mycaffe_hip_host.hpp"

using namespace mycaffe;

namespace {

// TransposeLayer.cs:127-213: strides and axis map live in device blobs created at reshape time
struct Transpose {
    CudaDnn& cuda;
    long hXCounts, hYCounts, hMap, hBuffer;
    long long count;
    int axes;
    Transpose(CudaDnn& c, const std::vector<int>& shape, const std::vector<int>& dim) : cuda(c)
    {
        axes = (int)shape.size();
        std::vector<int> top(axes);
        for (int i = 0; i < axes; i++) top[i] = shape[dim[i]];
        std::vector<float> bc(axes), tc(axes), mp(axes);
        count = 1;
        for (int i = 0; i < axes; i++) count *= shape[i];
        for (int i = 0; i < axes; i++) {
            long long b = 1, t = 1;
            for (int j = i + 1; j < axes; j++) { b *= shape[j]; t *= top[j]; }
            bc[i] = (float)b; tc[i] = (float)t; mp[i] = (float)dim[i];
        }
        hXCounts = cuda.AllocMemory(bc); hYCounts = cuda.AllocMemory(tc); hMap = cuda.AllocMemory(mp);
        hBuffer = cuda.AllocMemory(count * axes);
    }
    void Forward(long hX, long hY) { cuda.transpose(count, hX, hY, hXCounts, hYCounts, hMap, axes, hBuffer); }
    void Free() { for (long h : {hXCounts, hYCounts, hMap, hBuffer}) cuda.FreeMemory(h); }
};

std::vector<float> normal(size_t n, float std, unsigned seed)
{
    std::mt19937 g(seed);
    std::normal_distribution<float> d(0.f, std);
    std::vector<float> v(n);
    for (auto& x : v) x = d(g);
    return v;
}

double run(CudaDnn& cuda, bool half, bool fused, int reps, int calls = 0)
{
    const int B = 8, T = 1024, C = 768, H = 12, hs = C / H, M = B * T;
    const long long MC = (long long)M * C;
    long hX = cuda.AllocMemory(normal((size_t)MC, 1.f, 1), half);
    long hWa = cuda.AllocMemory(normal((size_t)3 * C * C, 0.02f, 2), half), hBa = cuda.AllocMemory(std::vector<float>(3 * C, 0.f), half);
    long hWp = cuda.AllocMemory(normal((size_t)C * C, 0.02f, 3), half), hBp = cuda.AllocMemory(std::vector<float>(C, 0.f), half);
    long hOnes = cuda.AllocMemory(std::vector<float>(M, 1.f), half);
    long hIp = cuda.AllocMemory(3 * MC, half);
    long hQ = cuda.AllocMemory(MC, half), hK = cuda.AllocMemory(MC, half), hV = cuda.AllocMemory(MC, half);
    long hQt = cuda.AllocMemory(MC, half), hKt = cuda.AllocMemory(MC, half), hVt = cuda.AllocMemory(MC, half);
    long hWork = cuda.AllocMemory(MC, half), hY = cuda.AllocMemory(MC, half), hTop = cuda.AllocMemory(MC, half);
    std::vector<float> tril((size_t)T * T, 0.f);                     // fillMask, CausalSelfAttentionLayer.cs:276-291
    for (int i = 0; i < T; i++)
        for (int j = 0; j <= i; j++) tril[(size_t)i * T + j] = 1.f;
    long hMask = cuda.AllocMemory(tril);
    Transpose split(cuda, {B, T, H, hs}, {0, 2, 1, 3}), merge(cuda, {B, H, T, hs}, {0, 2, 1, 3}), kT(cuda, {B, H, T, hs}, {0, 1, 3, 2});
    long hCudnn = cuda.CreateCuDNN(), hAttn = cuda.CreateAttn();
    cuda.SetAttn(hCudnn, hAttn, 0, false, B, T, H, hs, 0.f);
    long hKt1 = 0, hAttA = 0, hAttB = 0, hBtmDesc = 0, hTopDesc = 0;
    const long long nAtt = (long long)B * H * T * T;
    if (!fused) {
        hKt1 = cuda.AllocMemory(MC, half);
        hAttA = cuda.AllocMemory(nAtt, half);
        hAttB = cuda.AllocMemory(nAtt, half);
        hBtmDesc = cuda.CreateTensorDesc();
        hTopDesc = cuda.CreateTensorDesc();
        cuda.SetTensorDesc(hBtmDesc, B * H * T, T, 1, 1, half);
        cuda.SetTensorDesc(hTopDesc, B * H * T, T, 1, 1, half);
    }
    auto forward = [&]() {
        if (calls) {
            cuda.QkvProjHeads(B, T, H, hs, hX, hWa, hBa, hQt, hKt, hVt);
            cuda.AttnScaledDotProductForward(hCudnn, hAttn, T, hQt, hKt, hVt, hMask, hY, 0, true);
            if (calls == 3) {
                cuda.LinearForward(M, C, C, hY, hWp, hBp, hTop);
                return;
            }
            cuda.gemm(false, true, M, C, C, 1.f, hY, hWp, 0.f, hTop);
            cuda.gemm(false, false, M, C, 1, 1.f, hOnes, hBp, 1.f, hTop);
            return;
        }
        // q, k, v = c_attn(x).split(n_embd, dim = 2)   (InnerProductLayer.cs:372-417: gemm, then the bias as a rank-1 gemm)
        cuda.gemm(false, true, M, 3 * C, C, 1.f, hX, hWa, 0.f, hIp);
        cuda.gemm(false, false, M, 3 * C, 1, 1.f, hOnes, hBa, 1.f, hIp);
        cuda.channel_copy(MC, B, T, 3, C, 0, hIp, hQ, FWD);
        cuda.channel_copy(MC, B, T, 3, C, 1, hIp, hK, FWD);
        cuda.channel_copy(MC, B, T, 3, C, 2, hIp, hV, FWD);
        split.Forward(hQ, hQt);
        split.Forward(hK, hKt);
        split.Forward(hV, hVt);
        if (fused) {
            cuda.AttnScaledDotProductForward(hCudnn, hAttn, T, hQt, hKt, hVt, hMask, hWork, 0);
        } else {
            kT.Forward(hKt, hKt1);
            cuda.matmul(B * H, T, T, hs, hQt, hKt1, hAttA);
            cuda.scal(nAtt, 1.f / std::sqrt((float)hs), hAttA);
            cuda.mask(nAtt, (long long)T * T, 0.f, -1e29f, hAttA, hMask, hAttA);
            cuda.SoftmaxForward(hCudnn, hBtmDesc, hAttA, hTopDesc, hAttB);
            cuda.matmul(B * H, T, hs, T, hAttB, hVt, hWork);
        }
        merge.Forward(hWork, hY);
        cuda.gemm(false, true, M, C, C, 1.f, hY, hWp, 0.f, hTop);
        cuda.gemm(false, false, M, C, 1, 1.f, hOnes, hBp, 1.f, hTop);
    };
    // The GPU's clocks ramp for some 40 ms after an idle gap (a 28 us kernel measures 28.4 us in the first 2 ms and 24.9 us
    // from 40 ms on), and the set-up above is such a gap: the timed forwards follow 60 ms of untimed ones.
    {
        const auto w0 = std::chrono::steady_clock::now();
        do {
            for (int i = 0; i < 3; i++) forward();
            cuda.SynchronizeDevice();
        } while (std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - w0).count() < 60.0);
    }
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < reps; i++) forward();
    cuda.SynchronizeDevice();
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / reps;
    split.Free(); merge.Free(); kT.Free();
    cuda.FreeAttn(hAttn);
    cuda.FreeCuDNN(hCudnn);
    for (long h : {hX, hWa, hBa, hWp, hBp, hOnes, hIp, hQ, hK, hV, hQt, hKt, hVt, hWork, hY, hTop, hMask}) cuda.FreeMemory(h);
    if (!fused) {
        for (long h : {hKt1, hAttA, hAttB}) cuda.FreeMemory(h);
        cuda.FreeTensorDesc(hBtmDesc);
        cuda.FreeTensorDesc(hTopDesc);
    }
    return ms;
}

}  // namespace

int main(int argc, char** argv)
{
    if (argc < 2) {
        std::fprintf(stderr, "usage: %s <libmycaffe_hip.so> [reps]\n", argv[0]);
        return 2;
    }
    const int reps = argc > 2 ? std::max(1, std::atoi(argv[2])) : 20;
    try {
        CudaDnn cuda(0, argv[1]);
        const double a = run(cuda, false, true, reps);
        const double b = run(cuda, false, false, reps);
        const double c = run(cuda, true, true, reps);
        const double d = run(cuda, false, true, reps, 4);
        const double e = run(cuda, true, true, reps, 4);
        const double f = run(cuda, false, true, reps, 3);
        const double g = run(cuda, true, true, reps, 3);
        std::printf("{\"reps\": %d, \"f32_fused_ms\": %.4f, \"f32_explicit_ms\": %.4f, \"bf16_fused_ms\": %.4f, \"f32_4call_ms\": %.4f, "
                    "\"bf16_4call_ms\": %.4f, \"f32_3call_ms\": %.4f, \"bf16_3call_ms\": %.4f}\n", reps, a, b, c, d, e, f, g);
    } catch (const std::exception& e) {
        std::fprintf(stderr, "csa_layer_bench: %s\n", e.what());
        return 1;
    }
    return 0;
}
