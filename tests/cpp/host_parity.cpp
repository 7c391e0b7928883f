// C++ host-side parity program: drives the HIP libraries only through include/mycaffe_hip_host.hpp (the C++
// counterpart of the C# CudaDnn<float> + CudaControl pair) and checks
//   1. the inline known-answer vector of TestCudaDnn.cs TestGemm (:5586-5686), all four transpose combinations;
//   2. error codes crossing the ABI as exceptions;
//   3. the CausalSelfAttentionLayer forward call sequence (CausalSelfAttentionLayer.cs:526-628) on the
//      gpt-pico-csa* tensors held by the reference's test data, against the recorded layer output y;
//   4. optionally a greedy generation through the llama2 extension, whose ids are printed for the caller to compare.
// usage: host_parity <libmycaffe_hip.so> <golden dir> [<libmycaffe_hip_llama2.so> <checkpoint.bin> <nSteps> <id> <id> ...]
// Prints one line per check; exit status 0 only when every check passed.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <sstream>

#include "../../include/mycaffe_hip_host.hpp"

using namespace mycaffe;

static int g_failed = 0;
static void report(const char* what, bool ok, double err = 0.0)
{
    printf("%s %s (max rel err %.3g)\n", ok ? "PASS" : "FAIL", what, err);
    fflush(stdout);
    if (!ok) g_failed++;
}

struct Tensor {
    std::vector<int> shape;
    std::vector<float> data;
    long long count() const { return (long long)data.size(); }
};

// reference text tensor: first line "# (d0, d1, ...)", then one value per line
static Tensor load_txt(const std::string& path)
{
    std::ifstream f(path);
    if (!f) throw std::runtime_error("cannot open " + path);
    Tensor t;
    std::string line;
    std::getline(f, line);
    for (char& ch : line)
        if (ch == '#' || ch == '(' || ch == ')' || ch == ',') ch = ' ';
    std::istringstream hs(line);
    int d;
    while (hs >> d) t.shape.push_back(d);
    double v;
    while (f >> v) t.data.push_back((float)v);
    return t;
}

static double max_rel_err(const std::vector<float>& a, const std::vector<float>& b)
{
    double scale = 0, err = 0;
    for (size_t i = 0; i < b.size(); i++) scale = std::fmax(scale, std::fabs((double)b[i]));
    for (size_t i = 0; i < b.size(); i++) err = std::fmax(err, std::fabs((double)a[i] - (double)b[i]));
    return a.size() == b.size() ? err / (scale > 0 ? scale : 1) : 1e30;
}

// TransposeLayer.cs:127-213: the generic transpose takes its strides and axis map as float blobs
struct TransposeLayer {
    CudaDnn& cuda;
    std::vector<int> dim;
    long hXCounts = 0, hYCounts = 0, hMap = 0, hBuffer = 0;
    TransposeLayer(CudaDnn& c, std::vector<int> d) : cuda(c), dim(std::move(d)) {}
    std::vector<int> Forward(const std::vector<int>& shape, long hX, long hY)
    {
        const int n = (int)shape.size();
        std::vector<int> top(n);
        for (int i = 0; i < n; i++) top[i] = shape[dim[i]];
        std::vector<float> bc(n), tc(n), mp(n);
        long long count = 1;
        for (int i = 0; i < n; i++) count *= shape[i];
        for (int i = 0; i < n; i++) {
            long long b = 1, t = 1;
            for (int j = i + 1; j < n; j++) { b *= shape[j]; t *= top[j]; }
            bc[i] = (float)b; tc[i] = (float)t; mp[i] = (float)dim[i];
        }
        if (!hXCounts) {
            hXCounts = cuda.AllocMemory(bc); hYCounts = cuda.AllocMemory(tc); hMap = cuda.AllocMemory(mp);
            hBuffer = cuda.AllocMemory(count * n);
        }
        cuda.transpose(count, hX, hY, hXCounts, hYCounts, hMap, n, hBuffer);
        return top;
    }
};

// InnerProductLayer.cs:372-417 with axis 2: y = x W^T, then y += ones (M,1) * bias (1,N) as a rank-1 gemm
static void inner_product(CudaDnn& cuda, int M, int N, int K, long hX, long hW, long hBias, long hOnes, long hY)
{
    cuda.gemm(false, true, M, N, K, 1.f, hX, hW, 0.f, hY);
    if (hBias) cuda.gemm(false, false, M, N, 1, 1.f, hOnes, hBias, 1.f, hY);
}

static void csa_golden(CudaDnn& cuda, const std::string& dir, int heads)
{
    Tensor x = load_txt(dir + "/x.txt"), wa = load_txt(dir + "/attn_weight.txt"), ba = load_txt(dir + "/attn_bias.txt");
    Tensor wp = load_txt(dir + "/attn_proj_weight.txt"), bp = load_txt(dir + "/attn_proj_bias.txt"), y = load_txt(dir + "/y.txt");
    const int B = x.shape[0], T = x.shape[1], C = x.shape[2], hs = C / heads, M = B * T;
    long hX = cuda.AllocMemory(x.data), hWa = cuda.AllocMemory(wa.data), hBa = cuda.AllocMemory(ba.data);
    long hWp = cuda.AllocMemory(wp.data), hBp = cuda.AllocMemory(bp.data), hOnes = cuda.AllocMemory(std::vector<float>(M, 1.f));
    long hIp = cuda.AllocMemory((long long)M * 3 * C), hQ = cuda.AllocMemory((long long)M * C), hK = cuda.AllocMemory((long long)M * C);
    long hV = cuda.AllocMemory((long long)M * C), hQt = cuda.AllocMemory((long long)M * C), hKt = cuda.AllocMemory((long long)M * C);
    long hVt = cuda.AllocMemory((long long)M * C), hWork = cuda.AllocMemory((long long)M * C), hY = cuda.AllocMemory((long long)M * C);
    long hTop = cuda.AllocMemory((long long)M * C);
    std::vector<float> tril((size_t)T * T, 0.f);                     // fillMask, CausalSelfAttentionLayer.cs:276-291
    for (int i = 0; i < T; i++)
        for (int j = 0; j <= i; j++) tril[(size_t)i * T + j] = 1.f;
    long hMask = cuda.AllocMemory(tril);
    // q, k, v = c_attn(x).split(n_embd, dim = 2)
    inner_product(cuda, M, 3 * C, C, hX, hWa, hBa, hOnes, hIp);
    for (int i = 0; i < 3; i++) cuda.channel_copy((long long)M * C, B, T, 3, C, i, hIp, i == 0 ? hQ : (i == 1 ? hK : hV), FWD);
    // (B, T, nh, hs) -> (B, nh, T, hs)
    TransposeLayer tr(cuda, {0, 2, 1, 3});
    tr.Forward({B, T, heads, hs}, hQ, hQt);
    tr.Forward({B, T, heads, hs}, hK, hKt);
    tr.Forward({B, T, heads, hs}, hV, hVt);
    long hCudnn = cuda.CreateCuDNN(), hAttn = cuda.CreateAttn();
    cuda.SetAttn(hCudnn, hAttn, 0, true, B, T, heads, hs, 0.f);    // training: the forward call keeps what ATTN_BWD needs
    cuda.AttnScaledDotProductForward(hCudnn, hAttn, T, hQt, hKt, hVt, hMask, hWork, 0);
    // y.transpose(1, 2).contiguous().view(B, T, C), then the output projection
    TransposeLayer tb(cuda, {0, 2, 1, 3});
    tb.Forward({B, heads, T, hs}, hWork, hY);
    inner_product(cuda, M, C, C, hY, hWp, hBp, hOnes, hTop);
    std::vector<float> out = cuda.GetMemoryFloat(hTop, (long long)M * C);
    const double err = max_rel_err(out, y.data);
    report(("causal self attention layer vs " + dir.substr(dir.find_last_of('/') + 1) + "/y.txt").c_str(), err <= 1e-4, err);
    // the same forward as three calls (ids with no counterpart in the reference: fused QKV projection written head by
    // head, attention output written merged, output projection with its bias), on an inference-mode handle
    {
        long hAttn2 = cuda.CreateAttn();
        cuda.SetAttn(hCudnn, hAttn2, 0, false, B, T, heads, hs, 0.f);
        for (long h : {hQt, hKt, hVt, hY, hTop}) cuda.set((long long)M * C, h, 0.f);
        cuda.QkvProjHeads(B, T, heads, hs, hX, hWa, hBa, hQt, hKt, hVt);
        cuda.AttnScaledDotProductForward(hCudnn, hAttn2, T, hQt, hKt, hVt, hMask, hY, 0, true);
        cuda.LinearForward(M, C, C, hY, hWp, hBp, hTop);
        const double e3 = max_rel_err(cuda.GetMemoryFloat(hTop, (long long)M * C), y.data);
        report(("the layer as three calls vs " + dir.substr(dir.find_last_of('/') + 1) + "/y.txt").c_str(), e3 <= 1e-4, e3);
        cuda.FreeAttn(hAttn2);
        // the training-mode handle's forward state is what the gradient below uses: run it again
        cuda.AttnScaledDotProductForward(hCudnn, hAttn, T, hQt, hKt, hVt, hMask, hWork, 0);
    }
    // gradients of the attention core against the reference's dump of the same layer (iter_0): dY (B,H,T,hs) -> dQ, dK, dV
    {
        Tensor gy = load_txt(dir + "/iter_0/grad_y_pre_transpose.txt");
        long hdY = cuda.AllocMemory(gy.data), hdQ = cuda.AllocMemory((long long)M * C), hdK = cuda.AllocMemory((long long)M * C);
        long hdV = cuda.AllocMemory((long long)M * C);
        cuda.AttnScaledDotProductBackward(hCudnn, hAttn, hQt, hdQ, hKt, hdK, hVt, hdV, hMask, hWork, hdY);
        double worst = 0;
        const char* names[3] = {"/iter_0/grad_qt.txt", "/iter_0/grad_kt.txt", "/iter_0/grad_vt.txt"};
        const long hs3[3] = {hdQ, hdK, hdV};
        for (int i = 0; i < 3; i++) worst = std::max(worst, max_rel_err(cuda.GetMemoryFloat(hs3[i], (long long)M * C), load_txt(dir + names[i]).data));
        report(("attention backward vs " + dir.substr(dir.find_last_of('/') + 1) + "/iter_0 grad_qt, grad_kt, grad_vt").c_str(), worst <= 1e-4, worst);
        for (long h : {hdY, hdQ, hdK, hdV}) cuda.FreeMemory(h);
    }
    cuda.FreeAttn(hAttn);
    cuda.FreeCuDNN(hCudnn);
    for (long h : {hX, hWa, hBa, hWp, hBp, hOnes, hIp, hQ, hK, hV, hQt, hKt, hVt, hWork, hY, hTop, hMask}) cuda.FreeMemory(h);
}

// LayerNorm handle forward and gradient on the reference's dump (x, y, grad_1a_y -> grad_9_x), eps 1e-10
static void layernorm_golden(CudaDnn& cuda, const std::string& dir)
{
    Tensor x = load_txt(dir + "/x.txt"), y = load_txt(dir + "/y.txt"), gy = load_txt(dir + "/grad_1a_y.txt"), gx = load_txt(dir + "/grad_9_x.txt");
    const int B = x.shape[0], T = x.shape[1], C = x.shape[2];
    const long long n = (long long)B * T * C;
    long h = cuda.CreateLayerNorm(0, n, B, T, C, 1e-10f);
    long hX = cuda.AllocMemory(x.data), hY = cuda.AllocMemory(n), hdY = cuda.AllocMemory(gy.data), hdX = cuda.AllocMemory(n);
    cuda.LayerNormForward(h, hX, hY);
    const double e1 = max_rel_err(cuda.GetMemoryFloat(hY, n), y.data);
    cuda.LayerNormBackward(h, hY, hdY, hdX);
    const double e2 = max_rel_err(cuda.GetMemoryFloat(hdX, n), gx.data);
    report(("layer norm forward + backward vs " + dir.substr(dir.find_last_of('/') + 1)).c_str(), e1 <= 1e-4 && e2 <= 1e-4, std::max(e1, e2));
    cuda.FreeLayerNorm(h);
    for (long m : {hX, hY, hdY, hdX}) cuda.FreeMemory(m);
}

static void gelu_golden(CudaDnn& cuda, const std::string& dir)
{
    Tensor x = load_txt(dir + "/1_x.txt"), y = load_txt(dir + "/2_y.txt"), gy = load_txt(dir + "/grad_1_y.txt"), gx = load_txt(dir + "/grad_2_x.txt");
    const long long n = (long long)x.data.size();
    long hX = cuda.AllocMemory(x.data), hY = cuda.AllocMemory(n), hdY = cuda.AllocMemory(gy.data), hdX = cuda.AllocMemory(n);
    cuda.gelu_fwd(n, hX, hY, true);
    const double e1 = max_rel_err(cuda.GetMemoryFloat(hY, n), y.data);
    cuda.gelu_bwd(n, hdY, hY, hdX, hX, true);
    const double e2 = max_rel_err(cuda.GetMemoryFloat(hdX, n), gx.data);
    report("gelu forward + backward vs gpt-pico-gelu", e1 <= 1e-4 && e2 <= 1e-4, std::max(e1, e2));
    for (long m : {hX, hY, hdY, hdX}) cuda.FreeMemory(m);
}

int main(int argc, char** argv)
{
    if (argc < 3) {
        fprintf(stderr, "usage: %s <libmycaffe_hip.so> <golden dir> [<llama2 extension> <checkpoint.bin> <nSteps> <ids...>]\n", argv[0]);
        return 2;
    }
    try {
        CudaDnn cuda(0, argv[1]);
        printf("device: %s\n", cuda.GetDeviceName(0).c_str());
        // 1. TestGemm known answers: A (2x3) = 1..6, B (3x4) = 1..12
        {
            const std::vector<float> A = {1, 2, 3, 4, 5, 6}, At = {1, 4, 2, 5, 3, 6};
            const std::vector<float> Bm = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}, Bt = {1, 5, 9, 2, 6, 10, 3, 7, 11, 4, 8, 12};
            const std::vector<float> expect = {38, 44, 50, 56, 83, 98, 113, 128};
            long hA = cuda.AllocMemory(A), hAt = cuda.AllocMemory(At), hB = cuda.AllocMemory(Bm), hBt = cuda.AllocMemory(Bt), hC = cuda.AllocMemory(8);
            bool ok = true;
            for (int tA = 0; tA < 2; tA++)
                for (int tB = 0; tB < 2; tB++) {
                    cuda.gemm(tA, tB, 2, 4, 3, 1.f, tA ? hAt : hA, tB ? hBt : hB, 0.f, hC);
                    ok = ok && cuda.GetMemoryFloat(hC) == expect;
                }
            report("gemm inline vector, four transpose combinations, exact", ok);
            // a fresh allocation is zero filled (memorycol.h:75-107)
            std::vector<float> z = cuda.GetMemoryFloat(cuda.AllocMemory(1000), 1000);
            bool zero = z.size() == 1000;
            for (float v : z) zero = zero && v == 0.f;
            report("new allocations are zero filled; GETMEM beyond the caller's buffer", zero);
            for (long h : {hA, hAt, hB, hBt, hC}) cuda.FreeMemory(h);
        }
        // 2. error codes become exceptions
        {
            long code = 0;
            try {
                cuda.gemm(false, false, 2, 2, 2, 1.f, 4242, 4243, 0.f, 4244);
            } catch (const CudaDnnError& e) {
                code = e.code();
            }
            report("unknown memory handle -> ERROR_MEMORY_NOT_FOUND", code == MCH_ERROR_MEMORY_NOT_FOUND);
            code = 0;
            try {
                cuda.Raw().RunFloatEx2(cuda.KernelHandle(), 480 /* CUDA_FN_LSTM_FWD, outside the path */, {}, {1});
            } catch (const CudaDnnError& e) {
                code = e.code();
            }
            report("function id outside the path -> ERROR_NOT_IMPLEMENTED", code == MCH_ERROR_NOT_IMPLEMENTED);
        }
        // 3. layer forward on the reference's golden tensors
        const std::string g = argv[2];
        csa_golden(cuda, g + "/gpt-pico-csa", 1);
        csa_golden(cuda, g + "/gpt-pico-csaB", 1);
        csa_golden(cuda, g + "/gpt-pico-csa3", 3);
        csa_golden(cuda, g + "/gpt-pico-csa3B", 3);
        layernorm_golden(cuda, g + "/gpt-pico-ln");
        layernorm_golden(cuda, g + "/gpt-pico-ln3B");
        gelu_golden(cuda, g + "/gpt-pico-gelu");
        // 4. llama2 extension
        if (argc >= 7) {
            LlmInference llm(cuda, argv[3]);
            llm.Load(argv[4]);
            const int nSteps = atoi(argv[5]);
            std::vector<int> prompt;
            for (int i = 6; i < argc; i++) prompt.push_back(atoi(argv[i]));
            std::vector<int> ids = llm.GenerateIds(prompt, nSteps);
            printf("IDS");
            for (int id : ids) printf(" %d", id);
            printf("\n");
        }
    } catch (const std::exception& e) {
        printf("FAIL exception: %s\n", e.what());
        return 1;
    }
    return g_failed ? 1 : 0;
}
