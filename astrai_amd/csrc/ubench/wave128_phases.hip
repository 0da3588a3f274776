// Where the four-wave 256x256x128 GEMM kernel's time goes, measured on the kernel itself:
//   1. phase stamps (the shader clock counter read by every wave at kernel start, main-loop
//      start, main-loop end and kernel end; workgroup 0) on all-zero operands, where the clock
//      stays at its maximum;
//   2. knock-outs: the same kernel with one class of instructions removed (LDS operand reads,
//      global->LDS loads, MFMAs, output stores), timed on zeros and on normally distributed fp8
//      operands (the config-1 distribution). On toggling operands the chip runs against its
//      power cap, so a knocked-out class gives back its issue slots AND its energy (clock).
// Build: make -C astrai_amd/csrc ubench     Run: astrai_amd/csrc/ubench/wave128_phases [M N K]
#define W8A8_PP_TIMING 1
#include "../gemm_wave128.cuh"
#include "../gemm_wave128_q16.cuh"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

using namespace w8a8;

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

template <class Op, int SK, int KO>
static float time_us(const GemmArgs& g) {
    auto kern = gemm_wave128_kernel<Op, SK, EPI_PLAIN, KO>;
    CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, Wave128Cfg::LDS_BYTES));
    const int tiles = ((g.m + 255) / 256) * ((g.n + 255) / 256);
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int i = 0; i < 300; ++i) kern<<<tiles, 256, Wave128Cfg::LDS_BYTES, 0>>>(g, RopeCacheArgs{});
    CK(hipDeviceSynchronize());
    std::vector<float> ts;
    for (int rep = 0; rep < 7; ++rep) {
        CK(hipEventRecord(e0));
        for (int i = 0; i < 100; ++i) kern<<<tiles, 256, Wave128Cfg::LDS_BYTES, 0>>>(g, RopeCacheArgs{});
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        ts.push_back(ms * 10.0f);
    }
    std::sort(ts.begin(), ts.end());
    return ts[3];
}

// the 16x16x128 instance of the four-wave kernel (fp8 only)
template <int SK, int KO>
static float time_q16_us(const GemmArgs& g) {
    auto kern = gemm_wave128_q16_kernel<0, SK, KO>;
    CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, Wave128Cfg::LDS_BYTES));
    const int tiles = ((g.m + 255) / 256) * ((g.n + 255) / 256);
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int i = 0; i < 300; ++i) kern<<<tiles, 256, Wave128Cfg::LDS_BYTES, 0>>>(g);
    CK(hipDeviceSynchronize());
    std::vector<float> ts;
    for (int rep = 0; rep < 7; ++rep) {
        CK(hipEventRecord(e0));
        for (int i = 0; i < 100; ++i) kern<<<tiles, 256, Wave128Cfg::LDS_BYTES, 0>>>(g);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        ts.push_back(ms * 10.0f);
    }
    std::sort(ts.begin(), ts.end());
    return ts[3];
}

// e4m3fn byte nearest to v (|v| <= 448)
static unsigned char e4m3_of(float v) {
    const float a = fabsf(v);
    const unsigned char s = v < 0 ? 0x80 : 0;
    if (a < 0.0009765625f) return s;
    int e;
    const float m = frexpf(a, &e);  // a = m * 2^e, m in [0.5, 1)
    int E = e - 1 + 7;
    if (E <= 0) return s | (unsigned char)std::min((int)lrintf(a / 0.001953125f), 7);
    int q = (int)lrintf((m * 2 - 1) * 8);
    if (q == 8) { q = 0; E++; }
    if (E > 15 || (E == 15 && q > 6)) { E = 15; q = 6; }
    return s | (unsigned char)((E << 3) | q);
}

// the eight-wave ping-pong kernel (block-scaled and per-tensor instances) with its stamps
template <class Op, int SK, class Cfg>
static float pingpong_us(const GemmArgs& g) {
    auto kern = gemm_pingpong_kernel<Op, SK, Cfg>;
    CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES));
    const int tiles = ((g.m + 255) / 256) * ((g.n + 255) / 256);
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    for (int i = 0; i < 200; ++i) kern<<<tiles, Cfg::THREADS, Cfg::LDS_BYTES, 0>>>(g);
    CK(hipDeviceSynchronize());
    std::vector<float> ts;
    for (int rep = 0; rep < 7; ++rep) {
        CK(hipEventRecord(e0));
        for (int i = 0; i < 50; ++i) kern<<<tiles, Cfg::THREADS, Cfg::LDS_BYTES, 0>>>(g);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        ts.push_back(ms * 20.0f);
    }
    std::sort(ts.begin(), ts.end());
    return ts[3];
}

static void print_stamps(unsigned long long* dbg, int k, std::initializer_list<int> waves) {
    std::vector<unsigned long long> hd(8 * 256);
    CK(hipMemcpy(hd.data(), dbg, hd.size() * 8, hipMemcpyDeviceToHost));
    for (int w : waves) {
        const unsigned long long* t = &hd[w * 256];
        printf("  wave %d: prologue %llu cycles, main loop %llu (%.0f per slab), epilogue %llu\n", w,
               t[1] - t[0], t[2] - t[1], (double)(t[2] - t[1]) / (k / 128), t[3] - t[2]);
    }
}

// config-3 shape: block-scaled instance against the per-tensor instance of the same kernel
static void pingpong_section(unsigned long long* dbg) {
    const int M = 8192, N = 2048, K = 7168;
    void *a, *b, *out;
    float* s;
    CK(hipMalloc(&a, (size_t)M * K));
    CK(hipMalloc(&b, (size_t)N * K));
    CK(hipMalloc(&out, (size_t)M * N * 2));
    CK(hipMalloc(&s, (size_t)4 * M * (K / 128)));
    std::vector<float> ones((size_t)M * (K / 128), 1.0f);
    CK(hipMemcpy(s, ones.data(), ones.size() * 4, hipMemcpyHostToDevice));
    GemmArgs g{a, b, s, s, nullptr, nullptr, out, M, N, K, OUT_BF16};
    for (int random = 0; random < 2; ++random) {
        if (random) {
            std::vector<unsigned char> ra((size_t)M * K), rb((size_t)N * K);
            auto gauss = [] { float u = 0; for (int i = 0; i < 12; ++i) u += (float)rand() / RAND_MAX; return u - 6.0f; };
            for (auto& x : ra) x = e4m3_of(gauss() * 448.0f / 4.5f);
            for (auto& x : rb) x = e4m3_of(gauss() * 448.0f / 4.5f);
            CK(hipMemcpy(a, ra.data(), ra.size(), hipMemcpyHostToDevice));
            CK(hipMemcpy(b, rb.data(), rb.size(), hipMemcpyHostToDevice));
        } else {
            CK(hipMemset(a, 0, (size_t)M * K));
            CK(hipMemset(b, 0, (size_t)N * K));
        }
        const double ops = 2.0 * M * N * (double)K;
        float us = pingpong_us<Op32F8<0>, SCALE_BLOCK128, PingPongCfgBlock>(g);
        printf("ping-pong kernel, 128-block scales, %s %dx%dx%d: %.2f us (%.0f Tops/s)\n",
               random ? "normal operands" : "zeros", M, N, K, us, ops / us / 1e6);
        if (!random) print_stamps(dbg, K, {0, 4});
        us = pingpong_us<Op32F8<0>, SCALE_TENSOR, PingPongCfg>(g);
        printf("ping-pong kernel, per-tensor scales, %s: %.2f us (%.0f Tops/s)\n",
               random ? "normal operands" : "zeros", us, ops / us / 1e6);
        if (!random) print_stamps(dbg, K, {0, 4});
        us = time_us<Op32F8<0>, SCALE_TENSOR, 0>(g);
        printf("four-wave kernel, per-tensor scales, %s: %.2f us (%.0f Tops/s)\n",
               random ? "normal operands" : "zeros", us, ops / us / 1e6);
    }
    CK(hipFree(a)); CK(hipFree(b)); CK(hipFree(out)); CK(hipFree(s));
}

template <class Op, int SK>
static void knockouts(const char* what, const GemmArgs& g) {
    const double ops = 2.0 * g.m * g.n * (double)g.k;
    const float base = time_us<Op, SK, 0>(g);
    printf("%s: whole kernel %.2f us (%.0f Tops/s)\n", what, base, ops / base / 1e6);
    printf("  without LDS operand reads      %.2f us\n", time_us<Op, SK, KO_LDS_READS>(g));
    printf("  without global->LDS loads      %.2f us\n", time_us<Op, SK, KO_LOADS>(g));
    printf("  without either                 %.2f us\n", time_us<Op, SK, KO_LDS_READS | KO_LOADS>(g));
    printf("  without output stores          %.2f us\n", time_us<Op, SK, KO_STORES>(g));
    printf("  without MFMAs                  %.2f us\n", time_us<Op, SK, KO_MFMA>(g));
}

template <int SK>
static void knockouts_q16(const char* what, const GemmArgs& g) {
    const double ops = 2.0 * g.m * g.n * (double)g.k;
    const float base = time_q16_us<SK, 0>(g);
    printf("%s, 16x16x128 instance: whole kernel %.2f us (%.0f Tops/s)\n", what, base, ops / base / 1e6);
    printf("  without LDS operand reads      %.2f us\n", time_q16_us<SK, KO_LDS_READS>(g));
    printf("  without global->LDS loads      %.2f us\n", time_q16_us<SK, KO_LOADS>(g));
    printf("  without either                 %.2f us\n", time_q16_us<SK, KO_LDS_READS | KO_LOADS>(g));
    printf("  without output stores          %.2f us\n", time_q16_us<SK, KO_STORES>(g));
    printf("  without MFMAs                  %.2f us\n", time_q16_us<SK, KO_MFMA>(g));
    printf("  without the per-slab barrier   %.2f us\n", time_q16_us<SK, KO_BARRIER>(g));
    printf("  without the per-slab waits     %.2f us\n", time_q16_us<SK, KO_WAITS>(g));
    printf("  without barrier and waits      %.2f us\n", time_q16_us<SK, KO_BARRIER | KO_WAITS>(g));
    printf("  without barrier, waits, loads and LDS reads %.2f us\n",
           time_q16_us<SK, KO_BARRIER | KO_WAITS | KO_LOADS | KO_LDS_READS>(g));
}

int main(int argc, char** argv) {
    int M = 4096, N = 4096, K = 4096;
    if (argc > 3) { M = atoi(argv[1]); N = atoi(argv[2]); K = atoi(argv[3]); }
    void *a, *b, *out;
    float* s;
    unsigned long long* dbg;
    CK(hipMalloc(&a, (size_t)M * K));
    CK(hipMalloc(&b, (size_t)N * K));
    CK(hipMalloc(&out, (size_t)M * N * 2));
    CK(hipMalloc(&s, (size_t)4 * (M + N)));
    CK(hipMalloc(&dbg, 8 * 256 * 8));
    CK(hipMemcpyToSymbol(HIP_SYMBOL(g_pp_dbg), &dbg, sizeof(dbg)));
    std::vector<float> steps(M + N, 1e-4f);
    CK(hipMemcpy(s, steps.data(), 4 * (M + N), hipMemcpyHostToDevice));
    GemmArgs g{a, b, s, s, nullptr, nullptr, out, M, N, K, OUT_BF16};

    CK(hipMemset(a, 0, (size_t)M * K));
    CK(hipMemset(b, 0, (size_t)N * K));
    for (int which = 0; which < 2; ++which) {
        const float us = which ? time_us<Op32I8, SCALE_ROWCOL, 0>(g) : time_us<Op32F8<0>, SCALE_TENSOR, 0>(g);
        printf("%s zeros %dx%dx%d: %.2f us; stamps of workgroup 0 in shader clock cycles\n",
               which ? "int8" : "fp8", M, N, K, us);
        print_stamps(dbg, K, {0, 3});
    }
    {
        const float us = time_q16_us<SCALE_TENSOR, 0>(g);
        printf("fp8 16x16x128 instance zeros %dx%dx%d: %.2f us; stamps of workgroup 0 in shader clock cycles\n", M, N, K, us);
        print_stamps(dbg, K, {0, 3});
    }
    knockouts<Op32F8<0>, SCALE_TENSOR>("fp8 zeros", g);
    knockouts_q16<SCALE_TENSOR>("fp8 zeros", g);
    knockouts<Op32I8, SCALE_ROWCOL>("int8 zeros", g);

    {
        std::vector<unsigned char> ra((size_t)M * K), rb((size_t)N * K);
        auto gauss = [] { float u = 0; for (int i = 0; i < 12; ++i) u += (float)rand() / RAND_MAX; return u - 6.0f; };
        for (auto& x : ra) x = e4m3_of(gauss() * 448.0f / 4.5f);
        for (auto& x : rb) x = e4m3_of(gauss() * 448.0f / 4.5f);
        CK(hipMemcpy(a, ra.data(), ra.size(), hipMemcpyHostToDevice));
        CK(hipMemcpy(b, rb.data(), rb.size(), hipMemcpyHostToDevice));
    }
    knockouts<Op32F8<0>, SCALE_TENSOR>("fp8 normal operands (amax at 4.5 sigma)", g);
    knockouts_q16<SCALE_TENSOR>("fp8 normal operands (amax at 4.5 sigma)", g);
    // the two instances in alternation on the same operands
    for (int rep = 0; rep < 3; ++rep)
        printf("alternating, normal operands: 32x32x64 %.2f us, 16x16x128 %.2f us\n",
               time_us<Op32F8<0>, SCALE_TENSOR, 0>(g), time_q16_us<SCALE_TENSOR, 0>(g));
    {
        std::vector<signed char> ra((size_t)M * K), rb((size_t)N * K);
        auto gauss = [] { float u = 0; for (int i = 0; i < 12; ++i) u += (float)rand() / RAND_MAX; return u - 6.0f; };
        for (auto& x : ra) x = (signed char)std::max(-127.0f, std::min(127.0f, rintf(gauss() * 127.0f / 4.5f)));
        for (auto& x : rb) x = (signed char)std::max(-127.0f, std::min(127.0f, rintf(gauss() * 127.0f / 4.5f)));
        CK(hipMemcpy(a, ra.data(), ra.size(), hipMemcpyHostToDevice));
        CK(hipMemcpy(b, rb.data(), rb.size(), hipMemcpyHostToDevice));
    }
    knockouts<Op32I8, SCALE_ROWCOL>("int8 normal operands (amax at 4.5 sigma)", g);
    pingpong_section(dbg);
    return 0;
}
