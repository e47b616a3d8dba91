// One fp16 contraction through the C ABI of libdaceml_hip.so from a C++ program (no Python, no torch): includes the
// public header, links against the library, runs the product, times it with HIP events and, with `check`, compares
// sampled outputs with a double-precision dot product on the host. tests/test_cabi_from_cpp.py builds it on the CPU
// (the header and the exported symbols are usable from C++) and runs it with `check` on a GPU; the per-configuration
// counter runs of the GEMM kernels are taken with it too.
//
//   gemm_from_cpp M N K a-layout b-layout config iterations [check|trace]
//     a-layout: k = A stored [m][k] (K-contiguous), r = A stored [k][m]
//     b-layout: k = B stored [n][k] (K-contiguous), r = B stored [k][n]
//     config:   tile configuration for dmlhip_debug_force_gemm_config (-1 = the library's own choice)
//     check:    compare 2000 sampled outputs with a double-precision dot product on the host
//     trace:    one more launch with dmlhip_debug_gemm_trace: where the workgroups' time goes (microseconds after the
//               first workgroup started; median and maximum over workgroups of: start, first tile in LDS, end of the K
//               loop, end of the epilogue)
//
// Build: python tests/cabi/build.py
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "daceml_hip.h"

#define PROBE_CHECK(x)                                                                    \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);    \
            std::exit(1);                                                                 \
        }                                                                                 \
    } while (0)

int main(int argc, char** argv) {
    if (argc < 8) {
        std::printf("usage: gemm_from_cpp M N K a-layout(k|r) b-layout(k|r) config iterations [check|trace]\n");
        return 1;
    }
    const long M = std::atol(argv[1]), N = std::atol(argv[2]), K = std::atol(argv[3]);
    const char al = argv[4][0], bl = argv[5][0];
    const int cfg = std::atoi(argv[6]), iters = std::atoi(argv[7]);
    const bool check = argc > 8 && std::strcmp(argv[8], "check") == 0;
    const bool trace = argc > 8 && std::strcmp(argv[8], "trace") == 0;
    if (M <= 0 || N <= 0 || K <= 0 || iters <= 0 || (al != 'k' && al != 'r') || (bl != 'k' && bl != 'r')) {
        std::printf("bad arguments\n");
        return 1;
    }
    std::vector<_Float16> ha((size_t)M * K), hb((size_t)N * K);
    std::mt19937 rng(1);
    std::normal_distribution<float> nd(0.f, 1.f);
    for (auto& v : ha) v = (_Float16)nd(rng);
    for (auto& v : hb) v = (_Float16)(nd(rng) * 0.05f);
    // GEMM_PITCH_PAD=<elements> in the environment: the operands' rows are that much longer than their contents (what a
    // pitch that is not a power of two does to the time of a launch)
    const long pad = std::getenv("GEMM_PITCH_PAD") ? std::atol(std::getenv("GEMM_PITCH_PAD")) : 0;
    const long a_rows = al == 'k' ? M : K, a_cols = al == 'k' ? K : M, b_rows = bl == 'k' ? N : K, b_cols = bl == 'k' ? K : N;
    const long a_pitch = a_cols + pad, b_pitch = b_cols + pad;
    _Float16 *a, *b, *c;
    PROBE_CHECK(hipMalloc(&a, (size_t)a_rows * a_pitch * 2));
    PROBE_CHECK(hipMalloc(&b, (size_t)b_rows * b_pitch * 2));
    PROBE_CHECK(hipMalloc(&c, (size_t)M * N * 2));
    PROBE_CHECK(hipMemcpy2D(a, a_pitch * 2, ha.data(), a_cols * 2, a_cols * 2, a_rows, hipMemcpyHostToDevice));
    PROBE_CHECK(hipMemcpy2D(b, b_pitch * 2, hb.data(), b_cols * 2, b_cols * 2, b_rows, hipMemcpyHostToDevice));
    dmlhip_gemm_desc d;
    std::memset(&d, 0, sizeof d);
    d.m = M; d.n = N; d.k = K;
    d.batch[0] = d.batch[1] = d.batch[2] = 1;
    if (al == 'k') { d.a_stride_m = a_pitch; d.a_stride_k = 1; } else { d.a_stride_m = 1; d.a_stride_k = a_pitch; }
    if (bl == 'k') { d.b_stride_n = b_pitch; d.b_stride_k = 1; } else { d.b_stride_n = 1; d.b_stride_k = b_pitch; }
    d.c_stride_m = N;
    d.alpha = 1.f;
    d.out_dtype = DMLHIP_F16;
    d.bias_dtype = DMLHIP_F16;
    dmlhip_debug_force_gemm_config(cfg);
    hipStream_t st;
    PROBE_CHECK(hipStreamCreate(&st));
    for (int i = 0; i < 3; ++i) {
        if (int e = dmlhip_gemm_f16(&d, a, b, c, nullptr, nullptr, nullptr, st)) {
            std::printf("dmlhip_gemm_f16 returned %d: %s\n", e, dmlhip_last_error_string());
            return 1;
        }
    }
    PROBE_CHECK(hipStreamSynchronize(st));
    hipEvent_t e0, e1;
    PROBE_CHECK(hipEventCreate(&e0));
    PROBE_CHECK(hipEventCreate(&e1));
    PROBE_CHECK(hipEventRecord(e0, st));
    for (int i = 0; i < iters; ++i) dmlhip_gemm_f16(&d, a, b, c, nullptr, nullptr, nullptr, st);
    PROBE_CHECK(hipEventRecord(e1, st));
    PROBE_CHECK(hipStreamSynchronize(st));
    float ms = 0.f;
    PROBE_CHECK(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1e3 / iters;
    std::printf("M=%ld N=%ld K=%ld %c%c config %d: %.2f us per launch, %.1f TFLOP/s\n", M, N, K, al, bl, cfg, us,
                2.0 * M * N * K / us / 1e6);
    if (trace) {
        const size_t slots = 4 * ((size_t)((M + 63) / 64) * ((N + 63) / 64) + 8);   // no tile is smaller than 64 x 64
        unsigned long long* buf;
        PROBE_CHECK(hipMalloc(&buf, slots * 8));
        PROBE_CHECK(hipMemset(buf, 0, slots * 8));
        dmlhip_debug_gemm_trace(buf);
        dmlhip_gemm_f16(&d, a, b, c, nullptr, nullptr, nullptr, st);
        PROBE_CHECK(hipStreamSynchronize(st));
        dmlhip_debug_gemm_trace(nullptr);
        std::vector<unsigned long long> h(slots);
        PROBE_CHECK(hipMemcpy(h.data(), buf, slots * 8, hipMemcpyDeviceToHost));
        std::vector<double> ph[4];
        unsigned long long t0 = ~0ULL;
        for (size_t w = 0; w * 4 < slots; ++w)
            if (h[4 * w] && h[4 * w] < t0) t0 = h[4 * w];
        for (size_t w = 0; w * 4 < slots; ++w)
            if (h[4 * w])
                for (int i = 0; i < 4; ++i) ph[i].push_back((double)(h[4 * w + i] - t0) * 0.01);   // 100 MHz -> us
        const char* names[4] = {"start", "first tile in LDS", "end of the K loop", "end of the epilogue"};
        std::printf("trace: %zu workgroups\n", ph[0].size());
        for (int i = 0; i < 4; ++i) {
            std::sort(ph[i].begin(), ph[i].end());
            const size_t n = ph[i].size();
            std::printf("  %-20s min %6.2f  p10 %6.2f  median %6.2f  p90 %6.2f  max %6.2f us\n", names[i], ph[i][0],
                        ph[i][n / 10], ph[i][n / 2], ph[i][n * 9 / 10], ph[i][n - 1]);
        }
    }
    if (check) {
        std::vector<_Float16> hc((size_t)M * N);
        PROBE_CHECK(hipMemcpy(hc.data(), c, hc.size() * 2, hipMemcpyDeviceToHost));
        double worst = 0;
        int bad = 0;
        for (int t = 0; t < 2000; ++t) {
            long m = rng() % M, n = rng() % N;
            if (t < 8) { m = (t & 1) ? M - 1 : 0; n = (t & 2) ? N - 1 : 0; }
            double s = 0;
            for (long k = 0; k < K; ++k) {
                const float av = al == 'k' ? (float)ha[m * K + k] : (float)ha[k * M + m];
                const float bv = bl == 'k' ? (float)hb[n * K + k] : (float)hb[k * N + n];
                s += (double)av * bv;
            }
            const double err = std::fabs((double)(float)hc[m * N + n] - s);
            if (err > 1e-2 + 2e-2 * std::fabs(s)) ++bad;
            if (err > worst) worst = err;
        }
        std::printf("check: %d of 2000 samples beyond rtol 2e-2 / atol 1e-2, worst absolute error %.4g\n", bad, worst);
        if (bad) return 2;
    }
    return 0;
}
