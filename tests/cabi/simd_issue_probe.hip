// What one SIMD of the GPU does with the instruction mixes of the fused-attention kernels: stand-alone loops without
// global memory traffic, 256 threads per workgroup, 256 or 512 workgroups (one or two wavefronts per SIMD on 256 compute
// units), timed with HIP events. MEASUREMENT TOOL; built by tests/cabi/build.py, run by hand.
//
//   part 1: a loop of 8 MFMAs (two accumulators) with NV independent vector instructions between them (fused
//           multiply-adds or exponentials): does vector work issue in the shadow of the matrix pipe, and what does
//           an exponential cost;
//   part 2: the LDS fragment reads and MFMAs of one 64-key attention tile (8 ds_read_b128 of K rows, 16
//           ds_read_b64_tr_b16 of V^T, 8 + 8 MFMAs) without the softmax arithmetic. The reads are plain LDS loads and the
//           transpose-read builtin: the compiler places every wait;
//   part 3: the instruction mix of one K step of the 128 x 128 GEMM tile (16 MFMAs, 16 or 8 ds_read_b128, 8 or 4
//           global -> LDS transfers per wavefront) on one wavefront per SIMD.
#include <hip/hip_runtime.h>

#include <cstdio>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef __fp16 fp16x4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define PROBE_CHECK(x)                                                                 \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

// ---------------------------------------------------------------- part 1
template <int NV, int KIND, int NM>   // KIND 0: v_fma_f32, 1: v_exp_f32; NM MFMAs per iteration (0 or 8)
__global__ __launch_bounds__(256) void issue_kernel(float* out, int iters, float seed) {
    floatx16 acc0, acc1;
    for (int e = 0; e < 16; ++e) { acc0[e] = 0.f; acc1[e] = 0.f; }
    half8 a, b;
    for (int e = 0; e < 8; ++e) { a[e] = (_Float16)(seed + threadIdx.x * 0.001f); b[e] = (_Float16)(seed * 0.5f); }
    float v[8];
    for (int i = 0; i < 8; ++i) v[i] = seed + i + threadIdx.x;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if (m < NM) {
                if (m & 1) acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc1, 0, 0, 0);
                else acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc0, 0, 0, 0);
            }
#pragma unroll
            for (int j = 0; j < NV / 8; ++j) {
                if (KIND == 0) v[j & 7] = __builtin_fmaf(v[j & 7], 1.0001f, 0.5f);
                else v[j & 7] = __builtin_amdgcn_exp2f(v[j & 7]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float s = 0.f;
    for (int e = 0; e < 16; ++e) s += acc0[e] + acc1[e];
    for (int i = 0; i < 8; ++i) s += v[i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// ---------------------------------------------------------------- part 2
__device__ __forceinline__ int swz_rt(int r) { return ((r >> 2) & 3) | (((r >> 1) & 1) << 2); }

template <int MODE>   // 0: reads + MFMAs; 1: MFMAs alone (operands read once); 2: reads alone (one MFMA keeps them live)
__global__ __launch_bounds__(256, 2) void tile_kernel(float* out, int iters, int barrier) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 64 * 1024 / 4; i += 256) ((float*)lds)[i] = (float)(i & 15) * 0.001f;
    __syncthreads();
    // the tile layout and fragment addresses of daceml_amd/csrc/attention.hip (conflict-free for both kinds of read)
    const int r = lane & 31, h = lane >> 5;
    int rowread[4], trread[2][2];
    for (int st = 0; st < 4; ++st) rowread[st] = r * 128 + (((st * 2 + h) ^ swz_rt(r)) << 4);
    const int s = lane & 15, grp = lane >> 4, hh = grp >> 1;
    for (int blk = 0; blk < 2; ++blk)
        for (int hi = 0; hi < 2; ++hi) {
            const int kk = 4 * hh + 8 * hi + (s >> 2);
            const int d0 = blk * 32 + (grp & 1) * 16 + 4 * (s & 3);
            trread[blk][hi] = 8192 + kk * 128 + (((d0 >> 3) ^ swz_rt(kk)) << 4) + (d0 & 7) * 2;
        }
    floatx16 sacc0, sacc1, oacc0, oacc1;
    for (int e = 0; e < 16; ++e) { sacc0[e] = 0.f; sacc1[e] = 0.f; oacc0[e] = 0.f; oacc1[e] = 0.f; }
    half8 qf[4], pf[4];
    for (int st = 0; st < 4; ++st)
        for (int e = 0; e < 8; ++e) { qf[st][e] = (_Float16)(0.01f * lane); pf[st][e] = (_Float16)(0.02f * lane); }
    half8 kf[2][4], vf[2][4];
    auto read_all = [&](int stage) {
        const char* base = lds + stage * 16384;
        for (int st = 0; st < 4; ++st) {
            kf[0][st] = *(const half8*)(base + rowread[st]);
            kf[1][st] = *(const half8*)(base + rowread[st] + 4096);
        }
        for (int blk = 0; blk < 2; ++blk)
            for (int st = 0; st < 4; ++st) {
                const half4 lo = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                    (__attribute__((address_space(3))) fp16x4*)(base + trread[blk][0] + st * 2048)));
                const half4 hi = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4f16(
                    (__attribute__((address_space(3))) fp16x4*)(base + trread[blk][1] + st * 2048)));
                vf[blk][st] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
    };
    read_all(0);
    for (int it = 0; it < iters; ++it) {
        if (MODE != 1) read_all(it & 3);
        if (barrier) __builtin_amdgcn_s_barrier();
        if (MODE != 2) {
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                sacc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[0][st], qf[st], sacc0, 0, 0, 0);
                sacc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[1][st], qf[st], sacc1, 0, 0, 0);
            }
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                oacc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[0][st], pf[st], oacc0, 0, 0, 0);
                oacc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[1][st], pf[st], oacc1, 0, 0, 0);
            }
        } else {
            half8 x = kf[0][0];
            for (int st = 0; st < 4; ++st) {
                x = x + kf[1][st] + vf[0][st] + vf[1][st];
                if (st) x = x + kf[0][st];
            }
            sacc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, qf[0], sacc0, 0, 0, 0);
        }
    }
    float sum = 0.f;
    for (int e = 0; e < 16; ++e) sum += sacc0[e] + sacc1[e] + oacc0[e] + oacc1[e];
    out[blockIdx.x * 256 + threadIdx.x] = sum;
}

// ---------------------------------------------------------------- part 3
// The per-K-step instruction mix of the 128 x 128 GEMM tile on one wavefront per SIMD: 16 MFMAs, NREADS ds_read_b128
// (16 = four wavefronts of 64 x 64 outputs each read their A and B fragments; 8 = what a split of K across the
// wavefronts would read) and NDMA global -> LDS transfers of 16 bytes per lane (8 = both operands through LDS) from a
// buffer that stays in L2. Data values do not matter here; every read feeds an MFMA so that nothing is dropped.
template <int NREADS, int NDMA, bool SHARED>
__global__ __launch_bounds__(256) void step_kernel(float* out, const _Float16* src, int iters) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 128 * 1024 / 4; i += 256) ((float*)lds)[i] = (float)(i & 15) * 0.001f;
    __syncthreads();
    floatx16 acc[4];
    for (int t = 0; t < 4; ++t)
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    const int r = lane & 31, h = lane >> 5;
    const char* rd = lds + (wave * 32 + r) * 128 + ((h ^ (r & 7)) << 4);
    // SHARED: every workgroup streams through the same 256 KB, 32 KB per iteration (what a GEMM's L2 does for tiles that
    // its workgroups share); otherwise through 256 KB of its own (64 MB in all: from the memory-side cache)
    const _Float16* gsrc = src + (SHARED ? 0 : (size_t)blockIdx.x * (128 * 1024)) + wave * 512 + lane * 8;
    half8 frag[16];
    for (int i = 0; i < 16; ++i) frag[i] = *(const half8*)(rd + (i & 7) * 16);
    for (int it = 0; it < iters; ++it) {
        const int stage = it & 3;
        const _Float16* g = gsrc + (size_t)(it & 7) * (16 * 1024);
        char* dst = lds + stage * 32768 + wave * 1024;
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(frag[m], frag[(m + 5) & 15], acc[m & 3], 0, 0, 0);
            if (m < NREADS) frag[m] = *(const half8*)(rd + ((stage + 1) & 3) * 32768 + m * 2048);
            if ((m & 1) == 0 && m / 2 < NDMA)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g + (m / 2) * 2048),
                                                 (__attribute__((address_space(3))) void*)(dst + (m / 2) * 4096), 16, 0, 0);
        }
        __builtin_amdgcn_s_barrier();
    }
    float sum = 0.f;
    for (int t = 0; t < 4; ++t)
        for (int e = 0; e < 16; ++e) sum += acc[t][e];
    out[blockIdx.x * 256 + threadIdx.x] = sum;
}

// ---------------------------------------------------------------- host
constexpr int kIters = 2000;

template <typename Launch>
int timed(const char* name, int blocks, const char* note, Launch launch) {
    hipEvent_t e0, e1;
    PROBE_CHECK(hipEventCreate(&e0));
    PROBE_CHECK(hipEventCreate(&e1));
    launch(10);
    PROBE_CHECK(hipDeviceSynchronize());
    PROBE_CHECK(hipEventRecord(e0));
    launch(kIters);
    PROBE_CHECK(hipEventRecord(e1));
    PROBE_CHECK(hipEventSynchronize(e1));
    float ms;
    PROBE_CHECK(hipEventElapsedTime(&ms, e0, e1));
    std::printf("%-26s %4d workgroups%s: %7.1f ns per iteration\n", name, blocks, note, ms * 1e6 / kIters);
    return 0;
}

template <int NV, int KIND, int NM>
int run_issue(const char* name, int blocks, float* out) {
    return timed(name, blocks, "", [&](int iters) { hipLaunchKernelGGL((issue_kernel<NV, KIND, NM>), blocks, 256, 0, 0, out, iters, 1.0f); });
}

template <int MODE>
int run_tile(const char* name, int blocks, int barrier, float* out) {
    return timed(name, blocks, barrier ? ", barrier per tile" : "",
                 [&](int iters) { hipLaunchKernelGGL((tile_kernel<MODE>), blocks, 256, 64 * 1024, 0, out, iters, barrier); });
}

template <int NREADS, int NDMA, bool SHARED = true>
int run_step(const char* name, float* out, const _Float16* src) {
    auto kern = step_kernel<NREADS, NDMA, SHARED>;
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024) != hipSuccess) return 1;
    return timed(name, 256, "", [&](int iters) { hipLaunchKernelGGL(kern, 256, 256, 128 * 1024, 0, out, src, iters); });
}

int main() {
    float* out;
    PROBE_CHECK(hipMalloc(&out, 1024 * 256 * 4));
    int bad = 0;
    for (int blocks : {256, 512}) {
        bad |= run_issue<0, 0, 8>("8 MFMA", blocks, out);
        bad |= run_issue<64, 0, 0>("64 fma", blocks, out);
        bad |= run_issue<64, 0, 8>("8 MFMA + 64 fma", blocks, out);
        bad |= run_issue<128, 0, 0>("128 fma", blocks, out);
        bad |= run_issue<128, 0, 8>("8 MFMA + 128 fma", blocks, out);
        bad |= run_issue<32, 1, 0>("32 exp", blocks, out);
        bad |= run_issue<32, 1, 8>("8 MFMA + 32 exp", blocks, out);
        bad |= run_issue<64, 1, 0>("64 exp", blocks, out);
        bad |= run_issue<64, 1, 8>("8 MFMA + 64 exp", blocks, out);
    }
    for (int blocks : {256, 512})
        for (int barrier : {0, 1}) {
            bad |= run_tile<0>("24 LDS reads + 16 MFMA", blocks, barrier, out);
            bad |= run_tile<1>("16 MFMA", blocks, barrier, out);
            bad |= run_tile<2>("24 LDS reads (+ 1 MFMA)", blocks, barrier, out);
        }
    _Float16* src;
    PROBE_CHECK(hipMalloc(&src, (size_t)64 << 20));
    PROBE_CHECK(hipMemset(src, 0, (size_t)64 << 20));
    bad |= run_step<0, 0>("step: 16 MFMA", out, src);
    bad |= run_step<16, 0>("step: + 16 reads", out, src);
    bad |= run_step<8, 0>("step: + 8 reads", out, src);
    bad |= run_step<0, 8>("step: + 8 transfers", out, src);
    bad |= run_step<16, 8>("step: + 16 reads + 8 tr.", out, src);
    bad |= run_step<8, 8>("step: + 8 reads + 8 tr.", out, src);
    bad |= run_step<16, 4>("step: + 16 reads + 4 tr.", out, src);
    bad |= run_step<16, 8, false>("step: 16 r. + 8 tr., own data", out, src);
    PROBE_CHECK(hipFree(src));
    PROBE_CHECK(hipFree(out));
    return bad;
}
