// Shared device/host helpers for the gfx950 kernels behind the dmlhip_* C ABI.
//
// Conventions used by every translation unit:
//   * every entry point validates its arguments on the host first and returns a
//     negative status without touching the device when they are bad;
//   * a positive return value is the hipError_t of the failed launch;
//   * all kernels are asynchronous on the caller's stream, never synchronise,
//     never allocate and never keep a caller pointer after returning.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/daceml_hip.h"

namespace dml {

// ---------------------------------------------------------------- error text
void set_error(const char* fmt, ...);
int launch_status(const char* what);

#define DML_REQUIRE(cond, code, ...)            \
    do {                                        \
        if (!(cond)) {                          \
            ::dml::set_error(__VA_ARGS__);      \
            return (code);                      \
        }                                       \
    } while (0)

// ---------------------------------------------------------------- vectors
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

template <typename T> struct VecOf;  // 16-byte vector of T
template <> struct VecOf<_Float16> { using type = half8; static constexpr int n = 8; };
template <> struct VecOf<float> { using type = floatx4; static constexpr int n = 4; };

__device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }
__device__ __forceinline__ float to_f32(float v) { return v; }
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ _Float16 from_f32<_Float16>(float v) { return (_Float16)v; }
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }

// ---------------------------------------------------------------- wave reductions
// Reduce over the 64 lanes of a wavefront with DPP lane permutes inside each row
// of 16 lanes and four scalar lane reads across rows. Every lane gets the result.
struct OpSum { __device__ __forceinline__ static float f(float a, float b) { return a + b; } };
struct OpMax { __device__ __forceinline__ static float f(float a, float b) { return fmaxf(a, b); } };
struct OpMin { __device__ __forceinline__ static float f(float a, float b) { return fminf(a, b); } };

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
    return __builtin_bit_cast(float, r);
}

template <typename Op>
__device__ __forceinline__ float wave_reduce(float v) {
    v = Op::f(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    v = Op::f(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    v = Op::f(v, dpp_move<0x141>(v));  // row_half_mirror
    v = Op::f(v, dpp_move<0x140>(v));  // row_mirror
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return Op::f(Op::f(r0, r1), Op::f(r2, r3));
}

// Reduce over a whole workgroup of NWAVES wavefronts through LDS. `scratch` must hold
// NWAVES floats; the call contains barriers, so every thread has to reach it.
template <typename Op, int NWAVES>
__device__ __forceinline__ float block_reduce(float v, float* scratch) {
    v = wave_reduce<Op>(v);
    if constexpr (NWAVES == 1) return v;
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) r = Op::f(r, scratch[i]);
    return r;
}

// Second stage of the two-stage column reductions: out[c] = scale * Op over p < parts of
// part[p*row_stride + c]. 64 columns per workgroup, 16 wavefronts striding over the partial rows with
// several independent loads in flight each (the partial matrix is small, so this stage is latency
// bound and wants many short chains rather than few long ones). With `out1` set, columns >= cols0 go to
// out1[c - cols0]: two results that share one partial matrix finish in one launch.
template <typename Op, typename TOut>
__global__ __launch_bounds__(1024) void reduce_partials_kernel(const float* __restrict__ part, TOut* __restrict__ out,
                                                               int parts, int64_t row_stride, int64_t cols, float init,
                                                               float scale, TOut* __restrict__ out1, int64_t cols0) {
    __shared__ float lds[16][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t c = (int64_t)blockIdx.x * kWave + lane;
    float a0 = init, a1 = init, a2 = init, a3 = init;
    if (c < cols) {
        const float* base = part + c;
        int p = wave;
        for (; p + 48 < parts; p += 64) {
            const float v0 = base[(int64_t)p * row_stride];
            const float v1 = base[(int64_t)(p + 16) * row_stride];
            const float v2 = base[(int64_t)(p + 32) * row_stride];
            const float v3 = base[(int64_t)(p + 48) * row_stride];
            a0 = Op::f(a0, v0); a1 = Op::f(a1, v1); a2 = Op::f(a2, v2); a3 = Op::f(a3, v3);
        }
        for (; p < parts; p += 16) a0 = Op::f(a0, base[(int64_t)p * row_stride]);
    }
    lds[wave][lane] = Op::f(Op::f(a0, a1), Op::f(a2, a3));
    __syncthreads();
    if (wave == 0 && c < cols) {
        float a = lds[0][lane];
#pragma unroll
        for (int w = 1; w < 16; ++w) a = Op::f(a, lds[w][lane]);
        if (out1 && c >= cols0) out1[c - cols0] = from_f32<TOut>(a * scale);
        else out[c] = from_f32<TOut>(a * scale);
    }
}

// Same reduction for few, wide partial rows (split-K sums): every thread owns four consecutive columns
// and walks the `parts` rows with 128-bit loads. Requires cols % 4 == 0 and 16-byte aligned rows.
template <typename TOut>
__global__ __launch_bounds__(256) void sum_partials_vec4_kernel(const float* __restrict__ part, TOut* __restrict__ out,
                                                                int parts, int64_t row_stride, int64_t cols, float scale) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i * 4 < cols; i += stride) {
        floatx4 acc = *reinterpret_cast<const floatx4*>(part + i * 4);
        for (int p = 1; p < parts; ++p) {
            const floatx4 v = *reinterpret_cast<const floatx4*>(part + (int64_t)p * row_stride + i * 4);
            acc += v;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) out[i * 4 + e] = from_f32<TOut>(acc[e] * scale);
    }
}

// ---------------------------------------------------------------- math
// exact-GELU pieces; no fast-math anywhere on fp32 paths.
__device__ __forceinline__ float gelu_f(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
__device__ __forceinline__ float gelu_grad_f(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
    const float pdf = 0.39894228040143267794f * expf(-0.5f * x * x);
    return cdf + x * pdf;
}
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
// Sigmoid for fused epilogues, on the hardware exp2 and reciprocal (each accurate to about one ulp, so the result
// is within a few 1e-7 relative of sigmoid_f): an epilogue runs once per output element while the matrix pipe waits,
// and the library expf plus a true division cost several times the arithmetic of the product itself there.
__device__ __forceinline__ float sigmoid_epilogue_f(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * x));
}

// GELU and its derivative for fp16 tensors (not used on fp32 paths). With cdf the standard normal distribution function,
//     tail(x) = cdf(-|x|) = erfc(|x| / sqrt 2) / 2 = q(t) exp(-x^2 / 2),   t = 1 / (1 + 0.3275911 |x| / sqrt 2)
// by Abramowitz-Stegun 7.1.26 with halved coefficients (absolute error < 0.8e-7, far below the half-precision rounding
// of the results) on the hardware reciprocal and exp2, and
//     x cdf(x)          = max(x, 0) - |x| tail(x)                      (no cancellation for negative x)
//     cdf(x) + x pdf(x) = (x > 0 ? 1 - tail : tail) + x exp(-x^2 / 2) / sqrt(2 pi)
// Both kernels are bound by vector-instruction issue, so the forms are chosen for the fewest instructions: 12 and 15
// besides the conversions, two of them (reciprocal, exp2) at half rate.
__device__ __forceinline__ float gelu_tail_half_f(float x, float& ex) {
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(fabsf(x), 0.3275911f * 0.70710678118654752440f, 1.0f));
    const float q = t * (0.127414796f + t * (-0.142248368f + t * (0.7107068705f + t * (-0.7265760135f + t * 0.5307027145f))));
    ex = __builtin_amdgcn_exp2f((x * -0.72134752044448170368f) * x);   // exp(-x^2 / 2)
    return q * ex;
}

__device__ __forceinline__ float gelu_half_f(float x) {
    float ex;
    const float tail = gelu_tail_half_f(x, ex);
    return __builtin_fmaf(-fabsf(x), tail, fmaxf(x, 0.f));
}

__device__ __forceinline__ float gelu_grad_half_f(float x) {
    float ex;
    const float tail = gelu_tail_half_f(x, ex);
    const float cdf = x > 0.f ? 1.0f - tail : tail;
    return __builtin_fmaf(x * 0.39894228040143267794f, ex, cdf);
}

__device__ __forceinline__ float apply_act_half(int act, float v) {
    switch (act) {
        case DMLHIP_ACT_GELU: return gelu_half_f(v);
        case DMLHIP_ACT_SWISH: return v * sigmoid_f(v);
        case DMLHIP_ACT_SIGMOID: return sigmoid_f(v);
        case DMLHIP_ACT_RELU: return fmaxf(v, 0.f);
        default: return v;
    }
}

__device__ __forceinline__ float apply_act(int act, float v) {
    switch (act) {
        case DMLHIP_ACT_GELU: return gelu_f(v);
        case DMLHIP_ACT_SWISH: return v * sigmoid_epilogue_f(v);
        case DMLHIP_ACT_SIGMOID: return sigmoid_epilogue_f(v);
        case DMLHIP_ACT_RELU: return fmaxf(v, 0.f);
        default: return v;
    }
}
inline bool valid_act(int act) { return act >= DMLHIP_ACT_NONE && act <= DMLHIP_ACT_RELU; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// a / b for 0 <= a < 2^22 and 0 < b, with inv_b = 1.0f / b computed once: the float quotient is within one of the
// result and the remainder says which way. A handful of instructions where the integer division costs dozens.
__device__ __forceinline__ int fast_div(int a, int b, float inv_b) {
    int q = (int)((float)a * inv_b);
    const int r = a - q * b;
    q += (r >= b) - (r < 0);
    return q;
}

}  // namespace dml
