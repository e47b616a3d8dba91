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

__device__ __forceinline__ float apply_act(int act, float v) {
    switch (act) {
        case DMLHIP_ACT_GELU: return gelu_f(v);
        case DMLHIP_ACT_SWISH: return v * sigmoid_f(v);
        case DMLHIP_ACT_SIGMOID: return sigmoid_f(v);
        case DMLHIP_ACT_RELU: return fmaxf(v, 0.f);
        default: return v;
    }
}
inline bool valid_act(int act) { return act >= DMLHIP_ACT_NONE && act <= DMLHIP_ACT_RELU; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace dml
