// Pieces shared by the fp16 GEMM kernels: launch arguments, the LDS chunk swizzle and the
// LDS-staged epilogue.
#pragma once

#include "common.h"

#include <type_traits>

namespace dml {
namespace gemm16 {

constexpr int kThreads = 256;
constexpr int BK = 64;         // K elements per step
constexpr int kRowBytes = BK * 2;
constexpr int kXcds = 8;

struct GemmArgs {
    int m, n, k;
    int64_t sam, sak, sbn, sbk, scm;
    int batch1, batch2;  // extents of the two inner batch dims (outer one is implied)
    int64_t sab[3], sbb[3], scb[3];
    float alpha, beta;
    int out_f32, bias_f32, act, bias_m, c_vec;
    int tiles_m, tiles_n;
    long long total_blocks;
};

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// ---------------------------------------------------------------- epilogue helper
// One wavefront writes a 32 x WN strip held in LDS (fp32, row pitch WN+4) to C: lane -> (row,
// eight consecutive columns). v = alpha*acc + bias; pre_out = v; v = act(v) + residual + beta*C.
// ACT = false compiles the activation switch out (most contractions have none).
template <typename OutT> struct OutVec;
template <> struct OutVec<_Float16> { typedef half8 type; };
template <> struct OutVec<float> { typedef float type __attribute__((ext_vector_type(8))); };

template <typename OutT, int WN, bool ACT>
__device__ __forceinline__ void store_strip(const GemmArgs& g, void* c_ptr, void* pre_ptr, const void* res_ptr,
                                            const void* bias_ptr, const float* strip, int mb, int nb, int64_t coff,
                                            int lane) {
    typedef typename OutVec<OutT>::type ovec;
    constexpr int PITCH = WN + 4;
    constexpr int CPR = WN / 8;
    constexpr int ITER = 32 * CPR / kWave;
    OutT* C = reinterpret_cast<OutT*>(c_ptr);
    OutT* P = reinterpret_cast<OutT*>(pre_ptr);
    const OutT* R = reinterpret_cast<const OutT*>(res_ptr);
    // A lane keeps its eight columns for the whole strip (64 % CPR == 0): the column bias is loaded once,
    // as one 128-bit access when it is aligned.
    float bias_n[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (bias_ptr && !g.bias_m) {
        const int n = nb + (lane % CPR) * 8;
        if (n + 8 <= g.n && ((reinterpret_cast<uintptr_t>(bias_ptr) + (size_t)n * (g.bias_f32 ? 4 : 2)) & 15) == 0) {
            if (g.bias_f32) {
                const floatx4 b0 = *reinterpret_cast<const floatx4*>(reinterpret_cast<const float*>(bias_ptr) + n);
                const floatx4 b1 = *reinterpret_cast<const floatx4*>(reinterpret_cast<const float*>(bias_ptr) + n + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { bias_n[e] = b0[e]; bias_n[e + 4] = b1[e]; }
            } else {
                const half8 b = *reinterpret_cast<const half8*>(reinterpret_cast<const _Float16*>(bias_ptr) + n);
#pragma unroll
                for (int e = 0; e < 8; ++e) bias_n[e] = (float)b[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int ne = min(n + e, g.n - 1);
                if (n < g.n) bias_n[e] = g.bias_f32 ? reinterpret_cast<const float*>(bias_ptr)[ne]
                                                     : (float)reinterpret_cast<const _Float16*>(bias_ptr)[ne];
            }
        }
    }
    // without an activation the body is small: unroll so that LDS reads and global stores of
    // several rows overlap; with one, keep few copies of the activation code
#pragma unroll(ACT ? 2 : 4)
    for (int it = 0; it < ITER; ++it) {
        const int idx = it * kWave + lane;
        const int r = idx / CPR, c8 = (idx % CPR) * 8;
        const int m = mb + r, n = nb + c8;
        if (m >= g.m || n >= g.n) continue;
        const floatx4 lo = *reinterpret_cast<const floatx4*>(strip + r * PITCH + c8);
        const floatx4 hi = *reinterpret_cast<const floatx4*>(strip + r * PITCH + c8 + 4);
        float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const int64_t off = coff + (int64_t)m * g.scm + n;
        const bool full = g.c_vec && n + 8 <= g.n;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= g.alpha;
        if (bias_ptr) {
            if (g.bias_m) {
                const float b = g.bias_f32 ? reinterpret_cast<const float*>(bias_ptr)[m]
                                           : (float)reinterpret_cast<const _Float16*>(bias_ptr)[m];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += b;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += bias_n[e];
            }
        }
        if (full) {
            if (P) {
                ovec pv;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    pv[e] = (OutT)v[e];
                    v[e] = (float)pv[e];  // the un-fused graph reads the stored pre-activation back
                }
                *reinterpret_cast<ovec*>(P + off) = pv;
            }
            if constexpr (ACT) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = apply_act_half(g.act, v[e]);
            }
            if (R) {
                const ovec rv = *reinterpret_cast<const ovec*>(R + off);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += (float)rv[e];
            }
            if (g.beta != 0.f) {
                const ovec cv = *reinterpret_cast<const ovec*>(C + off);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += g.beta * (float)cv[e];
            }
            ovec ov;
#pragma unroll
            for (int e = 0; e < 8; ++e) ov[e] = (OutT)v[e];
            *reinterpret_cast<ovec*>(C + off) = ov;
        } else {
            // ragged or unaligned tail: element by element (rare; kept out of line by the branch)
            const int cnt = min(8, g.n - n);
            float x = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (e < cnt) {
                    x = v[e];
                    if (P) {
                        const OutT h = (OutT)x;
                        P[off + e] = h;
                        x = (float)h;
                    }
                    if constexpr (ACT) x = apply_act_half(g.act, x);
                    if (R) x += (float)R[off + e];
                    if (g.beta != 0.f) x += g.beta * (float)C[off + e];
                    C[off + e] = (OutT)x;
                }
            }
        }
    }
}

// Launches the fully pipelined kernel (both operands straight to LDS). amode / bmode: 3 = K-contiguous,
// 4 = row-contiguous. Returns DMLHIP_ERR_UNSUPPORTED when no instantiation fits.
int launch_pipelined(GemmArgs& g, const _Float16* a, const _Float16* b, void* c, const void* bias, const void* residual,
                     void* pre, int amode, int bmode, int cfg, long long batch, hipStream_t st);

}  // namespace gemm16
}  // namespace dml
