// Pieces shared by the fp16 GEMM kernels: launch arguments, the LDS chunk swizzle and the
// LDS-staged epilogue.
#pragma once

#include "common.h"
#include "lds_ops.h"

#include <type_traits>

namespace dml {
namespace gemm16 {

constexpr int kThreads = 256;
constexpr int BK = 64;         // K elements per step
constexpr int kRowBytes = BK * 2;
constexpr int kXcds = 8;
constexpr int kCus = 256;   // compute units of an MI355X: what a "round" of workgroups means in the tile choice

struct GemmArgs {
    int m, n, k;
    int64_t sam, sak, sbn, sbk, scm;
    int batch1, batch2;  // extents of the two inner batch dims (outer one is implied)
    int64_t sab[3], sbb[3], scb[3];
    float alpha, beta;
    int out_f32, bias_f32, act, bias_m, c_vec;
    int tiles_m, tiles_n;
    long long total_blocks;
    // grouped launch: the outer batch index selects one of `groups` independent problems of identical shape and
    // strides (0 = an ordinary launch, pointers come from the kernel parameters). With `ksum` the groups are instead
    // concatenated along K: one output C = sum over groups of A_g B_g (only ga / gb are used).
    int groups, ksum;
    // optional second result: asum[m] = sum over k of A[m, k] (per group: gasum), written by the workgroups of the
    // first tile column; fp32 or fp16 elements
    void* asum;
    void* gasum[DMLHIP_GROUP_MAX];
    int asum_f32;
    // diagnostic (dmlhip_debug_gemm_trace): when set, every workgroup stores four readings of the 100 MHz wall clock -
    // start, first tile in LDS, end of the K loop, end of the epilogue - at trace[4 * workgroup]
    unsigned long long* trace;
    const _Float16* ga[DMLHIP_GROUP_MAX];
    const _Float16* gb[DMLHIP_GROUP_MAX];
    void* gc[DMLHIP_GROUP_MAX];
    const void* gbias[DMLHIP_GROUP_MAX];
};

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }
__device__ __forceinline__ int swz16(int row) { return (row & 7) ^ ((row >> 3) & 1); }  // period 16 rows

// ---------------------------------------------------------------- epilogue helpers
// The kernels issue the MFMA with the operands swapped (B fragment first): a lane then holds, for the
// output row m = lane % 32 of a 32x32 block, the columns n = 8*(e/4) + 4*(lane/32) + e%4 — four
// consecutive columns per group of four accumulator registers, which go to the LDS strip as one
// 128-bit write. PITCH = WN + 4 floats keeps both these writes and the row-wise reads of store_strip
// free of bank conflicts.
template <int TN, int PITCH>
__device__ __forceinline__ void stage_strip(float* strip, const floatx16 (&acc)[TN], int lane) {
    float* row = strip + (lane & 31) * PITCH + (lane >> 5) * 4;
    static_for<0, TN>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            floatx4 v = {acc[j][4 * q], acc[j][4 * q + 1], acc[j][4 * q + 2], acc[j][4 * q + 3]};
            *reinterpret_cast<floatx4*>(row + j * 32 + q * 8) = v;
        }
    });
}

// One wavefront writes a 32 x WN strip held in LDS (fp32, row pitch WN+4) to C: lane -> (row,
// eight consecutive columns). v = alpha*acc + bias; pre_out = v; v = act(v) + residual + beta*C.
// ACT = false compiles the activation switch out (most contractions have none).
template <typename OutT> struct OutVec;
template <> struct OutVec<_Float16> { typedef half8 type; };
template <> struct OutVec<float> { typedef float type __attribute__((ext_vector_type(8))); };

// Epilogue variants (template parameter EPI), chosen on the host so that the common cases carry no
// loads inside the store loop: on this target loads and stores share one completion counter and
// complete out of order with respect to each other, so any wait for a load also waits for every
// store issued before it (a full write round trip per iteration).
//   EPI_PLAIN    v = alpha*acc + bias[n]                       -> C
//   EPI_ACT      same, pre_out = v, v = act(v)                 -> C (and pre-activation)   no loads
//   EPI_GENERAL  + bias along m, residual, beta*C               (loads per strip, issued before the stores)
//   EPI_GENERAL_ACT  EPI_GENERAL with the activation switch compiled in
constexpr int EPI_PLAIN = 0, EPI_ACT = 1, EPI_GENERAL = 2, EPI_GENERAL_ACT = 3;

inline int epilogue_kind(const GemmArgs& g, const void* bias, const void* residual, const void* pre) {
    const bool loads = residual || g.beta != 0.f || (bias && g.bias_m);
    const bool act = g.act != DMLHIP_ACT_NONE;
    if (loads) return act ? EPI_GENERAL_ACT : EPI_GENERAL;
    return (act || pre) ? EPI_ACT : EPI_PLAIN;
}

// The eight column-bias values of a lane (its columns are the same for every strip of the wavefront's tile, so
// this runs once, before the first store).
template <int WN>
__device__ __forceinline__ void load_bias_n(const GemmArgs& g, const void* bias_ptr, int nb, int lane, float (&bias_n)[8]) {
    constexpr int CPR = WN / 8;
    const int n = nb + (lane % CPR) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) bias_n[e] = 0.f;
    if (!bias_ptr || g.bias_m || n >= g.n) return;
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
            bias_n[e] = g.bias_f32 ? reinterpret_cast<const float*>(bias_ptr)[ne]
                                   : (float)reinterpret_cast<const _Float16*>(bias_ptr)[ne];
        }
    }
}

template <typename OutT, int WN, int EPI>
__device__ __forceinline__ void store_strip(const GemmArgs& g, void* c_ptr, void* pre_ptr, const void* res_ptr,
                                            const void* bias_ptr, const float (&bias_n)[8], const float* strip, int mb,
                                            int nb, int64_t coff, int lane) {
    typedef typename OutVec<OutT>::type ovec;
    constexpr int PITCH = WN + 4;
    constexpr int CPR = WN / 8;
    constexpr int ITER = 32 * CPR / kWave;
    constexpr int RSTEP = kWave / CPR;  // rows between two iterations of a lane
    constexpr bool ACT = EPI == EPI_ACT || EPI == EPI_GENERAL_ACT;
    constexpr bool GENERAL = EPI == EPI_GENERAL || EPI == EPI_GENERAL_ACT;
    OutT* C = reinterpret_cast<OutT*>(c_ptr);
    OutT* P = reinterpret_cast<OutT*>(pre_ptr);
    const OutT* R = reinterpret_cast<const OutT*>(res_ptr);
    // A lane keeps its eight columns for the whole strip (64 % CPR == 0).
    const int r0 = lane / CPR, c8 = (lane % CPR) * 8;
    const int n = nb + c8;
    if (n >= g.n) return;
    const bool full = g.c_vec && n + 8 <= g.n;
    const int64_t off0 = coff + (int64_t)(mb + r0) * g.scm + n;
    const int64_t rstep = (int64_t)RSTEP * g.scm;

    if (full) {
        // operands that have to be loaded (general variants only): all of the strip's loads first
        ovec rv[GENERAL ? ITER : 1], cv[GENERAL ? ITER : 1];
        float bm[GENERAL ? ITER : 1];
        if constexpr (GENERAL) {
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const int m = min(mb + r0 + it * RSTEP, g.m - 1);
                const int64_t off = coff + (int64_t)m * g.scm + n;
                if (R) rv[it] = *reinterpret_cast<const ovec*>(R + off);
                if (g.beta != 0.f) cv[it] = *reinterpret_cast<const ovec*>(C + off);
                bm[it] = 0.f;
                if (bias_ptr && g.bias_m)
                    bm[it] = g.bias_f32 ? reinterpret_cast<const float*>(bias_ptr)[m]
                                        : (float)reinterpret_cast<const _Float16*>(bias_ptr)[m];
            }
        }
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int r = r0 + it * RSTEP;
            if (mb + r >= g.m) break;
            const floatx4 lo = *reinterpret_cast<const floatx4*>(strip + r * PITCH + c8);
            const floatx4 hi = *reinterpret_cast<const floatx4*>(strip + r * PITCH + c8 + 4);
            float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const int64_t off = off0 + it * rstep;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = v[e] * g.alpha + bias_n[e];
            if constexpr (GENERAL) {
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += bm[it];
            }
            if constexpr (EPI != EPI_PLAIN) {
                if (P) {
                    ovec pv;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        pv[e] = (OutT)v[e];
                        v[e] = (float)pv[e];  // the un-fused graph reads the stored pre-activation back
                    }
                    *reinterpret_cast<ovec*>(P + off) = pv;
                }
            }
            if constexpr (ACT) {
                // the activation is chosen once per store, not once per element: with the five-way choice inside the
                // unrolled element loop the epilogue grows to tens of thousands of instructions and runs out of the
                // instruction cache
                if (g.act == DMLHIP_ACT_GELU) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = gelu_half_f(v[e]);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = apply_act_half(g.act, v[e]);
                }
            }
            if constexpr (GENERAL) {
                if (R) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += (float)rv[it][e];
                }
                if (g.beta != 0.f) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += g.beta * (float)cv[it][e];
                }
            }
            ovec ov;
#pragma unroll
            for (int e = 0; e < 8; ++e) ov[e] = (OutT)v[e];
            // fp16 results (what the next kernel reads) go through the L2 as they are written; the fp32 ones (weight
            // gradients, read by nobody in the step) measured no faster that way
            if constexpr (sizeof(OutT) == 2) global_store_b128_through(C + off, ov);
            else *reinterpret_cast<ovec*>(C + off) = ov;
        }
    } else {
        // ragged or unaligned columns: element by element (rare)
        const int cnt = min(8, g.n - n);
        for (int it = 0; it < ITER; ++it) {
            const int r = r0 + it * RSTEP, m = mb + r;
            if (m >= g.m) break;
            const int64_t off = off0 + it * rstep;
            float bmv = 0.f;
            if (bias_ptr && g.bias_m)
                bmv = g.bias_f32 ? reinterpret_cast<const float*>(bias_ptr)[m]
                                 : (float)reinterpret_cast<const _Float16*>(bias_ptr)[m];
            for (int e = 0; e < cnt; ++e) {
                float x = strip[r * PITCH + c8 + e] * g.alpha + bias_n[e] + bmv;
                if (P) {
                    const OutT h = (OutT)x;
                    P[off + e] = h;
                    x = (float)h;
                }
                if (g.act != DMLHIP_ACT_NONE) x = apply_act_half(g.act, x);
                if (R) x += (float)R[off + e];
                if (g.beta != 0.f) x += g.beta * (float)C[off + e];
                C[off + e] = (OutT)x;
            }
        }
    }
}

// Launches the fully pipelined kernel (both operands straight to LDS). amode / bmode: 3 = K-contiguous,
// 4 = row-contiguous. Returns DMLHIP_ERR_UNSUPPORTED when no instantiation fits.
int launch_pipelined(GemmArgs& g, const _Float16* a, const _Float16* b, void* c, const void* bias, const void* residual,
                     void* pre, int amode, int bmode, int cfg, long long batch, hipStream_t st);
// Configurations 4 - 7 and 9 (the interleaved K loop on the tiles of 2, 0, 1, 3 and 8); ak / bk: 0 = K-contiguous, 1 = row-contiguous.
int launch_pipelined_ilv(GemmArgs& g, const _Float16* a, const _Float16* b, void* c, const void* bias, const void* residual,
                         void* pre, int ak, int bk, int cfg, long long batch, hipStream_t st);

}  // namespace gemm16
}  // namespace dml
