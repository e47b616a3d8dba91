// Fused scaled-dot-product attention for fp16 tensors with head dimension 64:
//     O = softmax(scale * Q K^T [+ mask]) V          (no dropout; softmax over the key axis)
// without materialising the [Sq, Sk] score matrix in HBM, and its backward pass. It replaces the chain
// Einsum(Q,K) -> Mul/Div(scale) [-> Add(mask)] -> Softmax(axis=-1) -> Einsum(P,V) of the reference
// (daceml/onnx/op_implementations/pure_implementations.py:219-252, 34-36, 309-319) and, in backward, the nodes
// emitted by daceml/autodiff/implementations/onnx_ops.py:25-138 and :237-275 for that chain. The optional additive
// mask is one fp16 row of seq_k values per (batch0, batch1), the same for every query (the padding mask of a BERT
// encoder, [batch, 1, 1, keys]); the kernels without it are separate instantiations.
//
// Work decomposition (forward): a workgroup of four wavefronts owns 128 query rows of one (batch, head);
// each wavefront owns 32 of them. K and V stream through a three-stage LDS ring in tiles of 64 keys
// (global_load_lds, 16 bytes per lane). Per tile a wavefront computes
//     S^T[key, q] = K Q^T           v_mfma_f32_32x32x16_f16, A = K rows from LDS, B = Q (registers)
// so that a lane holds ONE query column and 32 keys: the running row maximum and sum of the online
// softmax are per-lane scalars (one exchange with lane^32 per tile), and the fp16 probabilities are,
// without any shuffle, the B operand of
//     O^T[d, q] += V^T P^T          A = V^T via LDS transpose reads (ds_read_b64_tr_b16)
// The key order inside a 16-key MFMA step is permuted ({0..3, 8..11} for lanes 0-31, {4..7, 12..15} for
// lanes 32-63) — harmless for a contraction index as long as V^T is read with the same permutation.
//
// LDS tile layout (K, V, and Q / dO in the backward kernels): [64 rows][64 halves], 128-byte rows, the
// 16-byte chunk c of row r stored at slot c ^ f(r), f(r) = (r>>2 & 3) | ((r>>1 & 1) << 2): conflict-free both
// for 128-bit row reads (contraction over d) and for transpose reads (contraction over rows).
#include "common.h"
#include "lds_ops.h"

#include <type_traits>

namespace dml {
namespace {

constexpr int kAttnThreads = 256;
constexpr float kLog2eF = 1.44269504088896340736f;
constexpr int kTileBytes = 64 * 128;  // one [64][64] fp16 tile

struct AttnArgs {
    int batch1, seq_q, seq_k, q_tiles, k_tiles;
    long long total_blocks;
    int64_t qs[3], ks[3], vs[3], os[3];       // element strides: batch0, batch1, sequence (head dim stride 1)
    int64_t dqs[3], dks[3], dvs[3], dos[3];   // gradient tensors (backward only)
    float scale, scale_log2;
    unsigned long long* trace;                // diagnostic: 16 readings of the 100 MHz clock per workgroup, or NULL
};

// the additive mask: row (b0, b1) starts at mask + b0 * ms[0] + b1 * ms[1] (a stride of 0 broadcasts), keys contiguous
struct AttnArgsMasked : AttnArgs {
    const _Float16* mask;
    int64_t ms[2];
};
template <bool MASK> using AttnArgsFor = std::conditional_t<MASK, AttnArgsMasked, AttnArgs>;

template <int I, int N, typename F>
__device__ __forceinline__ void static_for_attn(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_attn<I + 1, N>(f);
    }
}

// slot 0: start; 1: first tile in LDS; 2 + j: end of key tile j (j < 12); 15: end of the kernel
__device__ __forceinline__ void trace_stamp(const AttnArgs& a, int slot) {
    if (a.trace && threadIdx.x == 0) a.trace[16 * (size_t)blockIdx.x + slot] = wall_clock64();
}

__device__ __forceinline__ int swz_rt(int r) { return ((r >> 2) & 3) | (((r >> 1) & 1) << 2); }

// Per-lane geometry of the 16-byte DMA pieces of a [64][64] tile: two instructions per wavefront.
struct TileDma {
    int row[2], col[2];
    __device__ __forceinline__ void init(int wave, int lane) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int r = (i * 4 + wave) * 8 + (lane >> 3);
            row[i] = r;
            col[i] = ((lane & 7) ^ swz_rt(r)) * 8;
        }
    }
    // rows r0 .. r0+63 of a matrix with `stride` elements between rows; rows beyond rmax re-read row rmax
    __device__ __forceinline__ void issue(const _Float16* base, int64_t stride, int r0, int rmax, char* tile,
                                          int wave) const {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int r = min(r0 + row[i], rmax);
            lds_dma16(base + (int64_t)r * stride + col[i], tile + (i * 4 + wave) * 1024);
        }
    }
};

// Fragment addresses inside a tile (relative to the tile base).
struct TileFrags {
    uint32_t rowread[4];   // 128-bit row reads: [16-wide step of the contracted (head) dimension]
    uint32_t trread[2][2]; // transpose reads: [32-wide block of the head dimension][first / second 4 rows]
    __device__ __forceinline__ void init(int lane) {
        const int r = lane & 31, h = lane >> 5;
#pragma unroll
        for (int st = 0; st < 4; ++st) rowread[st] = r * 128 + (((st * 2 + h) ^ swz_rt(r)) << 4);
        const int s = lane & 15, grp = lane >> 4, hh = grp >> 1;
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) {
                const int k = 4 * hh + 8 * hi + (s >> 2);            // row inside a 16-row step
                const int d0 = blk * 32 + (grp & 1) * 16 + 4 * (s & 3);
                trread[blk][hi] = k * 128 + (((d0 >> 3) ^ swz_rt(k)) << 4) + (d0 & 7) * 2;
            }
    }
};

// Lanes l and l^32 hold the two halves of one row's keys (or head elements): combine through the LDS
// crossbar (ds_bpermute), which moves no data through LDS memory.
__device__ __forceinline__ float other_half(float v) {
    const int idx = ((int)(threadIdx.x & 63) ^ 32) << 2;
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(idx, __builtin_bit_cast(int, v)));
}
__device__ __forceinline__ float cross_half_max(float v) { return fmaxf(v, other_half(v)); }
__device__ __forceinline__ float cross_half_sum(float v) { return v + other_half(v); }

// Two transpose reads (rows 0..3 and 8..11 of a 16-row step, say) joined into one MFMA operand.
template <int OFF>
[[nodiscard]] __device__ __forceinline__ half8 tr_pair(uint32_t lo_addr, uint32_t hi_addr) {
    const half4v lo = lds_read_tr16_b64<OFF>(lo_addr);
    const half4v hi = lds_read_tr16_b64<OFF>(hi_addr);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// The mask values of the 32 keys a lane holds of key tile j in the forward and dQ kernels, as loaded:
// mk[blk * 4 + g][e] belongs to key 64*j + 32*blk + 8*g + 4*h + e. Whole tiles are read eight bytes at a time (the host
// checks the alignment); the last, partial tile element by element with the index clamped to the row.
__device__ __forceinline__ void load_mask_tile(const _Float16* row, int j, int h, int seq_k, half4v (&mk)[8]) {
    const int base = j * 64 + h * 4;
    if ((j + 1) * 64 <= seq_k) {
#pragma unroll
        for (int i = 0; i < 8; ++i) mk[i] = *reinterpret_cast<const half4v*>(row + base + (i >> 2) * 32 + (i & 3) * 8);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) mk[i][e] = row[min(base + (i >> 2) * 32 + (i & 3) * 8 + e, seq_k - 1)];
    }
}

__device__ __forceinline__ void decode_block(const AttnArgs& a, int tiles, long long& bid, int& b0, int& b1, int& tile) {
    // XCD-aware: consecutive tiles of one (batch, head) share K/V (or Q/dO) and should share an L2. 32-bit arithmetic
    // (the host checks total_blocks < 2^31): 64-bit divisions are long software sequences, and nothing can be requested
    // from memory before this is done.
    const uint32_t total = (uint32_t)a.total_blocks, b = (uint32_t)bid;
    const uint32_t xcd = b % 8u, idx = b / 8u;
    const uint32_t base = total / 8u, rem = total % 8u;
    const uint32_t id = xcd * base + (xcd < rem ? xcd : rem) + idx;
    const uint32_t bh = id / (uint32_t)tiles;
    tile = (int)(id - bh * (uint32_t)tiles);
    const uint32_t hi = bh / (uint32_t)a.batch1;
    b1 = (int)(bh - hi * (uint32_t)a.batch1);
    b0 = (int)hi;
    bid = id;
}

// One [32 q] x [64 d] fp16 result per wavefront, held transposed (acc[blk][e]: d = 32*blk + 8*(e/4) + 4*(lane/32)
// + e%4, q = lane%32), written through a 4 KB LDS region so that global stores are 128-bit and row-contiguous.
__device__ __forceinline__ void store_rows_t(const floatx16 (&acc)[2], float mul, char* region, _Float16* out,
                                             int64_t stride, int row0, int rows, int lane) {
    const int q = lane & 31, h = lane >> 5;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            half4v v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = (_Float16)(acc[blk][4 * g + e] * mul);
            *reinterpret_cast<half4v*>(region + q * 128 + (((blk * 4 + g) ^ ((q >> 1) & 7)) << 4) + h * 8) = v;
        }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int r = it * 8 + (lane >> 3), c = lane & 7;
        const half8 v = *reinterpret_cast<const half8*>(region + r * 128 + ((c ^ ((r >> 1) & 7)) << 4));
        if (row0 + r < rows) global_store_b128_through(out + (int64_t)(row0 + r) * stride + c * 8, v);
    }
    __builtin_amdgcn_wave_barrier();
}

// ---------------------------------------------------------------- forward
constexpr int kFwdStages = 3;

template <bool MASK>
__global__ __launch_bounds__(kAttnThreads, 2) void attention_fwd_kernel(const _Float16* __restrict__ q_ptr,
                                                                        const _Float16* __restrict__ k_ptr,
                                                                        const _Float16* __restrict__ v_ptr,
                                                                        _Float16* __restrict__ o_ptr,
                                                                        float* __restrict__ lse_ptr,
                                                                        const AttnArgsFor<MASK> a) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    constexpr int STAGE = 2 * kTileBytes;
    trace_stamp(a, 0);
    long long bid = blockIdx.x;
    int b0, b1, qt;
    decode_block(a, a.q_tiles, bid, b0, b1, qt);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5;
    const int q0 = qt * 128 + wave * 32;

    const _Float16* Q = q_ptr + b0 * a.qs[0] + b1 * a.qs[1];
    const _Float16* K = k_ptr + b0 * a.ks[0] + b1 * a.ks[1];
    const _Float16* V = v_ptr + b0 * a.vs[0] + b1 * a.vs[1];
    const _Float16* mask_row = nullptr;
    if constexpr (MASK) mask_row = a.mask + b0 * a.ms[0] + b1 * a.ms[1];

    // Q fragments (B operand of S^T = K Q^T): lane -> query row lane%32, head elements 16*st + 8*h .. +7
    half8 qf[4];
    {
        const _Float16* qp = Q + (int64_t)min(q0 + (lane & 31), a.seq_q - 1) * a.qs[2] + h * 8;
#pragma unroll
        for (int st = 0; st < 4; ++st) qf[st] = *reinterpret_cast<const half8*>(qp + st * 16);
    }

    TileDma dma;
    dma.init(wave, lane);
    TileFrags fr;
    fr.init(lane);
    const uint32_t lds0 = lds_addr(lds);
    const int nk = a.k_tiles;
    const int kmax = a.seq_k - 1;

    // prologue: tiles 0 and 1 in flight
#pragma unroll
    for (int s = 0; s < kFwdStages - 1; ++s)
        if (s < nk) {
            dma.issue(K, a.ks[2], s * 64, kmax, lds + s * STAGE, wave);
            dma.issue(V, a.vs[2], s * 64, kmax, lds + s * STAGE + kTileBytes, wave);
        }

    floatx16 oacc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[i][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    int stage = 0;
    for (int j = 0; j < nk; ++j) {
        // tile j has landed for this wavefront once at most the newer tile's four transfers are outstanding
        if (j + 1 < nk) wait_vm_lgkm0<4>();
        else wait_vm_lgkm0<0>();
        __builtin_amdgcn_s_barrier();
        if (j == 0) trace_stamp(a, 1);
        // ahead of the refill below, so that waiting for these loads does not wait for the transfers issued after them
        half4v mk[MASK ? 8 : 1];
        if constexpr (MASK) load_mask_tile(mask_row, j, h, a.seq_k, mk);
        // every wavefront has finished tile j-1: its stage takes tile j+2
        if (j + kFwdStages - 1 < nk) {
            const int fs = stage == 0 ? kFwdStages - 1 : stage - 1;
            dma.issue(K, a.ks[2], (j + kFwdStages - 1) * 64, kmax, lds + fs * STAGE, wave);
            dma.issue(V, a.vs[2], (j + kFwdStages - 1) * 64, kmax, lds + fs * STAGE + kTileBytes, wave);
        }
        const uint32_t kt = lds0 + stage * STAGE, vt = kt + kTileBytes;

        // ---- S^T = K Q^T for 64 keys x 32 queries
        half8 kf[2][4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            kf[0][st] = lds_read_b128<0>(kt + fr.rowread[st]);
            kf[1][st] = lds_read_b128<4096>(kt + fr.rowread[st]);
        }
        floatx16 sacc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[i][e] = 0.f;
        wait_lgkm<0>();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[0][st], qf[st], sacc[0], 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[1][st], qf[st], sacc[1], 0, 0, 0);
        }

        // ---- V^T fragments for the second product: in flight during the softmax arithmetic
        half8 vf[2][4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            half4v lo, hi;
            lo = lds_read_tr16_b64<0 * 2048>(vt + fr.trread[blk][0]); hi = lds_read_tr16_b64<0 * 2048>(vt + fr.trread[blk][1]);
            vf[blk][0] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            lo = lds_read_tr16_b64<1 * 2048>(vt + fr.trread[blk][0]); hi = lds_read_tr16_b64<1 * 2048>(vt + fr.trread[blk][1]);
            vf[blk][1] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            lo = lds_read_tr16_b64<2 * 2048>(vt + fr.trread[blk][0]); hi = lds_read_tr16_b64<2 * 2048>(vt + fr.trread[blk][1]);
            vf[blk][2] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            lo = lds_read_tr16_b64<3 * 2048>(vt + fr.trread[blk][0]); hi = lds_read_tr16_b64<3 * 2048>(vt + fr.trread[blk][1]);
            vf[blk][3] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }

        // ---- online softmax over the key axis; the lane's query is lane%32, its keys are
        // 64*j + 32*blk + 8*(e/4) + 4*h + e%4
        // (scale > 0, checked on the host: the maximum is taken over the raw scores and scaled once, and scale and
        // shift of the exponent's argument are one fused multiply-add per score)
        float mt = -INFINITY;
        const bool ragged = (j + 1) * 64 > a.seq_k;
        if constexpr (MASK) {
            // the mask shifts every score by its own amount: scale and shift first, then the maximum
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    sacc[blk][e] = __builtin_fmaf(sacc[blk][e], a.scale_log2, (float)mk[blk * 4 + (e >> 2)][e & 3] * kLog2eF);
        }
        if (ragged) {
            // a branch of its own (the empty statement keeps the compiler from turning it into 32 compare-and-select
            // pairs that every tile would pay for): only a last, partial tile has keys to take out
            asm volatile("");
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = j * 64 + blk * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
                    if (key >= a.seq_k) sacc[blk][e] = -INFINITY;
                }
        }
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int e = 0; e < 16; ++e) mt = fmaxf(mt, sacc[blk][e]);
        mt = cross_half_max(mt);
        const float m_new = fmaxf(m_run, MASK ? mt : mt * a.scale_log2);
        // a mask may hold -inf for every key seen so far: keep the exponents' arguments free of (-inf) - (-inf)
        const float m_use = MASK && m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        m_run = m_new;
        float psum = 0.f;
        half8 pf[4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float p = MASK ? __builtin_amdgcn_exp2f(sacc[blk][e] - m_use)
                                     : __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[blk][e], a.scale_log2, -m_new));
                psum += p;
                pf[blk * 2 + (e >> 3)][e & 7] = (_Float16)p;
            }
        l_run = l_run * alpha + psum;
        // once the running maxima have settled every alpha is 1 and the accumulators need no rescaling
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int e = 0; e < 16; ++e) oacc[blk][e] *= alpha;
        }

        // ---- O^T += V^T P^T
        wait_lgkm<0>();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            oacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[0][s], pf[s], oacc[0], 0, 0, 0);
            oacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[1][s], pf[s], oacc[1], 0, 0, 0);
        }
        stage = stage + 1 == kFwdStages ? 0 : stage + 1;
        if (j < 12) trace_stamp(a, 2 + j);
    }

    const float l_tot = cross_half_sum(l_run);
    const float inv = 1.0f / l_tot;
    if (lse_ptr && lane < 32 && q0 + lane < a.seq_q)
        lse_ptr[((int64_t)b0 * a.batch1 + b1) * a.seq_q + q0 + lane] =
            (m_run + __builtin_amdgcn_logf(l_tot)) * 0.69314718055994530942f;
    __syncthreads();  // all fragment reads of the last tiles are done: the ring becomes staging space
    store_rows_t(oacc, inv, lds + wave * 4096, o_ptr + b0 * a.os[0] + b1 * a.os[1], a.os[2], q0, a.seq_q, lane);
    trace_stamp(a, 15);
}


// ---------------------------------------------------------------- backward
// Two kernels, no atomics (results are deterministic):
//   attention_bwd_dq_kernel   workgroup = 128 query rows, streams K and V tiles. Recomputes
//       P^T = exp(scale*K Q^T - lse), dP^T = V dO^T, dS^T = P^T * (dP^T - D), accumulates dQ^T += K^T dS^T.
//       Also produces D[q] = sum_d dO[q,d] O[q,d] (its dO / O fragments hold the rows) for the second kernel.
//   attention_bwd_dkv_kernel  workgroup = 128 key rows, streams Q and dO tiles (with lse and D).
//       Recomputes P = exp(scale*Q K^T - lse), dP = dO V^T, dS = P * (dP - D); dV^T += dO^T P, dK^T += Q^T dS.
// In both, the lane that owns an output row keeps it across the whole loop, the recomputed probabilities are
// used as MFMA B operands straight from the accumulator registers (same key/query permutation trick as the
// forward kernel) and the transposed operands come from LDS transpose reads of the same tiles.
constexpr int kBwdStages = 3;
constexpr float kLog2e = 1.44269504088896340736f;

[[nodiscard]] __device__ __forceinline__ floatx4 lds_read_f32x4(uint32_t addr) {
    floatx4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}

template <bool MASK>
__global__ __launch_bounds__(kAttnThreads, 2) void attention_bwd_dq_kernel(
    const _Float16* __restrict__ q_ptr, const _Float16* __restrict__ k_ptr, const _Float16* __restrict__ v_ptr,
    const _Float16* __restrict__ o_ptr, const float* __restrict__ lse_ptr, const _Float16* __restrict__ do_ptr,
    _Float16* __restrict__ dq_ptr, float* __restrict__ dvec_ptr, const AttnArgsFor<MASK> a) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    constexpr int STAGE = 2 * kTileBytes;
    trace_stamp(a, 0);
    long long bid = blockIdx.x;
    int b0, b1, qt;
    decode_block(a, a.q_tiles, bid, b0, b1, qt);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5;
    const int q0 = qt * 128 + wave * 32;
    const int qrow = min(q0 + (lane & 31), a.seq_q - 1);
    const int64_t bh = (int64_t)b0 * a.batch1 + b1;

    const _Float16* K = k_ptr + b0 * a.ks[0] + b1 * a.ks[1];
    const _Float16* V = v_ptr + b0 * a.vs[0] + b1 * a.vs[1];
    const _Float16* mask_row = nullptr;
    if constexpr (MASK) mask_row = a.mask + b0 * a.ms[0] + b1 * a.ms[1];

    // the first two K / V tiles are requested before anything else: the row loads below (and the row dots that wait for
    // them) then run while the tiles are on their way, instead of ahead of them
    TileDma dma;
    dma.init(wave, lane);
    TileFrags fr;
    fr.init(lane);
    const uint32_t lds0 = lds_addr(lds);
    const int nk = a.k_tiles;
    const int kmax = a.seq_k - 1;
#pragma unroll
    for (int s = 0; s < kBwdStages - 1; ++s)
        if (s < nk) {
            dma.issue(K, a.ks[2], s * 64, kmax, lds + s * STAGE, wave);
            dma.issue(V, a.vs[2], s * 64, kmax, lds + s * STAGE + kTileBytes, wave);
        }

    half8 qf[4], dof[4];
    float dsum = 0.f;
    {
        const _Float16* qp = q_ptr + b0 * a.qs[0] + b1 * a.qs[1] + (int64_t)qrow * a.qs[2] + h * 8;
        const _Float16* gp = do_ptr + b0 * a.dos[0] + b1 * a.dos[1] + (int64_t)qrow * a.dos[2] + h * 8;
        const _Float16* op = o_ptr + b0 * a.os[0] + b1 * a.os[1] + (int64_t)qrow * a.os[2] + h * 8;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            qf[st] = *reinterpret_cast<const half8*>(qp + st * 16);
            dof[st] = *reinterpret_cast<const half8*>(gp + st * 16);
            const half8 of = *reinterpret_cast<const half8*>(op + st * 16);
#pragma unroll
            for (int e = 0; e < 8; ++e) dsum += (float)dof[st][e] * (float)of[e];
        }
    }
    const float dvec = cross_half_sum(dsum);
    if (lane < 32 && q0 + lane < a.seq_q) dvec_ptr[bh * a.seq_q + q0 + lane] = dvec;
    const float lse2 = lse_ptr[bh * a.seq_q + qrow] * kLog2e;

    floatx16 dqacc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) dqacc[i][e] = 0.f;

    int stage = 0;
    for (int j = 0; j < nk; ++j) {
        if (j + 1 < nk) wait_vm_lgkm0<4>();
        else wait_vm_lgkm0<0>();
        __builtin_amdgcn_s_barrier();
        if (j == 0) trace_stamp(a, 1);
        half4v mk[MASK ? 8 : 1];   // ahead of the refill, as in the forward kernel
        if constexpr (MASK) load_mask_tile(mask_row, j, h, a.seq_k, mk);
        if (j + kBwdStages - 1 < nk) {
            const int fs = stage == 0 ? kBwdStages - 1 : stage - 1;
            dma.issue(K, a.ks[2], (j + kBwdStages - 1) * 64, kmax, lds + fs * STAGE, wave);
            dma.issue(V, a.vs[2], (j + kBwdStages - 1) * 64, kmax, lds + fs * STAGE + kTileBytes, wave);
        }
        const uint32_t kt = lds0 + stage * STAGE, vt = kt + kTileBytes;

        half8 kf[2][4], vr[2][4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            kf[0][st] = lds_read_b128<0>(kt + fr.rowread[st]);
            kf[1][st] = lds_read_b128<4096>(kt + fr.rowread[st]);
        }
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            vr[0][st] = lds_read_b128<0>(vt + fr.rowread[st]);
            vr[1][st] = lds_read_b128<4096>(vt + fr.rowread[st]);
        }
        floatx16 sacc[2], pacc[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) { sacc[i][e] = 0.f; pacc[i][e] = 0.f; }
        wait_lgkm<0>();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[0][st], qf[st], sacc[0], 0, 0, 0);
            sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[1][st], qf[st], sacc[1], 0, 0, 0);
            pacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vr[0][st], dof[st], pacc[0], 0, 0, 0);
            pacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vr[1][st], dof[st], pacc[1], 0, 0, 0);
        }
        // K^T fragments for dQ^T += K^T dS^T, in flight during the elementwise part
        half8 ktf[2][4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            ktf[blk][0] = tr_pair<0 * 2048>(kt + fr.trread[blk][0], kt + fr.trread[blk][1]);
            ktf[blk][1] = tr_pair<1 * 2048>(kt + fr.trread[blk][0], kt + fr.trread[blk][1]);
            ktf[blk][2] = tr_pair<2 * 2048>(kt + fr.trread[blk][0], kt + fr.trread[blk][1]);
            ktf[blk][3] = tr_pair<3 * 2048>(kt + fr.trread[blk][0], kt + fr.trread[blk][1]);
        }
        // only a last, partial tile has keys to take out: their scores become -inf in a branch of its own, ahead of the
        // exponentials (the empty statement keeps the compiler from turning the branch into 32 compare-and-select
        // pairs that every tile would pay for)
        if ((j + 1) * 64 > a.seq_k) {
            asm volatile("");
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = j * 64 + blk * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
                    if (key >= a.seq_k) sacc[blk][e] = -INFINITY;
                }
        }
        // dS^T = P^T * (dP^T - D), P^T recomputed from the scores
        half8 dsf[4];
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float p;
                if constexpr (MASK)
                    p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[blk][e], a.scale_log2,
                                                              (float)mk[blk * 4 + (e >> 2)][e & 3] * kLog2eF) - lse2);
                else
                    p = __builtin_amdgcn_exp2f(sacc[blk][e] * a.scale_log2 - lse2);
                dsf[blk * 2 + (e >> 3)][e & 7] = (_Float16)(p * (pacc[blk][e] - dvec));
            }
        wait_lgkm<0>();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            dqacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ktf[0][s], dsf[s], dqacc[0], 0, 0, 0);
            dqacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ktf[1][s], dsf[s], dqacc[1], 0, 0, 0);
        }
        stage = stage + 1 == kBwdStages ? 0 : stage + 1;
        if (j < 12) trace_stamp(a, 2 + j);
    }
    __syncthreads();
    store_rows_t(dqacc, a.scale, lds + wave * 4096, dq_ptr + b0 * a.dqs[0] + b1 * a.dqs[1], a.dqs[2], q0, a.seq_q, lane);
    trace_stamp(a, 15);
}

template <bool MASK>
__global__ __launch_bounds__(kAttnThreads, 2) void attention_bwd_dkv_kernel(
    const _Float16* __restrict__ q_ptr, const _Float16* __restrict__ k_ptr, const _Float16* __restrict__ v_ptr,
    const float* __restrict__ lse_ptr, const float* __restrict__ dvec_ptr, const _Float16* __restrict__ do_ptr,
    _Float16* __restrict__ dk_ptr, _Float16* __restrict__ dv_ptr, const AttnArgsFor<MASK> a) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    constexpr int STAGE = 2 * kTileBytes + 512;  // Q tile, dO tile, 64 lse, 64 D
    trace_stamp(a, 0);
    long long bid = blockIdx.x;
    int b0, b1, ktile;
    decode_block(a, (a.seq_k + 127) / 128, bid, b0, b1, ktile);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5;
    const int k0 = ktile * 128 + wave * 32;
    const int krow = min(k0 + (lane & 31), a.seq_k - 1);
    const int64_t bh = (int64_t)b0 * a.batch1 + b1;

    const _Float16* Q = q_ptr + b0 * a.qs[0] + b1 * a.qs[1];
    const _Float16* G = do_ptr + b0 * a.dos[0] + b1 * a.dos[1];
    const float* LSE = lse_ptr + bh * a.seq_q;
    const float* DV = dvec_ptr + bh * a.seq_q;

    // this lane's key row carries one mask value, whatever the query
    float mask2 = 0.f;
    if constexpr (MASK) mask2 = (float)a.mask[b0 * a.ms[0] + b1 * a.ms[1] + krow] * kLog2eF;

    // K and V fragments of this lane's key row (B operands)
    half8 kfr[4], vfr[4];
    {
        const _Float16* kp = k_ptr + b0 * a.ks[0] + b1 * a.ks[1] + (int64_t)krow * a.ks[2] + h * 8;
        const _Float16* vp = v_ptr + b0 * a.vs[0] + b1 * a.vs[1] + (int64_t)krow * a.vs[2] + h * 8;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            kfr[st] = *reinterpret_cast<const half8*>(kp + st * 16);
            vfr[st] = *reinterpret_cast<const half8*>(vp + st * 16);
        }
    }

    TileDma dma;
    dma.init(wave, lane);
    TileFrags fr;
    fr.init(lane);
    const uint32_t lds0 = lds_addr(lds);
    const int nq = (a.seq_q + 63) / 64;
    const int qmax = a.seq_q - 1;
    // per tile every wavefront moves two pieces of Q, two of dO and one 256-byte vector: wavefronts 0 and 2
    // the 64 lse values, 1 and 3 the 64 D values (duplicates keep the transfer count uniform)
    const float* vec_src = (wave & 1) ? DV : LSE;
    const int vec_off = 2 * kTileBytes + (wave & 1) * 256;
    auto issue_tile = [&](int t, int st) {
        dma.issue(Q, a.qs[2], t * 64, qmax, lds + st * STAGE, wave);
        dma.issue(G, a.dos[2], t * 64, qmax, lds + st * STAGE + kTileBytes, wave);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(vec_src + min(t * 64 + lane, qmax)),
                                         (__attribute__((address_space(3))) void*)(lds + st * STAGE + vec_off), 4, 0, 0);
    };
#pragma unroll
    for (int s = 0; s < kBwdStages - 1; ++s)
        if (s < nq) issue_tile(s, s);

    floatx16 dkacc[2], dvacc[2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) { dkacc[i][e] = 0.f; dvacc[i][e] = 0.f; }

    int stage = 0;
    for (int j = 0; j < nq; ++j) {
        if (j + 1 < nq) wait_vm_lgkm0<5>();
        else wait_vm_lgkm0<0>();
        __builtin_amdgcn_s_barrier();
        if (j == 0) trace_stamp(a, 1);
        if (j + kBwdStages - 1 < nq) issue_tile(j + kBwdStages - 1, stage == 0 ? kBwdStages - 1 : stage - 1);
        const uint32_t qt = lds0 + stage * STAGE, gt = qt + kTileBytes, lt = gt + kTileBytes, dt = lt + 256;
        // Only a last, partial tile has query rows to take out (the transfers re-read the last row for them). Their
        // log-sum-exp becomes +inf here, which makes their probabilities, and with them their dS, exactly zero: the
        // arithmetic below carries no test.
        if ((j + 1) * 64 > a.seq_q) {
            if (wave == 0 && j * 64 + lane >= a.seq_q)
                reinterpret_cast<float*>(lds + stage * STAGE + 2 * kTileBytes)[lane] = INFINITY;
            __syncthreads();
        }

        static_for_attn<0, 2>([&](auto qbc) {
            constexpr int qb = decltype(qbc)::value;
            half8 qa[4], ga[4];
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                qa[st] = lds_read_b128<qb * 4096>(qt + fr.rowread[st]);
                ga[st] = lds_read_b128<qb * 4096>(gt + fr.rowread[st]);
            }
            floatx4 lv[4], dvv[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                lv[g] = lds_read_f32x4(lt + (qb * 32 + g * 8 + h * 4) * 4);
                dvv[g] = lds_read_f32x4(dt + (qb * 32 + g * 8 + h * 4) * 4);
            }
            floatx16 sacc, pacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) { sacc[e] = 0.f; pacc[e] = 0.f; }
            wait_lgkm<0>();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int st = 0; st < 4; ++st) {
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa[st], kfr[st], sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ga[st], vfr[st], pacc, 0, 0, 0);
            }
            // transposed operands: dO^T (for dV^T) and Q^T (for dK^T), steps 2*qb and 2*qb+1 of the tile
            half8 gtf[2][2], qtf[2][2];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                gtf[blk][0] = tr_pair<(2 * qb) * 2048>(gt + fr.trread[blk][0], gt + fr.trread[blk][1]);
                gtf[blk][1] = tr_pair<(2 * qb + 1) * 2048>(gt + fr.trread[blk][0], gt + fr.trread[blk][1]);
                qtf[blk][0] = tr_pair<(2 * qb) * 2048>(qt + fr.trread[blk][0], qt + fr.trread[blk][1]);
                qtf[blk][1] = tr_pair<(2 * qb + 1) * 2048>(qt + fr.trread[blk][0], qt + fr.trread[blk][1]);
            }
            half8 pf[2], dsf[2];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float p = MASK ? __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[e], a.scale_log2, mask2) - lv[e >> 2][e & 3] * kLog2e)
                                     : __builtin_amdgcn_exp2f(sacc[e] * a.scale_log2 - lv[e >> 2][e & 3] * kLog2e);
                pf[e >> 3][e & 7] = (_Float16)p;
                dsf[e >> 3][e & 7] = (_Float16)(p * (pacc[e] - dvv[e >> 2][e & 3]));
            }
            wait_lgkm<0>();
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                dvacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(gtf[0][t], pf[t], dvacc[0], 0, 0, 0);
                dvacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(gtf[1][t], pf[t], dvacc[1], 0, 0, 0);
                dkacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qtf[0][t], dsf[t], dkacc[0], 0, 0, 0);
                dkacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(qtf[1][t], dsf[t], dkacc[1], 0, 0, 0);
            }
        });
        stage = stage + 1 == kBwdStages ? 0 : stage + 1;
        if (j < 12) trace_stamp(a, 2 + j);
    }
    __syncthreads();
    store_rows_t(dkacc, a.scale, lds + wave * 4096, dk_ptr + b0 * a.dks[0] + b1 * a.dks[1], a.dks[2], k0, a.seq_k, lane);
    store_rows_t(dvacc, 1.0f, lds + wave * 4096, dv_ptr + b0 * a.dvs[0] + b1 * a.dvs[1], a.dvs[2], k0, a.seq_k, lane);
    trace_stamp(a, 15);
}

// ---------------------------------------------------------------- host side
thread_local unsigned long long* g_attn_trace = nullptr;   // per-workgroup clock readings (diagnostic)

int fill_args(const dmlhip_attention_desc* d, const dmlhip_attention_desc* g, AttnArgs& a, const char* what) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "%s: NULL descriptor", what);
    DML_REQUIRE(d->head_dim == 64, DMLHIP_ERR_UNSUPPORTED, "%s: head_dim %lld (only 64 is implemented)", what,
                (long long)d->head_dim);
    DML_REQUIRE(d->batch[0] >= 0 && d->batch[1] >= 0 && d->seq_q >= 0 && d->seq_k >= 0, DMLHIP_ERR_SHAPE,
                "%s: negative extent", what);
    DML_REQUIRE(d->seq_q <= (1 << 24) && d->seq_k <= (1 << 24) && d->batch[1] <= (1 << 24) && d->batch[0] <= (1 << 24),
                DMLHIP_ERR_SHAPE, "%s: extent too large", what);
    DML_REQUIRE(d->seq_k > 0 || d->seq_q == 0, DMLHIP_ERR_SHAPE, "%s: softmax over an empty key axis", what);
    a.batch1 = (int)d->batch[1];
    a.seq_q = (int)d->seq_q;
    a.seq_k = (int)d->seq_k;
    a.q_tiles = (int)ceil_div(d->seq_q, 128);
    a.k_tiles = (int)ceil_div(d->seq_k, 64);
    const dmlhip_attention_desc* src[2] = {d, g};
    for (int t = 0; t < 2; ++t) {
        if (!src[t]) continue;
        for (int i = 0; i < 3; ++i) {
            const int64_t s4[4] = {src[t]->q_stride[i], src[t]->k_stride[i], src[t]->v_stride[i], src[t]->o_stride[i]};
            for (int m = 0; m < 4; ++m)
                DML_REQUIRE(s4[m] >= 0 && s4[m] % 8 == 0, DMLHIP_ERR_ALIGN,
                            "%s: strides must be non-negative multiples of 8 elements (16 bytes)", what);
            if (t == 0) { a.qs[i] = s4[0]; a.ks[i] = s4[1]; a.vs[i] = s4[2]; a.os[i] = s4[3]; }
            else { a.dqs[i] = s4[0]; a.dks[i] = s4[1]; a.dvs[i] = s4[2]; a.dos[i] = s4[3]; }
        }
    }
    DML_REQUIRE(d->scale > 0.f, DMLHIP_ERR_SHAPE, "%s: the scale must be positive, got %g", what, (double)d->scale);
    a.scale = d->scale;
    a.scale_log2 = d->scale * 1.44269504088896340736f;
    a.trace = g_attn_trace;
    return 0;
}

// `m` = the arguments with the mask row pointer and strides added (checked here)
int fill_mask(const AttnArgs& a, const void* mask, const int64_t* ms, AttnArgsMasked& m, const char* what) {
    DML_REQUIRE(reinterpret_cast<uintptr_t>(mask) % 8 == 0, DMLHIP_ERR_ALIGN, "%s: the mask must be 8-byte aligned", what);
    DML_REQUIRE(ms[0] >= 0 && ms[1] >= 0 && ms[0] % 4 == 0 && ms[1] % 4 == 0, DMLHIP_ERR_ALIGN,
                "%s: mask strides must be non-negative multiples of 4 elements (0 = broadcast)", what);
    static_cast<AttnArgs&>(m) = a;
    m.mask = static_cast<const _Float16*>(mask);
    m.ms[0] = ms[0];
    m.ms[1] = ms[1];
    return 0;
}

int attention_forward(const dmlhip_attention_desc* d, const void* q, const void* k, const void* v, const void* mask,
                      const int64_t* ms, void* o, void* lse, void* stream, const char* what) {
    AttnArgs a = {};
    if (int e = fill_args(d, nullptr, a, what)) return e;
    const long long bh = (long long)d->batch[0] * d->batch[1];
    if (bh == 0 || d->seq_q == 0) return 0;
    DML_REQUIRE(q && k && v && o, DMLHIP_ERR_NULL, "%s: NULL tensor pointer", what);
    DML_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o), DMLHIP_ERR_ALIGN,
                "%s: tensors must be 16-byte aligned", what);
    a.total_blocks = bh * a.q_tiles;
    DML_REQUIRE(a.total_blocks <= 2147483647LL, DMLHIP_ERR_SHAPE, "%s: too many workgroups", what);
    if (mask) {
        AttnArgsMasked m;
        if (int e = fill_mask(a, mask, ms, m, what)) return e;
        hipLaunchKernelGGL(attention_fwd_kernel<true>, (unsigned)a.total_blocks, kAttnThreads, kFwdStages * 2 * kTileBytes,
                           (hipStream_t)stream, (const _Float16*)q, (const _Float16*)k, (const _Float16*)v, (_Float16*)o,
                           (float*)lse, m);
    } else {
        hipLaunchKernelGGL(attention_fwd_kernel<false>, (unsigned)a.total_blocks, kAttnThreads, kFwdStages * 2 * kTileBytes,
                           (hipStream_t)stream, (const _Float16*)q, (const _Float16*)k, (const _Float16*)v, (_Float16*)o,
                           (float*)lse, a);
    }
    return launch_status(what);
}

int attention_backward(const dmlhip_attention_desc* d, const dmlhip_attention_desc* grad, const void* q, const void* k,
                       const void* v, const void* mask, const int64_t* ms, const void* o, const void* lse, const void* d_o,
                       void* dq, void* dk, void* dv, void* workspace, size_t workspace_bytes, void* stream, const char* what) {
    AttnArgs a = {};
    DML_REQUIRE(grad, DMLHIP_ERR_NULL, "%s: NULL gradient descriptor", what);
    if (int e = fill_args(d, grad, a, what)) return e;
    const long long bh = (long long)d->batch[0] * d->batch[1];
    if (bh == 0 || (d->seq_q == 0 && d->seq_k == 0)) return 0;
    DML_REQUIRE(d->seq_q > 0, DMLHIP_ERR_SHAPE, "%s: no query rows but %lld key rows", what, (long long)d->seq_k);
    DML_REQUIRE(q && k && v && o && lse && d_o && dq && dk && dv, DMLHIP_ERR_NULL, "%s: NULL tensor pointer", what);
    DML_REQUIRE(aligned16(q) && aligned16(k) && aligned16(v) && aligned16(o) && aligned16(d_o) && aligned16(dq) &&
                    aligned16(dk) && aligned16(dv),
                DMLHIP_ERR_ALIGN, "%s: tensors must be 16-byte aligned", what);
    const size_t need = dmlhip_attention_backward_workspace_bytes(d);
    DML_REQUIRE(workspace && workspace_bytes >= need, DMLHIP_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given",
                what, need, workspace_bytes);
    AttnArgsMasked m;
    if (mask)
        if (int e = fill_mask(a, mask, ms, m, what)) return e;
    hipStream_t st = (hipStream_t)stream;
    const long long dq_blocks = bh * a.q_tiles, dkv_blocks = bh * ((a.seq_k + 127) / 128);
    DML_REQUIRE(dq_blocks <= 2147483647LL && dkv_blocks <= 2147483647LL, DMLHIP_ERR_SHAPE, "%s: too many workgroups", what);
    a.total_blocks = m.total_blocks = dq_blocks;
    if (mask)
        hipLaunchKernelGGL(attention_bwd_dq_kernel<true>, (unsigned)dq_blocks, kAttnThreads, kBwdStages * 2 * kTileBytes, st,
                           (const _Float16*)q, (const _Float16*)k, (const _Float16*)v, (const _Float16*)o, (const float*)lse,
                           (const _Float16*)d_o, (_Float16*)dq, (float*)workspace, m);
    else
        hipLaunchKernelGGL(attention_bwd_dq_kernel<false>, (unsigned)dq_blocks, kAttnThreads, kBwdStages * 2 * kTileBytes, st,
                           (const _Float16*)q, (const _Float16*)k, (const _Float16*)v, (const _Float16*)o, (const float*)lse,
                           (const _Float16*)d_o, (_Float16*)dq, (float*)workspace, a);
    if (int e = launch_status(what)) return e;
    a.total_blocks = m.total_blocks = dkv_blocks;
    if (a.trace) a.trace = m.trace = a.trace + 16 * dq_blocks;   // the second kernel's readings follow the first's
    if (mask)
        hipLaunchKernelGGL(attention_bwd_dkv_kernel<true>, (unsigned)dkv_blocks, kAttnThreads,
                           kBwdStages * (2 * kTileBytes + 512), st, (const _Float16*)q, (const _Float16*)k, (const _Float16*)v,
                           (const float*)lse, (const float*)workspace, (const _Float16*)d_o, (_Float16*)dk, (_Float16*)dv, m);
    else
        hipLaunchKernelGGL(attention_bwd_dkv_kernel<false>, (unsigned)dkv_blocks, kAttnThreads,
                           kBwdStages * (2 * kTileBytes + 512), st, (const _Float16*)q, (const _Float16*)k, (const _Float16*)v,
                           (const float*)lse, (const float*)workspace, (const _Float16*)d_o, (_Float16*)dk, (_Float16*)dv, a);
    return launch_status(what);
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

void dmlhip_debug_attention_trace(void* buffer) { g_attn_trace = (unsigned long long*)buffer; }

int dmlhip_attention_f16(const dmlhip_attention_desc* d, const void* q, const void* k, const void* v, void* o, void* lse,
                         void* stream) {
    return attention_forward(d, q, k, v, nullptr, nullptr, o, lse, stream, "attention");
}

int dmlhip_attention_masked_f16(const dmlhip_attention_desc* d, const void* q, const void* k, const void* v,
                                const void* mask, const int64_t* mask_stride, void* o, void* lse, void* stream) {
    DML_REQUIRE(mask && mask_stride, DMLHIP_ERR_NULL, "attention_masked: NULL mask or mask strides");
    return attention_forward(d, q, k, v, mask, mask_stride, o, lse, stream, "attention_masked");
}

size_t dmlhip_attention_backward_workspace_bytes(const dmlhip_attention_desc* d) {
    if (!d || d->batch[0] <= 0 || d->batch[1] <= 0 || d->seq_q <= 0) return 0;
    return (size_t)d->batch[0] * d->batch[1] * d->seq_q * sizeof(float);
}

int dmlhip_attention_backward_f16(const dmlhip_attention_desc* d, const dmlhip_attention_desc* grad, const void* q,
                                  const void* k, const void* v, const void* o, const void* lse, const void* d_o, void* dq,
                                  void* dk, void* dv, void* workspace, size_t workspace_bytes, void* stream) {
    return attention_backward(d, grad, q, k, v, nullptr, nullptr, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes,
                              stream, "attention_backward");
}

int dmlhip_attention_masked_backward_f16(const dmlhip_attention_desc* d, const dmlhip_attention_desc* grad, const void* q,
                                         const void* k, const void* v, const void* mask, const int64_t* mask_stride,
                                         const void* o, const void* lse, const void* d_o, void* dq, void* dk, void* dv,
                                         void* workspace, size_t workspace_bytes, void* stream) {
    DML_REQUIRE(mask && mask_stride, DMLHIP_ERR_NULL, "attention_masked_backward: NULL mask or mask strides");
    return attention_backward(d, grad, q, k, v, mask, mask_stride, o, lse, d_o, dq, dk, dv, workspace, workspace_bytes,
                              stream, "attention_masked_backward");
}

}  // extern "C"
