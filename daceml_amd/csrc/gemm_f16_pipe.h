// Fully pipelined fp16 MFMA GEMM: both operands stream from global memory straight into a ring of
// NSTAGE LDS tiles (global_load_lds, 16 bytes per lane, no staging registers, no LDS store
// instructions), with loads for tile t+NSTAGE-1 in flight while tile t is multiplied. Waiting is
// explicit: s_waitcnt vmcnt(n) lets the newest NSTAGE-2 tiles stay outstanding across the barrier
// that publishes tile t+1.
//
// Operand kinds
//   KC  K-contiguous (stride_k == 1): LDS tile [rows][64 k], 128-byte rows, 16-byte chunk c of row r at
//       slot c ^ (r & 7) ^ (r>>3 & 1) (rows r and r+8 share a bank window, the second term separates them;
//       the pattern repeats every 16 rows, so fragment blocks 32 rows apart differ by a constant offset);
//       fragments are ds_read_b128.
//   RC  row-contiguous (stride_row == 1, the transposed storage): LDS tile [64 k][rows], chunk (8 rows)
//       c of K row k at slot c ^ ((k & 3) << 2); fragments are two ds_read_b64_tr_b16 — the LDS
//       transpose read of gfx950 hands every lane four consecutive k of its row, which is exactly the
//       MFMA operand layout, so no transpose is done in registers or in a separate pass.
// Requirements (checked by the host): K % 64 == 0, 16-byte aligned bases and strides, rows % 8 == 0
// for RC operands, 32-bit element offsets.
#pragma once

#include "gemm_f16_common.h"
#include "lds_ops.h"

namespace dml {
namespace gemm16 {
namespace {

// ---------------------------------------------------------------- operand streams
// A stream owns one operand: where each lane's 16-byte DMA pieces come from, and where each lane
// reads its MFMA fragments. `T` = number of 32-row MFMA blocks this wavefront multiplies.
template <int R, int KIND, int T> struct Stream;

template <int R, int T>
struct Stream<R, 0, T> {  // K-contiguous: tile [R][64 k], chunk c of row r at slot c ^ swz16(r)
    static constexpr int N = R / 32;   // DMA instructions per wavefront per tile
    static constexpr int READS = T;    // LDS read instructions per K sub-step
    int off[N];
    uint32_t faddr[4];                 // fragment address of block 0 for each K sub-step (stage 0)
    __device__ __forceinline__ void init(int64_t s_row, int64_t, int row0, int rows, int wave, int lane, int wrow0,
                                         uint32_t tile0) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int r = (i * 4 + wave) * 8 + (lane >> 3);
            const int c = (lane & 7) ^ swz16(r);
            off[i] = (int)(min(row0 + r, rows - 1) * s_row) + c * 8;
        }
        const int r = wrow0 + (lane & 31);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
            faddr[kk] = tile0 + r * kRowBytes + ((((kk * 2 + (lane >> 5))) ^ swz16(r)) << 4);
    }
    __device__ __forceinline__ void issue(const _Float16* base, int64_t, int k0, char* tile, int wave) const {
#pragma unroll
        for (int i = 0; i < N; ++i) lds_dma16(base + off[i] + k0, tile + (i * 4 + wave) * 1024);
    }
    template <int I>
    __device__ __forceinline__ void issue_one(const _Float16* base, int64_t, int k0, char* tile, int wave) const {
        lds_dma16(base + off[I] + k0, tile + (I * 4 + wave) * 1024);
    }
    template <int KK>
    __device__ __forceinline__ void frags(uint32_t stage_off, half8 (&f)[T]) const {
        const uint32_t a = faddr[KK] + stage_off;
        static_for<0, T>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            f[i] = lds_read_b128<i * 32 * kRowBytes>(a);
        });
    }
    // fragment I of K sub-step KK alone (the interleaved loop requests fragments one at a time, between MFMAs)
    template <int KK, int I>
    __device__ __forceinline__ void frag_one(uint32_t stage_off, half8& f) const {
        f = lds_read_b128<I * 32 * kRowBytes>(faddr[KK] + stage_off);
    }
};

template <int R, int T>
struct Stream<R, 1, T> {  // row-contiguous: tile [64 k][R], chunk c (8 rows) of K row k at slot c ^ shift(k)
    static constexpr int N = R / 32;
    static constexpr int P = R * 2;    // bytes per K row of the tile
    static constexpr int READS = 2 * T;
    // A transpose read touches four consecutive K rows, 32 bytes of each. With 256-byte K rows (R = 128) they would
    // all start in the same bank: K row k is shifted by 64 (k % 4) bytes. With 128-byte K rows (R = 64) rows k and
    // k + 2 collide: shifted by 64 ((k / 2) % 2) bytes. Both depend on k % 4 only, so the reads' immediate offsets
    // (multiples of four K rows) leave the shift alone.
    static_assert(R == 64 || R % 128 == 0, "K rows of 128 bytes or of a multiple of 256");
    int off[N];
    uint32_t faddr[T];                 // per 32-row block: address of this lane's first transpose read (stage 0)
    __device__ __forceinline__ void init(int64_t, int64_t s_k, int row0, int rows, int wave, int lane, int wrow0,
                                         uint32_t tile0) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int o = (i * 4 + wave) * 1024 + lane * 16;
            const int kl = o / P, pos = (o % P) >> 4;
            int cidx;
            if constexpr (R == 64) cidx = pos ^ (((kl >> 1) & 1) << 2);
            else cidx = pos ^ ((kl & 3) << 2);
            off[i] = (int)(kl * s_k) + min(row0 + cidx * 8, rows - 8);
        }
        // transpose read: the 16 lanes of group G = l/16 jointly read K rows kq..kq+3 of 16 tile rows; lane
        // s = l%16 points at K row s/4, rows 4*(s%4)..+3 of them, and receives four consecutive K of row s.
        // G%2 picks the 16-row half of the 32-row block, G/2 the K half of the 16-k sub-step.
        const int s = lane & 15, grp = lane >> 4;
        const int kq = (grp >> 1) * 8 + (s >> 2);
#pragma unroll
        for (int i = 0; i < T; ++i) {
            const int row = wrow0 + i * 32 + (grp & 1) * 16 + 4 * (s & 3);
            if constexpr (R == 64) faddr[i] = tile0 + kq * P + (((row >> 3) ^ (((kq >> 1) & 1) << 2)) << 4) + (row & 7) * 2;
            else faddr[i] = tile0 + kq * P + (((row >> 3) ^ ((kq & 3) << 2)) << 4) + (row & 7) * 2;
        }
    }
    __device__ __forceinline__ void issue(const _Float16* base, int64_t s_k, int k0, char* tile, int wave) const {
        const _Float16* p = base + (int64_t)k0 * s_k;
#pragma unroll
        for (int i = 0; i < N; ++i) lds_dma16(p + off[i], tile + (i * 4 + wave) * 1024);
    }
    template <int I>
    __device__ __forceinline__ void issue_one(const _Float16* base, int64_t s_k, int k0, char* tile, int wave) const {
        lds_dma16(base + (int64_t)k0 * s_k + off[I], tile + (I * 4 + wave) * 1024);
    }
    template <int KK>
    __device__ __forceinline__ void frags(uint32_t stage_off, half8 (&f)[T]) const {
        static_for<0, T>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            const uint32_t a = faddr[i] + stage_off;
            const half4v lo = lds_read_tr16_b64<KK * 16 * P>(a);
            const half4v hi = lds_read_tr16_b64<KK * 16 * P + 4 * P>(a);
            f[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        });
    }
    template <int KK, int I>
    __device__ __forceinline__ void frag_one(uint32_t stage_off, half8& f) const {
        const uint32_t a = faddr[I] + stage_off;
        const half4v lo = lds_read_tr16_b64<KK * 16 * P>(a);
        const half4v hi = lds_read_tr16_b64<KK * 16 * P + 4 * P>(a);
        f = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
};


// ---------------------------------------------------------------- kernel
// KSUM: the operand pairs g.ga[i] / g.gb[i] are concatenated along K (one output, see GemmArgs::ksum). A template
// parameter, so that the ordinary kernels keep loop-invariant operand bases.
// ASUM: the workgroups of tile column 0 also produce asum[m] = sum_k A[m, k] (GemmArgs::asum) — the bias gradient
// that accompanies a weight gradient — from the A fragments they hold anyway: four packed dot products against ones
// per fragment, vector instructions that issue while the matrix pipe works on the MFMAs of the same sub-step.
// ILV: the interleaved K loop. Instead of issuing a sub-step's fragment reads and a K step's global -> LDS transfers as
// bursts ahead of the MFMAs (during which the matrix pipe of this SIMD has nothing queued), every MFMA is followed by at
// most a few fragment reads for the NEXT sub-step and, in the early sub-steps of a K step, by one transfer of the tile
// that is being refilled: the wavefront's other instructions issue in the shadow of the MFMA before them.
template <int BM, int BN, int WM, int WN, int AKIND, int BKIND, int NSTAGE, int EPI, bool KSUM = false, bool ASUM = false,
          bool ILV = false>
__global__ __launch_bounds__(kThreads) void gemm_f16_pipe_kernel(const _Float16* a_ptr, const _Float16* b_ptr, void* c_ptr,
                                                                 const void* bias_ptr, const void* res_ptr,
                                                                 void* pre_ptr, const GemmArgs g) {
    static_assert((BM / WM) * (BN / WN) == kThreads / kWave, "four wavefronts per workgroup");
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes, STAGE = A_BYTES + B_BYTES;
    constexpr int LPT = BM / 32 + BN / 32;  // DMA instructions per wavefront per tile
    extern __shared__ __attribute__((aligned(16))) char lds[];

    // All of this is wave-uniform integer arithmetic in 32 bits (the host checks total_blocks < 2^31): 64-bit
    // divisions are long software sequences, and this prologue runs before the first load can be issued.
    if (g.trace && threadIdx.x == 0) g.trace[4 * (size_t)blockIdx.x] = wall_clock64();
    uint32_t bid = blockIdx.x;
    {
        const uint32_t total = (uint32_t)g.total_blocks;
        const uint32_t xcd = bid % kXcds, idx = bid / kXcds;
        const uint32_t base = total / kXcds, rem = total % kXcds;
        bid = xcd * base + (xcd < rem ? xcd : rem) + idx;
    }
    const uint32_t tiles = (uint32_t)(g.tiles_m * g.tiles_n);
    uint32_t batch = 0, tile = bid;
    if (bid >= tiles) {   // more than one batch entry / group
        batch = bid / tiles;
        tile = bid - batch * tiles;
    }
    // Tiles are walked in groups of kGroupM tile rows, column by column inside a group: the workgroups that
    // are resident together (and the contiguous run of tiles an XCD gets) then cover a squarish patch of C and
    // share few rows of A and few columns of B, which is what fits an XCD's 4 MB L2.
    constexpr uint32_t kGroupM = 8;
    const uint32_t per_group = kGroupM * (uint32_t)g.tiles_n;
    const uint32_t group = tile / per_group, in_group = tile - group * per_group;
    const uint32_t rows_here = min((uint32_t)g.tiles_m - group * kGroupM, kGroupM);
    const uint32_t tn_u = in_group / rows_here;
    const int tm = (int)(group * kGroupM + (in_group - tn_u * rows_here)), tn = (int)tn_u;
    int z0 = 0, z1 = 0, z2 = 0;
    if (batch != 0) {
        const uint32_t b2 = (uint32_t)g.batch2, b1 = (uint32_t)g.batch1;
        const uint32_t q = batch / b2;
        z2 = (int)(batch - q * b2);
        z0 = (int)(q / b1);
        z1 = (int)(q - (uint32_t)z0 * b1);
    }
    void* asum_ptr = g.asum;
    if (!KSUM && g.groups) {  // uniform: one of several same-shaped problems (host sets the outer batch strides to 0)
        a_ptr = g.ga[z0];
        b_ptr = g.gb[z0];
        c_ptr = g.gc[z0];
        bias_ptr = g.gbias[z0];
        asum_ptr = g.gasum[z0];
    }
    const int64_t aoff = z0 * g.sab[0] + z1 * g.sab[1] + z2 * g.sab[2];
    const int64_t boff = z0 * g.sbb[0] + z1 * g.sbb[1] + z2 * g.sbb[2];
    const _Float16* A = a_ptr + aoff;
    const _Float16* B = b_ptr + boff;
    const int64_t coff = z0 * g.scb[0] + z1 * g.scb[1] + z2 * g.scb[2];
    const int m0 = tm * BM, n0 = tn * BN;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // wave-uniform: the wavefronts of tile column 0 sum the A rows they multiply; wn = 0 writes the result
    static_assert(!ASUM || BN / WN == 2, "the row sums are shared by two wavefronts per row block");
    const bool do_asum = ASUM && tn == 0 && asum_ptr != nullptr;
    const int asum_parity = do_asum ? wn : -1;
    float acc_sum[ASUM ? TM : 1];   // per lane: row lane % 32 of block i, the k half lane / 32 of every sub-step
    if constexpr (ASUM) {
#pragma unroll
        for (int i = 0; i < TM; ++i) acc_sum[i] = 0.f;
    }

    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
    Stream<BM, AKIND, TM> sa;
    Stream<BN, BKIND, TN> sb;
    sa.init(g.sam, g.sak, m0, g.m, wave, lane, wm * WM, lds0);
    sb.init(g.sbn, g.sbk, n0, g.n, wave, lane, wn * WN, lds0 + A_BYTES);
    constexpr int READS = Stream<BM, AKIND, TM>::READS + Stream<BN, BKIND, TN>::READS;
    constexpr int READS_W = READS > 15 ? 15 : READS;  // lgkmcnt saturates at 15: waiting for one more is harmless

    // K steps: g.k / BK per operand pair; with ksum the pairs follow each other (the accumulators simply keep
    // running), and the fill cursor (fa, fb, fk) walks pair by pair.
    const int nkg = g.k / BK;
    const int nk = KSUM ? nkg * g.groups : nkg;
    const _Float16* fa = A;
    const _Float16* fb = B;
    int fk = 0, fgrp = 0;
    auto advance = [&]() {
        ++fk;
        if constexpr (KSUM) {
            if (fk == nkg && fgrp + 1 < g.groups) {
                fk = 0;
                ++fgrp;
                // constant indices: the table stays in the kernel-argument segment, the choice in scalar registers
                fa = (fgrp == 1 ? g.ga[1] : fgrp == 2 ? g.ga[2] : g.ga[3]) + aoff;
                fb = (fgrp == 1 ? g.gb[1] : fgrp == 2 ? g.gb[2] : g.gb[3]) + boff;
            }
        }
    };
    static_assert(DMLHIP_GROUP_MAX == 4, "the operand-pair selection above lists four entries");
    // prologue: tiles 0 .. NSTAGE-2 in flight
#pragma unroll
    for (int s = 0; s < NSTAGE - 1; ++s) {
        if (s < nk) {
            sa.issue(KSUM ? fa : A, g.sak, (KSUM ? fk : s) * BK, lds + s * STAGE, wave);
            sb.issue(KSUM ? fb : B, g.sbk, (KSUM ? fk : s) * BK, lds + s * STAGE + A_BYTES, wave);
            if constexpr (KSUM) advance();
        }
    }
    if (nk >= NSTAGE - 1) wait_vm_lgkm0<(NSTAGE - 2) * LPT>();
    else wait_vm_lgkm0<0>();
    __builtin_amdgcn_s_barrier();
    if (g.trace && threadIdx.x == 0) g.trace[4 * (size_t)blockIdx.x + 1] = wall_clock64();

    half8 af[2][TM], bf[2][TN];
    if (nk > 0) {
        sa.template frags<0>(0u, af[0]);
        sb.template frags<0>(0u, bf[0]);
    }

    int cur_stage = 0;
    if constexpr (ILV) {
        constexpr int NM = TM * TN;                   // MFMAs per K sub-step
        constexpr int NU = TM + TN;                   // fragments to fetch per K sub-step
        // fragments requested after one MFMA: all of them within the first half of the sub-step's MFMAs, so that the
        // last one still has half a sub-step of MFMAs to land under
        constexpr int UPS = (NU + NM / 2 - 1) / (NM / 2);
        // Transfers go out in the early sub-steps only: with two stages the tile is needed at the end of this very
        // step, so its last transfer leaves half a step of cover; with a deeper ring the last sub-step stays free so
        // that the wait below can count whole tiles.
        constexpr int DSUB = NSTAGE == 2 ? 2 : 3;
        constexpr int DSLOTS = DSUB * NM;
        constexpr int NA = BM / 32;
        static_assert(LPT <= DSLOTS, "more transfers than MFMA slots to put them behind");
        // One K step. FILL: the ring is still being refilled (every step but the last NSTAGE-1), so the transfers are
        // issued unconditionally. MORE: another step follows, whose first fragments are requested during this step's
        // last sub-step. Three copies of the body (filling; draining; the very last step) and no per-slot branches in
        // any of them.
        int kt = 0;
        auto step = [&](auto fill_c, auto more_c) {
            constexpr bool FILL = decltype(fill_c)::value;
            constexpr bool MORE = decltype(more_c)::value;
            static_assert(MORE || !FILL, "a step that refills the ring is never the last");
            const uint32_t cur_off = (uint32_t)cur_stage * STAGE;
            const int nxt_stage = cur_stage + 1 == NSTAGE ? 0 : cur_stage + 1;
            const uint32_t nxt_off = (uint32_t)nxt_stage * STAGE;
            const int fs = cur_stage == 0 ? NSTAGE - 1 : cur_stage - 1;
            char* fill_tile = lds + fs * STAGE;
            const _Float16* const fill_a = KSUM ? fa : A;
            const _Float16* const fill_b = KSUM ? fb : B;
            const int fill_k = (KSUM ? fk : kt + NSTAGE - 1) * BK;
            if constexpr (KSUM && FILL) advance();
            static_for<0, BK / 16>([&](auto kc) {
                constexpr int kk = decltype(kc)::value;
                constexpr int nb = (kk + 1) & 1;
                constexpr bool last = kk + 1 == BK / 16;
                // the fragments of this sub-step were requested during the previous one
                if constexpr (last) {
                    // tile kt+1 must have landed for every wavefront before anybody reads it (below)
                    if constexpr (FILL) wait_vm_lgkm0<(NSTAGE - 2) * LPT>();
                    else wait_vm_lgkm0<0>();
                    __builtin_amdgcn_s_barrier();
                } else {
                    wait_lgkm<0>();
                }
                __builtin_amdgcn_sched_barrier(0);
                static_for<0, NM>([&](auto mc) {
                    constexpr int m = decltype(mc)::value;
                    constexpr int i = m / TN, j = m % TN;
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[kk & 1][j], af[kk & 1][i], acc[i][j], 0, 0, 0);
                    static_for<m * UPS, ((m + 1) * UPS < NU ? (m + 1) * UPS : NU)>([&](auto uc) {
                        constexpr int u = decltype(uc)::value;
                        if constexpr (!last) {
                            if constexpr (u < TM) sa.template frag_one<kk + 1, u>(cur_off, af[nb][u]);
                            else sb.template frag_one<kk + 1, u - TM>(cur_off, bf[nb][u - TM]);
                        } else if constexpr (MORE) {
                            if constexpr (u < TM) sa.template frag_one<0, u>(nxt_off, af[nb][u]);
                            else sb.template frag_one<0, u - TM>(nxt_off, bf[nb][u - TM]);
                        }
                    });
                    if constexpr (FILL && kk < DSUB) {
                        static_for<0, LPT>([&](auto dc) {
                            constexpr int d = decltype(dc)::value;
                            if constexpr ((d * DSLOTS) / LPT == kk * NM + m) {
                                if constexpr (d < NA) sa.template issue_one<d>(fill_a, g.sak, fill_k, fill_tile, wave);
                                else sb.template issue_one<d - NA>(fill_b, g.sbk, fill_k, fill_tile + A_BYTES, wave);
                            }
                        });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
                if constexpr (ASUM) {
                    // as in the plain loop below: the two wavefronts that share these A rows take alternate sub-steps
                    // (the fragments of this sub-step stay untouched until the reads of sub-step kk + 2 are issued)
                    if (asum_parity == (kk & 1)) {
                        const half2v one2 = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
                        for (int i = 0; i < TM; ++i) {
                            const half8 f = af[kk & 1][i];
#pragma unroll
                            for (int e = 0; e < 8; e += 2) {
                                const half2v p = {f[e], f[e + 1]};
                                acc_sum[i] = __builtin_amdgcn_fdot2(p, one2, acc_sum[i], false);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            cur_stage = nxt_stage;
        };
        for (; kt + NSTAGE - 1 < nk; ++kt) step(std::true_type{}, std::true_type{});
        if constexpr (NSTAGE > 2) {
            for (; kt + 1 < nk; ++kt) step(std::false_type{}, std::true_type{});
        }
        step(std::false_type{}, std::false_type{});  // kt == nk - 1 (the host passes k >= one K step)
    } else {
        for (int kt = 0; kt < nk; ++kt) {
            const uint32_t cur_off = (uint32_t)cur_stage * STAGE;
            const int nxt_stage = cur_stage + 1 == NSTAGE ? 0 : cur_stage + 1;
            // the stage that held tile kt-1 is free (every wavefront passed the barrier of step kt-1 after
            // its last read of it had completed): refill it with tile kt+NSTAGE-1
            // With three or more stages the transfers are issued in three portions, each right after the MFMAs of
            // sub-steps 0..2 have been queued: the matrix pipe keeps running while this wavefront computes
            // addresses and issues them. With two stages the tile is needed at the end of this very step, so it
            // is requested at once.
            constexpr bool SPREAD = NSTAGE >= 3;
            const int fill = kt + NSTAGE - 1;
            const int fs = cur_stage == 0 ? NSTAGE - 1 : cur_stage - 1;
            char* fill_tile = lds + fs * STAGE;
            const _Float16* const fill_a = KSUM ? fa : A;
            const _Float16* const fill_b = KSUM ? fb : B;
            const int fill_k = (KSUM ? fk : fill) * BK;
            if (KSUM && fill < nk) advance();
            if constexpr (!SPREAD) {
                if (fill < nk) {
                    sa.issue(fill_a, g.sak, fill_k, fill_tile, wave);
                    sb.issue(fill_b, g.sbk, fill_k, fill_tile + A_BYTES, wave);
                }
            }
            const bool more = kt + 1 < nk;
            static_for<0, BK / 16>([&](auto kc) {
                constexpr int kk = decltype(kc)::value;
                constexpr int nb = (kk + 1) & 1;
                if constexpr (kk + 1 < BK / 16) {
                    // fragments of the next sub-step, then wait for everything older than them (measured: fetching
                    // a whole K step of fragments ahead instead does not shorten the step)
                    sa.template frags<kk + 1>(cur_off, af[nb]);
                    sb.template frags<kk + 1>(cur_off, bf[nb]);
                    wait_lgkm<READS_W>();
                } else {
                    // last sub-step: its fragments are the only reads outstanding. Tile kt+1 must have
                    // landed for every wavefront before anybody reads it.
                    if (fill < nk) wait_vm_lgkm0<(NSTAGE - 2) * LPT>();
                    else wait_vm_lgkm0<0>();
                    __builtin_amdgcn_s_barrier();
                    if (more) {
                        sa.template frags<0>((uint32_t)nxt_stage * STAGE, af[0]);
                        sb.template frags<0>((uint32_t)nxt_stage * STAGE, bf[0]);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
    #pragma unroll
                for (int i = 0; i < TM; ++i)
    #pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[kk & 1][j], af[kk & 1][i], acc[i][j], 0, 0, 0);
                if constexpr (ASUM) {
                    // the two wavefronts that share these A rows (wn = 0, 1) take alternate sub-steps
                    if (asum_parity == (kk & 1)) {
                        const half2v one2 = {(_Float16)1.0f, (_Float16)1.0f};
    #pragma unroll
                        for (int i = 0; i < TM; ++i) {
                            const half8 f = af[kk & 1][i];
    #pragma unroll
                            for (int e = 0; e < 8; e += 2) {
                                const half2v p = {f[e], f[e + 1]};
                                acc_sum[i] = __builtin_amdgcn_fdot2(p, one2, acc_sum[i], false);
                            }
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (SPREAD && kk < 3) {
                    if (fill < nk) {
                        constexpr int NA = BM / 32;
                        static_for<kk * LPT / 3, (kk + 1) * LPT / 3>([&](auto jc) {
                            constexpr int j = decltype(jc)::value;
                            if constexpr (j < NA) sa.template issue_one<j>(fill_a, g.sak, fill_k, fill_tile, wave);
                            else sb.template issue_one<j - NA>(fill_b, g.sbk, fill_k, fill_tile + A_BYTES, wave);
                        });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            cur_stage = nxt_stage;
        }
    }
    wait_vm_lgkm0<0>();
    __syncthreads();
    if (g.trace && threadIdx.x == 0) g.trace[4 * (size_t)blockIdx.x + 2] = wall_clock64();

    // ---- epilogue (see store_strip): 32 x WN strips through this wavefront's LDS region
    constexpr int PITCH = WN + 4;
    float* strip = reinterpret_cast<float*>(lds) + wave * 32 * PITCH;
    float bias_n[8];
    load_bias_n<WN>(g, bias_ptr, n0 + wn * WN, lane, bias_n);
    static_for<0, TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        stage_strip<TN, PITCH>(strip, acc[i], lane);
        __builtin_amdgcn_wave_barrier();  // LDS serves a wavefront's accesses in program order
        const int mb = m0 + wm * WM + i * 32, nb = n0 + wn * WN;
        if (g.out_f32) store_strip<float, WN, EPI>(g, c_ptr, pre_ptr, res_ptr, bias_ptr, bias_n, strip, mb, nb, coff, lane);
        else store_strip<_Float16, WN, EPI>(g, c_ptr, pre_ptr, res_ptr, bias_ptr, bias_n, strip, mb, nb, coff, lane);
        __builtin_amdgcn_wave_barrier();
    });
    if (g.trace && threadIdx.x == 0) {
        wait_vm_lgkm0<0>();   // this wavefront's stores have been accepted
        g.trace[4 * (size_t)blockIdx.x + 3] = wall_clock64();
    }
    if constexpr (ASUM) {
        // lanes l and l + 32 hold the two k halves of row l; wavefront wn = 1 hands its share over through LDS
        __syncthreads();   // the epilogue strips in LDS are done with
        float* hand = reinterpret_cast<float*>(lds) + wm * (TM * 32);
        float v[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int other = __builtin_amdgcn_ds_bpermute(((lane + 32) & 63) << 2, __builtin_bit_cast(int, acc_sum[i]));
            v[i] = acc_sum[i] + __builtin_bit_cast(float, other);
            if (do_asum && wn == 1 && lane < 32) hand[i * 32 + lane] = v[i];
        }
        __syncthreads();
        if (do_asum && wn == 0 && lane < 32) {
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = m0 + wm * WM + i * 32 + lane;
                const float r = v[i] + hand[i * 32 + lane];
                if (m < g.m) {
                    if (g.asum_f32) reinterpret_cast<float*>(asum_ptr)[m] = r;
                    else reinterpret_cast<_Float16*>(asum_ptr)[m] = (_Float16)r;
                }
            }
        }
    }
}

template <int BM, int BN, int WM, int WN, int NSTAGE, bool KSUM = false, bool ASUM = false, bool ILV = false>
int launch_tile(GemmArgs& g, const _Float16* a, const _Float16* b, void* c, const void* bias, const void* res, void* pre,
                int akind, int bkind, long long batch, hipStream_t st) {
    g.tiles_m = (g.m + BM - 1) / BM;
    g.tiles_n = (g.n + BN - 1) / BN;
    const long long total = (long long)g.tiles_m * g.tiles_n * batch;
    DML_REQUIRE(total <= 2147483647LL, DMLHIP_ERR_SHAPE, "gemm_f16: %lld workgroups exceed the grid limit", total);
    g.total_blocks = total;
    size_t lds = (size_t)NSTAGE * (BM + BN) * kRowBytes;
    const size_t epi = (size_t)4 * 32 * (WN + 4) * sizeof(float);
    if (lds < epi) lds = epi;
    const int ek = epilogue_kind(g, bias, res, pre);
    if (ek == EPI_GENERAL_ACT) {
        set_error("gemm_f16: the pipelined kernel has no activation + residual/beta/row-bias epilogue");
        return DMLHIP_ERR_UNSUPPORTED;
    }
#define DML_PIPE_CASE(AK, BKD, ACTV)                                                                          \
    if (akind == AK && bkind == BKD && ek == ACTV) {                                                          \
        auto kern = gemm_f16_pipe_kernel<BM, BN, WM, WN, AK, BKD, NSTAGE, ACTV, KSUM, ASUM, ILV>;                  \
        if (lds > 64 * 1024) {                                                                                \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               (int)lds);                                                     \
            if (e != hipSuccess) {                                                                            \
                set_error("gemm_f16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));        \
                return (int)e;                                                                                \
            }                                                                                                 \
        }                                                                                                     \
        hipLaunchKernelGGL(kern, (unsigned)total, kThreads, lds, st, a, b, c, bias, res, pre, g);             \
        return launch_status("gemm_f16(pipelined)");                                                          \
    }
    DML_PIPE_CASE(0, 0, EPI_PLAIN) DML_PIPE_CASE(0, 1, EPI_PLAIN) DML_PIPE_CASE(1, 0, EPI_PLAIN) DML_PIPE_CASE(1, 1, EPI_PLAIN)
    if constexpr (ASUM) {
        set_error("gemm_f16: the row-sum result needs a plain epilogue");
        return DMLHIP_ERR_UNSUPPORTED;
    } else {
        if constexpr (!KSUM) {
            DML_PIPE_CASE(0, 0, EPI_ACT) DML_PIPE_CASE(0, 1, EPI_ACT) DML_PIPE_CASE(1, 0, EPI_ACT) DML_PIPE_CASE(1, 1, EPI_ACT)
        }
        DML_PIPE_CASE(0, 0, EPI_GENERAL) DML_PIPE_CASE(0, 1, EPI_GENERAL) DML_PIPE_CASE(1, 0, EPI_GENERAL)
        DML_PIPE_CASE(1, 1, EPI_GENERAL)
        set_error("gemm_f16: no pipelined kernel for operand kinds %d/%d", akind, bkind);
        return DMLHIP_ERR_UNSUPPORTED;
    }
#undef DML_PIPE_CASE
}

}  // namespace
}  // namespace gemm16
}  // namespace dml
