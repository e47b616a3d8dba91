// fp16 x fp16 -> fp32-accumulate strided batched GEMM on the gfx950 matrix cores
// (v_mfma_f32_32x32x16_f16), the kernel behind MatMul / Einsum / Gemm and their backward
// contractions.
//
// Tiling: a workgroup of 4 wavefronts owns a BM x BN tile of C and walks K in steps of 64.
// Each K step stages an A tile [BM][64] and a B tile [BN][64] (both K-contiguous, 128 bytes per
// row) in LDS, double-buffered, so one barrier per step. Global loads for step t+1 are issued
// before the MFMAs of step t and written to the other LDS buffer afterwards.
//
// LDS layout: rows are split into eight 16-byte chunks; chunk c of row r is stored at chunk slot
// c ^ ((r ^ (r >> 3)) & 7). A fragment read (lane -> row l%32, chunk 2*kk + l/32) then touches
// eight distinct slots per eight consecutive rows, and so do both kinds of tile stores.
//
// Operand layout: each operand may be K-contiguous (stride_k == 1; 128-bit loads straight to LDS)
// or row-contiguous (stride_m/n == 1, i.e. the transposed storage). The latter is transposed in
// registers on the way to LDS: a thread loads eight K-rows of RU adjacent rows and re-packs them
// into RU chunks of eight K values, so no separate transpose kernel or HBM round trip is needed.
#include "gemm_f16_common.h"

#include <atomic>

namespace dml {
using namespace gemm16;
namespace {

// ---------------------------------------------------------------- global -> registers
// The loaders are branch-free in the steady state. Rows past the end of the operand are clamped to
// the last valid row (they only feed rows/columns of C that are never stored); K past the end is
// zero-filled, and only the last K step takes that path. Offsets are 32-bit element offsets from
// the operand's batch base (the host falls back to the generic loader when they would not fit).

// K-contiguous operand (k % 8 == 0): thread t loads chunks q = t + i*256 of the [R][64] tile.
// Loads never branch: a chunk past the end of K is fetched from the last valid chunk instead and
// replaced by zeros when it is written to LDS.
template <int R>
struct LoaderKC {
    static constexpr int N = R * 8 / kThreads;
    u32x4 v[N];
    int off[N];
    int c8;       // first k of this thread's chunk inside a K step
    int k_valid;  // k of the tile held in v[] minus its k0 (chunks with c8 >= k_valid are zero)
    __device__ __forceinline__ void init(int64_t s_row, int64_t, int row0, int rows) {
        c8 = (threadIdx.x & 7) * 8;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = min(row0 + (q >> 3), rows - 1);
            off[i] = (int)(r * s_row);
        }
    }
    __device__ __forceinline__ void load(const _Float16* base, int64_t, int k0, int k) {
        k_valid = k - k0;
        const int kc = min(k0 + c8, k - 8);
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = *reinterpret_cast<const u32x4*>(base + off[i] + kc);
    }
    __device__ __forceinline__ void store(char* tile) const {
        const bool ok = c8 < k_valid;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = q >> 3, c = q & 7;
            const u32x4 z = {0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4*>(tile + r * kRowBytes + ((c ^ swz(r)) << 4)) = ok ? v[i] : z;
        }
    }
};

// K-contiguous operand with k % 64 == 0, loaded straight into LDS (global_load_lds, 16 bytes per
// lane): no staging registers and no LDS store instructions. One wave instruction fills 1 KiB =
// eight tile rows; lane l lands at (row l/8, chunk slot l%8) of that group, so it fetches the
// global chunk that the swizzle maps to this slot.
template <int R>
struct LoaderKCDirect {
    static constexpr int N = R / 32;  // instructions per wavefront per tile
    int off[N];
    int wave;
    __device__ __forceinline__ void init(int64_t s_row, int64_t, int row0, int rows) {
        const int lane = threadIdx.x & (kWave - 1);
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int r = (i * 4 + wave) * 8 + (lane >> 3);
            const int c = (lane & 7) ^ swz(r);
            off[i] = (int)(min(row0 + r, rows - 1) * s_row) + c * 8;
        }
    }
    __device__ __forceinline__ void issue(const _Float16* base, int k0, char* tile) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(base + off[i] + k0),
                (__attribute__((address_space(3))) void*)(tile + (i * 4 + wave) * 1024), 16, 0, 0);
        }
    }
    __device__ __forceinline__ void load(const _Float16*, int64_t, int, int) {}
    __device__ __forceinline__ void store(char*) const {}
};

// Row-contiguous operand (element (row, k) at k*s_k + row; rows % RU == 0): thread t owns K block
// kb = t/32 (eight K values) of the RU rows starting at (t%32)*RU and transposes them in registers.
// K rows past the end are fetched from row k-1 and zeroed on the way to LDS.
template <int R>
struct LoaderRC {
    static constexpr int RU = R / 32;  // 4 for R=128, 8 for R=256
    typedef _Float16 rowvec __attribute__((ext_vector_type(RU)));
    rowvec v[8];
    int off;
    int k_valid;
    __device__ __forceinline__ void init(int64_t, int64_t, int row0, int rows) {
        const int rg = threadIdx.x & 31;
        off = min(row0 + rg * RU, rows - RU);
    }
    __device__ __forceinline__ void load(const _Float16* base, int64_t s_k, int k0, int k) {
        const int kb8 = (threadIdx.x >> 5) * 8;
        k_valid = k - k0 - kb8;
        const _Float16* p = base + off;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int gk = min(k0 + kb8 + j, k - 1);
            v[j] = *reinterpret_cast<const rowvec*>(p + (int64_t)gk * s_k);
        }
    }
    __device__ __forceinline__ void store(char* tile) const {
        const int kb = threadIdx.x >> 5, rg = threadIdx.x & 31;
#pragma unroll
        for (int e = 0; e < RU; ++e) {
            half8 o;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = j < k_valid ? v[j][e] : (_Float16)0;
            const int r = rg * RU + e;
            *reinterpret_cast<half8*>(tile + r * kRowBytes + ((kb ^ swz(r)) << 4)) = o;
        }
    }
};

// Any strides, any alignment: guarded element loads. Correct everywhere, fast nowhere.
template <int R>
struct LoaderGeneric {
    static constexpr int N = R * 8 / kThreads;
    half8 v[N];
    int64_t s_row_, s_k_;
    int row0_, rows_;
    __device__ __forceinline__ void init(int64_t s_row, int64_t s_k, int row0, int rows) {
        s_row_ = s_row; s_k_ = s_k; row0_ = row0; rows_ = rows;
    }
    __device__ __forceinline__ void load(const _Float16* base, int64_t, int k0, int k) {
#pragma unroll 1
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = q >> 3, c = q & 7;
            const int gr = row0_ + r, gk = k0 + c * 8;
            half8 h = {};
            if (gr < rows_) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (gk + e < k) h[e] = base[(int64_t)gr * s_row_ + (int64_t)(gk + e) * s_k_];
            }
            v[i] = h;
        }
    }
    __device__ __forceinline__ void store(char* tile) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = q >> 3, c = q & 7;
            *reinterpret_cast<half8*>(tile + r * kRowBytes + ((c ^ swz(r)) << 4)) = v[i];
        }
    }
};

template <int R, int MODE> struct LoaderSel;
template <int R> struct LoaderSel<R, 0> { using type = LoaderKC<R>; };
template <int R> struct LoaderSel<R, 1> { using type = LoaderRC<R>; };
template <int R> struct LoaderSel<R, 2> { using type = LoaderGeneric<R>; };
template <int R> struct LoaderSel<R, 3> { using type = LoaderKCDirect<R>; };

// ---------------------------------------------------------------- the kernel
// AMODE / BMODE: 0 = K-contiguous via registers, 1 = row-contiguous, 2 = generic strides,
// 3 = K-contiguous straight to LDS (k % 64 == 0).
template <int BM, int BN, int WM, int WN, int AMODE, int BMODE, bool ACT>
__global__ __launch_bounds__(kThreads) void gemm_f16_kernel(const _Float16* __restrict__ a_ptr,
                                                            const _Float16* __restrict__ b_ptr, void* c_ptr,
                                                            const void* bias_ptr, const void* res_ptr, void* pre_ptr,
                                                            const GemmArgs g) {
    static_assert((BM / WM) * (BN / WN) == kThreads / kWave, "four wavefronts per workgroup");
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes;
    extern __shared__ __attribute__((aligned(16))) char lds[];

    // ---- block -> (batch, tile): blocks are dealt round-robin to the eight XCDs, so give each
    // XCD a contiguous run of tiles (neighbouring tiles share operand panels in that XCD's L2).
    long long bid = blockIdx.x;
    {
        const long long total = g.total_blocks;
        const long long xcd = bid % kXcds, idx = bid / kXcds;
        const long long base = total / kXcds, rem = total % kXcds;
        bid = xcd * base + (xcd < rem ? xcd : rem) + idx;
    }
    const int tiles = g.tiles_m * g.tiles_n;
    const long long batch = bid / tiles;
    const int tile = (int)(bid % tiles);
    const int tm = tile / g.tiles_n, tn = tile % g.tiles_n;
    const int z2 = (int)(batch % g.batch2);
    const int z1 = (int)((batch / g.batch2) % g.batch1);
    const int z0 = (int)(batch / ((long long)g.batch2 * g.batch1));
    const _Float16* A = a_ptr + z0 * g.sab[0] + z1 * g.sab[1] + z2 * g.sab[2];
    const _Float16* B = b_ptr + z0 * g.sbb[0] + z1 * g.sbb[1] + z2 * g.sbb[2];
    const int64_t coff = z0 * g.scb[0] + z1 * g.scb[1] + z2 * g.scb[2];
    const int m0 = tm * BM, n0 = tn * BN;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    typename LoaderSel<BM, AMODE>::type la;
    typename LoaderSel<BN, BMODE>::type lb;

    const int nk = (g.k + BK - 1) / BK;
    la.init(g.sam, g.sak, m0, g.m);
    lb.init(g.sbn, g.sbk, n0, g.n);
    if (nk > 0) {
        if constexpr (AMODE == 3) la.issue(A, 0, lds);
        if constexpr (BMODE == 3) lb.issue(B, 0, lds + A_BYTES);
        la.load(A, g.sak, 0, g.k);
        lb.load(B, g.sbk, 0, g.k);
        la.store(lds);
        lb.store(lds + A_BYTES);
    }
    __syncthreads();

    // Fragment reads are software-pipelined one K sub-step (16) ahead of the MFMAs that consume
    // them, and the barrier that publishes the next tile sits before the last sub-step, so the LDS
    // latency of the first fragments of tile t+1 hides behind the last MFMAs of tile t.
    const int frow = lane & 31, fk = lane >> 5;
    const int a_row = wm * WM + frow, b_row = wn * WN + frow;
    half8 af[2][TM], bf[2][TN];
    auto read_frags = [&](const char* buf, int kk, half8(&fa)[TM], half8(&fb)[TN]) {
        const int c = kk * 2 + fk;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int r = a_row + i * 32;
            fa[i] = *reinterpret_cast<const half8*>(buf + r * kRowBytes + ((c ^ swz(r)) << 4));
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int r = b_row + j * 32;
            fb[j] = *reinterpret_cast<const half8*>(buf + A_BYTES + r * kRowBytes + ((c ^ swz(r)) << 4));
        }
    };
    if (nk > 0) read_frags(lds, 0, af[0], bf[0]);
    for (int kt = 0; kt < nk; ++kt) {
        char* cur = lds + (kt & 1) * (A_BYTES + B_BYTES);
        char* nxt = lds + ((kt + 1) & 1) * (A_BYTES + B_BYTES);
        const bool more = kt + 1 < nk;
        if (more) {
            if constexpr (AMODE == 3) la.issue(A, (kt + 1) * BK, nxt);
            if constexpr (BMODE == 3) lb.issue(B, (kt + 1) * BK, nxt + A_BYTES);
            la.load(A, g.sak, (kt + 1) * BK, g.k);
            lb.load(B, g.sbk, (kt + 1) * BK, g.k);
        }
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            if (kk + 1 < BK / 16) {
                read_frags(cur, kk + 1, af[(kk + 1) & 1], bf[(kk + 1) & 1]);
            } else {
                if (more) {
                    la.store(nxt);
                    lb.store(nxt + A_BYTES);
                }
                __syncthreads();
                if (more) read_frags(nxt, 0, af[0], bf[0]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[kk & 1][j], af[kk & 1][i], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();

    // ---- epilogue. With the swapped MFMA operands acc[i][j][e] is C[m, n] with m = l%32 and
    // n = (e/4)*8 + (l/32)*4 + e%4 inside the 32x32 block. Each wavefront stages one 32 x WN strip at a
    // time in its own LDS region and reads it back row-wise, so that global accesses are 128-bit and
    // contiguous along n.
    constexpr int PITCH = WN + 4;
    float* strip = reinterpret_cast<float*>(lds) + wave * 32 * PITCH;
    float bias_n[8];
    load_bias_n<WN>(g, bias_ptr, n0 + wn * WN, lane, bias_n);
    static_for<0, TM>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        stage_strip<TN, PITCH>(strip, acc[i], lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int mb = m0 + wm * WM + i * 32, nb = n0 + wn * WN;
        if (g.out_f32) store_strip<float, WN, ACT ? EPI_GENERAL_ACT : EPI_GENERAL>(g, c_ptr, pre_ptr, res_ptr, bias_ptr, bias_n, strip, mb, nb, coff, lane);
        else store_strip<_Float16, WN, ACT ? EPI_GENERAL_ACT : EPI_GENERAL>(g, c_ptr, pre_ptr, res_ptr, bias_ptr, bias_n, strip, mb, nb, coff, lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    });
}

// ---------------------------------------------------------------- host side
enum { CFG_128x128 = 0, CFG_256x128 = 1, CFG_256x256 = 2 };

template <int BM, int BN, int WM, int WN>
int launch_cfg(GemmArgs& g, const _Float16* pa, const _Float16* pb, void* pc, const void* pbias, const void* pres,
               void* ppre, int amode, int bmode, long long batch, hipStream_t st) {
    g.tiles_m = (g.m + BM - 1) / BM;
    g.tiles_n = (g.n + BN - 1) / BN;
    const long long total = (long long)g.tiles_m * g.tiles_n * batch;
    DML_REQUIRE(total <= 2147483647LL, DMLHIP_ERR_SHAPE, "gemm_f16: %lld workgroups exceed the grid limit", total);
    g.total_blocks = total;
    const size_t lds = (size_t)2 * (BM + BN) * kRowBytes;
#define DML_GEMM_CASE(AM, BMD)                                                                                \
    if (amode == AM && bmode == BMD) {                                                                        \
        auto kern = g.act != DMLHIP_ACT_NONE ? gemm_f16_kernel<BM, BN, WM, WN, AM, BMD, true>                  \
                                             : gemm_f16_kernel<BM, BN, WM, WN, AM, BMD, false>;                \
        if (lds > 64 * 1024) {                                                                                \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               (int)lds);                                                     \
            if (e != hipSuccess) {                                                                            \
                set_error("gemm_f16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));        \
                return (int)e;                                                                                \
            }                                                                                                 \
        }                                                                                                     \
        hipLaunchKernelGGL(kern, (unsigned)total, kThreads, lds, st, pa, pb, pc, pbias, pres, ppre, g);                                      \
        return launch_status("gemm_f16");                                                                     \
    }
    DML_GEMM_CASE(0, 0)
    DML_GEMM_CASE(0, 1)
    DML_GEMM_CASE(1, 0)
    DML_GEMM_CASE(1, 1)
    if constexpr (BM == 128 && BN == 128) {
        DML_GEMM_CASE(2, 2)
    }
#undef DML_GEMM_CASE
    set_error("gemm_f16: no kernel for operand modes %d/%d", amode, bmode);
    return DMLHIP_ERR_UNSUPPORTED;
}

// 0 = K-contiguous, 1 = row-contiguous (both with 16-byte-aligned vectors, extents that are
// multiples of the vector length and 32-bit element offsets), 2 = anything else.
int operand_mode(const void* p, int64_t rows, int64_t k, int64_t s_row, int64_t s_k, const int64_t* sb,
                 const int64_t* batch) {
    bool bs_ok = true;
    for (int i = 0; i < 3; ++i)
        if (batch[i] > 1 && sb[i] % 8 != 0) bs_ok = false;
    if (!aligned16(p) || !bs_ok) return 2;
    if ((double)(rows - 1) * s_row + (double)(k + 64) * s_k > 2.0e9) return 2;
    if (s_k == 1 && s_row % 8 == 0 && k % 8 == 0) return 0;
    if (s_row == 1 && s_k % 8 == 0 && rows % 8 == 0) return 1;
    return 2;
}

// Diagnostic switches (declared in the public header). Per calling thread, so that one thread pinning a configuration
// does not change what other threads launch.
thread_local int g_force_cfg = -1;  // pin the tile configuration
thread_local int g_direct_lds = 1;  // 0 forces the register-staged loaders
thread_local unsigned long long* g_trace = nullptr;  // per-workgroup clock readings of the pipelined kernel

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

void dmlhip_debug_force_gemm_config(int cfg) { g_force_cfg = cfg; }
void dmlhip_debug_gemm_direct_lds(int on) { g_direct_lds = on; }
void dmlhip_debug_gemm_trace(void* buffer) { g_trace = (unsigned long long*)buffer; }
static std::atomic<long long> g_grouped_single_launches{0};
// Number of grouped calls that went out as ONE launch (tests check that grouping really happens).
long long dmlhip_debug_grouped_single_launches() { return g_grouped_single_launches.load(); }

struct GemmGroup {
    int count;
    const void* const* a;
    const void* const* b;
    void* const* c;            // unused with ksum
    const void* const* bias;   // unused with ksum
    bool ksum;                 // concatenate the groups along K into one output instead of running them side by side
};

// grp != nullptr: a / b / c / bias are those of group 0 (used for the layout checks, which the caller has made sure
// hold for every group); returns DMLHIP_ERR_UNSUPPORTED when the grouped launch is not possible.
static int run_gemm_f16(const dmlhip_gemm_desc* d, const void* a, const void* b, void* c, const void* bias,
                        const void* residual, void* pre_out, void* stream, const GemmGroup* grp = nullptr,
                        void* const* asum = nullptr, int asum_f32 = 0) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "gemm_f16: NULL descriptor");
    DML_REQUIRE(d->m >= 0 && d->n >= 0 && d->k >= 0, DMLHIP_ERR_SHAPE, "gemm_f16: negative extent");
    DML_REQUIRE(d->m <= 2147483647 / 2 && d->n <= 2147483647 / 2 && d->k <= 2147483647 / 2, DMLHIP_ERR_SHAPE,
                "gemm_f16: extent exceeds 2^30");
    long long batch = 1;
    for (int i = 0; i < 3; ++i) {
        DML_REQUIRE(d->batch[i] >= 0 && d->batch[i] <= 2147483647, DMLHIP_ERR_SHAPE, "gemm_f16: bad batch extent");
        batch *= d->batch[i];
        DML_REQUIRE(batch <= 2147483647LL, DMLHIP_ERR_SHAPE, "gemm_f16: batch too large");
    }
    DML_REQUIRE(d->out_dtype == DMLHIP_F16 || d->out_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM, "gemm_f16: bad out_dtype");
    DML_REQUIRE(d->bias_dtype == DMLHIP_F16 || d->bias_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM,
                "gemm_f16: bad bias_dtype");
    DML_REQUIRE(valid_act(d->act), DMLHIP_ERR_ENUM, "gemm_f16: bad act");
    DML_REQUIRE(d->a_stride_m >= 0 && d->a_stride_k >= 0 && d->b_stride_k >= 0 && d->b_stride_n >= 0 &&
                    d->c_stride_m >= 0,
                DMLHIP_ERR_SHAPE, "gemm_f16: negative stride");
    DML_REQUIRE(d->c_stride_m >= d->n || d->m <= 1, DMLHIP_ERR_SHAPE, "gemm_f16: rows of C overlap (stride %lld < n)",
                (long long)d->c_stride_m);
    if (d->m == 0 || d->n == 0 || batch == 0) return 0;
    DML_REQUIRE(c, DMLHIP_ERR_NULL, "gemm_f16: NULL output");
    DML_REQUIRE(d->k == 0 || (a && b), DMLHIP_ERR_NULL, "gemm_f16: NULL operand");

    GemmArgs g;
    g.groups = 0;
    g.ksum = 0;
    g.trace = g_trace;
    g.asum = !grp && asum ? asum[0] : nullptr;
    g.asum_f32 = asum_f32;
    for (int i = 0; i < DMLHIP_GROUP_MAX; ++i) g.gasum[i] = grp && asum && i < grp->count ? asum[i] : nullptr;
    if (grp) {
        g.groups = grp->count;
        g.ksum = grp->ksum;
        if (!grp->ksum) batch *= grp->count;
        for (int i = 0; i < DMLHIP_GROUP_MAX; ++i) {
            const bool on = i < grp->count;
            g.ga[i] = on ? (const _Float16*)grp->a[i] : nullptr;
            g.gb[i] = on ? (const _Float16*)grp->b[i] : nullptr;
            g.gc[i] = on && !grp->ksum ? grp->c[i] : nullptr;
            g.gbias[i] = on && !grp->ksum && grp->bias ? grp->bias[i] : nullptr;
        }
    }
    g.m = (int)d->m; g.n = (int)d->n; g.k = (int)d->k;
    g.sam = d->a_stride_m; g.sak = d->a_stride_k; g.sbn = d->b_stride_n; g.sbk = d->b_stride_k;
    g.scm = d->c_stride_m;
    g.batch1 = (int)d->batch[1]; g.batch2 = (int)d->batch[2];
    for (int i = 0; i < 3; ++i) {
        g.sab[i] = d->a_stride_batch[i]; g.sbb[i] = d->b_stride_batch[i]; g.scb[i] = d->c_stride_batch[i];
    }
    g.alpha = d->alpha; g.beta = d->beta;
    g.out_f32 = d->out_dtype == DMLHIP_F32; g.bias_f32 = d->bias_dtype == DMLHIP_F32; g.act = d->act;
    g.bias_m = d->bias_along_m != 0;
    {
        // 128-bit accesses to C / pre_out / residual need 8-element granularity everywhere
        const int gran = 8;
        bool ok = aligned16(c) && (!residual || aligned16(residual)) && (!pre_out || aligned16(pre_out)) &&
                  d->c_stride_m % gran == 0;
        if (g.out_f32)
            ok = ok && (reinterpret_cast<uintptr_t>(c) % 32 == 0) &&
                 (!residual || reinterpret_cast<uintptr_t>(residual) % 32 == 0) &&
                 (!pre_out || reinterpret_cast<uintptr_t>(pre_out) % 32 == 0);
        for (int i = 0; i < 3; ++i)
            if (d->batch[i] > 1 && d->c_stride_batch[i] % gran != 0) ok = false;
        g.c_vec = ok;
    }

    int amode = d->k == 0 ? 0 : operand_mode(a, d->m, d->k, d->a_stride_m, d->a_stride_k, d->a_stride_batch, d->batch);
    int bmode = d->k == 0 ? 0 : operand_mode(b, d->n, d->k, d->b_stride_n, d->b_stride_k, d->b_stride_batch, d->batch);
    if (amode == 2 || bmode == 2) amode = bmode = 2;
    hipStream_t st = (hipStream_t)stream;

    int cfg = g_force_cfg;
    // Both operands vector-loadable and K a whole number of steps: the fully pipelined kernel.
    if (amode != 2 && d->k % BK == 0 && d->k > 0 && g_direct_lds &&
        epilogue_kind(g, bias, residual, pre_out) != EPI_GENERAL_ACT) {
        if (cfg < 0) {
            auto blocks = [&](int bm, int bn) { return (long long)ceil_div(d->m, bm) * ceil_div(d->n, bn) * batch; };
            const bool extra = grp || asum;   // operand pairs / row sums: the 128 x 128 tile only
            const long long t256 = blocks(256, 256), t128 = blocks(128, 128);
            const long long slots256 = ceil_div(t256, (long long)kCus) * kCus;
            if (d->k < 512) {
                // a handful of K steps (the batched products of an unfused attention): bound by the epilogue, where two
                // resident workgroups per compute unit overlap one's stores with the other's loads
                cfg = t128 > kCus ? 3 : 0;
            } else if (!extra && t256 * 10 >= slots256 * 9) {
                // Measured on MI355X, alone and inside the BERT layer (4096 x 4096 x 1024: 39 us against 45 - 54 us for
                // every 128-wide tile; 8192^3: 1176 TFLOP/s): the 256 x 256 tile halves the bytes each compute unit
                // pulls through L2 and LDS per MFMA, and the interleaved loop keeps its single wavefront per SIMD
                // issuing MFMAs while transfers and fragment reads are in flight. Only when its tiles fill (nearly) every
                // round of compute units: 192 tiles on 256 units lose more than the tile gains.
                cfg = 4;
            } else if (!extra && t128 <= kCus / 2) {
                // few tiles and a long K (1024 x 1024 x 4096: 24 us against 29 - 38 us): the 128 x 64 tile doubles the
                // workgroups, two of them per compute unit
                cfg = 9;
            } else if (d->k <= 1024 && t128 >= 2 * kCus) {
                // several rounds of short K loops (the grouped q / k / v projections: 768 tiles of 16 steps): with two
                // LDS stages instead of four, two workgroups share a compute unit and one's epilogue and first loads
                // overlap the other's loop - 45.3 against 46 - 49 us
                cfg = 7;
            } else if (!extra && d->k <= 1024 && t128 <= kCus && residual) {
                // a short K loop whose epilogue also reads a residual tile (4096 x 1024 x 1024: 20.3 - 21.1 against
                // 22.9 - 23.2 us): 128 x 64 tiles, two workgroups per compute unit, for the same overlap (without the
                // residual the two tiles are level: 18.2 us)
                cfg = 9;
            } else {
                // one 128 x 128 tile per compute unit, four LDS stages, interleaved loop: 5 - 20 % faster than the plain
                // loop on every product of the layer with 4096 x 1024 or 1024 x 4096 outputs
                cfg = 5;
            }
        }
        return launch_pipelined(g, (const _Float16*)a, (const _Float16*)b, c, bias, residual, pre_out, amode == 1 ? 4 : 3,
                                bmode == 1 ? 4 : 3, cfg, batch, st);
    }
    if (grp || asum) return DMLHIP_ERR_UNSUPPORTED;  // only the pipelined kernel takes pointer groups / makes row sums
    if (cfg < 0 || cfg > 2) {
        // Largest tile that still yields at least one workgroup per CU.
        auto blocks = [&](int bm, int bn) { return (long long)ceil_div(d->m, bm) * ceil_div(d->n, bn) * batch; };
        if (blocks(256, 256) >= 256) cfg = CFG_256x256;
        else if (blocks(256, 128) >= 256) cfg = CFG_256x128;
        else cfg = CFG_128x128;
    }
    if (amode == 2) cfg = CFG_128x128;
    switch (cfg) {
        case CFG_256x256: return launch_cfg<256, 256, 128, 128>(g, (const _Float16*)a, (const _Float16*)b, c, bias, residual, pre_out, amode, bmode,
                                                   batch, st);
        case CFG_256x128: return launch_cfg<256, 128, 128, 64>(g, (const _Float16*)a, (const _Float16*)b, c, bias, residual, pre_out, amode, bmode,
                                                   batch, st);
        default: return launch_cfg<128, 128, 64, 64>(g, (const _Float16*)a, (const _Float16*)b, c, bias, residual, pre_out, amode, bmode,
                                                   batch, st);
    }
}

// Number of K splits worth taking for this problem (1 = none).
static int split_k_factor(const dmlhip_gemm_desc* d) {
    if (!d || d->m <= 0 || d->n <= 0 || d->k < 1024 || d->batch[0] != 1) return 1;
    long long batch = d->batch[1] * d->batch[2];
    const long long tiles = ceil_div(d->m, 128) * ceil_div(d->n, 128) * batch;
    if (tiles > 128) return 1;
    int s = 1;
    while (tiles * s * 2 <= 256 && d->k / (s * 2) >= 256 && d->k % (s * 2 * 64) == 0) s *= 2;
    return s;
}

size_t dmlhip_gemm_f16_workspace_bytes(const dmlhip_gemm_desc* d) {
    const int s = split_k_factor(d);
    if (s <= 1) return 0;
    return (size_t)s * d->batch[1] * d->batch[2] * d->m * d->n * sizeof(float);
}

int dmlhip_gemm_f16_ws(const dmlhip_gemm_desc* d, const void* a, const void* b, void* c, const void* bias,
                       const void* residual, void* pre_out, void* workspace, size_t workspace_bytes, void* stream) {
    const int s = split_k_factor(d);
    const bool plain = d && !bias && !residual && !pre_out && d->beta == 0.f && d->act == DMLHIP_ACT_NONE;
    if (s <= 1 || !plain || !workspace || workspace_bytes < dmlhip_gemm_f16_workspace_bytes(d) || !a || !b || !c ||
        d->c_stride_m != d->n || (d->batch[1] * d->batch[2] > 1))
        return run_gemm_f16(d, a, b, c, bias, residual, pre_out, stream);
    // stage 1: batch slot 0 enumerates the K slices; partial C tiles are dense fp32 [s][m][n]
    dmlhip_gemm_desc p = *d;
    p.k = d->k / s;
    p.batch[0] = s;
    p.a_stride_batch[0] = p.k * d->a_stride_k;
    p.b_stride_batch[0] = p.k * d->b_stride_k;
    p.c_stride_batch[0] = d->m * d->n;
    p.c_stride_m = d->n;
    p.alpha = 1.f;
    p.out_dtype = DMLHIP_F32;
    if (int e = run_gemm_f16(&p, a, b, workspace, nullptr, nullptr, nullptr, stream)) return e;
    // stage 2: sum the slices, scale by alpha, convert
    const int64_t cols = d->m * d->n;
    hipStream_t st = (hipStream_t)stream;
    if (cols % 4 == 0) {
        int64_t blocks = ceil_div(cols / 4, 256);
        if (blocks > 256 * 16) blocks = 256 * 16;
        if (d->out_dtype == DMLHIP_F32)
            hipLaunchKernelGGL((sum_partials_vec4_kernel<float>), (unsigned)blocks, 256, 0, st, (const float*)workspace,
                               (float*)c, s, cols, cols, d->alpha);
        else
            hipLaunchKernelGGL((sum_partials_vec4_kernel<_Float16>), (unsigned)blocks, 256, 0, st,
                               (const float*)workspace, (_Float16*)c, s, cols, cols, d->alpha);
        return launch_status("gemm_f16(split-K sum)");
    }
    const unsigned grid = (unsigned)ceil_div(cols, kWave);
    if (d->out_dtype == DMLHIP_F32)
        hipLaunchKernelGGL((reduce_partials_kernel<OpSum, float>), grid, 1024, 0, st, (const float*)workspace, (float*)c,
                           s, cols, cols, 0.f, d->alpha, (float*)nullptr, (int64_t)0);
    else
        hipLaunchKernelGGL((reduce_partials_kernel<OpSum, _Float16>), grid, 1024, 0, st, (const float*)workspace,
                           (_Float16*)c, s, cols, cols, 0.f, d->alpha, (_Float16*)nullptr, (int64_t)0);
    return launch_status("gemm_f16(split-K sum)");
}

int dmlhip_gemm_f16(const dmlhip_gemm_desc* d, const void* a, const void* b, void* c, const void* bias,
                    const void* residual, void* pre_out, void* stream) {
    return run_gemm_f16(d, a, b, c, bias, residual, pre_out, stream);
}

int dmlhip_gemm_f16_grouped(const dmlhip_gemm_desc* d, int groups, const void* const* a, const void* const* b,
                            void* const* c, const void* const* bias, void* workspace, size_t workspace_bytes,
                            void* stream) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "gemm_f16_grouped: NULL descriptor");
    DML_REQUIRE(groups >= 1 && groups <= DMLHIP_GROUP_MAX, DMLHIP_ERR_SHAPE, "gemm_f16_grouped: %d groups outside 1..%d",
                groups, DMLHIP_GROUP_MAX);
    DML_REQUIRE(a && b && c, DMLHIP_ERR_NULL, "gemm_f16_grouped: NULL pointer table");
    DML_REQUIRE(d->batch[0] == 1, DMLHIP_ERR_SHAPE, "gemm_f16_grouped: the outer batch extent must be 1");
    for (int i = 0; i < groups; ++i) DML_REQUIRE(c[i], DMLHIP_ERR_NULL, "gemm_f16_grouped: NULL output %d", i);
    // one launch when every group has the alignment of group 0 and the pipelined kernel applies
    bool same = d->k > 0 && d->beta == 0.f;
    for (int i = 0; i < groups && same; ++i) {
        same = a[i] && b[i] && aligned16(a[i]) && aligned16(b[i]) && reinterpret_cast<uintptr_t>(c[i]) % 32 == 0 &&
               (!bias == !(bias && bias[i])) && (!bias || aligned16(bias[i]));
    }
    if (same && groups > 1) {
        dmlhip_gemm_desc p = *d;
        p.a_stride_batch[0] = p.b_stride_batch[0] = p.c_stride_batch[0] = 0;   // the outer batch index selects the group
        GemmGroup grp = {groups, a, b, c, bias, false};
        const int e = run_gemm_f16(&p, a[0], b[0], c[0], bias ? bias[0] : nullptr, nullptr, nullptr, stream, &grp);
        if (e == 0) ++g_grouped_single_launches;
        if (e != DMLHIP_ERR_UNSUPPORTED) return e;
    }
    for (int i = 0; i < groups; ++i)
        if (int e = dmlhip_gemm_f16_ws(d, a[i], b[i], c[i], bias ? bias[i] : nullptr, nullptr, nullptr, workspace,
                                       workspace_bytes, stream))
            return e;
    return 0;
}

size_t dmlhip_gemm_f16_grouped_asum_workspace_bytes(const dmlhip_gemm_desc* d) {
    if (!d) return 0;
    const size_t g = dmlhip_gemm_f16_workspace_bytes(d);
    const size_t r = dmlhip_reduce_workspace_bytes(1, d->k, d->m);
    return g > r ? g : r;
}

int dmlhip_gemm_f16_grouped_asum(const dmlhip_gemm_desc* d, int groups, const void* const* a, const void* const* b,
                                 void* const* c, void* const* asum, int asum_dtype, void* workspace,
                                 size_t workspace_bytes, void* stream) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "gemm_f16_grouped_asum: NULL descriptor");
    DML_REQUIRE(groups >= 1 && groups <= DMLHIP_GROUP_MAX, DMLHIP_ERR_SHAPE,
                "gemm_f16_grouped_asum: %d groups outside 1..%d", groups, DMLHIP_GROUP_MAX);
    DML_REQUIRE(a && b && c && asum, DMLHIP_ERR_NULL, "gemm_f16_grouped_asum: NULL pointer table");
    DML_REQUIRE(asum_dtype == DMLHIP_F16 || asum_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM,
                "gemm_f16_grouped_asum: bad asum_dtype");
    DML_REQUIRE(d->batch[0] == 1 && d->batch[1] == 1 && d->batch[2] == 1, DMLHIP_ERR_SHAPE,
                "gemm_f16_grouped_asum: batched products are not supported");
    DML_REQUIRE(d->beta == 0.f && d->act == DMLHIP_ACT_NONE, DMLHIP_ERR_UNSUPPORTED,
                "gemm_f16_grouped_asum: beta and activations are not supported");
    DML_REQUIRE(d->a_stride_m == 1 && d->a_stride_k == d->m, DMLHIP_ERR_UNSUPPORTED,
                "gemm_f16_grouped_asum: A must be stored as a dense [k, m] matrix");
    for (int i = 0; i < groups; ++i)
        DML_REQUIRE(c[i] && asum[i] && (d->k == 0 || (a[i] && b[i])), DMLHIP_ERR_NULL,
                    "gemm_f16_grouped_asum: NULL tensor in group %d", i);
    bool same = d->k > 0;
    for (int i = 0; i < groups && same; ++i)
        same = aligned16(a[i]) && aligned16(b[i]) && reinterpret_cast<uintptr_t>(c[i]) % 32 == 0;
    if (same) {
        int e;
        if (groups > 1) {
            dmlhip_gemm_desc p = *d;
            p.a_stride_batch[0] = p.b_stride_batch[0] = p.c_stride_batch[0] = 0;
            GemmGroup grp = {groups, a, b, c, nullptr, false};
            e = run_gemm_f16(&p, a[0], b[0], c[0], nullptr, nullptr, nullptr, stream, &grp, asum, asum_dtype == DMLHIP_F32);
        } else {
            e = run_gemm_f16(d, a[0], b[0], c[0], nullptr, nullptr, nullptr, stream, nullptr, asum, asum_dtype == DMLHIP_F32);
        }
        if (e == 0) ++g_grouped_single_launches;
        if (e != DMLHIP_ERR_UNSUPPORTED) return e;
    }
    // products and column sums of the stored [k, m] matrices one after the other
    for (int i = 0; i < groups; ++i) {
        if (int e = dmlhip_gemm_f16_ws(d, a[i], b[i], c[i], nullptr, nullptr, nullptr, workspace, workspace_bytes, stream))
            return e;
        if (int e = dmlhip_reduce_f16(DMLHIP_RSUM, a[i], asum[i], asum_dtype, 1, d->k, d->m, workspace, workspace_bytes,
                                      stream))
            return e;
    }
    return 0;
}

int dmlhip_gemm_f16_ksum(const dmlhip_gemm_desc* d, int groups, const void* const* a, const void* const* b, void* c,
                         const void* bias, const void* residual, void* stream) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "gemm_f16_ksum: NULL descriptor");
    DML_REQUIRE(groups >= 1 && groups <= DMLHIP_GROUP_MAX, DMLHIP_ERR_SHAPE, "gemm_f16_ksum: %d groups outside 1..%d",
                groups, DMLHIP_GROUP_MAX);
    DML_REQUIRE(a && b && c, DMLHIP_ERR_NULL, "gemm_f16_ksum: NULL pointer");
    DML_REQUIRE(d->beta == 0.f && d->act == DMLHIP_ACT_NONE, DMLHIP_ERR_UNSUPPORTED,
                "gemm_f16_ksum: beta and activations are not supported");
    for (int i = 0; i < groups; ++i) DML_REQUIRE(a[i] && b[i], DMLHIP_ERR_NULL, "gemm_f16_ksum: NULL operand %d", i);
    bool same = d->k > 0 && groups > 1;
    for (int i = 0; i < groups && same; ++i) same = aligned16(a[i]) && aligned16(b[i]);
    if (same) {
        GemmGroup grp = {groups, a, b, nullptr, nullptr, true};
        const int e = run_gemm_f16(d, a[0], b[0], c, bias, residual, nullptr, stream, &grp);
        if (e == 0) ++g_grouped_single_launches;
        if (e != DMLHIP_ERR_UNSUPPORTED) return e;
    }
    // one product after the other, accumulating in C (rounded to C's type in between)
    dmlhip_gemm_desc p = *d;
    for (int i = 0; i < groups; ++i) {
        if (int e = run_gemm_f16(&p, a[i], b[i], c, i == 0 ? bias : nullptr, i == 0 ? residual : nullptr, nullptr, stream))
            return e;
        p.beta = 1.f;
    }
    return 0;
}

}  // extern "C"
