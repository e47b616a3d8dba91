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
#include "common.h"

namespace dml {
namespace {

constexpr int kThreads = 256;
constexpr int BK = 64;         // K elements per step
constexpr int kRowBytes = BK * 2;
constexpr int kXcds = 8;

struct GemmArgs {
    const _Float16* a;
    const _Float16* b;
    void* c;
    const void* bias;
    const void* residual;
    void* pre;
    int m, n, k;
    int64_t sam, sak, sbn, sbk, scm;
    int batch1, batch2;  // extents of the two inner batch dims (outer one is implied)
    int64_t sab[3], sbb[3], scb[3];
    float alpha, beta;
    int out_f32, bias_f32, act, bias_m;
    int tiles_m, tiles_n;
    long long total_blocks;
};

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// ---------------------------------------------------------------- global -> registers
// K-contiguous operand: thread t loads chunks q = t + i*256 of the [R][64] tile.
template <int R>
struct LoaderKC {
    static constexpr int N = R * 8 / kThreads;
    u32x4 v[N];
    __device__ __forceinline__ void load(const _Float16* base, int64_t s_row, int row0, int rows, int k0, int k) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = q >> 3, c = q & 7;
            const int gr = row0 + r, gk = k0 + c * 8;
            const _Float16* p = base + (int64_t)gr * s_row + gk;
            if (gr < rows && gk + 8 <= k) {
                v[i] = *reinterpret_cast<const u32x4*>(p);
            } else {
                half8 h = {};
                if (gr < rows) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (gk + e < k) h[e] = p[e];
                }
                v[i] = __builtin_bit_cast(u32x4, h);
            }
        }
    }
    __device__ __forceinline__ void store(char* tile) const {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = q >> 3, c = q & 7;
            *reinterpret_cast<u32x4*>(tile + r * kRowBytes + ((c ^ swz(r)) << 4)) = v[i];
        }
    }
};

// Row-contiguous operand (element (row, k) at k*s_k + row): thread t owns K block kb = t/32
// (eight K values) of the RU rows starting at (t%32)*RU.
template <int R>
struct LoaderRC {
    static constexpr int RU = R / 32;  // 4 for R=128, 8 for R=256
    typedef _Float16 rowvec __attribute__((ext_vector_type(RU)));
    rowvec v[8];
    __device__ __forceinline__ void load(const _Float16* base, int64_t s_k, int row0, int rows, int k0, int k) {
        const int kb = threadIdx.x >> 5, rg = threadIdx.x & 31;
        const int gr = row0 + rg * RU;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int gk = k0 + kb * 8 + j;
            const _Float16* p = base + (int64_t)gk * s_k + gr;
            if (gk < k && gr + RU <= rows) {
                v[j] = *reinterpret_cast<const rowvec*>(p);
            } else {
                rowvec h = {};
                if (gk < k) {
#pragma unroll
                    for (int e = 0; e < RU; ++e)
                        if (gr + e < rows) h[e] = p[e];
                }
                v[j] = h;
            }
        }
    }
    __device__ __forceinline__ void store(char* tile) const {
        const int kb = threadIdx.x >> 5, rg = threadIdx.x & 31;
#pragma unroll
        for (int e = 0; e < RU; ++e) {
            half8 o;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = v[j][e];
            const int r = rg * RU + e;
            *reinterpret_cast<half8*>(tile + r * kRowBytes + ((kb ^ swz(r)) << 4)) = o;
        }
    }
};

// Any strides, any alignment: element loads. Correct everywhere, fast nowhere.
template <int R>
struct LoaderGeneric {
    static constexpr int N = R * 8 / kThreads;
    half8 v[N];
    __device__ __forceinline__ void load(const _Float16* base, int64_t s_row, int64_t s_k, int row0, int rows, int k0,
                                         int k) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int q = threadIdx.x + i * kThreads;
            const int r = q >> 3, c = q & 7;
            const int gr = row0 + r, gk = k0 + c * 8;
            half8 h = {};
            if (gr < rows) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (gk + e < k) h[e] = base[(int64_t)gr * s_row + (int64_t)(gk + e) * s_k];
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

template <int MODE, typename L>
__device__ __forceinline__ void do_load(L& l, const _Float16* base, int64_t s_row, int64_t s_k, int row0, int rows,
                                        int k0, int k) {
    if constexpr (MODE == 0) l.load(base, s_row, row0, rows, k0, k);
    else if constexpr (MODE == 1) l.load(base, s_k, row0, rows, k0, k);
    else l.load(base, s_row, s_k, row0, rows, k0, k);
}

// ---------------------------------------------------------------- the kernel
// AMODE / BMODE: 0 = K-contiguous, 1 = row-contiguous, 2 = generic strides.
template <int BM, int BN, int WM, int WN, int AMODE, int BMODE>
__global__ __launch_bounds__(kThreads) void gemm_f16_kernel(GemmArgs g) {
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
    const _Float16* A = g.a + z0 * g.sab[0] + z1 * g.sab[1] + z2 * g.sab[2];
    const _Float16* B = g.b + z0 * g.sbb[0] + z1 * g.sbb[1] + z2 * g.sbb[2];
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
    do_load<AMODE>(la, A, g.sam, g.sak, m0, g.m, 0, g.k);
    do_load<BMODE>(lb, B, g.sbn, g.sbk, n0, g.n, 0, g.k);
    la.store(lds);
    lb.store(lds + A_BYTES);
    __syncthreads();

    const int frow = lane & 31, fk = lane >> 5;
    for (int kt = 0; kt < nk; ++kt) {
        char* cur = lds + (kt & 1) * (A_BYTES + B_BYTES);
        char* nxt = lds + ((kt + 1) & 1) * (A_BYTES + B_BYTES);
        const bool more = kt + 1 < nk;
        if (more) {
            do_load<AMODE>(la, A, g.sam, g.sak, m0, g.m, (kt + 1) * BK, g.k);
            do_load<BMODE>(lb, B, g.sbn, g.sbk, n0, g.n, (kt + 1) * BK, g.k);
        }
        const char* at = cur + (wm * WM + frow) * kRowBytes;
        const char* bt = cur + A_BYTES + (wn * WN + frow) * kRowBytes;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            half8 af[TM], bf[TN];
            const int c = kk * 2 + fk;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = wm * WM + i * 32 + frow;
                af[i] = *reinterpret_cast<const half8*>(at + i * 32 * kRowBytes + ((c ^ swz(r)) << 4));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = wn * WN + j * 32 + frow;
                bf[j] = *reinterpret_cast<const half8*>(bt + j * 32 * kRowBytes + ((c ^ swz(r)) << 4));
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            la.store(nxt);
            lb.store(nxt + A_BYTES);
        }
        __syncthreads();
    }

    // ---- epilogue. acc[i][j][e] is C[m, n] with n = l%32 and m = (e/4)*8 + (l/32)*4 + e%4
    // inside the 32x32 block.
    const int ncol = lane & 31, mgrp = lane >> 5;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * WN + j * 32 + ncol;
        if (n >= g.n) continue;
        float bias_n = 0.f;
        if (g.bias && !g.bias_m) bias_n = g.bias_f32 ? reinterpret_cast<const float*>(g.bias)[n]
                                                     : (float)reinterpret_cast<const _Float16*>(g.bias)[n];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * WM + i * 32 + (e >> 2) * 8 + mgrp * 4 + (e & 3);
                if (m >= g.m) continue;
                const int64_t off = coff + (int64_t)m * g.scm + n;
                float bias = bias_n;
                if (g.bias && g.bias_m) bias = g.bias_f32 ? reinterpret_cast<const float*>(g.bias)[m]
                                                          : (float)reinterpret_cast<const _Float16*>(g.bias)[m];
                float v = g.alpha * acc[i][j][e] + bias;
                if (g.out_f32) {
                    if (g.pre) reinterpret_cast<float*>(g.pre)[off] = v;
                    v = apply_act(g.act, v);
                    if (g.residual) v += reinterpret_cast<const float*>(g.residual)[off];
                    if (g.beta != 0.f) v += g.beta * reinterpret_cast<float*>(g.c)[off];
                    reinterpret_cast<float*>(g.c)[off] = v;
                } else {
                    if (g.pre) {
                        // the un-fused graph stores the pre-activation in fp16 and reads it back
                        const _Float16 h = (_Float16)v;
                        reinterpret_cast<_Float16*>(g.pre)[off] = h;
                        v = (float)h;
                    }
                    v = apply_act(g.act, v);
                    if (g.residual) v += (float)reinterpret_cast<const _Float16*>(g.residual)[off];
                    if (g.beta != 0.f) v += g.beta * (float)reinterpret_cast<_Float16*>(g.c)[off];
                    reinterpret_cast<_Float16*>(g.c)[off] = (_Float16)v;
                }
            }
        }
    }
}

// ---------------------------------------------------------------- host side
enum { CFG_128x128 = 0, CFG_256x128 = 1, CFG_256x256 = 2 };

template <int BM, int BN, int WM, int WN>
int launch_cfg(GemmArgs& g, int amode, int bmode, long long batch, hipStream_t st) {
    g.tiles_m = (g.m + BM - 1) / BM;
    g.tiles_n = (g.n + BN - 1) / BN;
    const long long total = (long long)g.tiles_m * g.tiles_n * batch;
    DML_REQUIRE(total <= 2147483647LL, DMLHIP_ERR_SHAPE, "gemm_f16: %lld workgroups exceed the grid limit", total);
    g.total_blocks = total;
    const size_t lds = (size_t)2 * (BM + BN) * kRowBytes;
#define DML_GEMM_CASE(AM, BMD)                                                                                \
    if (amode == AM && bmode == BMD) {                                                                        \
        auto kern = gemm_f16_kernel<BM, BN, WM, WN, AM, BMD>;                                                 \
        if (lds > 64 * 1024) {                                                                                \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               (int)lds);                                                     \
            if (e != hipSuccess) {                                                                            \
                set_error("gemm_f16: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));        \
                return (int)e;                                                                                \
            }                                                                                                 \
        }                                                                                                     \
        hipLaunchKernelGGL(kern, (unsigned)total, kThreads, lds, st, g);                                      \
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

// 0 = K-contiguous with 16-byte-aligned rows, 1 = row-contiguous likewise, 2 = anything else
int operand_mode(const void* p, int64_t s_row, int64_t s_k, const int64_t* sb, const int64_t* batch) {
    bool bs_ok = true;
    for (int i = 0; i < 3; ++i)
        if (batch[i] > 1 && sb[i] % 8 != 0) bs_ok = false;
    if (!aligned16(p) || !bs_ok) return 2;
    if (s_k == 1 && s_row % 8 == 0) return 0;
    if (s_row == 1 && s_k % 8 == 0) return 1;
    return 2;
}

int g_force_cfg = -1;  // test hook: pin the tile configuration

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

// Not part of the public header: lets the tests exercise every tile configuration.
void dmlhip_debug_force_gemm_config(int cfg) { g_force_cfg = cfg; }

int dmlhip_gemm_f16(const dmlhip_gemm_desc* d, const void* a, const void* b, void* c, const void* bias,
                    const void* residual, void* pre_out, void* stream) {
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
    g.a = (const _Float16*)a;
    g.b = (const _Float16*)b;
    g.c = c;
    g.bias = bias;
    g.residual = residual;
    g.pre = pre_out;
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

    int amode = d->k == 0 ? 0 : operand_mode(a, d->a_stride_m, d->a_stride_k, d->a_stride_batch, d->batch);
    int bmode = d->k == 0 ? 0 : operand_mode(b, d->b_stride_n, d->b_stride_k, d->b_stride_batch, d->batch);
    if (amode == 2 || bmode == 2) amode = bmode = 2;
    hipStream_t st = (hipStream_t)stream;

    int cfg = g_force_cfg;
    if (cfg < 0) {
        // Largest tile that still yields at least one workgroup per CU.
        auto blocks = [&](int bm, int bn) { return (long long)ceil_div(d->m, bm) * ceil_div(d->n, bn) * batch; };
        if (blocks(256, 256) >= 256) cfg = CFG_256x256;
        else if (blocks(256, 128) >= 256) cfg = CFG_256x128;
        else cfg = CFG_128x128;
    }
    if (amode == 2) cfg = CFG_128x128;
    switch (cfg) {
        case CFG_256x256: return launch_cfg<256, 256, 128, 128>(g, amode, bmode, batch, st);
        case CFG_256x128: return launch_cfg<256, 128, 128, 64>(g, amode, bmode, batch, st);
        default: return launch_cfg<128, 128, 64, 64>(g, amode, bmode, batch, st);
    }
}

}  // extern "C"
