// fp32 strided batched GEMM on the matrix cores with true fp32 products
// (v_mfma_f32_32x32x2_f32; no reduced-precision path), for the fp32 MatMul / Einsum / Gemm
// nodes and the 1x1 convolutions.
//
// A workgroup of 4 wavefronts owns a 128x128 tile of C and walks K in steps of 16. Tiles are
// staged in LDS as [k][row] (row contiguous, padded), which is what the 32x32x2 fragments read
// conflict-free: lane l takes element (row l%32, k l/32). Operands that are row-contiguous in
// memory go to LDS with 128-bit loads and stores as they are; K-contiguous operands are loaded
// 128 bits along K and scattered; other strides use element loads.
#include "common.h"

namespace dml {
namespace {

constexpr int kThreads = 256;
constexpr int TB = 128;        // tile rows (BM == BN)
constexpr int BK = 16;
constexpr int LDT = TB + 4;    // padded LDS row (floats)
constexpr int kXcds = 8;

struct GemmArgs32 {
    const float* a;
    const float* b;
    float* c;
    const void* bias;
    const float* residual;
    float* pre;
    int m, n, k;
    int64_t sam, sak, sbn, sbk, scm;
    int batch1, batch2;
    int64_t sab[3], sbb[3], scb[3];
    float alpha, beta;
    int bias_f32, act, bias_m;
    int tiles_m, tiles_n;
    long long total_blocks;
};

// MODE 0: K-contiguous (stride_k == 1), 1: row-contiguous (stride_row == 1), 2: generic.
template <int MODE>
struct Loader32 {
    floatx4 v[2];
    __device__ __forceinline__ void load(const float* base, int64_t s_row, int64_t s_k, int row0, int rows, int k0,
                                         int k) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int q = threadIdx.x + i * kThreads;  // 512 float4 per tile
            floatx4 t = {0.f, 0.f, 0.f, 0.f};
            if constexpr (MODE == 0) {
                const int r = q >> 2, kq = (q & 3) * 4;
                const int gr = row0 + r, gk = k0 + kq;
                const float* p = base + (int64_t)gr * s_row + gk;
                if (gr < rows && gk + 4 <= k) t = *reinterpret_cast<const floatx4*>(p);
                else if (gr < rows) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gk + e < k) t[e] = p[e];
                }
            } else if constexpr (MODE == 1) {
                const int kk = q >> 5, r = (q & 31) * 4;
                const int gr = row0 + r, gk = k0 + kk;
                const float* p = base + (int64_t)gk * s_k + gr;
                if (gk < k && gr + 4 <= rows) t = *reinterpret_cast<const floatx4*>(p);
                else if (gk < k) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gr + e < rows) t[e] = p[e];
                }
            } else {
                const int kk = q >> 5, r = (q & 31) * 4;
                const int gk = k0 + kk;
                if (gk < k) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (row0 + r + e < rows) t[e] = base[(int64_t)(row0 + r + e) * s_row + (int64_t)gk * s_k];
                }
            }
            v[i] = t;
        }
    }
    __device__ __forceinline__ void store(float* tile) const {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int q = threadIdx.x + i * kThreads;
            if constexpr (MODE == 0) {
                const int r = q >> 2, kq = (q & 3) * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) tile[(kq + e) * LDT + r] = v[i][e];
            } else {
                const int kk = q >> 5, r = (q & 31) * 4;
                *reinterpret_cast<floatx4*>(tile + kk * LDT + r) = v[i];
            }
        }
    }
};

template <int AMODE, int BMODE>
__global__ __launch_bounds__(kThreads) void gemm_f32_kernel(GemmArgs32 g) {
    __shared__ __attribute__((aligned(16))) float lds[2][2][BK * LDT];  // [buffer][A|B]

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
    const float* A = g.a + z0 * g.sab[0] + z1 * g.sab[1] + z2 * g.sab[2];
    const float* B = g.b + z0 * g.sbb[0] + z1 * g.sbb[1] + z2 * g.sbb[2];
    const int64_t coff = z0 * g.scb[0] + z1 * g.scb[1] + z2 * g.scb[2];
    const int m0 = tm * TB, n0 = tn * TB;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int wm = wave >> 1, wn = wave & 1;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    Loader32<AMODE> la;
    Loader32<BMODE> lb;
    const int nk = (g.k + BK - 1) / BK;
    la.load(A, g.sam, g.sak, m0, g.m, 0, g.k);
    lb.load(B, g.sbn, g.sbk, n0, g.n, 0, g.k);
    la.store(lds[0][0]);
    lb.store(lds[0][1]);
    __syncthreads();

    const int frow = lane & 31, fk = lane >> 5;
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < nk;
        if (more) {
            la.load(A, g.sam, g.sak, m0, g.m, (kt + 1) * BK, g.k);
            lb.load(B, g.sbn, g.sbk, n0, g.n, (kt + 1) * BK, g.k);
        }
        const float* at = lds[cur][0] + wm * 64 + frow;
        const float* bt = lds[cur][1] + wn * 64 + frow;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) af[i] = at[(kk + fk) * LDT + i * 32];
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[j] = bt[(kk + fk) * LDT + j * 32];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            la.store(lds[cur ^ 1][0]);
            lb.store(lds[cur ^ 1][1]);
        }
        __syncthreads();
    }

    const int ncol = lane & 31, mgrp = lane >> 5;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + wn * 64 + j * 32 + ncol;
        if (n >= g.n) continue;
        float bias_n = 0.f;
        if (g.bias && !g.bias_m) bias_n = g.bias_f32 ? reinterpret_cast<const float*>(g.bias)[n]
                                                     : (float)reinterpret_cast<const _Float16*>(g.bias)[n];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * 64 + i * 32 + (e >> 2) * 8 + mgrp * 4 + (e & 3);
                if (m >= g.m) continue;
                const int64_t off = coff + (int64_t)m * g.scm + n;
                float bias = bias_n;
                if (g.bias && g.bias_m) bias = g.bias_f32 ? reinterpret_cast<const float*>(g.bias)[m]
                                                          : (float)reinterpret_cast<const _Float16*>(g.bias)[m];
                float v = g.alpha * acc[i][j][e] + bias;
                if (g.pre) g.pre[off] = v;
                v = apply_act(g.act, v);
                if (g.residual) v += g.residual[off];
                if (g.beta != 0.f) v += g.beta * g.c[off];
                g.c[off] = v;
            }
        }
    }
}

int operand_mode32(const void* p, int64_t s_row, int64_t s_k, const int64_t* sb, const int64_t* batch) {
    bool bs_ok = true;
    for (int i = 0; i < 3; ++i)
        if (batch[i] > 1 && sb[i] % 4 != 0) bs_ok = false;
    if (!aligned16(p) || !bs_ok) return 2;
    if (s_k == 1 && s_row % 4 == 0) return 0;
    if (s_row == 1 && s_k % 4 == 0) return 1;
    return 2;
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" int dmlhip_gemm_f32(const dmlhip_gemm_desc* d, const void* a, const void* b, void* c, const void* bias,
                               const void* residual, void* pre_out, void* stream) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "gemm_f32: NULL descriptor");
    DML_REQUIRE(d->m >= 0 && d->n >= 0 && d->k >= 0, DMLHIP_ERR_SHAPE, "gemm_f32: negative extent");
    DML_REQUIRE(d->m <= 2147483647 / 2 && d->n <= 2147483647 / 2 && d->k <= 2147483647 / 2, DMLHIP_ERR_SHAPE,
                "gemm_f32: extent exceeds 2^30");
    long long batch = 1;
    for (int i = 0; i < 3; ++i) {
        DML_REQUIRE(d->batch[i] >= 0 && d->batch[i] <= 2147483647, DMLHIP_ERR_SHAPE, "gemm_f32: bad batch extent");
        batch *= d->batch[i];
        DML_REQUIRE(batch <= 2147483647LL, DMLHIP_ERR_SHAPE, "gemm_f32: batch too large");
    }
    DML_REQUIRE(d->out_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM, "gemm_f32: out_dtype must be DMLHIP_F32");
    DML_REQUIRE(d->bias_dtype == DMLHIP_F16 || d->bias_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM,
                "gemm_f32: bad bias_dtype");
    DML_REQUIRE(valid_act(d->act), DMLHIP_ERR_ENUM, "gemm_f32: bad act");
    DML_REQUIRE(d->a_stride_m >= 0 && d->a_stride_k >= 0 && d->b_stride_k >= 0 && d->b_stride_n >= 0 &&
                    d->c_stride_m >= 0,
                DMLHIP_ERR_SHAPE, "gemm_f32: negative stride");
    DML_REQUIRE(d->c_stride_m >= d->n || d->m <= 1, DMLHIP_ERR_SHAPE, "gemm_f32: rows of C overlap");
    if (d->m == 0 || d->n == 0 || batch == 0) return 0;
    DML_REQUIRE(c, DMLHIP_ERR_NULL, "gemm_f32: NULL output");
    DML_REQUIRE(d->k == 0 || (a && b), DMLHIP_ERR_NULL, "gemm_f32: NULL operand");

    GemmArgs32 g;
    g.a = (const float*)a; g.b = (const float*)b; g.c = (float*)c;
    g.bias = bias; g.residual = (const float*)residual; g.pre = (float*)pre_out;
    g.m = (int)d->m; g.n = (int)d->n; g.k = (int)d->k;
    g.sam = d->a_stride_m; g.sak = d->a_stride_k; g.sbn = d->b_stride_n; g.sbk = d->b_stride_k; g.scm = d->c_stride_m;
    g.batch1 = (int)d->batch[1]; g.batch2 = (int)d->batch[2];
    for (int i = 0; i < 3; ++i) {
        g.sab[i] = d->a_stride_batch[i]; g.sbb[i] = d->b_stride_batch[i]; g.scb[i] = d->c_stride_batch[i];
    }
    g.alpha = d->alpha; g.beta = d->beta;
    g.bias_f32 = d->bias_dtype == DMLHIP_F32; g.act = d->act;
    g.bias_m = d->bias_along_m != 0;
    g.tiles_m = (g.m + TB - 1) / TB;
    g.tiles_n = (g.n + TB - 1) / TB;
    const long long total = (long long)g.tiles_m * g.tiles_n * batch;
    DML_REQUIRE(total <= 2147483647LL, DMLHIP_ERR_SHAPE, "gemm_f32: too many workgroups");
    g.total_blocks = total;
    const int am = d->k == 0 ? 1 : operand_mode32(a, d->a_stride_m, d->a_stride_k, d->a_stride_batch, d->batch);
    const int bm = d->k == 0 ? 1 : operand_mode32(b, d->b_stride_n, d->b_stride_k, d->b_stride_batch, d->batch);
    hipStream_t st = (hipStream_t)stream;
#define DML_G32(AM, BMD) \
    if (am == AM && bm == BMD) hipLaunchKernelGGL((gemm_f32_kernel<AM, BMD>), (unsigned)total, kThreads, 0, st, g)
    DML_G32(0, 0); DML_G32(0, 1); DML_G32(0, 2);
    DML_G32(1, 0); DML_G32(1, 1); DML_G32(1, 2);
    DML_G32(2, 0); DML_G32(2, 1); DML_G32(2, 2);
#undef DML_G32
    return launch_status("gemm_f32");
}
