// Gradients of the two convolution forms an inverted-residual block is made of (fp32): depthwise KxK and pointwise.
// All three kernels are organised around reading the large tensors once, in rows, and are deterministic (partial sums
// go through a workspace and a fixed-order reduction, never atomics).
//
//   * depthwise data gradient: dX[iy, ix] = sum_{hy, hx} W[hy, hx] dY[(iy + P - hy) / S, (ix + P - hx) / S] over the taps
//     for which the divisions are exact. A thread owns S rows of four dX pixels; which taps reach which of its pixels
//     is known at compile time, so there is no divisibility test, each dY value of the small neighbourhood is loaded
//     once and a row's four pixels leave as one 16-byte store.
//   * depthwise weight gradient: dW[hy, hx] = sum_{n, oy, ox} dY[n, oy, ox] X[n, oy S - P + hy, ox S - P + hx]; one
//     workgroup per (image, channel) plane keeps K*K running sums per thread, the planes' results are summed over the
//     images by the reduction kernel.
//   * pointwise weight gradient: dW[m, c] = sum_{n, p} dY[n, m, p] X[n, c, p], a product with a tiny output and a
//     contraction over millions of pixels. A workgroup takes a range of pixels of one image, streams 64-pixel slabs
//     of both tensors through LDS and accumulates up to 8 x 1 blocks of 32 x 32 on v_mfma_f32_32x32x2f32, its four
//     wavefronts splitting the slab; the per-workgroup results are summed by the reduction kernel.
#include "common.h"

namespace dml {
namespace {

typedef float floatx2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------- depthwise, data gradient
// offsets (relative to the thread's cell) of the dY rows / columns that reach an S-block of dX
template <int K, int S, int P> struct DwBack {
    static constexpr int q(int i) { return (i + P) / S; }          // cell offset of pixel i's first tap
    static constexpr int r(int i) { return (i + P) % S; }          // first tap index
    static constexpr int taps(int i) { return r(i) < K ? (K - 1 - r(i)) / S + 1 : 0; }
    static constexpr int lo() {
        int v = 1 << 20;
        for (int i = 0; i < S; ++i)
            if (taps(i) > 0 && q(i) - (taps(i) - 1) < v) v = q(i) - (taps(i) - 1);
        return v;
    }
    static constexpr int hi() {
        int v = -(1 << 20);
        for (int i = 0; i < S; ++i)
            if (taps(i) > 0 && q(i) > v) v = q(i);
        return v;
    }
    static constexpr int span() { return hi() - lo() + 1; }
};

// CX adjacent cells per thread: with S * CX == 4 a thread's pixels of a row are one aligned 16-byte store, and the dY
// columns shared by neighbouring cells are loaded once.
template <int K, int S, int P, int CX>
__global__ __launch_bounds__(256) void depthwise_bwd_data_kernel(const float* __restrict__ dy, const float* __restrict__ w,
                                                                 float* __restrict__ dx, int c, int h, int wd, int oh, int ow,
                                                                 int cw, int cells, uint32_t chunks, int vec) {
    using G = DwBack<K, S, P>;
    constexpr int LO = G::lo(), NB = G::span(), NBX = NB + CX - 1, PX = S * CX;
    const uint32_t plane = blockIdx.x / chunks, chunk = blockIdx.x - plane * chunks;
    const int ci = (int)(plane % (uint32_t)c);
    float wk[K * K];
#pragma unroll
    for (int i = 0; i < K * K; ++i) wk[i] = w[ci * K * K + i];
    const float* gp = dy + (size_t)plane * oh * ow;
    float* xp = dx + (size_t)plane * h * wd;
#pragma unroll 1
    for (int rep = 0; rep < 8; ++rep) {
        const int idx = (int)chunk * 2048 + rep * 256 + (int)threadIdx.x;
        if (idx >= cells) return;
        const int a = idx / cw, b = (idx - a * cw) * CX;     // first cell of the thread's group
        float nb[NB][NBX];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int oy = a + LO + u;
#pragma unroll
            for (int v = 0; v < NBX; ++v) {
                const int ox = b + LO + v;
                const bool ok = oy >= 0 && oy < oh && ox >= 0 && ox < ow;
                nb[u][v] = ok ? gp[(size_t)(ok ? oy : 0) * ow + (ok ? ox : 0)] : 0.f;
            }
        }
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int iy = a * S + i;
            float out[PX];
#pragma unroll
            for (int cx = 0; cx < CX; ++cx)
#pragma unroll
                for (int j = 0; j < S; ++j) {
                    float acc = 0.f;
#pragma unroll
                    for (int t = 0; t < G::taps(i); ++t)
#pragma unroll
                        for (int u = 0; u < G::taps(j); ++u)
                            acc += wk[(G::r(i) + S * t) * K + G::r(j) + S * u] *
                                   nb[G::q(i) - t - LO][cx + G::q(j) - u - LO];
                    out[cx * S + j] = acc;
                }
            if (iy < h) {
                float* row = xp + (size_t)iy * wd + b * S;
                if constexpr (PX == 4) {
                    // row length a multiple of 4 and a 16-byte aligned tensor: one store for the thread's four pixels
                    if (vec) {
                        *reinterpret_cast<floatx4*>(row) = floatx4{out[0], out[1], out[2], out[3]};
                        continue;
                    }
                }
#pragma unroll
                for (int j = 0; j < PX; ++j)
                    if (b * S + j < wd) row[j] = out[j];
            }
        }
    }
}

// ---------------------------------------------------------------- depthwise, weight gradient
template <int K, int S>
__global__ __launch_bounds__(256) void depthwise_bwd_weight_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                                   float* __restrict__ part, int h, int wd, int oh, int ow,
                                                                   int pad) {
    __shared__ float red[4][K * K];
    const size_t plane = blockIdx.x;
    const float* xp = x + plane * h * wd;
    const float* gp = dy + plane * oh * ow;
    float acc[K * K];
#pragma unroll
    for (int i = 0; i < K * K; ++i) acc[i] = 0.f;
    const int total = oh * ow;
    for (int idx = threadIdx.x; idx < total; idx += 256) {
        const int oy = idx / ow, ox = idx - oy * ow;
        const float g = gp[idx];
        const int iy0 = oy * S - pad, ix0 = ox * S - pad;
#pragma unroll
        for (int hy = 0; hy < K; ++hy) {
            const int iy = iy0 + hy;
            const bool rok = iy >= 0 && iy < h;
#pragma unroll
            for (int hx = 0; hx < K; ++hx) {
                const int ix = ix0 + hx;
                const bool ok = rok && ix >= 0 && ix < wd;
                const float v = xp[ok ? (size_t)iy * wd + ix : 0];
                acc[hy * K + hx] += ok ? g * v : 0.f;
            }
        }
    }
    // wavefront sums first, then one exchange through LDS for all K * K values (a single barrier)
#pragma unroll
    for (int i = 0; i < K * K; ++i) acc[i] = wave_reduce<OpSum>(acc[i]);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < K * K; ++i) red[wave][i] = acc[i];
    }
    __syncthreads();
    if (threadIdx.x < K * K)
        part[plane * (K * K) + threadIdx.x] =
            (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// ---------------------------------------------------------------- pointwise, weight gradient
constexpr int kSlab = 64;        // pixels per LDS slab
constexpr int kPitch = kSlab + 2;  // rows land two banks apart: the two k halves of a wavefront read disjoint banks

struct PwGradArgs {
    const float* a;       // operand whose rows form the accumulators' rows: [n][ra][hw]
    const float* b;       // operand whose rows form the accumulators' columns: [n][rb][hw]
    float* part;          // [workgroups along x][out_elems]
    int ra, rb;
    int64_t hw;
    int chunk_px, chunks_per_img;
    int a_groups;         // workgroups along y = a_groups * ceil(rb / 32)
    int out_sa, out_sb;   // element (row of a, row of b) of the result lives at row_a * out_sa + row_b * out_sb
    int64_t out_elems;
};

template <int TA>
__global__ __launch_bounds__(256, 2) void pointwise_bwd_weight_kernel(const PwGradArgs g) {
    extern __shared__ __attribute__((aligned(16))) float pg_lds[];
    constexpr int ROWS = (TA + 1) * 32;              // TA blocks of a, then one block of b
    constexpr int NV = ROWS * (kSlab / 4) / 256;     // float4 loads per thread per slab
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int img = blockIdx.x / g.chunks_per_img, chunk = blockIdx.x - img * g.chunks_per_img;
    const int ag = blockIdx.y % g.a_groups, bt = blockIdx.y / g.a_groups;
    const int a0 = ag * TA * 32, b0 = bt * 32;
    const int64_t p_begin = (int64_t)chunk * g.chunk_px;
    const int64_t p_end = p_begin + g.chunk_px < g.hw ? p_begin + g.chunk_px : g.hw;
    const float* an = g.a + (int64_t)img * g.ra * g.hw;
    const float* bn = g.b + (int64_t)img * g.rb * g.hw;

    floatx16 acc[TA];
#pragma unroll
    for (int t = 0; t < TA; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

    // row / column of the slab this thread moves, per load
    floatx4 pre[NV];
    auto fetch = [&](int64_t p0) {
#pragma unroll
        for (int r = 0; r < NV; ++r) {
            const int idx = r * 256 + threadIdx.x, row = idx / (kSlab / 4), c4 = idx % (kSlab / 4);
            const bool is_b = row >= TA * 32;
            const int gr = is_b ? b0 + row - TA * 32 : a0 + row;
            const int lim = is_b ? g.rb : g.ra;
            const float* base = is_b ? bn : an;
            const int64_t p = p0 + c4 * 4;
            const bool ok = gr < lim && p < p_end;      // hw % 4 == 0 and chunk_px % 64 == 0: whole float4s
            floatx4 v = *reinterpret_cast<const floatx4*>(base + (int64_t)(ok ? gr : 0) * g.hw + (ok ? p : 0));
            if (!ok) v = floatx4{0.f, 0.f, 0.f, 0.f};
            pre[r] = v;
        }
    };
    if (p_begin < p_end) fetch(p_begin);
    for (int64_t p0 = p_begin; p0 < p_end; p0 += kSlab) {
        __syncthreads();      // the previous slab has been consumed
#pragma unroll
        for (int r = 0; r < NV; ++r) {
            const int idx = r * 256 + threadIdx.x, row = idx / (kSlab / 4), c4 = idx % (kSlab / 4);
            float* dst = pg_lds + row * kPitch + c4 * 4;
            *reinterpret_cast<floatx2*>(dst) = floatx2{pre[r][0], pre[r][1]};
            *reinterpret_cast<floatx2*>(dst + 2) = floatx2{pre[r][2], pre[r][3]};
        }
        __syncthreads();
        if (p0 + kSlab < p_end) fetch(p0 + kSlab);     // in flight while this slab is multiplied
        const float* bl = pg_lds + (TA * 32 + l32) * kPitch + wave * 16 + hh;
        const float* al = pg_lds + l32 * kPitch + wave * 16 + hh;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const float bv = bl[2 * ks];
#pragma unroll
            for (int t = 0; t < TA; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(al[t * 32 * kPitch + 2 * ks], bv, acc[t], 0, 0, 0);
        }
    }
    // sum the four wavefronts' blocks through LDS and write the workgroup's result
    float* out = g.part + (int64_t)blockIdx.x * g.out_elems;
#pragma unroll
    for (int t = 0; t < TA; ++t) {
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 16; ++e) pg_lds[wave * 1024 + e * 64 + lane] = acc[t][e];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int q = r * 256 + threadIdx.x;
            const float s = (pg_lds[q] + pg_lds[1024 + q]) + (pg_lds[2048 + q] + pg_lds[3072 + q]);
            const int e = q >> 6, ln = q & 63;
            const int row_a = a0 + t * 32 + (e >> 2) * 8 + (ln >> 5) * 4 + (e & 3);
            const int row_b = b0 + (ln & 31);
            if (row_a < g.ra && row_b < g.rb) out[(int64_t)row_a * g.out_sa + (int64_t)row_b * g.out_sb] = s;
        }
    }
}

// ---------------------------------------------------------------- dense KxK, weight gradient
// dW[m, j] = sum_{n, p} dY[n, m, p] * X[n, c(j), oy(p) s - pad + hy(j) d, ox(p) s - pad + hx(j) d] with j = (c, hy, hx)
// flattened as in W. Same scheme as the pointwise kernel above — 64-pixel slabs, accumulators' rows = output
// channels, columns = 32 consecutive j — but the slab of the second operand is gathered: row j of it is X shifted by
// j's tap. A workgroup covers a range of images and a range of each image's pixels.
struct DenseGradArgs {
    const float* x;
    const float* dy;
    float* part;          // [groups of images * pixel ranges][m * c * kh * kw]
    int n, c, h, w, m, kh, kw, sh, sw, ph, pw, dh, dw, oh, ow;
    int imgs_per_group, chunk_px, chunks_per_img;
    int a_groups, b_tiles;   // workgroups = a_groups * b_tiles * (image groups * pixel ranges); the first two vary fastest
};

template <int TA>
__global__ __launch_bounds__(256, 2) void dense_bwd_weight_kernel(const DenseGradArgs g) {
    extern __shared__ __attribute__((aligned(16))) float dg_lds[];
    constexpr int RA = TA * 8, RB = 8;               // rows of dY / of the gathered operand a thread moves per slab
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int ytiles = g.a_groups * g.b_tiles;
    const int yt = blockIdx.x % ytiles, xb = blockIdx.x / ytiles;
    const int ag = yt % g.a_groups, bt = yt / g.a_groups;
    const int grp = xb / g.chunks_per_img, chunk = xb - grp * g.chunks_per_img;
    const int a0 = ag * TA * 32, b0 = bt * 32;
    const int ohw = g.oh * g.ow, kk = g.kh * g.kw, jn = g.c * kk, in_plane = g.h * g.w;
    const int p_begin = chunk * g.chunk_px, p_end = min(p_begin + g.chunk_px, ohw);
    const int n_begin = grp * g.imgs_per_group, n_end = min(n_begin + g.imgs_per_group, g.n);
    const float inv_ow = 1.0f / (float)g.ow, inv_kk = 1.0f / (float)kk, inv_kw = 1.0f / (float)g.kw;

    // the rows of the gathered operand this thread fills: channel offset and tap shift of j = b0 + wave + 4 e
    int coff[RB], tshift[RB];
#pragma unroll
    for (int e = 0; e < RB; ++e) {
        const int j = b0 + wave + 4 * e;
        const int ch = fast_div(min(j, jn - 1), kk, inv_kk), tap = min(j, jn - 1) - ch * kk;
        const int hy = fast_div(tap, g.kw, inv_kw), hx = tap - hy * g.kw;
        coff[e] = j < jn ? ch * in_plane : -1;
        tshift[e] = ((hy * g.dh) << 16) | (hx * g.dw);
    }

    floatx16 acc[TA];
#pragma unroll
    for (int t = 0; t < TA; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

    float pa[RA], pb[RB];
    auto fetch = [&](int img, int p0) {
        const int p = p0 + lane;
        const bool pok = p < p_end;
        const int pc = pok ? p : p_begin;
        const float* dyn = g.dy + (size_t)img * g.m * ohw + pc;
#pragma unroll
        for (int e = 0; e < RA; ++e) {
            const int row = a0 + wave + 4 * e;
            const bool ok = pok && row < g.m;
            pa[e] = dyn[(size_t)(ok ? row : 0) * ohw];
            pa[e] = ok ? pa[e] : 0.f;
        }
        const int oy = fast_div(pc, g.ow, inv_ow), ox = pc - oy * g.ow;
        const int by = oy * g.sh - g.ph, bx = ox * g.sw - g.pw;
        const float* xn = g.x + (size_t)img * g.c * in_plane;
#pragma unroll
        for (int e = 0; e < RB; ++e) {
            const int iy = by + (tshift[e] >> 16), ix = bx + (tshift[e] & 0xffff);
            const bool ok = pok && coff[e] >= 0 && iy >= 0 && iy < g.h && ix >= 0 && ix < g.w;
            pb[e] = xn[ok ? coff[e] + iy * g.w + ix : 0];
            pb[e] = ok ? pb[e] : 0.f;
        }
    };
    int img = n_begin, p0 = p_begin;
    const bool any = n_begin < n_end && p_begin < p_end;
    if (any) fetch(img, p0);
    while (any && img < n_end) {
        __syncthreads();      // the previous slab has been consumed
#pragma unroll
        for (int e = 0; e < RA; ++e) dg_lds[(wave + 4 * e) * kPitch + lane] = pa[e];
#pragma unroll
        for (int e = 0; e < RB; ++e) dg_lds[(TA * 32 + wave + 4 * e) * kPitch + lane] = pb[e];
        __syncthreads();
        p0 += kSlab;
        if (p0 >= p_end) {
            p0 = p_begin;
            ++img;
        }
        if (img < n_end) fetch(img, p0);     // in flight while this slab is multiplied
        const float* bl = dg_lds + (TA * 32 + l32) * kPitch + wave * 16 + hh;
        const float* al = dg_lds + l32 * kPitch + wave * 16 + hh;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const float bv = bl[2 * ks];
#pragma unroll
            for (int t = 0; t < TA; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(al[t * 32 * kPitch + 2 * ks], bv, acc[t], 0, 0, 0);
        }
    }
    float* out = g.part + (size_t)xb * g.m * jn;
#pragma unroll
    for (int t = 0; t < TA; ++t) {
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 16; ++e) dg_lds[wave * 1024 + e * 64 + lane] = acc[t][e];
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int q = r * 256 + threadIdx.x;
            const float s = (dg_lds[q] + dg_lds[1024 + q]) + (dg_lds[2048 + q] + dg_lds[3072 + q]);
            const int e = q >> 6, ln = q & 63;
            const int row_a = a0 + t * 32 + (e >> 2) * 8 + (ln >> 5) * 4 + (e & 3);
            const int row_b = b0 + (ln & 31);
            if (row_a < g.m && row_b < jn) out[(size_t)row_a * jn + row_b] = s;
        }
    }
}

struct DenseGradPlan {
    int ta, a_groups, b_tiles, imgs_per_group, chunk_px, chunks_per_img;
    int64_t xblocks;
};

bool plan_dense_bwd_weight(int n, int c, int m, int kk, int oh, int ow, int h, int w, DenseGradPlan* pl) {
    const int64_t ohw = (int64_t)oh * ow, jn = (int64_t)c * kk;
    if (n < 1 || c < 1 || m < 1 || ohw < 64 || ohw > (1 << 22) || (int64_t)h * w > (1 << 28) || jn > (1 << 22)) return false;
    if ((int64_t)n * ohw * m * jn < (1LL << 24)) return false;          // tiny: the direct kernel
    const int tm = (int)ceil_div(m, 32);
    pl->a_groups = (tm + 7) / 8;
    pl->ta = (tm + pl->a_groups - 1) / pl->a_groups;
    pl->b_tiles = (int)ceil_div(jn, (int64_t)32);
    const int64_t ytiles = (int64_t)pl->a_groups * pl->b_tiles;
    int64_t want = ceil_div((int64_t)2048, ytiles);                      // ranges of the (image, pixel) space
    const int64_t cap = (64LL << 20) / ((int64_t)m * jn);                // at most 256 MiB of per-range results
    if (want > cap) want = cap;
    if (want < 1) want = 1;
    if (want >= n) {
        pl->imgs_per_group = 1;
        int64_t per_img = want / n;
        const int64_t max_per_img = ceil_div(ohw, (int64_t)256);
        if (per_img > max_per_img) per_img = max_per_img;
        pl->chunk_px = (int)(ceil_div(ceil_div(ohw, per_img), (int64_t)kSlab) * kSlab);
        pl->chunks_per_img = (int)ceil_div(ohw, (int64_t)pl->chunk_px);
        pl->xblocks = (int64_t)n * pl->chunks_per_img;
    } else {
        pl->imgs_per_group = (int)ceil_div((int64_t)n, want);
        pl->chunk_px = (int)(ceil_div(ohw, (int64_t)kSlab) * kSlab);
        pl->chunks_per_img = 1;
        pl->xblocks = ceil_div((int64_t)n, (int64_t)pl->imgs_per_group);
    }
    return pl->xblocks * ytiles <= 2147483647LL && pl->xblocks * (int64_t)m * jn < (1LL << 31);
}

struct PwGradPlan {
    bool swap;            // a = X (rows = input channels) instead of a = dY
    int ta, a_groups, b_tiles, chunk_px, chunks_per_img;
    int64_t blocks_x;
};

bool plan_pointwise_bwd_weight(int n, int m, int c, int64_t hw, PwGradPlan* pl) {
    if (n < 1 || m < 1 || c < 1 || hw < 256 || hw % 4 != 0) return false;
    const int tm = (int)ceil_div(m, 32), tc = (int)ceil_div(c, 32);
    // traffic of the two orientations in units of one pixel of one channel: the operand on the accumulators' columns
    // is re-read once per group of a, the other once per 32 rows of b
    auto groups = [](int tiles) { return (tiles + 7) / 8; };
    const double cost_dy_rows = (double)m * tc + (double)c * groups(tm);
    const double cost_x_rows = (double)c * tm + (double)m * groups(tc);
    pl->swap = cost_x_rows < cost_dy_rows;
    const int ta_tiles = pl->swap ? tc : tm;
    pl->b_tiles = pl->swap ? tm : tc;
    pl->a_groups = groups(ta_tiles);
    pl->ta = (ta_tiles + pl->a_groups - 1) / pl->a_groups;
    if ((pl->swap ? cost_x_rows : cost_dy_rows) > 4.0 * (m + c)) return false;   // a tiled GEMM re-reads less
    const int64_t ygroups = (int64_t)pl->a_groups * pl->b_tiles;
    int64_t per_img = ceil_div((int64_t)1024, (int64_t)n * ygroups);
    const int64_t max_per_img = ceil_div(hw, (int64_t)256);
    if (per_img > max_per_img) per_img = max_per_img;
    if (per_img < 1) per_img = 1;
    int64_t px = ceil_div(ceil_div(hw, per_img), (int64_t)kSlab) * kSlab;
    if (px > (1 << 30)) return false;
    pl->chunk_px = (int)px;
    pl->chunks_per_img = (int)ceil_div(hw, px);
    pl->blocks_x = (int64_t)n * pl->chunks_per_img;
    return pl->blocks_x <= 2147483647LL && ygroups <= 65535;
}

}  // namespace

// ---------------------------------------------------------------- launchers (called from the entry points in conv.hip)
bool depthwise_bwd_supported(int k, int s, int p) {
    return (k == 3 && p == 1 && (s == 1 || s == 2)) || (k == 5 && p == 2 && (s == 1 || s == 2));
}

int launch_depthwise_bwd_data(const float* dy, const float* w, float* dx, int n, int c, int h, int wd, int oh, int ow, int k,
                              int s, hipStream_t st) {
    const int cx = 4 / s;                                         // cells per thread: four pixels of a row
    const int ch = (h + s - 1) / s, cw = (int)ceil_div((wd + s - 1) / s, cx);
    const int64_t cells = (int64_t)ch * cw;
    const int64_t chunks = ceil_div(cells, (int64_t)2048);
    const int64_t blocks = (int64_t)n * c * chunks;
    DML_REQUIRE(cells <= (1 << 30) && blocks <= 2147483647LL, DMLHIP_ERR_SHAPE, "conv2d_backward_data: too many workgroups");
    const int vec = wd % 4 == 0 && ((uintptr_t)dx & 15) == 0;
#define DML_DWB(K, S, P)                                                                                               \
    if (k == K && s == S) {                                                                                            \
        hipLaunchKernelGGL((depthwise_bwd_data_kernel<K, S, P, 4 / S>), (unsigned)blocks, 256, 0, st, dy, w, dx, c, h, wd, \
                           oh, ow, cw, (int)cells, (uint32_t)chunks, vec);                                             \
        return launch_status("conv2d_backward_data(depthwise)");                                                       \
    }
    DML_DWB(3, 1, 1) DML_DWB(3, 2, 1) DML_DWB(5, 1, 2) DML_DWB(5, 2, 2)
#undef DML_DWB
    set_error("conv2d_backward_data: no depthwise kernel for k %d stride %d", k, s);
    return DMLHIP_ERR_UNSUPPORTED;
}

size_t depthwise_bwd_weight_partials(int n, int c, int k) { return (size_t)n * c * k * k; }

int launch_depthwise_bwd_weight(const float* x, const float* dy, float* part, int n, int c, int h, int wd, int oh, int ow,
                                int k, int s, int p, hipStream_t st) {
    const int64_t planes = (int64_t)n * c;
    DML_REQUIRE(planes <= 2147483647LL && (int64_t)oh * ow <= (1 << 30), DMLHIP_ERR_SHAPE,
                "conv2d_backward_weight: too many workgroups");
#define DML_DWW(K, S)                                                                                                  \
    if (k == K && s == S) {                                                                                            \
        hipLaunchKernelGGL((depthwise_bwd_weight_kernel<K, S>), (unsigned)planes, 256, 0, st, x, dy, part, h, wd, oh, ow, p); \
        return launch_status("conv2d_backward_weight(depthwise)");                                                     \
    }
    DML_DWW(3, 1) DML_DWW(3, 2) DML_DWW(5, 1) DML_DWW(5, 2)
#undef DML_DWW
    set_error("conv2d_backward_weight: no depthwise kernel for k %d stride %d", k, s);
    return DMLHIP_ERR_UNSUPPORTED;
}

// number of per-workgroup-range results (each m * c * kh * kw floats) of the dense weight gradient; 0 = not applicable
int64_t dense_bwd_weight_partials(int n, int c, int m, int kh, int kw, int oh, int ow, int h, int w) {
    DenseGradPlan pl;
    return plan_dense_bwd_weight(n, c, m, kh * kw, oh, ow, h, w, &pl) ? pl.xblocks : 0;
}

int launch_dense_bwd_weight(const float* x, const float* dy, float* part, int n, int c, int h, int w, int m, int kh, int kw,
                            int sh, int sw, int ph, int pw, int dh, int dw, int oh, int ow, hipStream_t st) {
    DenseGradPlan pl;
    DML_REQUIRE(plan_dense_bwd_weight(n, c, m, kh * kw, oh, ow, h, w, &pl), DMLHIP_ERR_UNSUPPORTED,
                "conv2d_backward_weight: the implicit-GEMM kernel does not apply");
    DML_REQUIRE(kh * dh < 32768 && kw * dw < 32768, DMLHIP_ERR_UNSUPPORTED, "conv2d_backward_weight: stencil too large");
    DenseGradArgs g;
    g.x = x; g.dy = dy; g.part = part;
    g.n = n; g.c = c; g.h = h; g.w = w; g.m = m; g.kh = kh; g.kw = kw; g.sh = sh; g.sw = sw; g.ph = ph; g.pw = pw;
    g.dh = dh; g.dw = dw; g.oh = oh; g.ow = ow;
    g.imgs_per_group = pl.imgs_per_group; g.chunk_px = pl.chunk_px; g.chunks_per_img = pl.chunks_per_img;
    g.a_groups = pl.a_groups; g.b_tiles = pl.b_tiles;
    const unsigned blocks = (unsigned)(pl.xblocks * pl.a_groups * pl.b_tiles);
    const size_t lds = (size_t)(pl.ta + 1) * 32 * kPitch * sizeof(float);
#define DML_DG(TA)                                                                                                     \
    case TA: {                                                                                                         \
        auto kern = dense_bwd_weight_kernel<TA>;                                                                       \
        if (lds > 64 * 1024) {                                                                                         \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
            if (e != hipSuccess) {                                                                                     \
                set_error("conv2d_backward_weight: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));  \
                return (int)e;                                                                                         \
            }                                                                                                          \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, blocks, 256, lds, st, g);                                                             \
        break;                                                                                                         \
    }
    switch (pl.ta) {
        DML_DG(1) DML_DG(2) DML_DG(3) DML_DG(4) DML_DG(5) DML_DG(6) DML_DG(7) DML_DG(8)
        default:
            set_error("conv2d_backward_weight: bad block count %d", pl.ta);
            return DMLHIP_ERR_UNSUPPORTED;
    }
#undef DML_DG
    return launch_status("conv2d_backward_weight(implicit GEMM)");
}

// number of per-workgroup results (each m * c floats) the pointwise weight gradient writes; 0 = not applicable
int64_t pointwise_bwd_weight_partials(int n, int m, int c, int64_t hw) {
    PwGradPlan pl;
    return plan_pointwise_bwd_weight(n, m, c, hw, &pl) ? pl.blocks_x : 0;
}

int launch_pointwise_bwd_weight(const float* x, const float* dy, float* part, int n, int m, int c, int64_t hw,
                                hipStream_t st) {
    PwGradPlan pl;
    DML_REQUIRE(plan_pointwise_bwd_weight(n, m, c, hw, &pl), DMLHIP_ERR_UNSUPPORTED,
                "conv2d_backward_weight: the pointwise kernel does not apply");
    PwGradArgs g;
    g.a = pl.swap ? x : dy;
    g.b = pl.swap ? dy : x;
    g.part = part;
    g.ra = pl.swap ? c : m;
    g.rb = pl.swap ? m : c;
    g.hw = hw;
    g.chunk_px = pl.chunk_px;
    g.chunks_per_img = pl.chunks_per_img;
    g.a_groups = pl.a_groups;
    g.out_sa = pl.swap ? 1 : c;       // dW is [m][c]
    g.out_sb = pl.swap ? c : 1;
    g.out_elems = (int64_t)m * c;
    const dim3 grid((unsigned)pl.blocks_x, (unsigned)(pl.a_groups * pl.b_tiles));
    const size_t lds = (size_t)(pl.ta + 1) * 32 * kPitch * sizeof(float);
#define DML_PWG(TA)                                                                                                    \
    case TA: {                                                                                                         \
        auto kern = pointwise_bwd_weight_kernel<TA>;                                                                   \
        if (lds > 64 * 1024) {                                                                                         \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
            if (e != hipSuccess) {                                                                                     \
                set_error("conv2d_backward_weight: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));  \
                return (int)e;                                                                                         \
            }                                                                                                          \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, grid, 256, lds, st, g);                                                               \
        break;                                                                                                         \
    }
    switch (pl.ta) {
        DML_PWG(1) DML_PWG(2) DML_PWG(3) DML_PWG(4) DML_PWG(5) DML_PWG(6) DML_PWG(7) DML_PWG(8)
        default:
            set_error("conv2d_backward_weight: bad block count %d", pl.ta);
            return DMLHIP_ERR_UNSUPPORTED;
    }
#undef DML_PWG
    return launch_status("conv2d_backward_weight(pointwise)");
}

}  // namespace dml
