// Dense (group 1) KxK convolution, fp32, as an implicit GEMM on v_mfma_f32_32x32x2f32:
//   Y[n, m, p] = act(b[m] + sum_{c, hy, hx} W[m, c, hy, hx] * X[n, c, oy(p) s - pad + hy d, ox(p) s - pad + hx d])
// with M = output channels, N = the oh*ow output pixels of one image (contiguous in Y) and K = (c, hy, hx). Nothing is
// materialised: a workgroup takes 128 or 256 consecutive output pixels of one image and up to 128 output channels, and
// walks over the input channels in chunks of 8. Per chunk the rectangle of X those pixels can touch (whole rows, with
// the padding written as zeros) and the chunk's weights go to LDS; every tap is then a shifted read of the same
// rectangle. A = W (rows = output channels), B = X (columns = pixels): a lane's accumulators are 16 output channels
// of one pixel, so the stores of a wavefront run along the pixels.
#include "common.h"
#include "conv_geom.h"

#include <type_traits>

namespace dml {
namespace {

constexpr int kIgChunk = 8;   // input channels per LDS chunk

struct ImplicitArgs {
    int c, h, w, m, kh, kw, sh, sw, ph, pw, dh, dw, oh, ow, act;
    int prow, pwid, plane;    // rectangle rows / columns, and the per-channel pitch in LDS (== 32 mod 64: the two input
                              // channels a wavefront reads at once sit in different bank halves)
    int wpitch;               // LDS pitch of a weight row: kIgChunk * kh * kw + 1
    // data-gradient mode: the input (dY) is read as if ids - 1 zeros stood between its rows / columns (the forward
    // stride), and the weights as W[input channel][output channel] with the taps reversed
    int ids_h, ids_w, wflip;
};

// Few accumulators (MT * PT <= 2 blocks of 32 x 32) leave room for four workgroups per CU instead of two: their
// staging phases and matrix phases overlap each other.
template <int MT, int PT>
__global__ __launch_bounds__(256, (MT * PT <= 2 ? 4 : 2)) void conv_implicit_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                   const float* __restrict__ bias, float* __restrict__ y,
                                                                   const ImplicitArgs g) {
    constexpr int PX = 128 * PT;
    extern __shared__ __attribute__((aligned(16))) float ig_lds[];
    float* xs = ig_lds;                               // [kIgChunk][plane]
    float* ws = xs + kIgChunk * g.plane;              // [MT*32][wpitch]
    float* bs = ws + MT * 32 * g.wpitch;              // [MT*32]
    const int n = blockIdx.y;
    const int ohw = g.oh * g.ow;
    const int p0 = blockIdx.x * PX;
    const int m0 = blockIdx.z * MT * 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    const int kk = g.kh * g.kw;

    // rows of X the workgroup's pixels can touch
    const int oy_first = p0 / g.ow;
    const int iy_first = oy_first * g.sh - g.ph;
    const int ix_first = -g.pw;

    // per-lane offset of each of its pixels inside a channel's rectangle (tap 0)
    int base[PT];
#pragma unroll
    for (int j = 0; j < PT; ++j) {
        const int p = min(p0 + wave * 32 * PT + j * 32 + l32, ohw - 1);
        const int oy = p / g.ow, ox = p - oy * g.ow;
        base[j] = (oy - oy_first) * g.sh * g.pwid + ox * g.sw + hh * g.plane;
    }

    floatx16 acc[MT][PT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    if (threadIdx.x < MT * 32) bs[threadIdx.x] = (bias && m0 + (int)threadIdx.x < g.m) ? bias[m0 + threadIdx.x] : 0.f;
    const float* xn = x + (size_t)n * g.c * g.h * g.w;
    const int rect = g.prow * g.pwid;
    const int wrow = kIgChunk * kk;     // weights of a chunk per output channel (contiguous in W)
    const float inv_pwid = 1.0f / (float)g.pwid, inv_wrow = 1.0f / (float)wrow, inv_kk = 1.0f / (float)kk;
    const float inv_ids_h = 1.0f / (float)g.ids_h, inv_ids_w = 1.0f / (float)g.ids_w;
    const int in_plane = g.h * g.w;
    for (int kc = 0; kc < g.c; kc += kIgChunk) {
        __syncthreads();   // the previous chunk has been consumed
        const int cl = min(kIgChunk, g.c - kc);
        // rectangle: kIgChunk channels x prow rows x pwid columns, zeros outside the image and past the last channel.
        // A thread resolves (row, column) of two rectangle positions once and loads them for all channels of the
        // chunk: sixteen loads in flight per round trip.
        // uniform bases + 32-bit offsets: a chunk of X and the weight tensor have fewer than 2^31 elements
        const float* xc = xn + (size_t)kc * in_plane;
        const float* wc = w + (size_t)kc * (g.wflip ? g.m * kk : kk);
        for (int i0 = 0; i0 < rect; i0 += 512) {
            int pos[2], off[2];
            bool ok[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                pos[u] = i0 + u * 256 + (int)threadIdx.x;
                const int row = fast_div(pos[u], g.pwid, inv_pwid), col = pos[u] - row * g.pwid;
                int iy = iy_first + row, ix = ix_first + col;
                bool on_grid = iy >= 0 && ix >= 0;
                if (g.ids_h > 1 || g.ids_w > 1) {     // only every ids-th position of the dilated input holds a value
                    const int qy = fast_div(max(iy, 0), g.ids_h, inv_ids_h), qx = fast_div(max(ix, 0), g.ids_w, inv_ids_w);
                    on_grid = on_grid && qy * g.ids_h == iy && qx * g.ids_w == ix;
                    iy = qy;
                    ix = qx;
                }
                ok[u] = pos[u] < rect && on_grid && iy < g.h && ix < g.w;
                off[u] = ok[u] ? iy * g.w + ix : 0;
            }
            float v[2][kIgChunk];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int ch = 0; ch < kIgChunk; ++ch)
                    v[u][ch] = xc[(uint32_t)(min(ch, cl - 1) * in_plane + off[u])];
#pragma unroll
            for (int u = 0; u < 2; ++u)
                if (pos[u] < rect) {
#pragma unroll
                    for (int ch = 0; ch < kIgChunk; ++ch) xs[ch * g.plane + pos[u]] = (ok[u] && ch < cl) ? v[u][ch] : 0.f;
                }
        }
        // weights: the chunk's cl * kh * kw values of an output channel are contiguous in W. A thread stays on one
        // output channel and strides over k, so source and LDS index are a base plus k; six loads per round trip
        {
            constexpr int TPR = 8 / MT;                      // threads per output channel
            const int row = (int)threadIdx.x / TPR, q = (int)threadIdx.x % TPR;
            const bool rok = m0 + row < g.m;
            const int klim = rok ? cl * kk : 0;              // k at and beyond it is zero-filled
            const int sbase = (m0 + (rok ? row : 0)) * (g.wflip ? kk : g.c * kk);
            float* wdst = ws + row * g.wpitch;
            for (int k0 = q; k0 < wrow; k0 += 6 * TPR) {
                float v[6];
#pragma unroll
                for (int u = 0; u < 6; ++u) {
                    const int k = k0 + u * TPR;
                    const bool ok = k < klim;
                    int src = sbase + k;
                    if (g.wflip) {
                        const int ch = fast_div(ok ? k : 0, kk, inv_kk), tap = (ok ? k : 0) - ch * kk;
                        src = sbase + ch * g.m * kk + (kk - 1 - tap);
                    }
                    v[u] = wc[(uint32_t)(ok ? src : 0)];
                    v[u] = ok ? v[u] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 6; ++u)
                    if (k0 + u * TPR < wrow) wdst[k0 + u * TPR] = v[u];
            }
        }
        __syncthreads();
        for (int hy = 0; hy < g.kh; ++hy)
            for (int hx = 0; hx < g.kw; ++hx) {
                const int tap = hy * g.kw + hx;
                const int toff = hy * g.dh * g.pwid + hx * g.dw;
                const float* wl = ws + l32 * g.wpitch + hh * kk + tap;
#pragma unroll
                for (int cp = 0; cp < kIgChunk / 2; ++cp) {
                    float b[PT];
#pragma unroll
                    for (int j = 0; j < PT; ++j) b[j] = xs[base[j] + toff + 2 * cp * g.plane];
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        const float a = wl[i * 32 * g.wpitch + 2 * cp * kk];
#pragma unroll
                        for (int j = 0; j < PT; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[j], acc[i][j], 0, 0, 0);
                    }
                }
            }
    }
    float* yn = y + (size_t)n * g.m * ohw;
    auto store_all = [&](auto actc) {
        constexpr int ACT = decltype(actc)::value;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < PT; ++j) {
                const int p = p0 + wave * 32 * PT + j * 32 + l32;
                if (p >= ohw) continue;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int ml = i * 32 + (e >> 2) * 8 + hh * 4 + (e & 3);
                    if (m0 + ml < g.m) yn[(size_t)(m0 + ml) * ohw + p] = apply_act(ACT, acc[i][j][e] + bs[ml]);
                }
            }
    };
    switch (g.act) {
        case DMLHIP_ACT_GELU: store_all(std::integral_constant<int, DMLHIP_ACT_GELU>{}); break;
        case DMLHIP_ACT_SWISH: store_all(std::integral_constant<int, DMLHIP_ACT_SWISH>{}); break;
        case DMLHIP_ACT_SIGMOID: store_all(std::integral_constant<int, DMLHIP_ACT_SIGMOID>{}); break;
        case DMLHIP_ACT_RELU: store_all(std::integral_constant<int, DMLHIP_ACT_RELU>{}); break;
        default: store_all(std::integral_constant<int, DMLHIP_ACT_NONE>{}); break;
    }
}

struct ImplicitPlan {
    ImplicitArgs a;
    int mt, pt;
    size_t lds;
    dim3 grid;
};

// g describes the convolution the kernel runs: for a data gradient that is the stride-1 convolution of the
// (zero-dilated) dY with the reversed weights, not the forward one.
bool plan_implicit(const ConvGeom& g, int ids_h, int ids_w, int wflip, ImplicitPlan* pl) {
    if (g.group != 1 || g.c < 1 || g.m < 1 || g.oh < 1 || g.ow < 1 || g.n < 1 || g.n > 65535) return false;
    // worth the staging only with enough arithmetic per output; tiny products stay on the direct kernel
    const int64_t kdim = (int64_t)g.c * g.kh * g.kw;
    if (kdim < 32 || (int64_t)g.oh * g.ow < 64 || g.kh * g.kw > 121) return false;
    if ((int64_t)g.n * g.m * g.oh * g.ow * kdim < (1LL << 24)) return false;
    const int64_t ohw = (int64_t)g.oh * g.ow;
    if (ohw > (1 << 22) || (int64_t)g.h * g.w > (1 << 28) || (int64_t)g.h * ids_h > (1 << 22) ||
        (int64_t)g.w * ids_w > (1 << 22))
        return false;
    int mt = (int)ceil_div(g.m, 32);
    mt = mt >= 4 ? 4 : (mt == 3 ? 4 : mt);
    ImplicitArgs& a = pl->a;
    a.c = g.c; a.h = g.h; a.w = g.w; a.m = g.m; a.kh = g.kh; a.kw = g.kw; a.sh = g.sh; a.sw = g.sw; a.ph = g.ph; a.pw = g.pw;
    a.dh = g.dh; a.dw = g.dw; a.oh = g.oh; a.ow = g.ow; a.act = g.act;
    a.ids_h = ids_h; a.ids_w = ids_w; a.wflip = wflip;
    a.pwid = (g.ow - 1) * g.sw + (g.kw - 1) * g.dw + 1;
    a.wpitch = kIgChunk * g.kh * g.kw + 1;
    for (int pt = 2; pt >= 1; --pt) {
        const int px = 128 * pt;
        const int64_t blocks = ceil_div(ohw, (int64_t)px) * g.n * ceil_div(g.m, mt * 32);
        if (pt == 2 && blocks < 384) continue;          // few workgroups: smaller ones fill the chip better
        // output rows a block of px consecutive pixels can span, then the input rows under them
        const int span = (int)((px - 1 + g.ow - 1) / g.ow) + 1;
        const int rows = span < g.oh ? span : g.oh;
        a.prow = (rows - 1) * g.sh + (g.kh - 1) * g.dh + 1;
        const int64_t rect = (int64_t)a.prow * a.pwid;
        if (rect > (1 << 20) || (int64_t)mt * 32 * kIgChunk * g.kh * g.kw > (1 << 20)) continue;
        if ((int64_t)g.m * g.c * g.kh * g.kw >= (1LL << 31) || (int64_t)kIgChunk * g.h * g.w >= (1LL << 31)) continue;
        a.plane = (int)(ceil_div(rect + 32, (int64_t)64) * 64 - 32);   // >= rect, == 32 (mod 64)
        const size_t lds = ((size_t)kIgChunk * a.plane + (size_t)mt * 32 * a.wpitch + mt * 32) * sizeof(float);
        if (lds > 72 * 1024) continue;                  // two workgroups per CU
        pl->mt = mt;
        pl->pt = pt;
        pl->lds = lds;
        pl->grid = dim3((unsigned)ceil_div(ohw, (int64_t)px), (unsigned)g.n, (unsigned)ceil_div(g.m, mt * 32));
        return true;
    }
    return false;
}

// The data gradient of a dense convolution as a convolution: dX = conv(dY with s - 1 zeros between its elements,
// W with input / output channels exchanged and the taps reversed, stride 1, padding (k - 1) d - p).
bool data_gradient_problem(const ConvGeom& f, ConvGeom* b) {
    const int ph = (f.kh - 1) * f.dh - f.ph, pw = (f.kw - 1) * f.dw - f.pw;
    if (f.group != 1 || ph < 0 || pw < 0) return false;
    *b = f;
    b->c = f.m; b->m = f.c;            // channels exchanged
    b->h = f.oh; b->w = f.ow;          // the input is dY ...
    b->oh = f.h; b->ow = f.w;          // ... the output dX
    b->sh = b->sw = 1;
    b->ph = ph; b->pw = pw;
    b->cg = b->c; b->mg = b->m;
    b->act = DMLHIP_ACT_NONE;
    return true;
}

int launch_planned(const ImplicitPlan& pl, const float* x, const float* w, const float* bias, float* y, hipStream_t st,
                   const char* what) {
#define DML_IG(MT, PT)                                                                                                 \
    if (pl.mt == MT && pl.pt == PT) {                                                                                  \
        auto kern = conv_implicit_f32_kernel<MT, PT>;                                                                  \
        if (pl.lds > 64 * 1024) {                                                                                      \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds); \
            if (e != hipSuccess) {                                                                                     \
                set_error("%s: cannot reserve %zu bytes of LDS: %s", what, pl.lds, hipGetErrorString(e));             \
                return (int)e;                                                                                         \
            }                                                                                                          \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, pl.grid, 256, pl.lds, st, x, w, bias, y, pl.a);                                       \
        return launch_status(what);                                                                                    \
    }
    DML_IG(1, 1) DML_IG(1, 2) DML_IG(2, 1) DML_IG(2, 2) DML_IG(4, 1) DML_IG(4, 2)
#undef DML_IG
    set_error("%s: no implicit-GEMM kernel for %d x %d blocks", what, pl.mt, pl.pt);
    return DMLHIP_ERR_UNSUPPORTED;
}

}  // namespace

bool conv_implicit_applicable(const ConvGeom& g) {
    ImplicitPlan pl;
    return plan_implicit(g, 1, 1, 0, &pl);
}

int launch_conv_implicit_f32(const ConvGeom& g, const float* x, const float* w, const float* bias, float* y, hipStream_t st) {
    ImplicitPlan pl;
    DML_REQUIRE(plan_implicit(g, 1, 1, 0, &pl), DMLHIP_ERR_UNSUPPORTED, "conv2d: the implicit-GEMM kernel does not apply");
    return launch_planned(pl, x, w, bias, y, st, "conv2d(implicit GEMM)");
}

bool conv_implicit_bwd_data_applicable(const ConvGeom& g) {
    ConvGeom b;
    ImplicitPlan pl;
    return data_gradient_problem(g, &b) && plan_implicit(b, g.sh, g.sw, 1, &pl);
}

int launch_conv_implicit_bwd_data_f32(const ConvGeom& g, const float* dy, const float* w, float* dx, hipStream_t st) {
    ConvGeom b;
    ImplicitPlan pl;
    DML_REQUIRE(data_gradient_problem(g, &b) && plan_implicit(b, g.sh, g.sw, 1, &pl), DMLHIP_ERR_UNSUPPORTED,
                "conv2d_backward_data: the implicit-GEMM kernel does not apply");
    return launch_planned(pl, dy, w, nullptr, dx, st, "conv2d_backward_data(implicit GEMM)");
}

}  // namespace dml
