// Pointwise (1x1) convolution + activation followed by a 3x3 depthwise convolution + activation, in one kernel: the
// expanded tensor of an inverted-residual (MBConv) block — six times the block's input — lives only in LDS.
//
// Separately the two nodes are HBM-bound (write 6x, read 6x); fused they read X and write the depthwise output, and
// the work that remains is the pointwise product on the fp32 matrix pipe.
//
// Workgroup = (image, block of 32 expanded channels, strip of TOH output rows). Phase 1 computes the expanded,
// activated values of the IH = (TOH-1)*stride + 3 input rows the strip needs with v_mfma_f32_32x32x2f32 (A = the 32 x Cin
// weight block from LDS, B = 32 consecutive pixels of X straight from global memory, which are contiguous because
// strips span whole rows) and stores them to LDS as E[channel][row][1 + col], with zero columns left and right and
// zero rows outside the image — the depthwise convolution's padding. Phase 2 is the stencil: one wavefront per
// (channel, output row), lanes along the output columns.
#include "common.h"

namespace dml {
namespace {

constexpr int kFusedThreads = 256;
constexpr int kCB = 32;   // expanded channels per workgroup

struct FusedArgs {
    int n, cin, cmid, h, w, oh, ow, stride;
    int toh, ih, wp;          // output rows per strip, expanded rows per strip, LDS row pitch (w + 2)
    int strips, cblocks;
};

template <int ACT>
__device__ __forceinline__ float act_f(float v) {
    if constexpr (ACT == DMLHIP_ACT_SWISH) return v * sigmoid_epilogue_f(v);
    else if constexpr (ACT == DMLHIP_ACT_SIGMOID) return sigmoid_epilogue_f(v);
    else if constexpr (ACT == DMLHIP_ACT_RELU) return fmaxf(v, 0.f);
    else return v;
}

template <int ACT1, int ACT2>
__global__ __launch_bounds__(kFusedThreads) void expand_depthwise_kernel(const float* __restrict__ x,
                                                                         const float* __restrict__ we,
                                                                         const float* __restrict__ be,
                                                                         const float* __restrict__ wd,
                                                                         const float* __restrict__ bd,
                                                                         float* __restrict__ y, const FusedArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds_f[];
    float* E = lds_f;                                   // [kCB][ih][wp]
    float* WE = lds_f + kCB * a.ih * a.wp;              // [kCB][cin + 1]: the odd pitch spreads a column over the banks
    const int wep = a.cin + 1;
    float* WD = WE + kCB * wep;                         // [kCB][9 taps + bias]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    uint32_t bid = blockIdx.x;
    const int cb = (int)(bid % (uint32_t)a.cblocks);
    bid /= (uint32_t)a.cblocks;
    const int strip = (int)(bid % (uint32_t)a.strips);
    const int n = (int)(bid / (uint32_t)a.strips);
    const int c0 = cb * kCB;
    const int oy0 = strip * a.toh;
    const int iy0 = oy0 * a.stride - 1;                 // pad 1

    // ---- phase 0: weight blocks to LDS, zero border columns
    for (int i = threadIdx.x; i < kCB * a.cin; i += kFusedThreads)
        WE[(i / a.cin) * wep + i % a.cin] = we[(size_t)c0 * a.cin + i];
    for (int i = threadIdx.x; i < kCB * 10; i += kFusedThreads) {
        const int c = i / 10, t = i - c * 10;
        WD[i] = t < 9 ? wd[(size_t)(c0 + c) * 9 + t] : (bd ? bd[c0 + c] : 0.f);
    }
    for (int i = threadIdx.x; i < kCB * a.ih * 2; i += kFusedThreads) {
        const int r = i >> 1;
        E[r * a.wp + ((i & 1) ? a.wp - 1 : 0)] = 0.f;
    }
    __syncthreads();

    // ---- phase 1: E = act1(We X + be) for the strip's rows. The loads of the next chunk of 16 input channels are in
    // flight while the current one is multiplied.
    const int npix = a.ih * a.w;
    const int ntiles = (npix + 31) / 32;
    const int j = lane & 31, hh = lane >> 5;
    const int plane = a.h * a.w;
    const float* xn = x + (size_t)n * a.cin * plane;     // uniform base; per-lane offsets fit 32 bits (checked on the host)
    float bias1[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) bias1[e] = 0.f;
    if (be) {
#pragma unroll
        for (int e = 0; e < 16; ++e) bias1[e] = be[c0 + (e >> 2) * 8 + hh * 4 + (e & 3)];
    }
    const int chunks = a.cin / 16;
    constexpr int kWaves = kFusedThreads / 64;
    const int my_tiles = wave < ntiles ? (ntiles - wave + kWaves - 1) / kWaves : 0;
    const int steps = my_tiles * chunks;
    auto pixel_off = [&](int t) -> uint32_t {
        const int p = min(t * 32 + j, npix - 1);
        const int row = p / a.w;
        return (uint32_t)(hh * plane + min(max(iy0 + row, 0), a.h - 1) * a.w + (p - row * a.w));
    };
    // ring of kDepth chunks (16 input channels each) in flight per wavefront
    constexpr int kDepth = 4;
    float ring[kDepth][8];
    int it = wave, ich = 0;
    uint32_t ixo = steps > 0 ? pixel_off(it) : 0u;
    auto issue = [&](float (&dst)[8], int k) {
        if (k >= steps) return;
#pragma unroll
        for (int s = 0; s < 8; ++s) dst[s] = xn[ixo + (uint32_t)((ich * 16 + 2 * s) * plane)];
        if (++ich == chunks) {
            ich = 0;
            it += kWaves;
            if (k + 1 < steps) ixo = pixel_off(it);
        }
    };
#pragma unroll
    for (int d = 0; d < kDepth; ++d) issue(ring[d], d);
    floatx16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    int ct = wave, cch = 0;
    for (int i0 = 0; i0 < steps; i0 += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int i = i0 + d;
            if (i >= steps) break;
            float bc[8];
#pragma unroll
            for (int s = 0; s < 8; ++s) bc[s] = ring[d][s];
            issue(ring[d], i + kDepth);
            const float* wrow = WE + j * wep + cch * 16 + hh;
#pragma unroll
            for (int s = 0; s < 8; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(wrow[2 * s], bc[s], acc, 0, 0, 0);
            if (++cch == chunks) {
                cch = 0;
                const int p = ct * 32 + j;
                if (p < npix) {
                    const int row = p / a.w;
                    float* ep = E + row * a.wp + (p - row * a.w) + 1 + hh * 4 * a.ih * a.wp;
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        ep[((e >> 2) * 8 + (e & 3)) * a.ih * a.wp] = act_f<ACT1>(acc[e] + bias1[e]);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[e] = 0.f;
                ct += kWaves;
            }
        }
    }
    __syncthreads();
    // rows above / below the image are the depthwise convolution's zero padding (first and last strips only)
    if (iy0 < 0 || iy0 + a.ih > a.h) {
        for (int i = threadIdx.x; i < kCB * a.ih * a.w; i += kFusedThreads) {
            const int cr = i / a.w, cc = i - cr * a.w;
            const int iy = iy0 + cr % a.ih;
            if (iy < 0 || iy >= a.h) E[cr * a.wp + cc + 1] = 0.f;
        }
        __syncthreads();
    }

    // ---- phase 2: depthwise 3x3 stencil, lanes along the output columns; a wavefront takes a channel and two output
    // rows of the strip at a time, so that two independent chains of LDS reads and activations are in flight
    const int row_pairs = (a.toh + 1) / 2;
    for (int pr = wave; pr < kCB * row_pairs; pr += kWaves) {
        const int c = pr % kCB, orow = (pr / kCB) * 2;
        const int oy = oy0 + orow;
        if (oy >= a.oh) continue;
        const bool two = orow + 1 < a.toh && oy + 1 < a.oh;
        float wv[10];
#pragma unroll
        for (int i = 0; i < 10; ++i) wv[i] = WD[c * 10 + i];
        const float* e0 = E + (c * a.ih + orow * a.stride) * a.wp;
        const float* e1 = e0 + (two ? a.stride * a.wp : 0);
        float* yrow = y + (((size_t)n * a.cmid + c0 + c) * a.oh + oy) * a.ow;
        for (int oc = lane; oc < a.ow; oc += 64) {
            float s0 = wv[9], s1 = wv[9];
#pragma unroll
            for (int ky = 0; ky < 3; ++ky) {
                const float* r0 = e0 + ky * a.wp + oc * a.stride;
                const float* r1 = e1 + ky * a.wp + oc * a.stride;
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    s0 += wv[ky * 3 + kx] * r0[kx];
                    s1 += wv[ky * 3 + kx] * r1[kx];
                }
            }
            yrow[oc] = act_f<ACT2>(s0);
            if (two) yrow[a.ow + oc] = act_f<ACT2>(s1);
        }
    }
}

size_t fused_lds_bytes(int toh, int stride, int w, int cin) {
    const int ih = (toh - 1) * stride + 3;
    return ((size_t)kCB * ih * (w + 2) + (size_t)kCB * (cin + 1) + (size_t)kCB * 10) * sizeof(float);
}

thread_local int g_fused_toh = 0;   // diagnostic switch (per calling thread): pin the strip height

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

void dmlhip_debug_force_fused_strip(int toh) { g_fused_toh = toh; }

size_t dmlhip_conv2d_expand_depthwise_lds_bytes(int64_t w, int64_t cin, int64_t stride) {
    if (w <= 0 || w > 4096 || cin <= 0 || cin > (1 << 20) || (stride != 1 && stride != 2)) return 0;
    const size_t need = fused_lds_bytes(1, (int)stride, (int)w, (int)cin);
    return need <= 156 * 1024 ? need : 0;
}

int dmlhip_conv2d_expand_depthwise_f32(const dmlhip_conv2d_desc* pw, const dmlhip_conv2d_desc* dw, const void* x,
                                       const void* w_pw, const void* b_pw, const void* w_dw, const void* b_dw, void* y,
                                       void* stream) {
    DML_REQUIRE(pw && dw, DMLHIP_ERR_NULL, "conv2d_expand_depthwise: NULL descriptor");
    DML_REQUIRE(pw->n >= 0 && pw->c > 0 && pw->h > 0 && pw->w > 0 && pw->m > 0, DMLHIP_ERR_SHAPE,
                "conv2d_expand_depthwise: extents must be positive");
    DML_REQUIRE(valid_act(pw->act) && valid_act(dw->act) && pw->act != DMLHIP_ACT_GELU && dw->act != DMLHIP_ACT_GELU,
                DMLHIP_ERR_ENUM, "conv2d_expand_depthwise: unsupported activation");
    const bool pointwise = pw->kh == 1 && pw->kw == 1 && pw->stride_h == 1 && pw->stride_w == 1 && pw->pad_h == 0 &&
                           pw->pad_w == 0 && pw->group == 1;
    const bool depthwise = dw->kh == 3 && dw->kw == 3 && dw->pad_h == 1 && dw->pad_w == 1 && dw->dil_h == 1 &&
                           dw->dil_w == 1 && dw->stride_h == dw->stride_w && (dw->stride_h == 1 || dw->stride_h == 2) &&
                           dw->group == dw->c && dw->m == dw->c;
    DML_REQUIRE(pointwise && depthwise, DMLHIP_ERR_UNSUPPORTED,
                "conv2d_expand_depthwise: needs a 1x1 / stride 1 / unpadded convolution followed by a 3x3 depthwise "
                "convolution with padding 1 and stride 1 or 2");
    DML_REQUIRE(dw->n == pw->n && dw->c == pw->m && dw->h == pw->h && dw->w == pw->w, DMLHIP_ERR_SHAPE,
                "conv2d_expand_depthwise: the depthwise input must be the pointwise output");
    DML_REQUIRE(pw->c % 16 == 0 && pw->m % kCB == 0, DMLHIP_ERR_UNSUPPORTED,
                "conv2d_expand_depthwise: needs input channels %% 16 == 0 and expanded channels %% 32 == 0");
    DML_REQUIRE(pw->h * pw->w < (1LL << 30) && pw->w <= 4096 && pw->c * pw->h * pw->w < (1LL << 31), DMLHIP_ERR_UNSUPPORTED,
                "conv2d_expand_depthwise: image too large");
    if (pw->n == 0) return 0;
    DML_REQUIRE(x && w_pw && w_dw && y, DMLHIP_ERR_NULL, "conv2d_expand_depthwise: NULL tensor pointer");
    const int stride = (int)dw->stride_h;
    FusedArgs a;
    a.n = (int)pw->n; a.cin = (int)pw->c; a.cmid = (int)pw->m; a.h = (int)pw->h; a.w = (int)pw->w;
    a.stride = stride;
    a.oh = (a.h + 2 - 3) / stride + 1;
    a.ow = (a.w + 2 - 3) / stride + 1;
    // tallest strip that lets two workgroups share a CU's LDS, else the tallest that fits at all
    int toh = 0;
    for (int cand : {8, 4, 2, 1})
        if (!toh && fused_lds_bytes(cand, stride, a.w, a.cin) <= 78 * 1024) toh = cand;
    if (!toh) for (int cand : {4, 2, 1})
        if (!toh && fused_lds_bytes(cand, stride, a.w, a.cin) <= 156 * 1024) toh = cand;
    if (g_fused_toh > 0 && fused_lds_bytes(g_fused_toh, stride, a.w, a.cin) <= 156 * 1024) toh = g_fused_toh;
    DML_REQUIRE(toh > 0, DMLHIP_ERR_UNSUPPORTED, "conv2d_expand_depthwise: a row strip of width %d does not fit LDS", a.w);
    if (toh > a.oh) toh = a.oh;
    a.toh = toh;
    a.ih = (toh - 1) * stride + 3;
    a.wp = a.w + 2;
    a.strips = (a.oh + toh - 1) / toh;
    a.cblocks = a.cmid / kCB;
    const long long blocks = (long long)a.n * a.strips * a.cblocks;
    DML_REQUIRE(blocks <= 2147483647LL, DMLHIP_ERR_SHAPE, "conv2d_expand_depthwise: too many workgroups");
    const size_t lds = fused_lds_bytes(toh, stride, a.w, a.cin);
    hipStream_t st = (hipStream_t)stream;
#define DML_FUSED_CASE(A1, A2)                                                                                       \
    if (pw->act == A1 && dw->act == A2) {                                                                            \
        auto kern = expand_depthwise_kernel<A1, A2>;                                                                 \
        if (lds > 64 * 1024) {                                                                                       \
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
            if (e != hipSuccess) {                                                                                   \
                set_error("conv2d_expand_depthwise: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e)); \
                return (int)e;                                                                                       \
            }                                                                                                        \
        }                                                                                                            \
        hipLaunchKernelGGL(kern, (unsigned)blocks, kFusedThreads, lds, st, (const float*)x, (const float*)w_pw,      \
                           (const float*)b_pw, (const float*)w_dw, (const float*)b_dw, (float*)y, a);                \
        return launch_status("conv2d_expand_depthwise");                                                             \
    }
    DML_FUSED_CASE(DMLHIP_ACT_SWISH, DMLHIP_ACT_SWISH)
    DML_FUSED_CASE(DMLHIP_ACT_NONE, DMLHIP_ACT_NONE)
    DML_FUSED_CASE(DMLHIP_ACT_RELU, DMLHIP_ACT_RELU)
    DML_FUSED_CASE(DMLHIP_ACT_SWISH, DMLHIP_ACT_NONE)
    DML_FUSED_CASE(DMLHIP_ACT_NONE, DMLHIP_ACT_SWISH)
    DML_FUSED_CASE(DMLHIP_ACT_RELU, DMLHIP_ACT_NONE)
    DML_FUSED_CASE(DMLHIP_ACT_NONE, DMLHIP_ACT_RELU)
#undef DML_FUSED_CASE
    set_error("conv2d_expand_depthwise: no kernel for activations %d / %d", pw->act, dw->act);
    return DMLHIP_ERR_UNSUPPORTED;
}

}  // extern "C"
