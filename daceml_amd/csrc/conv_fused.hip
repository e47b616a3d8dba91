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

// ---- the same product with a rolling window: a workgroup keeps its (image, channel block) and walks down a segment
// of output rows, R rows at a time. The expanded rows live in a ring in LDS, so a row is expanded once per segment
// instead of once per strip (the strips above share 3 - stride of their (TOH - 1) * stride + 3 rows with each
// neighbour), weights and borders are set up once per segment, and the two phases run at the same time: the lower
// half of the wavefronts expands the rows of the next batch on the matrix pipe while the upper half runs the stencil
// of the current one on the vector pipe, one barrier per batch.
//
// Ring: the rows a batch reads, [lo_b, hi_b] with lo_b = oy_b * stride - 1 and hi_b = (oy_b + R - 1) * stride + 1, plus
// the rows the next batch adds, (hi_b, hi_{b+1}], are 2 R stride + 3 - stride consecutive rows; row iy sits in slot
// (iy - lo_0) mod ring.
struct RollArgs {
    int n, cin, cmid, h, w, oh, ow, stride;
    int r, ring, wp;             // output rows per batch, expanded rows in LDS, LDS row pitch (w + 2)
    int seg_rows, segs, cblocks; // output rows per segment, segments per image, blocks of kCB expanded channels
    uint32_t total;              // workgroups
    uint32_t magic_w, magic_ow;  // ceil(2^32 / w), ceil(2^32 / ow), 0 for a divisor of 1: see div_small
};

// p / d for p * d < 2^32 through the high half of a product with magic = ceil(2^32 / d); the quotient of a division by 1
// has no such constant in 32 bits and is marked by magic == 0.
__device__ __forceinline__ int div_small(int p, uint32_t magic) {
    return magic ? (int)__umulhi((uint32_t)p, magic) : p;
}
inline uint32_t div_magic(int d) { return d == 1 ? 0u : (uint32_t)((0x100000000ULL + (uint32_t)d - 1) / (uint32_t)d); }

inline size_t rolling_lds_bytes(int r, int stride, int w, int cin) {
    const int ring = 2 * r * stride + 3 - stride;
    return ((size_t)kCB * ring * (w + 2) + (size_t)kCB * (cin + 1) + (size_t)kCB * 10) * sizeof(float);
}

// Geometry of a launch: at most `rows` output rows per batch (-1: the most that fit, 0: the library's choice), workgroups
// spread over `cus` compute units. Returns false when not even one row per batch fits LDS.
inline bool fill_rolling(int n, int cin, int cmid, int h, int w, int stride, int rows, int cus, RollArgs& a) {
    a.n = n; a.cin = cin; a.cmid = cmid; a.h = h; a.w = w; a.stride = stride;
    a.oh = (h + 2 - 3) / stride + 1;
    a.ow = (w + 2 - 3) / stride + 1;
    int r = 0;
    // the library's own choice (rows == 0): the most rows whose ring leaves room for a second workgroup on the compute
    // unit (measured on the MBConv block [96,32,112,112] -> 192 channels, stride 2: 352 us with one row per batch and two
    // workgroups of 8 wavefronts, 402 us with two rows and one workgroup, 508 us for the strips)
    if (rows == 0)
        for (int cand : {8, 4, 2, 1})
            if (!r && rolling_lds_bytes(cand, stride, w, cin) <= 78 * 1024) r = cand;
    for (int cand : {8, 4, 2, 1})
        if (!r && (rows <= 0 || cand <= rows) && rolling_lds_bytes(cand, stride, w, cin) <= 156 * 1024) r = cand;
    if (!r) return false;
    while (r > 1 && r / 2 >= a.oh) r /= 2;
    a.r = r;
    a.ring = 2 * r * stride + 3 - stride;
    a.wp = w + 2;
    a.cblocks = cmid / kCB;
    // segments: each costs one batch of lead-in (its first rows are expanded before any stencil runs) and the halo rows;
    // more segments fill the chip more evenly. Cost in batch slots of the busiest compute unit:
    const int batches = (a.oh + r - 1) / r;
    long long best = -1;
    for (int segs = 1; segs <= batches; segs *= 2) {
        const int per = (batches + segs - 1) / segs;           // batches per segment
        const int used = (batches + per - 1) / per;            // segments that hold rows
        const long long wgs = (long long)n * a.cblocks * used;
        const long long cost = ((wgs + cus - 1) / cus) * (per + 1);
        if (best < 0 || cost < best) {
            best = cost;
            a.seg_rows = per * r;
            a.segs = used;
        }
    }
    a.total = (uint32_t)((long long)n * a.cblocks * a.segs);
    a.magic_w = div_magic(w);
    a.magic_ow = div_magic(a.ow);
    return true;
}

template <int ACT1, int ACT2, int STRIDE, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void expand_depthwise_rolling_kernel(const float* __restrict__ x,
                                                                              const float* __restrict__ we,
                                                                              const float* __restrict__ be,
                                                                              const float* __restrict__ wd,
                                                                              const float* __restrict__ bd,
                                                                              float* __restrict__ y, const RollArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds_f[];
    constexpr int kThreads = WAVES * 64;
    const int cpitch = a.ring * a.wp;                   // one channel's rows
    float* E = lds_f;                                   // [kCB][ring][wp]
    float* WE = lds_f + kCB * cpitch;                   // [kCB][cin + 1]
    const int wep = a.cin + 1;
    float* WD = WE + kCB * wep;                         // [kCB][9 taps + bias]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    // the channel blocks of one image segment read the same rows of X: consecutive workgroup numbers go to different
    // XCDs, so renumber to keep them on one (and in one L2)
    uint32_t bid = blockIdx.x;
    if (a.total % 8u == 0) bid = (bid % 8u) * (a.total / 8u) + bid / 8u;
    const int cb = (int)(bid % (uint32_t)a.cblocks);
    bid /= (uint32_t)a.cblocks;
    const int seg = (int)(bid % (uint32_t)a.segs);
    const int n = (int)(bid / (uint32_t)a.segs);
    const int c0 = cb * kCB;
    const int oy_a = seg * a.seg_rows, oy_b = min(a.oh, oy_a + a.seg_rows);
    const int iy_base = oy_a * STRIDE - 1;              // the row in slot 0

    for (int i = threadIdx.x; i < kCB * a.cin; i += kThreads)
        WE[(i / a.cin) * wep + i % a.cin] = we[(size_t)c0 * a.cin + i];
    for (int i = threadIdx.x; i < kCB * 10; i += kThreads) {
        const int c = i / 10, t = i - c * 10;
        WD[i] = t < 9 ? wd[(size_t)(c0 + c) * 9 + t] : (bd ? bd[c0 + c] : 0.f);
    }
    for (int i = threadIdx.x; i < kCB * a.ring * 2; i += kThreads) {
        const int r = i >> 1;
        E[r * a.wp + ((i & 1) ? a.wp - 1 : 0)] = 0.f;    // left and right padding of every row, never written again
    }
    __syncthreads();

    const int j = lane & 31, hh = lane >> 5;
    const int plane = a.h * a.w;
    const float* xn = x + (size_t)n * a.cin * plane;
    float bias1[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) bias1[e] = 0.f;
    if (be) {
#pragma unroll
        for (int e = 0; e < 16; ++e) bias1[e] = be[c0 + (e >> 2) * 8 + hh * 4 + (e & 3)];
    }
    const int chunks = a.cin / 16;

    // expanded rows lo..hi (image rows; rows outside the image are the stencil's zero padding) by `nw` wavefronts, of
    // which this is number `widx`: tiles of 32 consecutive pixels, 16 input channels per step, kDepth steps in flight
    auto produce = [&](int lo, int hi, int widx, int nw) {
        const int npix = (hi - lo + 1) * a.w;
        const int ntiles = (npix + 31) / 32;
        const int my_tiles = widx < ntiles ? (ntiles - widx + nw - 1) / nw : 0;
        const int steps = my_tiles * chunks;
        const int slot_lo = (lo - iy_base) % a.ring;
        auto pixel_off = [&](int t) -> uint32_t {
            const int p = min(t * 32 + j, npix - 1);
            const int row = div_small(p, a.magic_w);
            return (uint32_t)(hh * plane + min(max(lo + row, 0), a.h - 1) * a.w + (p - row * a.w));
        };
        constexpr int kDepth = 4;
        float ring[kDepth][8];
        int it = widx, ich = 0;
        uint32_t ixo = steps > 0 ? pixel_off(it) : 0u;
        auto issue = [&](float (&dst)[8], int k) {
            if (k >= steps) return;
#pragma unroll
            for (int s = 0; s < 8; ++s) dst[s] = xn[ixo + (uint32_t)((ich * 16 + 2 * s) * plane)];
            if (++ich == chunks) {
                ich = 0;
                it += nw;
                if (k + 1 < steps) ixo = pixel_off(it);
            }
        };
#pragma unroll
        for (int d = 0; d < kDepth; ++d) issue(ring[d], d);
        floatx16 acc;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] = 0.f;
        int ct = widx, cch = 0;
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
                        const int row = div_small(p, a.magic_w);
                        const int iy = lo + row;
                        int slot = slot_lo + row;              // row < ring: one wrap at most
                        if (slot >= a.ring) slot -= a.ring;
                        // rows outside the image hold zeros; as a bit mask, so that the activations stay branch-free
                        const uint32_t keep = iy >= 0 && iy < a.h ? 0xffffffffu : 0u;
                        float* ep = E + slot * a.wp + (p - row * a.w) + 1 + hh * 4 * cpitch;
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            ep[((e >> 2) * 8 + (e & 3)) * cpitch] =
                                __uint_as_float(__float_as_uint(act_f<ACT1>(acc[e] + bias1[e])) & keep);
                    }
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
                    ct += nw;
                }
            }
        }
    };

    // output rows oy0..oy1-1 by `nw` wavefronts: a lane takes one (channel, output column) and moves down the rows,
    // keeping the rows two consecutive outputs share in registers
    auto consume = [&](int oy0, int oy1, int widx, int nw) {
        const int ntask = kCB * a.ow;
        for (int idx = widx * 64 + lane; idx < ntask; idx += nw * 64) {
            const int c = div_small(idx, a.magic_ow);
            const int ocol = idx - c * a.ow;
            float wv[10];
#pragma unroll
            for (int i = 0; i < 10; ++i) wv[i] = WD[c * 10 + i];
            const float* ecol = E + c * cpitch + ocol * STRIDE;
            float* yp = y + (((size_t)n * a.cmid + c0 + c) * a.oh) * a.ow + ocol;
            int slot = (oy0 * STRIDE - 1 - iy_base) % a.ring;
            float win[3][3];
            auto load_row = [&](float (&r)[3]) {
                const float* p = ecol + slot * a.wp;
                r[0] = p[0]; r[1] = p[1]; r[2] = p[2];
                if (++slot == a.ring) slot = 0;
            };
            load_row(win[0]);
            load_row(win[1]);
            load_row(win[2]);
            for (int oy = oy0; oy < oy1; ++oy) {
                float s = wv[9];
#pragma unroll
                for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                    for (int kx = 0; kx < 3; ++kx) s += wv[ky * 3 + kx] * win[ky][kx];
                yp[(size_t)oy * a.ow] = act_f<ACT2>(s);
                if (oy + 1 < oy1) {
                    if constexpr (STRIDE == 1) {
#pragma unroll
                        for (int kx = 0; kx < 3; ++kx) { win[0][kx] = win[1][kx]; win[1][kx] = win[2][kx]; }
                        load_row(win[2]);
                    } else {
#pragma unroll
                        for (int kx = 0; kx < 3; ++kx) win[0][kx] = win[2][kx];
                        load_row(win[1]);
                        load_row(win[2]);
                    }
                }
            }
        }
    };

    const int nb = (oy_b - oy_a + a.r - 1) / a.r;
    auto last_row = [&](int b) { return (min(oy_a + (b + 1) * a.r, oy_b) - 1) * STRIDE + 1; };
    produce(iy_base, last_row(0), wave, WAVES);
    __syncthreads();
    for (int b = 0; b < nb; ++b) {
        const int oy0 = oy_a + b * a.r, oy1 = min(oy0 + a.r, oy_b);
        if (b + 1 < nb) {
            if (wave < WAVES / 2) produce(last_row(b) + 1, last_row(b + 1), wave, WAVES / 2);
            else consume(oy0, oy1, wave - WAVES / 2, WAVES / 2);
        } else {
            consume(oy0, oy1, wave, WAVES);
        }
        __syncthreads();
    }
}

size_t fused_lds_bytes(int toh, int stride, int w, int cin) {
    const int ih = (toh - 1) * stride + 3;
    return ((size_t)kCB * ih * (w + 2) + (size_t)kCB * (cin + 1) + (size_t)kCB * 10) * sizeof(float);
}

thread_local int g_fused_toh = 0;   // diagnostic switch (per calling thread): pin the strip height
thread_local int g_rolling_rows = 0;    // diagnostic switch (per calling thread): 0 = the library's choice, -1 = rolling window
thread_local int g_rolling_waves = 8;   // with the most rows per batch that fit, > 0 = at most that many, -2 = strips;
                                        // wavefronts per workgroup

int compute_units() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (!cached[dev]) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev] = cus;
    }
    return cached[dev];
}

template <int A1, int A2, int STRIDE, int WAVES>
int launch_rolling(const RollArgs& a, const float* x, const float* w_pw, const float* b_pw, const float* w_dw,
                   const float* b_dw, float* y, hipStream_t st) {
    auto kern = expand_depthwise_rolling_kernel<A1, A2, STRIDE, WAVES>;
    const size_t lds = rolling_lds_bytes(a.r, a.stride, a.w, a.cin);
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            set_error("conv2d_expand_depthwise: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
            return (int)e;
        }
    }
    hipLaunchKernelGGL(kern, a.total, WAVES * 64, lds, st, x, w_pw, b_pw, w_dw, b_dw, y, a);
    return launch_status("conv2d_expand_depthwise");
}

template <int A1, int A2>
int launch_rolling_act(const RollArgs& a, int waves, const float* x, const float* w_pw, const float* b_pw,
                       const float* w_dw, const float* b_dw, float* y, hipStream_t st) {
    if (a.stride == 1)
        return waves == 16 ? launch_rolling<A1, A2, 1, 16>(a, x, w_pw, b_pw, w_dw, b_dw, y, st)
                           : launch_rolling<A1, A2, 1, 8>(a, x, w_pw, b_pw, w_dw, b_dw, y, st);
    return waves == 16 ? launch_rolling<A1, A2, 2, 16>(a, x, w_pw, b_pw, w_dw, b_dw, y, st)
                       : launch_rolling<A1, A2, 2, 8>(a, x, w_pw, b_pw, w_dw, b_dw, y, st);
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

void dmlhip_debug_force_fused_strip(int toh) { g_fused_toh = toh; }

void dmlhip_debug_fused_rolling(int rows, int waves) {
    g_rolling_rows = rows;
    g_rolling_waves = waves == 16 ? 16 : 8;
}

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
    hipStream_t st = (hipStream_t)stream;
    RollArgs ra;
    // a pinned strip height asks for the strip kernel
    if (g_rolling_rows != -2 && g_fused_toh <= 0 && fill_rolling((int)pw->n, (int)pw->c, (int)pw->m, (int)pw->h, (int)pw->w, stride,
                                            g_rolling_rows, compute_units(), ra)) {
#define DML_ROLLING_CASE(A1, A2)                                                                                     \
    if (pw->act == A1 && dw->act == A2)                                                                              \
        return launch_rolling_act<A1, A2>(ra, g_rolling_waves, (const float*)x, (const float*)w_pw,                  \
                                          (const float*)b_pw, (const float*)w_dw, (const float*)b_dw, (float*)y, st);
        DML_ROLLING_CASE(DMLHIP_ACT_SWISH, DMLHIP_ACT_SWISH)
        DML_ROLLING_CASE(DMLHIP_ACT_NONE, DMLHIP_ACT_NONE)
        DML_ROLLING_CASE(DMLHIP_ACT_RELU, DMLHIP_ACT_RELU)
        DML_ROLLING_CASE(DMLHIP_ACT_SWISH, DMLHIP_ACT_NONE)
        DML_ROLLING_CASE(DMLHIP_ACT_NONE, DMLHIP_ACT_SWISH)
        DML_ROLLING_CASE(DMLHIP_ACT_RELU, DMLHIP_ACT_NONE)
        DML_ROLLING_CASE(DMLHIP_ACT_NONE, DMLHIP_ACT_RELU)
#undef DML_ROLLING_CASE
    }
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
