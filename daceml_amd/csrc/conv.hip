// ONNX Conv (2-D, NCHW / OIHW, cross-correlation), forward and backward.
//   * 1x1 / stride 1 / no pad / group 1 is a batched GEMM per image, Y[b] = W . X[b], and is
//     handed to the MFMA GEMM with the channel bias and activation in its epilogue;
//   * depthwise (group == C == M) stages the input rows a strip of outputs needs in LDS with
//     coalesced loads and computes the stencil from LDS (HBM-bound: every input byte is read
//     once per strip);
//   * everything else runs a direct kernel, one thread per output, accumulating c, hy, hx
//     sequentially in fp32 — the summation order of the reference's pure expansion.
#include "common.h"
#include "conv_geom.h"

#include <type_traits>

namespace dml {

// conv_backward.hip
bool depthwise_bwd_supported(int k, int s, int p);
int launch_depthwise_bwd_data(const float* dy, const float* w, float* dx, int n, int c, int h, int wd, int oh, int ow, int k,
                              int s, hipStream_t st);
size_t depthwise_bwd_weight_partials(int n, int c, int k);
int launch_depthwise_bwd_weight(const float* x, const float* dy, float* part, int n, int c, int h, int wd, int oh, int ow,
                                int k, int s, int p, hipStream_t st);
int64_t dense_bwd_weight_partials(int n, int c, int m, int kh, int kw, int oh, int ow, int h, int w);
int launch_dense_bwd_weight(const float* x, const float* dy, float* part, int n, int c, int h, int w, int m, int kh, int kw,
                            int sh, int sw, int ph, int pw, int dh, int dw, int oh, int ow, hipStream_t st);
int64_t pointwise_bwd_weight_partials(int n, int m, int c, int64_t hw);
int launch_pointwise_bwd_weight(const float* x, const float* dy, float* part, int n, int m, int c, int64_t hw,
                                hipStream_t st);

// conv_implicit.hip
bool conv_implicit_applicable(const ConvGeom& g);
int launch_conv_implicit_f32(const ConvGeom& g, const float* x, const float* w, const float* bias, float* y, hipStream_t st);
bool conv_implicit_bwd_data_applicable(const ConvGeom& g);
int launch_conv_implicit_bwd_data_f32(const ConvGeom& g, const float* dy, const float* w, float* dx, hipStream_t st);

namespace {

// ---------------------------------------------------------------- direct forward
template <typename T>
__global__ __launch_bounds__(256) void conv_direct_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                          const T* __restrict__ bias, T* __restrict__ y, ConvGeom g,
                                                          int64_t total) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        const int ox = (int)(i % g.ow);
        const int oy = (int)((i / g.ow) % g.oh);
        const int m = (int)((i / ((int64_t)g.ow * g.oh)) % g.m);
        const int b = (int)(i / ((int64_t)g.ow * g.oh * g.m));
        const int grp = m / g.mg;
        float acc = bias ? to_f32(bias[m]) : 0.f;
        for (int c = 0; c < g.cg; ++c) {
            const T* xp = x + ((int64_t)b * g.c + grp * g.cg + c) * g.h * g.w;
            const T* wp = w + ((int64_t)m * g.cg + c) * g.kh * g.kw;
            for (int hy = 0; hy < g.kh; ++hy) {
                const int iy = oy * g.sh - g.ph + hy * g.dh;
                if (iy < 0 || iy >= g.h) continue;
                for (int hx = 0; hx < g.kw; ++hx) {
                    const int ix = ox * g.sw - g.pw + hx * g.dw;
                    if (ix < 0 || ix >= g.w) continue;
                    acc += to_f32(wp[hy * g.kw + hx]) * to_f32(xp[(int64_t)iy * g.w + ix]);
                }
            }
        }
        y[i] = from_f32<T>(apply_act(g.act, acc));
    }
}

// ---------------------------------------------------------------- depthwise forward
// One workgroup per (image, channel, strip of output rows). LDS holds the input rows of the strip with the data
// of a row starting at a 16-byte aligned column (left margin kLeft >= pad, zero-filled like the right margin), so
// the stencil needs no bounds checks along x, global loads are 128-bit when the row length allows, and the
// output loop has no integer divisions: lanes run along x, wavefronts along y.
constexpr int kDwLeft = 4;

__host__ __device__ inline int dw_pitch(int w, int pw) { return ((kDwLeft + w + pw + 3) / 4) * 4; }

template <typename T, int KH, int KW, int ACT>
__device__ __forceinline__ void depthwise_body(const T* __restrict__ x, const T* __restrict__ w, const T* __restrict__ bias,
                                               T* __restrict__ y, const ConvGeom& g, int rows_per_strip, int strips,
                                               float* tile) {
    const int strip = blockIdx.x % strips;
    const int64_t plane = blockIdx.x / strips;  // b * C + c
    const int c = (int)(plane % g.c);
    const int oy0 = strip * rows_per_strip;
    const int oy1 = min(oy0 + rows_per_strip, g.oh);
    const int pitch = dw_pitch(g.w, g.pw);
    const int iy0 = oy0 * g.sh - g.ph;
    const int in_rows = (oy1 - oy0 - 1) * g.sh + (KH - 1) * g.dh + 1;
    const T* xp = x + plane * g.h * g.w;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // margins: kDwLeft columns on the left, the rest of the pitch on the right
    const int right0 = kDwLeft + g.w, margin = kDwLeft + pitch - right0;
    for (int i = threadIdx.x; i < in_rows * margin; i += 256) {
        const int r = i / margin, m = i % margin;
        tile[r * pitch + (m < kDwLeft ? m : right0 + m - kDwLeft)] = 0.f;
    }
    if constexpr (sizeof(T) == 4) {
        if (g.w % 4 == 0 && (reinterpret_cast<uintptr_t>(xp) & 15) == 0) {
            const int vec = g.w / 4;
            for (int i = threadIdx.x; i < in_rows * vec; i += 256) {
                const int r = i / vec, c4 = i % vec;
                const int iy = iy0 + r;
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (iy >= 0 && iy < g.h) v = *reinterpret_cast<const floatx4*>(xp + (int64_t)iy * g.w + c4 * 4);
                *reinterpret_cast<floatx4*>(tile + r * pitch + kDwLeft + c4 * 4) = v;
            }
        } else {
            for (int r = wave; r < in_rows; r += 4) {
                const int iy = iy0 + r;
                for (int col = lane; col < g.w; col += 64)
                    tile[r * pitch + kDwLeft + col] = (iy >= 0 && iy < g.h) ? to_f32(xp[(int64_t)iy * g.w + col]) : 0.f;
            }
        }
    } else {
        for (int r = wave; r < in_rows; r += 4) {
            const int iy = iy0 + r;
            for (int col = lane; col < g.w; col += 64)
                tile[r * pitch + kDwLeft + col] = (iy >= 0 && iy < g.h) ? to_f32(xp[(int64_t)iy * g.w + col]) : 0.f;
        }
    }
    float wr[KH * KW];
#pragma unroll
    for (int i = 0; i < KH * KW; ++i) wr[i] = to_f32(w[(int64_t)c * KH * KW + i]);
    const float bv = bias ? to_f32(bias[c]) : 0.f;
    __syncthreads();
    T* yp = y + plane * g.oh * g.ow;
    for (int oy = wave; oy < oy1 - oy0; oy += 4) {
        for (int ox = lane; ox < g.ow; ox += 64) {
            const float* tp = tile + (oy * g.sh) * pitch + kDwLeft - g.pw + ox * g.sw;
            float acc = bv;
#pragma unroll
            for (int hy = 0; hy < KH; ++hy)
#pragma unroll
                for (int hx = 0; hx < KW; ++hx) acc += wr[hy * KW + hx] * tp[hy * g.dh * pitch + hx * g.dw];
            yp[(int64_t)(oy0 + oy) * g.ow + ox] = from_f32<T>(apply_act(ACT, acc));
        }
    }
}

template <typename T, int KH, int KW>
__global__ __launch_bounds__(256) void conv_depthwise_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                             const T* __restrict__ bias, T* __restrict__ y, ConvGeom g,
                                                             int rows_per_strip, int strips) {
    extern __shared__ float tile[];  // [in_rows][pitch]
    switch (g.act) {  // the activation is selected once per workgroup, not once per output
        case DMLHIP_ACT_SWISH: depthwise_body<T, KH, KW, DMLHIP_ACT_SWISH>(x, w, bias, y, g, rows_per_strip, strips, tile); break;
        case DMLHIP_ACT_SIGMOID: depthwise_body<T, KH, KW, DMLHIP_ACT_SIGMOID>(x, w, bias, y, g, rows_per_strip, strips, tile); break;
        case DMLHIP_ACT_RELU: depthwise_body<T, KH, KW, DMLHIP_ACT_RELU>(x, w, bias, y, g, rows_per_strip, strips, tile); break;
        case DMLHIP_ACT_GELU: depthwise_body<T, KH, KW, DMLHIP_ACT_GELU>(x, w, bias, y, g, rows_per_strip, strips, tile); break;
        default: depthwise_body<T, KH, KW, DMLHIP_ACT_NONE>(x, w, bias, y, g, rows_per_strip, strips, tile); break;
    }
}

// ---------------------------------------------------------------- direct backward
// dX[b,c,iy,ix] = sum_{m in group, hy, hx : iy = oy*sh - ph + hy*dh, ...} W[m,c',hy,hx] * dY[b,m,oy,ox]
__global__ __launch_bounds__(256) void conv_bwd_data_kernel(const float* __restrict__ dy, const float* __restrict__ w,
                                                            float* __restrict__ dx, ConvGeom g, int64_t total) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        const int ix = (int)(i % g.w);
        const int iy = (int)((i / g.w) % g.h);
        const int c = (int)((i / ((int64_t)g.w * g.h)) % g.c);
        const int b = (int)(i / ((int64_t)g.w * g.h * g.c));
        const int grp = c / g.cg, cc = c % g.cg;
        float acc = 0.f;
        for (int mm = 0; mm < g.mg; ++mm) {
            const int m = grp * g.mg + mm;
            const float* gp = dy + ((int64_t)b * g.m + m) * g.oh * g.ow;
            const float* wp = w + ((int64_t)m * g.cg + cc) * g.kh * g.kw;
            for (int hy = 0; hy < g.kh; ++hy) {
                const int ty = iy + g.ph - hy * g.dh;
                if (ty < 0 || ty % g.sh) continue;
                const int oy = ty / g.sh;
                if (oy >= g.oh) continue;
                for (int hx = 0; hx < g.kw; ++hx) {
                    const int tx = ix + g.pw - hx * g.dw;
                    if (tx < 0 || tx % g.sw) continue;
                    const int ox = tx / g.sw;
                    if (ox >= g.ow) continue;
                    acc += wp[hy * g.kw + hx] * gp[(int64_t)oy * g.ow + ox];
                }
            }
        }
        dx[i] = acc;
    }
}

// dW[m,c',hy,hx] = sum_{b,oy,ox} dY[b,m,oy,ox] * X[b, grp*cg+c', oy*sh-ph+hy*dh, ox*sw-pw+hx*dw];
// one workgroup per weight element.
__global__ __launch_bounds__(256) void conv_bwd_weight_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                              float* __restrict__ dw, ConvGeom g) {
    __shared__ float scratch[4];
    int64_t i = blockIdx.x;
    const int hx = (int)(i % g.kw); i /= g.kw;
    const int hy = (int)(i % g.kh); i /= g.kh;
    const int cc = (int)(i % g.cg); i /= g.cg;
    const int m = (int)i;
    const int c = (m / g.mg) * g.cg + cc;
    const int64_t per_img = (int64_t)g.oh * g.ow;
    float acc = 0.f;
    for (int64_t j = threadIdx.x; j < per_img * g.n; j += 256) {
        const int b = (int)(j / per_img);
        const int r = (int)(j % per_img);
        const int oy = r / g.ow, ox = r % g.ow;
        const int iy = oy * g.sh - g.ph + hy * g.dh, ix = ox * g.sw - g.pw + hx * g.dw;
        if (iy < 0 || iy >= g.h || ix < 0 || ix >= g.w) continue;
        acc += dy[((int64_t)b * g.m + m) * per_img + r] * x[(((int64_t)b * g.c + c) * g.h + iy) * g.w + ix];
    }
    acc = block_reduce<OpSum, 4>(acc, scratch);
    if (threadIdx.x == 0) dw[blockIdx.x] = acc;
}


// ---------------------------------------------------------------- pointwise (1x1) convolution, fp32
// Y[n, m, p] = act(sum_c W[m, c] * s[n, c] * X[n, c, p] + b[m]) with p running over the h*w pixels: per image a
// GEMM with a short K (the input channels) and a very long, contiguous N. It is bound by the output write, so the
// kernel is organised around reading X exactly once and writing Y in full 128-byte rows: a workgroup takes 256
// pixels of one image and up to 192 output channels; X goes through LDS in chunks of 32 channels, W chunk by chunk
// as well; every wavefront multiplies all output channels with its 64 pixels on v_mfma_f32_32x32x2f32 (true fp32).
// A = W (rows = output channels), B = X (columns = pixels): a lane's accumulators are 16 output channels of ONE
// pixel, so stores of a wavefront run along the pixels. `in_scale` (optional) is a per-image, per-input-channel
// factor applied to X on its way into LDS (the squeeze-excite gate in front of a projection).
// WT: the weights are given transposed, as [cin][cout] (the data gradient of a pointwise convolution is a pointwise
// convolution of dY with W^T); cin may then be any positive number, the last chunk is zero-filled.
template <int MT, int PT, bool WT>  // 32-channel blocks per workgroup; 32-pixel blocks per wavefront
__global__ __launch_bounds__(256, 2) void conv_pointwise_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                    const float* __restrict__ bias,
                                                                    const float* __restrict__ in_scale, float* __restrict__ y,
                                                                    int cin, int cout, int64_t hw, int act) {
    constexpr int PX = 128 * PT, KC = 32, XP = PX + 32, WP = KC + 1;
    extern __shared__ float pw_lds[];
    float* xs = pw_lds;                 // [KC][XP]   pitch: rows k and k+1 land in different bank halves
    float* ws = xs + KC * XP;           // [MT*32][WP]
    float* bs = ws + MT * 32 * WP;      // [MT*32]
    const int n = blockIdx.y;
    const int64_t p0 = (int64_t)blockIdx.x * PX;
    const int m0 = blockIdx.z * MT * 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int pwv = wave * 32 * PT;

    floatx16 acc[MT][PT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < PT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    if (threadIdx.x < MT * 32) bs[threadIdx.x] = (bias && m0 + (int)threadIdx.x < cout) ? bias[m0 + threadIdx.x] : 0.f;
    const float* xn = x + (int64_t)n * cin * hw;
    for (int kc = 0; kc < cin; kc += KC) {
        __syncthreads();  // the previous chunk has been consumed
        // all loads of the chunk are issued before the first one is used (branch-free: out-of-range pixels read
        // a clamped address and are zeroed afterwards), so the chunk costs one memory round trip, not eight
        constexpr int XL = KC * (PX / 4) / 256, WL = (MT * 32 * (KC / 4) + 255) / 256, WS = MT * 32 * KC / 256;
        floatx4 xv[XL], wv[WT ? 1 : WL];
        float wt[WT ? WS : 1];
#pragma unroll
        for (int r = 0; r < XL; ++r) {
            const int idx = r * 256 + threadIdx.x, row = idx / (PX / 4), c4 = idx % (PX / 4);
            const int64_t p = p0 + c4 * 4 < hw ? p0 + c4 * 4 : hw - 4;
            xv[r] = *reinterpret_cast<const floatx4*>(xn + (int64_t)min(kc + row, cin - 1) * hw + p);
        }
        if constexpr (WT) {
#pragma unroll
            for (int r = 0; r < WS; ++r) {
                const int idx = r * 256 + threadIdx.x, col = idx / (MT * 32), row = idx % (MT * 32);
                wt[r] = w[(int64_t)min(kc + col, cin - 1) * cout + min(m0 + row, cout - 1)];
            }
        } else {
#pragma unroll
            for (int r = 0; r < WL; ++r) {
                const int idx = r * 256 + threadIdx.x, row = min(idx / (KC / 4), MT * 32 - 1), c4 = idx % (KC / 4);
                wv[r] = *reinterpret_cast<const floatx4*>(w + (int64_t)min(m0 + row, cout - 1) * cin + kc + c4 * 4);
            }
        }
#pragma unroll
        for (int r = 0; r < XL; ++r) {
            const int idx = r * 256 + threadIdx.x, row = idx / (PX / 4), c4 = idx % (PX / 4);
            floatx4 v = xv[r];
            if (in_scale) v *= in_scale[(int64_t)n * cin + min(kc + row, cin - 1)];
            if (!(p0 + c4 * 4 < hw) || kc + row >= cin) v = floatx4{0.f, 0.f, 0.f, 0.f};
            *reinterpret_cast<floatx4*>(xs + row * XP + c4 * 4) = v;
        }
        if constexpr (WT) {
#pragma unroll
            for (int r = 0; r < WS; ++r) {
                const int idx = r * 256 + threadIdx.x, col = idx / (MT * 32), row = idx % (MT * 32);
                ws[row * WP + col] = (kc + col < cin && m0 + row < cout) ? wt[r] : 0.f;
            }
        } else {
#pragma unroll
            for (int r = 0; r < WL; ++r) {
                const int idx = r * 256 + threadIdx.x, row = idx / (KC / 4), c4 = idx % (KC / 4);
                if (idx < MT * 32 * (KC / 4)) {
                    const bool ok = m0 + row < cout;
#pragma unroll
                    for (int e = 0; e < 4; ++e) ws[row * WP + c4 * 4 + e] = ok ? wv[r][e] : 0.f;
                }
            }
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < KC / 2; ++kk) {
            float b[PT];
#pragma unroll
            for (int j = 0; j < PT; ++j) b[j] = xs[(2 * kk + h) * XP + pwv + j * 32 + l32];
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const float a = ws[(i * 32 + l32) * WP + 2 * kk + h];
#pragma unroll
                for (int j = 0; j < PT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    float* yn = y + (int64_t)n * cout * hw;
    // the activation is selected once, outside the 32*MT stores of a lane
    auto store_all = [&](auto actc) {
        constexpr int ACT = decltype(actc)::value;
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < PT; ++j) {
                const int64_t p = p0 + pwv + j * 32 + l32;
                if (p >= hw) continue;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int ml = i * 32 + (e >> 2) * 8 + h * 4 + (e & 3);
                    if (m0 + ml < cout) yn[(int64_t)(m0 + ml) * hw + p] = apply_act(ACT, acc[i][j][e] + bs[ml]);
                }
            }
    };
    switch (act) {
        case DMLHIP_ACT_GELU: store_all(std::integral_constant<int, DMLHIP_ACT_GELU>{}); break;
        case DMLHIP_ACT_SWISH: store_all(std::integral_constant<int, DMLHIP_ACT_SWISH>{}); break;
        case DMLHIP_ACT_SIGMOID: store_all(std::integral_constant<int, DMLHIP_ACT_SIGMOID>{}); break;
        case DMLHIP_ACT_RELU: store_all(std::integral_constant<int, DMLHIP_ACT_RELU>{}); break;
        default: store_all(std::integral_constant<int, DMLHIP_ACT_NONE>{}); break;
    }
}

// Squeeze-excite sized products ([n, c, 1, 1] inputs): Y[n, m] = act(b[m] + sum_c X[n, c] W[m, c]). A few hundred
// outputs with a short dot product each: one wavefront per output, lanes along c, so the whole product is one
// memory round trip plus a wavefront reduction instead of a tiled GEMM's chain of synchronised K steps.
template <typename T>
__global__ __launch_bounds__(256) void conv_1x1_spatial1_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                                const T* __restrict__ bias, T* __restrict__ y, int n, int c,
                                                                int m, int act) {
    const int lane = threadIdx.x & 63;
    const int64_t o = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (o >= (int64_t)n * m) return;
    const int in = (int)(o / m), im = (int)(o % m);
    const T* xr = x + (int64_t)in * c;
    const T* wr = w + (int64_t)im * c;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int k = lane;
    for (; k + 192 < c; k += 256) {
        a0 += to_f32(xr[k]) * to_f32(wr[k]);
        a1 += to_f32(xr[k + 64]) * to_f32(wr[k + 64]);
        a2 += to_f32(xr[k + 128]) * to_f32(wr[k + 128]);
        a3 += to_f32(xr[k + 192]) * to_f32(wr[k + 192]);
    }
    for (; k < c; k += 64) a0 += to_f32(xr[k]) * to_f32(wr[k]);
    const float s = wave_reduce<OpSum>((a0 + a1) + (a2 + a3));
    if (lane == 0) y[o] = from_f32<T>(apply_act(act, s + (bias ? to_f32(bias[im]) : 0.f)));
}

// Gradients of those squeeze-excite sized products. One thread per output, a short loop, coalesced along the
// output's fast index: dX[n, c] = sum_m dY[n, m] W[m, c] and dW[m, c] = sum_n dY[n, m] X[n, c].
__global__ __launch_bounds__(256) void conv_1x1_spatial1_bwd_data_kernel(const float* __restrict__ dy,
                                                                         const float* __restrict__ w, float* __restrict__ dx,
                                                                         int n, int c, int m) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= (int64_t)n * c) return;
    const int in = (int)(o / c), ic = (int)(o % c);
    const float* g = dy + (int64_t)in * m;
    // four running sums: independent chains for the loads, and a shorter chain of roundings for the result
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int k = 0;
    for (; k + 3 < m; k += 4) {
        a0 += g[k] * w[(int64_t)k * c + ic];
        a1 += g[k + 1] * w[(int64_t)(k + 1) * c + ic];
        a2 += g[k + 2] * w[(int64_t)(k + 2) * c + ic];
        a3 += g[k + 3] * w[(int64_t)(k + 3) * c + ic];
    }
    for (; k < m; ++k) a0 += g[k] * w[(int64_t)k * c + ic];
    dx[o] = (a0 + a1) + (a2 + a3);
}

__global__ __launch_bounds__(256) void conv_1x1_spatial1_bwd_weight_kernel(const float* __restrict__ x,
                                                                           const float* __restrict__ dy,
                                                                           float* __restrict__ dw, int n, int c, int m) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= (int64_t)m * c) return;
    const int im = (int)(o / c), ic = (int)(o % c);
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    int b = 0;
    for (; b + 3 < n; b += 4) {
        a0 += dy[(int64_t)b * m + im] * x[(int64_t)b * c + ic];
        a1 += dy[(int64_t)(b + 1) * m + im] * x[(int64_t)(b + 1) * c + ic];
        a2 += dy[(int64_t)(b + 2) * m + im] * x[(int64_t)(b + 2) * c + ic];
        a3 += dy[(int64_t)(b + 3) * m + im] * x[(int64_t)(b + 3) * c + ic];
    }
    for (; b < n; ++b) a0 += dy[(int64_t)b * m + im] * x[(int64_t)b * c + ic];
    dw[o] = (a0 + a1) + (a2 + a3);
}

int launch_pointwise_f32(const float* x, const float* w, const float* bias, const float* in_scale, float* y, int n, int cin,
                         int cout, int64_t hw, int act, hipStream_t st, bool w_transposed = false) {
    int mt = (int)ceil_div(cout, 32);
    if (mt > 6) mt = 6;
    // many output channels: 32 pixels per wavefront keep the accumulators (16 registers per 32x32 block) and the
    // load registers within what two resident workgroups per CU may use
    const int pt = mt >= 5 ? 1 : 2;
    const dim3 grid((unsigned)ceil_div(hw, 128 * pt), (unsigned)n, (unsigned)ceil_div(cout, mt * 32));
    const size_t lds = (size_t)(32 * (128 * pt + 32) + mt * 32 * 33 + mt * 32) * sizeof(float);
#define DML_PW(MT, PT)                                                                                                 \
    case MT:                                                                                                           \
        if (w_transposed)                                                                                              \
            hipLaunchKernelGGL((conv_pointwise_f32_kernel<MT, PT, true>), grid, 256, lds, st, x, w, bias, in_scale, y, \
                               cin, cout, hw, act);                                                                    \
        else                                                                                                           \
            hipLaunchKernelGGL((conv_pointwise_f32_kernel<MT, PT, false>), grid, 256, lds, st, x, w, bias, in_scale, y, \
                               cin, cout, hw, act);                                                                    \
        break
    switch (mt) {
        DML_PW(1, 2); DML_PW(2, 2); DML_PW(3, 2); DML_PW(4, 2); DML_PW(5, 1);
        default: DML_PW(6, 1);
    }
#undef DML_PW
    return launch_status("conv2d(pointwise)");
}

// ---------------------------------------------------------------- host side
int make_geom(const dmlhip_conv2d_desc* d, ConvGeom* g, const char* what) {
    DML_REQUIRE(d, DMLHIP_ERR_NULL, "%s: NULL descriptor", what);
    DML_REQUIRE(d->n >= 0 && d->c >= 0 && d->h >= 0 && d->w >= 0 && d->m >= 0, DMLHIP_ERR_SHAPE,
                "%s: negative tensor extent", what);
    DML_REQUIRE(d->kh >= 1 && d->kw >= 1 && d->stride_h >= 1 && d->stride_w >= 1 && d->dil_h >= 1 && d->dil_w >= 1 &&
                    d->pad_h >= 0 && d->pad_w >= 0 && d->group >= 1,
                DMLHIP_ERR_SHAPE, "%s: kernel/stride/dilation/group must be >= 1 and pads >= 0", what);
    DML_REQUIRE(d->c % d->group == 0 && d->m % d->group == 0, DMLHIP_ERR_SHAPE,
                "%s: channels (%lld in, %lld out) not divisible by group %lld", what, (long long)d->c, (long long)d->m,
                (long long)d->group);
    const int64_t lim = 1 << 30;
    DML_REQUIRE(d->n < lim && d->c < lim && d->h < lim && d->w < lim && d->m < lim && d->kh < lim && d->kw < lim &&
                    d->stride_h < lim && d->stride_w < lim && d->pad_h < lim && d->pad_w < lim && d->dil_h < lim &&
                    d->dil_w < lim,
                DMLHIP_ERR_SHAPE, "%s: extent exceeds 2^30", what);
    DML_REQUIRE(valid_act(d->act), DMLHIP_ERR_ENUM, "%s: bad act", what);
    const int64_t eh = (d->kh - 1) * d->dil_h + 1, ew = (d->kw - 1) * d->dil_w + 1;
    const int64_t oh = d->h + 2 * d->pad_h >= eh ? (d->h + 2 * d->pad_h - eh) / d->stride_h + 1 : 0;
    const int64_t ow = d->w + 2 * d->pad_w >= ew ? (d->w + 2 * d->pad_w - ew) / d->stride_w + 1 : 0;
    DML_REQUIRE((double)d->n * d->m * oh * ow < 9e18 / 16 && (double)d->n * d->c * d->h * d->w < 9e18 / 16,
                DMLHIP_ERR_SHAPE, "%s: tensor size overflows", what);
    g->n = (int)d->n; g->c = (int)d->c; g->h = (int)d->h; g->w = (int)d->w; g->m = (int)d->m;
    g->kh = (int)d->kh; g->kw = (int)d->kw; g->sh = (int)d->stride_h; g->sw = (int)d->stride_w;
    g->ph = (int)d->pad_h; g->pw = (int)d->pad_w; g->dh = (int)d->dil_h; g->dw = (int)d->dil_w;
    g->group = (int)d->group; g->oh = (int)oh; g->ow = (int)ow;
    g->cg = g->c / g->group; g->mg = g->m / g->group; g->act = d->act;
    return 0;
}

inline bool is_pointwise(const ConvGeom& g) {
    return g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && g.group == 1;
}

// depthwise with a stencil, stride and "same" padding the gradient kernels are built for
inline bool is_depthwise_grad(const ConvGeom& g) {
    return g.group == g.c && g.m == g.c && g.c > 0 && g.kh == g.kw && g.sh == g.sw && g.ph == g.pw && g.dh == 1 &&
           g.dw == 1 && depthwise_bwd_supported(g.kh, g.sh, g.ph) && g.oh > 0 && g.ow > 0;
}

inline unsigned grid_for(int64_t total) {
    int64_t gsz = ceil_div(total, 256);
    if (gsz > 256 * 64) gsz = 256 * 64;
    return (unsigned)(gsz < 1 ? 1 : gsz);
}

template <typename T>
int conv_forward(const dmlhip_conv2d_desc* d, const void* x, const void* w, const void* bias, void* y, void* stream) {
    ConvGeom g;
    if (int e = make_geom(d, &g, "conv2d")) return e;
    const int64_t total = (int64_t)g.n * g.m * g.oh * g.ow;
    if (total == 0) return 0;
    DML_REQUIRE(y && w && (x || g.c == 0), DMLHIP_ERR_NULL, "conv2d: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;

    // 1x1, stride 1, no pad, group 1: Y[b] (M x HW) = W (M x C) . X[b] (C x HW)
    if (g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && g.group == 1 && g.c > 0) {
        const int64_t hw = (int64_t)g.h * g.w;
        if constexpr (sizeof(T) == 4) {
            // many pixels, few channels: the streaming kernel (reads X once, writes Y in full rows)
            if (g.c % 32 == 0 && hw % 4 == 0 && hw >= 128 && g.n <= 65535 && aligned16(x) && aligned16(w))
                return launch_pointwise_f32((const float*)x, (const float*)w, (const float*)bias, nullptr, (float*)y, g.n,
                                            g.c, g.m, hw, g.act, st);
        }
        dmlhip_gemm_desc gd = {};
        if (hw == 1 && (int64_t)g.n * g.m <= (1 << 22)) {
            hipLaunchKernelGGL((conv_1x1_spatial1_kernel<T>), (unsigned)ceil_div((int64_t)g.n * g.m, 4), 256, 0, st,
                               (const T*)x, (const T*)w, (const T*)bias, (T*)y, g.n, g.c, g.m, g.act);
            return launch_status("conv2d(1x1 on 1x1)");
        }
        gd.m = g.m; gd.n = hw; gd.k = g.c;
        gd.batch[0] = 1; gd.batch[1] = 1; gd.batch[2] = g.n;
        gd.a_stride_m = g.c; gd.a_stride_k = 1;
        gd.b_stride_k = hw; gd.b_stride_n = 1; gd.b_stride_batch[2] = (int64_t)g.c * hw;
        gd.c_stride_m = hw; gd.c_stride_batch[2] = (int64_t)g.m * hw;
        gd.alpha = 1.f; gd.beta = 0.f;
        gd.out_dtype = sizeof(T) == 2 ? DMLHIP_F16 : DMLHIP_F32;
        gd.bias_dtype = gd.out_dtype;
        gd.act = g.act;
        gd.bias_along_m = 1;
        return sizeof(T) == 2 ? dmlhip_gemm_f16(&gd, w, x, y, bias, nullptr, nullptr, stream)
                              : dmlhip_gemm_f32(&gd, w, x, y, bias, nullptr, nullptr, stream);
    }
    // depthwise with a small square-ish stencil
    if (g.group == g.c && g.m == g.c && ((g.kh == 3 && g.kw == 3) || (g.kh == 5 && g.kw == 5))) {
        if (g.pw > kDwLeft) goto direct;
        const int wp = dw_pitch(g.w, g.pw);
        // rows per strip: keep the LDS tile under 32 KiB so several workgroups share a CU
        int rows = g.oh;
        while (rows > 1 && (size_t)((rows - 1) * g.sh + (g.kh - 1) * g.dh + 1) * wp * sizeof(float) > 32 * 1024)
            rows = (rows + 1) / 2;
        const size_t lds = (size_t)((rows - 1) * g.sh + (g.kh - 1) * g.dh + 1) * wp * sizeof(float);
        if (lds <= 64 * 1024) {
            const int strips = (g.oh + rows - 1) / rows;
            const int64_t blocks = (int64_t)g.n * g.c * strips;
            DML_REQUIRE(blocks <= 2147483647LL, DMLHIP_ERR_SHAPE, "conv2d: too many depthwise strips");
            if (g.kh == 3)
                hipLaunchKernelGGL((conv_depthwise_kernel<T, 3, 3>), (unsigned)blocks, 256, lds, st, (const T*)x,
                                   (const T*)w, (const T*)bias, (T*)y, g, rows, strips);
            else
                hipLaunchKernelGGL((conv_depthwise_kernel<T, 5, 5>), (unsigned)blocks, 256, lds, st, (const T*)x,
                                   (const T*)w, (const T*)bias, (T*)y, g, rows, strips);
            return launch_status("conv2d(depthwise)");
        }
    }
direct:
    if constexpr (sizeof(T) == 4) {
        // dense convolutions with enough work per output: implicit GEMM on the fp32 matrix pipe
        if (conv_implicit_applicable(g))
            return launch_conv_implicit_f32(g, (const float*)x, (const float*)w, (const float*)bias, (float*)y, st);
    }
    hipLaunchKernelGGL((conv_direct_kernel<T>), grid_for(total), 256, 0, st, (const T*)x, (const T*)w, (const T*)bias,
                       (T*)y, g, total);
    return launch_status("conv2d(direct)");
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

int dmlhip_conv2d_out_shape(const dmlhip_conv2d_desc* d, int64_t* oh, int64_t* ow) {
    ConvGeom g;
    if (int e = make_geom(d, &g, "conv2d_out_shape")) return e;
    DML_REQUIRE(oh && ow, DMLHIP_ERR_NULL, "conv2d_out_shape: NULL output pointer");
    *oh = g.oh;
    *ow = g.ow;
    return 0;
}

int dmlhip_conv2d_f32(const dmlhip_conv2d_desc* d, const void* x, const void* w, const void* bias, void* y,
                      void* stream) {
    return conv_forward<float>(d, x, w, bias, y, stream);
}

int dmlhip_conv2d_gated_f32(const dmlhip_conv2d_desc* d, const void* x, const void* gate, const void* w, const void* bias,
                            void* y, void* stream) {
    ConvGeom g;
    if (int e = make_geom(d, &g, "conv2d_gated")) return e;
    const int64_t hw = (int64_t)g.h * g.w;
    DML_REQUIRE(g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && g.group == 1,
                DMLHIP_ERR_UNSUPPORTED, "conv2d_gated: only 1x1, stride 1, no padding, group 1");
    DML_REQUIRE(g.c > 0 && g.c % 32 == 0 && hw % 4 == 0 && hw >= 128 && g.n <= 65535, DMLHIP_ERR_UNSUPPORTED,
                "conv2d_gated: needs channels %% 32 == 0, h*w %% 4 == 0, h*w >= 128, n <= 65535");
    if ((int64_t)g.n * g.m == 0) return 0;
    DML_REQUIRE(x && gate && w && y, DMLHIP_ERR_NULL, "conv2d_gated: NULL tensor pointer");
    DML_REQUIRE(aligned16(x) && aligned16(w), DMLHIP_ERR_ALIGN, "conv2d_gated: x and w must be 16-byte aligned");
    return launch_pointwise_f32((const float*)x, (const float*)w, (const float*)bias, (const float*)gate, (float*)y, g.n, g.c,
                                g.m, hw, g.act, (hipStream_t)stream);
}

int dmlhip_conv2d_f16(const dmlhip_conv2d_desc* d, const void* x, const void* w, const void* bias, void* y,
                      void* stream) {
    return conv_forward<_Float16>(d, x, w, bias, y, stream);
}

int dmlhip_conv2d_backward_data_f32(const dmlhip_conv2d_desc* d, const void* dy, const void* w, void* dx,
                                    void* stream) {
    ConvGeom g;
    if (int e = make_geom(d, &g, "conv2d_backward_data")) return e;
    const int64_t total = (int64_t)g.n * g.c * g.h * g.w;
    if (total == 0) return 0;
    DML_REQUIRE(dx && w && (dy || (int64_t)g.oh * g.ow * g.m == 0), DMLHIP_ERR_NULL,
                "conv2d_backward_data: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    if (g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && g.group == 1 && g.m > 0) {
        // dX[b] (C x HW) = W^T (C x M) . dY[b] (M x HW)
        const int64_t hw = (int64_t)g.h * g.w;
        if (hw == 1 && (int64_t)g.n * g.c <= (1 << 22)) {
            hipLaunchKernelGGL(conv_1x1_spatial1_bwd_data_kernel, (unsigned)ceil_div((int64_t)g.n * g.c, 256), 256, 0, st,
                               (const float*)dy, (const float*)w, (float*)dx, g.n, g.c, g.m);
            return launch_status("conv2d_backward_data(1x1 on 1x1)");
        }
        // many pixels: the streaming pointwise kernel with dY as its input and W read as [cin = M][cout = C]
        if (hw % 4 == 0 && hw >= 128 && g.n <= 65535 && aligned16(dy) && aligned16(dx))
            return launch_pointwise_f32((const float*)dy, (const float*)w, nullptr, nullptr, (float*)dx, g.n, g.m, g.c, hw,
                                        DMLHIP_ACT_NONE, st, true);
        dmlhip_gemm_desc gd = {};
        gd.m = g.c; gd.n = hw; gd.k = g.m;
        gd.batch[0] = 1; gd.batch[1] = 1; gd.batch[2] = g.n;
        gd.a_stride_m = 1; gd.a_stride_k = g.c;
        gd.b_stride_k = hw; gd.b_stride_n = 1; gd.b_stride_batch[2] = (int64_t)g.m * hw;
        gd.c_stride_m = hw; gd.c_stride_batch[2] = (int64_t)g.c * hw;
        gd.alpha = 1.f; gd.out_dtype = DMLHIP_F32; gd.bias_dtype = DMLHIP_F32;
        return dmlhip_gemm_f32(&gd, w, dy, dx, nullptr, nullptr, nullptr, stream);
    }
    if (is_depthwise_grad(g))
        return launch_depthwise_bwd_data((const float*)dy, (const float*)w, (float*)dx, g.n, g.c, g.h, g.w, g.oh, g.ow, g.kh,
                                         g.sh, st);
    if (conv_implicit_bwd_data_applicable(g))
        return launch_conv_implicit_bwd_data_f32(g, (const float*)dy, (const float*)w, (float*)dx, st);
    hipLaunchKernelGGL(conv_bwd_data_kernel, grid_for(total), 256, 0, st, (const float*)dy, (const float*)w, (float*)dx,
                       g, total);
    return launch_status("conv2d_backward_data");
}

size_t dmlhip_conv2d_backward_weight_workspace_bytes(const dmlhip_conv2d_desc* d) {
    ConvGeom g;
    if (make_geom(d, &g, "conv2d_backward_weight")) return 0;
    if (is_pointwise(g) && (int64_t)g.h * g.w == 1 && (int64_t)g.m * g.c <= (1 << 22)) return 0;   // one small kernel
    if (is_pointwise(g) && g.n >= 1) {
        // the larger of what the two paths need: per-workgroup results of the streaming kernel, or per-image
        // products of the batched GEMM (taken when the streaming kernel does not apply or an operand is unaligned)
        const int64_t mc = (int64_t)g.m * g.c;
        size_t need = g.n > 1 ? (size_t)g.n * mc * sizeof(float) + dmlhip_reduce_workspace_bytes(1, g.n, mc) : 0;
        const int64_t parts = pointwise_bwd_weight_partials(g.n, g.m, g.c, (int64_t)g.h * g.w);
        if (parts > 1) {
            const size_t streaming = (size_t)parts * mc * sizeof(float) + dmlhip_reduce_workspace_bytes(1, parts, mc);
            if (streaming > need) need = streaming;
        }
        return need;
    }
    if (is_depthwise_grad(g) && g.n > 1) {
        const int64_t per = (int64_t)g.c * g.kh * g.kw;
        return (size_t)g.n * per * sizeof(float) + dmlhip_reduce_workspace_bytes(1, g.n, per);
    }
    if (g.group == 1) {
        const int64_t parts = dense_bwd_weight_partials(g.n, g.c, g.m, g.kh, g.kw, g.oh, g.ow, g.h, g.w);
        const int64_t per = (int64_t)g.m * g.c * g.kh * g.kw;
        if (parts > 1) return (size_t)parts * per * sizeof(float) + dmlhip_reduce_workspace_bytes(1, parts, per);
    }
    return 0;
}

int dmlhip_conv2d_backward_weight_f32(const dmlhip_conv2d_desc* d, const void* x, const void* dy, void* dw,
                                      void* workspace, size_t workspace_bytes, void* stream) {
    ConvGeom g;
    if (int e = make_geom(d, &g, "conv2d_backward_weight")) return e;
    const int64_t total = (int64_t)g.m * g.cg * g.kh * g.kw;
    if (total == 0) return 0;
    DML_REQUIRE(dw, DMLHIP_ERR_NULL, "conv2d_backward_weight: NULL output");
    const int64_t red = (int64_t)g.n * g.oh * g.ow;
    DML_REQUIRE(red == 0 || (x && dy), DMLHIP_ERR_NULL, "conv2d_backward_weight: NULL tensor pointer");
    DML_REQUIRE(total <= 2147483647LL, DMLHIP_ERR_SHAPE, "conv2d_backward_weight: too many weights");
    hipStream_t st = (hipStream_t)stream;
    const int64_t dense_parts =
        (!is_pointwise(g) && g.group == 1 && red > 0)
            ? dense_bwd_weight_partials(g.n, g.c, g.m, g.kh, g.kw, g.oh, g.ow, g.h, g.w) : 0;
    if ((is_pointwise(g) || is_depthwise_grad(g) || dense_parts > 0) && red > 0) {
        const size_t need = dmlhip_conv2d_backward_weight_workspace_bytes(d);
        DML_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), DMLHIP_ERR_WORKSPACE,
                    "conv2d_backward_weight: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    }
    if (is_depthwise_grad(g) && red > 0) {
        // one result per (image, channel) plane, summed over the images in a fixed order
        const int64_t per = (int64_t)g.c * g.kh * g.kw;
        float* part = g.n > 1 ? (float*)workspace : (float*)dw;
        if (int e = launch_depthwise_bwd_weight((const float*)x, (const float*)dy, part, g.n, g.c, g.h, g.w, g.oh, g.ow,
                                                g.kh, g.sh, g.ph, st))
            return e;
        if (g.n == 1) return 0;
        const size_t part_bytes = (size_t)g.n * per * sizeof(float);
        return dmlhip_reduce_f32(DMLHIP_RSUM, part, dw, DMLHIP_F32, 1, g.n, per, (char*)workspace + part_bytes,
                                 workspace_bytes - part_bytes, stream);
    }
    if (dense_parts > 0) {
        // implicit GEMM over ranges of the (image, pixel) space, then their sum in a fixed order
        float* part = dense_parts > 1 ? (float*)workspace : (float*)dw;
        if (int e = launch_dense_bwd_weight((const float*)x, (const float*)dy, part, g.n, g.c, g.h, g.w, g.m, g.kh, g.kw,
                                            g.sh, g.sw, g.ph, g.pw, g.dh, g.dw, g.oh, g.ow, st))
            return e;
        if (dense_parts == 1) return 0;
        const size_t part_bytes = (size_t)dense_parts * total * sizeof(float);
        return dmlhip_reduce_f32(DMLHIP_RSUM, part, dw, DMLHIP_F32, 1, dense_parts, total, (char*)workspace + part_bytes,
                                 workspace_bytes - part_bytes, stream);
    }
    if (is_pointwise(g) && red > 0 && (int64_t)g.h * g.w == 1 && total <= (1 << 22)) {
        hipLaunchKernelGGL(conv_1x1_spatial1_bwd_weight_kernel, (unsigned)ceil_div(total, 256), 256, 0, st,
                           (const float*)x, (const float*)dy, (float*)dw, g.n, g.c, g.m);
        return launch_status("conv2d_backward_weight(1x1 on 1x1)");
    }
    if (is_pointwise(g) && red > 0) {
        const int64_t hw = (int64_t)g.h * g.w;
        const int64_t parts = pointwise_bwd_weight_partials(g.n, g.m, g.c, hw);
        if (parts > 0 && aligned16(x) && aligned16(dy)) {
            // streaming kernel: every workgroup's M x C result, then their sum in a fixed order
            const int64_t mc = (int64_t)g.m * g.c;
            float* part = parts > 1 ? (float*)workspace : (float*)dw;
            if (int e = launch_pointwise_bwd_weight((const float*)x, (const float*)dy, part, g.n, g.m, g.c, hw, st)) return e;
            if (parts == 1) return 0;
            const size_t part_bytes = (size_t)parts * mc * sizeof(float);
            return dmlhip_reduce_f32(DMLHIP_RSUM, part, dw, DMLHIP_F32, 1, parts, mc, (char*)workspace + part_bytes,
                                     workspace_bytes - part_bytes, stream);
        }
        // per image: P[b] (M x C) = dY[b] (M x HW) . X[b]^T (HW x C); then dW = sum_b P[b]
        dmlhip_gemm_desc gd = {};
        gd.m = g.m; gd.n = g.c; gd.k = hw;
        gd.batch[0] = 1; gd.batch[1] = 1; gd.batch[2] = g.n;
        gd.a_stride_m = hw; gd.a_stride_k = 1; gd.a_stride_batch[2] = (int64_t)g.m * hw;
        gd.b_stride_k = 1; gd.b_stride_n = hw; gd.b_stride_batch[2] = (int64_t)g.c * hw;
        gd.c_stride_m = g.c; gd.c_stride_batch[2] = (int64_t)g.m * g.c;
        gd.alpha = 1.f; gd.out_dtype = DMLHIP_F32; gd.bias_dtype = DMLHIP_F32;
        if (g.n == 1) return dmlhip_gemm_f32(&gd, dy, x, dw, nullptr, nullptr, nullptr, stream);
        float* part = (float*)workspace;
        if (int e = dmlhip_gemm_f32(&gd, dy, x, part, nullptr, nullptr, nullptr, stream)) return e;
        const size_t part_bytes = (size_t)g.n * g.m * g.c * sizeof(float);
        return dmlhip_reduce_f32(DMLHIP_RSUM, part, dw, DMLHIP_F32, 1, g.n, (int64_t)g.m * g.c,
                                 (char*)workspace + part_bytes, workspace_bytes - part_bytes, stream);
    }
    hipLaunchKernelGGL(conv_bwd_weight_kernel, (unsigned)total, 256, 0, st, (const float*)x, (const float*)dy,
                       (float*)dw, g);
    return launch_status("conv2d_backward_weight");
}

}  // extern "C"
