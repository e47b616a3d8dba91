// MaxPool over the two trailing axes (PureMaxPool2D, img_op_implementations.py:28-161: no padding, no dilation,
// floor output extents) and its gradient (DefaultMaxPoolBackward, autodiff/implementations/onnx_ops.py:284-335: the
// gradient of an output goes to the first position of its window that holds the maximum, windows scanned row by row).
//
// Forward: one output element per thread. Backward: one INPUT element per thread, which sums the gradients of the
// windows that cover it and have their maximum there - a gather, so overlapping windows need no atomics and the result
// does not depend on the order in which threads run. Both are passes over memory.
#include "common.h"

namespace dml {
namespace {

struct PoolArgs {
    int64_t planes;              // batch * channels
    int h, w, oh, ow;
    int kh, kw, sh, sw;
};

template <typename T>
__global__ __launch_bounds__(256) void maxpool2d_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n,
                                                        PoolArgs a) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const int ox = (int)(i % a.ow);
        const int64_t r = i / a.ow;
        const int oy = (int)(r % a.oh);
        const int64_t p = r / a.oh;
        const T* xp = x + (p * a.h + (int64_t)oy * a.sh) * a.w + (int64_t)ox * a.sw;
        float best = to_f32(xp[0]);
        for (int ky = 0; ky < a.kh; ++ky)
            for (int kx = 0; kx < a.kw; ++kx) best = fmaxf(best, to_f32(xp[(int64_t)ky * a.w + kx]));
        y[i] = from_f32<T>(best);
    }
}

// position (row-major inside the window) of the first maximum of the window whose top-left corner is `xp`
template <typename T>
__device__ __forceinline__ int window_argmax(const T* xp, const PoolArgs& a) {
    float best = to_f32(xp[0]);
    int arg = 0;
    for (int ky = 0; ky < a.kh; ++ky)
        for (int kx = 0; kx < a.kw; ++kx) {
            const float v = to_f32(xp[(int64_t)ky * a.w + kx]);
            if (v > best) {
                best = v;
                arg = ky * a.kw + kx;
            }
        }
    return arg;
}

template <typename T>
__global__ __launch_bounds__(256) void maxpool2d_bwd_kernel(const T* __restrict__ x, const T* __restrict__ dy,
                                                            T* __restrict__ dx, int64_t n, PoolArgs a) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const int ix = (int)(i % a.w);
        const int64_t r = i / a.w;
        const int iy = (int)(r % a.h);
        const int64_t p = r / a.h;
        // windows (oy, ox) with oy*sh <= iy < oy*sh + kh, likewise along x, inside the output
        const int oy_lo = iy >= a.kh ? (iy - a.kh) / a.sh + 1 : 0, oy_hi = min(iy / a.sh, a.oh - 1);
        const int ox_lo = ix >= a.kw ? (ix - a.kw) / a.sw + 1 : 0, ox_hi = min(ix / a.sw, a.ow - 1);
        float g = 0.f;
        for (int oy = oy_lo; oy <= oy_hi; ++oy)
            for (int ox = ox_lo; ox <= ox_hi; ++ox) {
                const T* xp = x + (p * a.h + (int64_t)oy * a.sh) * a.w + (int64_t)ox * a.sw;
                const int arg = window_argmax(xp, a);
                if (arg == (iy - oy * a.sh) * a.kw + (ix - ox * a.sw)) g += to_f32(dy[(p * a.oh + oy) * a.ow + ox]);
            }
        dx[i] = from_f32<T>(g);
    }
}

int fill_pool(int64_t planes, int64_t h, int64_t w, int64_t kh, int64_t kw, int64_t sh, int64_t sw, PoolArgs& a,
              const char* what) {
    DML_REQUIRE(planes >= 0 && h >= 0 && w >= 0, DMLHIP_ERR_SHAPE, "%s: negative extent", what);
    DML_REQUIRE(kh >= 1 && kw >= 1 && sh >= 1 && sw >= 1, DMLHIP_ERR_SHAPE, "%s: window and strides must be positive", what);
    DML_REQUIRE(h <= 2147483647 && w <= 2147483647 && kh <= 65535 && kw <= 65535 && sh <= 65535 && sw <= 65535,
                DMLHIP_ERR_SHAPE, "%s: extent out of range", what);
    a.planes = planes;
    a.h = (int)h; a.w = (int)w; a.kh = (int)kh; a.kw = (int)kw; a.sh = (int)sh; a.sw = (int)sw;
    a.oh = h >= kh ? (int)((h - kh) / sh + 1) : 0;
    a.ow = w >= kw ? (int)((w - kw) / sw + 1) : 0;
    DML_REQUIRE(planes == 0 || ((int64_t)a.h * a.w <= (INT64_MAX / 16) / planes), DMLHIP_ERR_SHAPE, "%s: size overflows", what);
    return 0;
}

unsigned grid_for(int64_t n) {
    int64_t g = ceil_div(n, 256);
    return (unsigned)(g > 256 * 32 ? 256 * 32 : g);
}

template <typename T>
int maxpool_impl(const void* x, void* y, int64_t planes, int64_t h, int64_t w, int64_t kh, int64_t kw, int64_t sh,
                 int64_t sw, void* stream) {
    PoolArgs a;
    if (int e = fill_pool(planes, h, w, kh, kw, sh, sw, a, "maxpool2d")) return e;
    const int64_t n = planes * a.oh * a.ow;
    if (n == 0) return 0;
    DML_REQUIRE(x && y, DMLHIP_ERR_NULL, "maxpool2d: NULL tensor pointer");
    hipLaunchKernelGGL((maxpool2d_kernel<T>), grid_for(n), 256, 0, (hipStream_t)stream, (const T*)x, (T*)y, n, a);
    return launch_status("maxpool2d");
}

template <typename T>
int maxpool_bwd_impl(const void* x, const void* dy, void* dx, int64_t planes, int64_t h, int64_t w, int64_t kh,
                     int64_t kw, int64_t sh, int64_t sw, void* stream) {
    PoolArgs a;
    if (int e = fill_pool(planes, h, w, kh, kw, sh, sw, a, "maxpool2d_backward")) return e;
    const int64_t n = planes * a.h * a.w;
    if (n == 0) return 0;
    DML_REQUIRE(x && dx && (dy || a.oh == 0 || a.ow == 0), DMLHIP_ERR_NULL, "maxpool2d_backward: NULL tensor pointer");
    hipLaunchKernelGGL((maxpool2d_bwd_kernel<T>), grid_for(n), 256, 0, (hipStream_t)stream, (const T*)x, (const T*)dy,
                       (T*)dx, n, a);
    return launch_status("maxpool2d_backward");
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {
int dmlhip_maxpool2d_f16(const void* x, void* y, int64_t planes, int64_t h, int64_t w, int64_t kh, int64_t kw,
                         int64_t sh, int64_t sw, void* stream) {
    return maxpool_impl<_Float16>(x, y, planes, h, w, kh, kw, sh, sw, stream);
}
int dmlhip_maxpool2d_f32(const void* x, void* y, int64_t planes, int64_t h, int64_t w, int64_t kh, int64_t kw,
                         int64_t sh, int64_t sw, void* stream) {
    return maxpool_impl<float>(x, y, planes, h, w, kh, kw, sh, sw, stream);
}
int dmlhip_maxpool2d_backward_f16(const void* x, const void* dy, void* dx, int64_t planes, int64_t h, int64_t w,
                                  int64_t kh, int64_t kw, int64_t sh, int64_t sw, void* stream) {
    return maxpool_bwd_impl<_Float16>(x, dy, dx, planes, h, w, kh, kw, sh, sw, stream);
}
int dmlhip_maxpool2d_backward_f32(const void* x, const void* dy, void* dx, int64_t planes, int64_t h, int64_t w,
                                  int64_t kh, int64_t kw, int64_t sh, int64_t sw, void* stream) {
    return maxpool_bwd_impl<float>(x, dy, dx, planes, h, w, kh, kw, sh, sw, stream);
}
}
