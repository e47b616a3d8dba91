// Pad with a constant (ONNX Pad, mode "constant"): y[i] = x[i - begin] where that lies inside x, the fill value
// elsewhere. Negative amounts crop, as in ONNX - which also makes this the reverse of itself: the gradient of a Pad is
// the Pad with the amounts negated. One output element per thread and iteration; a pass over memory, nothing more.
#include "common.h"

namespace dml {
namespace {

struct PadDims {
    int ndim;
    int64_t out[DMLHIP_MAX_DIMS];    // output extents
    int64_t in[DMLHIP_MAX_DIMS];     // input extents
    int64_t begin[DMLHIP_MAX_DIMS];  // amount added in front of each axis (negative: removed)
    int64_t xs[DMLHIP_MAX_DIMS];     // input strides (dense)
};

template <typename T>
__global__ __launch_bounds__(256) void pad_constant_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n,
                                                           PadDims d, float value) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    const T fill = from_f32<T>(value);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        int64_t rem = i, off = 0;
        bool inside = true;
#pragma unroll
        for (int k = DMLHIP_MAX_DIMS - 1; k >= 0; --k) {
            if (k < d.ndim) {
                const int64_t s = rem % d.out[k] - d.begin[k];
                rem /= d.out[k];
                inside = inside && s >= 0 && s < d.in[k];
                off += s * d.xs[k];
            }
        }
        y[i] = inside ? x[off] : fill;
    }
}

template <typename T>
int pad_impl(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* begin, const int64_t* end,
             float value, void* stream) {
    DML_REQUIRE(ndim >= 0 && ndim <= DMLHIP_MAX_DIMS, DMLHIP_ERR_SHAPE, "pad: ndim %d outside [0, %d]", ndim,
                DMLHIP_MAX_DIMS);
    DML_REQUIRE(ndim == 0 || (shape && begin && end), DMLHIP_ERR_NULL, "pad: NULL shape / amounts");
    PadDims d;
    d.ndim = ndim;
    int64_t n_out = 1, n_in = 1;
    for (int k = 0; k < ndim; ++k) {
        DML_REQUIRE(shape[k] >= 0, DMLHIP_ERR_SHAPE, "pad: negative extent");
        const int64_t lim = INT64_MAX / 64;
        DML_REQUIRE(begin[k] > -lim && begin[k] < lim && end[k] > -lim && end[k] < lim && shape[k] < lim, DMLHIP_ERR_SHAPE,
                    "pad: amounts out of range");
        d.in[k] = shape[k];
        d.begin[k] = begin[k];
        d.out[k] = shape[k] + begin[k] + end[k];
        DML_REQUIRE(d.out[k] >= 0, DMLHIP_ERR_SHAPE, "pad: axis %d is cropped by more than its extent", k);
        DML_REQUIRE(d.out[k] == 0 || n_out <= (INT64_MAX / 16) / d.out[k], DMLHIP_ERR_SHAPE, "pad: size overflows");
        DML_REQUIRE(d.in[k] == 0 || n_in <= (INT64_MAX / 16) / d.in[k], DMLHIP_ERR_SHAPE, "pad: size overflows");
        n_out *= d.out[k];
        n_in *= d.in[k];
    }
    for (int k = ndim; k < DMLHIP_MAX_DIMS; ++k) { d.in[k] = d.out[k] = 1; d.begin[k] = 0; }
    int64_t s = 1;
    for (int k = DMLHIP_MAX_DIMS - 1; k >= 0; --k) { d.xs[k] = k < ndim ? s : 0; if (k < ndim) s *= d.in[k]; }
    if (n_out == 0) return 0;
    DML_REQUIRE(y && (x || n_in == 0), DMLHIP_ERR_NULL, "pad: NULL tensor pointer");
    int64_t grid = ceil_div(n_out, 256);
    if (grid > 256 * 32) grid = 256 * 32;
    hipLaunchKernelGGL((pad_constant_kernel<T>), (unsigned)grid, 256, 0, (hipStream_t)stream, (const T*)x, (T*)y, n_out, d,
                       value);
    return launch_status("pad");
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {
int dmlhip_pad_constant_f16(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* begin,
                            const int64_t* end, float value, void* stream) {
    return pad_impl<_Float16>(x, y, ndim, shape, begin, end, value, stream);
}
int dmlhip_pad_constant_f32(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* begin,
                            const int64_t* end, float value, void* stream) {
    return pad_impl<float>(x, y, ndim, shape, begin, end, value, stream);
}
}
