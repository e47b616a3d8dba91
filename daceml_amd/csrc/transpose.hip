// Transpose (np.transpose with an arbitrary permutation, up to DMLHIP_MAX_DIMS dims).
//   * permutations that keep the innermost dim innermost are row copies: 128-bit vector moves;
//   * everything else goes through a 32x32 LDS tile spanned by the input's innermost dim and the
//     output's innermost dim, so both the global reads and the global writes are coalesced.
#include "common.h"

namespace dml {
namespace {

struct TrDims {
    int ndim;                        // dims of the output
    int64_t shape[DMLHIP_MAX_DIMS];  // output extents
    int64_t xs[DMLHIP_MAX_DIMS];     // stride in x of output dim k
    int64_t ys[DMLHIP_MAX_DIMS];     // stride in y of output dim k
};

// innermost dim preserved: y[..., :] = x[..., :] in units of V elements
template <typename T, int V>
__global__ __launch_bounds__(256) void transpose_rows_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t nvec,
                                                             TrDims d) {
    typedef T vec_t __attribute__((ext_vector_type(V)));
    const int64_t stride = (int64_t)gridDim.x * 256;
    const int last = d.ndim - 1;
    const int64_t inner_vecs = d.shape[last] / V;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += stride) {
        int64_t rem = i / inner_vecs;
        int64_t off = (i % inner_vecs) * V;
#pragma unroll
        for (int k = DMLHIP_MAX_DIMS - 2; k >= 0; --k) {
            if (k < last) {
                off += (rem % d.shape[k]) * d.xs[k];
                rem /= d.shape[k];
            }
        }
        if constexpr (V > 1) *reinterpret_cast<vec_t*>(y + i * V) = *reinterpret_cast<const vec_t*>(x + off);
        else y[i] = x[off];
    }
}

// general case. `a` = output dim that is innermost in x (xs[a] == 1); b = ndim-1 (ys[b] == 1).
template <typename T>
__global__ __launch_bounds__(256) void transpose_tile_kernel(const T* __restrict__ x, T* __restrict__ y, TrDims d,
                                                             int a, int64_t tiles_a, int64_t tiles_b) {
    __shared__ T tile[32][33];
    const int b = d.ndim - 1;
    int64_t bid = blockIdx.x;
    const int64_t ta = bid % tiles_a; bid /= tiles_a;
    const int64_t tb = bid % tiles_b; bid /= tiles_b;
    int64_t xo = 0, yo = 0;
#pragma unroll
    for (int k = DMLHIP_MAX_DIMS - 1; k >= 0; --k) {
        if (k < d.ndim && k != a && k != b) {
            const int64_t idx = bid % d.shape[k];
            bid /= d.shape[k];
            xo += idx * d.xs[k];
            yo += idx * d.ys[k];
        }
    }
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int64_t a0 = ta * 32, b0 = tb * 32;
    for (int j = ty; j < 32; j += 8) {
        if (a0 + tx < d.shape[a] && b0 + j < d.shape[b]) tile[j][tx] = x[xo + (a0 + tx) * d.xs[a] + (b0 + j) * d.xs[b]];
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        if (a0 + j < d.shape[a] && b0 + tx < d.shape[b]) y[yo + (a0 + j) * d.ys[a] + (b0 + tx) * d.ys[b]] = tile[tx][j];
    }
}

template <typename T>
int transpose_impl(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* perm, void* stream) {
    DML_REQUIRE(ndim >= 0 && ndim <= DMLHIP_MAX_DIMS, DMLHIP_ERR_SHAPE, "transpose: ndim %d outside [0, %d]", ndim,
                DMLHIP_MAX_DIMS);
    DML_REQUIRE(ndim == 0 || (shape && perm), DMLHIP_ERR_NULL, "transpose: NULL shape/perm");
    bool seen[DMLHIP_MAX_DIMS] = {};
    int64_t n = 1;
    int64_t xstride[DMLHIP_MAX_DIMS];
    for (int i = 0; i < ndim; ++i) {
        DML_REQUIRE(perm[i] >= 0 && perm[i] < ndim && !seen[perm[i]], DMLHIP_ERR_SHAPE,
                    "transpose: perm is not a permutation");
        seen[perm[i]] = true;
        DML_REQUIRE(shape[i] >= 0, DMLHIP_ERR_SHAPE, "transpose: negative extent");
        DML_REQUIRE(shape[i] == 0 || n <= (INT64_MAX / 16) / shape[i], DMLHIP_ERR_SHAPE, "transpose: size overflows");
        n *= shape[i];
    }
    if (n == 0) return 0;
    DML_REQUIRE(x && y, DMLHIP_ERR_NULL, "transpose: NULL tensor pointer");
    int64_t s = 1;
    for (int i = ndim - 1; i >= 0; --i) { xstride[i] = s; s *= shape[i]; }

    // output dims with extent 1 dropped and runs that stay adjacent in x merged
    TrDims d;
    d.ndim = 0;
    for (int k = 0; k < ndim; ++k) {
        const int64_t ext = shape[perm[k]], xs = xstride[perm[k]];
        if (ext == 1) continue;
        if (d.ndim > 0 && d.xs[d.ndim - 1] == xs * ext) {
            d.shape[d.ndim - 1] *= ext;
            d.xs[d.ndim - 1] = xs;
        } else {
            d.shape[d.ndim] = ext;
            d.xs[d.ndim] = xs;
            ++d.ndim;
        }
    }
    if (d.ndim == 0) { d.ndim = 1; d.shape[0] = 1; d.xs[0] = 1; }
    for (int k = d.ndim; k < DMLHIP_MAX_DIMS; ++k) { d.shape[k] = 1; d.xs[k] = 0; }
    s = 1;
    for (int k = DMLHIP_MAX_DIMS - 1; k >= 0; --k) { d.ys[k] = k < d.ndim ? s : 0; if (k < d.ndim) s *= d.shape[k]; }

    hipStream_t st = (hipStream_t)stream;
    const T* xp = (const T*)x;
    T* yp = (T*)y;
    const int last = d.ndim - 1;
    if (d.xs[last] == 1) {
        constexpr int VN = VecOf<T>::n;
        bool vec = d.shape[last] % VN == 0 && aligned16(x) && aligned16(y);
        for (int k = 0; k < last; ++k) vec = vec && d.xs[k] % VN == 0;
        const int64_t nvec = vec ? n / VN : n;
        int64_t grid = ceil_div(nvec, 256);
        if (grid > 256 * 32) grid = 256 * 32;
        if (vec) hipLaunchKernelGGL((transpose_rows_kernel<T, VN>), (unsigned)grid, 256, 0, st, xp, yp, nvec, d);
        else hipLaunchKernelGGL((transpose_rows_kernel<T, 1>), (unsigned)grid, 256, 0, st, xp, yp, nvec, d);
        return launch_status("transpose(rows)");
    }
    int a = -1;
    for (int k = 0; k < d.ndim; ++k)
        if (d.xs[k] == 1) a = k;
    DML_REQUIRE(a >= 0 && a != last, DMLHIP_ERR_UNSUPPORTED, "transpose: internal layout error");
    const int64_t tiles_a = ceil_div(d.shape[a], 32), tiles_b = ceil_div(d.shape[last], 32);
    int64_t blocks = tiles_a * tiles_b;
    for (int k = 0; k < d.ndim; ++k)
        if (k != a && k != last) blocks *= d.shape[k];
    DML_REQUIRE(blocks <= 2147483647LL, DMLHIP_ERR_SHAPE, "transpose: too many tiles");
    hipLaunchKernelGGL((transpose_tile_kernel<T>), (unsigned)blocks, 256, 0, st, xp, yp, d, a, tiles_a, tiles_b);
    return launch_status("transpose(tiles)");
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {
int dmlhip_transpose_f16(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* perm, void* stream) {
    return transpose_impl<_Float16>(x, y, ndim, shape, perm, stream);
}
int dmlhip_transpose_f32(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* perm, void* stream) {
    return transpose_impl<float>(x, y, ndim, shape, perm, stream);
}
}
