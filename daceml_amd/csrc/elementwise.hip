// Element-wise nodes: broadcasting binary ops, unary maps and their derivatives, variadic Sum,
// bias+GELU, Cast. All are one HBM pass with 128-bit accesses on the dense fast paths; any
// stride pattern falls back to an index-decoding kernel with the same arithmetic.
#include "common.h"
#include "lds_ops.h"

namespace dml {
namespace {

constexpr int kEwBlock = 256;

inline unsigned ew_grid(int64_t work_items) {
    int64_t g = ceil_div(work_items, kEwBlock);
    const int64_t cap = 256 * 32;  // 32 workgroups per CU, grid-stride beyond that
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return (unsigned)g;
}

// ------------------------------------------------------------------ op functors
template <int OP> __device__ __forceinline__ float binary_apply(float a, float b) {
    if constexpr (OP == DMLHIP_ADD) return a + b;
    else if constexpr (OP == DMLHIP_SUB) return a - b;
    else if constexpr (OP == DMLHIP_MUL) return a * b;
    else if constexpr (OP == DMLHIP_DIV) return a / b;
    else return powf(a, b);
}

template <int OP> __device__ __forceinline__ float unary_apply(float x, float p) {
    if constexpr (OP == DMLHIP_ERF) return erff(x);
    else if constexpr (OP == DMLHIP_SQRT) return sqrtf(x);
    else if constexpr (OP == DMLHIP_EXP) return expf(x);
    else if constexpr (OP == DMLHIP_LOG) return logf(x);
    else if constexpr (OP == DMLHIP_TANH) return tanhf(x);
    else if constexpr (OP == DMLHIP_RELU) return fmaxf(x, 0.f);
    else if constexpr (OP == DMLHIP_SIGMOID) return sigmoid_f(x);
    else if constexpr (OP == DMLHIP_RECIPROCAL) return 1.0f / x;
    else if constexpr (OP == DMLHIP_GELU) return gelu_f(x);
    else if constexpr (OP == DMLHIP_SWISH) return x * sigmoid_f(x);
    else if constexpr (OP == DMLHIP_SCALE) return x * p;
    else return x;
}

template <int OP> __device__ __forceinline__ float unary_grad(float x, float p) {
    if constexpr (OP == DMLHIP_ERF) return 1.12837916709551257390f * expf(-x * x);
    else if constexpr (OP == DMLHIP_SQRT) return 0.5f / sqrtf(x);
    else if constexpr (OP == DMLHIP_EXP) return expf(x);
    else if constexpr (OP == DMLHIP_LOG) return 1.0f / x;
    else if constexpr (OP == DMLHIP_TANH) { const float t = tanhf(x); return 1.0f - t * t; }
    else if constexpr (OP == DMLHIP_RELU) return x > 0.f ? 1.f : 0.f;
    else if constexpr (OP == DMLHIP_SIGMOID) { const float s = sigmoid_f(x); return s * (1.0f - s); }
    else if constexpr (OP == DMLHIP_RECIPROCAL) return -1.0f / (x * x);
    else if constexpr (OP == DMLHIP_GELU) return gelu_grad_f(x);
    else if constexpr (OP == DMLHIP_SWISH) { const float s = sigmoid_f(x); return s * (1.0f + x * (1.0f - s)); }
    else if constexpr (OP == DMLHIP_SCALE) return p;
    else return 1.0f;
}

// ------------------------------------------------------------------ binary, dense fast paths
// MODE 0: a and b dense and equal-shaped. MODE 1: b is a row vector of `period` elements repeated
// along the flattened output (bias add). MODE 2: b is one scalar. MODE 3: b holds one value per row of `period`
// output elements (a per-image, per-channel factor against [N, C, H, W]; n < 2^32). MODE 4: a holds one value per row
// and b is one scalar (a reduced tensor expanded back over its rows and scaled). SWAP evaluates op(b, a) so that
// the same layouts serve a broadcast first operand.
template <typename T, int OP, int MODE, bool SWAP>
__global__ __launch_bounds__(kEwBlock) void binary_vec_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                              T* __restrict__ c, int64_t n, int64_t period) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const int64_t nvec = n / VN;
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    float bs = 0.f, as = 0.f;
    if constexpr (MODE == 2 || MODE == 4) bs = to_f32(b[0]);
    for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < nvec; i += stride) {
        V av, bv;
        if constexpr (MODE == 4) as = to_f32(a[(uint32_t)(i * VN) / (uint32_t)period]);
        else av = reinterpret_cast<const V*>(a)[i];
        if constexpr (MODE == 0) bv = reinterpret_cast<const V*>(b)[i];
        if constexpr (MODE == 1) bv = reinterpret_cast<const V*>(b)[(i * VN % period) / VN];
        if constexpr (MODE == 3) bs = to_f32(b[(uint32_t)(i * VN) / (uint32_t)period]);   // period % VN == 0: one row
        V cv;
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            const float x = MODE == 4 ? as : to_f32(av[e]);
            const float y = (MODE == 2 || MODE == 3 || MODE == 4) ? bs : to_f32(bv[e]);
            cv[e] = from_f32<T>(SWAP ? binary_apply<OP>(y, x) : binary_apply<OP>(x, y));
        }
        reinterpret_cast<V*>(c)[i] = cv;
    }
    // tail (n not a multiple of the vector width; MODE 1, 3 and 4 are launched with whole vectors only)
    for (int64_t i = nvec * VN + (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < n; i += stride) {
        const float x = to_f32(a[MODE == 4 ? i / period : i]);
        const float y = (MODE == 2 || MODE == 4) ? bs : to_f32(b[MODE == 1 ? i % period : (MODE == 3 ? i / period : i)]);
        c[i] = from_f32<T>(SWAP ? binary_apply<OP>(y, x) : binary_apply<OP>(x, y));
    }
}

// y[r, j] = a[r, j] * s[r] + t[r] * scale[0]: a dense tensor times one factor per row plus one (scaled) value per row
// expanded over the row — the two gradient contributions that meet at the input of a squeeze-excite block (through
// the gate multiplication and through the average pool), without their two intermediate tensors and the Sum pass.
template <typename T>
__global__ __launch_bounds__(kEwBlock) void row_affine_kernel(const T* __restrict__ a, const T* __restrict__ s,
                                                              const T* __restrict__ t, const T* __restrict__ scale,
                                                              T* __restrict__ y, int64_t rows, int64_t cols, int vec) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const float k = scale ? to_f32(scale[0]) : 1.0f;
    const int64_t n = rows * cols;
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    if (vec) {   // whole vectors inside one row, n < 2^32
        const int64_t nvec = n / VN;
        for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < nvec; i += stride) {
            const uint32_t row = (uint32_t)(i * VN) / (uint32_t)cols;
            const float sv = to_f32(s[row]), tv = to_f32(t[row]) * k;
            V av = reinterpret_cast<const V*>(a)[i], yv;
#pragma unroll
            for (int e = 0; e < VN; ++e) yv[e] = from_f32<T>(to_f32(av[e]) * sv + tv);
            reinterpret_cast<V*>(y)[i] = yv;
        }
    } else {
        for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < n; i += stride) {
            const int64_t row = i / cols;
            y[i] = from_f32<T>(to_f32(a[i]) * to_f32(s[row]) + to_f32(t[row]) * k);
        }
    }
}

template <typename T>
int row_affine_impl(const void* a, const void* s, const void* t, const void* scale, void* y, int64_t rows, int64_t cols,
                    void* stream) {
    DML_REQUIRE(rows >= 0 && cols >= 0, DMLHIP_ERR_SHAPE, "row_affine: negative extent");
    DML_REQUIRE(cols == 0 || rows <= (INT64_MAX / 16) / cols, DMLHIP_ERR_SHAPE, "row_affine: size overflows");
    const int64_t n = rows * cols;
    if (n == 0) return 0;
    DML_REQUIRE(a && s && t && y, DMLHIP_ERR_NULL, "row_affine: NULL tensor pointer");
    const int vec = aligned16(a) && aligned16(y) && cols % VecOf<T>::n == 0 && n < (1LL << 32);
    hipLaunchKernelGGL((row_affine_kernel<T>), ew_grid(ceil_div(n, vec ? VecOf<T>::n : 1)), kEwBlock, 0, (hipStream_t)stream,
                       (const T*)a, (const T*)s, (const T*)t, (const T*)scale, (T*)y, rows, cols, vec);
    return launch_status("row_affine");
}

struct BcastDims {
    int ndim;
    int64_t shape[DMLHIP_MAX_DIMS];
    int64_t sa[DMLHIP_MAX_DIMS];
    int64_t sb[DMLHIP_MAX_DIMS];
};

template <typename T, int OP>
__global__ __launch_bounds__(kEwBlock) void binary_general_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                                  T* __restrict__ c, int64_t n, BcastDims d) {
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < n; i += stride) {
        int64_t rem = i, oa = 0, ob = 0;
#pragma unroll
        for (int k = DMLHIP_MAX_DIMS - 1; k >= 0; --k) {
            if (k < d.ndim) {
                const int64_t idx = rem % d.shape[k];
                rem /= d.shape[k];
                oa += idx * d.sa[k];
                ob += idx * d.sb[k];
            }
        }
        c[i] = from_f32<T>(binary_apply<OP>(to_f32(a[oa]), to_f32(b[ob])));
    }
}

// ------------------------------------------------------------------ unary
// y may be the very buffer of dy (the gradient written over the gradient it was computed from: a thread reads its
// elements before it writes them, and no other thread touches them), so these two carry no __restrict__.
template <typename T, int OP, bool GRAD>
__global__ __launch_bounds__(kEwBlock) void unary_kernel(const T* __restrict__ x, const T* dy, T* y, int64_t n, float p) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const int64_t nvec = n / VN;
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < nvec; i += stride) {
        V xv = reinterpret_cast<const V*>(x)[i];
        V gv;
        if constexpr (GRAD) gv = reinterpret_cast<const V*>(dy)[i];
        V yv;
#pragma unroll
        for (int e = 0; e < VN; ++e) {
            if constexpr (GRAD && OP == DMLHIP_GELU && sizeof(T) == 2)
                yv[e] = from_f32<T>(to_f32(gv[e]) * gelu_grad_half_f(to_f32(xv[e])));
            else if constexpr (GRAD) yv[e] = from_f32<T>(to_f32(gv[e]) * unary_grad<OP>(to_f32(xv[e]), p));
            else if constexpr (OP == DMLHIP_GELU && sizeof(T) == 2) yv[e] = from_f32<T>(gelu_half_f(to_f32(xv[e])));
            else yv[e] = from_f32<T>(unary_apply<OP>(to_f32(xv[e]), p));
        }
        // fp16 results go through the L2 as they are written (see global_store_b128_through): Gelu on 32 MB 15.5 ->
        // 14.5 us, its gradient 19.9 -> 19.0 us inside the BERT step
        if constexpr (sizeof(T) == 2) global_store_b128_through(reinterpret_cast<V*>(y) + i, yv);
        else reinterpret_cast<V*>(y)[i] = yv;
    }
    for (int64_t i = nvec * VN + (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < n; i += stride) {
        if constexpr (GRAD) y[i] = from_f32<T>(to_f32(dy[i]) * unary_grad<OP>(to_f32(x[i]), p));
        else y[i] = from_f32<T>(unary_apply<OP>(to_f32(x[i]), p));
    }
}

// ------------------------------------------------------------------ variadic sum
struct SumPtrs { const void* p[8]; };

template <typename T, int N>
__global__ __launch_bounds__(kEwBlock) void sum_kernel(SumPtrs in, T* __restrict__ out, int64_t n) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const int64_t nvec = n / VN;
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < nvec; i += stride) {
        float acc[VN];
#pragma unroll
        for (int e = 0; e < VN; ++e) acc[e] = 0.f;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            V v = reinterpret_cast<const V*>(in.p[k])[i];
#pragma unroll
            for (int e = 0; e < VN; ++e) acc[e] += to_f32(v[e]);
        }
        V o;
#pragma unroll
        for (int e = 0; e < VN; ++e) o[e] = from_f32<T>(acc[e]);
        reinterpret_cast<V*>(out)[i] = o;
    }
    for (int64_t i = nvec * VN + (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < n; i += stride) {
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < N; ++k) acc += to_f32(reinterpret_cast<const T*>(in.p[k])[i]);
        out[i] = from_f32<T>(acc);
    }
}

// ------------------------------------------------------------------ bias + GELU
template <typename T, bool VEC>
__global__ __launch_bounds__(kEwBlock) void bias_gelu_kernel(const T* __restrict__ x, const T* __restrict__ bias,
                                                             T* __restrict__ y, T* __restrict__ pre, int64_t n,
                                                             int64_t cols) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VEC ? VecOf<T>::n : 1;
    const int64_t nvec = n / VN;
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < nvec; i += stride) {
        if constexpr (VEC) {
            V xv = reinterpret_cast<const V*>(x)[i];
            V yv, pv;
            V bv = {};
            if (bias) bv = reinterpret_cast<const V*>(bias)[(i * VN % cols) / VN];
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                // the Add node rounds to the tensor dtype before the GELU chain reads it
                pv[e] = from_f32<T>(to_f32(xv[e]) + to_f32(bv[e]));
                yv[e] = from_f32<T>(gelu_f(to_f32(pv[e])));
            }
            if (pre) reinterpret_cast<V*>(pre)[i] = pv;
            reinterpret_cast<V*>(y)[i] = yv;
        } else {
            const T u = from_f32<T>(to_f32(x[i]) + (bias ? to_f32(bias[i % cols]) : 0.f));
            if (pre) pre[i] = u;
            y[i] = from_f32<T>(gelu_f(to_f32(u)));
        }
    }
}

// ------------------------------------------------------------------ cast
template <typename S, typename D>
__global__ __launch_bounds__(kEwBlock) void cast_kernel(const S* __restrict__ x, D* __restrict__ y, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * kEwBlock;
    for (int64_t i = (int64_t)blockIdx.x * kEwBlock + threadIdx.x; i < n; i += stride) y[i] = (D)x[i];
}

// ------------------------------------------------------------------ host side
// Merge adjacent output dims that are laid out contiguously in both operands (broadcast dims
// merge with broadcast dims), and drop extent-1 dims.
BcastDims collapse(int ndim, const int64_t* shape, const int64_t* sa, const int64_t* sb) {
    BcastDims d;
    d.ndim = 0;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] == 1) continue;
        if (d.ndim > 0) {
            const int p = d.ndim - 1;
            if (d.sa[p] == sa[i] * shape[i] && d.sb[p] == sb[i] * shape[i]) {
                d.shape[p] *= shape[i];
                d.sa[p] = sa[i];
                d.sb[p] = sb[i];
                continue;
            }
        }
        d.shape[d.ndim] = shape[i];
        d.sa[d.ndim] = sa[i];
        d.sb[d.ndim] = sb[i];
        ++d.ndim;
    }
    if (d.ndim == 0) {
        d.ndim = 1;
        d.shape[0] = 1;
        d.sa[0] = 0;
        d.sb[0] = 0;
    }
    for (int i = d.ndim; i < DMLHIP_MAX_DIMS; ++i) { d.shape[i] = 1; d.sa[i] = 0; d.sb[i] = 0; }
    return d;
}

template <typename T, int OP>
int binary_launch(const T* a, const T* b, T* c, int64_t n, const BcastDims& d, hipStream_t st) {
    constexpr int VN = VecOf<T>::n;
    const bool al = aligned16(a) && aligned16(b) && aligned16(c);
    const unsigned gv = ew_grid(ceil_div(n, VN));
#define DML_BIN(MODE, SWAP, A, B, PERIOD) \
    hipLaunchKernelGGL((binary_vec_kernel<T, OP, MODE, SWAP>), gv, kEwBlock, 0, st, A, B, c, n, (int64_t)(PERIOD))
    if (al && d.ndim == 1 && d.sa[0] == 1 && d.sb[0] == 1) { DML_BIN(0, false, a, b, 1); return 0; }
    if (al && d.ndim == 1 && d.sa[0] == 1 && d.sb[0] == 0) { DML_BIN(2, false, a, b, 1); return 0; }
    if (al && d.ndim == 1 && d.sa[0] == 0 && d.sb[0] == 1) { DML_BIN(2, true, b, a, 1); return 0; }
    if (al && d.ndim == 2 && d.shape[1] % VN == 0) {
        if (d.sa[0] == d.shape[1] && d.sa[1] == 1 && d.sb[0] == 0 && d.sb[1] == 1) { DML_BIN(1, false, a, b, d.shape[1]); return 0; }
        if (d.sb[0] == d.shape[1] && d.sb[1] == 1 && d.sa[0] == 0 && d.sa[1] == 1) { DML_BIN(1, true, b, a, d.shape[1]); return 0; }
        if (n < (1LL << 32)) {   // one operand dense, the other one value per row
            if (d.sa[0] == d.shape[1] && d.sa[1] == 1 && d.sb[0] == 1 && d.sb[1] == 0) { DML_BIN(3, false, a, b, d.shape[1]); return 0; }
            if (d.sb[0] == d.shape[1] && d.sb[1] == 1 && d.sa[0] == 1 && d.sa[1] == 0) { DML_BIN(3, true, b, a, d.shape[1]); return 0; }
            if (d.sa[0] == 1 && d.sa[1] == 0 && d.sb[0] == 0 && d.sb[1] == 0) { DML_BIN(4, false, a, b, d.shape[1]); return 0; }
            if (d.sb[0] == 1 && d.sb[1] == 0 && d.sa[0] == 0 && d.sa[1] == 0) { DML_BIN(4, true, b, a, d.shape[1]); return 0; }
        }
    }
#undef DML_BIN
    hipLaunchKernelGGL((binary_general_kernel<T, OP>), ew_grid(n), kEwBlock, 0, st, a, b, c, n, d);
    return 0;
}

template <typename T>
int binary_impl(int op, const void* a, const void* b, void* c, int ndim, const int64_t* shape,
                const int64_t* a_strides, const int64_t* b_strides, void* stream) {
    DML_REQUIRE(op >= DMLHIP_ADD && op <= DMLHIP_POW, DMLHIP_ERR_ENUM, "binary: unknown op %d", op);
    DML_REQUIRE(ndim >= 0 && ndim <= DMLHIP_MAX_DIMS, DMLHIP_ERR_SHAPE, "binary: ndim %d outside [0, %d]", ndim,
                DMLHIP_MAX_DIMS);
    DML_REQUIRE(ndim == 0 || (shape && a_strides && b_strides), DMLHIP_ERR_NULL, "binary: NULL shape/stride array");
    int64_t n = 1;
    for (int i = 0; i < ndim; ++i) {
        DML_REQUIRE(shape[i] >= 0 && a_strides[i] >= 0 && b_strides[i] >= 0, DMLHIP_ERR_SHAPE,
                    "binary: negative extent or stride in dim %d", i);
        DML_REQUIRE(shape[i] == 0 || n <= (INT64_MAX / 16) / shape[i], DMLHIP_ERR_SHAPE, "binary: size overflows");
        n *= shape[i];
    }
    if (n == 0) return 0;
    DML_REQUIRE(a && b && c, DMLHIP_ERR_NULL, "binary: NULL tensor pointer");
    const BcastDims d = collapse(ndim, shape, a_strides, b_strides);
    hipStream_t st = (hipStream_t)stream;
    const T* ap = (const T*)a;
    const T* bp = (const T*)b;
    T* cp = (T*)c;
    switch (op) {
        case DMLHIP_ADD: binary_launch<T, DMLHIP_ADD>(ap, bp, cp, n, d, st); break;
        case DMLHIP_SUB: binary_launch<T, DMLHIP_SUB>(ap, bp, cp, n, d, st); break;
        case DMLHIP_MUL: binary_launch<T, DMLHIP_MUL>(ap, bp, cp, n, d, st); break;
        case DMLHIP_DIV: binary_launch<T, DMLHIP_DIV>(ap, bp, cp, n, d, st); break;
        default: binary_launch<T, DMLHIP_POW>(ap, bp, cp, n, d, st); break;
    }
    return launch_status("binary");
}

template <typename T, bool GRAD>
int unary_impl(int op, const void* x, const void* dy, void* y, int64_t n, float p, void* stream) {
    DML_REQUIRE(op >= DMLHIP_ERF && op <= DMLHIP_IDENTITY, DMLHIP_ERR_ENUM, "unary: unknown op %d", op);
    DML_REQUIRE(n >= 0, DMLHIP_ERR_SHAPE, "unary: negative size");
    if (n == 0) return 0;
    DML_REQUIRE(x && y && (!GRAD || dy), DMLHIP_ERR_NULL, "unary: NULL tensor pointer");
    DML_REQUIRE(aligned16(x) && aligned16(y) && (!GRAD || aligned16(dy)), DMLHIP_ERR_ALIGN,
                "unary: tensors must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const unsigned g = ew_grid(ceil_div(n, VecOf<T>::n));
    const T* xp = (const T*)x;
    const T* gp = (const T*)dy;
    T* yp = (T*)y;
#define DML_UN(OP) case OP: hipLaunchKernelGGL((unary_kernel<T, OP, GRAD>), g, kEwBlock, 0, st, xp, gp, yp, n, p); break
    switch (op) {
        DML_UN(DMLHIP_ERF); DML_UN(DMLHIP_SQRT); DML_UN(DMLHIP_EXP); DML_UN(DMLHIP_LOG); DML_UN(DMLHIP_TANH);
        DML_UN(DMLHIP_RELU); DML_UN(DMLHIP_SIGMOID); DML_UN(DMLHIP_RECIPROCAL); DML_UN(DMLHIP_GELU);
        DML_UN(DMLHIP_SWISH); DML_UN(DMLHIP_SCALE); DML_UN(DMLHIP_IDENTITY);
    }
#undef DML_UN
    return launch_status("unary");
}

template <typename T>
int sum_impl(const void* const* inputs, int n_inputs, void* out, int64_t n, void* stream) {
    DML_REQUIRE(n_inputs >= 1 && n_inputs <= 8, DMLHIP_ERR_SHAPE, "sum: %d inputs, 1..8 supported per call", n_inputs);
    DML_REQUIRE(n >= 0, DMLHIP_ERR_SHAPE, "sum: negative size");
    DML_REQUIRE(inputs, DMLHIP_ERR_NULL, "sum: NULL input array");
    if (n == 0) return 0;
    DML_REQUIRE(out && aligned16(out), out ? DMLHIP_ERR_ALIGN : DMLHIP_ERR_NULL, "sum: output NULL or not 16-byte aligned");
    SumPtrs sp = {};
    for (int i = 0; i < n_inputs; ++i) {
        DML_REQUIRE(inputs[i], DMLHIP_ERR_NULL, "sum: input %d is NULL", i);
        DML_REQUIRE(aligned16(inputs[i]), DMLHIP_ERR_ALIGN, "sum: input %d not 16-byte aligned", i);
        sp.p[i] = inputs[i];
    }
    hipStream_t st = (hipStream_t)stream;
    const unsigned g = ew_grid(ceil_div(n, VecOf<T>::n));
    T* op = (T*)out;
#define DML_SUM(N) case N: hipLaunchKernelGGL((sum_kernel<T, N>), g, kEwBlock, 0, st, sp, op, n); break
    switch (n_inputs) { DML_SUM(1); DML_SUM(2); DML_SUM(3); DML_SUM(4); DML_SUM(5); DML_SUM(6); DML_SUM(7); DML_SUM(8); }
#undef DML_SUM
    return launch_status("sum");
}

template <typename T>
int bias_gelu_impl(const void* x, const void* bias, void* y, void* pre, int64_t rows, int64_t cols, void* stream) {
    DML_REQUIRE(rows >= 0 && cols >= 0, DMLHIP_ERR_SHAPE, "bias_gelu: negative extent");
    DML_REQUIRE(cols == 0 || rows <= (INT64_MAX / 16) / cols, DMLHIP_ERR_SHAPE, "bias_gelu: size overflows");
    const int64_t n = rows * cols;
    if (n == 0) return 0;
    DML_REQUIRE(x && y, DMLHIP_ERR_NULL, "bias_gelu: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const bool vec = cols % VecOf<T>::n == 0 && aligned16(x) && aligned16(y) && (!bias || aligned16(bias)) &&
                     (!pre || aligned16(pre));
    if (vec)
        hipLaunchKernelGGL((bias_gelu_kernel<T, true>), ew_grid(n / VecOf<T>::n), kEwBlock, 0, st, (const T*)x,
                           (const T*)bias, (T*)y, (T*)pre, n, cols);
    else
        hipLaunchKernelGGL((bias_gelu_kernel<T, false>), ew_grid(n), kEwBlock, 0, st, (const T*)x, (const T*)bias,
                           (T*)y, (T*)pre, n, cols);
    return launch_status("bias_gelu");
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

int dmlhip_binary_f16(int op, const void* a, const void* b, void* c, int ndim, const int64_t* shape,
                      const int64_t* a_strides, const int64_t* b_strides, void* stream) {
    return binary_impl<_Float16>(op, a, b, c, ndim, shape, a_strides, b_strides, stream);
}
int dmlhip_binary_f32(int op, const void* a, const void* b, void* c, int ndim, const int64_t* shape,
                      const int64_t* a_strides, const int64_t* b_strides, void* stream) {
    return binary_impl<float>(op, a, b, c, ndim, shape, a_strides, b_strides, stream);
}
int dmlhip_unary_f16(int op, const void* x, void* y, int64_t n, float param, void* stream) {
    return unary_impl<_Float16, false>(op, x, nullptr, y, n, param, stream);
}
int dmlhip_unary_f32(int op, const void* x, void* y, int64_t n, float param, void* stream) {
    return unary_impl<float, false>(op, x, nullptr, y, n, param, stream);
}
int dmlhip_unary_backward_f16(int op, const void* x, const void* dy, void* dx, int64_t n, float param,
                              void* stream) {
    return unary_impl<_Float16, true>(op, x, dy, dx, n, param, stream);
}
int dmlhip_unary_backward_f32(int op, const void* x, const void* dy, void* dx, int64_t n, float param,
                              void* stream) {
    return unary_impl<float, true>(op, x, dy, dx, n, param, stream);
}
int dmlhip_sum_f16(const void* const* inputs, int n_inputs, void* out, int64_t n, void* stream) {
    return sum_impl<_Float16>(inputs, n_inputs, out, n, stream);
}
int dmlhip_sum_f32(const void* const* inputs, int n_inputs, void* out, int64_t n, void* stream) {
    return sum_impl<float>(inputs, n_inputs, out, n, stream);
}
int dmlhip_bias_gelu_f16(const void* x, const void* bias, void* y, void* pre_out, int64_t rows, int64_t cols,
                         void* stream) {
    return bias_gelu_impl<_Float16>(x, bias, y, pre_out, rows, cols, stream);
}
int dmlhip_bias_gelu_f32(const void* x, const void* bias, void* y, void* pre_out, int64_t rows, int64_t cols,
                         void* stream) {
    return bias_gelu_impl<float>(x, bias, y, pre_out, rows, cols, stream);
}
int dmlhip_row_affine_f16(const void* a, const void* s, const void* t, const void* scale, void* y, int64_t rows,
                          int64_t cols, void* stream) {
    return row_affine_impl<_Float16>(a, s, t, scale, y, rows, cols, stream);
}
int dmlhip_row_affine_f32(const void* a, const void* s, const void* t, const void* scale, void* y, int64_t rows,
                          int64_t cols, void* stream) {
    return row_affine_impl<float>(a, s, t, scale, y, rows, cols, stream);
}
int dmlhip_cast(int src_dtype, int dst_dtype, const void* x, void* y, int64_t n, void* stream) {
    DML_REQUIRE((src_dtype == DMLHIP_F16 || src_dtype == DMLHIP_F32) &&
                    (dst_dtype == DMLHIP_F16 || dst_dtype == DMLHIP_F32),
                DMLHIP_ERR_ENUM, "cast: unknown dtype code");
    DML_REQUIRE(n >= 0, DMLHIP_ERR_SHAPE, "cast: negative size");
    if (n == 0) return 0;
    DML_REQUIRE(x && y, DMLHIP_ERR_NULL, "cast: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const unsigned g = ew_grid(n);
    if (src_dtype == DMLHIP_F16 && dst_dtype == DMLHIP_F32)
        hipLaunchKernelGGL((cast_kernel<_Float16, float>), g, kEwBlock, 0, st, (const _Float16*)x, (float*)y, n);
    else if (src_dtype == DMLHIP_F32 && dst_dtype == DMLHIP_F16)
        hipLaunchKernelGGL((cast_kernel<float, _Float16>), g, kEwBlock, 0, st, (const float*)x, (_Float16*)y, n);
    else if (src_dtype == DMLHIP_F16)
        hipLaunchKernelGGL((cast_kernel<_Float16, _Float16>), g, kEwBlock, 0, st, (const _Float16*)x, (_Float16*)y, n);
    else
        hipLaunchKernelGGL((cast_kernel<float, float>), g, kEwBlock, 0, st, (const float*)x, (float*)y, n);
    return launch_status("cast");
}

}  // extern "C"
