// Row-wise, HBM-bound nodes: Softmax and the fused LayerNormalization chain, forward and
// backward. One wavefront owns one row: the row is read once with 128-bit loads, kept in
// registers, reduced with DPP lane permutes, and written once. Rows that do not fit the
// register budget or are not 16-byte aligned take a workgroup-per-row fallback.
#include "common.h"
#include "lds_ops.h"

#include <mutex>

namespace dml {
namespace {

constexpr int kRowBlock = 256;                 // threads per workgroup
constexpr int kRowsPerBlock = kRowBlock / kWave;

template <typename T> struct ExpFn;
// fp16 I/O: the result is rounded to 11 bits, so the hardware exp2 is exact enough.
template <> struct ExpFn<_Float16> {
    __device__ __forceinline__ static float f(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }
    // exp(v - m) with the subtraction and the base change in one fma; m2 = m * log2(e)
    __device__ __forceinline__ static float prep(float m) { return m * 1.44269504088896340736f; }
    __device__ __forceinline__ static float shifted(float v, float m2) {
        return __builtin_amdgcn_exp2f(__builtin_fmaf(v, 1.44269504088896340736f, -m2));
    }
};
template <> struct ExpFn<float> {
    __device__ __forceinline__ static float f(float x) { return expf(x); }
    __device__ __forceinline__ static float prep(float m) { return m; }
    __device__ __forceinline__ static float shifted(float v, float m) { return expf(v - m); }
};

// ------------------------------------------------------------------ softmax, wave per row
// RPW rows per wavefront: the loads of all its rows are issued before the first reduction, so a wavefront keeps
// RPW * VPL 16-byte loads in flight per lane instead of VPL (short rows otherwise leave the memory system idle
// between a row's load and its store).
template <typename T, int VPL, int RPW>
__global__ __launch_bounds__(kRowBlock) void softmax_wave_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                 int64_t rows, int cols) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row0 = ((int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave) * RPW;
    if (row0 >= rows) return;
    const int nvec = cols / VN;

    V raw[RPW][VPL];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        const int64_t row = row0 + r < rows ? row0 + r : rows - 1;
        const V* xr = reinterpret_cast<const V*>(x + row * cols);
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int vi = lane + j * kWave;
            if (vi < nvec) raw[r][j] = __builtin_nontemporal_load(xr + vi);
        }
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
        if (row0 + r >= rows) break;
        float v[VPL][VN];
        float m = -INFINITY;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int vi = lane + j * kWave;
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                v[j][e] = vi < nvec ? to_f32(raw[r][j][e]) : -INFINITY;
                m = fmaxf(m, v[j][e]);
            }
        }
        m = ExpFn<T>::prep(wave_reduce<OpMax>(m));
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < VPL; ++j)
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                v[j][e] = ExpFn<T>::shifted(v[j][e], m);
                s += v[j][e];
            }
        s = wave_reduce<OpSum>(s);
        // one true division per row; each element is then scaled (fp16 results: the hardware reciprocal would do,
        // but the row total is shared by fp32 outputs that must hold 1e-5)
        const float inv = 1.0f / s;
        V* yr = reinterpret_cast<V*>(y + (row0 + r) * cols);
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int vi = lane + j * kWave;
            if (vi < nvec) {
                V t;
#pragma unroll
                for (int e = 0; e < VN; ++e) t[e] = from_f32<T>(v[j][e] * inv);
                __builtin_nontemporal_store(t, yr + vi);
            }
        }
    }
}

// ------------------------------------------------------------------ softmax, block per row
template <typename T>
__global__ __launch_bounds__(kRowBlock) void softmax_block_kernel(const T* __restrict__ x, T* __restrict__ y,
                                                                  int64_t cols) {
    __shared__ float scratch[kRowsPerBlock];
    const T* xr = x + (int64_t)blockIdx.x * cols;
    T* yr = y + (int64_t)blockIdx.x * cols;
    float m = -INFINITY;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) m = fmaxf(m, to_f32(xr[c]));
    m = block_reduce<OpMax, kRowsPerBlock>(m, scratch);
    float s = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) s += ExpFn<T>::f(to_f32(xr[c]) - m);
    s = block_reduce<OpSum, kRowsPerBlock>(s, scratch);
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock)
        yr[c] = from_f32<T>(ExpFn<T>::f(to_f32(xr[c]) - m) / s);
}

// ------------------------------------------------------------------ softmax backward
template <typename T, int VPL>
__global__ __launch_bounds__(kRowBlock) void softmax_bwd_wave_kernel(const T* __restrict__ y,
                                                                     const T* __restrict__ dy,
                                                                     T* __restrict__ dx, int64_t rows,
                                                                     int cols) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (row >= rows) return;
    const V* yr = reinterpret_cast<const V*>(y + row * cols);
    const V* gr = reinterpret_cast<const V*>(dy + row * cols);
    V* dr = reinterpret_cast<V*>(dx + row * cols);
    const int nvec = cols / VN;
    float yv[VPL][VN], pv[VPL][VN];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
            V a = __builtin_nontemporal_load(yr + vi);
            V b = __builtin_nontemporal_load(gr + vi);
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                yv[j][e] = to_f32(a[e]);
                pv[j][e] = yv[j][e] * to_f32(b[e]);
                s += pv[j][e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < VN; ++e) { yv[j][e] = 0.f; pv[j][e] = 0.f; }
        }
    }
    s = wave_reduce<OpSum>(s);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
            V t;
#pragma unroll
            for (int e = 0; e < VN; ++e) t[e] = from_f32<T>(pv[j][e] - yv[j][e] * s);
            __builtin_nontemporal_store(t, dr + vi);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kRowBlock) void softmax_bwd_block_kernel(const T* __restrict__ y,
                                                                      const T* __restrict__ dy,
                                                                      T* __restrict__ dx, int64_t cols) {
    __shared__ float scratch[kRowsPerBlock];
    const int64_t off = (int64_t)blockIdx.x * cols;
    float s = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) s += to_f32(y[off + c]) * to_f32(dy[off + c]);
    s = block_reduce<OpSum, kRowsPerBlock>(s, scratch);
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) {
        const float yy = to_f32(y[off + c]);
        dx[off + c] = from_f32<T>(yy * to_f32(dy[off + c]) - yy * s);
    }
}

// ------------------------------------------------------------------ layernorm forward, wave per row
template <typename T, int VPL>
__global__ __launch_bounds__(kRowBlock) void layernorm_wave_kernel(
    const T* __restrict__ x, const T* __restrict__ res, const T* __restrict__ gamma,
    const T* __restrict__ beta, T* __restrict__ y, T* __restrict__ sum_out, float* __restrict__ mean,
    float* __restrict__ rstd, int64_t rows, int cols, float eps) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kWave;
    if (row >= rows) return;
    const int nvec = cols / VN;
    const V* xr = reinterpret_cast<const V*>(x + row * cols);
    const V* rr = res ? reinterpret_cast<const V*>(res + row * cols) : nullptr;
    float v[VPL][VN];
    float s = 0.f;
    // gamma and beta are requested together with the row, not after the two reductions: their latency (they come from
    // L2 for all but the first rows) then runs under the row's
    const V* gv = reinterpret_cast<const V*>(gamma);
    const V* bv = reinterpret_cast<const V*>(beta);
    V gvec[VPL], bvec[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
            gvec[j] = gv[vi];
            bvec[j] = bv[vi];
        }
    }
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
            V t = xr[vi];
            if (rr) {
                V r = rr[vi];
                // the fused ONNXAdd rounds to the tensor dtype, as the separate node would
#pragma unroll
                for (int e = 0; e < VN; ++e) t[e] = from_f32<T>(to_f32(t[e]) + to_f32(r[e]));
                if (sum_out) reinterpret_cast<V*>(sum_out + row * cols)[vi] = t;
            } else if (sum_out) {
                reinterpret_cast<V*>(sum_out + row * cols)[vi] = t;
            }
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                v[j][e] = to_f32(t[e]);
                s += v[j][e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < VN; ++e) v[j][e] = 0.f;
        }
    }
    const float mu = wave_reduce<OpSum>(s) / (float)cols;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
#pragma unroll
            for (int e = 0; e < VN; ++e) {
                v[j][e] -= mu;
                q += v[j][e] * v[j][e];
            }
        }
    }
    const float var = wave_reduce<OpSum>(q) / (float)cols;
    const float inv = 1.0f / sqrtf(var + eps);
    if (lane == 0) {
        if (mean) mean[row] = mu;
        if (rstd) rstd[row] = inv;
    }
    V* yr = reinterpret_cast<V*>(y + row * cols);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
            const V g = gvec[j], b = bvec[j];
            V t;
#pragma unroll
            for (int e = 0; e < VN; ++e) t[e] = from_f32<T>(v[j][e] * inv * to_f32(g[e]) + to_f32(b[e]));
            if constexpr (sizeof(T) == 2) global_store_b128_through(yr + vi, t);
            else yr[vi] = t;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kRowBlock) void layernorm_block_kernel(
    const T* __restrict__ x, const T* __restrict__ res, const T* __restrict__ gamma,
    const T* __restrict__ beta, T* __restrict__ y, T* __restrict__ sum_out, float* __restrict__ mean,
    float* __restrict__ rstd, int64_t cols, float eps) {
    __shared__ float scratch[kRowsPerBlock];
    const int64_t off = (int64_t)blockIdx.x * cols;
    auto load = [&](int64_t c) -> float {
        if (res) return to_f32(from_f32<T>(to_f32(x[off + c]) + to_f32(res[off + c])));
        return to_f32(x[off + c]);
    };
    float s = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) {
        const float t = load(c);
        if (sum_out) sum_out[off + c] = from_f32<T>(t);
        s += t;
    }
    const float mu = block_reduce<OpSum, kRowsPerBlock>(s, scratch) / (float)cols;
    float q = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) {
        const float d = load(c) - mu;
        q += d * d;
    }
    const float var = block_reduce<OpSum, kRowsPerBlock>(q, scratch) / (float)cols;
    const float inv = 1.0f / sqrtf(var + eps);
    if (threadIdx.x == 0) {
        if (mean) mean[blockIdx.x] = mu;
        if (rstd) rstd[blockIdx.x] = inv;
    }
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock)
        y[off + c] = from_f32<T>((load(c) - mu) * inv * to_f32(gamma[c]) + to_f32(beta[c]));
}

// ------------------------------------------------------------------ layernorm backward
// Stage 1: a workgroup walks a slab of rows, one wavefront per row at a time. Each lane keeps
// the running column sums of dy*xhat (dgamma) and dy (dbeta) for the columns it owns; after the
// slab the four wavefronts are combined through LDS and one partial row per workgroup goes to the
// workspace. Stage 2 sums the partial rows. dx is written in stage 1.
template <typename T, int VPL>
__global__ __launch_bounds__(kRowBlock) void layernorm_bwd_wave_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dx,
    float* __restrict__ part, int64_t rows, int cols) {
    using V = typename VecOf<T>::type;
    constexpr int VN = VecOf<T>::n;
    extern __shared__ float lds[];  // [2][kRowsPerBlock][cols]
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nvec = cols / VN;
    float g[VPL][VN], accg[VPL][VN], accb[VPL][VN];
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        V t = {};
        if (vi < nvec) t = reinterpret_cast<const V*>(gamma)[vi];
#pragma unroll
        for (int e = 0; e < VN; ++e) { g[j][e] = to_f32(t[e]); accg[j][e] = 0.f; accb[j][e] = 0.f; }
    }
    // The rows of a wavefront are software-pipelined: the loads of its next row are issued before the current
    // row is reduced, so a workgroup's short chain of rows is not a chain of full memory round trips.
    const int64_t row_step = (int64_t)gridDim.x * kRowsPerBlock;
    int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + wave;
    V a_nxt[VPL], b_nxt[VPL];
    float mu_nxt = 0.f, inv_nxt = 0.f;
    auto fetch = [&](int64_t r) {
        mu_nxt = mean[r];
        inv_nxt = rstd[r];
        const V* xr = reinterpret_cast<const V*>(x + r * cols);
        const V* gr = reinterpret_cast<const V*>(dy + r * cols);
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int vi = lane + j * kWave;
            if (vi < nvec) { a_nxt[j] = xr[vi]; b_nxt[j] = gr[vi]; }
        }
    };
    if (row < rows) fetch(row);
    for (; row < rows; row += row_step) {
        const float mu = mu_nxt, inv = inv_nxt;
        V a_cur[VPL], b_cur[VPL];
#pragma unroll
        for (int j = 0; j < VPL; ++j) { a_cur[j] = a_nxt[j]; b_cur[j] = b_nxt[j]; }
        if (row + row_step < rows) fetch(row + row_step);
        float xh[VPL][VN], gd[VPL][VN];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int vi = lane + j * kWave;
            if (vi < nvec) {
                const V a = a_cur[j], b = b_cur[j];
#pragma unroll
                for (int e = 0; e < VN; ++e) {
                    const float d = to_f32(b[e]);
                    xh[j][e] = (to_f32(a[e]) - mu) * inv;
                    accg[j][e] += d * xh[j][e];
                    accb[j][e] += d;
                    gd[j][e] = d * g[j][e];
                    s1 += gd[j][e];
                    s2 += gd[j][e] * xh[j][e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < VN; ++e) { xh[j][e] = 0.f; gd[j][e] = 0.f; }
            }
        }
        s1 = wave_reduce<OpSum>(s1) / (float)cols;
        s2 = wave_reduce<OpSum>(s2) / (float)cols;
        V* dr = reinterpret_cast<V*>(dx + row * cols);
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
            const int vi = lane + j * kWave;
            if (vi < nvec) {
                V t;
#pragma unroll
                for (int e = 0; e < VN; ++e) t[e] = from_f32<T>((gd[j][e] - s1 - xh[j][e] * s2) * inv);
                if constexpr (sizeof(T) == 2) global_store_b128_through(dr + vi, t);
                else dr[vi] = t;
            }
        }
    }
    float* lg = lds + (size_t)wave * cols;
    float* lb = lds + (size_t)(kRowsPerBlock + wave) * cols;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        const int vi = lane + j * kWave;
        if (vi < nvec) {
#pragma unroll
            for (int e = 0; e < VN; ++e) { lg[vi * VN + e] = accg[j][e]; lb[vi * VN + e] = accb[j][e]; }
        }
    }
    __syncthreads();
    float* pg = part + (size_t)blockIdx.x * 2 * cols;
    for (int c = threadIdx.x; c < cols; c += kRowBlock) {
        float a = 0.f, b = 0.f;
#pragma unroll
        for (int w = 0; w < kRowsPerBlock; ++w) {
            a += lds[(size_t)w * cols + c];
            b += lds[(size_t)(kRowsPerBlock + w) * cols + c];
        }
        pg[c] = a;
        pg[cols + c] = b;
    }
}

// dgamma / dbeta: fp32, or (grads_f16) fp16 - the fp32 column sums rounded once as they are stored
void launch_ln_bwd_finish(const float* part, void* dgamma, void* dbeta, bool grads_f16, int nparts, int64_t cols,
                          hipStream_t st) {
    // partial rows are [dgamma | dbeta]: one launch finishes both
    const unsigned grid = (unsigned)ceil_div(2 * cols, kWave);
    if (grads_f16)
        hipLaunchKernelGGL((reduce_partials_kernel<OpSum, _Float16>), grid, 1024, 0, st, part, (_Float16*)dgamma, nparts,
                           2 * cols, 2 * cols, 0.f, 1.f, (_Float16*)dbeta, cols);
    else
        hipLaunchKernelGGL((reduce_partials_kernel<OpSum, float>), grid, 1024, 0, st, part, (float*)dgamma, nparts, 2 * cols,
                           2 * cols, 0.f, 1.f, (float*)dbeta, cols);
}

// fallback: dx, workgroup per row
template <typename T>
__global__ __launch_bounds__(kRowBlock) void layernorm_bwd_dx_block_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ mean,
    const float* __restrict__ rstd, const T* __restrict__ gamma, T* __restrict__ dx, int64_t cols) {
    __shared__ float scratch[kRowsPerBlock];
    const int64_t off = (int64_t)blockIdx.x * cols;
    const float mu = mean[blockIdx.x], inv = rstd[blockIdx.x];
    float s1 = 0.f, s2 = 0.f;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) {
        const float gd = to_f32(dy[off + c]) * to_f32(gamma[c]);
        const float xh = (to_f32(x[off + c]) - mu) * inv;
        s1 += gd;
        s2 += gd * xh;
    }
    s1 = block_reduce<OpSum, kRowsPerBlock>(s1, scratch) / (float)cols;
    s2 = block_reduce<OpSum, kRowsPerBlock>(s2, scratch) / (float)cols;
    for (int64_t c = threadIdx.x; c < cols; c += kRowBlock) {
        const float gd = to_f32(dy[off + c]) * to_f32(gamma[c]);
        const float xh = (to_f32(x[off + c]) - mu) * inv;
        dx[off + c] = from_f32<T>((gd - s1 - xh * s2) * inv);
    }
}

// fallback: dgamma/dbeta partials, thread per column over a slab of rows
template <typename T>
__global__ void layernorm_bwd_cols_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                          const float* __restrict__ mean, const float* __restrict__ rstd,
                                          float* __restrict__ part, int64_t rows, int64_t cols) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    float a = 0.f, b = 0.f;
    for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const float d = to_f32(dy[r * cols + c]);
        a += d * (to_f32(x[r * cols + c]) - mean[r]) * rstd[r];
        b += d;
    }
    part[(size_t)blockIdx.y * 2 * cols + c] = a;
    part[(size_t)blockIdx.y * 2 * cols + cols + c] = b;
}

// ------------------------------------------------------------------ host dispatch
int check_rows(const char* what, int64_t rows, int64_t cols) {
    DML_REQUIRE(rows >= 0 && cols >= 0, DMLHIP_ERR_SHAPE, "%s: negative extent (rows=%lld, cols=%lld)", what,
                (long long)rows, (long long)cols);
    DML_REQUIRE(rows <= (int64_t)2147483647 * kRowsPerBlock, DMLHIP_ERR_SHAPE, "%s: too many rows (%lld)", what,
                (long long)rows);
    DML_REQUIRE(cols == 0 || rows <= (INT64_MAX / 16) / cols, DMLHIP_ERR_SHAPE, "%s: rows*cols overflows", what);
    return 0;
}

template <typename T>
bool wave_path_ok(int64_t cols, int max_vpl) {
    constexpr int VN = VecOf<T>::n;
    return cols % VN == 0 && cols <= (int64_t)kWave * VN * max_vpl;
}

template <typename T>
int softmax_impl(const void* x, void* y, int64_t rows, int64_t cols, void* stream) {
    if (int e = check_rows("softmax", rows, cols)) return e;
    if (rows == 0 || cols == 0) return 0;
    DML_REQUIRE(x && y, DMLHIP_ERR_NULL, "softmax: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const T* xp = (const T*)x;
    T* yp = (T*)y;
    constexpr int VN = VecOf<T>::n;
    const unsigned grid = (unsigned)ceil_div(rows, kRowsPerBlock);
    if (wave_path_ok<T>(cols, 4) && aligned16(x) && aligned16(y)) {
        const int vpl = (int)ceil_div(cols, kWave * VN);
        // short rows and many of them: several rows per wavefront
        const bool many = rows >= 16384;
        const unsigned grid4 = (unsigned)ceil_div(rows, kRowsPerBlock * 4), grid2 = (unsigned)ceil_div(rows, kRowsPerBlock * 2);
        switch (vpl) {
            case 1:
                if (many) hipLaunchKernelGGL((softmax_wave_kernel<T, 1, 4>), grid4, kRowBlock, 0, st, xp, yp, rows, (int)cols);
                else hipLaunchKernelGGL((softmax_wave_kernel<T, 1, 1>), grid, kRowBlock, 0, st, xp, yp, rows, (int)cols);
                break;
            case 2:
                if (many) hipLaunchKernelGGL((softmax_wave_kernel<T, 2, 2>), grid2, kRowBlock, 0, st, xp, yp, rows, (int)cols);
                else hipLaunchKernelGGL((softmax_wave_kernel<T, 2, 1>), grid, kRowBlock, 0, st, xp, yp, rows, (int)cols);
                break;
            case 3: hipLaunchKernelGGL((softmax_wave_kernel<T, 3, 1>), grid, kRowBlock, 0, st, xp, yp, rows, (int)cols); break;
            default: hipLaunchKernelGGL((softmax_wave_kernel<T, 4, 1>), grid, kRowBlock, 0, st, xp, yp, rows, (int)cols); break;
        }
    } else {
        DML_REQUIRE(rows <= 2147483647, DMLHIP_ERR_SHAPE, "softmax: too many rows for the generic path");
        hipLaunchKernelGGL((softmax_block_kernel<T>), (unsigned)rows, kRowBlock, 0, st, xp, yp, cols);
    }
    return launch_status("softmax");
}

template <typename T>
int softmax_bwd_impl(const void* y, const void* dy, void* dx, int64_t rows, int64_t cols, void* stream) {
    if (int e = check_rows("softmax_backward", rows, cols)) return e;
    if (rows == 0 || cols == 0) return 0;
    DML_REQUIRE(y && dy && dx, DMLHIP_ERR_NULL, "softmax_backward: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const T* yp = (const T*)y;
    const T* gp = (const T*)dy;
    T* dp = (T*)dx;
    constexpr int VN = VecOf<T>::n;
    const unsigned grid = (unsigned)ceil_div(rows, kRowsPerBlock);
    if (wave_path_ok<T>(cols, 4) && aligned16(y) && aligned16(dy) && aligned16(dx)) {
        const int vpl = (int)ceil_div(cols, kWave * VN);
        switch (vpl) {
            case 1: hipLaunchKernelGGL((softmax_bwd_wave_kernel<T, 1>), grid, kRowBlock, 0, st, yp, gp, dp, rows, (int)cols); break;
            case 2: hipLaunchKernelGGL((softmax_bwd_wave_kernel<T, 2>), grid, kRowBlock, 0, st, yp, gp, dp, rows, (int)cols); break;
            case 3: hipLaunchKernelGGL((softmax_bwd_wave_kernel<T, 3>), grid, kRowBlock, 0, st, yp, gp, dp, rows, (int)cols); break;
            default: hipLaunchKernelGGL((softmax_bwd_wave_kernel<T, 4>), grid, kRowBlock, 0, st, yp, gp, dp, rows, (int)cols); break;
        }
    } else {
        DML_REQUIRE(rows <= 2147483647, DMLHIP_ERR_SHAPE, "softmax_backward: too many rows for the generic path");
        hipLaunchKernelGGL((softmax_bwd_block_kernel<T>), (unsigned)rows, kRowBlock, 0, st, yp, gp, dp, cols);
    }
    return launch_status("softmax_backward");
}

template <typename T>
int layernorm_impl(const void* x, const void* residual, const void* gamma, const void* beta, void* y,
                   void* sum_out, float* mean, float* rstd, int64_t rows, int64_t cols, float eps, void* stream) {
    if (int e = check_rows("layernorm", rows, cols)) return e;
    DML_REQUIRE(eps >= 0.f, DMLHIP_ERR_SHAPE, "layernorm: negative epsilon");
    if (rows == 0 || cols == 0) return 0;
    DML_REQUIRE(x && gamma && beta && y, DMLHIP_ERR_NULL, "layernorm: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    const T *xp = (const T*)x, *rp = (const T*)residual, *gp = (const T*)gamma, *bp = (const T*)beta;
    T *yp = (T*)y, *sp = (T*)sum_out;
    constexpr int VN = VecOf<T>::n;
    const bool al = aligned16(x) && aligned16(y) && aligned16(gamma) && aligned16(beta) &&
                    (!residual || aligned16(residual)) && (!sum_out || aligned16(sum_out));
    if (wave_path_ok<T>(cols, 4) && al) {
        const unsigned grid = (unsigned)ceil_div(rows, kRowsPerBlock);
        const int vpl = (int)ceil_div(cols, kWave * VN);
#define DML_LN_LAUNCH(V) hipLaunchKernelGGL((layernorm_wave_kernel<T, V>), grid, kRowBlock, 0, st, xp, rp, gp, bp, yp, sp, mean, rstd, rows, (int)cols, eps)
        switch (vpl) {
            case 1: DML_LN_LAUNCH(1); break;
            case 2: DML_LN_LAUNCH(2); break;
            case 3: DML_LN_LAUNCH(3); break;
            default: DML_LN_LAUNCH(4); break;
        }
#undef DML_LN_LAUNCH
    } else {
        DML_REQUIRE(rows <= 2147483647, DMLHIP_ERR_SHAPE, "layernorm: too many rows for the generic path");
        hipLaunchKernelGGL((layernorm_block_kernel<T>), (unsigned)rows, kRowBlock, 0, st, xp, rp, gp, bp, yp, sp, mean,
                           rstd, cols, eps);
    }
    return launch_status("layernorm");
}

int ln_bwd_parts(int64_t rows) {
    int64_t p = ceil_div(rows, kRowsPerBlock * 4);
    if (p < 1) p = 1;
    if (p > 512) p = 512;
    return (int)p;
}

template <typename T>
int layernorm_bwd_impl(const void* dy, const void* x, const float* mean, const float* rstd, const void* gamma,
                       void* dx, void* dgamma, void* dbeta, int64_t rows, int64_t cols, void* workspace,
                       size_t workspace_bytes, void* stream, bool grads_f16 = false) {
    if (int e = check_rows("layernorm_backward", rows, cols)) return e;
    if (cols == 0) return 0;
    DML_REQUIRE(dgamma && dbeta, DMLHIP_ERR_NULL, "layernorm_backward: NULL gradient pointer");
    hipStream_t st = (hipStream_t)stream;
    if (rows == 0) {
        launch_ln_bwd_finish(nullptr, dgamma, dbeta, grads_f16, 0, cols, st);
        return launch_status("layernorm_backward");
    }
    DML_REQUIRE(dy && x && mean && rstd && gamma && dx, DMLHIP_ERR_NULL, "layernorm_backward: NULL tensor pointer");
    DML_REQUIRE(cols <= 2147483647, DMLHIP_ERR_SHAPE, "layernorm_backward: cols too large");
    const size_t need = dmlhip_layernorm_backward_workspace_bytes(rows, cols);
    DML_REQUIRE(workspace && workspace_bytes >= need, DMLHIP_ERR_WORKSPACE,
                "layernorm_backward: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    const T *gp = (const T*)dy, *xp = (const T*)x, *gm = (const T*)gamma;
    T* dp = (T*)dx;
    float* part = (float*)workspace;
    const int parts = ln_bwd_parts(rows);
    constexpr int VN = VecOf<T>::n;
    const bool al = aligned16(dy) && aligned16(x) && aligned16(gamma) && aligned16(dx);
    const size_t lds = (size_t)2 * kRowsPerBlock * cols * sizeof(float);
    if (wave_path_ok<T>(cols, 4) && al && lds <= 64 * 1024) {
        const int vpl = (int)ceil_div(cols, kWave * VN);
#define DML_LNB_LAUNCH(V) hipLaunchKernelGGL((layernorm_bwd_wave_kernel<T, V>), (unsigned)parts, kRowBlock, lds, st, gp, xp, mean, rstd, gm, dp, part, rows, (int)cols)
        switch (vpl) {
            case 1: DML_LNB_LAUNCH(1); break;
            case 2: DML_LNB_LAUNCH(2); break;
            case 3: DML_LNB_LAUNCH(3); break;
            default: DML_LNB_LAUNCH(4); break;
        }
#undef DML_LNB_LAUNCH
    } else {
        DML_REQUIRE(rows <= 2147483647, DMLHIP_ERR_SHAPE, "layernorm_backward: too many rows for the generic path");
        hipLaunchKernelGGL((layernorm_bwd_dx_block_kernel<T>), (unsigned)rows, kRowBlock, 0, st, gp, xp, mean, rstd, gm,
                           dp, cols);
        if (int e = launch_status("layernorm_backward(dx)")) return e;
        dim3 grid((unsigned)ceil_div(cols, 256), (unsigned)parts);
        hipLaunchKernelGGL((layernorm_bwd_cols_kernel<T>), grid, 256, 0, st, gp, xp, mean, rstd, part, rows, cols);
    }
    if (int e = launch_status("layernorm_backward(stage 1)")) return e;
    launch_ln_bwd_finish(part, dgamma, dbeta, grads_f16, parts, cols, st);
    return launch_status("layernorm_backward(stage 2)");
}

// ------------------------------------------------------------------ scratch for callers that cannot allocate
// A fixed-size device array that stands in for the caller's workspace in dmlhip_layernorm_backward_noalloc_f16.
// One copy per GPU, resident until the process ends. In host code the array's name is only a handle for
// hipGetSymbolAddress: the device address is looked up once per device and that pointer is what kernels get.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// Device address of the current device's copy of `scratch`.
int static_scratch(void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        set_error("layernorm_backward_noalloc: hipGetDevice failed: %s", hipGetErrorString(e));
        return (int)e;
    }
    DML_REQUIRE(dev >= 0 && dev < kMaxDevices, DMLHIP_ERR_UNSUPPORTED,
                "layernorm_backward_noalloc: device index %d beyond the %d devices the scratch table holds", dev,
                kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error("layernorm_backward_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

int dmlhip_softmax_f16(const void* x, void* y, int64_t rows, int64_t cols, void* stream) {
    return softmax_impl<_Float16>(x, y, rows, cols, stream);
}
int dmlhip_softmax_f32(const void* x, void* y, int64_t rows, int64_t cols, void* stream) {
    return softmax_impl<float>(x, y, rows, cols, stream);
}
int dmlhip_softmax_backward_f16(const void* y, const void* dy, void* dx, int64_t rows, int64_t cols, void* stream) {
    return softmax_bwd_impl<_Float16>(y, dy, dx, rows, cols, stream);
}
int dmlhip_softmax_backward_f32(const void* y, const void* dy, void* dx, int64_t rows, int64_t cols, void* stream) {
    return softmax_bwd_impl<float>(y, dy, dx, rows, cols, stream);
}
int dmlhip_layernorm_f16(const void* x, const void* residual, const void* gamma, const void* beta, void* y,
                         void* sum_out, float* mean, float* rstd, int64_t rows, int64_t cols, float eps,
                         void* stream) {
    return layernorm_impl<_Float16>(x, residual, gamma, beta, y, sum_out, mean, rstd, rows, cols, eps, stream);
}
int dmlhip_layernorm_f32(const void* x, const void* residual, const void* gamma, const void* beta, void* y,
                         void* sum_out, float* mean, float* rstd, int64_t rows, int64_t cols, float eps,
                         void* stream) {
    return layernorm_impl<float>(x, residual, gamma, beta, y, sum_out, mean, rstd, rows, cols, eps, stream);
}
size_t dmlhip_layernorm_backward_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    return (size_t)ln_bwd_parts(rows) * 2 * (size_t)cols * sizeof(float);
}
int dmlhip_layernorm_backward_f16(const void* dy, const void* x, const float* mean, const float* rstd,
                                  const void* gamma, void* dx, float* dgamma, float* dbeta, int64_t rows,
                                  int64_t cols, void* workspace, size_t workspace_bytes, void* stream) {
    return layernorm_bwd_impl<_Float16>(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, rows, cols, workspace,
                                        workspace_bytes, stream);
}
int dmlhip_layernorm_backward_f32(const void* dy, const void* x, const float* mean, const float* rstd,
                                  const void* gamma, void* dx, float* dgamma, float* dbeta, int64_t rows,
                                  int64_t cols, void* workspace, size_t workspace_bytes, void* stream) {
    return layernorm_bwd_impl<float>(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, rows, cols, workspace,
                                     workspace_bytes, stream);
}
int dmlhip_layernorm_backward_grads_f16(const void* dy, const void* x, const float* mean, const float* rstd,
                                        const void* gamma, void* dx, void* dgamma, void* dbeta, int grad_dtype,
                                        int64_t rows, int64_t cols, void* workspace, size_t workspace_bytes,
                                        void* stream) {
    DML_REQUIRE(grad_dtype == DMLHIP_F16 || grad_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM,
                "layernorm_backward_grads: bad grad_dtype %d", grad_dtype);
    return layernorm_bwd_impl<_Float16>(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, rows, cols, workspace,
                                        workspace_bytes, stream, grad_dtype == DMLHIP_F16);
}
size_t dmlhip_layernorm_backward_noalloc_max_bytes(void) { return kStaticScratchBytes; }
int dmlhip_layernorm_backward_noalloc_f16(const void* dy, const void* x, const float* mean, const float* rstd,
                                          const void* gamma, void* dx, float* dgamma, float* dbeta, int64_t rows,
                                          int64_t cols, void* stream) {
    if (int e = check_rows("layernorm_backward_noalloc", rows, cols)) return e;
    const size_t need = dmlhip_layernorm_backward_workspace_bytes(rows, cols);
    DML_REQUIRE(need <= kStaticScratchBytes, DMLHIP_ERR_WORKSPACE,
                "layernorm_backward_noalloc: %lld x %lld needs %zu bytes of scratch, the built-in buffer holds %zu; "
                "use dmlhip_layernorm_backward_f16 with a workspace", (long long)rows, (long long)cols, need,
                kStaticScratchBytes);
    void* ws = nullptr;
    if (int e = static_scratch(&ws)) return e;
    // every partial row that stage 2 reads is written by stage 1 of the same call: nothing has to start at zero
    return layernorm_bwd_impl<_Float16>(dy, x, mean, rstd, gamma, dx, dgamma, dbeta, rows, cols, ws,
                                        kStaticScratchBytes, stream);
}

}  // extern "C"
