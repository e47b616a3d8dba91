// Reductions over one (collapsed) axis of a dense tensor viewed as [outer, r, inner]:
// ReduceSum / ReduceMax / ReduceMin / ReduceMean and GlobalAveragePool. fp32 accumulation.
//   inner == 1 : each row of r elements is reduced by a wavefront (short rows) or a workgroup.
//   inner  > 1 : column reduction; lanes run along `inner` (coalesced, 128-bit when aligned),
//                four wavefronts stride over r, and r is split across workgroups when
//                outer*inner alone cannot fill the chip; partial results go through a caller
//                workspace and a second, tiny pass, so the result is deterministic.
#include "common.h"

namespace dml {
namespace {

constexpr int kRedBlock = 256;
constexpr int kRedWaves = kRedBlock / kWave;

template <int OP> struct RedOp;
template <> struct RedOp<DMLHIP_RSUM> { using op = OpSum; __device__ __host__ static float init() { return 0.f; } };
template <> struct RedOp<DMLHIP_RMEAN> { using op = OpSum; __device__ __host__ static float init() { return 0.f; } };
template <> struct RedOp<DMLHIP_RMAX> { using op = OpMax; __device__ __host__ static float init() { return -INFINITY; } };
template <> struct RedOp<DMLHIP_RMIN> { using op = OpMin; __device__ __host__ static float init() { return INFINITY; } };

// ---------------------------------------------------------------- inner == 1
template <typename TIn, typename TOut, int OP, bool WAVE>
__global__ __launch_bounds__(kRedBlock) void row_reduce_kernel(const TIn* __restrict__ x, TOut* __restrict__ y,
                                                               int64_t rows, int64_t r, float scale) {
    using Op = typename RedOp<OP>::op;
    __shared__ float scratch[kRedWaves];
    const int64_t row = WAVE ? (int64_t)blockIdx.x * kRedWaves + threadIdx.x / kWave : (int64_t)blockIdx.x;
    const int tid = WAVE ? (threadIdx.x & (kWave - 1)) : threadIdx.x;
    const int nth = WAVE ? kWave : kRedBlock;
    float a0 = RedOp<OP>::init(), a1 = a0, a2 = a0, a3 = a0;
    if (row < rows) {
        const TIn* xr = x + row * r;
        int64_t c = tid;
        for (; c + 3 * nth < r; c += 4 * nth) {
            a0 = Op::f(a0, to_f32(xr[c]));
            a1 = Op::f(a1, to_f32(xr[c + nth]));
            a2 = Op::f(a2, to_f32(xr[c + 2 * nth]));
            a3 = Op::f(a3, to_f32(xr[c + 3 * nth]));
        }
        for (; c < r; c += nth) a0 = Op::f(a0, to_f32(xr[c]));
    }
    float a = Op::f(Op::f(a0, a1), Op::f(a2, a3));
    if constexpr (WAVE) {
        a = wave_reduce<Op>(a);
    } else {
        a = block_reduce<Op, kRedWaves>(a, scratch);
    }
    if (row < rows && tid == 0) y[row] = from_f32<TOut>(a * scale);
}

// y[row] = sum_j a[row, j] * b[row, j]: a Mul whose only reader is a ReduceSum over the trailing axes, without the
// product tensor (the gradient of a per-row factor such as a squeeze-excite gate)
template <typename T, bool WAVE>
__global__ __launch_bounds__(kRedBlock) void row_dot_kernel(const T* __restrict__ a, const T* __restrict__ b,
                                                            T* __restrict__ y, int64_t rows, int64_t r) {
    __shared__ float scratch[kRedWaves];
    const int64_t row = WAVE ? (int64_t)blockIdx.x * kRedWaves + threadIdx.x / kWave : (int64_t)blockIdx.x;
    const int tid = WAVE ? (threadIdx.x & (kWave - 1)) : threadIdx.x;
    const int nth = WAVE ? kWave : kRedBlock;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (row < rows) {
        const T* ar = a + row * r;
        const T* br = b + row * r;
        int64_t c = tid;
        for (; c + 3 * nth < r; c += 4 * nth) {
            a0 += to_f32(ar[c]) * to_f32(br[c]);
            a1 += to_f32(ar[c + nth]) * to_f32(br[c + nth]);
            a2 += to_f32(ar[c + 2 * nth]) * to_f32(br[c + 2 * nth]);
            a3 += to_f32(ar[c + 3 * nth]) * to_f32(br[c + 3 * nth]);
        }
        for (; c < r; c += nth) a0 += to_f32(ar[c]) * to_f32(br[c]);
    }
    float s = (a0 + a1) + (a2 + a3);
    if constexpr (WAVE) {
        s = wave_reduce<OpSum>(s);
    } else {
        s = block_reduce<OpSum, kRedWaves>(s, scratch);
    }
    if (row < rows && tid == 0) y[row] = from_f32<T>(s);
}

template <typename T>
int row_dot_impl(const void* a, const void* b, void* y, int64_t rows, int64_t r, void* stream) {
    DML_REQUIRE(rows >= 0 && r >= 0, DMLHIP_ERR_SHAPE, "row_dot: negative extent");
    DML_REQUIRE(rows <= 2147483647LL, DMLHIP_ERR_SHAPE, "row_dot: too many rows");
    DML_REQUIRE(r == 0 || rows <= (INT64_MAX / 16) / r, DMLHIP_ERR_SHAPE, "row_dot: size overflows");
    if (rows == 0) return 0;
    DML_REQUIRE(y && (r == 0 || (a && b)), DMLHIP_ERR_NULL, "row_dot: NULL tensor pointer");
    hipStream_t st = (hipStream_t)stream;
    if (r <= 2048)
        hipLaunchKernelGGL((row_dot_kernel<T, true>), (unsigned)ceil_div(rows, kRedWaves), kRedBlock, 0, st, (const T*)a,
                           (const T*)b, (T*)y, rows, r);
    else
        hipLaunchKernelGGL((row_dot_kernel<T, false>), (unsigned)rows, kRedBlock, 0, st, (const T*)a, (const T*)b, (T*)y,
                           rows, r);
    return launch_status("row_dot");
}

// ---------------------------------------------------------------- inner > 1
// grid: x = column tiles, y = outer, z = splits of r. V = elements per lane along inner.
template <typename TIn, typename TOut, int OP, int V>
__global__ __launch_bounds__(kRedBlock) void col_reduce_kernel(const TIn* __restrict__ x, TOut* __restrict__ y,
                                                               int64_t outer, int64_t r, int64_t inner,
                                                               int64_t r_per_split, float scale) {
    using Op = typename RedOp<OP>::op;
    typedef TIn vec_t __attribute__((ext_vector_type(V)));
    __shared__ float lds[kRedWaves][kWave * V];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t col = ((int64_t)blockIdx.x * kWave + lane) * V;
    const int64_t o = blockIdx.y;
    const int64_t r0 = (int64_t)blockIdx.z * r_per_split;
    const int64_t r1 = r0 + r_per_split < r ? r0 + r_per_split : r;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = RedOp<OP>::init();
    if (col < inner) {
        const TIn* base = x + o * r * inner + col;
        for (int64_t i = r0 + wave; i < r1; i += kRedWaves) {
            if constexpr (V > 1) {
                vec_t v = *reinterpret_cast<const vec_t*>(base + i * inner);
#pragma unroll
                for (int e = 0; e < V; ++e) acc[e] = Op::f(acc[e], to_f32(v[e]));
            } else {
                acc[0] = Op::f(acc[0], to_f32(base[i * inner]));
            }
        }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) lds[wave][lane * V + e] = acc[e];
    __syncthreads();
    if (wave == 0 && col < inner) {
        TOut* out = y + ((int64_t)blockIdx.z * outer + o) * inner + col;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            float a = lds[0][lane * V + e];
#pragma unroll
            for (int w = 1; w < kRedWaves; ++w) a = Op::f(a, lds[w][lane * V + e]);
            out[e] = from_f32<TOut>(a * scale);
        }
    }
}

struct ColPlan {
    int v;           // elements per lane
    int64_t tiles;   // column tiles
    int64_t splits;  // splits of r
    int64_t r_per_split;
};

template <typename TIn>
ColPlan plan_cols(const void* x, int64_t outer, int64_t r, int64_t inner) {
    ColPlan p;
    constexpr int VN = VecOf<TIn>::n;
    p.v = (inner % VN == 0 && aligned16(x)) ? VN : 1;
    p.tiles = ceil_div(inner, (int64_t)kWave * p.v);
    const int64_t blocks = p.tiles * outer;
    int64_t splits = 1;
    if (blocks < 1024) {
        splits = ceil_div(1024, blocks);
        const int64_t max_splits = ceil_div(r, 4 * kRedWaves);  // at least 16 rows per workgroup
        if (splits > max_splits) splits = max_splits;
        if (splits < 1) splits = 1;
        if (splits > 65535) splits = 65535;
    }
    p.r_per_split = r > 0 ? ceil_div(r, splits) : 1;
    p.splits = r > 0 ? ceil_div(r, p.r_per_split) : 1;
    return p;
}

template <typename TIn, typename TOut, int OP>
int col_launch(const TIn* x, TOut* y, int64_t outer, int64_t r, int64_t inner, int v, int64_t tiles, int64_t splits,
               int64_t r_per_split, float scale, hipStream_t st) {
    dim3 grid((unsigned)tiles, (unsigned)outer, (unsigned)splits);
    constexpr int VN = VecOf<TIn>::n;
    if (v == VN)
        hipLaunchKernelGGL((col_reduce_kernel<TIn, TOut, OP, VN>), grid, kRedBlock, 0, st, x, y, outer, r, inner,
                           r_per_split, scale);
    else
        hipLaunchKernelGGL((col_reduce_kernel<TIn, TOut, OP, 1>), grid, kRedBlock, 0, st, x, y, outer, r, inner,
                           r_per_split, scale);
    return launch_status("reduce(columns)");
}

template <typename TIn, typename TOut, int OP>
int reduce_typed(const TIn* x, TOut* y, int64_t outer, int64_t r, int64_t inner, void* ws, size_t ws_bytes,
                 hipStream_t st) {
    const float scale = OP == DMLHIP_RMEAN ? 1.0f / (float)r : 1.0f;
    if (inner == 1) {
        if (r <= 2048) {
            hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, OP, true>), (unsigned)ceil_div(outer, kRedWaves), kRedBlock,
                               0, st, x, y, outer, r, scale);
        } else {
            hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, OP, false>), (unsigned)outer, kRedBlock, 0, st, x, y,
                               outer, r, scale);
        }
        return launch_status("reduce(rows)");
    }
    const ColPlan p = plan_cols<TIn>(x, outer, r, inner);
    if (p.splits == 1) return col_launch<TIn, TOut, OP>(x, y, outer, r, inner, p.v, p.tiles, 1, r, scale, st);
    const size_t need = (size_t)p.splits * outer * inner * sizeof(float);
    DML_REQUIRE(ws && ws_bytes >= need, DMLHIP_ERR_WORKSPACE, "reduce: workspace of %zu bytes needed, %zu given", need,
                ws_bytes);
    float* part = (float*)ws;
    if (int e = col_launch<TIn, float, OP>(x, part, outer, r, inner, p.v, p.tiles, p.splits, p.r_per_split, 1.0f, st))
        return e;
    // second pass over the fp32 partials [splits, outer*inner] -> TOut, same op, then the scale
    const int64_t inner2 = outer * inner;
    using Op = typename RedOp<OP>::op;
    hipLaunchKernelGGL((reduce_partials_kernel<Op, TOut>), (unsigned)ceil_div(inner2, kWave), 1024, 0, st,
                       (const float*)part, y, (int)p.splits, inner2, inner2, RedOp<OP>::init(), scale, (TOut*)nullptr,
                       (int64_t)0);
    return launch_status("reduce(partials)");
}

// ---------------------------------------------------------------- several column sums in one launch pair
// y_t[c] = sum_r x_t[r, c] for up to DMLHIP_MULTI_MAX independent row-major matrices (the bias gradients of a
// backward pass: each alone is a latency-bound pair of tiny launches). grid: x = column tiles of the widest
// matrix, y = row splits, z = matrix; fp32 partials [split][cols] per matrix, then one finishing launch.
struct MultiRedArgs {
    const void* x[DMLHIP_MULTI_MAX];
    void* y[DMLHIP_MULTI_MAX];
    long long rows[DMLHIP_MULTI_MAX], cols[DMLHIP_MULTI_MAX], part_off[DMLHIP_MULTI_MAX], rows_per_split[DMLHIP_MULTI_MAX];
    int splits[DMLHIP_MULTI_MAX];
    int count;
};

template <typename TIn>
__global__ __launch_bounds__(kRedBlock) void multi_col_sum_kernel(const MultiRedArgs a, float* __restrict__ part) {
    constexpr int V = VecOf<TIn>::n;
    typedef typename VecOf<TIn>::type vec_t;
    __shared__ float lds[kRedWaves][kWave * V];
    const int t = blockIdx.z;
    const long long cols = a.cols[t];
    if ((int)blockIdx.y >= a.splits[t] || (long long)blockIdx.x * kWave * V >= cols) return;  // whole workgroup leaves
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const long long col = ((long long)blockIdx.x * kWave + lane) * V;
    const long long r0 = (long long)blockIdx.y * a.rows_per_split[t];
    const long long r1 = r0 + a.rows_per_split[t] < a.rows[t] ? r0 + a.rows_per_split[t] : a.rows[t];
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = 0.f;
    if (col < cols) {
        const TIn* base = reinterpret_cast<const TIn*>(a.x[t]) + col;
        long long i = r0 + wave;
        constexpr int U = 8;  // independent 16-byte loads in flight per lane
        for (; i + (U - 1) * kRedWaves < r1; i += U * kRedWaves) {
            vec_t v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) v[u] = *reinterpret_cast<const vec_t*>(base + (i + u * kRedWaves) * cols);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float s = 0.f;
#pragma unroll
                for (int u = 0; u < U; ++u) s += to_f32(v[u][e]);
                acc[e] += s;
            }
        }
        for (; i < r1; i += kRedWaves) {
            const vec_t v = *reinterpret_cast<const vec_t*>(base + i * cols);
#pragma unroll
            for (int e = 0; e < V; ++e) acc[e] += to_f32(v[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) lds[wave][lane * V + e] = acc[e];
    __syncthreads();
    if (wave == 0 && col < cols) {
        float* out = part + a.part_off[t] + (long long)blockIdx.y * cols + col;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            float s = lds[0][lane * V + e];
#pragma unroll
            for (int w = 1; w < kRedWaves; ++w) s += lds[w][lane * V + e];
            out[e] = s;
        }
    }
}

template <typename TOut>
__global__ __launch_bounds__(1024) void multi_partials_kernel(const MultiRedArgs a, const float* __restrict__ part) {
    __shared__ float lds[16][kWave];
    const int t = blockIdx.y;
    const long long cols = a.cols[t];
    if ((long long)blockIdx.x * kWave >= cols) return;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const long long c = (long long)blockIdx.x * kWave + lane;
    float s = 0.f;
    if (c < cols) {
        const float* base = part + a.part_off[t] + c;
        for (int p = wave; p < a.splits[t]; p += 16) s += base[(long long)p * cols];
    }
    lds[wave][lane] = s;
    __syncthreads();
    if (wave == 0 && c < cols) {
        float v = lds[0][lane];
#pragma unroll
        for (int w = 1; w < 16; ++w) v += lds[w][lane];
        reinterpret_cast<TOut*>(a.y[t])[c] = from_f32<TOut>(v);
    }
}

int multi_plan(int count, const int64_t* rows, const int64_t* cols, MultiRedArgs& a, long long& part_floats, int& max_splits,
               long long& max_cols) {
    DML_REQUIRE(count >= 1 && count <= DMLHIP_MULTI_MAX, DMLHIP_ERR_SHAPE, "reduce_sum_multi: count %d outside 1..%d", count,
                DMLHIP_MULTI_MAX);
    DML_REQUIRE(rows && cols, DMLHIP_ERR_NULL, "reduce_sum_multi: NULL extents");
    part_floats = 0;
    max_splits = 1;
    max_cols = 0;
    a.count = count;
    for (int t = 0; t < count; ++t) {
        DML_REQUIRE(rows[t] >= 0 && cols[t] >= 0 && rows[t] <= (1LL << 40) && cols[t] <= (1LL << 31), DMLHIP_ERR_SHAPE,
                    "reduce_sum_multi: bad extent");
        a.rows[t] = rows[t];
        a.cols[t] = cols[t];
        long long splits = ceil_div(rows[t] > 0 ? rows[t] : 1, 128);   // 128 rows (32 per wavefront) per workgroup
        if (splits > 256) splits = 256;
        a.rows_per_split[t] = ceil_div(rows[t] > 0 ? rows[t] : 1, splits);
        a.splits[t] = (int)ceil_div(rows[t] > 0 ? rows[t] : 1, a.rows_per_split[t]);
        a.part_off[t] = part_floats;
        part_floats += (long long)a.splits[t] * cols[t];
        if (a.splits[t] > max_splits) max_splits = a.splits[t];
        if (cols[t] > max_cols) max_cols = cols[t];
    }
    return 0;
}

template <typename TIn>
int reduce_sum_multi_impl(int count, const void* const* x, void* const* y, int out_dtype, const int64_t* rows,
                          const int64_t* cols, void* ws, size_t ws_bytes, void* stream) {
    DML_REQUIRE(out_dtype == DMLHIP_F16 || out_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM, "reduce_sum_multi: unknown out_dtype");
    DML_REQUIRE(x && y, DMLHIP_ERR_NULL, "reduce_sum_multi: NULL pointer table");
    MultiRedArgs a = {};
    long long part_floats, max_cols;
    int max_splits;
    if (int e = multi_plan(count, rows, cols, a, part_floats, max_splits, max_cols)) return e;
    constexpr int V = VecOf<TIn>::n;
    for (int t = 0; t < count; ++t) {
        DML_REQUIRE(y[t] && (x[t] || rows[t] == 0 || cols[t] == 0), DMLHIP_ERR_NULL, "reduce_sum_multi: NULL tensor %d", t);
        DML_REQUIRE(cols[t] % V == 0 && aligned16(x[t]), DMLHIP_ERR_ALIGN,
                    "reduce_sum_multi: matrix %d needs 16-byte aligned rows (cols %% %d == 0)", t, V);
        a.x[t] = x[t];
        a.y[t] = y[t];
    }
    if (max_cols == 0) return 0;
    DML_REQUIRE(ws && ws_bytes >= (size_t)part_floats * sizeof(float), DMLHIP_ERR_WORKSPACE,
                "reduce_sum_multi: workspace of %zu bytes needed, %zu given", (size_t)part_floats * sizeof(float), ws_bytes);
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL((multi_col_sum_kernel<TIn>), dim3((unsigned)ceil_div(max_cols, (int64_t)kWave * V), (unsigned)max_splits,
                                                         (unsigned)count),
                       kRedBlock, 0, st, a, (float*)ws);
    if (int e = launch_status("reduce_sum_multi(stage 1)")) return e;
    const dim3 g2((unsigned)ceil_div(max_cols, kWave), (unsigned)count);
    if (out_dtype == DMLHIP_F32) hipLaunchKernelGGL((multi_partials_kernel<float>), g2, 1024, 0, st, a, (const float*)ws);
    else hipLaunchKernelGGL((multi_partials_kernel<_Float16>), g2, 1024, 0, st, a, (const float*)ws);
    return launch_status("reduce_sum_multi(stage 2)");
}

template <typename TIn>
int reduce_impl(int op, const void* x, void* y, int out_dtype, int64_t outer, int64_t r, int64_t inner, void* ws,
                size_t ws_bytes, void* stream) {
    DML_REQUIRE(op >= DMLHIP_RSUM && op <= DMLHIP_RMEAN, DMLHIP_ERR_ENUM, "reduce: unknown op %d", op);
    DML_REQUIRE(out_dtype == DMLHIP_F16 || out_dtype == DMLHIP_F32, DMLHIP_ERR_ENUM, "reduce: unknown out_dtype");
    DML_REQUIRE(outer >= 0 && r >= 0 && inner >= 0, DMLHIP_ERR_SHAPE, "reduce: negative extent");
    DML_REQUIRE(outer <= 2147483647 && (inner == 1 || outer <= 65535), DMLHIP_ERR_SHAPE,
                "reduce: outer extent %lld too large", (long long)outer);
    DML_REQUIRE(r == 0 || inner == 0 || outer <= (INT64_MAX / 16) / r / inner, DMLHIP_ERR_SHAPE,
                "reduce: size overflows");
    if (outer == 0 || inner == 0) return 0;
    DML_REQUIRE(r > 0 || op == DMLHIP_RSUM, DMLHIP_ERR_SHAPE, "reduce: empty axis only defined for sum");
    DML_REQUIRE(x || r == 0, DMLHIP_ERR_NULL, "reduce: NULL input");
    DML_REQUIRE(y, DMLHIP_ERR_NULL, "reduce: NULL output");
    hipStream_t st = (hipStream_t)stream;
    const TIn* xp = (const TIn*)x;
#define DML_RED(OP)                                                                                          \
    case OP:                                                                                                 \
        return out_dtype == DMLHIP_F32                                                                       \
                   ? reduce_typed<TIn, float, OP>(xp, (float*)y, outer, r, inner, ws, ws_bytes, st)          \
                   : reduce_typed<TIn, _Float16, OP>(xp, (_Float16*)y, outer, r, inner, ws, ws_bytes, st)
    switch (op) {
        DML_RED(DMLHIP_RSUM);
        DML_RED(DMLHIP_RMAX);
        DML_RED(DMLHIP_RMIN);
        default: DML_RED(DMLHIP_RMEAN);
    }
#undef DML_RED
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

size_t dmlhip_reduce_workspace_bytes(int64_t outer, int64_t r, int64_t inner) {
    if (outer <= 0 || r <= 0 || inner <= 1) return 0;
    // alignment-independent upper bound: the plan with the most splits
    const int64_t tiles_min = ceil_div(inner, (int64_t)kWave * 8);
    int64_t splits = ceil_div(1024, tiles_min * outer);
    const int64_t max_splits = ceil_div(r, 4 * kRedWaves);
    if (splits > max_splits) splits = max_splits;
    if (splits <= 1) return 0;
    return (size_t)(splits + 1) * outer * inner * sizeof(float);
}

size_t dmlhip_reduce_sum_multi_workspace_bytes(int count, const int64_t* rows, const int64_t* cols) {
    MultiRedArgs a = {};
    long long part_floats = 0, max_cols;
    int max_splits;
    if (multi_plan(count, rows, cols, a, part_floats, max_splits, max_cols)) return 0;
    return (size_t)part_floats * sizeof(float);
}
int dmlhip_reduce_sum_multi_f16(int count, const void* const* x, void* const* y, int out_dtype, const int64_t* rows,
                                const int64_t* cols, void* workspace, size_t workspace_bytes, void* stream) {
    return reduce_sum_multi_impl<_Float16>(count, x, y, out_dtype, rows, cols, workspace, workspace_bytes, stream);
}
int dmlhip_reduce_sum_multi_f32(int count, const void* const* x, void* const* y, int out_dtype, const int64_t* rows,
                                const int64_t* cols, void* workspace, size_t workspace_bytes, void* stream) {
    return reduce_sum_multi_impl<float>(count, x, y, out_dtype, rows, cols, workspace, workspace_bytes, stream);
}

int dmlhip_reduce_f16(int op, const void* x, void* y, int out_dtype, int64_t outer, int64_t r, int64_t inner,
                      void* workspace, size_t workspace_bytes, void* stream) {
    return reduce_impl<_Float16>(op, x, y, out_dtype, outer, r, inner, workspace, workspace_bytes, stream);
}
int dmlhip_reduce_f32(int op, const void* x, void* y, int out_dtype, int64_t outer, int64_t r, int64_t inner,
                      void* workspace, size_t workspace_bytes, void* stream) {
    return reduce_impl<float>(op, x, y, out_dtype, outer, r, inner, workspace, workspace_bytes, stream);
}

int dmlhip_row_dot_f16(const void* a, const void* b, void* y, int64_t rows, int64_t cols, void* stream) {
    return row_dot_impl<_Float16>(a, b, y, rows, cols, stream);
}
int dmlhip_row_dot_f32(const void* a, const void* b, void* y, int64_t rows, int64_t cols, void* stream) {
    return row_dot_impl<float>(a, b, y, rows, cols, stream);
}

}  // extern "C"
