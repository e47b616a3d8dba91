// BatchNormalization over NCHW tensors: inference, training forward (batch statistics + running-statistics update)
// and backward. HBM-bound: training reads X twice and writes Y once, backward reads dY and X twice and writes dX.
// A Relu or Swish that follows the normalisation can run inside the same kernels (template parameter ACT): the
// forward applies it before the store, the backward recomputes the normalised value from X and multiplies the incoming
// gradient by the activation's derivative, so neither pass touches the tensor more often than without it.
//
// A channel's data are N segments of HW contiguous elements. Segments are cut into chunks of at most kChunk
// elements; workgroup (c, s) of a grid C x S walks the chunks s, s+S, ... of channel c, so the launch fills the
// chip also when C is small. Statistics are accumulated in fp32 as sums of (x - K) and (x - K)^2 with K the
// channel's first element (shifted-data variance: no cancellation against a large mean), written as per-workgroup
// partials; the second kernel of each pair starts by combining its channel's partials (S <= kMaxSplit of them).
#include <initializer_list>
#include <type_traits>

#include "common.h"

namespace dml {
namespace {

constexpr int kThreads = 256;
constexpr int kChunk = 4096;
constexpr int kMaxSplit = 64;

struct BnGeom {
    int64_t n, c, hw;
    int64_t chunks_per_seg;   // ceil(hw / kChunk)
    int64_t chunks;           // n * chunks_per_seg
    int split;                // S
    int vec_ok;               // segments are 16-byte aligned and hw is a multiple of the vector length
};

// Calls f(index into the tensor, element count <= VecOf<T>::n) for this thread's share of the channel's chunks.
template <typename T, typename F>
__device__ __forceinline__ void for_each_piece(const BnGeom& g, int c, int s, F&& f) {
    constexpr int V = VecOf<T>::n;
    for (int64_t ch = s; ch < g.chunks; ch += g.split) {
        const int64_t n = ch / g.chunks_per_seg;
        const int64_t off = (ch - n * g.chunks_per_seg) * kChunk;
        const int64_t len = min((int64_t)kChunk, g.hw - off);
        const int64_t base = (n * g.c + c) * g.hw + off;
        if (g.vec_ok) {
            for (int64_t i = (int64_t)threadIdx.x * V; i < len; i += (int64_t)kThreads * V) f(base + i, V);
        } else {
            for (int64_t i = threadIdx.x; i < len; i += kThreads) f(base + i, 1);
        }
    }
}

template <typename T>
__device__ __forceinline__ void load_piece(const T* p, int64_t idx, int count, float (&v)[VecOf<T>::n]) {
    constexpr int V = VecOf<T>::n;
    if (count == V) {
        const typename VecOf<T>::type q = *reinterpret_cast<const typename VecOf<T>::type*>(p + idx);
#pragma unroll
        for (int j = 0; j < V; ++j) v[j] = to_f32(q[j]);
    } else {
        v[0] = to_f32(p[idx]);
    }
}

template <typename T>
__device__ __forceinline__ void store_piece(T* p, int64_t idx, int count, const float (&v)[VecOf<T>::n]) {
    constexpr int V = VecOf<T>::n;
    if (count == V) {
        typename VecOf<T>::type q;
#pragma unroll
        for (int j = 0; j < V; ++j) q[j] = from_f32<T>(v[j]);
        *reinterpret_cast<typename VecOf<T>::type*>(p + idx) = q;
    } else {
        p[idx] = from_f32<T>(v[0]);
    }
}

// The activation that may follow the normalisation inside the same kernel (NONE, RELU, SWISH), and its derivative
// with respect to the normalised value z — the backward kernels recompute z from X instead of reading a stored copy.
template <int ACT>
__device__ __forceinline__ float bn_act(float z) {
    if constexpr (ACT == DMLHIP_ACT_SWISH) return z * sigmoid_epilogue_f(z);
    else if constexpr (ACT == DMLHIP_ACT_RELU) return fmaxf(z, 0.f);
    else return z;
}
template <int ACT>
__device__ __forceinline__ float bn_act_grad(float z) {
    if constexpr (ACT == DMLHIP_ACT_SWISH) {
        const float sg = sigmoid_epilogue_f(z);
        return sg * (1.0f + z * (1.0f - sg));
    } else if constexpr (ACT == DMLHIP_ACT_RELU) return z > 0.f ? 1.f : 0.f;
    else return 1.f;
}

// partial[(c * S + s) * 2 + {0, 1}] = sum of (x - K), sum of (x - K)^2 over the workgroup's chunks
template <typename T>
__global__ __launch_bounds__(kThreads) void bn_stats_kernel(const T* __restrict__ x, float* __restrict__ partial,
                                                            BnGeom g) {
    __shared__ float scratch[kThreads / kWave];
    const int c = blockIdx.x, s = blockIdx.y;
    const float shift = to_f32(x[(int64_t)c * g.hw]);
    float s1 = 0.f, s2 = 0.f;
    for_each_piece<T>(g, c, s, [&](int64_t idx, int count) {
        float v[VecOf<T>::n];
        load_piece<T>(x, idx, count, v);
        for (int j = 0; j < count; ++j) {
            const float d = v[j] - shift;
            s1 += d;
            s2 += d * d;
        }
    });
    s1 = block_reduce<OpSum, kThreads / kWave>(s1, scratch);
    s2 = block_reduce<OpSum, kThreads / kWave>(s2, scratch);
    if (threadIdx.x == 0) {
        partial[((int64_t)c * g.split + s) * 2 + 0] = s1;
        partial[((int64_t)c * g.split + s) * 2 + 1] = s2;
    }
}

// Sum of the channel's partial pairs, by the first wavefront; every thread gets the result.
__device__ __forceinline__ void combine_partials(const float* partial, int c, int split, float* lds2, float& a, float& b) {
    if (threadIdx.x < kWave) {
        float p0 = 0.f, p1 = 0.f;
        for (int i = threadIdx.x; i < split; i += kWave) {
            p0 += partial[((int64_t)c * split + i) * 2 + 0];
            p1 += partial[((int64_t)c * split + i) * 2 + 1];
        }
        p0 = wave_reduce<OpSum>(p0);
        p1 = wave_reduce<OpSum>(p1);
        if (threadIdx.x == 0) {
            lds2[0] = p0;
            lds2[1] = p1;
        }
    }
    __syncthreads();
    a = lds2[0];
    b = lds2[1];
}

// TRAINING: statistics from `partial`; workgroup s == 0 also writes the saved and the running statistics.
// otherwise: statistics are the given mean / var.
template <typename T, bool TRAINING, int ACT>
__global__ __launch_bounds__(kThreads) void bn_apply_kernel(const T* __restrict__ x, const T* __restrict__ scale,
                                                            const T* __restrict__ bias, const T* __restrict__ in_mean,
                                                            const T* __restrict__ in_var, const float* __restrict__ partial,
                                                            T* __restrict__ y, T* __restrict__ out_mean,
                                                            T* __restrict__ out_var, T* __restrict__ saved_mean,
                                                            T* __restrict__ saved_var, float eps, float momentum,
                                                            BnGeom g) {
    __shared__ float lds2[2];
    const int c = blockIdx.x, s = blockIdx.y;
    float mean, var;
    if constexpr (TRAINING) {
        float s1, s2;
        combine_partials(partial, c, g.split, lds2, s1, s2);
        const float cnt = (float)(g.n * g.hw);
        const float shift = to_f32(x[(int64_t)c * g.hw]);
        const float dm = s1 / cnt;
        mean = shift + dm;
        var = fmaxf(s2 / cnt - dm * dm, 0.f);   // biased, as np.add.reduce(...) / N
        if (s == 0 && threadIdx.x == 0) {
            saved_mean[c] = from_f32<T>(mean);
            saved_var[c] = from_f32<T>(var);
            out_mean[c] = from_f32<T>(to_f32(in_mean[c]) * momentum + mean * (1.f - momentum));
            out_var[c] = from_f32<T>(to_f32(in_var[c]) * momentum + var * (1.f - momentum));
        }
    } else {
        mean = to_f32(in_mean[c]);
        var = to_f32(in_var[c]);
    }
    const float a = to_f32(scale[c]) * (1.0f / sqrtf(var + eps));
    const float b = to_f32(bias[c]);
    for_each_piece<T>(g, c, s, [&](int64_t idx, int count) {
        float v[VecOf<T>::n];
        load_piece<T>(x, idx, count, v);
        for (int j = 0; j < count; ++j) v[j] = bn_act<ACT>((v[j] - mean) * a + b);   // centred first: no cancellation for large means
        store_piece<T>(y, idx, count, v);
    });
}

// partial pairs: sum of dz, sum of dz * (x - mean), with dz = dy * act'(z) the gradient at the normalised value
template <typename T, int ACT>
__global__ __launch_bounds__(kThreads) void bn_bwd_stats_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                                const T* __restrict__ scale, const T* __restrict__ bias,
                                                                const T* __restrict__ saved_mean,
                                                                const T* __restrict__ saved_var, float eps,
                                                                float* __restrict__ partial, BnGeom g) {
    __shared__ float scratch[kThreads / kWave];
    const int c = blockIdx.x, s = blockIdx.y;
    const float mean = to_f32(saved_mean[c]);
    float a = 0.f, b = 0.f;
    if constexpr (ACT != DMLHIP_ACT_NONE) {
        a = to_f32(scale[c]) * (1.0f / sqrtf(to_f32(saved_var[c]) + eps));
        b = to_f32(bias[c]);
    }
    float s1 = 0.f, s2 = 0.f;
    for_each_piece<T>(g, c, s, [&](int64_t idx, int count) {
        float v[VecOf<T>::n], d[VecOf<T>::n];
        load_piece<T>(x, idx, count, v);
        load_piece<T>(dy, idx, count, d);
        for (int j = 0; j < count; ++j) {
            const float xc = v[j] - mean;
            const float dz = d[j] * bn_act_grad<ACT>(xc * a + b);
            s1 += dz;
            s2 += dz * xc;
        }
    });
    s1 = block_reduce<OpSum, kThreads / kWave>(s1, scratch);
    s2 = block_reduce<OpSum, kThreads / kWave>(s2, scratch);
    if (threadIdx.x == 0) {
        partial[((int64_t)c * g.split + s) * 2 + 0] = s1;
        partial[((int64_t)c * g.split + s) * 2 + 1] = s2;
    }
}

// dx = scale * invstd * (dz - mean(dz) - (x - mean) * invstd^2 * mean(dz * (x - mean)))
template <typename T, int ACT>
__global__ __launch_bounds__(kThreads) void bn_bwd_apply_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                                const T* __restrict__ scale, const T* __restrict__ bias,
                                                                const T* __restrict__ saved_mean,
                                                                const T* __restrict__ saved_var,
                                                                const float* __restrict__ partial, T* __restrict__ dx,
                                                                float* __restrict__ dscale, float* __restrict__ dbias,
                                                                float eps, BnGeom g) {
    __shared__ float lds2[2];
    const int c = blockIdx.x, s = blockIdx.y;
    float sum_dy, sum_dyxc;
    combine_partials(partial, c, g.split, lds2, sum_dy, sum_dyxc);
    const float mean = to_f32(saved_mean[c]);
    const float invstd = 1.0f / sqrtf(to_f32(saved_var[c]) + eps);
    if (s == 0 && threadIdx.x == 0) {
        if (dscale) dscale[c] = sum_dyxc * invstd;
        if (dbias) dbias[c] = sum_dy;
    }
    if (!dx) return;
    const float cnt = (float)(g.n * g.hw);
    const float k0 = to_f32(scale[c]) * invstd;
    const float k1 = sum_dy / cnt;
    const float k2 = invstd * invstd * sum_dyxc / cnt;
    float b = 0.f;
    if constexpr (ACT != DMLHIP_ACT_NONE) b = to_f32(bias[c]);
    for_each_piece<T>(g, c, s, [&](int64_t idx, int count) {
        float v[VecOf<T>::n], d[VecOf<T>::n];
        load_piece<T>(x, idx, count, v);
        load_piece<T>(dy, idx, count, d);
        for (int j = 0; j < count; ++j) {
            const float xc = v[j] - mean;
            v[j] = k0 * (d[j] * bn_act_grad<ACT>(xc * k0 + b) - k1 - xc * k2);
        }
        store_piece<T>(dx, idx, count, v);
    });
}

int make_geom(const char* what, int64_t n, int64_t c, int64_t hw, std::initializer_list<const void*> tensors, BnGeom* g) {
    DML_REQUIRE(n > 0 && c > 0 && hw > 0, DMLHIP_ERR_SHAPE, "%s: extents must be positive, got N=%lld C=%lld HW=%lld", what,
                (long long)n, (long long)c, (long long)hw);
    DML_REQUIRE(c <= 0x7fffffff, DMLHIP_ERR_SHAPE, "%s: %lld channels exceed the grid limit", what, (long long)c);
    g->n = n;
    g->c = c;
    g->hw = hw;
    g->chunks_per_seg = ceil_div(hw, kChunk);
    g->chunks = n * g->chunks_per_seg;
    // enough workgroups to fill 256 CUs several times over, never more than there are chunks
    int64_t split = ceil_div(2048, c);
    if (split > g->chunks) split = g->chunks;
    if (split > kMaxSplit) split = kMaxSplit;
    g->split = (int)(split < 1 ? 1 : split);
    bool vec = true;
    for (const void* p : tensors) vec = vec && (p == nullptr || aligned16(p));
    g->vec_ok = vec && hw % 8 == 0;   // 8 covers both vector lengths and keeps every segment 16-byte aligned
    return 0;
}

size_t bn_workspace(int64_t n, int64_t c, int64_t hw) {
    (void)n;
    (void)hw;
    return c > 0 ? (size_t)c * kMaxSplit * 2 * sizeof(float) : 0;
}

// runs `body(std::integral_constant<int, ACT>)` for the activation code, or reports an unsupported one
template <typename F>
int with_activation(const char* what, int act, F&& body) {
    switch (act) {
        case DMLHIP_ACT_NONE: return body(std::integral_constant<int, DMLHIP_ACT_NONE>{});
        case DMLHIP_ACT_RELU: return body(std::integral_constant<int, DMLHIP_ACT_RELU>{});
        case DMLHIP_ACT_SWISH: return body(std::integral_constant<int, DMLHIP_ACT_SWISH>{});
        default:
            set_error("%s: activation %d is not one of NONE, RELU, SWISH", what, act);
            return DMLHIP_ERR_ENUM;
    }
}

template <typename T>
int bn_inference(const void* x, const void* scale, const void* bias, const void* mean, const void* var, void* y,
                 int64_t n, int64_t c, int64_t hw, float eps, int act, void* stream) {
    DML_REQUIRE(x && scale && bias && mean && var && y, DMLHIP_ERR_NULL, "batchnorm_inference: NULL pointer");
    BnGeom g;
    if (int e = make_geom("batchnorm_inference", n, c, hw, {x, y}, &g)) return e;
    return with_activation("batchnorm_inference", act, [&](auto actc) {
        constexpr int ACT = decltype(actc)::value;
        hipLaunchKernelGGL((bn_apply_kernel<T, false, ACT>), dim3((unsigned)c, (unsigned)g.split), kThreads, 0,
                           (hipStream_t)stream, (const T*)x, (const T*)scale, (const T*)bias, (const T*)mean, (const T*)var,
                           (const float*)nullptr, (T*)y, (T*)nullptr, (T*)nullptr, (T*)nullptr, (T*)nullptr, eps, 0.f, g);
        return launch_status("batchnorm_inference");
    });
}

template <typename T>
int bn_training(const void* x, const void* scale, const void* bias, const void* in_mean, const void* in_var, void* y,
                void* out_mean, void* out_var, void* saved_mean, void* saved_var, int64_t n, int64_t c, int64_t hw,
                float eps, float momentum, int act, void* workspace, size_t workspace_bytes, void* stream) {
    DML_REQUIRE(x && scale && bias && in_mean && in_var && y && out_mean && out_var && saved_mean && saved_var,
                DMLHIP_ERR_NULL, "batchnorm_training: NULL pointer");
    BnGeom g;
    if (int e = make_geom("batchnorm_training", n, c, hw, {x, y}, &g)) return e;
    DML_REQUIRE(workspace && workspace_bytes >= bn_workspace(n, c, hw), DMLHIP_ERR_WORKSPACE,
                "batchnorm_training: workspace of %zu bytes needed, got %zu", bn_workspace(n, c, hw), workspace_bytes);
    const dim3 grid((unsigned)c, (unsigned)g.split);
    hipLaunchKernelGGL((bn_stats_kernel<T>), grid, kThreads, 0, (hipStream_t)stream, (const T*)x, (float*)workspace, g);
    if (int e = launch_status("batchnorm_training(statistics)")) return e;
    return with_activation("batchnorm_training", act, [&](auto actc) {
        constexpr int ACT = decltype(actc)::value;
        hipLaunchKernelGGL((bn_apply_kernel<T, true, ACT>), grid, kThreads, 0, (hipStream_t)stream, (const T*)x,
                           (const T*)scale, (const T*)bias, (const T*)in_mean, (const T*)in_var, (const float*)workspace,
                           (T*)y, (T*)out_mean, (T*)out_var, (T*)saved_mean, (T*)saved_var, eps, momentum, g);
        return launch_status("batchnorm_training");
    });
}

template <typename T>
int bn_backward(const void* dy, const void* x, const void* scale, const void* bias, const void* saved_mean,
                const void* saved_var, void* dx, float* dscale, float* dbias, int64_t n, int64_t c, int64_t hw, float eps,
                int act, void* workspace, size_t workspace_bytes, void* stream) {
    DML_REQUIRE(dy && x && scale && saved_mean && saved_var, DMLHIP_ERR_NULL, "batchnorm_backward: NULL pointer");
    DML_REQUIRE(bias || act == DMLHIP_ACT_NONE, DMLHIP_ERR_NULL,
                "batchnorm_backward: the bias is needed to recompute the activation's input");
    DML_REQUIRE(dx || dscale || dbias, DMLHIP_ERR_NULL, "batchnorm_backward: no gradient requested");
    BnGeom g;
    if (int e = make_geom("batchnorm_backward", n, c, hw, {dy, x, dx}, &g)) return e;
    DML_REQUIRE(workspace && workspace_bytes >= bn_workspace(n, c, hw), DMLHIP_ERR_WORKSPACE,
                "batchnorm_backward: workspace of %zu bytes needed, got %zu", bn_workspace(n, c, hw), workspace_bytes);
    const dim3 grid((unsigned)c, (unsigned)g.split);
    return with_activation("batchnorm_backward", act, [&](auto actc) {
        constexpr int ACT = decltype(actc)::value;
        hipLaunchKernelGGL((bn_bwd_stats_kernel<T, ACT>), grid, kThreads, 0, (hipStream_t)stream, (const T*)dy, (const T*)x,
                           (const T*)scale, (const T*)bias, (const T*)saved_mean, (const T*)saved_var, eps,
                           (float*)workspace, g);
        if (int e = launch_status("batchnorm_backward(sums)")) return e;
        hipLaunchKernelGGL((bn_bwd_apply_kernel<T, ACT>), grid, kThreads, 0, (hipStream_t)stream, (const T*)dy, (const T*)x,
                           (const T*)scale, (const T*)bias, (const T*)saved_mean, (const T*)saved_var,
                           (const float*)workspace, (T*)dx, dscale, dbias, eps, g);
        return launch_status("batchnorm_backward");
    });
}

}  // namespace
}  // namespace dml

using namespace dml;

extern "C" {

size_t dmlhip_batchnorm_workspace_bytes(int64_t n, int64_t c, int64_t hw) { return bn_workspace(n, c, hw); }

#define DML_BN_ENTRIES(SFX, T)                                                                                         \
    int dmlhip_batchnorm_inference_##SFX(const void* x, const void* scale, const void* bias, const void* mean,         \
                                         const void* var, void* y, int64_t n, int64_t c, int64_t hw, float eps,        \
                                         void* stream) {                                                               \
        return bn_inference<T>(x, scale, bias, mean, var, y, n, c, hw, eps, DMLHIP_ACT_NONE, stream);                  \
    }                                                                                                                  \
    int dmlhip_batchnorm_inference_act_##SFX(const void* x, const void* scale, const void* bias, const void* mean,     \
                                             const void* var, void* y, int64_t n, int64_t c, int64_t hw, float eps,    \
                                             int act, void* stream) {                                                  \
        return bn_inference<T>(x, scale, bias, mean, var, y, n, c, hw, eps, act, stream);                              \
    }                                                                                                                  \
    int dmlhip_batchnorm_training_##SFX(const void* x, const void* scale, const void* bias, const void* in_mean,       \
                                        const void* in_var, void* y, void* out_mean, void* out_var, void* saved_mean,  \
                                        void* saved_var, int64_t n, int64_t c, int64_t hw, float eps, float momentum,  \
                                        void* workspace, size_t workspace_bytes, void* stream) {                       \
        return bn_training<T>(x, scale, bias, in_mean, in_var, y, out_mean, out_var, saved_mean, saved_var, n, c, hw,  \
                              eps, momentum, DMLHIP_ACT_NONE, workspace, workspace_bytes, stream);                     \
    }                                                                                                                  \
    int dmlhip_batchnorm_training_act_##SFX(const void* x, const void* scale, const void* bias, const void* in_mean,   \
                                            const void* in_var, void* y, void* out_mean, void* out_var,                \
                                            void* saved_mean, void* saved_var, int64_t n, int64_t c, int64_t hw,       \
                                            float eps, float momentum, int act, void* workspace,                       \
                                            size_t workspace_bytes, void* stream) {                                    \
        return bn_training<T>(x, scale, bias, in_mean, in_var, y, out_mean, out_var, saved_mean, saved_var, n, c, hw,  \
                              eps, momentum, act, workspace, workspace_bytes, stream);                                 \
    }                                                                                                                  \
    int dmlhip_batchnorm_backward_##SFX(const void* dy, const void* x, const void* scale, const void* saved_mean,      \
                                        const void* saved_var, void* dx, float* dscale, float* dbias, int64_t n,       \
                                        int64_t c, int64_t hw, float eps, void* workspace, size_t workspace_bytes,     \
                                        void* stream) {                                                                \
        return bn_backward<T>(dy, x, scale, nullptr, saved_mean, saved_var, dx, dscale, dbias, n, c, hw, eps,          \
                              DMLHIP_ACT_NONE, workspace, workspace_bytes, stream);                                    \
    }                                                                                                                  \
    int dmlhip_batchnorm_backward_act_##SFX(const void* dy, const void* x, const void* scale, const void* bias,        \
                                            const void* saved_mean, const void* saved_var, void* dx, float* dscale,    \
                                            float* dbias, int64_t n, int64_t c, int64_t hw, float eps, int act,        \
                                            void* workspace, size_t workspace_bytes, void* stream) {                   \
        return bn_backward<T>(dy, x, scale, bias, saved_mean, saved_var, dx, dscale, dbias, n, c, hw, eps, act,        \
                              workspace, workspace_bytes, stream);                                                     \
    }

DML_BN_ENTRIES(f16, _Float16)
DML_BN_ENTRIES(f32, float)
#undef DML_BN_ENTRIES

}  // extern "C"
