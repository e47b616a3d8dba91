/*
 * daceml_hip.h — C ABI of libdaceml_hip.so: hand-written gfx950 (MI355X) kernels for the
 * ONNX library-node hot path of DaCeML.
 *
 * The reference (spcl/daceml) has no compiled sources; what these entry points replace are
 * the *call sites* through which its expansions reach native code:
 *   - the SDFG that a "pure" expansion returns and DaCe compiles
 *     (daceml/onnx/op_implementations/pure_implementations.py, img_op_implementations.py),
 *   - the cuDNN calls emitted as C++ tasklets
 *     (daceml/onnx/op_implementations/cudnn_implementations.py:360-410),
 *   - cuBLAS reached through DaCe's BLAS library nodes
 *     (daceml/util/utils.py:226-229).
 * Each declaration cites the reference expansion whose semantics it implements.
 *
 * Calling convention
 *   - tensors are dense row-major device pointers unless strides are passed explicitly;
 *   - every call is asynchronous on `stream` (a hipStream_t passed as void*; NULL = the
 *     null stream), never synchronises, never allocates or frees, and never keeps a pointer;
 *   - scratch memory is caller-provided and sized by the matching *_workspace_bytes query;
 *   - return value: 0 = launched; < 0 = argument error detected on the host before any device
 *     work (safe to call on a machine without a GPU); > 0 = hipError_t of a failed launch.
 *     dmlhip_last_error_string() describes the last failure on the calling thread.
 *   - "_f16" entry points read/write IEEE half and always compute and accumulate in fp32
 *     (the effect of daceml/transformation/mixed_precision.py:5-35); "_f32" entry points
 *     are fp32 end to end with no fast-math (daceml/__init__.py:13-19).
 */
#ifndef DACEML_HIP_H
#define DACEML_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DMLHIP_VERSION 100 /* major*10000 + minor*100 + patch */
#define DMLHIP_MAX_DIMS 6

enum {
    DMLHIP_OK = 0,
    DMLHIP_ERR_NULL = -1,        /* a required pointer is NULL */
    DMLHIP_ERR_SHAPE = -2,       /* negative / inconsistent / overflowing extents */
    DMLHIP_ERR_UNSUPPORTED = -3, /* valid ONNX, but outside what the kernels cover */
    DMLHIP_ERR_ALIGN = -4,       /* pointer or stride alignment requirement violated */
    DMLHIP_ERR_WORKSPACE = -5,   /* workspace NULL or smaller than the query says */
    DMLHIP_ERR_ENUM = -6         /* unknown op / dtype / epilogue code */
};

/* element types used for "out_dtype"/"bias_dtype" style arguments */
enum { DMLHIP_F16 = 0, DMLHIP_F32 = 1 };

int dmlhip_version(void);
const char* dmlhip_last_error_string(void);

/* ------------------------------------------------------------------ Softmax
 * Softmax "pure": pure_implementations.py:309-319. The caller coalesces
 * [shape[:axis], shape[axis:]] into rows x cols (opset-12 semantics); y = exp(x-max)/sum. */
int dmlhip_softmax_f16(const void* x, void* y, int64_t rows, int64_t cols, void* stream);
int dmlhip_softmax_f32(const void* x, void* y, int64_t rows, int64_t cols, void* stream);

/* DefaultSoftmaxBackward: autodiff/implementations/onnx_ops.py:237-275.
 * dx = y*dy - y*sum_row(y*dy), in one pass. */
int dmlhip_softmax_backward_f16(const void* y, const void* dy, void* dx, int64_t rows,
                                int64_t cols, void* stream);
int dmlhip_softmax_backward_f32(const void* y, const void* dy, void* dx, int64_t rows,
                                int64_t cols, void* stream);

/* ------------------------------------------------------------------ LayerNormalization
 * The opset-12 export has no LayerNormalization node; the reference runs the chain
 * ReduceMean, Sub, Pow, ReduceMean, Add, Sqrt, Div, Mul, Add
 * (pure_implementations.py:101-103,81-83,39-41,76-78,34-36,91-93). This is that chain fused:
 * mu = mean(s), var = mean((s-mu)^2) (biased, two-pass), y = (s-mu)/sqrt(var+eps)*gamma+beta,
 * with s = x (+ residual when residual != NULL: the preceding ONNXAdd fused in).
 * Optional outputs (NULL to skip): sum_out = s (same dtype as x), mean / rstd = per-row
 * fp32 statistics for the backward node. */
int dmlhip_layernorm_f16(const void* x, const void* residual, const void* gamma,
                         const void* beta, void* y, void* sum_out, float* mean, float* rstd,
                         int64_t rows, int64_t cols, float eps, void* stream);
int dmlhip_layernorm_f32(const void* x, const void* residual, const void* gamma,
                         const void* beta, void* y, void* sum_out, float* mean, float* rstd,
                         int64_t rows, int64_t cols, float eps, void* stream);

/* Backward of the chain above (what the SymPy tasklet reversal of
 * autodiff/backward_pass_generator.py:1284-1421 plus ReverseReduce, dace_nodes.py:13-105,
 * compute as many small maps). dx has x's dtype; dgamma/dbeta are fp32 master gradients
 * (overwritten, not accumulated). Needs a workspace. */
size_t dmlhip_layernorm_backward_workspace_bytes(int64_t rows, int64_t cols);
int dmlhip_layernorm_backward_f16(const void* dy, const void* x, const float* mean,
                                  const float* rstd, const void* gamma, void* dx,
                                  float* dgamma, float* dbeta, int64_t rows, int64_t cols,
                                  void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_layernorm_backward_f32(const void* dy, const void* x, const float* mean,
                                  const float* rstd, const void* gamma, void* dx,
                                  float* dgamma, float* dbeta, int64_t rows, int64_t cols,
                                  void* workspace, size_t workspace_bytes, void* stream);

/* dmlhip_layernorm_backward_f16 with the scale / shift gradients in the type the caller names (DMLHIP_F16 or
 * DMLHIP_F32): under the reference a gradient has the dtype of its forward array
 * (autodiff/backward_pass_generator.py:642-700), so an fp16 LayerNorm's scale and bias get fp16 gradients. The column
 * sums are formed in fp32 and rounded once when they are stored. */
int dmlhip_layernorm_backward_grads_f16(const void* dy, const void* x, const float* mean,
                                        const float* rstd, const void* gamma, void* dx,
                                        void* dgamma, void* dbeta, int grad_dtype, int64_t rows,
                                        int64_t cols, void* workspace, size_t workspace_bytes, void* stream);

/* dmlhip_layernorm_backward_f16 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the
 * reference. Same arguments and results as dmlhip_layernorm_backward_f16 without the workspace: the
 * per-workgroup partial sums go to a fixed device array inside the library (one copy per GPU, resident
 * until the process ends) of dmlhip_layernorm_backward_noalloc_max_bytes() = 8 MiB. Shapes whose
 * dmlhip_layernorm_backward_workspace_bytes(rows, cols) exceeds that are refused with
 * DMLHIP_ERR_WORKSPACE. The call allocates and frees nothing. Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (different streams or threads) race; calls on one stream do not.
 * The first call on a device looks up the array's device address (hipGetSymbolAddress): make one ordinary
 * call on each device before the first call under stream capture there. */
size_t dmlhip_layernorm_backward_noalloc_max_bytes(void);
int dmlhip_layernorm_backward_noalloc_f16(const void* dy, const void* x, const float* mean,
                                          const float* rstd, const void* gamma, void* dx,
                                          float* dgamma, float* dbeta, int64_t rows, int64_t cols,
                                          void* stream);

/* ------------------------------------------------------------------ elementwise
 * Add/Sub/Mul/Div/Pow "pure": pure_implementations.py:39-41,76-93 (NumPy broadcasting).
 * `shape` is the broadcast output shape (ndim <= DMLHIP_MAX_DIMS); a_strides / b_strides are
 * element strides per output dim, 0 where the operand is broadcast. c is dense. */
enum { DMLHIP_ADD = 0, DMLHIP_SUB = 1, DMLHIP_MUL = 2, DMLHIP_DIV = 3, DMLHIP_POW = 4 };
int dmlhip_binary_f16(int op, const void* a, const void* b, void* c, int ndim,
                      const int64_t* shape, const int64_t* a_strides,
                      const int64_t* b_strides, void* stream);
int dmlhip_binary_f32(int op, const void* a, const void* b, void* c, int ndim,
                      const int64_t* shape, const int64_t* a_strides,
                      const int64_t* b_strides, void* stream);

/* Unary maps: Erf (pure_implementations.py:106-108), Sqrt (:34-36), Exp/Log (:24-31),
 * Tanh (:289-291), Relu (:556-560), Sigmoid (:741-743), Reciprocal (:283-286).
 * GELU = the exported chain Div,Erf,Add,Mul,Mul fused: 0.5*x*(1+erf(x/sqrt(2))).
 * SWISH = Mul(x, Sigmoid(x)) fused. SCALE: y = x*param (Mul/Div by a scalar constant). */
enum {
    DMLHIP_ERF = 0, DMLHIP_SQRT = 1, DMLHIP_EXP = 2, DMLHIP_LOG = 3, DMLHIP_TANH = 4,
    DMLHIP_RELU = 5, DMLHIP_SIGMOID = 6, DMLHIP_RECIPROCAL = 7, DMLHIP_GELU = 8,
    DMLHIP_SWISH = 9, DMLHIP_SCALE = 10, DMLHIP_IDENTITY = 11
};
int dmlhip_unary_f16(int op, const void* x, void* y, int64_t n, float param, void* stream);
int dmlhip_unary_f32(int op, const void* x, void* y, int64_t n, float param, void* stream);

/* Backward of the unary maps above: dx = dy * f'(x), x being the forward *input* (the derivative the SymPy
 * tasklet reversal of autodiff/backward_pass_generator.py:1284-1421 writes for each of these maps). dx may be the
 * very buffer of dy (not a shifted or partial overlap of it, and not x). */
int dmlhip_unary_backward_f16(int op, const void* x, const void* dy, void* dx, int64_t n,
                              float param, void* stream);
int dmlhip_unary_backward_f32(int op, const void* x, const void* dy, void* dx, int64_t n,
                              float param, void* stream);

/* PureSum: pure_implementations.py:584-646 — variadic same-shape sum, 1..8 inputs. */
int dmlhip_sum_f16(const void* const* inputs, int n_inputs, void* out, int64_t n, void* stream);
int dmlhip_sum_f32(const void* const* inputs, int n_inputs, void* out, int64_t n, void* stream);

/* y[r, j] = a[r, j] * s[r] + t[r] * scale[0] over dense [rows, cols] (scale may be NULL = 1): ONNXSum
 * (pure_implementations.py:584-646) of an ONNXMul with a per-row factor (:86-88) and a per-row value broadcast back over
 * the row (ReverseReduce, autodiff/implementations/dace_nodes.py:13-105) — the gradient accumulation at the input of a
 * squeeze-excite block — in one pass. */
int dmlhip_row_affine_f16(const void* a, const void* s, const void* t, const void* scale, void* y, int64_t rows,
                          int64_t cols, void* stream);
int dmlhip_row_affine_f32(const void* a, const void* s, const void* t, const void* scale, void* y, int64_t rows,
                          int64_t cols, void* stream);

/* Add(bias[cols]) followed by the GELU chain, fused; bias may be NULL.
 * pre_out (nullable) receives x+bias, which the backward needs. */
int dmlhip_bias_gelu_f16(const void* x, const void* bias, void* y, void* pre_out, int64_t rows,
                         int64_t cols, void* stream);
int dmlhip_bias_gelu_f32(const void* x, const void* bias, void* y, void* pre_out, int64_t rows,
                         int64_t cols, void* stream);

/* Cast "pure": pure_implementations.py:329-377, between DMLHIP_F16 and DMLHIP_F32. */
int dmlhip_cast(int src_dtype, int dst_dtype, const void* x, void* y, int64_t n, void* stream);

/* ------------------------------------------------------------------ reductions
 * ReduceSum/Max/Min/Mean "pure": pure_implementations.py:101-103,294-306;
 * GlobalAveragePool "pure": img_op_implementations.py:415-417 (= MEAN with inner 1).
 * Input viewed as [outer, r, inner] (the reduced axes must be adjacent; the caller collapses
 * them); output [outer, inner] of out_dtype. Accumulates in fp32. */
enum { DMLHIP_RSUM = 0, DMLHIP_RMAX = 1, DMLHIP_RMIN = 2, DMLHIP_RMEAN = 3 };
size_t dmlhip_reduce_workspace_bytes(int64_t outer, int64_t r, int64_t inner);
int dmlhip_reduce_f16(int op, const void* x, void* y, int out_dtype, int64_t outer, int64_t r,
                      int64_t inner, void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_reduce_f32(int op, const void* x, void* y, int out_dtype, int64_t outer, int64_t r,
                      int64_t inner, void* workspace, size_t workspace_bytes, void* stream);
/* y[row] = sum_j a[row, j] * b[row, j] for dense [rows, cols] operands, fp32 accumulation, y in the operands' type:
 * ONNXMul (pure_implementations.py:86-88) read only by ONNXReduceSum over the trailing axes (:294-296) — what the
 * reversal of a broadcast multiplication emits for the broadcast operand (autodiff/backward_pass_generator.py:1284-1421
 * with ReverseReduce, autodiff/implementations/dace_nodes.py:13-105) — without writing the product. */
int dmlhip_row_dot_f16(const void* a, const void* b, void* y, int64_t rows, int64_t cols, void* stream);
int dmlhip_row_dot_f32(const void* a, const void* b, void* y, int64_t rows, int64_t cols, void* stream);
/* Several independent ReduceSum nodes over all leading axes (keepdims = 0) in one launch pair:
 * y[t][c] = sum_r x[t][r, c] for count <= DMLHIP_MULTI_MAX row-major matrices [rows[t], cols[t]].
 * This is the shape of the bias gradients DefaultEinsumBackward's callers need
 * (autodiff/implementations/onnx_ops.py:54-138 leaves them to ReduceSum, pure_implementations.py:
 * 294-306); each alone is two latency-bound launches. cols[t] must keep rows 16-byte aligned.
 * All outputs have element type out_dtype. */
#define DMLHIP_MULTI_MAX 8
size_t dmlhip_reduce_sum_multi_workspace_bytes(int count, const int64_t* rows, const int64_t* cols);
int dmlhip_reduce_sum_multi_f16(int count, const void* const* x, void* const* y, int out_dtype,
                                const int64_t* rows, const int64_t* cols, void* workspace,
                                size_t workspace_bytes, void* stream);
int dmlhip_reduce_sum_multi_f32(int count, const void* const* x, void* const* y, int out_dtype,
                                const int64_t* rows, const int64_t* cols, void* workspace,
                                size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ Transpose
 * Transpose "pure"/"einsum": pure_implementations.py:322-326,746-778.
 * y = transpose(x, perm); `shape` is x's shape, ndim <= DMLHIP_MAX_DIMS. */
int dmlhip_transpose_f16(const void* x, void* y, int ndim, const int64_t* shape,
                         const int64_t* perm, void* stream);
int dmlhip_transpose_f32(const void* x, void* y, int ndim, const int64_t* shape,
                         const int64_t* perm, void* stream);

/* ------------------------------------------------------------------ MaxPool
 * PureMaxPool2D (img_op_implementations.py:28-161): x is `planes` = batch * channels images of h x w, the window
 * kh x kw moves by sh, sw; no padding, no dilation, output extents (h - kh) / sh + 1 and (w - kw) / sw + 1 rounded
 * down. The backward entry point is DefaultMaxPoolBackward (autodiff/implementations/onnx_ops.py:284-335): dx receives
 * the gradient of every window at the first position (row by row) that holds the window's maximum, zero elsewhere;
 * it needs x, not the forward output. */
int dmlhip_maxpool2d_f16(const void* x, void* y, int64_t planes, int64_t h, int64_t w, int64_t kh, int64_t kw,
                         int64_t sh, int64_t sw, void* stream);
int dmlhip_maxpool2d_f32(const void* x, void* y, int64_t planes, int64_t h, int64_t w, int64_t kh, int64_t kw,
                         int64_t sh, int64_t sw, void* stream);
int dmlhip_maxpool2d_backward_f16(const void* x, const void* dy, void* dx, int64_t planes, int64_t h, int64_t w,
                                  int64_t kh, int64_t kw, int64_t sh, int64_t sw, void* stream);
int dmlhip_maxpool2d_backward_f32(const void* x, const void* dy, void* dx, int64_t planes, int64_t h, int64_t w,
                                  int64_t kh, int64_t kw, int64_t sh, int64_t sw, void* stream);

/* ------------------------------------------------------------------ Pad
 * ONNX Pad, mode "constant", with the amounts and the fill value known when the node is lowered. The reference has no
 * expansion for it (a stand-alone Pad runs in onnxruntime; PadConvFusion, transformation/pad_conv_fusion.py:13-104,
 * folds the common case into the Conv's padding, and so does this library's fusion pass). `shape` is x's shape,
 * ndim <= DMLHIP_MAX_DIMS; y has shape[k] + begin[k] + end[k] elements along axis k; negative amounts crop (the
 * gradient of a Pad is the Pad with the amounts negated). */
int dmlhip_pad_constant_f16(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* begin,
                            const int64_t* end, float value, void* stream);
int dmlhip_pad_constant_f32(const void* x, void* y, int ndim, const int64_t* shape, const int64_t* begin,
                            const int64_t* end, float value, void* stream);

/* ------------------------------------------------------------------ contractions
 * PureEinsum / PureMatMul / PureGemm: pure_implementations.py:111-252,380-553, which the
 * reference lowers to cuBLAS (strided-batched) GEMM through DaCe. One strided, batched GEMM:
 *
 *   C[b0,b1,b2][m,n] = epilogue( alpha * sum_k A[b...][m,k] * B[b...][k,n] ) (+ beta*C)
 *
 * with arbitrary element strides for m/k/n in A and B (so the Transpose nodes around a
 * contraction fold into operand layout, the effect of transformation/einsum_fusion.py:102-151)
 * and unit stride for n in C. Products accumulate in fp32 on MFMA.
 * epilogue: v = alpha*acc; if bias: v += bias[n] (or bias[m]); if pre_out: pre_out[m,n] = v;
 *           v = act(v); if residual: v += residual[m,n]; if beta: v += beta*C;
 */
enum {
    DMLHIP_ACT_NONE = 0, DMLHIP_ACT_GELU = 1, DMLHIP_ACT_SWISH = 2, DMLHIP_ACT_SIGMOID = 3,
    DMLHIP_ACT_RELU = 4
};
typedef struct dmlhip_gemm_desc {
    int64_t m, n, k;
    int64_t batch[3];       /* batch extents; use 1 for unused dims */
    int64_t a_stride_m, a_stride_k, a_stride_batch[3];
    int64_t b_stride_k, b_stride_n, b_stride_batch[3];
    int64_t c_stride_m, c_stride_batch[3]; /* stride of n in C is 1 */
    float alpha, beta;
    int out_dtype;          /* DMLHIP_F16 or DMLHIP_F32: type of C, pre_out and residual */
    int bias_dtype;         /* type of bias[n] */
    int act;                /* DMLHIP_ACT_* */
    int bias_along_m;       /* 0: bias[n] (Linear / Gemm C vector); 1: bias[m] (conv channel bias) */
} dmlhip_gemm_desc;
/* inputs fp16 */
int dmlhip_gemm_f16(const dmlhip_gemm_desc* desc, const void* a, const void* b, void* c,
                    const void* bias, const void* residual, void* pre_out, void* stream);
/* Same, with a scratch buffer: when C has too few tiles to fill the chip and K is long (the
 * weight-gradient contractions), K is split across workgroups, fp32 partial tiles go to the
 * workspace and a second pass sums them (deterministic, no atomics). Only plain products
 * (no bias / activation / residual / pre_out / beta) are split; everything else runs as above.
 * A NULL or short workspace simply disables the split. */
size_t dmlhip_gemm_f16_workspace_bytes(const dmlhip_gemm_desc* desc);
int dmlhip_gemm_f16_ws(const dmlhip_gemm_desc* desc, const void* a, const void* b, void* c,
                       const void* bias, const void* residual, void* pre_out, void* workspace,
                       size_t workspace_bytes, void* stream);
/* inputs fp32, true fp32 MFMA (no reduced-precision path); out_dtype must be DMLHIP_F32 */
/* Several products of identical shape, strides and epilogue (alpha, column bias) on different tensors in one
 * launch: groups <= DMLHIP_GROUP_MAX, tensor i uses a[i], b[i], c[i], bias[i] (bias may be NULL: none). This is
 * HorizontalEinsumFusion's purpose (daceml/transformation/einsum_fusion.py:102-151: the three Q/K/V projections of
 * an attention block as one contraction) without requiring the operands to be adjacent in memory. d->batch[0]
 * must be 1 and d->beta 0; no residual / pre-activation / activation. Falls back to `groups` separate calls of
 * dmlhip_gemm_f16_ws (with the given workspace) when one launch is not possible. */
#define DMLHIP_GROUP_MAX 4
int dmlhip_gemm_f16_grouped(const dmlhip_gemm_desc* d, int groups, const void* const* a,
                            const void* const* b, void* const* c, const void* const* bias,
                            void* workspace, size_t workspace_bytes, void* stream);
/* dmlhip_gemm_f16_grouped without bias, plus a second result per group: asum[i][m] = sum over k of a[i][m, k]
 * (element type asum_dtype). For a weight gradient dW = dY^T X this is the bias gradient, i.e. the ReduceSum node
 * that accompanies the two Einsum nodes of DefaultEinsumBackward's callers
 * (daceml/autodiff/implementations/onnx_ops.py:54-138) — produced inside the contraction from the operand tiles
 * that are in LDS anyway instead of by another pass over dY. groups may be 1. Unbatched products only; a[i] must be
 * stored as a dense [k, m] matrix (a_stride_m == 1, a_stride_k == m). Needs a workspace of
 * dmlhip_gemm_f16_grouped_asum_workspace_bytes(d) for the case that one launch is not possible. */
size_t dmlhip_gemm_f16_grouped_asum_workspace_bytes(const dmlhip_gemm_desc* d);
int dmlhip_gemm_f16_grouped_asum(const dmlhip_gemm_desc* d, int groups, const void* const* a,
                                 const void* const* b, void* const* c, void* const* asum, int asum_dtype,
                                 void* workspace, size_t workspace_bytes, void* stream);
/* c = alpha * sum_i a[i] b[i] (+ column bias) (+ residual): `groups` products of identical shape and strides that
 * are summed — the operand pairs are concatenated along K inside one launch, so the partial products never reach
 * memory. This is what autodiff's gradient accumulation (an ONNXSum over the contributions of several consumers,
 * daceml/autodiff/backward_pass_generator.py:715-752) amounts to when the contributions are contractions, e.g. the
 * input gradient of the Q/K/V projections. d->beta must be 0 and d->act NONE. Falls back to `groups` accumulating
 * calls of dmlhip_gemm_f16 when one launch is not possible. */
int dmlhip_gemm_f16_ksum(const dmlhip_gemm_desc* d, int groups, const void* const* a, const void* const* b,
                         void* c, const void* bias, const void* residual, void* stream);
int dmlhip_gemm_f32(const dmlhip_gemm_desc* desc, const void* a, const void* b, void* c,
                    const void* bias, const void* residual, void* pre_out, void* stream);

/* ------------------------------------------------------------------ Conv
 * ONNX Conv, 2-D, NCHW / OIHW, cross-correlation:
 *   Y[b,m,oy,ox] = B[m] + sum_{c,hy,hx} W[m,c,hy,hx] * X[b, g*C/G+c, oy*sy-pt+hy*dy, ox*sx-pl+hx*dx]
 * PureConv2D (img_op_implementations.py:164-330) covers stride 1 / no pad / group 1; the
 * general attribute handling follows CudnnConvolution (cudnn_implementations.py:148-275,
 * symmetric pads, groups incl. depthwise) and the output-size rule of
 * shape_inference/symbolic_shape_infer.py:466-526. bias may be NULL.
 * act: a DMLHIP_ACT_* code applied to the result (e.g. SWISH = the Sigmoid+Mul pair that
 * follows the conv in the exported graph, fused). */
typedef struct dmlhip_conv2d_desc {
    int64_t n, c, h, w;       /* X */
    int64_t m, kh, kw;        /* W is [m, c/group, kh, kw] */
    int64_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w, group;
    int act;
} dmlhip_conv2d_desc;
int dmlhip_conv2d_out_shape(const dmlhip_conv2d_desc* d, int64_t* oh, int64_t* ow);
int dmlhip_conv2d_f32(const dmlhip_conv2d_desc* d, const void* x, const void* w,
                      const void* bias, void* y, void* stream);
int dmlhip_conv2d_f16(const dmlhip_conv2d_desc* d, const void* x, const void* w,
                      const void* bias, void* y, void* stream);
/* Y = Conv1x1(X * gate) with gate [n, c] (the [n, c, 1, 1] squeeze-excite factor broadcast over the pixels):
 * the Mul node (pure_implementations.py:86-88) in front of a pointwise Conv folded into the conv's read of X.
 * Only 1x1 / stride 1 / no padding / group 1 with c % 32 == 0, h*w % 4 == 0, h*w >= 128 (DMLHIP_ERR_UNSUPPORTED
 * otherwise: the caller keeps Mul and Conv separate). */
int dmlhip_conv2d_gated_f32(const dmlhip_conv2d_desc* d, const void* x, const void* gate,
                            const void* w, const void* bias, void* y, void* stream);
/* A pointwise convolution + activation followed by a 3x3 depthwise convolution + activation — the expand and
 * depthwise stages of an MBConv block, i.e. two Conv nodes (PureConv2D / CudnnConvolution,
 * img_op_implementations.py:164-330, cudnn_implementations.py:123-410) with their Swish chains — in one kernel:
 * the expanded tensor stays in LDS. pw: 1x1, stride 1, no padding, group 1, c % 16 == 0, m % 32 == 0; dw: the
 * pointwise output as input, 3x3, padding 1, stride 1 or 2, group = channels. act of each descriptor: NONE, SWISH,
 * RELU. DMLHIP_ERR_UNSUPPORTED otherwise (the caller keeps the two convolutions). fp32. */
int dmlhip_conv2d_expand_depthwise_f32(const dmlhip_conv2d_desc* pw, const dmlhip_conv2d_desc* dw, const void* x,
                                       const void* w_pw, const void* b_pw, const void* w_dw, const void* b_dw,
                                       void* y, void* stream);
/* LDS bytes the smallest row strip of dmlhip_conv2d_expand_depthwise_f32 needs for images `w` wide with `cin` input
 * channels and depthwise stride `stride`; 0 when no strip fits (the call would return DMLHIP_ERR_UNSUPPORTED). */
size_t dmlhip_conv2d_expand_depthwise_lds_bytes(int64_t w, int64_t cin, int64_t stride);
/* cudnnConvolutionBackwardData / BackwardFilter (autodiff/implementations/onnx_ops.py:663-703)
 * and the ATen depthwise backward (onnx_ops.py:1201-1231). dw is overwritten. The bias
 * gradient is dmlhip_reduce over [n, m, oh*ow] done by the caller (two reduce calls). */
int dmlhip_conv2d_backward_data_f32(const dmlhip_conv2d_desc* d, const void* dy, const void* w,
                                    void* dx, void* stream);
size_t dmlhip_conv2d_backward_weight_workspace_bytes(const dmlhip_conv2d_desc* d);
int dmlhip_conv2d_backward_weight_f32(const dmlhip_conv2d_desc* d, const void* x,
                                      const void* dy, void* dw, void* workspace,
                                      size_t workspace_bytes, void* stream);

/* ---- fused attention ----------------------------------------------------------------------
 * O = softmax(scale * Q K^T, over keys) V for fp16 tensors, computed without writing the
 * [seq_q, seq_k] scores to memory. Replaces the node chain the reference expands separately:
 * Einsum / MatMul(Q, K) (pure_implementations.py:111-252), the scalar Mul / Div (:76-93),
 * Softmax(axis=-1) (:309-319) and Einsum(P, V); the backward entry point replaces the nodes
 * DefaultEinsumBackward and DefaultSoftmaxBackward emit for that chain
 * (autodiff/implementations/onnx_ops.py:25-138, 237-275). No dropout; the *_masked_* entry
 * points below add a mask row to the scaled scores first.
 * Tensors are [batch0, batch1, seq, head_dim] views: element strides for batch0, batch1 and
 * seq are given per tensor (multiples of 8), head_dim is contiguous and must be 64.
 * lse (optional in forward, required by backward): fp32 [batch0, batch1, seq_q] dense,
 * lse = log(sum_k exp(scale * q.k)) per query row. scale must be positive. */
typedef struct dmlhip_attention_desc {
    int64_t batch[2];
    int64_t seq_q, seq_k, head_dim;
    int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];
    float scale;
} dmlhip_attention_desc;
int dmlhip_attention_f16(const dmlhip_attention_desc* d, const void* q, const void* k,
                         const void* v, void* o, void* lse, void* stream);
/* grad: strides of dq / dk / dv / do in the q / k / v / o slots (extents and scale are taken
 * from d). workspace: dmlhip_attention_backward_workspace_bytes(d) bytes (row dots do.o). */
size_t dmlhip_attention_backward_workspace_bytes(const dmlhip_attention_desc* d);
int dmlhip_attention_backward_f16(const dmlhip_attention_desc* d,
                                  const dmlhip_attention_desc* grad, const void* q,
                                  const void* k, const void* v, const void* o, const void* lse,
                                  const void* d_o, void* dq, void* dk, void* dv,
                                  void* workspace, size_t workspace_bytes, void* stream);
/* The same with an additive mask between the scaling and the softmax - the elementwise Add of
 * pure_implementations.py:34-36 as the exporter places it in a BERT encoder (scores + mask, mask
 * [batch, 1, 1, keys]): O = softmax(scale * Q K^T + mask, over keys) V. mask: fp16, one row of seq_k
 * contiguous values per (batch0, batch1), the same for every query; row (b0, b1) starts at
 * mask + b0 * mask_stride[0] + b1 * mask_stride[1] elements (0 = broadcast over that dimension;
 * multiples of 4; mask 8-byte aligned). Values may be -inf; a query row whose keys are all at -inf
 * yields NaN, as the reference's Softmax does. The backward treats the mask as a constant (no gradient
 * for it) and must be given the mask the forward call was given. */
int dmlhip_attention_masked_f16(const dmlhip_attention_desc* d, const void* q, const void* k,
                                const void* v, const void* mask, const int64_t* mask_stride, void* o,
                                void* lse, void* stream);
int dmlhip_attention_masked_backward_f16(const dmlhip_attention_desc* d,
                                         const dmlhip_attention_desc* grad, const void* q,
                                         const void* k, const void* v, const void* mask,
                                         const int64_t* mask_stride, const void* o, const void* lse,
                                         const void* d_o, void* dq, void* dk, void* dv,
                                         void* workspace, size_t workspace_bytes, void* stream);

/* ---- BatchNormalization (NCHW) ------------------------------------------------------------------
 * Replaces PureBatchNormalization (daceml/onnx/op_implementations/img_op_implementations.py:333-412) and
 * CudnnBatchNormalizationTraining (daceml/onnx/op_implementations/cudnn_implementations.py:444-649);
 * backward replaces CuDNNBatchNormBackward (daceml/autodiff/implementations/onnx_ops.py:1268-1510).
 * x, y: [n, c, hw] dense; scale, bias and every statistic: [c] in the tensor's element type.
 * inference: y = (x - mean) / sqrt(var + eps) * scale + bias with the given statistics.
 * training:  saved_mean / saved_var = batch mean and biased batch variance per channel; y from those;
 *            out_mean = in_mean * momentum + saved_mean * (1 - momentum), likewise out_var (ONNX convention:
 *            `momentum` weighs the running value). out_* may alias in_*.
 * backward:  dx (tensor type, may be NULL), dscale / dbias (fp32, overwritten, may be NULL) from dy, x and the
 *            statistics saved by the training call.
 * training and backward need a workspace of dmlhip_batchnorm_workspace_bytes(n, c, hw) bytes. */
size_t dmlhip_batchnorm_workspace_bytes(int64_t n, int64_t c, int64_t hw);
int dmlhip_batchnorm_inference_f16(const void* x, const void* scale, const void* bias, const void* mean,
                                   const void* var, void* y, int64_t n, int64_t c, int64_t hw, float eps,
                                   void* stream);
int dmlhip_batchnorm_inference_f32(const void* x, const void* scale, const void* bias, const void* mean,
                                   const void* var, void* y, int64_t n, int64_t c, int64_t hw, float eps,
                                   void* stream);
int dmlhip_batchnorm_training_f16(const void* x, const void* scale, const void* bias, const void* in_mean,
                                  const void* in_var, void* y, void* out_mean, void* out_var, void* saved_mean,
                                  void* saved_var, int64_t n, int64_t c, int64_t hw, float eps, float momentum,
                                  void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_batchnorm_training_f32(const void* x, const void* scale, const void* bias, const void* in_mean,
                                  const void* in_var, void* y, void* out_mean, void* out_var, void* saved_mean,
                                  void* saved_var, int64_t n, int64_t c, int64_t hw, float eps, float momentum,
                                  void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_batchnorm_backward_f16(const void* dy, const void* x, const void* scale, const void* saved_mean,
                                  const void* saved_var, void* dx, float* dscale, float* dbias, int64_t n,
                                  int64_t c, int64_t hw, float eps, void* workspace, size_t workspace_bytes,
                                  void* stream);
int dmlhip_batchnorm_backward_f32(const void* dy, const void* x, const void* scale, const void* saved_mean,
                                  const void* saved_var, void* dx, float* dscale, float* dbias, int64_t n,
                                  int64_t c, int64_t hw, float eps, void* workspace, size_t workspace_bytes,
                                  void* stream);
/* The same three with an activation (DMLHIP_ACT_NONE, _RELU or _SWISH; anything else: DMLHIP_ERR_ENUM) applied to the
 * normalised value inside the kernel: the exported chains BatchNormalization -> Relu and BatchNormalization -> Sigmoid,
 * Mul (pure_implementations.py:556-560, 741-743, 86-88) without a second pass over the tensor. backward_act takes
 * the gradient with respect to the activated output, recomputes the normalised value from x, scale, bias and the
 * saved statistics (hence the bias argument) and returns the gradients of the fused pair. */
int dmlhip_batchnorm_inference_act_f16(const void* x, const void* scale, const void* bias, const void* mean,
                                       const void* var, void* y, int64_t n, int64_t c, int64_t hw, float eps, int act,
                                       void* stream);
int dmlhip_batchnorm_inference_act_f32(const void* x, const void* scale, const void* bias, const void* mean,
                                       const void* var, void* y, int64_t n, int64_t c, int64_t hw, float eps, int act,
                                       void* stream);
int dmlhip_batchnorm_training_act_f16(const void* x, const void* scale, const void* bias, const void* in_mean,
                                      const void* in_var, void* y, void* out_mean, void* out_var, void* saved_mean,
                                      void* saved_var, int64_t n, int64_t c, int64_t hw, float eps, float momentum,
                                      int act, void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_batchnorm_training_act_f32(const void* x, const void* scale, const void* bias, const void* in_mean,
                                      const void* in_var, void* y, void* out_mean, void* out_var, void* saved_mean,
                                      void* saved_var, int64_t n, int64_t c, int64_t hw, float eps, float momentum,
                                      int act, void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_batchnorm_backward_act_f16(const void* dy, const void* x, const void* scale, const void* bias,
                                      const void* saved_mean, const void* saved_var, void* dx, float* dscale,
                                      float* dbias, int64_t n, int64_t c, int64_t hw, float eps, int act,
                                      void* workspace, size_t workspace_bytes, void* stream);
int dmlhip_batchnorm_backward_act_f32(const void* dy, const void* x, const void* scale, const void* bias,
                                      const void* saved_mean, const void* saved_var, void* dx, float* dscale,
                                      float* dbias, int64_t n, int64_t c, int64_t hw, float eps, int act,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ diagnostics
 * Switches for tests and measurements; nothing in the reference corresponds to them (its cuDNN expansion exposes
 * `node._algorithm`, cudnn_implementations.py:131-146, for the same purpose). The two "force" switches and the
 * loader switch are per calling thread: they change only what that thread launches afterwards, and a value of
 * -1 / 0 / 1 respectively restores the default choice. The counter is process-wide and atomic. */
/* Pin the tile configuration of the fp16 contraction kernels: 0 = 128x128 tile with a 4-stage ring, 1 = 256x128,
 * 2 = 256x256, 3 = 128x128 with a 2-stage ring; -1 = chosen per problem (default). 4, 5, 6, 7 = the tiles of 2, 0, 1, 3
 * with the interleaved K loop (fragment reads and global->LDS transfers issued one at a time between the MFMAs):
 * never chosen by the library, not yet measured or validated on hardware. 8 = 128x64 tile with a 3-stage ring (twice
 * the workgroups, two per compute unit, for products that give each compute unit a single 128x128 tile), 9 = the same
 * with the interleaved loop: likewise. Products with row sums or K-concatenated operand pairs exist on the 128x128 tile
 * only: 5 and 7 run them with the interleaved loop, 4, 6, 8 and 9 leave them on the plain one. */
void dmlhip_debug_force_gemm_config(int cfg);
/* 0: the fp16 contractions stage their operands through registers instead of loading them straight into LDS;
 * 1 = default. */
void dmlhip_debug_gemm_direct_lds(int on);
/* Per-workgroup timing of the pipelined fp16 contraction kernel: with a device buffer of 4 x 8 bytes per workgroup of
 * the next launches set here, every workgroup stores four readings of the 100 MHz wall clock (start, first tile in
 * LDS, end of the K loop, end of the epilogue) at buffer[4 * workgroup]; NULL (default) switches it off. The caller
 * sizes the buffer for the largest grid it launches. Per calling thread. */
void dmlhip_debug_gemm_trace(void* buffer);
/* Number of grouped / K-concatenated / row-sum contraction calls that went out as one launch so far. */
long long dmlhip_debug_grouped_single_launches(void);
/* Run dmlhip_conv2d_expand_depthwise_f32 on its strip kernel with this output-row strip height (used if it fits LDS);
 * 0 = default (the library's choice of kernel and geometry). */
void dmlhip_debug_force_fused_strip(int toh);
/* dmlhip_conv2d_expand_depthwise_f32 with a rolling window instead of strips: a workgroup walks down a segment of output
 * rows with the expanded rows in a ring in LDS, half of its wavefronts expanding the next rows while the other half runs
 * the stencil. This is what the library runs; the switch pins its geometry. rows: 0 = the library's choice (default: the
 * most output rows per batch whose ring lets two workgroups share a compute unit's LDS, else the most that fit), -1 = as
 * many output rows per batch as fit LDS, > 0 = at most that many, -2 = the strip kernel; waves: 8 or 16 wavefronts per
 * workgroup. Shapes of which not one row fits LDS run on the strips. Per calling thread. */
void dmlhip_debug_fused_rolling(int rows, int waves);
/* Where the attention workgroups' time goes: with a non-NULL buffer (device memory, 16 x 8 bytes per workgroup) thread 0
 * of every workgroup stores readings of the 100 MHz wall clock: [0] start, [1] first tile in LDS, [2 + j] end of tile j
 * (j < 12), [15] end. A forward call has batch0 x batch1 x ceil(seq_q / 128) workgroups; a backward call writes the
 * readings of its first kernel (dQ, as many workgroups as forward) and behind them those of the second (dK / dV:
 * batch0 x batch1 x ceil(seq_k / 128) workgroups). NULL (default) = off. Per calling thread. */
void dmlhip_debug_attention_trace(void* buffer);

#ifdef __cplusplus
}
#endif
#endif /* DACEML_HIP_H */
