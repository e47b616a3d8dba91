"""ctypes binding of libdaceml_hip.so (declared in include/daceml_hip.h).

The library is the only compute path of this package: if it is missing the import of any
kernel wrapper raises, there is no eager / CPU fallback.
"""
import ctypes
import os
import sys
from ctypes import (POINTER, Structure, c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libdaceml_hip.so")

OK = 0
ERR_NULL, ERR_SHAPE, ERR_UNSUPPORTED, ERR_ALIGN, ERR_WORKSPACE, ERR_ENUM = -1, -2, -3, -4, -5, -6
F16, F32 = 0, 1
ADD, SUB, MUL, DIV, POW = range(5)
MULTI_MAX = 8  # DMLHIP_MULTI_MAX
GROUP_MAX = 4  # DMLHIP_GROUP_MAX
(ERF, SQRT, EXP, LOG, TANH, RELU, SIGMOID, RECIPROCAL, GELU, SWISH, SCALE, IDENTITY) = range(12)
RSUM, RMAX, RMIN, RMEAN = range(4)
ACT_NONE, ACT_GELU, ACT_SWISH, ACT_SIGMOID, ACT_RELU = range(5)
MAX_DIMS = 6


class GemmDesc(Structure):
    """struct dmlhip_gemm_desc"""
    _fields_ = [
        ("m", c_int64), ("n", c_int64), ("k", c_int64),
        ("batch", c_int64 * 3),
        ("a_stride_m", c_int64), ("a_stride_k", c_int64), ("a_stride_batch", c_int64 * 3),
        ("b_stride_k", c_int64), ("b_stride_n", c_int64), ("b_stride_batch", c_int64 * 3),
        ("c_stride_m", c_int64), ("c_stride_batch", c_int64 * 3),
        ("alpha", c_float), ("beta", c_float),
        ("out_dtype", c_int), ("bias_dtype", c_int), ("act", c_int), ("bias_along_m", c_int),
    ]


class Conv2dDesc(Structure):
    """struct dmlhip_conv2d_desc"""
    _fields_ = [
        ("n", c_int64), ("c", c_int64), ("h", c_int64), ("w", c_int64),
        ("m", c_int64), ("kh", c_int64), ("kw", c_int64),
        ("stride_h", c_int64), ("stride_w", c_int64), ("pad_h", c_int64), ("pad_w", c_int64),
        ("dil_h", c_int64), ("dil_w", c_int64), ("group", c_int64),
        ("act", c_int),
    ]


class AttentionDesc(Structure):
    """struct dmlhip_attention_desc"""
    _fields_ = [
        ("batch", c_int64 * 2), ("seq_q", c_int64), ("seq_k", c_int64), ("head_dim", c_int64),
        ("q_stride", c_int64 * 3), ("k_stride", c_int64 * 3), ("v_stride", c_int64 * 3), ("o_stride", c_int64 * 3),
        ("scale", c_float),
    ]


_P = c_void_p
_I64P = POINTER(c_int64)

# name -> (restype, argtypes); mirrors include/daceml_hip.h declaration by declaration.
SIGNATURES = {
    "dmlhip_version": (c_int, []),
    "dmlhip_last_error_string": (c_char_p, []),
    "dmlhip_softmax_f16": (c_int, [_P, _P, c_int64, c_int64, _P]),
    "dmlhip_softmax_f32": (c_int, [_P, _P, c_int64, c_int64, _P]),
    "dmlhip_softmax_backward_f16": (c_int, [_P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_softmax_backward_f32": (c_int, [_P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_layernorm_f16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_float, _P]),
    "dmlhip_layernorm_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_float, _P]),
    "dmlhip_layernorm_backward_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "dmlhip_layernorm_backward_f16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, _P, c_size_t, _P]),
    "dmlhip_layernorm_backward_grads_f16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int64, c_int64, _P, c_size_t,
                                                    _P]),
    "dmlhip_layernorm_backward_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, _P, c_size_t, _P]),
    "dmlhip_layernorm_backward_noalloc_max_bytes": (c_size_t, []),
    "dmlhip_layernorm_backward_noalloc_f16": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_batchnorm_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "dmlhip_batchnorm_inference_f16": (c_int, [_P] * 6 + [c_int64, c_int64, c_int64, c_float, _P]),
    "dmlhip_batchnorm_inference_f32": (c_int, [_P] * 6 + [c_int64, c_int64, c_int64, c_float, _P]),
    "dmlhip_batchnorm_training_f16": (c_int, [_P] * 10 + [c_int64, c_int64, c_int64, c_float, c_float, _P, c_size_t, _P]),
    "dmlhip_batchnorm_training_f32": (c_int, [_P] * 10 + [c_int64, c_int64, c_int64, c_float, c_float, _P, c_size_t, _P]),
    "dmlhip_batchnorm_backward_f16": (c_int, [_P] * 8 + [c_int64, c_int64, c_int64, c_float, _P, c_size_t, _P]),
    "dmlhip_batchnorm_backward_f32": (c_int, [_P] * 8 + [c_int64, c_int64, c_int64, c_float, _P, c_size_t, _P]),
    "dmlhip_batchnorm_inference_act_f16": (c_int, [_P] * 6 + [c_int64, c_int64, c_int64, c_float, c_int, _P]),
    "dmlhip_batchnorm_inference_act_f32": (c_int, [_P] * 6 + [c_int64, c_int64, c_int64, c_float, c_int, _P]),
    "dmlhip_batchnorm_training_act_f16": (c_int, [_P] * 10 + [c_int64, c_int64, c_int64, c_float, c_float, c_int, _P,
                                                              c_size_t, _P]),
    "dmlhip_batchnorm_training_act_f32": (c_int, [_P] * 10 + [c_int64, c_int64, c_int64, c_float, c_float, c_int, _P,
                                                              c_size_t, _P]),
    "dmlhip_batchnorm_backward_act_f16": (c_int, [_P] * 9 + [c_int64, c_int64, c_int64, c_float, c_int, _P, c_size_t, _P]),
    "dmlhip_batchnorm_backward_act_f32": (c_int, [_P] * 9 + [c_int64, c_int64, c_int64, c_float, c_int, _P, c_size_t, _P]),
    "dmlhip_binary_f16": (c_int, [c_int, _P, _P, _P, c_int, _I64P, _I64P, _I64P, _P]),
    "dmlhip_binary_f32": (c_int, [c_int, _P, _P, _P, c_int, _I64P, _I64P, _I64P, _P]),
    "dmlhip_unary_f16": (c_int, [c_int, _P, _P, c_int64, c_float, _P]),
    "dmlhip_unary_f32": (c_int, [c_int, _P, _P, c_int64, c_float, _P]),
    "dmlhip_unary_backward_f16": (c_int, [c_int, _P, _P, _P, c_int64, c_float, _P]),
    "dmlhip_unary_backward_f32": (c_int, [c_int, _P, _P, _P, c_int64, c_float, _P]),
    "dmlhip_sum_f16": (c_int, [POINTER(c_void_p), c_int, _P, c_int64, _P]),
    "dmlhip_sum_f32": (c_int, [POINTER(c_void_p), c_int, _P, c_int64, _P]),
    "dmlhip_bias_gelu_f16": (c_int, [_P, _P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_bias_gelu_f32": (c_int, [_P, _P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_cast": (c_int, [c_int, c_int, _P, _P, c_int64, _P]),
    "dmlhip_reduce_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "dmlhip_reduce_f16": (c_int, [c_int, _P, _P, c_int, c_int64, c_int64, c_int64, _P, c_size_t, _P]),
    "dmlhip_reduce_f32": (c_int, [c_int, _P, _P, c_int, c_int64, c_int64, c_int64, _P, c_size_t, _P]),
    "dmlhip_row_affine_f16": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_row_affine_f32": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_row_dot_f16": (c_int, [_P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_row_dot_f32": (c_int, [_P, _P, _P, c_int64, c_int64, _P]),
    "dmlhip_transpose_f16": (c_int, [_P, _P, c_int, _I64P, _I64P, _P]),
    "dmlhip_transpose_f32": (c_int, [_P, _P, c_int, _I64P, _I64P, _P]),
    "dmlhip_maxpool2d_f16": (c_int, [_P, _P] + [c_int64] * 7 + [_P]),
    "dmlhip_maxpool2d_f32": (c_int, [_P, _P] + [c_int64] * 7 + [_P]),
    "dmlhip_maxpool2d_backward_f16": (c_int, [_P, _P, _P] + [c_int64] * 7 + [_P]),
    "dmlhip_maxpool2d_backward_f32": (c_int, [_P, _P, _P] + [c_int64] * 7 + [_P]),
    "dmlhip_pad_constant_f16": (c_int, [_P, _P, c_int, _I64P, _I64P, _I64P, c_float, _P]),
    "dmlhip_pad_constant_f32": (c_int, [_P, _P, c_int, _I64P, _I64P, _I64P, c_float, _P]),
    "dmlhip_gemm_f16": (c_int, [POINTER(GemmDesc), _P, _P, _P, _P, _P, _P, _P]),
    "dmlhip_gemm_f16_workspace_bytes": (c_size_t, [POINTER(GemmDesc)]),
    "dmlhip_gemm_f16_ws": (c_int, [POINTER(GemmDesc), _P, _P, _P, _P, _P, _P, _P, c_size_t, _P]),
    "dmlhip_gemm_f16_grouped": (c_int, [POINTER(GemmDesc), c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                        POINTER(c_void_p), _P, c_size_t, _P]),
    "dmlhip_gemm_f16_grouped_asum_workspace_bytes": (c_size_t, [POINTER(GemmDesc)]),
    "dmlhip_gemm_f16_grouped_asum": (c_int, [POINTER(GemmDesc), c_int, POINTER(c_void_p), POINTER(c_void_p),
                                             POINTER(c_void_p), POINTER(c_void_p), c_int, _P, c_size_t, _P]),
    "dmlhip_gemm_f16_ksum": (c_int, [POINTER(GemmDesc), c_int, POINTER(c_void_p), POINTER(c_void_p), _P, _P, _P, _P]),
    "dmlhip_gemm_f32": (c_int, [POINTER(GemmDesc), _P, _P, _P, _P, _P, _P, _P]),
    "dmlhip_conv2d_out_shape": (c_int, [POINTER(Conv2dDesc), _I64P, _I64P]),
    "dmlhip_conv2d_f32": (c_int, [POINTER(Conv2dDesc), _P, _P, _P, _P, _P]),
    "dmlhip_conv2d_f16": (c_int, [POINTER(Conv2dDesc), _P, _P, _P, _P, _P]),
    "dmlhip_conv2d_gated_f32": (c_int, [POINTER(Conv2dDesc), _P, _P, _P, _P, _P, _P]),
    "dmlhip_conv2d_expand_depthwise_f32": (c_int, [POINTER(Conv2dDesc), POINTER(Conv2dDesc), _P, _P, _P, _P, _P, _P, _P]),
    "dmlhip_conv2d_backward_data_f32": (c_int, [POINTER(Conv2dDesc), _P, _P, _P, _P]),
    "dmlhip_conv2d_backward_weight_workspace_bytes": (c_size_t, [POINTER(Conv2dDesc)]),
    "dmlhip_conv2d_backward_weight_f32": (c_int, [POINTER(Conv2dDesc), _P, _P, _P, _P, c_size_t, _P]),
    "dmlhip_reduce_sum_multi_workspace_bytes": (c_size_t, [c_int, _I64P, _I64P]),
    "dmlhip_reduce_sum_multi_f16": (c_int, [c_int, POINTER(c_void_p), POINTER(c_void_p), c_int, _I64P, _I64P, _P, c_size_t,
                                            _P]),
    "dmlhip_reduce_sum_multi_f32": (c_int, [c_int, POINTER(c_void_p), POINTER(c_void_p), c_int, _I64P, _I64P, _P, c_size_t,
                                            _P]),
    "dmlhip_attention_f16": (c_int, [POINTER(AttentionDesc), _P, _P, _P, _P, _P, _P]),
    "dmlhip_attention_backward_workspace_bytes": (c_size_t, [POINTER(AttentionDesc)]),
    "dmlhip_attention_backward_f16": (c_int, [POINTER(AttentionDesc), POINTER(AttentionDesc), _P, _P, _P, _P, _P, _P, _P,
                                              _P, _P, _P, c_size_t, _P]),
    "dmlhip_attention_masked_f16": (c_int, [POINTER(AttentionDesc), _P, _P, _P, _P, _I64P, _P, _P, _P]),
    "dmlhip_attention_masked_backward_f16": (c_int, [POINTER(AttentionDesc), POINTER(AttentionDesc), _P, _P, _P, _P, _I64P,
                                                     _P, _P, _P, _P, _P, _P, _P, c_size_t, _P]),
    # diagnostics (switches for tests and measurements, declared at the end of the header)
    "dmlhip_conv2d_expand_depthwise_lds_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "dmlhip_debug_force_gemm_config": (None, [c_int]),
    "dmlhip_debug_gemm_direct_lds": (None, [c_int]),
    "dmlhip_debug_grouped_single_launches": (ctypes.c_longlong, []),
    "dmlhip_debug_force_fused_strip": (None, [c_int]),
    "dmlhip_debug_fused_rolling": (None, [c_int, c_int]),
    "dmlhip_debug_attention_trace": (None, [c_void_p]),
    "dmlhip_debug_gemm_trace": (None, [c_void_p]),
}

_lib = None


class HipLibraryMissing(RuntimeError):
    pass


class HipKernelError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("libdaceml_hip status %d: %s" % (status, message))
        self.status = status


def load():
    """Load the shared library once and attach the signatures. Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipLibraryMissing(
            "%s not found. Build it with `python -m daceml_amd.csrc.build` (needs hipcc); "
            "this package has no fallback compute path." % LIB_PATH)
    # A process that uses PyTorch must have PyTorch's HIP runtime loaded before this library, so that both bind to the
    # same one: loaded the other way round, launches on torch's streams fail with "no ROCm-capable device is detected".
    if "torch" not in sys.modules:
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error() -> str:
    return load().dmlhip_last_error_string().decode("utf-8", "replace")


def check(status: int) -> None:
    if status != 0:
        raise HipKernelError(status, last_error())


def i64_array(values):
    return (c_int64 * len(values))(*[int(v) for v in values])
