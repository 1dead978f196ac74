"""ctypes binding of libnncase_hip.so -- the same C ABI a C# `[DllImport("nncase_hip")]`
or the native `hip` runtime module would bind (include/nncase_hip.h).

There is no CPU fallback: if the library has not been built, or no gfx950 device is
present, creating a Context raises.
"""
from __future__ import annotations

import ctypes as C
import errno
import weakref
import os
from typing import Optional, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnncase_hip.so")

# nncase typecodes (src/Native/include/nncase/runtime/typecodes.def)
DT_I8, DT_I16, DT_I32, DT_U8, DT_F16, DT_F32 = 0x02, 0x03, 0x04, 0x06, 0x0A, 0x0B
NP_TO_DT = {np.dtype(np.int8): DT_I8, np.dtype(np.int16): DT_I16, np.dtype(np.int32): DT_I32,
            np.dtype(np.uint8): DT_U8, np.dtype(np.float16): DT_F16, np.dtype(np.float32): DT_F32}
DT_TO_NP = {v: k for k, v in NP_TO_DT.items()}
FLT_MAX = float(np.finfo(np.float32).max)

ERR_DATATYPE_MISMATCH, ERR_SHAPE_MISMATCH, ERR_INVALID_MEMORY_LOCATION, ERR_HIP_BASE = 0x05, 0x06, 0x07, 0x1000
ERR_INVALID_MODEL_IDENTIFIER, ERR_INVALID_MODEL_VERSION, ERR_RUNTIME_NOT_FOUND = 0x01, 0x03, 0x04


class QuantParam(C.Structure):
    """quant_param_t (src/Native/include/nncase/runtime/simple_types.h:157-165)."""
    _fields_ = [("zero_point", C.c_int32), ("scale", C.c_float)]

    def __repr__(self):
        return f"QuantParam(zero_point={self.zero_point}, scale={self.scale!r})"


class Conv2dDesc(C.Structure):
    _fields_ = [("in_channels", C.c_int32), ("out_channels", C.c_int32), ("kernel_h", C.c_int32),
                ("kernel_w", C.c_int32), ("groups", C.c_int32), ("w_qp", QuantParam), ("expected_pixels", C.c_int64)]


class Conv2dArgs(C.Structure):
    _fields_ = [("batch", C.c_int32), ("in_h", C.c_int32), ("in_w", C.c_int32),
                ("stride_h", C.c_int32), ("stride_w", C.c_int32),
                ("dilation_h", C.c_int32), ("dilation_w", C.c_int32),
                ("pad_h_before", C.c_int32), ("pad_h_after", C.c_int32),
                ("pad_w_before", C.c_int32), ("pad_w_after", C.c_int32),
                ("x_qp", QuantParam), ("y_qp", QuantParam),
                ("clamp_min", C.c_float), ("clamp_max", C.c_float), ("out_dtype", C.c_int32),
                ("residual_dev", C.c_void_p), ("residual_qp", QuantParam), ("sum_qp", QuantParam),
                ("sum_clamp_min", C.c_float), ("sum_clamp_max", C.c_float),
                ("out_channel_stride", C.c_int32), ("out_channel_offset", C.c_int32),
                ("dequantize_output", C.c_int32), ("reserved", C.c_int32)]


class QBlockDesc(C.Structure):
    _fields_ = [("in_channels", C.c_int32), ("mid_channels", C.c_int32), ("out_channels", C.c_int32),
                ("expand_w_qp", QuantParam), ("dw_w_qp", QuantParam), ("project_w_qp", QuantParam)]


class QBlockArgs(C.Structure):
    _fields_ = [("batch", C.c_int32), ("in_h", C.c_int32), ("in_w", C.c_int32), ("stride", C.c_int32),
                ("pad_h_before", C.c_int32), ("pad_h_after", C.c_int32), ("pad_w_before", C.c_int32), ("pad_w_after", C.c_int32),
                ("x_qp", QuantParam), ("expand_qp", QuantParam), ("dw_qp", QuantParam), ("y_qp", QuantParam),
                ("expand_clamp_min", C.c_float), ("expand_clamp_max", C.c_float),
                ("dw_clamp_min", C.c_float), ("dw_clamp_max", C.c_float),
                ("clamp_min", C.c_float), ("clamp_max", C.c_float),
                ("add_input", C.c_int32), ("sum_qp", QuantParam), ("sum_clamp_min", C.c_float), ("sum_clamp_max", C.c_float)]


class MatmulArgs(C.Structure):
    _fields_ = [("m", C.c_int32), ("a_qp", QuantParam), ("y_qp", QuantParam),
                ("clamp_min", C.c_float), ("clamp_max", C.c_float), ("out_dtype", C.c_int32)]


class PagedAttnArgs(C.Structure):
    _fields_ = [("batch", C.c_int32), ("num_q_heads", C.c_int32), ("num_kv_heads", C.c_int32),
                ("head_dim", C.c_int32), ("block_size", C.c_int32), ("max_blocks_per_seq", C.c_int32),
                ("num_blocks", C.c_int32), ("scale", C.c_float), ("out_dtype", C.c_int32), ("ctx_len_offset", C.c_int32)]


# name -> (restype, argtypes); every symbol include/nncase_hip.h declares
_VP, _I, _SZ = C.c_void_p, C.c_int, C.c_size_t
_I32P = C.POINTER(C.c_int32)
_I64P = C.POINTER(C.c_int64)
SYMBOLS = {
    "nncase_hip_version": (_I, []),
    "nncase_hip_ctx_create": (_I, [_I, C.POINTER(_VP)]),
    "nncase_hip_ctx_destroy": (_I, [_VP]),
    "nncase_hip_ctx_get_stream": (_I, [_VP, C.POINTER(_VP)]),
    "nncase_hip_ctx_set_stream": (_I, [_VP, _VP]),
    "nncase_hip_last_error_string": (C.c_char_p, [_VP]),
    "nncase_hip_device_info": (_I, [_VP, C.POINTER(_I), C.POINTER(_I), C.POINTER(_SZ)]),
    "nncase_hip_malloc": (_I, [_VP, _SZ, C.POINTER(_VP)]),
    "nncase_hip_free": (_I, [_VP, _VP]),
    "nncase_hip_memcpy_h2d": (_I, [_VP, _VP, _VP, _SZ]),
    "nncase_hip_memcpy_d2h": (_I, [_VP, _VP, _VP, _SZ]),
    "nncase_hip_memset": (_I, [_VP, _VP, _I, _SZ]),
    "nncase_hip_stream_sync": (_I, [_VP]),
    "nncase_hip_quantize": (_I, [_VP, _VP, _I, _VP, _I, _SZ, QuantParam]),
    "nncase_hip_dequantize": (_I, [_VP, _VP, _I, _VP, _I, _SZ, QuantParam]),
    "nncase_hip_quantize_strided": (_I, [_VP, _VP, _I, _VP, _I, C.c_int32, _I64P, _I64P, _I64P, QuantParam]),
    "nncase_hip_dequantize_strided": (_I, [_VP, _VP, _I, _VP, _I, C.c_int32, _I64P, _I64P, _I64P, QuantParam]),
    "nncase_hip_qconv2d_prepack": (_I, [_VP, C.POINTER(Conv2dDesc), _VP, _VP, C.POINTER(_VP)]),
    "nncase_hip_weights_destroy": (_I, [_VP, _VP]),
    "nncase_hip_weights_set_post_lut": (_I, [_VP, _VP, _VP, QuantParam]),
    "nncase_hip_qconv2d": (_I, [_VP, _VP, _VP, _VP, C.POINTER(Conv2dArgs)]),
    "nncase_hip_requant_plan": (_I, [C.c_float, C.c_float, QuantParam, C.c_float, C.c_float, C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "nncase_hip_requant_host": (_I, [C.c_float, C.c_float, QuantParam, C.c_float, C.c_float, _VP, _SZ, _VP, _I32P]),
    "nncase_hip_requant_host_magic": (_I, [C.c_float, C.c_float, QuantParam, C.c_float, C.c_float, _VP, _SZ, _VP, C.POINTER(C.c_float),
                                           C.POINTER(C.c_float), _I32P]),
    "nncase_hip_qblock_supported": (_I, [C.POINTER(QBlockDesc)]),
    "nncase_hip_qblock_prepack": (_I, [_VP, C.POINTER(QBlockDesc), _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(_VP)]),
    "nncase_hip_qblock_destroy": (_I, [_VP, _VP]),
    "nncase_hip_qblock": (_I, [_VP, _VP, _VP, _VP, C.POINTER(QBlockArgs)]),
    "nncase_hip_function_add_qblock": (_I, [_VP, _VP, _VP, _VP, C.POINTER(QBlockArgs)]),
    "nncase_hip_qpointwise_pair_supported": (_I, [C.c_int32, C.c_int32, C.c_int32]),
    "nncase_hip_qpointwise_pair_create": (_I, [_VP, _VP, _VP, _VP, _VP, C.POINTER(_VP)]),
    "nncase_hip_qpointwise_pair_destroy": (_I, [_VP, _VP]),
    "nncase_hip_qpointwise_pair": (_I, [_VP, _VP, _VP, _VP, _VP, C.POINTER(Conv2dArgs), C.POINTER(Conv2dArgs)]),
    "nncase_hip_function_add_qpointwise_pair": (_I, [_VP, _VP, _VP, _VP, _VP, C.POINTER(Conv2dArgs), C.POINTER(Conv2dArgs)]),
    "nncase_hip_qglobal_avgpool_qconv2d_supported": (_I, [_VP, C.POINTER(Conv2dArgs), C.c_int32, C.c_int32]),
    "nncase_hip_qglobal_avgpool_qconv2d": (_I, [_VP, _VP, C.c_int32, C.c_int32, QuantParam, _VP, _VP, C.POINTER(Conv2dArgs)]),
    "nncase_hip_function_add_qglobal_avgpool_qconv2d": (_I, [_VP, _VP, C.c_int32, C.c_int32, QuantParam, _VP, _VP, C.POINTER(Conv2dArgs)]),
    "nncase_hip_qdepthwise_pointwise_pair": (_I, [_VP, _VP, _VP, C.POINTER(Conv2dArgs), _VP, _VP, _VP, C.POINTER(Conv2dArgs), C.POINTER(Conv2dArgs)]),
    "nncase_hip_function_add_qdepthwise_pointwise_pair": (_I, [_VP, _VP, _VP, C.POINTER(Conv2dArgs), _VP, _VP, _VP, C.POINTER(Conv2dArgs),
                                                           C.POINTER(Conv2dArgs)]),
    "nncase_hip_qmatmul_prepack": (_I, [_VP, _VP, C.c_int32, C.c_int32, QuantParam, _VP, C.c_int64, C.POINTER(_VP)]),
    "nncase_hip_qmatmul": (_I, [_VP, _VP, _VP, _VP, C.POINTER(MatmulArgs)]),
    "nncase_hip_qadd": (_I, [_VP, _VP, QuantParam, _VP, QuantParam, _VP, QuantParam, C.c_float, C.c_float, _SZ]),
    "nncase_hip_qglobal_avgpool": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int32, QuantParam,
                                        QuantParam]),
    "nncase_hip_make_unary_lut": (_I, [C.c_int32, QuantParam, QuantParam, _VP]),
    "nncase_hip_lut_u8": (_I, [_VP, _VP, _VP, _SZ, _VP]),
    "nncase_hip_qconcat_channels": (_I, [_VP, C.c_int32, C.POINTER(_VP), _I32P, C.POINTER(QuantParam), _VP, QuantParam,
                                         C.c_int64]),
    "nncase_hip_resize_nearest": (_I, [_VP, _VP, _VP] + [C.c_int32] * 9),
    "nncase_hip_function_add_lut_u8": (_I, [_VP, _VP, _VP, _SZ, _VP]),
    "nncase_hip_function_add_qconcat_channels": (_I, [_VP, C.c_int32, C.POINTER(_VP), _I32P, C.POINTER(QuantParam), _VP,
                                                      QuantParam, C.c_int64]),
    "nncase_hip_function_add_resize_nearest": (_I, [_VP, _VP, _VP] + [C.c_int32] * 9),
    "nncase_hip_function_add_layout": (_I, [_VP, _VP, _VP] + [C.c_int32] * 6),
    "nncase_hip_qmaxpool2d": (_I, [_VP, _VP, _VP] + [C.c_int32] * 12 + [QuantParam, QuantParam]),
    "nncase_hip_function_add_qmaxpool2d": (_I, [_VP, _VP, _VP] + [C.c_int32] * 12 + [QuantParam, QuantParam]),
    "nncase_hip_function_add_pack": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, _I32P, C.c_int32, _I32P, _I32P]),
    "nncase_hip_function_add_quantize_pack": (_I, [_VP, _VP, _VP, C.c_int32, _I32P, C.c_int32, _I32P, _I32P, QuantParam]),
    "nncase_hip_w8a16_prepack": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.POINTER(_VP)]),
    "nncase_hip_w8a16_destroy": (_I, [_VP, _VP]),
    "nncase_hip_w8a16_gemm": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, _VP, C.c_int32]),
    "nncase_hip_rmsnorm_f16": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.c_float]),
    "nncase_hip_rope_kv_append": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs), C.c_float]),
    "nncase_hip_argmax_f32": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32]),
    "nncase_hip_embedding_f16": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32]),
    "nncase_hip_add_i32": (_I, [_VP, _VP, C.c_int32, C.c_int32]),
    "nncase_hip_function_add_w8a16_gemm": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, _VP, C.c_int32]),
    "nncase_hip_rmsnorm_w8a16_gemm": (_I, [_VP, _VP, _VP, C.c_float, _VP, _VP, C.c_int32, C.c_int32, _VP, C.c_int32]),
    "nncase_hip_function_add_rmsnorm_w8a16_gemm": (_I, [_VP, _VP, _VP, C.c_float, _VP, _VP, C.c_int32, C.c_int32, _VP, C.c_int32]),
    "nncase_hip_function_add_rmsnorm_f16": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.c_float]),
    "nncase_hip_function_add_rope_kv_append": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs), C.c_float]),
    "nncase_hip_function_add_w8a16_gemm_rope_kv_append": (_I, [_VP, _VP, _VP, C.c_float, _VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs), C.c_float]),
    "nncase_hip_w8a16_gemm_rope_kv_append": (_I, [_VP, _VP, _VP, C.c_float, _VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs), C.c_float]),
    "nncase_hip_function_add_paged_attention_decode": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs)]),
    "nncase_hip_function_add_argmax_f32": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32]),
    "nncase_hip_function_add_embedding_f16": (_I, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32]),
    "nncase_hip_function_add_add_i32": (_I, [_VP, _VP, C.c_int32, C.c_int32]),
    "nncase_hip_function_set_lane": (_I, [_VP, C.c_int32]),
    "nncase_hip_kmodel_load": (_I, [_VP, _VP, _SZ, C.POINTER(_VP)]),
    "nncase_hip_kmodel_load_function": (_I, [_VP, _VP, _SZ, _VP, _SZ, C.POINTER(_VP)]),
    "nncase_hip_kmodel_destroy": (_I, [_VP]),
    "nncase_hip_kmodel_function": (_I, [_VP, C.POINTER(_VP)]),
    "nncase_hip_kmodel_tensor": (_I, [_VP, C.c_int32, C.POINTER(_VP), _I32P, _I32P]),
    "nncase_hip_fill_queue_pool": (_I, [C.c_int]),
    "nncase_hip_release_queue_pool": (_I, [C.c_int]),
    "nncase_hip_pack": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, _I32P, C.c_int32, _I32P, _I32P]),
    "nncase_hip_unpack": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, _I32P, C.c_int32, _I32P, _I32P]),
    "nncase_hip_quantize_pack": (_I, [_VP, _VP, _VP, C.c_int32, _I32P, C.c_int32, _I32P, _I32P, QuantParam]),
    "nncase_hip_nchw_to_nhwc": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "nncase_hip_nhwc_to_nchw": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "nncase_hip_paged_attention_decode": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs)]),
    "nncase_hip_paged_attention_decode_noalloc": (_I, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, C.POINTER(PagedAttnArgs)]),
    "nncase_hip_function_create": (_I, [_VP, C.POINTER(_VP)]),
    "nncase_hip_function_destroy": (_I, [_VP]),
    "nncase_hip_function_add_quantize": (_I, [_VP, _VP, _I, _VP, _I, _SZ, QuantParam]),
    "nncase_hip_function_add_dequantize": (_I, [_VP, _VP, _I, _VP, _I, _SZ, QuantParam]),
    "nncase_hip_function_add_qconv2d": (_I, [_VP, _VP, _VP, _VP, C.POINTER(Conv2dArgs)]),
    "nncase_hip_function_add_qadd": (_I, [_VP, _VP, QuantParam, _VP, QuantParam, _VP, QuantParam, C.c_float, C.c_float,
                                          _SZ]),
    "nncase_hip_function_add_qglobal_avgpool": (_I, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                                     QuantParam, QuantParam]),
    "nncase_hip_function_size": (_I, [_VP, C.POINTER(C.c_int32)]),
    "nncase_hip_function_invoke": (_I, [_VP]),
    "nncase_hip_function_invoke_one": (_I, [_VP, C.c_int32]),
    "nncase_hip_function_capture": (_I, [_VP]),
    "nncase_hip_function_profile": (_I, [_VP, C.c_int32, C.POINTER(C.c_float)]),
    "nncase_hip_function_op_kernel": (_I, [_VP, C.c_int32, C.c_char_p, _SZ]),
}

_lib: Optional[C.CDLL] = None


def load_library() -> C.CDLL:
    """Loads the built library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m nncase_amd.build` "
                               "(there is no CPU fallback for the hip target)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the export is missing
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


class HipError(RuntimeError):
    """Mirrors the C# interop's `InvalidOperationException("Status code: N")`
    (src/Nncase.Simulator/Runtime/Interop/ErrorCode.cs:25-31)."""

    def __init__(self, code: int, where: str, detail: str = ""):
        self.code = code
        name = errno.errorcode.get(-code, "") if -code < ERR_HIP_BASE else f"hipError {-code - ERR_HIP_BASE}"
        super().__init__(f"{where}: status code {code} {name} {detail}".strip())


def fill_queue_pool(device: int = 0) -> int:
    """Creates the idle streams that fill HIP's pool of hardware queues (once per process), so that the contexts
    created afterwards get a hardware queue each; returns the number of hardware queues."""
    rc = load_library().nncase_hip_fill_queue_pool(device)
    if rc <= 0:
        raise HipError(rc, "fill_queue_pool")
    return rc


def release_queue_pool(device: int = 0) -> int:
    """Destroys the idle streams fill_queue_pool created on the device; returns how many there were."""
    rc = load_library().nncase_hip_release_queue_pool(device)
    if rc < 0:
        raise HipError(rc, "release_queue_pool")
    return rc


def qp(zero_point: int, scale: float) -> QuantParam:
    return QuantParam(int(zero_point), float(np.float32(scale)))


GEMM_PLAIN, GEMM_SWIGLU = 0, 1
MAX_LANES = 8  # NNCASE_HIP_MAX_LANES
LUT_REQUANT, LUT_SWISH = 0, 1
RESIZE_HALF_PIXEL, RESIZE_PYTORCH_HALF_PIXEL, RESIZE_ALIGN_CORNERS, RESIZE_ASYMMETRIC, RESIZE_TFCROP_AND_RESIZE = range(5)
NEAREST_ROUND_PREFER_FLOOR, NEAREST_ROUND_PREFER_CEIL, NEAREST_FLOOR, NEAREST_CEIL = range(4)


def make_unary_lut(kind: int, x_qp: "QuantParam", y_qp: "QuantParam") -> np.ndarray:
    """Host-side 256-entry table lut[v] = Q_y(f(DQ_x(v))) built by the library (same libm as the CPU kernels)."""
    lut = np.empty(256, np.uint8)
    rc = load_library().nncase_hip_make_unary_lut(kind, x_qp, y_qp, lut.ctypes.data)
    if rc != 0:
        raise HipError(rc, "make_unary_lut", "invalid kind or zero output scale")
    return lut


def requant_plan(sx, sw, y_qp: "QuantParam", clamp=(-FLT_MAX, FLT_MAX)):
    """(found, c1, c2): the one-FMA form of the u8 requantisation the kernels would use for this layer, if the
    library's host-side search proved one equal to the three-rounding sequence (host-only, no device needed)."""
    c1, c2 = C.c_float(), C.c_float()
    rc = load_library().nncase_hip_requant_plan(float(sx), float(sw), y_qp, clamp[0], clamp[1], C.byref(c1), C.byref(c2))
    if rc < 0:
        raise HipError(rc, "requant_plan", "scales outside the supported range")
    return bool(rc), c1.value, c2.value


def requant_host(acc: np.ndarray, sx, sw, y_qp: "QuantParam", clamp=(-FLT_MAX, FLT_MAX)):
    """(bytes, form): the requantised codes of int32 accumulators by the form the kernels pick (1 = FMA form)."""
    acc = np.ascontiguousarray(acc, np.int32)
    out = np.empty(acc.shape, np.uint8)
    form = C.c_int32()
    rc = load_library().nncase_hip_requant_host(float(sx), float(sw), y_qp, clamp[0], clamp[1], acc.ctypes.data, acc.size,
                                                out.ctypes.data, C.byref(form))
    if rc != 0:
        raise HipError(rc, "requant_host", "scales outside the supported range")
    return out, form.value


def requant_host_magic(acc: np.ndarray, sx, sw, y_qp: "QuantParam", clamp=(-FLT_MAX, FLT_MAX)):
    """(bytes, m1, m2, limit) by the conversion-free form RN(fma(as_float(0x4B400000 + acc), m1, m2)) that the dense row /
    window kernels and the stride-2 depthwise kernel use where the library's search found one, or None."""
    acc = np.ascontiguousarray(acc, np.int32)
    out = np.empty(acc.shape, np.uint8)
    m1, m2, limit = C.c_float(), C.c_float(), C.c_int32()
    rc = load_library().nncase_hip_requant_host_magic(float(sx), float(sw), y_qp, clamp[0], clamp[1], acc.ctypes.data, acc.size,
                                                      out.ctypes.data, C.byref(m1), C.byref(m2), C.byref(limit))
    if rc < 0:
        raise HipError(rc, "requant_host_magic", "scales outside the supported range")
    return (out, m1.value, m2.value, limit.value) if rc else None


def _concat_args(inputs, channels, in_qps):
    n = len(inputs)
    ptrs = (_VP * n)(*[None if b is None else b.ptr for b in inputs])   # None: the slice is already in place
    ch = (C.c_int32 * n)(*channels)
    qps = (QuantParam * n)(*in_qps)
    return n, ptrs, ch, qps


class DeviceBuffer:
    """An HBM allocation owned through the context (nncase_hip_malloc / _free)."""

    def __init__(self, ctx: "Context", nbytes: int):
        self.ctx, self.nbytes = ctx, int(nbytes)
        p = C.c_void_p()
        ctx._check(ctx.lib.nncase_hip_malloc(ctx.handle, max(1, self.nbytes), C.byref(p)), "malloc")
        self.ptr = p.value

    def upload(self, arr: np.ndarray) -> "DeviceBuffer":
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        self.ctx._check(self.ctx.lib.nncase_hip_memcpy_h2d(self.ctx.handle, self.ptr, arr.ctypes.data, arr.nbytes), "h2d")
        return self

    def download(self, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        self.ctx._check(self.ctx.lib.nncase_hip_memcpy_d2h(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes), "d2h")
        return out

    def fill(self, byte: int) -> "DeviceBuffer":
        self.ctx._check(self.ctx.lib.nncase_hip_memset(self.ctx.handle, self.ptr, byte, self.nbytes), "memset")
        return self

    def free(self):
        if self.ptr:
            if self.ctx.handle:
                self.ctx.lib.nncase_hip_free(self.ctx.handle, self.ptr)
            self.ptr = None

    def view(self, offset: int, nbytes: int) -> "DeviceView":
        return DeviceView(self, offset, nbytes)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class DeviceView:
    """A byte range of a DeviceBuffer (keeps the allocation alive; owns nothing)."""

    def __init__(self, base: DeviceBuffer, offset: int, nbytes: int):
        assert 0 <= offset and offset + nbytes <= base.nbytes
        self.base, self.ctx, self.nbytes = base, base.ctx, int(nbytes)
        self.ptr = base.ptr + int(offset)

    def view(self, offset: int, nbytes: int) -> "DeviceView":
        assert 0 <= offset and offset + nbytes <= self.nbytes
        return DeviceView(self.base, self.ptr - self.base.ptr + offset, nbytes)

    upload, download, fill = DeviceBuffer.upload, DeviceBuffer.download, DeviceBuffer.fill


class Weights:
    """Pre-packed constants of one conv / matmul (nncase_hip_weights_t)."""

    def __init__(self, ctx: "Context", handle, out_channels: int, kernel: Tuple[int, int], in_channels: int, groups: int):
        self.ctx, self.handle = ctx, handle
        self.out_channels, self.kernel, self.in_channels, self.groups = out_channels, kernel, in_channels, groups

    def set_post_lut(self, lut: Optional[np.ndarray], lut_qp: "QuantParam" = None):
        """Attaches a fused 256-entry byte table (make_unary_lut) applied behind the requantisation of every
        u8-output call with these weights; None detaches it."""
        if lut is None:
            self.ctx._check(self.ctx.lib.nncase_hip_weights_set_post_lut(self.ctx.handle, self.handle, None, qp(0, 1.0)), "weights_set_post_lut")
            return self
        t = np.ascontiguousarray(lut, np.uint8)
        assert t.size == 256
        self.ctx._check(self.ctx.lib.nncase_hip_weights_set_post_lut(self.ctx.handle, self.handle, t.ctypes.data, lut_qp), "weights_set_post_lut")
        return self

    def destroy(self):
        if self.handle:
            if self.ctx.handle:
                self.ctx.lib.nncase_hip_weights_destroy(self.ctx.handle, self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class QPair:
    """Two pointwise convolutions packed to run as one launch (nncase_hip_qpair_t); keeps both Weights alive."""

    def __init__(self, ctx: "Context", handle, first: "Weights", second: "Weights"):
        self.ctx, self.handle, self.first, self.second = ctx, handle, first, second

    def destroy(self):
        if self.handle:
            if self.ctx.handle:
                self.ctx.lib.nncase_hip_qpointwise_pair_destroy(self.ctx.handle, self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class QBlock:
    """Pre-packed constants of a fused expand -> depthwise -> project block (nncase_hip_qblock_t)."""

    def __init__(self, ctx: "Context", handle, channels: Tuple[int, int, int]):
        self.ctx, self.handle, self.channels = ctx, handle, channels

    def destroy(self):
        if self.handle:
            if self.ctx.handle:
                self.ctx.lib.nncase_hip_qblock_destroy(self.ctx.handle, self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def windowed_output_size(size, filt, stride, dilation, before, after) -> int:
    """src/Native/include/nncase/kernels/kernel_utils.h:86-93."""
    eff = (filt - 1) * dilation + 1
    return (size + before + after - eff + stride) // stride


class Context:
    """One device + stream (nncase_hip_ctx_t)."""

    def __init__(self, device: int = 0):
        self.lib = load_library()
        h = C.c_void_p()
        rc = self.lib.nncase_hip_ctx_create(device, C.byref(h))
        if rc != 0:
            raise HipError(rc, "nncase_hip_ctx_create", "(no gfx950 device?)")
        self.handle = h.value
        cu, khz, mem = C.c_int(), C.c_int(), C.c_size_t()
        self.lib.nncase_hip_device_info(self.handle, C.byref(cu), C.byref(khz), C.byref(mem))
        self.compute_units, self.clock_khz, self.hbm_bytes = cu.value, khz.value, mem.value

    # -- plumbing ---------------------------------------------------------------------
    def _check(self, rc: int, where: str):
        if rc != 0:
            msg = self.lib.nncase_hip_last_error_string(self.handle)
            raise HipError(rc, where, msg.decode() if msg else "")

    def _adopt(self, child):
        """Functions and loaded kmodels hold a pointer to the native context: they are destroyed with it."""
        if not hasattr(self, "_children"):
            self._children = weakref.WeakSet()
        self._children.add(child)

    def close(self):
        if getattr(self, "handle", None):
            for child in list(getattr(self, "_children", ())):
                child.destroy()
            self.lib.nncase_hip_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def stream(self) -> int:
        s = C.c_void_p()
        self._check(self.lib.nncase_hip_ctx_get_stream(self.handle, C.byref(s)), "get_stream")
        return s.value or 0

    def set_stream(self, hip_stream: int):
        self._check(self.lib.nncase_hip_ctx_set_stream(self.handle, C.c_void_p(hip_stream)), "set_stream")

    def sync(self):
        self._check(self.lib.nncase_hip_stream_sync(self.handle), "stream_sync")

    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr: np.ndarray) -> DeviceBuffer:
        arr = np.ascontiguousarray(arr)
        return DeviceBuffer(self, arr.nbytes).upload(arr)

    # -- operators (raw device pointers) ----------------------------------------------
    def quantize(self, src: DeviceBuffer, in_dtype: int, dst: DeviceBuffer, out_dtype: int, count: int, q: QuantParam):
        self._check(self.lib.nncase_hip_quantize(self.handle, src.ptr, in_dtype, dst.ptr, out_dtype, count, q), "quantize")

    def dequantize(self, src: DeviceBuffer, in_dtype: int, dst: DeviceBuffer, out_dtype: int, count: int, q: QuantParam):
        self._check(self.lib.nncase_hip_dequantize(self.handle, src.ptr, in_dtype, dst.ptr, out_dtype, count, q),
                    "dequantize")

    def _strided(self, fn, what, src, in_dtype, dst, out_dtype, shape, in_strides, out_strides, q):
        rank = len(shape)
        arr = lambda v: (C.c_int64 * max(rank, 1))(*[int(e) for e in v])
        self._check(fn(self.handle, src.ptr, in_dtype, dst.ptr, out_dtype, rank, arr(shape), arr(in_strides), arr(out_strides), q), what)

    def quantize_strided(self, src, in_dtype, dst, out_dtype, shape, in_strides, out_strides, q: QuantParam):
        """Strides in elements, as the reference's kernels take them (reference/quantize.cpp:29-47)."""
        self._strided(self.lib.nncase_hip_quantize_strided, "quantize_strided", src, in_dtype, dst, out_dtype, shape, in_strides, out_strides, q)

    def dequantize_strided(self, src, in_dtype, dst, out_dtype, shape, in_strides, out_strides, q: QuantParam):
        self._strided(self.lib.nncase_hip_dequantize_strided, "dequantize_strided", src, in_dtype, dst, out_dtype, shape, in_strides, out_strides, q)

    def prepack_conv2d(self, weights_oihw: np.ndarray, bias: Optional[np.ndarray], w_qp: QuantParam, groups: int = 1,
                       expected_pixels: int = 0) -> Weights:
        w = np.ascontiguousarray(weights_oihw, np.uint8)
        oc, gic, kh, kw = w.shape
        desc = Conv2dDesc(gic * groups, oc, kh, kw, groups, w_qp, int(expected_pixels))
        b = None if bias is None else np.ascontiguousarray(bias, np.int32)
        if b is not None:
            assert b.shape == (oc,)
        h = C.c_void_p()
        self._check(self.lib.nncase_hip_qconv2d_prepack(self.handle, C.byref(desc), w.ctypes.data,
                                                        None if b is None else b.ctypes.data, C.byref(h)), "qconv2d_prepack")
        return Weights(self, h.value, oc, (kh, kw), gic * groups, groups)

    def qconv2d(self, x: DeviceBuffer, w: Weights, y: DeviceBuffer, args: Conv2dArgs):
        self._check(self.lib.nncase_hip_qconv2d(self.handle, x.ptr, w.handle, y.ptr, C.byref(args)), "qconv2d")

    def qblock_supported(self, cin: int, mid: int, cout: int) -> bool:
        d = QBlockDesc(cin, mid, cout, qp(0, 1.0), qp(0, 1.0), qp(0, 1.0))
        return bool(self.lib.nncase_hip_qblock_supported(C.byref(d)))

    def prepack_qblock(self, w_expand, b_expand, qp_expand, w_dw, b_dw, qp_dw, w_project, b_project, qp_project) -> QBlock:
        """OIHW u8 weights [mid, in, 1, 1], [mid, 1, 3, 3], [out, mid, 1, 1] and int32 biases (or None)."""
        we, wd, wp = (np.ascontiguousarray(w, np.uint8) for w in (w_expand, w_dw, w_project))
        mid, cin = we.shape[:2]
        cout = wp.shape[0]
        assert we.shape == (mid, cin, 1, 1) and wd.shape == (mid, 1, 3, 3) and wp.shape == (cout, mid, 1, 1)
        bs = [None if b is None else np.ascontiguousarray(b, np.int32) for b in (b_expand, b_dw, b_project)]
        for b, n in zip(bs, (mid, mid, cout)):
            assert b is None or b.shape == (n,)
        bp = [None if b is None else b.ctypes.data for b in bs]
        desc = QBlockDesc(cin, mid, cout, qp_expand, qp_dw, qp_project)
        h = C.c_void_p()
        self._check(self.lib.nncase_hip_qblock_prepack(self.handle, C.byref(desc), we.ctypes.data, bp[0], wd.ctypes.data, bp[1],
                                                       wp.ctypes.data, bp[2], C.byref(h)), "qblock_prepack")
        return QBlock(self, h.value, (cin, mid, cout))

    def qblock(self, x, blk: QBlock, y, args: QBlockArgs):
        self._check(self.lib.nncase_hip_qblock(self.handle, x.ptr, blk.handle, y.ptr, C.byref(args)), "qblock")

    def qpointwise_pair_supported(self, cin: int, mid: int, cout: int) -> bool:
        return bool(self.lib.nncase_hip_qpointwise_pair_supported(cin, mid, cout))

    def prepack_qpointwise_pair(self, first: Weights, first_oihw: np.ndarray, second: Weights, second_oihw: np.ndarray) -> QPair:
        """`first` / `second` are the prepack_conv2d handles of the two 1x1 convolutions (bias, quantisation, tables),
        the arrays their OIHW u8 weights [mid, in, 1, 1] and [out, mid, 1, 1] once more."""
        wa, wb = (np.ascontiguousarray(w, np.uint8) for w in (first_oihw, second_oihw))
        assert wa.shape[2:] == (1, 1) and wb.shape[2:] == (1, 1)
        h = C.c_void_p()
        self._check(self.lib.nncase_hip_qpointwise_pair_create(self.handle, first.handle, wa.ctypes.data, second.handle, wb.ctypes.data,
                                                               C.byref(h)), "qpointwise_pair_create")
        return QPair(self, h.value, first, second)

    def qpointwise_pair(self, x, pair: QPair, y1, y2, first_args: Conv2dArgs, second_args: Conv2dArgs):
        self._check(self.lib.nncase_hip_qpointwise_pair(self.handle, x.ptr, pair.handle, y1.ptr, y2.ptr, C.byref(first_args),
                                                        C.byref(second_args)), "qpointwise_pair")

    def qglobal_avgpool_qconv2d_supported(self, w: Weights, args: Conv2dArgs, h: int, w_: int) -> bool:
        return bool(self.lib.nncase_hip_qglobal_avgpool_qconv2d_supported(w.handle, C.byref(args), h, w_))

    def qglobal_avgpool_qconv2d(self, x, h: int, w_: int, x_qp: QuantParam, w: Weights, y, args: Conv2dArgs):
        """Global average pool of x [batch, h, w, channels] and the 1x1 convolution on the pooled pixel, one launch."""
        self._check(self.lib.nncase_hip_qglobal_avgpool_qconv2d(self.handle, x.ptr, h, w_, x_qp, w.handle, y.ptr, C.byref(args)),
                    "qglobal_avgpool_qconv2d")

    def qdepthwise_pointwise_pair(self, x, dw: Weights, dw_args: Conv2dArgs, pair: QPair, y1, y2, first_args: Conv2dArgs,
                                  second_args: Conv2dArgs):
        """x is the 3x3 depthwise convolution's input; its result only exists inside the launch."""
        self._check(self.lib.nncase_hip_qdepthwise_pointwise_pair(self.handle, x.ptr, dw.handle, C.byref(dw_args), pair.handle, y1.ptr, y2.ptr,
                                                                  C.byref(first_args), C.byref(second_args)), "qdepthwise_pointwise_pair")

    def prepack_matmul(self, b_kn: np.ndarray, bias: Optional[np.ndarray], b_qp: QuantParam, expected_rows: int = 0) -> Weights:
        b = np.ascontiguousarray(b_kn, np.uint8)
        k, n = b.shape
        bi = None if bias is None else np.ascontiguousarray(bias, np.int32)
        h = C.c_void_p()
        self._check(self.lib.nncase_hip_qmatmul_prepack(self.handle, b.ctypes.data, k, n, b_qp,
                                                        None if bi is None else bi.ctypes.data, int(expected_rows), C.byref(h)),
                    "qmatmul_prepack")
        return Weights(self, h.value, n, (1, 1), k, 1)

    def qmatmul(self, a: DeviceBuffer, w: Weights, y: DeviceBuffer, args: MatmulArgs):
        self._check(self.lib.nncase_hip_qmatmul(self.handle, a.ptr, w.handle, y.ptr, C.byref(args)), "qmatmul")

    def qadd(self, a: DeviceBuffer, a_qp, b: DeviceBuffer, b_qp, out: DeviceBuffer, y_qp, count: int,
             clamp=(-FLT_MAX, FLT_MAX)):
        self._check(self.lib.nncase_hip_qadd(self.handle, a.ptr, a_qp, b.ptr, b_qp, out.ptr, y_qp, clamp[0], clamp[1], count),
                    "qadd")

    def qglobal_avgpool(self, x: DeviceBuffer, out: DeviceBuffer, batch, h, w, channels, x_qp, y_qp):
        self._check(self.lib.nncase_hip_qglobal_avgpool(self.handle, x.ptr, out.ptr, batch, h, w, channels, x_qp, y_qp),
                    "qglobal_avgpool")

    def lut_u8(self, src: DeviceBuffer, dst: DeviceBuffer, count: int, lut: np.ndarray):
        t = np.ascontiguousarray(lut, np.uint8)
        assert t.size == 256
        self._check(self.lib.nncase_hip_lut_u8(self.handle, src.ptr, dst.ptr, count, t.ctypes.data), "lut_u8")

    def qconcat_channels(self, inputs: Sequence[DeviceBuffer], channels: Sequence[int], in_qps, out: DeviceBuffer, out_qp,
                         pixels: int):
        n, ptrs, ch, qps = _concat_args(inputs, channels, in_qps)
        self._check(self.lib.nncase_hip_qconcat_channels(self.handle, n, ptrs, ch, qps, out.ptr, out_qp, pixels),
                    "qconcat_channels")

    def qmaxpool2d(self, x: DeviceBuffer, out: DeviceBuffer, batch, h, w, channels, kernel, stride, padding, x_qp, y_qp):
        (ph0, ph1), (pw0, pw1) = padding
        self._check(self.lib.nncase_hip_qmaxpool2d(self.handle, x.ptr, out.ptr, batch, h, w, channels, kernel[0], kernel[1],
                                                   stride[0], stride[1], ph0, ph1, pw0, pw1, x_qp, y_qp), "qmaxpool2d")

    def resize_nearest(self, src: DeviceBuffer, dst: DeviceBuffer, elem_size, batch, in_h, in_w, channels, out_h, out_w,
                       transformation_mode=0, nearest_mode=0):
        self._check(self.lib.nncase_hip_resize_nearest(self.handle, src.ptr, dst.ptr, elem_size, batch, in_h, in_w, channels,
                                                       out_h, out_w, transformation_mode, nearest_mode), "resize_nearest")

    def pack(self, src: DeviceBuffer, dst: DeviceBuffer, elem_size: int, shape: Sequence[int], axes: Sequence[int],
             lanes: Sequence[int]):
        sh, ax, ln = (C.c_int32 * len(shape))(*shape), (C.c_int32 * max(1, len(axes)))(*axes), (C.c_int32 * max(1, len(lanes)))(*lanes)
        self._check(self.lib.nncase_hip_pack(self.handle, src.ptr, dst.ptr, elem_size, len(shape), sh, len(axes), ax, ln), "pack")

    def quantize_pack(self, src: DeviceBuffer, dst: DeviceBuffer, shape: Sequence[int], axes: Sequence[int], lanes: Sequence[int],
                      q: QuantParam):
        """float32 -> u8 quantize and pack in one pass (the layouts in front of a stem convolution)."""
        sh, ax, ln = (C.c_int32 * len(shape))(*shape), (C.c_int32 * max(1, len(axes)))(*axes), (C.c_int32 * max(1, len(lanes)))(*lanes)
        self._check(self.lib.nncase_hip_quantize_pack(self.handle, src.ptr, dst.ptr, len(shape), sh, len(axes), ax, ln, q), "quantize_pack")

    def unpack(self, src: DeviceBuffer, dst: DeviceBuffer, elem_size: int, unpacked_shape: Sequence[int],
               axes: Sequence[int], lanes: Sequence[int]):
        sh = (C.c_int32 * len(unpacked_shape))(*unpacked_shape)
        ax, ln = (C.c_int32 * max(1, len(axes)))(*axes), (C.c_int32 * max(1, len(lanes)))(*lanes)
        self._check(self.lib.nncase_hip_unpack(self.handle, src.ptr, dst.ptr, elem_size, len(unpacked_shape), sh, len(axes),
                                               ax, ln), "unpack")

    def nchw_to_nhwc(self, src: DeviceBuffer, dst: DeviceBuffer, elem_size, n, c, h, w):
        self._check(self.lib.nncase_hip_nchw_to_nhwc(self.handle, src.ptr, dst.ptr, elem_size, n, c, h, w), "nchw_to_nhwc")

    def nhwc_to_nchw(self, src: DeviceBuffer, dst: DeviceBuffer, elem_size, n, c, h, w):
        self._check(self.lib.nncase_hip_nhwc_to_nchw(self.handle, src.ptr, dst.ptr, elem_size, n, c, h, w), "nhwc_to_nchw")

    # -- decode-step operators ---------------------------------------------------------------
    def prepack_w8a16(self, w_nk: np.ndarray, scale: np.ndarray, bias: Optional[np.ndarray] = None) -> "W8A16":
        return W8A16(self, w_nk, scale, bias)

    def w8a16_gemm(self, a: DeviceBuffer, w: "W8A16", out: DeviceBuffer, m: int, mode: int = GEMM_PLAIN,
                   residual: Optional[DeviceBuffer] = None, out_dtype: int = DT_F16):
        self._check(self.lib.nncase_hip_w8a16_gemm(self.handle, a.ptr, w.handle, out.ptr, m, mode,
                                                   residual.ptr if residual is not None else None, out_dtype), "w8a16_gemm")

    def rmsnorm_w8a16_gemm(self, x: DeviceBuffer, ln_weight: DeviceBuffer, eps: float, w: "W8A16", out: DeviceBuffer, m: int,
                           mode: int = GEMM_PLAIN, residual: Optional[DeviceBuffer] = None, out_dtype: int = DT_F16):
        """w8a16_gemm(rmsnorm_f16(x)) in one launch, bit for bit the two operators' result."""
        self._check(self.lib.nncase_hip_rmsnorm_w8a16_gemm(self.handle, x.ptr, ln_weight.ptr, eps, w.handle, out.ptr, m, mode,
                                                           residual.ptr if residual is not None else None, out_dtype),
                    "rmsnorm_w8a16_gemm")

    def rmsnorm_f16(self, x: DeviceBuffer, weight: DeviceBuffer, out: DeviceBuffer, rows: int, hidden: int, eps: float):
        self._check(self.lib.nncase_hip_rmsnorm_f16(self.handle, x.ptr, weight.ptr, out.ptr, rows, hidden, eps), "rmsnorm_f16")

    def w8a16_gemm_rope_kv_append(self, x, ln_weight, eps, w, qkv, q_out, k_cache, v_cache, block_table, ctx_lens, geometry, theta):
        self._check(self.lib.nncase_hip_w8a16_gemm_rope_kv_append(
            self.handle, x.ptr, ln_weight.ptr if ln_weight is not None else None, eps, w.handle, qkv.ptr, q_out.ptr, k_cache.ptr,
            v_cache.ptr, block_table.ptr, ctx_lens.ptr, C.byref(geometry), theta), "w8a16_gemm_rope_kv_append")

    def rope_kv_append(self, qkv, q_out, k_cache, v_cache, block_table, ctx_lens, geometry: PagedAttnArgs, theta: float):
        self._check(self.lib.nncase_hip_rope_kv_append(self.handle, qkv.ptr, q_out.ptr, k_cache.ptr, v_cache.ptr, block_table.ptr,
                                                       ctx_lens.ptr, C.byref(geometry), theta), "rope_kv_append")

    def argmax_f32(self, x: DeviceBuffer, out: DeviceBuffer, rows: int, cols: int):
        self._check(self.lib.nncase_hip_argmax_f32(self.handle, x.ptr, out.ptr, rows, cols), "argmax_f32")

    def embedding_f16(self, table: DeviceBuffer, ids: DeviceBuffer, out: DeviceBuffer, rows: int, hidden: int, vocab: int):
        self._check(self.lib.nncase_hip_embedding_f16(self.handle, table.ptr, ids.ptr, out.ptr, rows, hidden, vocab), "embedding_f16")

    def add_i32(self, x: DeviceBuffer, count: int, delta: int):
        self._check(self.lib.nncase_hip_add_i32(self.handle, x.ptr, count, delta), "add_i32")

    def paged_attention_decode(self, q: DeviceBuffer, k_cache: DeviceBuffer, v_cache: DeviceBuffer,
                               block_table: DeviceBuffer, ctx_lens: DeviceBuffer, out: DeviceBuffer, args: PagedAttnArgs):
        self._check(self.lib.nncase_hip_paged_attention_decode(self.handle, q.ptr, k_cache.ptr, v_cache.ptr, block_table.ptr,
                                                               ctx_lens.ptr, out.ptr, C.byref(args)), "paged_attention_decode")

    def paged_attention_decode_noalloc(self, q: DeviceBuffer, k_cache: DeviceBuffer, v_cache: DeviceBuffer,
                                       block_table: DeviceBuffer, ctx_lens: DeviceBuffer, out: DeviceBuffer, args: PagedAttnArgs):
        """The same operator on the library's static device scratch: allocates nothing (-ENOSPC beyond its size)."""
        self._check(self.lib.nncase_hip_paged_attention_decode_noalloc(self.handle, q.ptr, k_cache.ptr, v_cache.ptr,
                                                                       block_table.ptr, ctx_lens.ptr, out.ptr, C.byref(args)),
                    "paged_attention_decode_noalloc")


class Function:
    """Resident operator list (nncase_hip_function_t): the `hip` module's runtime_function."""

    def __init__(self, ctx: Context):
        self.ctx = ctx
        h = C.c_void_p()
        ctx._check(ctx.lib.nncase_hip_function_create(ctx.handle, C.byref(h)), "function_create")
        self.handle = h.value
        self._keep = []  # operands must outlive the function
        ctx._adopt(self)

    def _ck(self, rc, where):
        self.ctx._check(rc, where)

    def add_quantize(self, src, in_dtype, dst, out_dtype, count, q):
        self._keep += [src, dst]
        self._ck(self.ctx.lib.nncase_hip_function_add_quantize(self.handle, src.ptr, in_dtype, dst.ptr, out_dtype, count, q),
                 "function_add_quantize")

    def add_dequantize(self, src, in_dtype, dst, out_dtype, count, q):
        self._keep += [src, dst]
        self._ck(self.ctx.lib.nncase_hip_function_add_dequantize(self.handle, src.ptr, in_dtype, dst.ptr, out_dtype, count, q),
                 "function_add_dequantize")

    def add_qconv2d(self, x, w: Weights, y, args: Conv2dArgs):
        self._keep += [x, w, y]
        self._ck(self.ctx.lib.nncase_hip_function_add_qconv2d(self.handle, x.ptr, w.handle, y.ptr, C.byref(args)),
                 "function_add_qconv2d")

    def add_qblock(self, x, blk: QBlock, y, args: QBlockArgs):
        self._keep += [x, blk, y]
        self._ck(self.ctx.lib.nncase_hip_function_add_qblock(self.handle, x.ptr, blk.handle, y.ptr, C.byref(args)),
                 "function_add_qblock")

    def add_qpointwise_pair(self, x, pair: QPair, y1, y2, first_args: Conv2dArgs, second_args: Conv2dArgs):
        self._keep += [x, pair, y1, y2]
        self._ck(self.ctx.lib.nncase_hip_function_add_qpointwise_pair(self.handle, x.ptr, pair.handle, y1.ptr, y2.ptr, C.byref(first_args),
                                                                      C.byref(second_args)), "function_add_qpointwise_pair")

    def add_qglobal_avgpool_qconv2d(self, x, h: int, w_: int, x_qp: QuantParam, w: Weights, y, args: Conv2dArgs):
        self._keep += [x, w, y]
        self._ck(self.ctx.lib.nncase_hip_function_add_qglobal_avgpool_qconv2d(self.handle, x.ptr, h, w_, x_qp, w.handle, y.ptr, C.byref(args)),
                 "function_add_qglobal_avgpool_qconv2d")

    def add_qdepthwise_pointwise_pair(self, x, dw: Weights, dw_args: Conv2dArgs, pair: QPair, y1, y2, first_args: Conv2dArgs,
                                      second_args: Conv2dArgs):
        self._keep += [x, dw, pair, y1, y2]
        self._ck(self.ctx.lib.nncase_hip_function_add_qdepthwise_pointwise_pair(self.handle, x.ptr, dw.handle, C.byref(dw_args), pair.handle,
                                                                                y1.ptr, y2.ptr, C.byref(first_args), C.byref(second_args)),
                 "function_add_qdepthwise_pointwise_pair")

    def add_qadd(self, a, a_qp, b, b_qp, out, y_qp, count, clamp=(-FLT_MAX, FLT_MAX)):
        self._keep += [a, b, out]
        self._ck(self.ctx.lib.nncase_hip_function_add_qadd(self.handle, a.ptr, a_qp, b.ptr, b_qp, out.ptr, y_qp, clamp[0],
                                                          clamp[1], count), "function_add_qadd")

    def add_qglobal_avgpool(self, x, out, batch, h, w, channels, x_qp, y_qp):
        self._keep += [x, out]
        self._ck(self.ctx.lib.nncase_hip_function_add_qglobal_avgpool(self.handle, x.ptr, out.ptr, batch, h, w, channels,
                                                                     x_qp, y_qp), "function_add_qglobal_avgpool")

    def add_lut_u8(self, src, dst, count, lut):
        self._keep += [src, dst]
        t = np.ascontiguousarray(lut, np.uint8)
        assert t.size == 256
        self._ck(self.ctx.lib.nncase_hip_function_add_lut_u8(self.handle, src.ptr, dst.ptr, count, t.ctypes.data),
                 "function_add_lut_u8")

    def add_qconcat_channels(self, inputs, channels, in_qps, out, out_qp, pixels):
        self._keep += [b for b in inputs if b is not None] + [out]
        n, ptrs, ch, qps = _concat_args(inputs, channels, in_qps)
        self._ck(self.ctx.lib.nncase_hip_function_add_qconcat_channels(self.handle, n, ptrs, ch, qps, out.ptr, out_qp, pixels),
                 "function_add_qconcat_channels")

    def add_qmaxpool2d(self, x, out, batch, h, w, channels, kernel, stride, padding, x_qp, y_qp):
        self._keep += [x, out]
        (ph0, ph1), (pw0, pw1) = padding
        self._ck(self.ctx.lib.nncase_hip_function_add_qmaxpool2d(self.handle, x.ptr, out.ptr, batch, h, w, channels, kernel[0],
                                                                 kernel[1], stride[0], stride[1], ph0, ph1, pw0, pw1, x_qp, y_qp),
                 "function_add_qmaxpool2d")

    def add_pack(self, src, dst, elem_size, shape, axes, lanes):
        self._keep += [src, dst]
        sh, ax, ln = (C.c_int32 * len(shape))(*shape), (C.c_int32 * max(1, len(axes)))(*axes), (C.c_int32 * max(1, len(lanes)))(*lanes)
        self._ck(self.ctx.lib.nncase_hip_function_add_pack(self.handle, src.ptr, dst.ptr, elem_size, len(shape), sh, len(axes), ax, ln),
                 "function_add_pack")

    def add_quantize_pack(self, src, dst, shape, axes, lanes, q: QuantParam):
        self._keep += [src, dst]
        sh, ax, ln = (C.c_int32 * len(shape))(*shape), (C.c_int32 * max(1, len(axes)))(*axes), (C.c_int32 * max(1, len(lanes)))(*lanes)
        self._ck(self.ctx.lib.nncase_hip_function_add_quantize_pack(self.handle, src.ptr, dst.ptr, len(shape), sh, len(axes), ax, ln, q),
                 "function_add_quantize_pack")

    def add_w8a16_gemm(self, a, w, out, m, mode=GEMM_PLAIN, residual=None, out_dtype=DT_F16):
        self._keep += [a, w, out] + ([residual] if residual is not None else [])
        self._ck(self.ctx.lib.nncase_hip_function_add_w8a16_gemm(self.handle, a.ptr, w.handle, out.ptr, m, mode,
                                                                 residual.ptr if residual is not None else None, out_dtype),
                 "function_add_w8a16_gemm")

    def add_rmsnorm_w8a16_gemm(self, x, ln_weight, eps, w, out, m, mode=GEMM_PLAIN, residual=None, out_dtype=DT_F16):
        self._keep += [x, ln_weight, w, out] + ([residual] if residual is not None else [])
        self._ck(self.ctx.lib.nncase_hip_function_add_rmsnorm_w8a16_gemm(self.handle, x.ptr, ln_weight.ptr, eps, w.handle, out.ptr, m,
                                                                         mode, residual.ptr if residual is not None else None,
                                                                         out_dtype), "function_add_rmsnorm_w8a16_gemm")

    def add_rmsnorm_f16(self, x, weight, out, rows, hidden, eps):
        self._keep += [x, weight, out]
        self._ck(self.ctx.lib.nncase_hip_function_add_rmsnorm_f16(self.handle, x.ptr, weight.ptr, out.ptr, rows, hidden, eps),
                 "function_add_rmsnorm_f16")

    def add_rope_kv_append(self, qkv, q_out, k_cache, v_cache, block_table, ctx_lens, geometry, theta):
        self._keep += [qkv, q_out, k_cache, v_cache, block_table, ctx_lens]
        self._ck(self.ctx.lib.nncase_hip_function_add_rope_kv_append(self.handle, qkv.ptr, q_out.ptr, k_cache.ptr, v_cache.ptr,
                                                                     block_table.ptr, ctx_lens.ptr, C.byref(geometry), theta),
                 "function_add_rope_kv_append")

    def add_w8a16_gemm_rope_kv_append(self, x, ln_weight, eps, w, qkv, q_out, k_cache, v_cache, block_table, ctx_lens, geometry, theta):
        """The q / k / v projection (of rmsnorm(x) when ln_weight is given), rotary embedding and cache append as one operator."""
        self._keep += [x, ln_weight, w, qkv, q_out, k_cache, v_cache, block_table, ctx_lens]
        self._ck(self.ctx.lib.nncase_hip_function_add_w8a16_gemm_rope_kv_append(
            self.handle, x.ptr, ln_weight.ptr if ln_weight is not None else None, eps, w.handle, qkv.ptr, q_out.ptr, k_cache.ptr,
            v_cache.ptr, block_table.ptr, ctx_lens.ptr, C.byref(geometry), theta), "function_add_w8a16_gemm_rope_kv_append")

    def add_paged_attention_decode(self, q, k_cache, v_cache, block_table, ctx_lens, out, args):
        self._keep += [q, k_cache, v_cache, block_table, ctx_lens, out]
        self._ck(self.ctx.lib.nncase_hip_function_add_paged_attention_decode(self.handle, q.ptr, k_cache.ptr, v_cache.ptr,
                                                                             block_table.ptr, ctx_lens.ptr, out.ptr, C.byref(args)),
                 "function_add_paged_attention_decode")

    def add_argmax_f32(self, x, out, rows, cols):
        self._keep += [x, out]
        self._ck(self.ctx.lib.nncase_hip_function_add_argmax_f32(self.handle, x.ptr, out.ptr, rows, cols), "function_add_argmax_f32")

    def add_embedding_f16(self, table, ids, out, rows, hidden, vocab):
        self._keep += [table, ids, out]
        self._ck(self.ctx.lib.nncase_hip_function_add_embedding_f16(self.handle, table.ptr, ids.ptr, out.ptr, rows, hidden, vocab),
                 "function_add_embedding_f16")

    def add_add_i32(self, x, count, delta):
        self._keep += [x]
        self._ck(self.ctx.lib.nncase_hip_function_add_add_i32(self.handle, x.ptr, count, delta), "function_add_add_i32")

    def add_resize_nearest(self, src, dst, elem_size, batch, in_h, in_w, channels, out_h, out_w, transformation_mode=0,
                           nearest_mode=0):
        self._keep += [src, dst]
        self._ck(self.ctx.lib.nncase_hip_function_add_resize_nearest(self.handle, src.ptr, dst.ptr, elem_size, batch, in_h,
                                                                     in_w, channels, out_h, out_w, transformation_mode,
                                                                     nearest_mode), "function_add_resize_nearest")

    def add_layout(self, src, dst, elem_size, n, c, h, w, to_nchw: bool):
        """NCHW -> NHWC (to_nchw False) or back, as a step of the function."""
        self._keep += [src, dst]
        self._ck(self.ctx.lib.nncase_hip_function_add_layout(self.handle, src.ptr, dst.ptr, elem_size, n, c, h, w, int(to_nchw)),
                 "function_add_layout")

    LANE_JOINED = -1   # set_lane(LANE_JOINED): what follows waits for every lane (recorded last)

    def set_lane(self, lane: int):
        """Operators added from now on form independent chain `lane`; a captured function overlaps its lanes."""
        self._ck(self.ctx.lib.nncase_hip_function_set_lane(self.handle, lane), "function_set_lane")

    def __len__(self):
        n = C.c_int32()
        self._ck(self.ctx.lib.nncase_hip_function_size(self.handle, C.byref(n)), "function_size")
        return n.value

    def invoke(self):
        self._ck(self.ctx.lib.nncase_hip_function_invoke(self.handle), "function_invoke")

    def invoke_one(self, index: int):
        self._ck(self.ctx.lib.nncase_hip_function_invoke_one(self.handle, index), "function_invoke_one")

    def capture(self):
        self._ck(self.ctx.lib.nncase_hip_function_capture(self.handle), "function_capture")

    def profile(self, iterations: int = 10):
        """Mean device milliseconds per operator (HIP events on the context's stream)."""
        n = len(self)
        out = (C.c_float * n)()
        self._ck(self.ctx.lib.nncase_hip_function_profile(self.handle, iterations, out), "function_profile")
        return [float(v) for v in out]

    def op_kernel(self, index: int) -> str:
        buf = C.create_string_buffer(96)
        self._ck(self.ctx.lib.nncase_hip_function_op_kernel(self.handle, index, buf, 96), "function_op_kernel")
        return buf.value.decode()

    def destroy(self):
        if self.handle:
            if self.ctx.handle:  # a function of a closed context went with it
                self.ctx.lib.nncase_hip_function_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class W8A16:
    """Pre-packed int8 weight matrix [n, k] with per-output-channel fp32 scales (nncase_hip_w8a16_t)."""

    def __init__(self, ctx: Context, w_nk: np.ndarray, scale: np.ndarray, bias: Optional[np.ndarray] = None):
        w = np.ascontiguousarray(w_nk, np.int8)
        sc = np.ascontiguousarray(scale, np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        self.ctx, self.n, self.k = ctx, w.shape[0], w.shape[1]
        assert sc.shape == (self.n,) and (b is None or b.shape == (self.n,))
        h = C.c_void_p()
        ctx._check(ctx.lib.nncase_hip_w8a16_prepack(ctx.handle, w.ctypes.data, sc.ctypes.data, None if b is None else b.ctypes.data,
                                                    self.k, self.n, C.byref(h)), "w8a16_prepack")
        self.handle = h.value

    def destroy(self):
        if self.handle:
            if self.ctx.handle:
                self.ctx.lib.nncase_hip_w8a16_destroy(self.ctx.handle, self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class _Borrowed:
    """A device address owned by someone else (a loaded kmodel's tensor)."""

    def __init__(self, ctx, ptr, nbytes):
        self.ctx, self.ptr, self.nbytes = ctx, ptr, nbytes

    upload = DeviceBuffer.upload
    download = DeviceBuffer.download


class _BorrowedFunction(Function):
    def __init__(self, ctx, handle):  # no create: the kmodel owns the handle
        self.ctx, self.handle, self._keep = ctx, handle, []

    def destroy(self):
        self.handle = None


class LoadedKModel:
    """A kmodel with a `hip` entry module, loaded by the native loader: the counterpart of
    Interpreter.load_model / set_input_tensor / run / get_output_tensor
    (src/Nncase.Simulator/Runtime/Interop/RTInterpreter.cs) for this target."""
    INPUT, OUTPUT = -1, -2
    _NP = {DT_F32: np.float32, DT_U8: np.uint8, DT_F16: np.float16, DT_I32: np.int32, DT_I8: np.int8, DT_I16: np.int16}

    def __init__(self, ctx: Context, data: bytes = None, *, text: bytes = None, rdata: bytes = b""):
        """`data`: a whole kmodel file.  `text` / `rdata`: one function's slice of a hip module's .text
        section and the module's .rdata section, the pair a runtime_function's initialize_core receives."""
        self.ctx = ctx
        h = C.c_void_p()
        if (data is None) == (text is None):
            raise ValueError("LoadedKModel takes either a kmodel file or a function's text (+ rdata)")
        if data is not None:
            buf = (C.c_char * len(data)).from_buffer_copy(data)
            ctx._check(ctx.lib.nncase_hip_kmodel_load(ctx.handle, C.cast(buf, C.c_void_p), len(data), C.byref(h)), "kmodel_load")
        else:
            tbuf = (C.c_char * max(len(text), 1)).from_buffer_copy(text or b"\0")
            rbuf = (C.c_char * max(len(rdata), 1)).from_buffer_copy(rdata or b"\0")
            ctx._check(ctx.lib.nncase_hip_kmodel_load_function(ctx.handle, C.cast(tbuf, C.c_void_p), len(text),
                                                               C.cast(rbuf, C.c_void_p), len(rdata), C.byref(h)),
                       "kmodel_load_function")
        self.handle = h.value
        ctx._adopt(self)
        f = C.c_void_p()
        ctx._check(ctx.lib.nncase_hip_kmodel_function(self.handle, C.byref(f)), "kmodel_function")
        self.fn = _BorrowedFunction(ctx, f.value)
        self.input, self.input_shape, self.input_dtype = self.tensor(self.INPUT)
        self.output, self.output_shape, self.output_dtype = self.tensor(self.OUTPUT)
        self.outputs = [(self.output, self.output_shape, self.output_dtype)]
        while True:  # further outputs of a function that returns a tuple
            try:
                self.outputs.append(self.tensor(self.OUTPUT - len(self.outputs)))
            except HipError:
                break

    def tensor(self, which: int):
        p, dt, dims = C.c_void_p(), C.c_int32(), (C.c_int32 * 4)()
        self.ctx._check(self.ctx.lib.nncase_hip_kmodel_tensor(self.handle, which, C.byref(p), C.byref(dt), dims), "kmodel_tensor")
        shape, dtype = tuple(dims), np.dtype(self._NP[dt.value])
        buf = None if not p.value else _Borrowed(self.ctx, p.value, int(np.prod(shape)) * dtype.itemsize)
        return buf, shape, dtype

    def run(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, self.input_dtype)
        if x.shape != self.input_shape:
            raise HipError(-ERR_SHAPE_MISMATCH, "kmodel run", f"input {x.shape}, model expects {self.input_shape}")
        self.input.upload(x)
        self.fn.invoke()
        self.ctx.sync()
        ys = [b.download(shape, dt) for b, shape, dt in self.outputs]
        return ys[0] if len(ys) == 1 else ys

    def destroy(self):
        if self.handle:
            if self.ctx.handle:
                self.ctx.lib.nncase_hip_kmodel_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
