"""ctypes/numpy front end of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the product package never does.  Every function forwards to the C
restatement in nncase_oracle.c (which cites the reference file:line it follows)
or, for pack/unpack, states the definition in numpy.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnncase_oracle.so")

U8, I8, I16 = 0, 1, 2
OUT_U8, OUT_I32, OUT_F32 = 0, 1, 2
_NP_Q = {U8: np.uint8, I8: np.int8, I16: np.int16}
_NP_OUT = {OUT_U8: np.uint8, OUT_I32: np.int32, OUT_F32: np.float32}
FLT_MAX = float(np.finfo(np.float32).max)


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "nncase_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libnncase_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.ref_f16_to_f32.restype = C.c_float
        _lib.ref_f16_to_f32.argtypes = [C.c_uint16]
        _lib.ref_f32_to_f16.restype = C.c_uint16
        _lib.ref_f32_to_f16.argtypes = [C.c_float]
        _lib.oracle_windowed_output_size.restype = C.c_int32
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.asarray(a, dtype=dtype, order="C")  # keeps 0-d shapes, unlike ascontiguousarray


def _f(x):
    return C.c_float(float(x))


def _i(x):
    return C.c_int32(int(x))


def windowed_output_size(size, filt, stride, dilation, pad_before, pad_after) -> int:
    return int(lib().oracle_windowed_output_size(_i(size), _i(filt), _i(stride), _i(dilation), _i(pad_before), _i(pad_after)))


# ---------------------------------------------------------------- reference float kernels
def quantize(x, scale, zero_point, dtype=U8, ort_order=False):
    x = _c(x, np.float32)
    out = np.empty(x.shape, _NP_Q[dtype])
    if ort_order:
        rc = lib().ref_quantize_f32_ort_order(_p(x), _p(out), C.c_size_t(x.size), _f(scale), _i(zero_point), C.c_int(dtype))
    else:
        rc = lib().ref_quantize_f32(_p(x), _p(out), C.c_size_t(x.size), _f(scale), _f(np.float32(zero_point)), C.c_int(dtype))
    assert rc == 0
    return out


def dequantize(q, scale, zero_point):
    q = np.asarray(q, order="C")
    dtype = {np.dtype(np.uint8): U8, np.dtype(np.int8): I8, np.dtype(np.int16): I16}[q.dtype]
    out = np.empty(q.shape, np.float32)
    rc = lib().ref_dequantize_f32(_p(q), _p(out), C.c_size_t(q.size), _f(scale), _f(np.float32(zero_point)), C.c_int(dtype))
    assert rc == 0
    return out


def _conv_geom(xshape, wshape, stride, padding, dilation):
    n, c, h, w = xshape
    oc, _, kh, kw = wshape
    (ph0, ph1), (pw0, pw1) = padding
    oh = windowed_output_size(h, kh, stride[0], dilation[0], ph0, ph1)
    ow = windowed_output_size(w, kw, stride[1], dilation[1], pw0, pw1)
    return n, c, h, w, oc, kh, kw, ph0, ph1, pw0, pw1, oh, ow


def conv2d_f32(x, w, bias, stride=(1, 1), padding=((0, 0), (0, 0)), dilation=(1, 1), groups=1,
               fused_clamp=(-FLT_MAX, FLT_MAX)):
    """reference::conv2d_impl<float>, NCHW / OIHW."""
    x, w, bias = _c(x, np.float32), _c(w, np.float32), _c(bias, np.float32)
    n, c, h, ww, oc, kh, kw, ph0, ph1, pw0, pw1, oh, ow = _conv_geom(x.shape, w.shape, stride, padding, dilation)
    assert w.shape[1] == c // groups
    out = np.empty((n, oc, oh, ow), np.float32)
    rc = lib().ref_conv2d_f32(_p(x), _p(w), _p(bias), _p(out), _i(n), _i(c), _i(h), _i(ww), _i(oc), _i(kh), _i(kw),
                              _i(stride[0]), _i(stride[1]), _i(ph0), _i(ph1), _i(pw0), _i(pw1),
                              _i(dilation[0]), _i(dilation[1]), _i(groups), _f(fused_clamp[0]), _f(fused_clamp[1]))
    assert rc == 0
    return out


def _to4d(shape):
    return [1] * (4 - len(shape)) + list(shape)


def matmul_f32(a, b):
    """reference::matmul_impl<float> including its rank<=4 broadcast batching."""
    a, b = _c(a, np.float32), _c(b, np.float32)
    ash, bsh = list(a.shape), list(b.shape)
    a1, b1 = len(ash) == 1, len(bsh) == 1
    if a1:
        ash = [1] + ash
    if b1:
        bsh = bsh + [1]
    a4, b4 = _to4d(ash), _to4d(bsh)
    out4 = [max(a4[0], b4[0]), max(a4[1], b4[1]), a4[2], b4[3]]
    out = np.empty(out4, np.float32)
    rc = lib().ref_matmul_f32(_p(a), _p(b), _p(out), (C.c_int32 * 4)(*a4), (C.c_int32 * 4)(*b4))
    assert rc == 0
    lead = np.broadcast_shapes(tuple(ash[:-2]), tuple(bsh[:-2]))
    shape = list(lead) + [ash[-2], bsh[-1]]
    out = out.reshape(shape)
    if a1:
        out = out.reshape(shape[:-2] + [shape[-1]])
        shape = list(out.shape)
    if b1:
        out = out.reshape(shape[:-1])
    return out


def reduce_window2d_mean_f32(x, filt, stride, padding=((0, 0), (0, 0)), count_include_pad=False,
                             fused_clamp=(-FLT_MAX, FLT_MAX)):
    x = _c(x, np.float32)
    n, c, h, w = x.shape
    (ph0, ph1), (pw0, pw1) = padding
    oh = windowed_output_size(h, filt[0], stride[0], 1, ph0, ph1)
    ow = windowed_output_size(w, filt[1], stride[1], 1, pw0, pw1)
    out = np.empty((n, c, oh, ow), np.float32)
    rc = lib().ref_reduce_window2d_mean_f32(_p(x), _p(out), _i(n), _i(c), _i(h), _i(w), _i(filt[0]), _i(filt[1]),
                                            _i(stride[0]), _i(stride[1]), _i(ph0), _i(ph1), _i(pw0), _i(pw1),
                                            _i(int(count_include_pad)), _f(fused_clamp[0]), _f(fused_clamp[1]))
    assert rc == 0
    return out


def fixup_range(lo, hi, symmetric=False):
    out = (C.c_float * 2)()
    lib().ref_fixup_range(_f(lo), _f(hi), C.c_int(int(symmetric)), out)
    return np.float32(out[0]), np.float32(out[1])


def calib_fixup_range(lo, hi, symmetric=False):
    out = (C.c_float * 2)()
    lib().ref_calib_fixup_range(_f(lo), _f(hi), C.c_int(int(symmetric)), out)
    return np.float32(out[0]), np.float32(out[1])


UNSIGNED, SIGNED_SYMMETRIC, SIGNED_ASYMMETRIC = 0, 1, 2


def get_quant_param(lo, hi, bits=8, mode=UNSIGNED):
    zp, sc = C.c_int32(), C.c_float()
    rc = lib().ref_get_quant_param(_f(lo), _f(hi), C.c_int(bits), C.c_int(mode), C.byref(zp), C.byref(sc))
    assert rc == 0
    return int(zp.value), np.float32(sc.value)


def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().ref_f32_to_f16_array(_p(x), _p(out), C.c_size_t(x.size))
    return out


def f16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().ref_f16_to_f32_array(_p(h), _p(out), C.c_size_t(h.size))
    return out


# ---------------------------------------------------------------- integer-exact u8/u8 operators
def requant_u8(acc, sx, sw, sy, zy, fused_clamp=(-FLT_MAX, FLT_MAX)):
    acc = _c(acc, np.int32)
    out = np.empty(acc.shape, np.uint8)
    lib().q_requant_u8(_p(acc), _p(out), C.c_size_t(acc.size), _f(sx), _f(sw), _f(fused_clamp[0]), _f(fused_clamp[1]),
                       _f(sy), _i(zy))
    return out


def qconv2d(x, w, bias, zx, sx, zw, sw, zy=0, sy=1.0, stride=(1, 1), padding=((0, 0), (0, 0)), dilation=(1, 1),
            groups=1, fused_clamp=(-FLT_MAX, FLT_MAX), out_mode=OUT_U8):
    """Integer-exact u8/u8 conv, NCHW u8 input, OIHW u8 weights, int32 bias (or None)."""
    x, w = _c(x, np.uint8), _c(w, np.uint8)
    b = None if bias is None else _c(bias, np.int32)
    n, c, h, ww, oc, kh, kw, ph0, ph1, pw0, pw1, oh, ow = _conv_geom(x.shape, w.shape, stride, padding, dilation)
    assert w.shape[1] == c // groups
    out = np.empty((n, oc, oh, ow), _NP_OUT[out_mode])
    rc = lib().q_conv2d_u8(_p(x), _p(w), None if b is None else _p(b), _p(out), _i(n), _i(c), _i(h), _i(ww), _i(oc),
                           _i(kh), _i(kw), _i(stride[0]), _i(stride[1]), _i(ph0), _i(ph1), _i(pw0), _i(pw1),
                           _i(dilation[0]), _i(dilation[1]), _i(groups), _i(zx), _f(sx), _i(zw), _f(sw), _i(zy), _f(sy),
                           _f(fused_clamp[0]), _f(fused_clamp[1]), C.c_int(out_mode))
    assert rc == 0, f"q_conv2d_u8 rc={rc}"
    return out


def qmatmul(a, b, bias, za, sa, zb, sb, zy=0, sy=1.0, fused_clamp=(-FLT_MAX, FLT_MAX), out_mode=OUT_I32):
    a, b = _c(a, np.uint8), _c(b, np.uint8)
    bi = None if bias is None else _c(bias, np.int32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    out = np.empty((m, n), _NP_OUT[out_mode])
    rc = lib().q_matmul_u8(_p(a), _p(b), None if bi is None else _p(bi), _p(out), _i(m), _i(k), _i(n), _i(za), _f(sa),
                           _i(zb), _f(sb), _i(zy), _f(sy), _f(fused_clamp[0]), _f(fused_clamp[1]), C.c_int(out_mode))
    assert rc == 0, f"q_matmul_u8 rc={rc}"
    return out


def qadd(a, b, za, sa, zb, sb, zy, sy, fused_clamp=(-FLT_MAX, FLT_MAX)):
    a, b = _c(a, np.uint8), _c(b, np.uint8)
    assert a.shape == b.shape
    out = np.empty(a.shape, np.uint8)
    lib().q_add_u8(_p(a), _p(b), _p(out), C.c_size_t(a.size), _i(za), _f(sa), _i(zb), _f(sb), _i(zy), _f(sy),
                   _f(fused_clamp[0]), _f(fused_clamp[1]))
    return out


def qglobal_avgpool(x, zx, sx, zy, sy):
    """u8 NCHW -> u8 [N, C]."""
    x = _c(x, np.uint8)
    n, c, h, w = x.shape
    out = np.empty((n, c), np.uint8)
    lib().q_global_avgpool_u8(_p(x), _p(out), _i(n), _i(c), _i(h), _i(w), _i(zx), _f(sx), _i(zy), _f(sy))
    return out


def qconv2d_float_chain(x, w, bias, zx, sx, zw, sw, zy, sy, stride=(1, 1), padding=((0, 0), (0, 0)), dilation=(1, 1),
                        groups=1, fused_clamp=(-FLT_MAX, FLT_MAX)):
    """What the CPU target really runs for a u8/u8 conv: DQ -> float conv (+clamp) -> Q
    (QLinearConv.cs:61-75; bias quant param (0, sx*sw))."""
    xf = dequantize(x, sx, zx)
    wf = dequantize(w, sw, zw)
    oc = w.shape[0]
    bq = np.zeros(oc, np.int32) if bias is None else np.asarray(bias, np.int32)
    bf = (bq.astype(np.float32) - np.float32(0)) * (np.float32(sx) * np.float32(sw))
    y = conv2d_f32(xf, wf, bf, stride, padding, dilation, groups, fused_clamp)
    return quantize(y, sy, zy, U8)


# ---------------------------------------------------------------- no reference counterpart
LUT_REQUANT, LUT_SWISH = 0, 1


def unary_lut(kind, zx, sx, zy, sy) -> np.ndarray:
    """256-entry table lut[v] = Q(f(DQ(v))); kind LUT_REQUANT (identity) or LUT_SWISH."""
    lut = np.empty(256, np.uint8)
    lib().q_unary_lut_u8(_i(kind), _i(zx), _f(sx), _i(zy), _f(sy), _p(lut))
    return lut


def qconcat(xs, qps, out_qp, axis=1) -> np.ndarray:
    """Concat of u8 tensors carrying different quant params: every input is requantised to
    out_qp (Q(DQ(x)), the Quantize/Dequantize pair the graph holds around Concat), then joined."""
    parts = [unary_lut(LUT_REQUANT, z, s, out_qp[0], out_qp[1])[np.asarray(x, np.uint8)] for x, (z, s) in zip(xs, qps)]
    return np.concatenate(parts, axis=axis)


HALF_PIXEL, PYTORCH_HALF_PIXEL, ALIGN_CORNERS, ASYMMETRIC, TFCROP_AND_RESIZE = range(5)
ROUND_PREFER_FLOOR, ROUND_PREFER_CEIL, FLOOR, CEIL = range(4)


def resize_nearest(x: np.ndarray, out_h: int, out_w: int, transformation_mode=HALF_PIXEL, nearest_mode=ROUND_PREFER_FLOOR):
    """resize_image(nearest_neighbor) on an NCHW tensor of any 1/2/4-byte dtype."""
    x = np.ascontiguousarray(x)
    n, c, h, w = x.shape
    out = np.empty((n, c, out_h, out_w), x.dtype)
    lib().ref_resize_nearest(_p(x), _p(out), _i(x.dtype.itemsize), _i(n), _i(c), _i(h), _i(w), _i(out_h), _i(out_w),
                             _i(transformation_mode), _i(nearest_mode))
    return out


def qmaxpool(x, kernel, stride, padding, zx, sx, zy, sy) -> np.ndarray:
    """reduce_window2d(max) on u8 NCHW between Dequantize(zx, sx) and Quantize(zy, sy)."""
    x = _c(x, np.uint8)
    n, c, h, w = x.shape
    (ph0, ph1), (pw0, pw1) = padding
    oh = windowed_output_size(h, kernel[0], stride[0], 1, ph0, ph1)
    ow = windowed_output_size(w, kernel[1], stride[1], 1, pw0, pw1)
    out = np.empty((n, c, oh, ow), np.uint8)
    lib().q_maxpool_u8(_p(x), _p(out), _i(n), _i(c), _i(h), _i(w), _i(kernel[0]), _i(kernel[1]), _i(stride[0]), _i(stride[1]),
                       _i(ph0), _i(ph1), _i(pw0), _i(pw1), _i(zx), _f(sx), _i(zy), _f(sy))
    return out


def paged_attention_decode(q_bits, k_cache_bits, v_cache_bits, block_table, ctx_lens, scale):
    """float64 brute force.  q [B,Hq,D] f16 bits; K cache [blocks,Hkv,block,D], V cache [blocks,Hkv,D,block] f16 bits."""
    q = _c(q_bits, np.uint16)
    kc, vc = _c(k_cache_bits, np.uint16), _c(v_cache_bits, np.uint16)
    bt, cl = _c(block_table, np.int32), _c(ctx_lens, np.int32)
    bsz, hq, d = q.shape
    nb, hkv, blk, d2 = kc.shape
    assert d == d2 and vc.shape == (nb, hkv, d, blk)
    out = np.empty((bsz, hq, d), np.float64)
    rc = lib().attn_paged_decode_f64(_p(q), _p(kc), _p(vc), _p(bt), _p(cl), _p(out), _i(bsz), _i(hq), _i(hkv), _i(d),
                                     _i(blk), _i(bt.shape[1]), _i(nb), C.c_double(scale))
    assert rc == 0, f"attn rc={rc}"
    return out


def pack(x: np.ndarray, axes, lanes) -> np.ndarray:
    """pack(x, axes, lanes): every packed axis a of extent D becomes an outer axis of extent
    ceil(D / L) in place, and its lane index is appended as a trailing axis of extent L (in the
    order the axes are listed); missing elements are zero."""
    x = np.asarray(x)
    axes = [a % x.ndim for a in axes]
    pads = [(0, 0)] * x.ndim
    for a, l in zip(axes, lanes):
        pads[a] = (0, (-x.shape[a]) % l)
    xp = np.pad(x, pads)
    split_shape, lane_pos, pos = [], {}, 0
    for d in range(x.ndim):
        if d in axes:
            l = lanes[axes.index(d)]
            split_shape += [xp.shape[d] // l, l]
            lane_pos[d] = pos + 1
            pos += 2
        else:
            split_shape.append(xp.shape[d])
            pos += 1
    y = xp.reshape(split_shape)
    lane_dims = [lane_pos[a] for a in axes]
    outer = [i for i in range(y.ndim) if i not in lane_dims]
    return np.ascontiguousarray(y.transpose(outer + lane_dims))


def unpack(y: np.ndarray, axes, lanes, orig_shape) -> np.ndarray:
    """Inverse of pack with a crop back to orig_shape."""
    y = np.asarray(y)
    nd = len(orig_shape)
    axes = [a % nd for a in axes]
    # outer dims are y.shape[:nd], lane dims y.shape[nd:]
    perm, cur = [], 0
    for d in range(nd):
        perm.append(d)
        if d in axes:
            perm.append(nd + axes.index(d))
    z = y.transpose(perm)
    shape = [y.shape[d] * (lanes[axes.index(d)] if d in axes else 1) for d in range(nd)]
    z = z.reshape(shape)
    return np.ascontiguousarray(z[tuple(slice(0, s) for s in orig_shape)])


def cosine(gt, pred) -> float:
    """Cosine similarity as the reference's test harness computes it (tests/compare_util.py:27-54):
    NaN at the same position of both arrays is dropped, likewise Inf; any non-finite value left over on
    either side gives -1 (so a NaN produced where the expectation is finite fails every threshold);
    identical arrays give 1 (covers all-zero data); a NaN quotient gives -1."""
    gt = np.asarray(gt, np.float64).ravel()
    pred = np.asarray(pred, np.float64).ravel()
    if np.isnan(gt).any() and np.isnan(pred).any():
        keep = ~(np.isnan(gt) & np.isnan(pred))
        gt, pred = gt[keep], pred[keep]
    if np.isinf(gt).any() and np.isinf(pred).any():
        keep = ~(np.isinf(gt) & np.isinf(pred))
        gt, pred = gt[keep], pred[keep]
    if not (np.isfinite(gt).all() and np.isfinite(pred).all()):
        return -1.0
    if np.array_equal(gt, pred):
        return 1.0
    with np.errstate(invalid="ignore", divide="ignore"):
        r = (gt @ pred) / (np.linalg.norm(gt, 2) * np.linalg.norm(pred, 2))
    return -1.0 if np.isnan(r) else float(r)
