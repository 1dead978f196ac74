"""Host-side mirror of the reference's kernel interface for the operators the `hip`
target owns: same names, argument order and meaning as `kernels::stackvm::*`
(src/Native/include/nncase/kernels/stackvm/tensor_ops.h, tensor_ops.cpp:181-220,268-283,
553-565,681-695), operating on host arrays the way the reference's kernels operate on
host tensors.  Every call stages its operands into HBM, runs the HIP kernel through the
C ABI and copies the result back -- what the native `hip` runtime module does at an
EXTCALL boundary.  Tensors are NCHW / OIHW here, as in the reference; the library works on
NHWC internally and the relayout runs on the device.

Quantised operators take the quantisation parameters the reference's importer attaches as
Dequantize / Quantize nodes around the float op (QLinearConv.cs:61-75).
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np

from . import runtime as rt
from .runtime import Context, QuantParam, qp

_default_ctx: Optional[Context] = None


def default_context() -> Context:
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context(0)
    return _default_ctx


def _ctx(ctx):
    return ctx or default_context()


def _span(a: np.ndarray):
    """(first byte, byte count, strides in elements) of the memory a strided view covers; None for views the
    strided entry points do not take (negative or unaligned strides)."""
    if a.size == 0:
        return None
    if any(st < 0 or st % a.itemsize for st in a.strides):
        return None
    nbytes = sum((n - 1) * st for n, st in zip(a.shape, a.strides)) + a.itemsize
    return a.__array_interface__["data"][0], nbytes, [st // a.itemsize for st in a.strides]


def _elementwise_strided(c: Context, call, x: np.ndarray, out: Optional[np.ndarray], out_dtype: np.dtype, qp_):
    """Runs a strided quantize / dequantize: the operands' memory spans are mirrored on the device, so elements the
    strides skip keep their values, as with the reference's kernels on strided tensors."""
    import ctypes
    xs = _span(x)
    if out is None:
        out = np.empty(x.shape, out_dtype)
    os_ = _span(out)
    if xs is None or os_ is None or out.shape != x.shape or out.dtype != out_dtype or not out.flags.writeable:
        raise rt.HipError(-22, "strided operand", "views need non-negative element-aligned strides, equal shapes and a writable output")
    src = c.to_device(np.frombuffer((ctypes.c_char * xs[1]).from_address(xs[0]), np.uint8))
    host_out = np.frombuffer((ctypes.c_char * os_[1]).from_address(os_[0]), np.uint8)
    dst = c.to_device(host_out)
    call(src, rt.NP_TO_DT[x.dtype], dst, rt.NP_TO_DT.get(out_dtype, 0xFF), x.shape, xs[2], os_[2], qp_)
    host_out[:] = dst.download((os_[1],), np.uint8)
    return out


def quantize(input: np.ndarray, quant_param: QuantParam, out_dtype=np.uint8, ctx: Context = None,
             out: Optional[np.ndarray] = None) -> np.ndarray:
    """kernels::stackvm::quantize(out_type, input, quant_param).  A strided view as `input`, or a strided `out` to
    write into, goes through the strided entry point with the views' own strides, like the reference's call
    (tensor_ops.cpp:690-693 passes input_tensor->strides() and output_tensor->strides())."""
    c = _ctx(ctx)
    x = np.asarray(input)
    if x.dtype not in (np.float32, np.float16):
        raise rt.HipError(-rt.ERR_DATATYPE_MISMATCH, "quantize", f"input dtype {x.dtype}")
    out_dtype = np.dtype(out_dtype)
    if x.size == 0:
        return np.empty(x.shape, out_dtype) if out is None else out
    if out is not None or not x.flags.c_contiguous:
        return _elementwise_strided(c, c.quantize_strided, x, out, out_dtype, quant_param)
    src, dst = c.to_device(x), c.alloc(x.size * out_dtype.itemsize)
    c.quantize(src, rt.NP_TO_DT[x.dtype], dst, rt.NP_TO_DT.get(out_dtype, 0xFF), x.size, quant_param)
    return dst.download(x.shape, out_dtype)


def dequantize(input: np.ndarray, quant_param: QuantParam, out_dtype=np.float32, ctx: Context = None,
               out: Optional[np.ndarray] = None) -> np.ndarray:
    """kernels::stackvm::dequantize(out_type, input, quant_param); strided operands as for quantize."""
    c = _ctx(ctx)
    q = np.asarray(input)
    out_dtype = np.dtype(out_dtype)
    if q.dtype not in rt.NP_TO_DT:
        raise rt.HipError(-rt.ERR_DATATYPE_MISMATCH, "dequantize", f"input dtype {q.dtype}")
    if q.size == 0:
        return np.empty(q.shape, out_dtype) if out is None else out
    if out is not None or not q.flags.c_contiguous:
        return _elementwise_strided(c, c.dequantize_strided, q, out, out_dtype, quant_param)
    src, dst = c.to_device(q), c.alloc(q.size * out_dtype.itemsize)
    c.dequantize(src, rt.NP_TO_DT[q.dtype], dst, rt.NP_TO_DT.get(out_dtype, 0xFF), q.size, quant_param)
    return dst.download(q.shape, out_dtype)


def _out_dt(out_dtype) -> int:
    return rt.NP_TO_DT[np.dtype(out_dtype)]


def conv2d(input: np.ndarray, weights: np.ndarray, bias: Optional[np.ndarray], stride: Sequence[int],
           padding: Sequence[Sequence[int]], dilation: Sequence[int], groups: int, fused_clamp: Tuple[float, float],
           input_qp: QuantParam, weights_qp: QuantParam, output_qp: Optional[QuantParam] = None, out_dtype=np.uint8,
           ctx: Context = None, residual: Optional[np.ndarray] = None, residual_qp: Optional[QuantParam] = None,
           sum_qp: Optional[QuantParam] = None, sum_clamp: Tuple[float, float] = (-rt.FLT_MAX, rt.FLT_MAX),
           post_lut: Optional[np.ndarray] = None, post_lut_qp: Optional[QuantParam] = None) -> np.ndarray:
    """kernels::stackvm::conv2d(pad_mode=constant, input, weights, bias, stride, padding, dilation,
    groups, fused_clamp) on u8 NCHW input / u8 OIHW weights / int32 bias.

    out_dtype uint8 -> requantised with output_qp; int32 -> accumulators; float32 -> clamped
    acc * (sx * sw).  Returns NCHW.
    """
    c = _ctx(ctx)
    x = np.ascontiguousarray(input, np.uint8)
    w = np.ascontiguousarray(weights, np.uint8)
    n, ch, h, wd = x.shape
    oc, gic, kh, kw = w.shape
    if gic * groups != ch:
        raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "conv2d", f"weights expect {gic * groups} input channels, input has {ch}")
    (ph0, ph1), (pw0, pw1) = padding
    oh = rt.windowed_output_size(h, kh, stride[0], dilation[0], ph0, ph1)
    ow = rt.windowed_output_size(wd, kw, stride[1], dilation[1], pw0, pw1)
    wts = c.prepack_conv2d(w, bias, weights_qp, groups, expected_pixels=n * oh * ow)
    x_nchw = c.to_device(x)
    x_nhwc = c.alloc(x.size)
    c.nchw_to_nhwc(x_nchw, x_nhwc, 1, n, ch, h, wd)
    out_dtype = np.dtype(out_dtype)
    es = out_dtype.itemsize
    y_nhwc = c.alloc(max(1, n * oh * ow * oc * es))
    y_nchw = c.alloc(max(1, n * oh * ow * oc * es))
    args = rt.Conv2dArgs(n, h, wd, stride[0], stride[1], dilation[0], dilation[1], ph0, ph1, pw0, pw1, input_qp,
                         output_qp or qp(0, 1.0), fused_clamp[0], fused_clamp[1], _out_dt(out_dtype))
    if post_lut is not None:  # fused Quantize(unary(Dequantize(conv))) as a byte table attached to the weights
        wts.set_post_lut(post_lut, post_lut_qp)
    if residual is not None:  # fused Quantize(Dequantize(conv) + Dequantize(residual)), residual given as NCHW u8
        r = np.ascontiguousarray(residual, np.uint8)
        if r.shape != (n, oc, oh, ow):
            raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "conv2d", f"residual shape {r.shape} != output shape {(n, oc, oh, ow)}")
        r_nchw, r_nhwc = c.to_device(r), c.alloc(r.size)
        c.nchw_to_nhwc(r_nchw, r_nhwc, 1, n, oc, oh, ow)
        args.residual_dev, args.residual_qp, args.sum_qp = r_nhwc.ptr, residual_qp, sum_qp
        args.sum_clamp_min, args.sum_clamp_max = sum_clamp
    c.qconv2d(x_nhwc, wts, y_nhwc, args)
    c.nhwc_to_nchw(y_nhwc, y_nchw, es, n, oc, oh, ow)
    out = y_nchw.download((n, oc, oh, ow), out_dtype)
    wts.destroy()
    return out


def mat_mul(lhs: np.ndarray, rhs: np.ndarray, lhs_qp: QuantParam, rhs_qp: QuantParam,
            output_qp: Optional[QuantParam] = None, out_dtype=np.float32, bias: Optional[np.ndarray] = None,
            fused_clamp: Tuple[float, float] = (-rt.FLT_MAX, rt.FLT_MAX), ctx: Context = None) -> np.ndarray:
    """kernels::stackvm::mat_mul(lhs, rhs) on u8 operands with the reference's operand forms
    (reference/matmul.cpp:28-48): rank-1 operands are a row / a column, both operands may carry up to two batch
    dimensions (rank <= 4) which broadcast against each other where one of them is 1.  lhs [..., M, K] against a
    plain [K, N] matrix is one launch (the batch is stacked into rows); otherwise every distinct rhs matrix is
    pre-packed once and serves all the lhs matrices it is paired with."""
    c = _ctx(ctx)
    a = np.ascontiguousarray(lhs, np.uint8)
    b = np.ascontiguousarray(rhs, np.uint8)
    if a.ndim < 1 or b.ndim < 1 or a.ndim > 4 or b.ndim > 4:
        raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "mat_mul", f"{a.shape} x {b.shape}")
    a1, b1 = a.ndim == 1, b.ndim == 1
    if a1:
        a = a[None, :]
    if b1:
        b = b[:, None]
    if a.shape[-1] != b.shape[-2]:
        raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "mat_mul", f"{np.shape(lhs)} x {np.shape(rhs)}")
    out_dtype = np.dtype(out_dtype)
    k, n = b.shape[-2:]

    def run(a2d, wts):
        m = a2d.shape[0]
        dy = c.alloc(max(1, m * n * out_dtype.itemsize))
        args = rt.MatmulArgs(m, lhs_qp, output_qp or qp(0, 1.0), fused_clamp[0], fused_clamp[1], _out_dt(out_dtype))
        c.qmatmul(c.to_device(a2d), wts, dy, args)
        return dy.download((m, n), out_dtype)

    if b.ndim == 2:                                   # one constant matrix: every lhs row in one launch
        lead = a.shape[:-1]
        m = int(np.prod(lead)) if lead else 1
        wts = c.prepack_matmul(b, bias, rhs_qp, expected_rows=m)
        out = run(a.reshape(m, k), wts).reshape(tuple(lead) + (n,))
        wts.destroy()
    else:
        ab, bb = a.shape[:-2], b.shape[:-2]
        try:
            batch = np.broadcast_shapes(ab, bb)
        except ValueError:
            raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "mat_mul", f"{np.shape(lhs)} x {np.shape(rhs)}") from None
        m = a.shape[-2]
        ai = np.broadcast_to(np.arange(int(np.prod(ab)) if ab else 1).reshape(ab), batch).ravel()
        bi = np.broadcast_to(np.arange(int(np.prod(bb))).reshape(bb), batch).ravel()
        amats, bmats = a.reshape(-1, m, k), b.reshape(-1, k, n)
        out = np.empty((len(bi), m, n), out_dtype)
        for j in np.unique(bi):                       # one pre-pack per distinct rhs matrix
            sel = np.nonzero(bi == j)[0]
            wts = c.prepack_matmul(np.ascontiguousarray(bmats[j]), bias, rhs_qp, expected_rows=m * len(sel))
            out[sel] = run(np.ascontiguousarray(amats[ai[sel]]).reshape(-1, k), wts).reshape(len(sel), m, n)
            wts.destroy()
        out = out.reshape(tuple(batch) + (m, n))
    if a1:
        out = out.squeeze(-2)
    if b1:
        out = out.squeeze(-1)
    return out


def binary_add(lhs: np.ndarray, rhs: np.ndarray, lhs_qp: QuantParam, rhs_qp: QuantParam, output_qp: QuantParam,
               fused_clamp: Tuple[float, float] = (-rt.FLT_MAX, rt.FLT_MAX), ctx: Context = None) -> np.ndarray:
    """Quantize(Dequantize(lhs) + Dequantize(rhs)) on equal-shape u8 tensors."""
    c = _ctx(ctx)
    a, b = np.ascontiguousarray(lhs, np.uint8), np.ascontiguousarray(rhs, np.uint8)
    if a.shape != b.shape:
        raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "binary_add", f"{a.shape} vs {b.shape}")
    da, db, dy = c.to_device(a), c.to_device(b), c.alloc(a.size)
    c.qadd(da, lhs_qp, db, rhs_qp, dy, output_qp, a.size, fused_clamp)
    return dy.download(a.shape, np.uint8)


def global_average_pool(input: np.ndarray, input_qp: QuantParam, output_qp: QuantParam, ctx: Context = None) -> np.ndarray:
    """reduce_window2d(mean) over the whole image of a u8 NCHW tensor -> u8 [N, C, 1, 1]."""
    c = _ctx(ctx)
    x = np.ascontiguousarray(input, np.uint8)
    n, ch, h, w = x.shape
    d_nchw, d_nhwc, dy = c.to_device(x), c.alloc(x.size), c.alloc(n * ch)
    c.nchw_to_nhwc(d_nchw, d_nhwc, 1, n, ch, h, w)
    c.qglobal_avgpool(d_nhwc, dy, n, h, w, ch, input_qp, output_qp)
    return dy.download((n, ch, 1, 1), np.uint8)


def _to_nhwc_dev(c, x: np.ndarray):
    n, ch, h, w = x.shape
    d_nchw, d_nhwc = c.to_device(x), c.alloc(max(1, x.nbytes))
    c.nchw_to_nhwc(d_nchw, d_nhwc, x.itemsize, n, ch, h, w)
    return d_nhwc


def _from_nhwc_dev(c, d_nhwc, shape_nchw, dtype) -> np.ndarray:
    n, ch, h, w = shape_nchw
    dtype = np.dtype(dtype)
    d_nchw = c.alloc(max(1, int(np.prod(shape_nchw)) * dtype.itemsize))
    c.nhwc_to_nchw(d_nhwc, d_nchw, dtype.itemsize, n, ch, h, w)
    return d_nchw.download(tuple(shape_nchw), dtype)


def unary_u8(kind: int, input: np.ndarray, input_qp: QuantParam, output_qp: QuantParam, ctx: Context = None) -> np.ndarray:
    """Quantize(unary(Dequantize(x))) on u8 data of any shape as one byte-table pass;
    kind = runtime.LUT_REQUANT (identity) or runtime.LUT_SWISH (kernels::stackvm::unary swish)."""
    c = _ctx(ctx)
    x = np.ascontiguousarray(input, np.uint8)
    lut = rt.make_unary_lut(kind, input_qp, output_qp)
    src, dst = c.to_device(x), c.alloc(max(1, x.size))
    c.lut_u8(src, dst, x.size, lut)
    return dst.download(x.shape, np.uint8)


def concat(inputs: Sequence[np.ndarray], input_qps: Sequence[QuantParam], output_qp: QuantParam, ctx: Context = None) -> np.ndarray:
    """kernels::stackvm::concat on axis 1 of u8 NCHW tensors, every input requantised to output_qp."""
    c = _ctx(ctx)
    xs = [np.ascontiguousarray(x, np.uint8) for x in inputs]
    n, _, h, w = xs[0].shape
    for x in xs:
        if x.ndim != 4 or (x.shape[0], x.shape[2], x.shape[3]) != (n, h, w):
            raise rt.HipError(-rt.ERR_SHAPE_MISMATCH, "concat", f"{[x.shape for x in xs]}")
    chans = [x.shape[1] for x in xs]
    devs = [_to_nhwc_dev(c, x) for x in xs]
    out = c.alloc(max(1, n * h * w * sum(chans)))
    c.qconcat_channels(devs, chans, list(input_qps), out, output_qp, n * h * w)
    return _from_nhwc_dev(c, out, (n, sum(chans), h, w), np.uint8)


def resize_image_nearest(input: np.ndarray, out_h: int, out_w: int, transformation_mode: int = rt.RESIZE_HALF_PIXEL,
                         nearest_mode: int = rt.NEAREST_ROUND_PREFER_FLOOR, ctx: Context = None) -> np.ndarray:
    """kernels::stackvm::resize_image(nearest_neighbor) on an NCHW tensor with 1/2/4-byte elements."""
    c = _ctx(ctx)
    x = np.ascontiguousarray(input)
    n, ch, h, w = x.shape
    src = _to_nhwc_dev(c, x)
    dst = c.alloc(max(1, n * ch * out_h * out_w * x.itemsize))
    c.resize_nearest(src, dst, x.itemsize, n, h, w, ch, out_h, out_w, transformation_mode, nearest_mode)
    return _from_nhwc_dev(c, dst, (n, ch, out_h, out_w), x.dtype)


def max_pool2d(input: np.ndarray, kernel: Sequence[int], stride: Sequence[int], padding: Sequence[Sequence[int]],
               input_qp: QuantParam, output_qp: QuantParam, ctx: Context = None) -> np.ndarray:
    """reduce_window2d(max) on a u8 NCHW tensor between Dequantize(input_qp) and Quantize(output_qp)."""
    c = _ctx(ctx)
    x = np.ascontiguousarray(input, np.uint8)
    n, ch, h, w = x.shape
    (ph0, ph1), (pw0, pw1) = padding
    oh = rt.windowed_output_size(h, kernel[0], stride[0], 1, ph0, ph1)
    ow = rt.windowed_output_size(w, kernel[1], stride[1], 1, pw0, pw1)
    src = _to_nhwc_dev(c, x)
    dst = c.alloc(max(1, n * ch * oh * ow))
    c.qmaxpool2d(src, dst, n, h, w, ch, kernel, stride, padding, input_qp, output_qp)
    return _from_nhwc_dev(c, dst, (n, ch, oh, ow), np.uint8)


def pack(input: np.ndarray, axes: Sequence[int], lanes: Sequence[int], ctx: Context = None) -> np.ndarray:
    c = _ctx(ctx)
    x = np.ascontiguousarray(input)
    nd = x.ndim
    ax = [a % nd for a in axes]
    out_shape = [(-(-x.shape[d] // lanes[ax.index(d)])) if d in ax else x.shape[d] for d in range(nd)] + list(lanes)
    src, dst = c.to_device(x), c.alloc(int(np.prod(out_shape)) * x.itemsize)
    c.pack(src, dst, x.itemsize, list(x.shape), list(axes), list(lanes))
    return dst.download(tuple(out_shape), x.dtype)


def unpack(input: np.ndarray, axes: Sequence[int], lanes: Sequence[int], unpacked_shape: Sequence[int],
           ctx: Context = None) -> np.ndarray:
    c = _ctx(ctx)
    y = np.ascontiguousarray(input)
    src, dst = c.to_device(y), c.alloc(int(np.prod(unpacked_shape)) * y.itemsize)
    c.unpack(src, dst, y.itemsize, list(unpacked_shape), list(axes), list(lanes))
    return dst.download(tuple(unpacked_shape), y.dtype)


def transpose_nchw_to_nhwc(input: np.ndarray, ctx: Context = None) -> np.ndarray:
    c = _ctx(ctx)
    x = np.ascontiguousarray(input)
    n, ch, h, w = x.shape
    src, dst = c.to_device(x), c.alloc(x.nbytes)
    c.nchw_to_nhwc(src, dst, x.itemsize, n, ch, h, w)
    return dst.download((n, h, w, ch), x.dtype)


def transpose_nhwc_to_nchw(input: np.ndarray, ctx: Context = None) -> np.ndarray:
    c = _ctx(ctx)
    x = np.ascontiguousarray(input)
    n, h, w, ch = x.shape
    src, dst = c.to_device(x), c.alloc(x.nbytes)
    c.nhwc_to_nchw(src, dst, x.itemsize, n, ch, h, w)
    return dst.download((n, ch, h, w), x.dtype)


def v_cache_from_token_major(v_cache: np.ndarray) -> np.ndarray:
    """[blocks, Hkv, block, D] -> the d-major [blocks, Hkv, D, block] layout the decode kernel reads."""
    return np.ascontiguousarray(np.asarray(v_cache).transpose(0, 1, 3, 2))


def paged_attention_decode(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray, block_table: np.ndarray,
                           ctx_lens: np.ndarray, scale: float, out_dtype=np.float32, ctx: Context = None) -> np.ndarray:
    """q [B, Hq, D] f16; K cache [blocks, Hkv, block, D] f16; V cache [blocks, Hkv, D, block] f16 (d-major, see
    v_cache_from_token_major); block_table [B, max_blocks] i32; ctx_lens [B] i32."""
    c = _ctx(ctx)
    qh = np.ascontiguousarray(q, np.float16)
    kc, vc = np.ascontiguousarray(k_cache, np.float16), np.ascontiguousarray(v_cache, np.float16)
    bt, cl = np.ascontiguousarray(block_table, np.int32), np.ascontiguousarray(ctx_lens, np.int32)
    bsz, hq, d = qh.shape
    nb, hkv, blk, _ = kc.shape
    if vc.shape != (nb, hkv, d, blk):
        raise ValueError(f"v_cache shape {vc.shape}: expected the d-major layout {(nb, hkv, d, blk)}")
    out_dtype = np.dtype(out_dtype)
    dq, dk, dv, dbt, dcl = (c.to_device(t) for t in (qh, kc, vc, bt, cl))
    dout = c.alloc(bsz * hq * d * out_dtype.itemsize)
    args = rt.PagedAttnArgs(bsz, hq, hkv, d, blk, bt.shape[1], nb, float(scale), rt.NP_TO_DT[out_dtype])
    c.paged_attention_decode(dq, dk, dv, dbt, dcl, dout, args)
    return dout.download((bsz, hq, d), out_dtype)
