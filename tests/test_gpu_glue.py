"""GPU parity of the u8 glue operators (byte-table unary ops, channel concat with requantisation,
nearest-neighbour resize) through the C ABI vs the CPU oracle: all bit-exact."""
import itertools

import numpy as np
import pytest

from nncase_amd import kernels as K
from nncase_amd import runtime as rt
from nncase_amd.runtime import qp
from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", [rt.LUT_REQUANT, rt.LUT_SWISH])
@pytest.mark.parametrize("shape", [(1,), (15,), (16,), (3, 5, 7), (2, 24, 40, 40), (1, 1000003)])
def test_unary_tables(hip_ctx, kind, shape):
    rng = np.random.default_rng(len(shape) * 31 + shape[-1] + kind)
    x = rng.integers(0, 256, shape, dtype=np.uint8)
    zx, sx, zy, sy = 117, 0.061, 9, 0.047
    got = K.unary_u8(kind, x, qp(zx, sx), qp(zy, sy), ctx=hip_ctx)
    assert np.array_equal(got, O.unary_lut(kind, zx, sx, zy, sy)[x])
    # the library's host-side table is the oracle's, entry by entry
    assert np.array_equal(rt.make_unary_lut(kind, qp(zx, sx), qp(zy, sy)), O.unary_lut(kind, zx, sx, zy, sy))


def test_unary_on_unaligned_views(hip_ctx):
    """Device pointers that are not 16-byte aligned take the byte path."""
    x = np.random.default_rng(3).integers(0, 256, 4099, dtype=np.uint8)
    lut = O.unary_lut(O.LUT_SWISH, 100, 0.08, 12, 0.05)
    src, dst = hip_ctx.to_device(x), hip_ctx.alloc(x.size)
    dst.fill(0)

    class View:  # a device address inside a buffer
        def __init__(self, base, off):
            self.ptr = base.ptr + off
    hip_ctx.lut_u8(View(src, 3), View(dst, 5), 4000, lut)
    out = dst.download((x.size,), np.uint8)
    assert np.array_equal(out[5:4005], lut[x[3:4003]]) and (out[:5] == 0).all() and (out[4005:] == 0).all()


@pytest.mark.parametrize("chans", [(64, 64), (32, 96, 16), (3, 5), (128,), (8, 8, 8, 8, 8, 8, 8, 8), (20, 7, 4)])
def test_concat_requantises_every_input(hip_ctx, chans):
    rng = np.random.default_rng(sum(chans))
    n, h, w = 2, 9, 11
    xs = [rng.integers(0, 256, (n, c, h, w), dtype=np.uint8) for c in chans]
    qps = [(int(rng.integers(0, 256)), float(rng.uniform(0.01, 0.1))) for _ in chans]
    out_qp = (90, 0.07)
    got = K.concat(xs, [qp(*q) for q in qps], qp(*out_qp), ctx=hip_ctx)
    want = O.qconcat(xs, qps, out_qp)
    assert got.shape == want.shape and np.array_equal(got, want)
    # identical quant params everywhere: a plain concatenation
    same = K.concat(xs, [qp(*out_qp)] * len(xs), qp(*out_qp), ctx=hip_ctx)
    assert np.array_equal(same, np.concatenate(xs, axis=1))


RESIZE_CASES = [(t, m, size, out) for t, m in itertools.product(range(5), range(4))
                for size, out in (((5, 7), (10, 14)), ((8, 8), (5, 3)), ((3, 4), (3, 4)), ((1, 1), (4, 4)), ((6, 5), (1, 1)),
                                  ((20, 20), (40, 40)))]


@pytest.mark.parametrize("tmode,nmode,size,out", RESIZE_CASES)
def test_resize_nearest_modes(hip_ctx, tmode, nmode, size, out):
    rng = np.random.default_rng(tmode * 100 + nmode * 10 + size[0])
    for c, dt in ((16, np.uint8), (3, np.uint8), (6, np.uint16), (5, np.float32)):
        x = rng.integers(0, 250, (2, c) + size).astype(dt)
        got = K.resize_image_nearest(x, out[0], out[1], tmode, nmode, ctx=hip_ctx)
        want = O.resize_nearest(x, out[0], out[1], tmode, nmode)
        assert got.dtype == want.dtype and np.array_equal(got, want)


def test_resize_yolo_neck_shape(hip_ctx):
    """Config-4 neck upsample at batch 16: [16, 256, 20, 20] -> 40 x 40 (and 40 -> 80), u8; a 2x nearest
    upsample is a repeat in every coordinate mode that centres pixels."""
    rng = np.random.default_rng(8)
    for c, s in ((256, 20), (128, 40)):
        x = rng.integers(0, 256, (16, c, s, s), dtype=np.uint8)
        got = K.resize_image_nearest(x, 2 * s, 2 * s, rt.RESIZE_ASYMMETRIC, rt.NEAREST_FLOOR, ctx=hip_ctx)
        assert np.array_equal(got, x.repeat(2, axis=2).repeat(2, axis=3))
        got = K.resize_image_nearest(x, 2 * s, 2 * s, rt.RESIZE_HALF_PIXEL, rt.NEAREST_ROUND_PREFER_FLOOR, ctx=hip_ctx)
        assert np.array_equal(got, x.repeat(2, axis=2).repeat(2, axis=3))


def test_glue_ops_in_a_resident_function(hip_ctx):
    """conv -> swish table -> upsample -> concat with a skip tensor, recorded once and replayed as a HIP graph."""
    from nncase_amd.runtime import Function
    rng = np.random.default_rng(21)
    n, c, s = 2, 32, 10
    a = rng.integers(0, 256, (n, s, s, c), dtype=np.uint8)          # NHWC
    skip = rng.integers(0, 256, (n, 2 * s, 2 * s, 16), dtype=np.uint8)
    lut = rt.make_unary_lut(rt.LUT_SWISH, qp(128, 0.04), qp(7, 0.03))
    da, dskip = hip_ctx.to_device(a), hip_ctx.to_device(skip)
    d1, d2, d3 = hip_ctx.alloc(a.size), hip_ctx.alloc(a.size * 4), hip_ctx.alloc(n * 4 * s * s * (c + 16))
    fn = Function(hip_ctx)
    fn.add_lut_u8(da, d1, a.size, lut)
    fn.add_resize_nearest(d1, d2, 1, n, s, s, c, 2 * s, 2 * s, rt.RESIZE_ASYMMETRIC, rt.NEAREST_FLOOR)
    fn.add_qconcat_channels([d2, dskip], [c, 16], [qp(7, 0.03), qp(100, 0.05)], d3, qp(20, 0.045), n * 4 * s * s)
    assert [fn.op_kernel(i) for i in range(3)] == ["lut_u8", "resize_nearest", "qconcat<2>"]
    up = O.unary_lut(O.LUT_SWISH, 128, 0.04, 7, 0.03)[a].repeat(2, axis=1).repeat(2, axis=2)
    want = np.concatenate([O.unary_lut(O.LUT_REQUANT, 7, 0.03, 20, 0.045)[up],
                           O.unary_lut(O.LUT_REQUANT, 100, 0.05, 20, 0.045)[skip]], axis=3)
    fn.invoke()
    hip_ctx.sync()
    assert np.array_equal(d3.download(want.shape, np.uint8), want)
    fn.capture()
    for _ in range(3):
        d3.fill(0)
        fn.invoke()
        hip_ctx.sync()
        assert np.array_equal(d3.download(want.shape, np.uint8), want)


def test_error_paths(hip_ctx):
    x = hip_ctx.alloc(64)
    with pytest.raises(rt.HipError):
        hip_ctx.resize_nearest(x, x, 3, 1, 2, 2, 4, 4, 4)            # element size 3
    with pytest.raises(rt.HipError):
        hip_ctx.resize_nearest(x, x, 1, 1, 2, 2, 4, 4, 4, 7, 0)      # unknown coordinate mode
    with pytest.raises(rt.HipError):
        hip_ctx.qconcat_channels([x] * 9, [1] * 9, [qp(0, 1.0)] * 9, x, qp(0, 1.0), 1)   # more than 8 inputs
    with pytest.raises(rt.HipError):
        rt.make_unary_lut(5, qp(0, 1.0), qp(0, 1.0))
    with pytest.raises(rt.HipError):
        rt.make_unary_lut(rt.LUT_SWISH, qp(0, 1.0), qp(0, 0.0))      # zero output scale


@pytest.mark.parametrize("k,s,p", [(5, 1, 2), (3, 2, 1), (2, 2, 0), (3, 1, 0), (5, 1, (2, 1)), (9, 1, 4), (13, 1, 6)])
@pytest.mark.parametrize("c", [16, 3])
def test_maxpool_between_dequantize_and_quantize(hip_ctx, k, s, p, c):
    rng = np.random.default_rng(k * 10 + s + c)
    pad = ((p, p), (p, p)) if isinstance(p, int) else ((p[0], p[1]), (p[1], p[0]))
    x = rng.integers(0, 256, (2, c, 17, 13), dtype=np.uint8)
    for (zx, sx, zy, sy) in [(90, 0.05, 90, 0.05), (120, 0.04, 7, 0.031), (0, 0.1, 30, 0.12), (255, 0.02, 200, 0.02)]:
        got = K.max_pool2d(x, (k, k), (s, s), pad, qp(zx, sx), qp(zy, sy), ctx=hip_ctx)
        want = O.qmaxpool(x, (k, k), (s, s), pad, zx, sx, zy, sy)
        assert got.shape == want.shape and np.array_equal(got, want)


def test_maxpool_sppf_shape(hip_ctx):
    """Config-4 SPPF pooling: 5x5, stride 1, pad 2 on [16, 256, 20, 20]; the float path agrees."""
    rng = np.random.default_rng(2)
    x = rng.integers(0, 256, (16, 256, 20, 20), dtype=np.uint8)
    zx, sx = 13, 0.047
    got = K.max_pool2d(x, (5, 5), (1, 1), ((2, 2), (2, 2)), qp(zx, sx), qp(zx, sx), ctx=hip_ctx)
    assert np.array_equal(got, O.qmaxpool(x, (5, 5), (1, 1), ((2, 2), (2, 2)), zx, sx, zx, sx))
    xp = np.pad(np.maximum(x, 0), ((0, 0), (0, 0), (2, 2), (2, 2)), constant_values=zx)   # 0.0 is the code zx
    win = np.lib.stride_tricks.sliding_window_view(xp, (5, 5), axis=(2, 3)).max(axis=(-1, -2))
    assert np.array_equal(got, win)
