"""GPU parity of the pointwise pair ([3x3 depthwise convolution ->] 1x1 convolution [+ byte table] [+ residual] -> 1x1
convolution [+ byte table] as one launch) through the C ABI: both results must be bit-identical to the CPU oracle
running the operators one after the other, and to nncase_hip_qconv2d called once per convolution on the device."""
import numpy as np
import pytest

from nncase_amd import runtime as rt
from nncase_amd.runtime import qp
from oracle import oracle as O
from test_gpu_block import pick_quant

pytestmark = pytest.mark.gpu
f32 = np.float32
FULL = (-rt.FLT_MAX, rt.FLT_MAX)


def conv_args(n, h, w, x_qp, y_qp, clamp):
    return rt.Conv2dArgs(n, h, w, 1, 1, 1, 1, 0, 0, 0, 0, x_qp, y_qp, clamp[0], clamp[1], rt.DT_U8)


def run_pair(ctx, n, k1, n1, n2, h, w, seed, residual=False, lut_a=False, lut_b=False, relu_b=True, dw=None):
    """dw = (stride, padding): h x w is then the input of a 3x3 depthwise convolution in front of the pair."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, k1, h, w), dtype=np.uint8)
    front = None
    if dw is not None:
        stride, pad = dw
        x0, (z0, s0) = x, (11, f32(0.019))
        wd = rng.integers(0, 256, (k1, 1, 3, 3), dtype=np.uint8)
        bd = rng.integers(-3000, 3000, k1).astype(np.int32)
        zwd, swd = 119, f32(0.0123)
        dwk = dict(stride=(stride, stride), padding=pad, dilation=(1, 1), groups=k1)
        real = O.qconv2d(x0, wd, bd, z0, s0, zwd, swd, out_mode=O.OUT_F32, **dwk)
        cd, zd, sd = pick_quant(real)
        x = O.qconv2d(x0, wd, bd, z0, s0, zwd, swd, zd, sd, fused_clamp=cd, out_mode=O.OUT_U8, **dwk)
        in_h, in_w = h, w
        h, w = x.shape[2:]
        dww = ctx.prepack_conv2d(wd, bd, qp(zwd, swd), groups=k1)
        (ph0, ph1), (pw0, pw1) = pad
        da_ = rt.Conv2dArgs(n, in_h, in_w, stride, stride, 1, 1, ph0, ph1, pw0, pw1, qp(z0, s0), qp(zd, sd), cd[0], cd[1], rt.DT_U8)
        front = (x0, dww, da_)
    wa = rng.integers(0, 256, (n1, k1, 1, 1), dtype=np.uint8)
    wb = rng.integers(0, 256, (n2, n1, 1, 1), dtype=np.uint8)
    ba = rng.integers(-3000, 3000, n1).astype(np.int32)
    bb = rng.integers(-3000, 3000, n2).astype(np.int32)
    zx, sx = (9, f32(0.0235)) if front is None else (zd, sd)
    (zwa, swa), (zwb, swb) = (131, f32(0.0041)), (122, f32(0.0037))
    # the oracle, operator by operator
    real = O.qconv2d(x, wa, ba, zx, sx, zwa, swa, out_mode=O.OUT_F32)
    c1, z1, s1 = pick_quant(real, relu6_like=False)
    y1 = O.qconv2d(x, wa, ba, zx, sx, zwa, swa, z1, s1, fused_clamp=c1, out_mode=O.OUT_U8)
    zc, sc = z1, s1                                      # the first convolution's own output quantisation
    ta = tb = None
    if lut_a:
        ta = rng.permutation(256).astype(np.uint8)
        y1 = ta[y1]
        z1, s1 = 17, f32(s1 * 1.25)                      # the table's own output quantisation
    res = None
    if residual:
        res = rng.integers(0, 256, y1.shape, dtype=np.uint8)
        zr, sr = 101, f32(0.031)
        fa = (y1.astype(f32) - f32(z1)) * s1 + (res.astype(f32) - f32(zr)) * sr
        _, zs, ss = pick_quant(fa)
        y1 = O.qadd(y1, res, z1, s1, zr, sr, zs, ss)
        z_mid, s_mid = zs, ss
    else:
        z_mid, s_mid = z1, s1
    real = O.qconv2d(y1, wb, bb, z_mid, s_mid, zwb, swb, out_mode=O.OUT_F32)
    c2, z2, s2 = pick_quant(real, relu6_like=relu_b)
    y2 = O.qconv2d(y1, wb, bb, z_mid, s_mid, zwb, swb, z2, s2, fused_clamp=c2, out_mode=O.OUT_U8)
    if lut_b:
        tb = rng.permutation(256).astype(np.uint8)
        y2 = tb[y2]

    first = ctx.prepack_conv2d(wa, ba, qp(zwa, swa))
    second = ctx.prepack_conv2d(wb, bb, qp(zwb, swb))
    if lut_a:
        first.set_post_lut(ta, qp(z1, s1))
    if lut_b:
        second.set_post_lut(tb, qp(z2, s2))
    pair = ctx.prepack_qpointwise_pair(first, wa, second, wb)
    fa_ = conv_args(n, h, w, qp(zx, sx), qp(zc, sc), c1)
    sa_ = conv_args(n, h, w, qp(z_mid, s_mid), qp(z2, s2), c2)
    xd = ctx.alloc(x.size).upload(np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    keep = [xd]
    if front is not None:
        x0d = ctx.alloc(front[0].size).upload(np.ascontiguousarray(front[0].transpose(0, 2, 3, 1)))
        keep.append(x0d)
    if residual:
        rd = ctx.alloc(res.size).upload(np.ascontiguousarray(res.transpose(0, 2, 3, 1)))
        keep.append(rd)
        fa_.residual_dev = rd.ptr
        fa_.residual_qp = qp(zr, sr)
        fa_.sum_qp = qp(zs, ss)
        fa_.sum_clamp_min, fa_.sum_clamp_max = FULL
    y1d = ctx.alloc(n * h * w * n1).fill(0xA5)
    y2d = ctx.alloc(n * h * w * n2).fill(0xA5)
    if front is None:
        ctx.qpointwise_pair(xd, pair, y1d, y2d, fa_, sa_)
    else:
        ctx.qdepthwise_pointwise_pair(x0d, front[1], front[2], pair, y1d, y2d, fa_, sa_)
    ctx.sync()
    got1 = y1d.download((n, h, w, n1), np.uint8).transpose(0, 3, 1, 2)
    got2 = y2d.download((n, h, w, n2), np.uint8).transpose(0, 3, 1, 2)
    for name, got, want in (("first", got1, y1), ("second", got2, y2)):
        bad = got != want
        assert not bad.any(), f"{name}: {bad.sum()} of {want.size} bytes differ; first at {np.argwhere(bad)[0]}: got {got[bad][0]} want {want[bad][0]}"
    assert y2.size < 256 or len(np.unique(y2)) > 8
    # the two stand-alone operators on the device
    u1 = ctx.alloc(n * h * w * n1).fill(0x5A)
    u2 = ctx.alloc(n * h * w * n2).fill(0x5A)
    if front is not None:
        ctx.qconv2d(x0d, front[1], xd.fill(0x5A), front[2])
    ctx.qconv2d(xd, first, u1, fa_)
    ctx.qconv2d(u1, second, u2, sa_)
    ctx.sync()
    assert np.array_equal(u1.download((n, h, w, n1), np.uint8), y1d.download((n, h, w, n1), np.uint8))
    assert np.array_equal(u2.download((n, h, w, n2), np.uint8), y2d.download((n, h, w, n2), np.uint8))
    return pair, (xd if front is None else x0d, y1d, y2d, fa_, sa_, keep + ([front] if front is not None else []))


MOBILENET_PAIRS = [  # (in, mid, out, h, w, residual): every projection -> expansion pair of MobileNetV2 1.0 at batch 1
    (32, 16, 96, 112, 112, False), (96, 24, 144, 56, 56, False), (144, 24, 144, 56, 56, True), (144, 32, 192, 28, 28, False),
    (192, 32, 192, 28, 28, True), (192, 64, 384, 14, 14, False), (384, 64, 384, 14, 14, True), (384, 96, 576, 14, 14, False),
    (576, 96, 576, 14, 14, True), (576, 160, 960, 7, 7, False), (960, 160, 960, 7, 7, True), (960, 320, 1280, 7, 7, False),
]


@pytest.mark.parametrize("k1,n1,n2,h,w,residual", MOBILENET_PAIRS)
def test_mobilenet_pair_shapes(hip_ctx, k1, n1, n2, h, w, residual):
    hw = (h, w) if h <= 28 else (h // 4, w // 4 + 1)       # the oracle follows the larger maps on a part of them
    run_pair(hip_ctx, 1, k1, n1, n2, hw[0], hw[1], seed=k1 + n1 * 7 + n2, residual=residual)


RAGGED = [  # (n, in, mid, out, h, w, residual, lut_a, lut_b, relu_b): pixel counts that fill no tile, channels that fill no tile or k-step
    (1, 16, 4, 4, 1, 1, False, False, False, True), (3, 48, 20, 36, 5, 3, True, False, False, False),
    (2, 80, 68, 200, 9, 7, False, True, False, True), (1, 1024, 512, 24, 3, 3, True, True, True, True),
    (5, 16, 64, 132, 3, 3, False, False, True, False), (2, 272, 12, 1000, 4, 5, True, False, True, True),
]


@pytest.mark.parametrize("n,k1,n1,n2,h,w,residual,lut_a,lut_b,relu_b", RAGGED)
def test_ragged_pairs(hip_ctx, n, k1, n1, n2, h, w, residual, lut_a, lut_b, relu_b):
    run_pair(hip_ctx, n, k1, n1, n2, h, w, seed=n + k1 + n1 + n2 + h * w, residual=residual, lut_a=lut_a, lut_b=lut_b, relu_b=relu_b)


P1 = ((1, 1), (1, 1))
MOBILENET_TRIPLES = [  # (channels, mid, out, in_h, in_w, depthwise stride, residual): MobileNetV2's depthwise -> projection -> expansion
    (96, 24, 144, 28, 30, 2, False), (144, 24, 144, 14, 15, 1, True), (144, 32, 192, 56, 56, 2, False), (192, 32, 192, 28, 28, 1, True),
    (192, 64, 384, 28, 28, 2, False), (384, 64, 384, 14, 14, 1, True), (384, 96, 576, 14, 14, 1, False), (576, 96, 576, 14, 14, 1, True),
    (576, 160, 960, 14, 14, 2, False), (960, 160, 960, 7, 7, 1, True), (960, 320, 1280, 7, 7, 1, False),
]


@pytest.mark.parametrize("k1,n1,n2,h,w,stride,residual", MOBILENET_TRIPLES)
def test_mobilenet_depthwise_pair_shapes(hip_ctx, k1, n1, n2, h, w, stride, residual):
    pad = P1 if stride == 1 else ((0, 1), (0, 1))
    run_pair(hip_ctx, 1, k1, n1, n2, h, w, seed=k1 * 3 + n1 + n2 + stride, residual=residual, dw=(stride, pad))


RAGGED_TRIPLES = [  # (n, channels, mid, out, in_h, in_w, stride, padding, residual, lut_a): windows cut by every edge, images that end inside a pixel tile
    (3, 16, 8, 20, 5, 5, 1, P1, True, False), (2, 48, 20, 36, 9, 7, 2, P1, False, True), (1, 32, 12, 64, 3, 3, 1, ((0, 0), (0, 0)), False, False),
    (2, 80, 16, 48, 6, 11, 2, ((0, 1), (1, 0)), True, False), (5, 1024, 24, 32, 3, 4, 1, P1, False, False), (1, 64, 4, 4, 1, 1, 1, P1, False, False),
]


@pytest.mark.parametrize("n,k1,n1,n2,h,w,stride,pad,residual,lut_a", RAGGED_TRIPLES)
def test_ragged_depthwise_pairs(hip_ctx, n, k1, n1, n2, h, w, stride, pad, residual, lut_a):
    run_pair(hip_ctx, n, k1, n1, n2, h, w, seed=n * 5 + k1 + n1 + n2 + h * w, residual=residual, lut_a=lut_a, dw=(stride, pad))


def test_depthwise_pair_in_a_function_repeats(hip_ctx):
    pair, (x0d, y1d, y2d, fa_, sa_, keep) = run_pair(hip_ctx, 2, 96, 24, 144, 14, 14, seed=4, dw=(1, P1))
    _, dww, da_ = keep[-1]
    want1, want2 = y1d.download((y1d.nbytes,), np.uint8), y2d.download((y2d.nbytes,), np.uint8)
    fn = rt.Function(hip_ctx)
    fn.add_qdepthwise_pointwise_pair(x0d, dww, da_, pair, y1d, y2d, fa_, sa_)
    assert fn.op_kernel(0) == "dw3x3+qpointwise_pair_kernel"
    fn.capture()
    for _ in range(2):
        y1d.fill(0x33)
        y2d.fill(0x33)
        fn.invoke()
        hip_ctx.sync()
        assert np.array_equal(y1d.download((y1d.nbytes,), np.uint8), want1)
        assert np.array_equal(y2d.download((y2d.nbytes,), np.uint8), want2)
    # argument checks of the depthwise front
    other = rt.Conv2dArgs(2, 14, 14, 1, 1, 1, 1, 0, 0, 0, 0, da_.x_qp, da_.y_qp, da_.clamp_min, da_.clamp_max, rt.DT_U8)   # 12 x 12 result
    with pytest.raises(rt.HipError):
        hip_ctx.qdepthwise_pointwise_pair(x0d, dww, other, pair, y1d, y2d, fa_, sa_)
    other = rt.Conv2dArgs(2, 14, 14, 1, 1, 1, 1, 1, 1, 1, 1, da_.x_qp, qp(da_.y_qp.zero_point + 1, da_.y_qp.scale), da_.clamp_min, da_.clamp_max,
                          rt.DT_U8)
    with pytest.raises(rt.HipError):
        hip_ctx.qdepthwise_pointwise_pair(x0d, dww, other, pair, y1d, y2d, fa_, sa_)
    with pytest.raises(rt.HipError):
        hip_ctx.qdepthwise_pointwise_pair(x0d, pair.first, da_, pair, y1d, y2d, fa_, sa_)     # not a depthwise convolution


def test_pair_in_a_function_repeats(hip_ctx):
    """Recorded in a function and replayed as a graph, twice into poisoned outputs."""
    pair, (xd, y1d, y2d, fa_, sa_, keep) = run_pair(hip_ctx, 2, 96, 24, 144, 14, 14, seed=3)
    want1, want2 = y1d.download((y1d.nbytes,), np.uint8), y2d.download((y2d.nbytes,), np.uint8)
    fn = rt.Function(hip_ctx)
    fn.add_qpointwise_pair(xd, pair, y1d, y2d, fa_, sa_)
    assert fn.op_kernel(0) == "qpointwise_pair_kernel"
    fn.capture()
    for _ in range(2):
        y1d.fill(0x33)
        y2d.fill(0x33)
        fn.invoke()
        hip_ctx.sync()
        assert np.array_equal(y1d.download((y1d.nbytes,), np.uint8), want1)
        assert np.array_equal(y2d.download((y2d.nbytes,), np.uint8), want2)


def test_pair_argument_checks(hip_ctx):
    rng = np.random.default_rng(0)
    wa = rng.integers(0, 256, (24, 96, 1, 1), dtype=np.uint8)
    wb = rng.integers(0, 256, (144, 24, 1, 1), dtype=np.uint8)
    w3 = rng.integers(0, 256, (24, 96, 3, 3), dtype=np.uint8)
    first, second = hip_ctx.prepack_conv2d(wa, None, qp(128, 0.01)), hip_ctx.prepack_conv2d(wb, None, qp(128, 0.01))
    assert hip_ctx.qpointwise_pair_supported(96, 24, 144)
    assert not hip_ctx.qpointwise_pair_supported(24, 24, 144)         # rows of x must be whole 16-byte pieces
    assert not hip_ctx.qpointwise_pair_supported(96, 22, 144)
    assert not hip_ctx.qpointwise_pair_supported(2048, 24, 144)
    with pytest.raises(rt.HipError):
        hip_ctx.prepack_qpointwise_pair(first, wa, first, wa)            # 24 outputs feed a 96-channel reduction
    with pytest.raises(rt.HipError):
        hip_ctx.prepack_qpointwise_pair(hip_ctx.prepack_conv2d(w3, None, qp(128, 0.01)), w3[:, :, :1, :1], second, wb)
    pair = hip_ctx.prepack_qpointwise_pair(first, wa, second, wb)
    xd, y1d, y2d = hip_ctx.alloc(4 * 96), hip_ctx.alloc(4 * 24), hip_ctx.alloc(4 * 144)
    good = conv_args(1, 2, 2, qp(0, 0.02), qp(3, 0.05), FULL)
    hip_ctx.qpointwise_pair(xd, pair, y1d, y2d, good, good)
    hip_ctx.sync()
    for field, value in (("stride_h", 2), ("pad_w_before", 1), ("out_dtype", rt.DT_F32), ("out_channel_stride", 256)):
        bad = conv_args(1, 2, 2, qp(0, 0.02), qp(3, 0.05), FULL)
        setattr(bad, field, value)
        with pytest.raises(rt.HipError):
            hip_ctx.qpointwise_pair(xd, pair, y1d, y2d, good, bad)
    other = conv_args(1, 2, 3, qp(0, 0.02), qp(3, 0.05), FULL)
    with pytest.raises(rt.HipError):
        hip_ctx.qpointwise_pair(xd, pair, y1d, y2d, good, other)
    withres = conv_args(1, 2, 2, qp(0, 0.02), qp(3, 0.05), FULL)
    withres.residual_dev = y1d.ptr
    withres.residual_qp, withres.sum_qp = qp(0, 0.02), qp(0, 0.02)
    with pytest.raises(rt.HipError):
        hip_ctx.qpointwise_pair(xd, pair, y1d, y2d, good, withres)


# ---- the few-pixel path of one dense 1x1 convolution (weights in registers), alone and behind a global average pool ----
ROWS = [  # (rows, in, out, table, dequantised): m of a classifier head, channel counts that fill no tile / k-step, several pixel tiles
    (1, 1280, 1000, False, True), (2, 64, 4, False, False), (16, 16, 36, True, False), (17, 80, 200, False, False),
    (5, 2048, 24, True, True), (32, 272, 132, False, True), (3, 1024, 1024, False, False),
]


@pytest.mark.parametrize("m,k,n,lut,deq", ROWS)
def test_rows_path_of_qconv2d(hip_ctx, m, k, n, lut, deq):
    rng = np.random.default_rng(m * 31 + k + n)
    x = rng.integers(0, 256, (m, k, 1, 1), dtype=np.uint8)
    w = rng.integers(0, 256, (n, k, 1, 1), dtype=np.uint8)
    b = rng.integers(-3000, 3000, n).astype(np.int32)
    zx, sx, zw, sw = 9, f32(0.0235), 131, f32(0.0041)
    real = O.qconv2d(x, w, b, zx, sx, zw, sw, out_mode=O.OUT_F32)
    c, zy, sy = pick_quant(real)
    want = O.qconv2d(x, w, b, zx, sx, zw, sw, zy, sy, fused_clamp=c, out_mode=O.OUT_U8)
    zl, sl = zy, sy
    wt = hip_ctx.prepack_conv2d(w, b, qp(zw, sw), expected_pixels=m)
    if lut:
        table = rng.permutation(256).astype(np.uint8)
        want = table[want]
        zl, sl = 23, f32(sy * 1.5)
        wt.set_post_lut(table, qp(zl, sl))
    a = conv_args(m, 1, 1, qp(zx, sx), qp(zy, sy), c)
    if deq:
        a.out_dtype, a.dequantize_output = rt.DT_F32, 1
        want = ((want.astype(np.int32) - zl).astype(f32) * sl).astype(f32)
    fn = rt.Function(hip_ctx)
    xd = hip_ctx.alloc(x.size).upload(np.ascontiguousarray(x.reshape(m, k)))
    yd = hip_ctx.alloc(m * n * (4 if deq else 1)).fill(0xA5)
    fn.add_qconv2d(xd, wt, yd, a)
    assert fn.op_kernel(0).startswith("qpointwise_rows")          # the path under test is the one taken
    for _ in range(2):
        hip_ctx.qconv2d(xd, wt, yd, a)
        hip_ctx.sync()
        got = yd.download((m, n), f32 if deq else np.uint8)
        assert np.array_equal(got.view(np.uint32) if deq else got, want.reshape(m, n).view(np.uint32) if deq else want.reshape(m, n))
        yd.fill(0x5A)
    # the same weights packed for many pixels take the tiled kernels: same bytes
    big = hip_ctx.prepack_conv2d(w, b, qp(zw, sw), expected_pixels=1 << 20)
    if lut:
        big.set_post_lut(table, qp(zl, sl))
    fn2 = rt.Function(hip_ctx)
    fn2.add_qconv2d(xd, big, yd, a)
    assert not fn2.op_kernel(0).startswith("qpointwise_rows")
    hip_ctx.qconv2d(xd, big, yd, a)
    hip_ctx.sync()
    got = yd.download((m, n), f32 if deq else np.uint8)
    assert np.array_equal(got.view(np.uint32) if deq else got, want.reshape(m, n).view(np.uint32) if deq else want.reshape(m, n))


POOLED = [  # (batch, h, w, channels, out, dequantised)
    (1, 7, 7, 1280, 1000, True), (2, 7, 7, 320, 36, False), (3, 1, 1, 64, 20, False), (1, 10, 9, 96, 132, True), (5, 3, 3, 48, 8, False),
]


@pytest.mark.parametrize("n,h,w,c,oc,deq", POOLED)
def test_global_average_pool_in_front_of_a_convolution(hip_ctx, n, h, w, c, oc, deq):
    rng = np.random.default_rng(n + h * w + c + oc)
    x = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    wt_ = rng.integers(0, 256, (oc, c, 1, 1), dtype=np.uint8)
    b = rng.integers(-3000, 3000, oc).astype(np.int32)
    zx, sx, zw, sw = 9, f32(0.0235), 131, f32(0.0041)
    zp, sp = 13, f32(0.011)                                # the pooled tensor's quantisation
    pooled = O.qglobal_avgpool(x, zx, sx, zp, sp).reshape(n, c, 1, 1)
    assert len(np.unique(pooled)) > 4
    real = O.qconv2d(pooled, wt_, b, zp, sp, zw, sw, out_mode=O.OUT_F32)
    cl, zy, sy = pick_quant(real)
    want = O.qconv2d(pooled, wt_, b, zp, sp, zw, sw, zy, sy, fused_clamp=cl, out_mode=O.OUT_U8)
    wt = hip_ctx.prepack_conv2d(wt_, b, qp(zw, sw), expected_pixels=n)
    a = conv_args(n, 1, 1, qp(zp, sp), qp(zy, sy), cl)
    if deq:
        a.out_dtype, a.dequantize_output = rt.DT_F32, 1
        want = ((want.astype(np.int32) - zy).astype(f32) * sy).astype(f32)
    assert hip_ctx.qglobal_avgpool_qconv2d_supported(wt, a, h, w)
    xd = hip_ctx.alloc(x.size).upload(np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    yd = hip_ctx.alloc(n * oc * (4 if deq else 1)).fill(0xA5)
    fn = rt.Function(hip_ctx)
    fn.add_qglobal_avgpool_qconv2d(xd, h, w, qp(zx, sx), wt, yd, a)
    fn.capture()
    for _ in range(2):
        fn.invoke()
        hip_ctx.sync()
        got = yd.download((n, oc), f32 if deq else np.uint8)
        assert np.array_equal(got.view(np.uint32) if deq else got, want.reshape(n, oc).view(np.uint32) if deq else want.reshape(n, oc))
        yd.fill(0x5A)
    # the two operators one after the other on the device
    pd = hip_ctx.alloc(n * c).fill(0)
    hip_ctx.qglobal_avgpool(xd, pd, n, h, w, c, qp(zx, sx), qp(zp, sp))
    hip_ctx.qconv2d(pd, wt, yd, a)
    hip_ctx.sync()
    got = yd.download((n, oc), f32 if deq else np.uint8)
    assert np.array_equal(got.view(np.uint32) if deq else got, want.reshape(n, oc).view(np.uint32) if deq else want.reshape(n, oc))
    # refused: weights packed for many pixels, a convolution that is not on the pooled pixel, a pool too large for one workgroup
    big = hip_ctx.prepack_conv2d(wt_, b, qp(zw, sw), expected_pixels=1 << 20)
    assert not hip_ctx.qglobal_avgpool_qconv2d_supported(big, a, h, w)
    with pytest.raises(rt.HipError):
        hip_ctx.qglobal_avgpool_qconv2d(xd, h, w, qp(zx, sx), big, yd, a)
    assert not hip_ctx.qglobal_avgpool_qconv2d_supported(wt, a, 512, 512)
    bad = conv_args(n, 2, 1, qp(zp, sp), qp(zy, sy), cl)
    with pytest.raises(rt.HipError):
        hip_ctx.qglobal_avgpool_qconv2d(xd, h, w, qp(zx, sx), wt, yd, bad)


@pytest.mark.parametrize("seed", range(16))
def test_random_pairs(hip_ctx, seed):
    """Seeded random shapes, options and padding: with and without the depthwise convolution in front."""
    rng = np.random.default_rng(7000 + seed)
    n, k1, n1, n2 = int(rng.integers(1, 4)), int(rng.integers(1, 20)) * 16, int(rng.integers(1, 24)) * 4, int(rng.integers(1, 40)) * 4
    h, w = int(rng.integers(3, 12)), int(rng.integers(3, 12))
    options = dict(residual=bool(rng.integers(0, 2)), lut_a=bool(rng.integers(0, 2)), lut_b=bool(rng.integers(0, 2)), relu_b=bool(rng.integers(0, 2)))
    dw = None
    if seed % 2:
        dw = (int(rng.integers(1, 3)), [P1, ((0, 1), (0, 1)), ((1, 0), (1, 0)), ((0, 0), (0, 0))][int(rng.integers(0, 4))])
    run_pair(hip_ctx, n, k1, n1, n2, h, w, seed=seed, dw=dw, **options)
