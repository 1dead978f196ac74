"""GPU parity of the pointwise pair (1x1 convolution [+ byte table] [+ residual] -> 1x1 convolution [+ byte table] as one
launch) through the C ABI: both results must be bit-identical to the CPU oracle running the operators one after the
other, and to nncase_hip_qconv2d called twice on the device."""
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


def run_pair(ctx, n, k1, n1, n2, h, w, seed, residual=False, lut_a=False, lut_b=False, relu_b=True):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, k1, h, w), dtype=np.uint8)
    wa = rng.integers(0, 256, (n1, k1, 1, 1), dtype=np.uint8)
    wb = rng.integers(0, 256, (n2, n1, 1, 1), dtype=np.uint8)
    ba = rng.integers(-3000, 3000, n1).astype(np.int32)
    bb = rng.integers(-3000, 3000, n2).astype(np.int32)
    zx, sx = 9, f32(0.0235)
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
    if residual:
        rd = ctx.alloc(res.size).upload(np.ascontiguousarray(res.transpose(0, 2, 3, 1)))
        keep.append(rd)
        fa_.residual_dev = rd.ptr
        fa_.residual_qp = qp(zr, sr)
        fa_.sum_qp = qp(zs, ss)
        fa_.sum_clamp_min, fa_.sum_clamp_max = FULL
    y1d = ctx.alloc(n * h * w * n1).fill(0xA5)
    y2d = ctx.alloc(n * h * w * n2).fill(0xA5)
    ctx.qpointwise_pair(xd, pair, y1d, y2d, fa_, sa_)
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
    ctx.qconv2d(xd, first, u1, fa_)
    ctx.qconv2d(u1, second, u2, sa_)
    ctx.sync()
    assert np.array_equal(u1.download((n, h, w, n1), np.uint8), y1d.download((n, h, w, n1), np.uint8))
    assert np.array_equal(u2.download((n, h, w, n2), np.uint8), y2d.download((n, h, w, n2), np.uint8))
    return pair, (xd, y1d, y2d, fa_, sa_, keep)


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
