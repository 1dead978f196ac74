"""GPU parity: u8/u8 conv2d (dense, grouped, depthwise) and matmul through the C ABI vs
the CPU oracle.  int32 accumulators, clamped fp32 values and requantised u8 bytes are all
compared bit-exactly: the fp32 epilogue is the same sequence of single IEEE operations on
both sides."""
import itertools
import zlib

import numpy as np
import pytest

from nncase_amd import kernels as K
from nncase_amd import quant
from nncase_amd import runtime as rt
from nncase_amd.runtime import qp
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32
FULL = (-rt.FLT_MAX, rt.FLT_MAX)


def same_padding(size, k, stride, dilation):
    """TF 'SAME' padding as nncase's importer computes it (Util.GetPaddings)."""
    out = -(-size // stride)
    eff = (k - 1) * dilation + 1
    total = max((out - 1) * stride + eff - size, 0)
    return (total // 2, total - total // 2)


def run_case(ctx, n, c, h, w, oc, kh, kw, stride, pad, dil, groups, seed, zx=7, zw=131, clamp=None, modes=("u8", "i32", "f32"),
             bias_of=None):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    wt = rng.integers(0, 256, (oc, c // groups, kh, kw), dtype=np.uint8)
    bias = rng.integers(-3000, 3000, oc).astype(np.int32) if bias_of is None else bias_of(wt).astype(np.int32)
    sx, sw = f32(0.0235), f32(0.0041)
    common = dict(stride=stride, padding=pad, dilation=dil, groups=groups)
    # the real-valued output decides the clamp and the output quantisation, so that the
    # requantiser sees values spread over (and beyond) the u8 range whatever the shape is
    real = O.qconv2d(x, wt, bias, zx, sx, zw, sw, out_mode=O.OUT_F32, **common)
    if clamp is not FULL:
        lo, hi = np.percentile(real, [10, 90]).astype(f32)
        clamp = (float(lo), float(hi)) if hi > lo else FULL
    span = float(real.max() - real.min()) or 1.0
    sy = f32(span * 0.7 / 255)
    zy_free = int(np.rint(-40 - real.min() / sy))  # puts the smallest value 40 codes below 0
    zy = int(np.clip(zy_free, 0, 255))
    if "i32" in modes:
        got = K.conv2d(x, wt, bias, stride, pad, dil, groups, FULL, qp(zx, sx), qp(zw, sw), None, np.int32, ctx=ctx)
        want = O.qconv2d(x, wt, bias, zx, sx, zw, sw, out_mode=O.OUT_I32, **common)
        assert got.shape == want.shape
        assert np.array_equal(got, want), f"int32 accumulators differ in {(got != want).sum()} of {got.size}"
    if "f32" in modes:
        got = K.conv2d(x, wt, bias, stride, pad, dil, groups, clamp, qp(zx, sx), qp(zw, sw), None, np.float32, ctx=ctx)
        want = O.qconv2d(x, wt, bias, zx, sx, zw, sw, fused_clamp=clamp, out_mode=O.OUT_F32, **common)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if "u8" in modes:
        for cl in (clamp, FULL):
            got = K.conv2d(x, wt, bias, stride, pad, dil, groups, cl, qp(zx, sx), qp(zw, sw), qp(zy, sy), np.uint8, ctx=ctx)
            want = O.qconv2d(x, wt, bias, zx, sx, zw, sw, zy, sy, fused_clamp=cl, out_mode=O.OUT_U8, **common)
            assert np.array_equal(got, want), f"u8 outputs differ in {(got != want).sum()} of {got.size}"
        if len(np.unique(real)) > 64 and zy == zy_free:
            assert len(np.unique(want)) > 8  # the case really exercises the requantiser


# ---- reference grids ----------------------------------------------------------------------------
# tests/importer/tflite_/basic/test_depthwise_conv2d.py: n {1,3}, C {1,16}, HxW {1x1, 33x65}, k {1,3,5},
# stride {[1,1],[1,3]}, padding {SAME, VALID}
DW_GRID = [(n, c, hw, k, s, p) for n, c, hw, k, s, p in itertools.product(
    (1, 3), (1, 16), ((1, 1), (33, 65)), (1, 3, 5), ((1, 1), (1, 3)), ("SAME", "VALID"))
    if not (p == "VALID" and hw == (1, 1) and k > 1)]


@pytest.mark.parametrize("n,c,hw,k,stride,padding", DW_GRID)
def test_depthwise_reference_grid(hip_ctx, n, c, hw, k, stride, padding):
    h, w = hw
    pad = (same_padding(h, k, stride[0], 1), same_padding(w, k, stride[1], 1)) if padding == "SAME" else ((0, 0), (0, 0))
    run_case(hip_ctx, n, c, h, w, c, k, k, stride, pad, (1, 1), c, seed=zlib.crc32(repr((n, c, hw, k, stride, padding)).encode()))


# tests/importer/tflite_/basic/test_conv2d.py: same plus stride [5,5] and dilation [2,2]
CONV_GRID = [(n, c, hw, k, s, d, p) for n, c, hw, k, s, d, p in itertools.product(
    (1, 3), (1, 16), ((1, 1), (33, 65)), (1, 3, 5), ((1, 1), (1, 3), (5, 5)), ((1, 1), (2, 2)), ("SAME", "VALID"))
    if not (p == "VALID" and hw == (1, 1) and k > 1) and not (d == (2, 2) and s != (1, 1))]


@pytest.mark.parametrize("n,c,hw,k,stride,dil,padding", CONV_GRID)
def test_conv2d_reference_grid(hip_ctx, n, c, hw, k, stride, dil, padding):
    h, w = hw
    pad = (same_padding(h, k, stride[0], dil[0]), same_padding(w, k, stride[1], dil[1])) if padding == "SAME" else ((0, 0), (0, 0))
    eff = (k - 1) * dil[0] + 1
    if padding == "VALID" and (eff > h or eff > w):
        pytest.skip("window larger than the image")
    run_case(hip_ctx, n, c, h, w, 8, k, k, stride, pad, dil, 1, seed=zlib.crc32(repr((n, c, hw, k, stride, dil, padding)).encode()),
             modes=("u8", "i32"))


# tests/kernels/test_conv2d.json + tests/importer/onnx_/basic/test_conv.py
@pytest.mark.parametrize("case", [
    (1, 4, 5, 5, 8, 3, (1, 1), ((1, 1), (1, 1)), (1, 1), 1),
    (1, 4, 16, 16, 8, 1, (2, 2), ((1, 1), (1, 1)), (1, 1), 1),
    (1, 4, 16, 16, 8, 3, (2, 2), ((1, 1), (1, 1)), (2, 2), 1),
    (1, 3, 16, 16, 5, 3, (2, 2), ((0, 1), (0, 1)), (2, 2), 1),   # SAME_UPPER-like
    (1, 3, 16, 16, 5, 3, (2, 2), ((1, 0), (1, 0)), (1, 1), 1),   # SAME_LOWER-like
    (2, 6, 9, 7, 4, 3, (5, 5), ((0, 2), (1, 0)), (1, 1), 2),     # grouped, asymmetric padding
    (1, 32, 10, 10, 48, 3, (1, 1), ((1, 1), (1, 1)), (1, 1), 4), # grouped with 8 channels per group
    (1, 16, 6, 6, 32, 3, (1, 1), ((1, 1), (1, 1)), (1, 1), 16),  # depthwise with multiplier 2
])
def test_conv2d_kernel_grid(hip_ctx, case):
    n, c, h, w, oc, k, stride, pad, dil, groups = case
    run_case(hip_ctx, n, c, h, w, oc, k, k, stride, pad, dil, groups, seed=sum(case[:6]))


# ---- shapes of the benchmark configurations ------------------------------------------------------
# every distinct (Cin, Cout) pointwise layer of MobileNetV2 on a small image, plus stem / depthwise / FC shapes
MBV2_PW = [(32, 16), (16, 96), (96, 24), (24, 144), (144, 24), (144, 32), (32, 192), (192, 32), (192, 64), (64, 384),
           (384, 64), (384, 96), (96, 576), (576, 96), (576, 160), (160, 960), (960, 160), (960, 320), (320, 1280),
           (64, 144), (144, 64)]   # the last two: the conv block of BASELINE config 2


@pytest.mark.parametrize("cin,cout", [(64, 144), (144, 64)])
def test_conv_block_pointwise_layers_at_batch_32(hip_ctx, cin, cout):
    # config 2's two pointwise layers at their full launch size: M = 32 * 56 * 56 = 100 352 pixels
    run_case(hip_ctx, 32, cin, 56, 56, cout, 1, 1, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, seed=cin + cout, modes=("u8",))


@pytest.mark.parametrize("cin,cout", MBV2_PW)
def test_mobilenet_pointwise_shapes(hip_ctx, cin, cout):
    # 2 x 13 x 11 = 286 pixels: not a multiple of the pixel tile, exercises the ragged last tile
    run_case(hip_ctx, 2, cin, 13, 11, cout, 1, 1, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, seed=cin * 7 + cout, modes=("u8", "i32"))


def test_mobilenet_stem_fc_and_depthwise_shapes(hip_ctx):
    run_case(hip_ctx, 2, 3, 32, 32, 32, 3, 3, (2, 2), ((0, 1), (0, 1)), (1, 1), 1, seed=1)           # stem 3x3 s2, 3 channels
    run_case(hip_ctx, 4, 1280, 1, 1, 1000, 1, 1, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, seed=2, clamp=FULL)  # FC as 1x1
    for c, s, hw in ((32, 1, 28), (96, 2, 28), (144, 1, 14), (192, 2, 14), (576, 1, 7), (960, 1, 7)):
        pad = ((1, 1), (1, 1)) if s == 1 else ((0, 1), (0, 1))
        run_case(hip_ctx, 2, c, hw, hw, c, 3, 3, (s, s), pad, (1, 1), c, seed=c + s)


# Large launches make the depthwise kernel walk strips of several output rows per thread (the strip
# length grows with the number of waves per SIMD); small shapes only ever take one-row strips.  On a
# 256-CU device these shapes give strips of 7, 8, 7, 2, 4, 2, 4 (MobileNetV2's depthwise layers at batch
# 64), then 5, and 8 / 4 / 2 with a ragged last strip, for stride 1 and 2.
DW_LARGE = [(64, 32, 112, 1), (64, 96, 112, 2), (64, 144, 56, 1), (64, 144, 56, 2), (64, 192, 28, 1), (64, 384, 14, 1),
            (64, 576, 14, 1), (64, 960, 7, 1), (48, 144, 75, 1), (32, 96, 75, 1), (64, 144, 30, 1), (32, 96, 37, 1),
            (64, 96, 75, 2), (96, 144, 37, 2)]


@pytest.mark.parametrize("n,c,hw,s", DW_LARGE)
def test_depthwise_multi_row_strips_at_full_batch(hip_ctx, n, c, hw, s):
    pad = ((1, 1), (1, 1)) if s == 1 else ((0, 1), (0, 1))
    run_case(hip_ctx, n, c, hw, hw, c, 3, 3, (s, s), pad, (1, 1), c, seed=n + c + hw + s, modes=("u8", "i32"))


# 3x3 depthwise layers over patches narrower and lower than a thread's strip, images smaller than one strip, stride 2
# with odd extents, every padding, and zero points at both ends; the second half of each case maps the accumulators
# one to one onto the output codes, so that any error in a sum is a different byte.
DW_SHAPES = [(2, 16, 37, 45, 1, ((1, 1), (1, 1))), (2, 48, 37, 45, 2, ((0, 1), (0, 1))), (3, 32, 7, 7, 1, ((1, 1), (1, 1))),
             (1, 16, 1, 1, 1, ((1, 1), (1, 1))), (2, 16, 14, 14, 2, ((1, 1), (1, 1))), (1, 64, 112, 112, 1, ((1, 1), (1, 1))),
             (1, 16, 113, 57, 2, ((1, 0), (0, 1))), (2, 32, 5, 70, 1, ((0, 0), (0, 0))), (1, 16, 40, 3, 1, ((2, 2), (2, 2)))]


@pytest.mark.parametrize("zx,zw", [(0, 0), (255, 255), (255, 0), (0, 255), (7, 131), (3, 128), (128, 1)])
@pytest.mark.parametrize("shape", DW_SHAPES)
def test_depthwise_3x3_exact_sums_and_zero_points(hip_ctx, shape, zx, zw):
    n, c, h, w, s, pad = shape
    run_case(hip_ctx, n, c, h, w, c, 3, 3, (s, s), pad, (1, 1), c, seed=c + h * 3 + w * 5 + s + zx + zw, zx=zx, zw=zw, modes=("u8",))
    # accumulators mapped one to one onto the codes (scales 1, zero point 128, values near the zero points):
    # any error in a sum shows up as a different byte
    rng = np.random.default_rng(zx * 256 + zw + h)
    x = np.clip(zx + rng.integers(-3, 4, (n, c, h, w)), 0, 255).astype(np.uint8)
    wt = np.clip(zw + rng.integers(-3, 4, (c, 1, 3, 3)), 0, 255).astype(np.uint8)
    bias = rng.integers(-20, 21, c).astype(np.int32)
    got = K.conv2d(x, wt, bias, (s, s), pad, (1, 1), c, FULL, qp(zx, 1.0), qp(zw, 1.0), qp(128, 1.0), np.uint8, ctx=hip_ctx)
    acc = O.qconv2d(x, wt, bias, zx, 1.0, zw, 1.0, stride=(s, s), padding=pad, groups=c, out_mode=O.OUT_I32)
    assert np.abs(acc).max() <= 127 and len(np.unique(acc)) > min(20, acc.size // 4)
    assert np.array_equal(got, (acc + 128).astype(np.uint8))


# Reductions of at least 512 over at least 65 536 pixels and 64 channels take the wide-tile kernels (a wave owns 64 pixels
# x 64 or 128 channels): windows, strides, dilation, groups, reductions that end inside a k-step, pixel and channel counts
# that end inside a tile, 255 channels (unaligned rows), and the matmul form with a long contiguous reduction.  Cases are
# (n, c, h, w, oc, k, stride, pad, dilation, groups); the oracle needs about 2.5 s per 10^9 multiply-adds.
WIDE = [
    (1, 64, 256, 257, 72, 3, (1, 1), ((1, 1), (1, 1)), (1, 1), 1),      # K = 576 (one tap per k-step), 72 channels, ragged pixel tile
    (1, 512, 256, 256, 64, 1, (1, 1), ((0, 0), (0, 0)), (1, 1), 1),     # 1x1 rows, K = 512, 64 channels (T = 4)
    (2, 528, 181, 182, 66, 1, (1, 1), ((0, 0), (0, 0)), (1, 1), 1),     # 1x1 rows, K = 528: the last k-step ends inside the row
    (1, 16, 256, 258, 64, 7, (1, 1), ((3, 3), (3, 3)), (1, 1), 1),      # 7x7 over 16 channels: K = 784, four taps per k-step
    (1, 48, 520, 516, 80, 4, (2, 2), ((1, 1), (1, 1)), (1, 1), 1),      # K = 768, 48 channels per tap, stride 2, even window
    (1, 128, 258, 258, 130, 3, (1, 1), ((2, 2), (2, 2)), (2, 2), 2),    # two groups of 64 -> 65 channels, dilation 2
]


@pytest.mark.parametrize("case", WIDE)
def test_wide_tile_kernels(hip_ctx, case):
    n, c, h, w, oc, k, stride, pad, dil, groups = case
    rng = np.random.default_rng(sum(case[:6]) + 11)
    x = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    wt = rng.integers(0, 256, (oc, c // groups, k, k), dtype=np.uint8)
    bias = rng.integers(-3000, 3000, oc).astype(np.int32)
    zx, sx, zw, sw = 7, f32(0.0235), 131, f32(0.0041)
    common = dict(stride=stride, padding=pad, dilation=dil, groups=groups)
    # one oracle convolution gives the accumulators; the other output forms are the oracle's epilogue applied to them
    acc = O.qconv2d(x, wt, bias, zx, sx, zw, sw, out_mode=O.OUT_I32, **common)
    assert acc.shape[0] * acc.shape[2] * acc.shape[3] >= 65536
    got = K.conv2d(x, wt, bias, stride, pad, dil, groups, FULL, qp(zx, sx), qp(zw, sw), None, np.int32, ctx=hip_ctx)
    assert np.array_equal(got, acc), f"int32 accumulators differ in {(got != acc).sum()} of {acc.size}"
    real = acc.astype(np.float64) * float(sx * sw)
    sy = f32((real.max() - real.min()) * 0.7 / 255)
    zy = int(np.clip(np.rint(-40 - real.min() / sy), 0, 255))
    lo, hi = (float(v) for v in np.percentile(real, [10, 90]).astype(f32))
    for clamp in ((lo, hi), FULL):
        got = K.conv2d(x, wt, bias, stride, pad, dil, groups, clamp, qp(zx, sx), qp(zw, sw), qp(zy, sy), np.uint8, ctx=hip_ctx)
        want = O.requant_u8(acc, sx, sw, sy, zy, clamp)
        assert np.array_equal(got, want), f"u8 outputs differ in {(got != want).sum()} of {want.size}"
    assert len(np.unique(want)) > 8
    got = K.conv2d(x, wt, bias, stride, pad, dil, groups, (lo, hi), qp(zx, sx), qp(zw, sw), None, np.float32, ctx=hip_ctx)
    want = np.clip((acc.astype(f32) * f32(sx * sw)), f32(lo), f32(hi))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("c,hw,oc,k", [(512, (256, 256), 136, 1), (64, (256, 256), 192, 3),
                                       (528, (255, 259), 200, 1),    # rows that end inside the ninth k-step, a ragged last pixel tile
                                       (256, (128, 512), 800, 1),    # four channel chunks per pixel tile, the last one an eighth full
                                       (48, (256, 257), 160, 3)])    # windows over 48 channels: seven k-steps, taps that straddle them
def test_wide_tile_kernels_with_256_channel_blocks(hip_ctx, c, hw, oc, k):
    """From 65 536 pixels on, layers of more than 128 channels run blocks of 256 pixels x 256 channels (two waves side by side
    share the block's activations).  One oracle convolution gives the accumulators; the u8 expectation is the oracle's
    requantisation of them."""
    rng = np.random.default_rng(c + oc)
    x = rng.integers(0, 256, (1, c, hw[0], hw[1]), dtype=np.uint8)
    w = rng.integers(0, 256, (oc, c, k, k), dtype=np.uint8)
    bias = rng.integers(-3000, 3000, oc).astype(np.int32)
    pad = ((k // 2, k // 2), (k // 2, k // 2))
    zx, sx, zw, sw = 7, f32(0.0235), 131, f32(0.0041)
    acc = O.qconv2d(x, w, bias, zx, sx, zw, sw, padding=pad, out_mode=O.OUT_I32)
    got = K.conv2d(x, w, bias, (1, 1), pad, (1, 1), 1, FULL, qp(zx, sx), qp(zw, sw), None, np.int32, ctx=hip_ctx)
    assert np.array_equal(got, acc)
    real = acc.astype(np.float64) * float(sx * sw)
    sy = f32((real.max() - real.min()) * 0.7 / 255)
    zy = 60
    lo, hi = (float(v) for v in np.percentile(real, [10, 90]).astype(f32))
    got = K.conv2d(x, w, bias, (1, 1), pad, (1, 1), 1, (lo, hi), qp(zx, sx), qp(zw, sw), qp(zy, sy), np.uint8, ctx=hip_ctx)
    want = O.requant_u8(acc, sx, sw, sy, zy, (lo, hi))
    assert np.array_equal(got, want) and len(np.unique(want)) > 8


def test_wide_tile_kernel_is_selected_and_zero_points_at_the_extremes(hip_ctx):
    w8 = np.zeros((128, 64, 3, 3), np.uint8)
    wts = hip_ctx.prepack_conv2d(w8, None, qp(131, 0.004), 1, expected_pixels=2 * 256 * 256)
    args = rt.Conv2dArgs(2, 256, 256, 1, 1, 1, 1, 1, 1, 1, 1, qp(7, 0.02), qp(0, 1.0), -rt.FLT_MAX, rt.FLT_MAX, rt.DT_I32)
    fn = rt.Function(hip_ctx)
    xb, yb = hip_ctx.alloc(2 * 256 * 256 * 64), hip_ctx.alloc(2 * 256 * 256 * 128 * 4)
    fn.add_qconv2d(xb, wts, yb, args)
    assert fn.op_kernel(0).startswith("qconv_wide<T=8")
    fn.destroy()
    # all-255 activations against all-0 and all-255 weights, zero points at both ends: the largest accumulators
    rng = np.random.default_rng(3)
    for xv, wv, zx, zw in ((255, 0, 0, 255), (255, 255, 0, 0), (0, 255, 255, 0), (255, 255, 255, 255)):
        x = np.full((1, 64, 256, 256), xv, np.uint8)
        w = np.full((64, 64, 3, 3), wv, np.uint8)
        got = K.conv2d(x, w, None, (1, 1), ((1, 1), (1, 1)), (1, 1), 1, FULL, qp(zx, 1.0), qp(zw, 1.0), None, np.int32, ctx=hip_ctx)
        want = O.qconv2d(x, w, np.zeros(64, np.int32), zx, 1.0, zw, 1.0, padding=((1, 1), (1, 1)), out_mode=O.OUT_I32)
        assert np.array_equal(got, want)


def test_large_reduction_stages_weights_through_lds_in_chunks(hip_ctx):
    # 3x3 over 256 channels: K = 2304 (36 k-steps) -> weights staged in several LDS chunks
    run_case(hip_ctx, 1, 256, 10, 10, 64, 3, 3, (1, 1), ((1, 1), (1, 1)), (1, 1), 1, seed=3, modes=("u8", "i32"))
    run_case(hip_ctx, 1, 128, 12, 12, 256, 3, 3, (2, 2), ((1, 1), (1, 1)), (1, 1), 1, seed=4, modes=("u8",))


def test_extreme_values_and_zero_points(hip_ctx):
    for zx, zw in ((0, 0), (255, 255), (0, 255), (128, 128), (1, 254)):
        for fill_x, fill_w in ((0, 0), (255, 255), (255, 0), (0, 255)):
            x = np.full((1, 64, 4, 4), fill_x, np.uint8)
            w = np.full((16, 64, 3, 3), fill_w, np.uint8)
            args = ((1, 1), ((1, 1), (1, 1)), (1, 1), 1, FULL, qp(zx, 1.0), qp(zw, 1.0), None, np.int32)
            got = K.conv2d(x, w, None, *args, ctx=hip_ctx)
            want = O.qconv2d(x, w, None, zx, 1.0, zw, 1.0, stride=(1, 1), padding=((1, 1), (1, 1)), out_mode=O.OUT_I32)
            assert np.array_equal(got, want)


@pytest.mark.parametrize("zw", [0, 1, 2, 127, 128, 129, 254, 255])
@pytest.mark.parametrize("cin,k,pad", [(16, 1, 0), (24, 1, 0), (32, 1, 0), (3, 3, 1), (8, 2, 0), (33, 1, 0), (48, 1, 0)])
def test_short_reductions_for_every_weight_zero_point(hip_ctx, zw, cin, k, pad):
    """Reductions of at most 32 carry the weight zero point's term inside the multiplication (except zw = 0, whose
    negative is no s8 value); just above 32 they do not.  Random and saturated operands, padding included."""
    run_case(hip_ctx, 2, cin, 9, 11, 40, k, k, (1, 1), ((pad, pad), (pad, pad)), (1, 1), 1, seed=zw * 7 + cin, zx=zw ^ 0x5a, zw=zw,
             modes=("u8", "i32"))
    for fill_x, fill_w in ((255, 255), (255, 0), (0, 255)):
        x = np.full((1, cin, 5, 5), fill_x, np.uint8)
        w = np.full((20, cin, k, k), fill_w, np.uint8)
        args = ((1, 1), ((pad, pad), (pad, pad)), (1, 1), 1, FULL, qp(3, 1.0), qp(zw, 1.0), None, np.int32)
        got = K.conv2d(x, w, None, *args, ctx=hip_ctx)
        want = O.qconv2d(x, w, None, 3, 1.0, zw, 1.0, stride=(1, 1), padding=((pad, pad), (pad, pad)), out_mode=O.OUT_I32)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("cin,groups", [(8, 1), (24, 1), (40, 1), (56, 1), (72, 1), (136, 1), (200, 1), (600, 1), (16, 2), (48, 2), (120, 3)])
@pytest.mark.parametrize("n,h,w", [(1, 1, 1), (1, 1, 2), (1, 1, 3), (2, 7, 9), (3, 16, 16)])
def test_pointwise_rows_with_half_used_last_load(hip_ctx, cin, groups, n, h, w):
    """1x1 layers whose channels per group are a multiple of 8 but not of 16 read rows in 16-byte pieces of which the
    last is half used; the tensor's last pixel (and a tensor smaller than one piece) must not be read past its end.
    Short reductions carry the weight zero point's term inside the multiplication here as well."""
    run_case(hip_ctx, n, cin, h, w, 24 * groups, 1, 1, (1, 1), ((0, 0), (0, 0)), (1, 1), groups,
             seed=cin * 13 + n * 5 + h + w, zx=(cin * 3 + h) & 255, zw=(cin * 7 + w) & 255, modes=("u8", "i32"))


@pytest.mark.parametrize("edge", [0, 1, -1, 2000, 10 ** 9])
@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("sign", [1, -1])
@pytest.mark.parametrize("zx,zw", [(0, 0), (255, 255), (255, 0), (7, 131)])
def test_depthwise_3x3_sums_at_the_edge_of_exact_fp32(hip_ctx, edge, stride, sign, zx, zw):
    """The stride-1 3x3 kernel keeps its sums in fp32 while |bias - zx * sum(w - zw)| + 9 * 255 * 255 cannot exceed
    2^24, and in int32 beyond: biases that put every channel exactly at that limit (edge 0), just below and above it,
    and far above it (where the conversion of the int32 sum to fp32 rounds, as the reference's does)."""
    limit = (1 << 24) - 9 * 255 * 255

    def bias_of(wt):
        wsum = (wt.astype(np.int64) - zw).reshape(wt.shape[0], -1).sum(axis=1)
        return sign * (limit - 255 * np.abs(wsum) + edge)

    run_case(hip_ctx, 2, 24, 13, 10, 24, 3, 3, (stride, stride), ((1, 1), (1, 1)), (1, 1), 24, seed=edge % 1000 + zx + zw + stride + sign,
             zx=zx, zw=zw, modes=("u8", "i32"), bias_of=bias_of)


def _random_conv_cases(count, seed):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        k = int(rng.choice([1, 1, 1, 3, 2, 5]))
        cin = int(rng.choice([1, 3, 4, 8, 12, 16, 24, 32, 40, 48, 64, 80, 96, 144, 160, 320, 384, 576, 960]))
        if k > 1 and cin > 96:
            continue
        cout = int(rng.choice([4, 8, 16, 20, 24, 32, 40, 64, 96, 100, 144, 160, 255, 320]))
        n = int(rng.integers(1, 4))
        h, w = int(rng.integers(k, 15)), int(rng.integers(k, 15))
        stride = int(rng.choice([1, 1, 2]))
        pad = int(rng.integers(0, (k + 1) // 2 + 1)) if k > 1 else 0
        cases.append((n, cin, h, w, cout, k, stride, pad, int(rng.integers(0, 256)), int(rng.integers(0, 256))))
    return cases


@pytest.mark.parametrize("case", _random_conv_cases(48, 20251))
def test_random_dense_shapes_and_zero_points(hip_ctx, case):
    """Shapes drawn at random across the loaders (row, 16/8/4-byte vectors, bytes), the single-tile and persistent
    forms, short and long reductions, and every pairing of zero points."""
    n, cin, h, w, cout, k, stride, pad, zx, zw = case
    run_case(hip_ctx, n, cin, h, w, cout, k, k, (stride, stride), ((pad, pad), (pad, pad)), (1, 1), 1,
             seed=n + cin * 3 + cout * 5 + h * 7 + w * 11, zx=zx, zw=zw, modes=("u8", "i32"))


def test_config2_conv_block(hip_ctx):
    """BASELINE config 2 at batch 1: 1x1 64->144, 3x3 depthwise, 1x1 144->64 on 56x56, ReLU6, per-tensor PTQ."""
    rng = np.random.default_rng(1)
    xf = rng.random((1, 64, 56, 56), dtype=f32)
    zx, sx = quant.get_quant_param((xf.min(), xf.max()))
    x = O.quantize(xf, sx, zx)

    def kaiming(shape):
        fan_in = shape[1] * shape[2] * shape[3]
        return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(f32)

    stages = [(kaiming((144, 64, 1, 1)), 1, ((0, 0), (0, 0))), (kaiming((144, 1, 3, 3)), 144, ((1, 1), (1, 1))),
              (kaiming((64, 144, 1, 1)), 1, ((0, 0), (0, 0)))]
    cur, cur_qp = x, (zx, sx)
    for wf, groups, pad in stages:
        wq, zw, sw = quant.quantize_weights(wf)
        bq = np.rint(rng.standard_normal(wf.shape[0]) * 0.01 / (cur_qp[1] * sw)).astype(np.int32)
        yq = quant.get_quant_param((0.0, 6.0))
        want = O.qconv2d(cur, wq, bq, cur_qp[0], cur_qp[1], zw, sw, yq[0], yq[1], padding=pad, groups=groups, fused_clamp=(0.0, 6.0))
        got = K.conv2d(cur, wq, bq, (1, 1), pad, (1, 1), groups, (0.0, 6.0), qp(*cur_qp), qp(zw, sw), qp(*yq), np.uint8, ctx=hip_ctx)
        assert np.array_equal(got, want)
        chain = O.qconv2d_float_chain(cur, wq, bq, cur_qp[0], cur_qp[1], zw, sw, yq[0], yq[1], padding=pad, groups=groups,
                                      fused_clamp=(0.0, 6.0))
        d = np.abs(got.astype(np.int32) - chain.astype(np.int32))
        assert d.max() <= 1 and O.cosine(got, chain) > 0.999  # the reference's own bar is cosine >= 0.98 with PTQ
        cur, cur_qp = got, yq


# ---- matmul --------------------------------------------------------------------------------------
def test_config1_matmul(hip_ctx):
    """BASELINE config 1: A[512,1024] u8 (0.02, 128) x B[1024,1024] u8 per-tensor asymmetric -> fp32."""
    rng = np.random.default_rng(0)
    a = rng.integers(0, 256, (512, 1024), dtype=np.uint8)
    bq, zb, sb = quant.quantize_weights((rng.standard_normal((1024, 1024)) * 0.05).astype(f32))
    acc = K.mat_mul(a, bq, qp(128, 0.02), qp(zb, sb), None, np.int32, ctx=hip_ctx)
    assert np.array_equal(acc, O.qmatmul(a, bq, None, 128, 0.02, zb, sb, out_mode=O.OUT_I32))
    out = K.mat_mul(a, bq, qp(128, 0.02), qp(zb, sb), None, np.float32, ctx=hip_ctx)
    want = O.qmatmul(a, bq, None, 128, 0.02, zb, sb, out_mode=O.OUT_F32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    # against what the CPU target computes (float matmul of dequantised operands): north-star tolerance 1e-3 relative
    ref = O.matmul_f32(O.dequantize(a[:64], 0.02, 128), O.dequantize(bq, sb, zb))
    np.testing.assert_allclose(out[:64], ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max())


@pytest.mark.parametrize("m,k,n", [(1, 6, 3), (6, 6, 1), (7, 70, 13), (130, 257, 100), (33, 64, 1000), (3, 1, 5)])
def test_matmul_shapes(hip_ctx, m, k, n):
    rng = np.random.default_rng(m * 100 + n)
    a = rng.integers(0, 256, (m, k), dtype=np.uint8)
    b = rng.integers(0, 256, (k, n), dtype=np.uint8)
    bias = rng.integers(-500, 500, n).astype(np.int32)
    got = K.mat_mul(a, b, qp(9, 0.02), qp(200, 0.003), None, np.int32, bias=bias, ctx=hip_ctx)
    assert np.array_equal(got, O.qmatmul(a, b, bias, 9, 0.02, 200, 0.003))
    gotq = K.mat_mul(a, b, qp(9, 0.02), qp(200, 0.003), qp(128, 0.5), np.uint8, bias=bias, ctx=hip_ctx)
    assert np.array_equal(gotq, O.qmatmul(a, b, bias, 9, 0.02, 200, 0.003, 128, 0.5, out_mode=O.OUT_U8))


def test_matmul_batched_lhs_is_flattened(hip_ctx):
    # the reference broadcasts rank<=4 batches of lhs against a constant rhs: rows are independent
    rng = np.random.default_rng(77)
    a = rng.integers(0, 256, (2, 3, 6, 6), dtype=np.uint8)
    b = rng.integers(0, 256, (6, 3), dtype=np.uint8)
    got = K.mat_mul(a, b, qp(1, 1.0), qp(2, 1.0), None, np.int32, ctx=hip_ctx)
    want = (a.astype(np.int64) - 1) @ (b.astype(np.int64) - 2)
    assert got.shape == (2, 3, 6, 3) and np.array_equal(got, want)


# reference/matmul.cpp:56-87: rank-1 operands become a row / a column, both operands are extended to four
# dimensions and the two batch dimensions broadcast where one side has extent 1 (shapes from
# tests/kernels/test_matmul.cpp's grid and ones where the rhs carries the batch)
@pytest.mark.parametrize("ashape,bshape", [
    ((3, 5), (5,)), ((5,), (5, 4)), ((5,), (5,)),
    ((2, 3, 4, 5), (2, 3, 5, 6)), ((2, 1, 4, 5), (1, 3, 5, 6)), ((4, 5), (2, 3, 5, 6)), ((3, 4, 5), (1, 1, 5, 6)),
    ((2, 3, 7, 70), (3, 70, 20)), ((1, 3, 16, 64), (2, 1, 64, 24)),
])
def test_matmul_two_sided_batches_and_vectors(hip_ctx, ashape, bshape):
    rng = np.random.default_rng(sum(ashape) * 31 + sum(bshape))
    a = rng.integers(0, 256, ashape, dtype=np.uint8)
    b = rng.integers(0, 256, bshape, dtype=np.uint8)
    za, zb = 17, 201
    want = np.matmul(a.astype(np.int64) - za, b.astype(np.int64) - zb)          # numpy broadcasts the same way
    got = K.mat_mul(a, b, qp(za, 0.02), qp(zb, 0.003), None, np.int32, ctx=hip_ctx)
    assert got.shape == want.shape and np.array_equal(got, want)
    gotf = K.mat_mul(a, b, qp(za, 0.02), qp(zb, 0.003), None, np.float32, ctx=hip_ctx)
    assert np.array_equal(gotf, want.astype(f32) * (f32(0.02) * f32(0.003)))
    # and against the float kernel of the reference restated in the oracle (its own batching), to 1e-3 relative
    ref = O.matmul_f32(O.dequantize(a, 0.02, za), O.dequantize(b, 0.003, zb))
    assert ref.shape == want.shape
    assert np.abs(gotf - ref).max() <= 1e-3 * max(1.0, np.abs(ref).max())
    with pytest.raises(rt.HipError) as e:
        K.mat_mul(np.zeros((2, 3, 4, 5), np.uint8), np.zeros((3, 2, 5, 6), np.uint8), qp(0, 1.0), qp(0, 1.0), None, np.int32, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH


@pytest.mark.parametrize("cin,cout,k,stride_c,offset,with_res", [
    (16, 24, 1, 64, 8, False), (32, 64, 3, 200, 136, False), (16, 20, 1, 33, 13, False),     # unaligned stride and offset
    (64, 32, 1, 96, 64, True), (128, 64, 3, 128, 64, False)])
def test_conv_output_inside_a_wider_tensor(hip_ctx, cin, cout, k, stride_c, offset, with_res):
    """out_channel_stride / out_channel_offset: the conv writes channels [offset, offset + cout) of every pixel of a
    tensor with stride_c channels (its slice of a concat) and leaves the other channels alone; a fused residual is
    still read as a dense tensor."""
    rng = np.random.default_rng(cin + cout + stride_c)
    n, h, w = 2, 19, 23
    x = rng.integers(0, 256, (n, cin, h, w), dtype=np.uint8)
    wt = rng.integers(0, 256, (cout, cin, k, k), dtype=np.uint8)
    bias = rng.integers(-2000, 2000, cout).astype(np.int32)
    pad = ((k // 2, k // 2), (k // 2, k // 2))
    zx, sx, zw, sw, zy, sy = 7, 0.0235, 131, 0.0041, 101, 0.21
    res = rng.integers(0, 256, (n, cout, h, w), dtype=np.uint8) if with_res else None
    want = O.qconv2d(x, wt, bias, zx, sx, zw, sw, zy, sy, padding=pad, out_mode=O.OUT_U8)
    if with_res:
        want = O.qadd(want, res, zy, sy, 33, 0.11, 90, 0.3)
    store = rng.integers(0, 256, (n, h, w, stride_c), dtype=np.uint8)
    wts = hip_ctx.prepack_conv2d(wt, bias, qp(zw, sw), 1, expected_pixels=n * h * w)
    xb = hip_ctx.to_device(np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    yb = hip_ctx.to_device(store)
    args = rt.Conv2dArgs(n, h, w, 1, 1, 1, 1, pad[0][0], pad[0][1], pad[1][0], pad[1][1], qp(zx, sx), qp(zy, sy), -rt.FLT_MAX, rt.FLT_MAX, rt.DT_U8)
    args.out_channel_stride, args.out_channel_offset = stride_c, offset
    if with_res:
        rb = hip_ctx.to_device(np.ascontiguousarray(res.transpose(0, 2, 3, 1)))
        args.residual_dev, args.residual_qp, args.sum_qp = rb.ptr, qp(33, 0.11), qp(90, 0.3)
        args.sum_clamp_min, args.sum_clamp_max = -rt.FLT_MAX, rt.FLT_MAX
    hip_ctx.qconv2d(xb, wts, yb, args)
    got = yb.download(store.shape, np.uint8)
    assert np.array_equal(got[..., offset:offset + cout], want.transpose(0, 2, 3, 1))
    keep = np.ones(stride_c, bool)
    keep[offset:offset + cout] = False
    assert np.array_equal(got[..., keep], store[..., keep])
    for bad_stride, bad_off in ((cout - 1, 0), (stride_c, stride_c - cout + 1), (0, 4)):
        args.out_channel_stride, args.out_channel_offset = bad_stride, bad_off
        with pytest.raises(rt.HipError) as e:
            hip_ctx.qconv2d(xb, wts, yb, args)
        assert e.value.code == -22


@pytest.mark.parametrize("cin,cout,k,hw,with_lut,with_res", [
    (128, 255, 1, 20, False, False),      # a detection head: 255 channels, rows of 1020 bytes
    (64, 64, 3, 13, True, False), (32, 48, 1, 9, True, True), (16, 24, 1, 7, False, True), (320, 1000, 1, 1, False, False),
    (512, 255, 1, 20, False, False)])
def test_conv_stores_the_dequantised_output(hip_ctx, cin, cout, k, hw, with_lut, with_res):
    """dequantize_output: conv (+ table, + residual add) with float32 output == the same conv with u8 output followed by
    Dequantize (oracle: conv, table, add, dequantize), bit for bit."""
    rng = np.random.default_rng(cin * 3 + cout + k)
    n = 2
    x = rng.integers(0, 256, (n, cin, hw, hw), dtype=np.uint8)
    wt = rng.integers(0, 256, (cout, cin, k, k), dtype=np.uint8)
    bias = rng.integers(-2000, 2000, cout).astype(np.int32)
    pad = ((k // 2, k // 2), (k // 2, k // 2))
    zx, sx, zw, sw = 7, 0.0235, 131, 0.0041
    real = O.qconv2d(x, wt, bias, zx, sx, zw, sw, padding=pad, out_mode=O.OUT_F32)
    zy, sy = quant.get_quant_param((float(real.min()), float(real.max())))
    zy, sy = int(zy), float(sy)
    want = O.qconv2d(x, wt, bias, zx, sx, zw, sw, zy, sy, padding=pad, out_mode=O.OUT_U8)
    last = (zy, sy)
    wts = hip_ctx.prepack_conv2d(wt, bias, qp(zw, sw), 1, expected_pixels=n * hw * hw)
    if with_lut:
        lut = rng.integers(0, 256, 256, dtype=np.uint8)
        last = (77, 0.043)
        wts.set_post_lut(lut, qp(*last))
        want = lut[want]
    args = rt.Conv2dArgs(n, hw, hw, 1, 1, 1, 1, pad[0][0], pad[0][1], pad[1][0], pad[1][1], qp(zx, sx), qp(zy, sy), -rt.FLT_MAX, rt.FLT_MAX, rt.DT_F32)
    args.dequantize_output = 1
    if with_res:
        res = rng.integers(0, 256, (n, cout, hw, hw), dtype=np.uint8)
        want = O.qadd(want, res, last[0], last[1], 33, 0.11, 90, 0.3)
        last = (90, 0.3)
        rb = hip_ctx.to_device(np.ascontiguousarray(res.transpose(0, 2, 3, 1)))
        args.residual_dev, args.residual_qp, args.sum_qp = rb.ptr, qp(33, 0.11), qp(90, 0.3)
        args.sum_clamp_min, args.sum_clamp_max = -rt.FLT_MAX, rt.FLT_MAX
    want_f = O.dequantize(want, last[1], last[0])
    xb = hip_ctx.to_device(np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    yb = hip_ctx.alloc(want_f.size * 4)
    hip_ctx.qconv2d(xb, wts, yb, args)
    got = yb.download((n, hw, hw, cout), np.float32)
    assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(want_f.transpose(0, 2, 3, 1)).view(np.uint32))
    args.out_dtype = rt.DT_U8                      # the flag needs a float32 output ...
    with pytest.raises(rt.HipError) as e:
        hip_ctx.qconv2d(xb, wts, yb, args)
    assert e.value.code == -rt.ERR_DATATYPE_MISMATCH
    args.out_dtype, args.out_channel_stride = rt.DT_F32, cout + 4     # ... and a dense one
    with pytest.raises(rt.HipError) as e:
        hip_ctx.qconv2d(xb, wts, yb, args)
    assert e.value.code == -22


def test_depthwise_conv_refuses_an_output_inside_a_wider_tensor(hip_ctx):
    wts = hip_ctx.prepack_conv2d(np.zeros((32, 1, 3, 3), np.uint8), None, qp(128, 0.01), 32)
    xb, yb = hip_ctx.alloc(8 * 8 * 32), hip_ctx.alloc(8 * 8 * 64)
    args = rt.Conv2dArgs(1, 8, 8, 1, 1, 1, 1, 1, 1, 1, 1, qp(0, 1.0), qp(0, 1.0), -rt.FLT_MAX, rt.FLT_MAX, rt.DT_U8)
    args.out_channel_stride = 64
    with pytest.raises(rt.HipError) as e:
        hip_ctx.qconv2d(xb, wts, yb, args)
    assert e.value.code == -22


def test_linearity_at_full_size(hip_ctx):
    """Size-independent check at a BASELINE-sized layer (56x56x24 -> 144, batch 32): with zero
    points 0, acc(x1 + x2) == acc(x1) + acc(x2), and acc(x, w = 1) is the per-pixel channel sum."""
    rng = np.random.default_rng(5)
    n, c, hw, oc = 32, 24, 56, 144
    x1 = rng.integers(0, 128, (n, c, hw, hw), dtype=np.uint8)
    x2 = rng.integers(0, 128, (n, c, hw, hw), dtype=np.uint8)
    w = rng.integers(0, 256, (oc, c, 1, 1), dtype=np.uint8)
    args = ((1, 1), ((0, 0), (0, 0)), (1, 1), 1, FULL, qp(0, 1.0), qp(0, 1.0), None, np.int32)
    a1 = K.conv2d(x1, w, None, *args, ctx=hip_ctx)
    a2 = K.conv2d(x2, w, None, *args, ctx=hip_ctx)
    a12 = K.conv2d(x1 + x2, w, None, *args, ctx=hip_ctx)
    assert np.array_equal(a12, a1 + a2)
    ones = K.conv2d(x1, np.ones_like(w), None, *args, ctx=hip_ctx)
    assert np.array_equal(ones[:, 0], x1.astype(np.int32).sum(1)) and np.array_equal(ones[:, 0], ones[:, oc - 1])


def test_error_paths(hip_ctx):
    x = np.zeros((1, 8, 4, 4), np.uint8)
    w = np.zeros((4, 8, 3, 3), np.uint8)
    with pytest.raises(rt.HipError) as e:   # window larger than the padded input
        K.conv2d(x[:, :, :2, :2], w, None, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, FULL, qp(0, 1), qp(0, 1), None, np.int32, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    with pytest.raises(rt.HipError) as e:   # channel mismatch
        K.conv2d(x, np.zeros((4, 6, 3, 3), np.uint8), None, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, FULL, qp(0, 1), qp(0, 1), None, np.int32, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    with pytest.raises(rt.HipError) as e:   # groups do not divide channels
        hip_ctx.prepack_conv2d(np.zeros((4, 3, 1, 1), np.uint8), None, qp(0, 1), groups=3)
    assert e.value.code == -rt.ERR_SHAPE_MISMATCH
    with pytest.raises(rt.HipError) as e:   # output scale must be positive for u8 output
        K.conv2d(x, w, None, (1, 1), ((1, 1), (1, 1)), (1, 1), 1, FULL, qp(0, 1), qp(0, 1), qp(0, 0.0), np.uint8, ctx=hip_ctx)
    assert e.value.code == -22
    with pytest.raises(rt.HipError) as e:   # zero point outside u8
        K.conv2d(x, w, None, (1, 1), ((1, 1), (1, 1)), (1, 1), 1, FULL, qp(300, 1), qp(0, 1), None, np.int32, ctx=hip_ctx)
    assert e.value.code == -22


def test_requantisation_is_exact_for_many_scales(hip_ctx):
    """The device replaces y / sy by a multiply and two FMAs with a pre-rounded reciprocal; the
    bytes must still equal the oracle's true fp32 division for every accumulator, including
    scales that are powers of two (exact .5 ties), have an all-ones mantissa, or are tiny/huge."""
    rng = np.random.default_rng(2024)
    x = rng.integers(0, 256, (1, 64, 64, 64), dtype=np.uint8)      # 4096 pixels
    w = rng.integers(0, 256, (64, 64, 1, 1), dtype=np.uint8)       # 262144 accumulators per case
    bias = rng.integers(-20000, 20000, 64).astype(np.int32)
    acc = O.qconv2d(x, w, bias, 3, 1.0, 128, 1.0, out_mode=O.OUT_I32)
    span = float(acc.max() - acc.min())
    special = [np.float32(2.0 ** -7), np.float32(0.5), np.nextafter(np.float32(1.0), np.float32(0)),
               np.nextafter(np.float32(0.03125), np.float32(0)), np.float32(1.0) + np.float32(2.0 ** -23)]
    for i in range(48):
        sx = f32(10.0 ** rng.uniform(-3, 0))
        sw = f32(10.0 ** rng.uniform(-4, -1))
        m = float(sx) * float(sw)
        sy = special[i] if i < len(special) else f32(span * m / 255 * 10.0 ** rng.uniform(-1.0, 0.5))
        if i < len(special):  # choose sx * sw so that the u8 range is covered for the special scales too
            sx, sw = f32(float(sy) * 255 / span), f32(1.0)
        zy = int(rng.integers(0, 256))
        clamp = FULL if i % 3 else (0.0, float(sy) * 200)
        got = K.conv2d(x, w, bias, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, clamp, qp(3, sx), qp(128, sw), qp(zy, sy), np.uint8, ctx=hip_ctx)
        want = O.qconv2d(x, w, bias, 3, sx, 128, sw, zy, sy, fused_clamp=clamp)
        assert np.array_equal(got, want), f"case {i}: sx={sx} sw={sw} sy={sy} zy={zy}: {(got != want).sum()} bytes differ"
    # extreme but supported scales, and the documented rejection beyond them
    for sy in (f32(2.0 ** -60), f32(2.0 ** 60)):
        got = K.conv2d(x, w, bias, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, FULL, qp(3, 1.0), qp(128, float(sy) / 100), qp(7, sy), np.uint8, ctx=hip_ctx)
        want = O.qconv2d(x, w, bias, 3, 1.0, 128, float(sy) / 100, 7, sy)
        assert np.array_equal(got, want)
    with pytest.raises(rt.HipError) as e:
        K.conv2d(x, w, bias, (1, 1), ((0, 0), (0, 0)), (1, 1), 1, FULL, qp(3, 1.0), qp(128, 1.0), qp(7, 2.0 ** -70), np.uint8, ctx=hip_ctx)
    assert e.value.code == -34  # ERANGE


@pytest.mark.parametrize("cin,cout,hw,k", [(144, 24, 13, 1), (960, 160, 7, 1), (32, 40, 9, 3), (24, 30, 5, 1)])
def test_fused_residual_equals_conv_then_add(hip_ctx, cin, cout, hw, k):
    """conv with a fused residual == the same conv followed by the separate add, bit for bit (oracle: conv then qadd)."""
    rng = np.random.default_rng(cin + cout)
    x = rng.integers(0, 256, (2, cin, hw, hw), dtype=np.uint8)
    w = rng.integers(0, 256, (cout, cin, k, k), dtype=np.uint8)
    bias = rng.integers(-3000, 3000, cout).astype(np.int32)
    res = rng.integers(0, 256, (2, cout, hw, hw), dtype=np.uint8)
    pad = ((k // 2, k // 2), (k // 2, k // 2))
    sx, sw = f32(0.0235), f32(0.0041)
    real = O.qconv2d(x, w, bias, 7, sx, 131, sw, padding=pad, out_mode=O.OUT_F32)
    sy = f32((real.max() - real.min()) / 255)
    zy = int(np.clip(np.rint(-real.min() / sy), 0, 255))
    conv = O.qconv2d(x, w, bias, 7, sx, 131, sw, zy, sy, padding=pad)
    want = O.qadd(conv, res, zy, sy, 99, 0.031, 101, float(sy) * 1.3)
    got = K.conv2d(x, w, bias, (1, 1), pad, (1, 1), 1, FULL, qp(7, sx), qp(131, sw), qp(zy, sy), np.uint8, ctx=hip_ctx,
                   residual=res, residual_qp=qp(99, 0.031), sum_qp=qp(101, float(sy) * 1.3))
    assert np.array_equal(got, want)
    assert len(np.unique(want)) > 16


@pytest.mark.parametrize("cin,cout,hw,k,with_residual", [(64, 32, 12, 1, False), (32, 32, 9, 3, True), (128, 255, 5, 1, False),
                                                         (4, 32, 20, 6, False), (256, 128, 7, 3, True),
                                                         (64, 72, 182, 3, True), (512, 255, 182, 1, True)])   # the last two: wide-tile kernels
def test_fused_table_equals_conv_then_table(hip_ctx, cin, cout, hw, k, with_residual):
    """conv with a fused swish table (and a residual add behind it) == conv, then the table, then the add."""
    rng = np.random.default_rng(cin + cout + k)
    x = rng.integers(0, 256, (2, cin, hw, hw), dtype=np.uint8)
    w = rng.integers(0, 256, (cout, cin, k, k), dtype=np.uint8)
    bias = rng.integers(-2000, 2000, cout).astype(np.int32)
    pad = ((k // 2, k // 2), (k // 2, k // 2)) if k != 6 else ((2, 2), (2, 2))
    stride = (2, 2) if k == 6 else (1, 1)
    zx, sx, zw, sw = 9, f32(0.031), 127, f32(0.004)
    real = O.qconv2d(x, w, bias, zx, sx, zw, sw, stride=stride, padding=pad, out_mode=O.OUT_F32)
    sy = f32((real.max() - real.min()) / 255)
    zy = int(np.clip(np.rint(-real.min() / sy), 0, 255))
    y = O.qconv2d(x, w, bias, zx, sx, zw, sw, zy, sy, stride=stride, padding=pad, out_mode=O.OUT_U8)
    lz, ls = 18, f32(sy * 0.9)
    lut = O.unary_lut(O.LUT_SWISH, zy, sy, lz, ls)
    want = lut[y]
    kw = {}
    if with_residual:
        r = rng.integers(0, 256, y.shape, dtype=np.uint8)
        rq, sq = (77, f32(0.02)), (40, f32(ls * 1.3))
        want = O.qadd(want, r, lz, ls, rq[0], rq[1], sq[0], sq[1])
        kw = dict(residual=r, residual_qp=qp(*rq), sum_qp=qp(*sq))
    got = K.conv2d(x, w, bias, stride, pad, (1, 1), 1, FULL, qp(zx, sx), qp(zw, sw), qp(zy, sy), np.uint8, ctx=hip_ctx,
                   post_lut=rt.make_unary_lut(rt.LUT_SWISH, qp(zy, sy), qp(lz, ls)), post_lut_qp=qp(lz, ls), **kw)
    assert np.array_equal(got, want), f"{(got != want).sum()} of {want.size} bytes differ"
