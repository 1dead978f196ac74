"""GPU parity of the fused inverted-residual block (1x1 expansion -> 3x3 depthwise -> 1x1 projection,
optionally + input) through the C ABI against the CPU oracle running the three convolutions and the add
one after the other: the u8 output must be bit-identical (every stage requantises to u8 exactly as the
stand-alone operators do; the two mid tensors only ever exist in LDS)."""
import numpy as np
import pytest

from nncase_amd import runtime as rt
from nncase_amd.runtime import qp
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32
FULL = (-rt.FLT_MAX, rt.FLT_MAX)


def pick_quant(real, relu6_like=True):
    """Clamp and output quantisation that spread the stage's real values over (and past) the u8 range."""
    lo, hi = np.percentile(real, [10, 90]).astype(f32)
    clamp = (float(lo), float(hi)) if (relu6_like and hi > lo) else FULL
    span = float(real.max() - real.min()) or 1.0
    sy = f32(span * 0.7 / 255)
    zy = int(np.clip(np.rint(-40 - real.min() / sy), 0, 255))
    return clamp, zy, sy


def oracle_block(x, we, be, wd, bd, wp, bp, zx, sx, zws, sws, stride, pad, add):
    mid = we.shape[0]
    real = O.qconv2d(x, we, be, zx, sx, zws[0], sws[0], out_mode=O.OUT_F32)
    c1, z1, s1 = pick_quant(real)
    e = O.qconv2d(x, we, be, zx, sx, zws[0], sws[0], z1, s1, fused_clamp=c1, out_mode=O.OUT_U8)
    dwk = dict(stride=(stride, stride), padding=pad, dilation=(1, 1), groups=mid)
    real = O.qconv2d(e, wd, bd, z1, s1, zws[1], sws[1], out_mode=O.OUT_F32, **dwk)
    c2, z2, s2 = pick_quant(real)
    d = O.qconv2d(e, wd, bd, z1, s1, zws[1], sws[1], z2, s2, fused_clamp=c2, out_mode=O.OUT_U8, **dwk)
    real = O.qconv2d(d, wp, bp, z2, s2, zws[2], sws[2], out_mode=O.OUT_F32)
    c3, z3, s3 = pick_quant(real, relu6_like=False)
    y = O.qconv2d(d, wp, bp, z2, s2, zws[2], sws[2], z3, s3, fused_clamp=c3, out_mode=O.OUT_U8)
    quant = dict(expand=(c1, z1, s1), dw=(c2, z2, s2), project=(c3, z3, s3), sum=None)
    if add:
        fa = (y.astype(f32) - f32(z3)) * s3 + (x.astype(f32) - f32(zx)) * sx
        _, z4, s4 = pick_quant(fa)
        y = O.qadd(y, x, z3, s3, zx, sx, z4, s4)
        quant["sum"] = (z4, s4)
    return y, quant, (e, d)


def run_block(ctx, n, cin, mid, cout, h, w, stride, pad, add, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, cin, h, w), dtype=np.uint8)
    we = rng.integers(0, 256, (mid, cin, 1, 1), dtype=np.uint8)
    wd = rng.integers(0, 256, (mid, 1, 3, 3), dtype=np.uint8)
    wp = rng.integers(0, 256, (cout, mid, 1, 1), dtype=np.uint8)
    be = rng.integers(-3000, 3000, mid).astype(np.int32)
    bd = rng.integers(-3000, 3000, mid).astype(np.int32)
    bp = rng.integers(-3000, 3000, cout).astype(np.int32)
    zx, sx = 7, f32(0.0235)
    zws, sws = (131, 120, 140), (f32(0.0041), f32(0.0123), f32(0.0037))
    want, quant, _ = oracle_block(x, we, be, wd, bd, wp, bp, zx, sx, zws, sws, stride, pad, add)
    blk = ctx.prepack_qblock(we, be, qp(zws[0], sws[0]), wd, bd, qp(zws[1], sws[1]), wp, bp, qp(zws[2], sws[2]))
    a = rt.QBlockArgs()
    a.batch, a.in_h, a.in_w, a.stride = n, h, w, stride
    (a.pad_h_before, a.pad_h_after), (a.pad_w_before, a.pad_w_after) = pad
    a.x_qp = qp(zx, sx)
    (c1, z1, s1), (c2, z2, s2), (c3, z3, s3) = quant["expand"], quant["dw"], quant["project"]
    a.expand_qp, a.dw_qp, a.y_qp = qp(z1, s1), qp(z2, s2), qp(z3, s3)
    a.expand_clamp_min, a.expand_clamp_max = c1
    a.dw_clamp_min, a.dw_clamp_max = c2
    a.clamp_min, a.clamp_max = c3
    a.add_input = int(add)
    if add:
        a.sum_qp = qp(*quant["sum"])
        a.sum_clamp_min, a.sum_clamp_max = FULL
    oh, ow = want.shape[2:]
    xd = ctx.alloc(x.size).upload(np.ascontiguousarray(x.transpose(0, 2, 3, 1)))
    yd = ctx.alloc(n * oh * ow * cout).fill(0xA5)
    ctx.qblock(xd, blk, yd, a)
    ctx.sync()
    got = yd.download((n, oh, ow, cout), np.uint8).transpose(0, 3, 1, 2)
    bad = got != want
    assert not bad.any(), f"{bad.sum()} of {want.size} bytes differ; first at {np.argwhere(bad)[0]}: got {got[bad][0]} want {want[bad][0]}"
    assert want.size < 256 or len(np.unique(want)) > 8
    return blk, a, xd, yd, want


P1 = ((1, 1), (1, 1))
MOBILENET_BLOCKS = [  # (cin, mid, cout, h, w, stride, add): every inverted-residual block shape of MobileNetV2 1.0
    (16, 96, 24, 28, 28, 2, False), (24, 144, 24, 21, 21, 1, True), (24, 144, 32, 28, 28, 2, False),
    (32, 192, 32, 14, 14, 1, True), (32, 192, 64, 14, 14, 2, False), (64, 384, 64, 14, 14, 1, True),
    (64, 384, 96, 14, 14, 1, False), (96, 576, 96, 14, 14, 1, True), (96, 576, 160, 14, 14, 2, False),
    (160, 960, 160, 7, 7, 1, True), (160, 960, 320, 7, 7, 1, False),
]


@pytest.mark.parametrize("cin,mid,cout,h,w,stride,add", MOBILENET_BLOCKS)
def test_mobilenet_block_shapes(hip_ctx, cin, mid, cout, h, w, stride, add):
    run_block(hip_ctx, 2, cin, mid, cout, h, w, stride, P1, add, seed=cin * 1000 + mid + cout + stride)


RAGGED = [  # tiles cut by the image edge, channel counts that fill no chunk / tile, asymmetric (TF 'SAME') padding
    (1, 8, 24, 8, 10, 13, 1, P1, True), (3, 20, 40, 17, 5, 3, 1, P1, False), (2, 8, 100, 33, 16, 9, 2, P1, False),
    (2, 16, 96, 24, 12, 12, 2, ((0, 1), (0, 1)), False), (1, 12, 48, 12, 8, 8, 1, ((0, 0), (0, 0)), False),
    (2, 24, 144, 24, 9, 20, 1, ((1, 0), (0, 1)), False), (1, 192, 64, 320, 7, 7, 1, P1, False),
    (1, 32, 68, 300, 15, 8, 2, ((1, 0), (1, 0)), False), (1, 4, 4, 4, 1, 1, 1, P1, True), (5, 16, 64, 16, 3, 3, 1, P1, True),
]


@pytest.mark.parametrize("n,cin,mid,cout,h,w,stride,pad,add", RAGGED)
def test_ragged_blocks(hip_ctx, n, cin, mid, cout, h, w, stride, pad, add):
    run_block(hip_ctx, n, cin, mid, cout, h, w, stride, pad, add, seed=n + cin + mid + cout + h * w)


def test_block_equals_three_operators_and_repeats(hip_ctx):
    """The fused kernel against the three stand-alone operators on the device (larger batch than the oracle
    is asked to follow), twice in a row into a poisoned output."""
    from nncase_amd import kernels as K
    n, cin, mid, cout, h, w = 16, 32, 192, 32, 28, 28
    blk, a, xd, yd, want = run_block(hip_ctx, 2, cin, mid, cout, h, w, 1, P1, True, seed=99)
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, (n, h, w, cin), dtype=np.uint8)
    a.batch = n
    xb = hip_ctx.alloc(x.size).upload(x)
    outs = []
    for _ in range(2):
        yb = hip_ctx.alloc(n * h * w * cout).fill(0x5A)
        hip_ctx.qblock(xb, blk, yb, a)
        hip_ctx.sync()
        outs.append(yb.download((n, h, w, cout), np.uint8))
    assert np.array_equal(outs[0], outs[1])
    # images 0 and 1 of the big batch are not those of the small one, so compare against a per-image run
    a.batch = 1
    for i in (0, 7, 15):
        xi = hip_ctx.alloc(h * w * cin).upload(x[i])
        yi = hip_ctx.alloc(h * w * cout).fill(0)
        hip_ctx.qblock(xi, blk, yi, a)
        hip_ctx.sync()
        assert np.array_equal(yi.download((h, w, cout), np.uint8), outs[0][i])


def test_block_argument_checks(hip_ctx):
    assert hip_ctx.qblock_supported(16, 96, 24) and hip_ctx.qblock_supported(160, 960, 320)
    assert not hip_ctx.qblock_supported(3, 32, 16) and not hip_ctx.qblock_supported(256, 512, 64)
    assert not hip_ctx.qblock_supported(32, 192, 336)
    we = np.zeros((32, 6, 1, 1), np.uint8)
    with pytest.raises(rt.HipError):
        hip_ctx.prepack_qblock(we, None, qp(0, 1.0), np.zeros((32, 1, 3, 3), np.uint8), None, qp(0, 1.0),
                               np.zeros((8, 32, 1, 1), np.uint8), None, qp(0, 1.0))
    blk, a, xd, yd, _ = run_block(hip_ctx, 1, 8, 32, 8, 6, 6, 1, P1, True, seed=3)
    for field, value in (("stride", 3), ("pad_h_before", 2), ("batch", 0)):
        b = rt.QBlockArgs.from_buffer_copy(a)
        setattr(b, field, value)
        with pytest.raises(rt.HipError):
            hip_ctx.qblock(xd, blk, yd, b)
    b = rt.QBlockArgs.from_buffer_copy(a)
    b.stride = 2                                   # a residual needs the input's shape
    with pytest.raises(rt.HipError):
        hip_ctx.qblock(xd, blk, yd, b)
