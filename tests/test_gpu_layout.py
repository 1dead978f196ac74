"""GPU parity: pack / unpack and NCHW<->NHWC relayout (pure permutations, bit-exact)."""
import numpy as np
import pytest

from nncase_amd import kernels as K
from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,axes,lanes,dtype", [
    ((2, 64, 3, 5), [1], [32], np.uint8),          # NCHW -> NC/32 HW 32
    ((2, 5, 3, 7), [1], [4], np.uint8),            # ragged: 5 channels into lanes of 4
    ((6, 10), [1, 0], [4, 2], np.float32),         # two axes, lanes appended in the listed order
    ((1024, 144), [0, 1], [16, 64], np.uint8),     # [K, N] -> weight-tile style blocking
    ((3, 1, 17), [2], [8], np.float16),
    ((7,), [0], [16], np.int32),
    ((2, 3, 4, 5, 6), [-1, 1], [4, 2], np.uint8),
    ((2, 9, 11, 3), [3], [4], np.uint8),           # RGB -> RGBX: the dword fast path
    ((5, 7, 1), [2], [4], np.uint8),
    ((4, 6, 4), [-1], [4], np.uint8),              # already 4 wide
    ((2, 6, 10, 3), [1, 2, 3], [2, 2, 4], np.uint8),   # 2 x 2 blocks of RGB -> 16-channel pixels: one thread per block
    ((3, 4, 2, 1), [1, 2, 3], [2, 2, 4], np.uint8),
    ((1, 8, 6, 4), [1, 2, 3], [2, 2, 4], np.uint8),
    ((2, 5, 6, 3), [1, 2, 3], [2, 2, 4], np.uint8),    # odd height: the general kernel
    ((2, 6, 10, 3), [2, 1, 3], [2, 2, 4], np.uint8),   # lanes in another order: the general kernel
    # the LDS-tile kernel: lanes of the last packed axis against the innermost plain axis, ragged both ways
    ((2, 33, 300), [1], [32], np.uint8),
    ((2, 33, 300), [1], [32], np.float32),
    ((4, 96, 14, 14), [1], [32], np.float16),          # trailing unpacked axes taken as one (H x W)
    ((70, 40), [1, 0], [16, 64], np.uint8),            # the innermost axis packed under an earlier lane entry
    ((520, 272), [1, 0], [16, 64], np.uint8),
    ((5, 3, 10, 4), [0, 2], [4, 4], np.uint8),         # another packed axis among the block coordinates, ragged
    ((2, 2, 130, 4), [2], [128], np.uint8),
    ((3, 20, 6), [0, 1], [2, 8], np.float16),
    ((2, 5, 3, 7), [1], [4], np.float32),
    ((3, 7, 6), [1], [4], np.uint8),                   # rows of 6 bytes: not dword multiples, the element-wise kernel
    ((2, 70, 4, 16), [1], [32], np.uint8),             # plain rows of whole 16-byte pieces: the tile kernel's wide loads, ragged lanes
    ((2, 40, 8, 8), [1], [8], np.float16),
    ((3, 1100, 48), [1], [64], np.uint8),              # many lane groups (the last one ragged), one short stretch
    ((2, 36, 2100), [1], [4], np.uint8),               # few lanes, a long stretch split evenly over its tiles
])
def test_pack_unpack(hip_ctx, shape, axes, lanes, dtype):
    rng = np.random.default_rng(len(shape) + shape[0])
    x = rng.integers(1, 120, shape).astype(dtype)
    y = K.pack(x, axes, lanes, ctx=hip_ctx)
    want = O.pack(x, axes, lanes)
    assert y.shape == want.shape and np.array_equal(y.view(np.uint8), want.view(np.uint8))
    back = K.unpack(y, axes, lanes, shape, ctx=hip_ctx)
    assert np.array_equal(back.view(np.uint8), x.view(np.uint8))


def test_pack_roundtrip_full_size(hip_ctx):
    # round trip at a BASELINE size (batch-32 conv-block activation), ragged lanes
    x = (np.arange(32 * 144 * 56 * 56, dtype=np.uint32) * 2654435761 >> 11).astype(np.uint8).reshape(32, 144, 56, 56)
    y = K.pack(x, [1], [64], ctx=hip_ctx)
    assert y.shape == (32, 3, 56, 56, 64) and (y[:, 2, :, :, 16:] == 0).all()
    assert np.array_equal(K.unpack(y, [1], [64], x.shape, ctx=hip_ctx), x)


@pytest.mark.parametrize("shape,axes,lanes", [
    ((2, 6, 10, 3), [1, 2, 3], [2, 2, 4]), ((1, 64, 48, 3), [1, 2, 3], [2, 2, 4]), ((3, 2, 2, 1), [1, 2, -1], [2, 2, 4]),
    ((2, 4, 6, 4), [1, 2, 3], [2, 2, 4]), ((2, 9, 11, 3), [3], [4]), ((7, 2), [1], [4]), ((5, 4), [-1], [4])])
def test_quantize_pack_equals_quantize_then_pack(hip_ctx, shape, axes, lanes):
    """Quantize and Pack in one pass over a float32 tensor == the two operators one after the other (oracle: quantize,
    then pack), for the two layouts that stand in front of a stem convolution; values beyond the u8 range, halves that
    round to even included."""
    from nncase_amd.runtime import qp
    rng = np.random.default_rng(sum(shape))
    x = ((rng.random(shape, dtype=np.float32) - 0.3) * 3).astype(np.float32)
    flat = x.reshape(-1)
    flat[::7] = (np.arange(flat[::7].size) - 3 + 0.5).astype(np.float32) * np.float32(0.0125)     # exact halves before rounding
    scale, zp = np.float32(0.0125), 17
    want = O.pack(O.quantize(x, scale, zp, O.U8), axes, lanes)
    src, dst = hip_ctx.to_device(x), hip_ctx.alloc(want.size)
    hip_ctx.quantize_pack(src, dst, list(shape), axes, lanes, qp(zp, scale))
    assert np.array_equal(dst.download(want.shape, np.uint8), want)


def test_quantize_pack_refuses_other_layouts(hip_ctx):
    from nncase_amd import runtime as rt
    src, dst = hip_ctx.alloc(4 * 2 * 6 * 10 * 8), hip_ctx.alloc(2 * 6 * 10 * 8)
    for shape, axes, lanes, q in (((2, 6, 10, 8), [3], [4], rt.qp(0, 1.0)),            # more than 4 channels
                                  ((2, 5, 10, 3), [1, 2, 3], [2, 2, 4], rt.qp(0, 1.0)),   # odd height
                                  ((2, 6, 10, 3), [2, 1, 3], [2, 2, 4], rt.qp(0, 1.0)),   # another lane order
                                  ((2, 6, 10, 3), [3], [8], rt.qp(0, 1.0)),
                                  ((2, 6, 10, 3), [3], [4], rt.qp(0, 0.0))):             # zero scale
        with pytest.raises(rt.HipError) as e:
            hip_ctx.quantize_pack(src, dst, list(shape), axes, lanes, q)
        assert e.value.code == -22


@pytest.mark.parametrize("shape", [(1, 3, 224, 224), (2, 144, 7, 5), (3, 1, 1, 1), (1, 33, 65, 2), (2, 256, 14, 14), (1, 64, 56, 56), (2, 132, 6, 6),
                                   (3, 4, 2, 600)])
@pytest.mark.parametrize("dtype", [np.uint8, np.float16, np.float32])
def test_nchw_nhwc(hip_ctx, shape, dtype):
    rng = np.random.default_rng(shape[1])
    x = rng.integers(0, 200, shape).astype(dtype)
    y = K.transpose_nchw_to_nhwc(x, ctx=hip_ctx)
    assert np.array_equal(y, x.transpose(0, 2, 3, 1))
    assert np.array_equal(K.transpose_nhwc_to_nchw(y, ctx=hip_ctx), x)
