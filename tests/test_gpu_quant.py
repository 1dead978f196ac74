"""GPU parity: quantize / dequantize / u8 glue through the C ABI vs the CPU oracle.
Bit-exact for integer outputs and for the fp32 dequantised values (each is one fp32
subtract and one multiply); fp16 outputs equal the fp32 value rounded to nearest even."""
import json
import os

import numpy as np
import pytest

from nncase_amd import kernels as K
from nncase_amd import runtime as rt
from nncase_amd.runtime import qp
from oracle import oracle as O

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
f32 = np.float32
NPQ = {"uint8": (np.uint8, O.U8), "int8": (np.int8, O.I8), "int16": (np.int16, O.I16)}


def test_golden_vectors(hip_ctx):
    g = GOLD["K1_dequantize"]
    y = K.dequantize(np.array(g["input_u8"], np.uint8), qp(g["zero_point"], g["scale"]), ctx=hip_ctx)
    assert y.view(np.uint32).tolist() == g["expected_f32_bits"]
    g = GOLD["K2_quantize_u8"]
    assert K.quantize(np.array(g["input_f32"], f32), qp(g["zero_point"], g["scale"]), np.uint8, ctx=hip_ctx).tolist() == g["expected"]
    g = GOLD["K3_quantize_i16"]
    assert K.quantize(np.array(g["input_f32"], f32), qp(g["zero_point"], g["scale"]), np.int16, ctx=hip_ctx).tolist() == g["expected"]
    g = GOLD["K3b_ties"]
    assert K.quantize(np.array(g["input_f32"], f32), qp(g["zero_point"], g["scale"]), np.uint8, ctx=hip_ctx).tolist() == g["expected_native"]


def test_reference_parameter_grids(hip_ctx):
    rng = np.random.default_rng(101)
    g = GOLD["K7_quantize_grid"]
    for shape in g["shapes"]:
        x = (rng.standard_normal(shape) * 2).astype(f32)
        for name in g["dtypes"]:
            npdt, code = NPQ[name]
            got = K.quantize(x, qp(g["zero_point"], g["scale"]), npdt, ctx=hip_ctx)
            assert got.shape == tuple(shape)
            assert np.array_equal(got, O.quantize(x, g["scale"], g["zero_point"], code))
    g = GOLD["K8_quantizelinear_grid"]
    x = rng.standard_normal(g["shape"]).astype(f32)
    for name in g["dtypes"]:
        npdt, code = NPQ[name]
        assert np.array_equal(K.quantize(x, qp(g["zero_point"], g["scale"]), npdt, ctx=hip_ctx),
                              O.quantize(x, g["scale"], g["zero_point"], code))


@pytest.mark.parametrize("count", [0, 1, 3, 4, 5, 1023, 4096 + 7, 200704, 1 << 22])
def test_quantize_sizes_ties_and_saturation(hip_ctx, count):
    rng = np.random.default_rng(count)
    scale, zp = f32(0.0235), 3
    x = (rng.standard_normal(count) * 3).astype(f32)
    if count >= 1023:
        k = rng.integers(-40, 300, count // 4)
        x[: count // 4] = ((k + 0.5).astype(f32) - f32(zp)) * scale  # lands on or next to .5 ties
        x[-8:] = np.array([1e9, -1e9, 3e38, -3e38, 6.0, 0.0, -0.0, 1e-30], f32)
    for npdt, code in NPQ.values():
        got = K.quantize(x, qp(zp, scale), npdt, ctx=hip_ctx)
        assert np.array_equal(got, O.quantize(x, scale, zp, code))


def test_quantize_f16_input(hip_ctx):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(5000) * 4).astype(np.float16)
    got = K.quantize(x, qp(100, 0.02), np.uint8, ctx=hip_ctx)
    assert np.array_equal(got, O.quantize(x.astype(f32), 0.02, 100, O.U8))


@pytest.mark.parametrize("count", [1, 7, 4096 + 3, 1 << 20])
def test_dequantize(hip_ctx, count):
    rng = np.random.default_rng(count)
    for npdt in (np.uint8, np.int8, np.int16):
        info = np.iinfo(npdt)
        q = rng.integers(info.min, info.max + 1, count).astype(npdt)
        want = O.dequantize(q, 0.0173, 11)
        got = K.dequantize(q, qp(11, 0.0173), np.float32, ctx=hip_ctx)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        got16 = K.dequantize(q, qp(11, 0.0173), np.float16, ctx=hip_ctx)
        assert np.array_equal(got16.view(np.uint16), O.f32_to_f16_bits(want))


@pytest.mark.parametrize("count", [1, 2, 3, 4, 5, 7, 16, 1027])
def test_dequantize_to_fp16_rounds_the_fp32_product(hip_ctx, count):
    """(q - zp) * scale lands exactly half way between two fp16 values after its fp32 rounding while the exact product
    does not: the fp16 result is the nearest-even of the rounded fp32 value, in the vector body of the kernel and in
    its scalar tail alike (a fused multiply-convert would round the exact product and give the neighbour)."""
    scale = np.float32(0.026969021186232567)
    codes = np.array([-172, -86, -43, 43, 86, 172], np.int16)
    q = np.resize(codes, count).astype(np.int16)
    want = O.dequantize(q, float(scale), 0)
    got16 = K.dequantize(q, qp(0, float(scale)), np.float16, ctx=hip_ctx)
    assert np.array_equal(got16.view(np.uint16), O.f32_to_f16_bits(want))
    exact = np.float16(q.astype(np.float64) * np.float64(scale))
    assert (exact.view(np.uint16) != O.f32_to_f16_bits(want)).all()  # the case really separates the two roundings


def test_quantize_dequantize_roundtrip_full_size(hip_ctx):
    # size-independent property at a BASELINE size: Q(DQ(q)) == q for every code
    n = 32 * 64 * 56 * 56
    q = (np.arange(n, dtype=np.uint32) * 2654435761 >> 13).astype(np.uint8)
    src = hip_ctx.to_device(q)
    mid = hip_ctx.alloc(n * 4)
    dst = hip_ctx.alloc(n)
    p = qp(17, 0.0471)
    hip_ctx.dequantize(src, rt.DT_U8, mid, rt.DT_F32, n, p)
    hip_ctx.quantize(mid, rt.DT_F32, dst, rt.DT_U8, n, p)
    assert np.array_equal(dst.download((n,), np.uint8), q)


def test_unaligned_pointers_take_the_scalar_path(hip_ctx):
    rng = np.random.default_rng(9)
    x = rng.standard_normal(1001).astype(f32)
    buf = hip_ctx.to_device(np.concatenate([np.zeros(1, f32), x]))
    out = hip_ctx.alloc(1001 + 16)

    class View:  # a device pointer 4 bytes / 1 byte into an allocation
        def __init__(self, ptr):
            self.ptr = ptr

    hip_ctx.quantize(View(buf.ptr + 4), rt.DT_F32, View(out.ptr + 1), rt.DT_U8, 1001, qp(128, 0.03))
    got = out.download((1001 + 16,), np.uint8)[1:1002]
    assert np.array_equal(got, O.quantize(x, 0.03, 128, O.U8))


def test_error_codes(hip_ctx):
    x = np.zeros(4, f32)
    with pytest.raises(rt.HipError) as e:
        K.quantize(x, qp(0, 0.0), np.uint8, ctx=hip_ctx)
    assert e.value.code == -22  # EINVAL: zero scale
    with pytest.raises(rt.HipError) as e:
        K.quantize(x, qp(0, 1.0), np.int32, ctx=hip_ctx)
    assert e.value.code == -rt.ERR_DATATYPE_MISMATCH
    assert "unsupported" in str(e.value)


@pytest.mark.parametrize("count", [5, 16, 1000, 64 * 56 * 56 * 24])
def test_qadd(hip_ctx, count):
    rng = np.random.default_rng(count)
    a = rng.integers(0, 256, count, dtype=np.uint8)
    b = rng.integers(0, 256, count, dtype=np.uint8)
    got = K.binary_add(a, b, qp(3, 0.02), qp(128, 0.011), qp(77, 0.031), ctx=hip_ctx)
    assert np.array_equal(got, O.qadd(a, b, 3, 0.02, 128, 0.011, 77, 0.031))
    got = K.binary_add(a, b, qp(3, 0.02), qp(128, 0.011), qp(0, 0.02), fused_clamp=(0.0, 6.0), ctx=hip_ctx)
    assert np.array_equal(got, O.qadd(a, b, 3, 0.02, 128, 0.011, 0, 0.02, (0.0, 6.0)))


@pytest.mark.parametrize("shape", [(1, 5, 7, 7), (3, 1280, 7, 7), (2, 17, 3, 5), (2, 8, 1, 1), (5, 64, 4, 4), (2, 12, 9, 5), (64, 1280, 7, 7)])
def test_qglobal_avgpool(hip_ctx, shape):
    rng = np.random.default_rng(shape[1])
    x = rng.integers(0, 256, shape, dtype=np.uint8)
    got = K.global_average_pool(x, qp(5, 0.02), qp(9, 0.015), ctx=hip_ctx)
    assert np.array_equal(got[:, :, 0, 0], O.qglobal_avgpool(x, 5, 0.02, 9, 0.015))


# ---- strided operands: the reference's kernels address both tensors through their strides
# (reference/quantize.cpp:36-47, dequantize.cpp:36-44); views with gaps, transposes, broadcasts (stride 0 on the
# input), rank 1..6, and an output view whose gaps must keep what they held.
STRIDED_VIEWS = [
    ("rows with gaps", lambda a: a[:, ::2, 1:9]),
    ("transposed", lambda a: a.transpose(2, 0, 1)),
    ("inner stride 3", lambda a: a[1, :, ::3]),
    ("single row", lambda a: a[2, 3, :]),
    ("rank 6", lambda a: a[:4, :6, :12].reshape(2, 2, 3, 2, 3, 4)[:, :, ::2, :, 1:, ::3]),
    ("broadcast row", lambda a: np.broadcast_to(a[0, 0, :8], (5, 8))),
]


@pytest.mark.parametrize("name,view", STRIDED_VIEWS)
def test_quantize_and_dequantize_strided_views(hip_ctx, name, view):
    rng = np.random.default_rng(len(name))
    base = ((rng.random((6, 10, 20), dtype=f32) - 0.3) * 9).astype(f32)
    x = view(base)
    assert not x.flags.c_contiguous or x.ndim == 1
    for out_np, out_code in ((np.uint8, O.U8), (np.int16, O.I16)):
        q = K.quantize(x, qp(37, 0.043), out_np, ctx=hip_ctx)
        want = O.quantize(np.ascontiguousarray(x), 0.043, 37, out_code)
        assert q.shape == x.shape and np.array_equal(q, want)
    codes = view(rng.integers(0, 256, (6, 10, 20), dtype=np.uint8))
    y = K.dequantize(codes, qp(131, 0.0123), np.float32, ctx=hip_ctx)
    assert np.array_equal(y.view(np.uint32), O.dequantize(np.ascontiguousarray(codes), 0.0123, 131).view(np.uint32))


def test_strided_output_keeps_the_elements_its_strides_skip(hip_ctx):
    rng = np.random.default_rng(3)
    x = ((rng.random((7, 5, 12), dtype=f32) - 0.5) * 6).astype(f32)
    store = np.full((7, 11, 40), 0xAB, np.uint8)
    out = store[:, 1::2, 3:39:3]                      # a [7, 5, 12] window into a larger tensor
    got = K.quantize(x[:, ::-1][:, ::-1], qp(128, 0.02), np.uint8, ctx=hip_ctx, out=out)
    assert got is out
    want = O.quantize(x, 0.02, 128, O.U8)
    assert np.array_equal(out, want)
    mask = np.ones(store.shape, bool)
    mask[:, 1::2, 3:39:3] = False
    assert (store[mask] == 0xAB).all()                # nothing outside the window was touched
    fstore = np.full((7, 5, 30), -7.5, f32)
    fout = fstore[:, :, 2:26:2]
    K.dequantize(want, qp(128, 0.02), np.float32, ctx=hip_ctx, out=fout)
    assert np.array_equal(fout.view(np.uint32), O.dequantize(want, 0.02, 128).view(np.uint32))
    assert (fstore[:, :, 0:2] == -7.5).all() and (fstore[:, :, 3:26:2] == -7.5).all() and (fstore[:, :, 26:] == -7.5).all()


def test_strided_argument_checks(hip_ctx):
    src, dst = hip_ctx.alloc(1024), hip_ctx.alloc(1024)
    for shape, ins, outs, code in (((4,) * 7, (1,) * 7, (1,) * 7, -22),          # rank 7
                                   ((4, 4), (4, -1), (4, 1), -22),               # negative stride
                                   ((1 << 20, 1 << 12), (1 << 12, 1), (1 << 12, 1), -22)):   # 2^32 elements
        with pytest.raises(rt.HipError) as e:
            hip_ctx.quantize_strided(src, rt.DT_F32, dst, rt.DT_U8, shape, ins, outs, qp(0, 1.0))
        assert e.value.code == code
    with pytest.raises(rt.HipError) as e:
        hip_ctx.dequantize_strided(src, rt.DT_F32, dst, rt.DT_U8, (4, 2), (4, 1), (2, 2), qp(0, 1.0))
    assert e.value.code == -rt.ERR_DATATYPE_MISMATCH
    hip_ctx.quantize_strided(src, rt.DT_F32, dst, rt.DT_U8, (0, 4), (4, 1), (4, 1), qp(0, 1.0))   # empty: nothing to do
