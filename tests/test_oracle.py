"""Pins the CPU oracle (oracle/nncase_oracle.c) before anything is compared against it:
the reference's own literal vectors (tests/golden/reference_vectors.json), closed forms,
float64 / int64 brute force and invariants chosen so that a dropped term, a wrong sign or
index or a transposed operand fails at least one check.  No GPU needed."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
f32 = np.float32


# ----------------------------------------------------------------------------- quantize / dequantize
def test_k1_dequantize_literals():
    g = GOLD["K1_dequantize"]
    y = O.dequantize(np.array(g["input_u8"], np.uint8), g["scale"], g["zero_point"])
    assert y.view(np.uint32).tolist() == g["expected_f32_bits"]


def test_k2_k3_quantize_literals():
    g = GOLD["K2_quantize_u8"]
    assert O.quantize(np.array(g["input_f32"], f32), g["scale"], g["zero_point"], O.U8).tolist() == g["expected"]
    g = GOLD["K3_quantize_i16"]
    assert O.quantize(np.array(g["input_f32"], f32), g["scale"], g["zero_point"], O.I16).tolist() == g["expected"]


def test_k3b_ties_distinguish_native_from_ort_order():
    g = GOLD["K3b_ties"]
    x = np.array(g["input_f32"], f32)
    assert O.quantize(x, g["scale"], g["zero_point"], O.U8).tolist() == g["expected_native"]
    assert O.quantize(x, g["scale"], g["zero_point"], O.U8, ort_order=True).tolist() == g["expected_ort_order"]


def test_quantize_round_half_even_and_saturation():
    # x / 1 + 0 = k + 0.5 must go to the even neighbour (half-away would give 1, 2, 3, 4 ...)
    x = np.array([0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5], f32)
    assert O.quantize(x, 1.0, 0, O.I8).tolist() == [0, 2, 2, 4, 0, -2, -2]
    big = np.array([1e9, -1e9, 300.0, -300.0, 255.4, 255.5, -0.5, -0.51], f32)
    assert O.quantize(big, 1.0, 0, O.U8).tolist() == [255, 0, 255, 0, 255, 255, 0, 0]
    assert O.quantize(big, 1.0, 0, O.I8).tolist() == [127, -128, 127, -128, 127, 127, 0, -1]
    assert O.quantize(big, 1.0, 0, O.I16).tolist() == [32767, -32768, 300, -300, 255, 256, 0, -1]


def test_quantize_matches_numpy_fp32_formula_on_reference_grids():
    rng = np.random.default_rng(7)
    g = GOLD["K7_quantize_grid"]
    for shape in g["shapes"]:
        x = (rng.standard_normal(shape) * 2).astype(f32)
        for name, code in (("uint8", O.U8), ("int8", O.I8), ("int16", O.I16)):
            info = np.iinfo(name)
            want = np.clip(np.rint(x / f32(g["scale"]) + f32(g["zero_point"])), info.min, info.max).astype(name)
            got = O.quantize(x, g["scale"], g["zero_point"], code)
            assert got.shape == tuple(shape) and np.array_equal(got, want)
    g = GOLD["K8_quantizelinear_grid"]
    x = rng.standard_normal(g["shape"]).astype(f32)
    want = np.clip(np.rint(x / f32(g["scale"]) + f32(g["zero_point"])), 0, 255).astype(np.uint8)
    assert np.array_equal(O.quantize(x, g["scale"], g["zero_point"], O.U8), want)


def test_quantize_dequantize_idempotent_for_all_256_codes():
    for scale, zp in ((0.0235, 0), (0.1, 128), (3.7e-3, 255), (1.0, 17)):
        q = np.arange(256, dtype=np.uint8)
        assert np.array_equal(O.quantize(O.dequantize(q, scale, zp), scale, zp, O.U8), q)


# ----------------------------------------------------------------------------- quant params
def test_k4_k6_get_quant_param_literals():
    for g in GOLD["K4_get_quant_param"] + [GOLD["K6_quant_param_of"]]:
        mode = {"UnsignedMode": O.UNSIGNED, "SignedSymmetricMode": O.SIGNED_SYMMETRIC,
                "SignedAsymmetricMode": O.SIGNED_ASYMMETRIC}[g["mode"]]
        zp, sc = O.get_quant_param(g["range"][0], g["range"][1], g["bits"], mode)
        assert zp == g["zero_point"] and sc == f32(g["scale"])


def test_k5_fixup_range_literals():
    for g in GOLD["K5_fixup_range"]:
        lo, hi = O.fixup_range(g["range"][0], g["range"][1], g["symmetric"])
        assert (lo, hi) == (f32(g["expected"][0]), f32(g["expected"][1]))


def test_get_quant_param_bankers_rounding_and_zero_inclusion():
    # min * (0 - 255) / (max - min) = 0.5 * 255 / 1 = 127.5 -> 128 (even); 0.25 -> 63.75 -> 64
    assert O.get_quant_param(-0.5, 0.5)[0] == 128
    assert O.get_quant_param(-0.25, 0.75)[0] == 64
    # -2.5/5*255 = 127.5 as well; -1.5/3 -> 127.5; a tie that must go DOWN to even: 0.1*(255)/0.2=127.5 -> 128,
    # (min=-0.3, max=0.1): 0.3*255/0.4 = 191.25 -> 191
    assert O.get_quant_param(-0.3, 0.1)[0] == 191
    # ranges that exclude zero are widened to include it
    zp, sc = O.get_quant_param(1.0, 3.0)
    assert zp == 0 and sc == f32(3.0 / 255.0)
    zp, sc = O.get_quant_param(-3.0, -1.0)
    assert zp == 255 and sc == f32(3.0 / 255.0)
    # calibrator variant: span below 1e-6 becomes 0.1, small spans are NOT widened to 0.01
    assert O.calib_fixup_range(0.0, 0.005) == (f32(0), f32(0.005))
    assert O.calib_fixup_range(0.0, 0.0) == (f32(0), f32(0.1))
    assert O.calib_fixup_range(2.0, 3.0) == (f32(0), f32(3.0))


# ----------------------------------------------------------------------------- half
def test_half_conversion_exhaustive_and_rounding():
    allh = np.arange(65536, dtype=np.uint16)
    f = O.f16_bits_to_f32(allh)
    want = allh.view(np.float16).astype(f32)
    nan = np.isnan(want)
    assert np.array_equal(f[~nan].view(np.uint32), want[~nan].view(np.uint32)) and np.isnan(f[nan]).all()
    # every finite half round-trips
    back = O.f32_to_f16_bits(want[~nan])
    assert np.array_equal(back, allh[~nan])
    # random floats, midpoints between adjacent halves, subnormal range, overflow
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(200000).astype(f32) * f32(100),
        (rng.standard_normal(100000) * 1e-5).astype(f32),
        rng.integers(0, 2 ** 32, 300000, dtype=np.uint32).view(f32),
    ])
    fin = allh[np.isfinite(want)]
    lo = fin.view(np.float16).astype(np.float64)
    nxt = (fin + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    ok = np.isfinite(nxt)
    mid = ((lo[ok] + nxt[ok]) / 2).astype(f32)  # exactly representable in fp32
    x = np.concatenate([x, mid, np.nextafter(mid, f32(np.inf)), np.nextafter(mid, f32(-np.inf)),
                        np.array([65504, 65519.99, 65520, 1e9, -1e9, np.inf, -np.inf, 5.96e-8, 2.98e-8, 2.9e-8, 0, -0.0], f32)])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want_bits = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16_bits(x), want_bits)
    assert int(O.f32_to_f16_bits(np.array([np.nan], f32))[0]) & 0x7fff == 0x7e00


# ----------------------------------------------------------------------------- float conv / matmul
def _conv_f64(x, w, b, stride, padding, dilation, groups):
    n, c, h, wd = x.shape
    oc, gic, kh, kw = w.shape
    (ph0, ph1), (pw0, pw1) = padding
    xp = np.zeros((n, c, h + ph0 + ph1, wd + pw0 + pw1))
    xp[:, :, ph0:ph0 + h, pw0:pw0 + wd] = x
    oh = (h + ph0 + ph1 - ((kh - 1) * dilation[0] + 1) + stride[0]) // stride[0]
    ow = (wd + pw0 + pw1 - ((kw - 1) * dilation[1] + 1) + stride[1]) // stride[1]
    out = np.zeros((n, oc, oh, ow))
    goc = oc // groups
    for o in range(oc):
        g = o // goc
        for ky in range(kh):
            for kx in range(kw):
                ys = slice(ky * dilation[0], ky * dilation[0] + (oh - 1) * stride[0] + 1, stride[0])
                xs = slice(kx * dilation[1], kx * dilation[1] + (ow - 1) * stride[1] + 1, stride[1])
                patch = xp[:, g * gic:(g + 1) * gic, ys, xs]
                out[:, o] += np.einsum("nchw,c->nhw", patch, w[o, :, ky, kx].astype(np.float64))
        out[:, o] += b[o]
    return out


CONV_CASES = [
    # (N, C, H, W, OC, k, stride, pad, dilation, groups)   -- reference grids test_conv2d.json / tflite tests
    (1, 4, 5, 5, 8, 3, (1, 1), ((1, 1), (1, 1)), (1, 1), 1),
    (1, 4, 16, 16, 8, 1, (2, 2), ((1, 1), (1, 1)), (1, 1), 1),
    (1, 4, 16, 16, 8, 3, (2, 2), ((1, 1), (1, 1)), (2, 2), 1),
    (3, 16, 33, 65, 16, 3, (1, 3), ((1, 1), (1, 1)), (1, 1), 16),
    (1, 16, 33, 65, 16, 5, (1, 1), ((2, 2), (2, 2)), (1, 1), 16),
    (2, 6, 9, 7, 4, 3, (5, 5), ((0, 2), (1, 0)), (1, 1), 2),
    (1, 3, 16, 16, 5, 3, (2, 2), ((0, 1), (0, 1)), (2, 2), 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_ref_conv2d_f32_matches_float64_bruteforce(case):
    n, c, h, w, oc, k, stride, pad, dil, groups = case
    rng = np.random.default_rng(11)
    x = rng.standard_normal((n, c, h, w)).astype(f32)
    wt = rng.standard_normal((oc, c // groups, k, k)).astype(f32)
    b = rng.standard_normal(oc).astype(f32)
    got = O.conv2d_f32(x, wt, b, stride, pad, dil, groups)
    want = _conv_f64(x.astype(np.float64), wt, b.astype(np.float64), stride, pad, dil, groups)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)
    # fused clamp is a plain clamp of the unclamped result
    gc = O.conv2d_f32(x, wt, b, stride, pad, dil, groups, fused_clamp=(0.0, 6.0))
    assert np.array_equal(gc, np.clip(got, 0, 6))


def test_ref_conv2d_f32_sequential_summation_order():
    # 1e8 + 1 - 1e8: the reference's sequential float order gives 0, pairwise/double would give 1
    x = np.array([1e8, 1.0, -1e8], f32).reshape(1, 3, 1, 1)
    w = np.ones((1, 3, 1, 1), f32)
    assert O.conv2d_f32(x, w, np.zeros(1, f32))[0, 0, 0, 0] == 0.0
    # and the bias is the FIRST term: (1e8 + 1) - 1e8 = 0 with bias 1e8 first
    x2 = np.array([1.0, -1e8], f32).reshape(1, 2, 1, 1)
    assert O.conv2d_f32(x2, np.ones((1, 2, 1, 1), f32), np.array([1e8], f32))[0, 0, 0, 0] == 0.0


@pytest.mark.parametrize("ash,bsh", [((6,), (6,)), ((6,), (6, 3)), ((6,), (2, 3, 6, 3)), ((4, 6), (6, 3)),
                                     ((2, 1, 4, 6), (3, 6, 5)), ((5, 4, 6), (6,)), ((2, 3, 4, 6), (2, 3, 6, 2))])
def test_ref_matmul_f32_matches_numpy_with_broadcast(ash, bsh):
    rng = np.random.default_rng(5)
    a, b = rng.standard_normal(ash).astype(f32), rng.standard_normal(bsh).astype(f32)
    got = O.matmul_f32(a, b)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_ref_matmul_not_transposed():
    a = np.array([[1, 2], [3, 4]], f32)
    b = np.array([[0, 1], [1, 0]], f32)
    assert O.matmul_f32(a, b).tolist() == [[2, 1], [4, 3]]


def test_ref_reduce_window_mean():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 3, 7, 7)).astype(f32)
    got = O.reduce_window2d_mean_f32(x, (7, 7), (1, 1))
    np.testing.assert_allclose(got[:, :, 0, 0], x.astype(np.float64).mean(axis=(2, 3)), rtol=1e-6, atol=1e-6)
    # sequential order: ((a + b) + c) / 3 in fp32
    v = np.array([1e8, 1.0, -1e8], f32).reshape(1, 1, 1, 3)
    assert O.reduce_window2d_mean_f32(v, (1, 3), (1, 1))[0, 0, 0, 0] == 0.0
    # padded 3x3 mean: count excludes the padding unless count_include_pad
    ones = np.ones((1, 1, 2, 2), f32)
    assert O.reduce_window2d_mean_f32(ones, (3, 3), (1, 1), ((1, 1), (1, 1)))[0, 0, 0, 0] == 1.0
    assert O.reduce_window2d_mean_f32(ones, (3, 3), (1, 1), ((1, 1), (1, 1)), True)[0, 0, 0, 0] == f32(4) / f32(9)


# ----------------------------------------------------------------------------- integer-exact operators
def _qconv_i64(x, w, bias, zx, zw, stride, padding, dilation, groups):
    xs = x.astype(np.int64) - zx
    ws = w.astype(np.int64) - zw
    out = _conv_f64(xs.astype(np.float64), ws, np.zeros(w.shape[0]), stride, padding, dilation, groups)
    out = np.rint(out).astype(np.int64)  # exact: all partial sums are integers far below 2^53
    return out + np.asarray(bias, np.int64).reshape(1, -1, 1, 1)


@pytest.mark.parametrize("case", CONV_CASES)
def test_qconv_accumulators_equal_int64_bruteforce(case):
    n, c, h, w, oc, k, stride, pad, dil, groups = case
    rng = np.random.default_rng(13)
    x = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    wt = rng.integers(0, 256, (oc, c // groups, k, k), dtype=np.uint8)
    b = rng.integers(-5000, 5000, oc).astype(np.int32)
    zx, zw = 7, 131
    got = O.qconv2d(x, wt, b, zx, 0.02, zw, 0.01, stride=stride, padding=pad, dilation=dil, groups=groups, out_mode=O.OUT_I32)
    assert np.array_equal(got.astype(np.int64), _qconv_i64(x, wt, b, zx, zw, stride, pad, dil, groups))


def test_qconv_invariants():
    rng = np.random.default_rng(17)
    x = rng.integers(0, 256, (2, 8, 6, 6), dtype=np.uint8)
    w = rng.integers(0, 256, (4, 8, 3, 3), dtype=np.uint8)
    kw = dict(stride=(1, 1), padding=((1, 1), (1, 1)), out_mode=O.OUT_I32)
    # weights all equal to their zero point, or input all equal to its zero point -> accumulators == bias
    b = np.array([5, -7, 0, 11], np.int32)
    assert np.array_equal(O.qconv2d(x, np.full_like(w, 99), b, 3, 1, 99, 1, **kw), np.broadcast_to(b.reshape(1, 4, 1, 1), (2, 4, 6, 6)))
    assert np.array_equal(O.qconv2d(np.full_like(x, 42), w, b, 42, 1, 120, 1, **kw), np.broadcast_to(b.reshape(1, 4, 1, 1), (2, 4, 6, 6)))
    # padding is a real zero: equals an unpadded conv over an input padded explicitly with zx
    zx = 37
    xp = np.full((2, 8, 8, 8), zx, np.uint8)
    xp[:, :, 1:7, 1:7] = x
    a1 = O.qconv2d(x, w, None, zx, 1, 120, 1, **kw)
    a2 = O.qconv2d(xp, w, None, zx, 1, 120, 1, stride=(1, 1), padding=((0, 0), (0, 0)), out_mode=O.OUT_I32)
    assert np.array_equal(a1, a2)
    # zero-point identity on a 1x1 conv: sum (x-zx)(w-zw) = sum xw - zw sum x - zx sum w + K zx zw
    w1 = rng.integers(0, 256, (4, 8, 1, 1), dtype=np.uint8)
    acc = O.qconv2d(x, w1, None, zx, 1, 120, 1, out_mode=O.OUT_I32).astype(np.int64)
    xi, wi = x.astype(np.int64), w1[:, :, 0, 0].astype(np.int64)
    ident = (np.einsum("nchw,oc->nohw", xi, wi) - 120 * xi.sum(1, keepdims=True) - zx * wi.sum(1).reshape(1, 4, 1, 1) + 8 * zx * 120)
    assert np.array_equal(acc, ident)
    # extremes: all-255 against all-0 weights with zw = 255 reaches K * 255 * 255 in magnitude
    xe, we = np.full((1, 64, 1, 1), 255, np.uint8), np.zeros((1, 64, 1, 1), np.uint8)
    assert O.qconv2d(xe, we, None, 0, 1, 255, 1, out_mode=O.OUT_I32)[0, 0, 0, 0] == -64 * 255 * 255


def test_qmatmul_equals_int64_and_is_not_transposed():
    rng = np.random.default_rng(19)
    a = rng.integers(0, 256, (9, 70), dtype=np.uint8)
    b = rng.integers(0, 256, (70, 13), dtype=np.uint8)
    bias = rng.integers(-100, 100, 13).astype(np.int32)
    got = O.qmatmul(a, b, bias, 128, 0.02, 101, 0.003)
    want = (a.astype(np.int64) - 128) @ (b.astype(np.int64) - 101) + bias
    assert np.array_equal(got.astype(np.int64), want)
    f = O.qmatmul(a, b, bias, 128, 0.02, 101, 0.003, out_mode=O.OUT_F32)
    assert np.array_equal(f, want.astype(f32) * (f32(0.02) * f32(0.003)))


def test_requant_formula_dense_sweep_monotone_and_ties():
    # numpy fp32 restatement, step by step (each numpy op rounds to fp32 once)
    def np_requant(acc, sx, sw, sy, zy, lo, hi):
        m = f32(sx) * f32(sw)
        y = acc.astype(f32) * m
        y = np.maximum(np.minimum(y, f32(hi)), f32(lo))
        t = y / f32(sy) + f32(zy)
        return np.clip(np.rint(t), 0, 255).astype(np.uint8)

    params = [(0.02, 0.004, 0.0235, 0, 0.0, 6.0), (0.5, 0.5, 0.25, 3, -O.FLT_MAX, O.FLT_MAX), (0.017, 0.0031, 0.05, 128, -1.0, 1.0),
              (1.0, 1.0, 2.0, 0, -O.FLT_MAX, O.FLT_MAX)]
    acc = np.concatenate([np.arange(-(1 << 17), 1 << 17, dtype=np.int32),
                          np.arange(-(1 << 24), 1 << 24, 127, dtype=np.int32),
                          np.array([np.iinfo(np.int32).min, np.iinfo(np.int32).max], np.int32)])
    acc.sort()
    for sx, sw, sy, zy, lo, hi in params:
        got = O.requant_u8(acc, sx, sw, sy, zy, (lo, hi))
        assert np.array_equal(got, np_requant(acc, sx, sw, sy, zy, lo, hi))
        assert (np.diff(got.astype(np.int32)) >= 0).all()  # monotone in acc
    # exact ties: M = 1, sy = 2 -> acc / 2 = k + 0.5 for odd acc, must round to even
    got = O.requant_u8(np.array([1, 3, 5, 7, -1], np.int32), 1.0, 1.0, 2.0, 0)
    assert got.tolist() == [0, 2, 2, 4, 0]


def test_qconv_u8_within_one_lsb_of_reference_float_chain():
    rng = np.random.default_rng(23)
    x = rng.integers(0, 256, (2, 16, 9, 9), dtype=np.uint8)
    w = rng.integers(0, 256, (24, 16, 3, 3), dtype=np.uint8)
    b = rng.integers(-2000, 2000, 24).astype(np.int32)
    args = dict(stride=(1, 1), padding=((1, 1), (1, 1)), fused_clamp=(0.0, 6.0))
    qi = O.qconv2d(x, w, b, 3, 0.0235, 119, 0.004, 0, 0.0235, **args)
    qf = O.qconv2d_float_chain(x, w, b, 3, 0.0235, 119, 0.004, 0, 0.0235, **args)
    d = np.abs(qi.astype(np.int32) - qf.astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() < 0.02
    assert O.cosine(qi, qf) > 0.999


def test_qadd_and_avgpool_against_numpy_fp32():
    rng = np.random.default_rng(29)
    a = rng.integers(0, 256, 4096, dtype=np.uint8)
    b = rng.integers(0, 256, 4096, dtype=np.uint8)
    got = O.qadd(a, b, 3, 0.02, 128, 0.011, 77, 0.031)
    fa = (a.astype(f32) - f32(3)) * f32(0.02)
    fb = (b.astype(f32) - f32(128)) * f32(0.011)
    want = np.clip(np.rint((fa + fb) / f32(0.031) + f32(77)), 0, 255).astype(np.uint8)
    assert np.array_equal(got, want)
    x = rng.integers(0, 256, (2, 5, 7, 7), dtype=np.uint8)
    got = O.qglobal_avgpool(x, 5, 0.02, 9, 0.015)
    xf = O.dequantize(x, 0.02, 5)
    mean = O.reduce_window2d_mean_f32(xf, (7, 7), (1, 1))[:, :, 0, 0]
    assert np.array_equal(got, O.quantize(mean, 0.015, 9, O.U8))


# ----------------------------------------------------------------------------- attention / pack
def test_paged_attention_closed_forms():
    rng = np.random.default_rng(31)
    bsz, hq, hkv, d, blk, nb = 3, 4, 2, 64, 16, 12
    q = rng.standard_normal((bsz, hq, d)).astype(np.float16)
    kc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    vc = rng.standard_normal((nb, hkv, blk, d)).astype(np.float16)
    bt = np.stack([rng.permutation(nb)[:4] for _ in range(bsz)]).astype(np.int32)
    cl = np.array([1, 17, 64], np.int32)
    def dmajor(v):  # the V cache is d-major: [blocks, Hkv, D, block]
        return np.ascontiguousarray(v.transpose(0, 1, 3, 2)).view(np.uint16)
    out = O.paged_attention_decode(q.view(np.uint16), kc.view(np.uint16), dmajor(vc), bt, cl, 0.125)
    # ctx == 1 -> the V row of the first cached token, kv head = h // 2
    for h in range(hq):
        assert np.array_equal(out[0, h], vc[bt[0, 0], h // 2, 0].astype(np.float64))
    # dense float64 softmax attention on gathered K/V
    for b in range(bsz):
        toks = [(bt[b, t // blk], t % blk) for t in range(cl[b])]
        for h in range(hq):
            K = np.stack([kc[p, h // 2, o] for p, o in toks]).astype(np.float64)
            V = np.stack([vc[p, h // 2, o] for p, o in toks]).astype(np.float64)
            s = K @ q[b, h].astype(np.float64) * 0.125
            p_ = np.exp(s - s.max())
            p_ /= p_.sum()
            np.testing.assert_allclose(out[b, h], p_ @ V, rtol=1e-12, atol=1e-12)
    # uniform K -> mean of V
    kc2 = np.ones_like(kc)
    out2 = O.paged_attention_decode(q.view(np.uint16), kc2.view(np.uint16), dmajor(vc), bt, cl, 0.125)
    toks = [(bt[1, t // blk], t % blk) for t in range(17)]
    np.testing.assert_allclose(out2[1, 3], np.mean([vc[p, 1, o].astype(np.float64) for p, o in toks], axis=0), rtol=1e-12, atol=1e-12)
    # relabelling physical blocks (cache permuted together with the table) changes nothing
    perm = rng.permutation(nb)
    inv = np.argsort(perm)
    out3 = O.paged_attention_decode(q.view(np.uint16), kc[perm].view(np.uint16), dmajor(vc[perm]), inv[bt].astype(np.int32), cl, 0.125)
    assert np.array_equal(out, out3)


def test_pack_unpack_definition():
    rng = np.random.default_rng(37)
    x = rng.integers(0, 255, (2, 5, 3, 7), dtype=np.uint8)
    y = O.pack(x, [1], [4])
    assert y.shape == (2, 2, 3, 7, 4)
    assert y[1, 1, 2, 6, 0] == x[1, 4, 2, 6] and (y[:, 1, :, :, 1:] == 0).all()
    assert np.array_equal(O.unpack(y, [1], [4], x.shape), x)
    # NCHW -> NC/32 HW 32 is a reshape + transpose when C divides
    x2 = rng.integers(0, 255, (2, 64, 3, 5), dtype=np.uint8)
    assert np.array_equal(O.pack(x2, [1], [32]), x2.reshape(2, 2, 32, 3, 5).transpose(0, 1, 3, 4, 2))
    # two axes: lanes appended in the order listed
    x3 = rng.standard_normal((6, 10)).astype(np.float32)
    y3 = O.pack(x3, [1, 0], [4, 2])
    assert y3.shape == (3, 3, 4, 2)
    assert y3[2, 1, 3, 1] == x3[2 * 2 + 1, 1 * 4 + 3] and y3[0, 2, 2, 0] == 0
    assert np.array_equal(O.unpack(y3, [1, 0], [4, 2], x3.shape), x3)


# ----------------------------------------------------------------------------- u8 glue: byte tables, concat, resize
def test_unary_tables():
    v = np.arange(256, dtype=np.uint8)
    # the requantisation table is the composition of the (separately pinned) dequantize and quantize
    for zx, sx, zy, sy in [(128, 0.05, 3, 0.023), (7, 0.0235, 131, 0.0041), (0, 0.1, 0, 0.1), (255, 1.0, 0, 0.5)]:
        lut = O.unary_lut(O.LUT_REQUANT, zx, sx, zy, sy)
        assert np.array_equal(lut, O.quantize(O.dequantize(v, sx, zx), sy, zy, O.U8))
    assert np.array_equal(O.unary_lut(O.LUT_REQUANT, 9, 0.25, 9, 0.25), v)            # same params: identity
    # swish: zero maps to the zero point, the table follows the float64 function to <= 1 code and agrees
    # with it almost everywhere, saturates at both ends, and is monotone right of the function's minimum
    zx, sx, zy, sy = 100, 0.08, 12, 0.05
    lut = O.unary_lut(O.LUT_SWISH, zx, sx, zy, sy).astype(np.int64)
    x = (v.astype(np.float64) - zx) * np.float64(np.float32(sx))
    want = np.clip(np.rint(x / (1 + np.exp(-x)) / np.float64(np.float32(sy)) + zy), 0, 255)
    assert lut[zx] == zy and np.abs(lut - want).max() <= 1 and (lut == want).sum() >= 250
    assert lut[-1] == 255 and (np.diff(lut[zx:]) >= 0).all()
    assert lut.min() == zy + round(-0.27846 / 0.05)                                    # min of swish = -0.27846
    parts = O.qconcat([np.full((1, 2, 1, 1), 10, np.uint8), np.full((1, 3, 1, 1), 20, np.uint8)], [(0, 0.5), (10, 0.25)], (1, 0.5))
    assert parts.shape == (1, 5, 1, 1) and parts.ravel().tolist() == [11, 11, 6, 6, 6]


def test_resize_nearest_known_answers():
    """Outputs printed in the ONNX operator documentation of Resize (the operator the reference's
    kernel test compares with through onnxruntime, tests/kernels/test_resize_image.cpp)."""
    a = np.arange(1, 17, dtype=np.float32).reshape(1, 1, 4, 4)
    pat = lambda cols: np.array([[a[0, 0, r, c] for c in cols] for r in cols], np.float32).reshape(1, 1, 8, 8)
    # resize_upsample_sizes_nearest_ceil_half_pixel
    assert np.array_equal(O.resize_nearest(a, 8, 8, O.HALF_PIXEL, O.CEIL), pat([0, 1, 1, 2, 2, 3, 3, 3]))
    # resize_upsample_sizes_nearest_floor_align_corners
    assert np.array_equal(O.resize_nearest(a, 8, 8, O.ALIGN_CORNERS, O.FLOOR), pat([0, 0, 0, 1, 1, 2, 2, 3]))
    # resize_upsample_sizes_nearest_round_prefer_ceil_asymmetric
    assert np.array_equal(O.resize_nearest(a, 8, 8, O.ASYMMETRIC, O.ROUND_PREFER_CEIL), pat([0, 1, 1, 2, 2, 3, 3, 3]))
    # resize_downsample_scales_nearest: [[1,2,3,4],[5,6,7,8]] scaled by 0.6 -> [[1, 3]]
    b = np.arange(1, 9, dtype=np.float32).reshape(1, 1, 2, 4)
    assert O.resize_nearest(b, 1, 2).ravel().tolist() == [1, 3]
    # resize_upsample_scales_nearest: scales (2, 3) repeat every pixel
    c = np.array([[1, 2], [3, 4]], np.uint8).reshape(1, 1, 2, 2)
    assert np.array_equal(O.resize_nearest(c, 4, 6), c.repeat(2, axis=2).repeat(3, axis=3))
    # integer factors in the other modes; identity; element sizes 2 and 4
    rng = np.random.default_rng(41)
    x = rng.integers(0, 255, (2, 3, 5, 7), dtype=np.uint8)
    assert np.array_equal(O.resize_nearest(x, 10, 14, O.ASYMMETRIC, O.FLOOR), x.repeat(2, axis=2).repeat(2, axis=3))
    assert np.array_equal(O.resize_nearest(x, 5, 7, O.PYTORCH_HALF_PIXEL), x)
    assert np.array_equal(O.resize_nearest(x[:, :, ::1, :6], 5, 3, O.ASYMMETRIC, O.FLOOR), x[:, :, :, 0:6:2])
    assert (O.resize_nearest(x, 4, 4, O.TFCROP_AND_RESIZE) == x[:, :, :1, :1]).all()      # roi (0, 0): every index 0
    for dt in (np.uint16, np.float32):
        y = rng.integers(0, 60000, (1, 2, 3, 3)).astype(dt)
        assert np.array_equal(O.resize_nearest(y, 6, 6, O.ASYMMETRIC, O.FLOOR), y.repeat(2, axis=2).repeat(2, axis=3))


def test_maxpool_restatement():
    rng = np.random.default_rng(43)
    x = rng.integers(0, 256, (2, 3, 9, 7), dtype=np.uint8)
    zx, sx, zy, sy = 100, 0.05, 20, 0.07
    xf = O.dequantize(x, sx, zx)
    for k, s, p in ((3, 1, 1), (5, 1, 2), (2, 2, 0), (3, 2, 1)):
        got = O.qmaxpool(x, (k, k), (s, s), ((p, p), (p, p)), zx, sx, zy, sy)
        # float definition: pad with 0.0 (the value the reference folds in for padded positions), window max, quantize
        xp = np.pad(xf, ((0, 0), (0, 0), (p, p), (p, p)), constant_values=0.0)
        win = np.lib.stride_tricks.sliding_window_view(xp, (k, k), axis=(2, 3))[:, :, ::s, ::s].max(axis=(-1, -2))
        assert np.array_equal(got, O.quantize(win.astype(np.float32), sy, zy, O.U8))
    # all-negative window at the border: the padding's 0 wins; in the interior it does not
    neg = np.full((1, 1, 4, 4), 10, np.uint8)
    out = O.qmaxpool(neg, (3, 3), (1, 1), ((1, 1), (1, 1)), 50, 0.1, 50, 0.1)
    assert out[0, 0, 0, 0] == 50 and out[0, 0, 1, 1] == 10 and out[0, 0, 3, 2] == 50
