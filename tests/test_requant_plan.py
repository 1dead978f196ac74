"""The u8 epilogues replace the three-rounding requantisation (quantize.cpp:36-43 on Conv2D's clamped fp32
value) by one FMA wherever the library's host-side search proves both maps equal.  These tests need no GPU:
they pin the search against the independent C restatement in oracle/ -- densely around every step of the
staircase, on random accumulators and at the ends of the int32 range -- for the quant params of real layers
and for awkward ones (coarse and fine scales, clamps, zero points at both ends)."""
import numpy as np
import pytest

from nncase_amd import runtime as rt
from nncase_amd.runtime import qp
from oracle import oracle as O

f32 = np.float32
FULL = (-rt.FLT_MAX, rt.FLT_MAX)

CASES = [  # sx, sw, sy, zy, clamp
    (0.0235, 0.0041, 0.0118965, 0, (0.0, 6.0)),          # ReLU6 expansion of a MobileNetV2 block
    (0.0192766, 0.0067, 0.0180625, 135, FULL),           # linear projection
    (0.05, 0.0011367, 0.0617623, 139, FULL),             # ~1000 accumulators per code: usually no FMA form
    (1.0, 1.0, 1.0, 0, FULL), (1.0, 1.0, 2.0, 3, FULL),  # exact ties at every step
    (0.5, 0.5, 0.125, 128, (-3.0, 3.0)), (0.02, 0.004, 0.7, 255, FULL), (0.02, 0.004, 1e-4, 0, (0.0, 6.0)),
    (3.1e-3, 7.7e-3, 0.0313, 17, (-0.4, 2.2)), (1e-3, 1e-3, 2.3e-5, 200, (-1.0, 0.001)),
]


def staircase_points(sx, sw, sy, zy, clamp, rng):
    """Accumulators that matter: a dense run over the un-saturated range (or around its steps when it is long),
    random ones, and the int32 extremes."""
    m = float(f32(sx) * f32(sw))
    centre = lambda code: (code - zy) * float(sy) / m
    lo, hi = centre(-2), centre(258)
    pts = [np.array([-2**31 + 1, -2**31 + 2, -1, 0, 1, 2**31 - 2, 2**31 - 1], np.int64)]
    if hi - lo < 3e6:
        pts.append(np.arange(int(lo), int(hi) + 1, dtype=np.int64))
    else:
        for code in range(-1, 258):                      # +-600 accumulators around every half-integer code
            c = int(centre(code + 0.5))
            pts.append(np.arange(c - 600, c + 601, dtype=np.int64))
    pts.append(rng.integers(int(lo * 1.5) - 10, int(hi * 1.5) + 10, 200000))
    v = np.concatenate(pts)
    return np.unique(v[(v > -2**31) & (v < 2**31)]).astype(np.int32)


@pytest.mark.parametrize("sx,sw,sy,zy,clamp", CASES)
def test_picked_form_equals_the_reference_sequence(sx, sw, sy, zy, clamp):
    rng = np.random.default_rng(int(zy) + 7)
    acc = staircase_points(sx, sw, sy, zy, clamp, rng)
    got, form = rt.requant_host(acc, sx, sw, qp(zy, sy), clamp)
    want = O.requant_u8(acc, sx, sw, sy, zy, clamp)
    bad = got != want
    assert not bad.any(), f"form {form}: {bad.sum()} of {acc.size} differ, first at acc={acc[bad][0]}: {got[bad][0]} vs {want[bad][0]}"
    assert np.all(np.diff(want.astype(np.int32)) >= 0) and len(np.unique(want)) >= 2     # a staircase, not a constant


@pytest.mark.parametrize("sx,sw,sy,zy,clamp", CASES)
def test_conversion_free_form_equals_the_reference_sequence(sx, sw, sy, zy, clamp):
    """Where the search finds the form on sums started from 0x4B400000 (their bits read as a float), it gives the reference's
    bytes on every accumulator of the range it vouches for: densely around every step, on random ones, and at the range's ends
    (far beyond 2^22, where the float no longer equals 12582912 + acc but still grows with it)."""
    rng = np.random.default_rng(int(zy) + 11)
    acc = staircase_points(sx, sw, sy, zy, clamp, rng)
    res = rt.requant_host_magic(acc, sx, sw, qp(zy, sy), clamp)
    if res is None:
        pytest.skip("no conversion-free pair for these quant params (the kernels use the other forms)")
    got, m1, m2, limit = res
    assert limit >= 2**29
    acc = np.concatenate([acc[np.abs(acc.astype(np.int64)) <= limit], np.array([-limit, -limit + 1, -2**22 - 1, -2**22, 2**22 - 1, 2**22, limit - 1, limit], np.int32)])
    got = rt.requant_host_magic(acc, sx, sw, qp(zy, sy), clamp)[0]
    want = O.requant_u8(acc, sx, sw, sy, zy, clamp)
    bad = got != want
    assert not bad.any(), f"{bad.sum()} of {acc.size} differ, first at acc={acc[bad][0]}: {got[bad][0]} vs {want[bad][0]}"
    # what the pair is: m1 with two spare mantissa bits, m2 = zy - 12582912 * m1 without rounding
    assert (np.array([m1], f32).view(np.uint32)[0] & 3) == 0
    assert float(f32(m2)) == float(zy) - 12582912.0 * float(f32(m1))


def test_conversion_free_form_exists_for_the_layers_it_is_meant_for():
    # a ReLU6 expansion, a linear projection and a depthwise layer of MobileNetV2 (calibrated scales)
    found = [rt.requant_host_magic(np.zeros(1, np.int32), sx, sw, qp(zy, sy), clamp) is not None
             for sx, sw, sy, zy, clamp in ((0.0235, 0.0041, 0.0118965, 0, (0.0, 6.0)), (0.0192766, 0.0067, 0.0180625, 135, FULL),
                                           (0.0235294, 0.0125, 0.0235294, 0, (0.0, 6.0)), (0.02, 0.011, 0.0235, 0, (0.0, 6.0)))]
    assert sum(found) >= 2, found


def test_fma_form_is_found_for_typical_layers_and_is_what_it_says():
    found, c1, c2 = rt.requant_plan(0.0235, 0.0041, qp(0, 0.0118965), (0.0, 6.0))
    assert found and abs(c1 / (float(f32(0.0235) * f32(0.0041)) / 0.0118965) - 1) < 1e-5 and abs(c2) < 1e-3
    # the constants reproduce the bytes with plain arithmetic (exact rational FMA, rounded once to float32)
    from fractions import Fraction
    acc = np.arange(-50, 1500, dtype=np.int32)
    want = O.requant_u8(acc, 0.0235, 0.0041, 0.0118965, 0, (0.0, 6.0))
    qhi = float(f32(f32(f32(6.0) / f32(0.0118965)) + f32(0)))
    for a, w in zip(acc[::37], want[::37]):
        exact = Fraction(int(a)) * Fraction(float(f32(c1))) + Fraction(float(f32(c2)))
        u = float(f32(float(exact)))                      # |exact| < 2^24 * 2^-8: the double is exact enough to round once
        u = min(max(u, 0.0), min(qhi, 255.0))
        assert int(np.rint(f32(u))) == int(w)
    assert rt.requant_plan(1.0, 1.0, qp(0, 1.0))[0]       # identity scale: trivially a line


def test_out_of_range_scales_are_refused():
    with pytest.raises(rt.HipError):
        rt.requant_plan(1.0, 1.0, qp(0, 1e-30))


def test_output_zero_points_outside_u8_are_refused():
    # every u8 epilogue (dense, depthwise, the three stages of the fused block) is set up through the same check
    import errno
    for zp in (-1, 256, 1 << 20):
        with pytest.raises(rt.HipError) as e:
            rt.requant_plan(0.02, 0.004, qp(zp, 0.05))
        assert e.value.code == -errno.EINVAL
    assert rt.requant_plan(0.02, 0.004, qp(255, 0.05))[0] in (True, False)
