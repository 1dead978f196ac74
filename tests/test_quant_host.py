"""Host-side quantisation-parameter maths (nncase_amd.quant) against the reference's literal
expectations and against the oracle's independent restatement."""
import json
import os

import numpy as np

from nncase_amd import quant
from oracle import oracle as O

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
f32 = np.float32


def test_literals():
    for g in GOLD["K4_get_quant_param"] + [GOLD["K6_quant_param_of"]]:
        zp, sc = quant.get_quant_param(tuple(g["range"]), g["bits"], quant.QuantMode[g["mode"]])
        assert zp == g["zero_point"] and sc == f32(g["scale"])
    for g in GOLD["K5_fixup_range"]:
        assert quant.fixup_range(tuple(g["range"]), g["symmetric"]) == (f32(g["expected"][0]), f32(g["expected"][1]))


def test_matches_oracle_on_random_ranges():
    rng = np.random.default_rng(0)
    for _ in range(3000):
        lo, hi = np.sort(rng.standard_normal(2).astype(f32) * f32(10 ** rng.uniform(-4, 3)))
        for mode in quant.QuantMode:
            assert quant.get_quant_param((lo, hi), 8, mode) == O.get_quant_param(lo, hi, 8, int(mode))
        assert quant.fixup_range((lo, hi)) == O.fixup_range(lo, hi)
        assert quant.calib_fixup_range((lo, hi)) == O.calib_fixup_range(lo, hi)


def test_calibration_union_and_weight_quantisation():
    samples = [np.array([0.5, 2.0, np.inf], f32), np.array([-1.0, 1.0, np.nan], f32)]
    assert quant.calibrate_range(samples) == (f32(-1.0), f32(2.0))
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((8, 4, 3, 3)) * 0.05).astype(f32)
    q, zp, sc = quant.quantize_weights(w)
    assert (zp, sc) == O.get_quant_param(w.min(), w.max())
    assert np.array_equal(q, O.quantize(w, sc, zp, O.U8))
