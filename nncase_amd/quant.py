"""Host-side quantisation parameter maths of the `hip` target.

Mirrors, name for name, the reference's
  QuantUtility.GetQuantParam / FixupRange   src/Nncase.Core/Utilities/QuantUtility.cs:41-97
  Quantizer.FixUpRange (calibrator variant) src/Nncase.Quantization/Quantization/Quantizer.cs:358-386
  RangeOf evaluator                         src/Nncase.Evaluator/Math/RangeOf.cs:20-35
  ValueRange.Union                          running min/max over calibration samples, Quantizer.cs:389-408
C# evaluates `range.Max - range.Min` on floats and everything around it on doubles, and
Math.Round is round-half-to-even; numpy scalars reproduce both.
"""
from __future__ import annotations

import enum
from typing import Iterable, Tuple

import numpy as np

f32 = np.float32


class QuantMode(enum.IntEnum):
    """src/Nncase.Core/Quantization/QuantMode (UnsignedMode / SignedSymmetricMode / SignedAsymmetricMode)."""
    UnsignedMode = 0
    SignedSymmetricMode = 1
    SignedAsymmetricMode = 2


def fixup_range(rng: Tuple[float, float], symmetric: bool = False) -> Tuple[np.float32, np.float32]:
    lo, hi = f32(rng[0]), f32(rng[1])
    if symmetric:
        r = max(max(abs(lo), abs(hi)), f32(0.01))
        return f32(-r), f32(r)
    hi = max(f32(0), hi)
    lo = min(f32(0), lo)
    r = f32(hi - lo)
    if r == 0:
        r = f32(0.1)
    elif r < f32(0.01):
        r = f32(0.01)
    return lo, f32(lo + r)


def calib_fixup_range(rng: Tuple[float, float], symmetric: bool = False) -> Tuple[np.float32, np.float32]:
    lo, hi = f32(rng[0]), f32(rng[1])
    if symmetric:
        r = max(f32(0.01), max(abs(lo), abs(hi)))
        return f32(-r), f32(r)
    if hi < 0:
        hi = f32(0)
    if lo > 0:
        lo = f32(0)
    r = f32(hi - lo)
    if r < f32(1e-6):
        r = f32(0.1)
    return lo, f32(lo + r)


def get_quant_param(rng: Tuple[float, float], bits: int = 8, mode: QuantMode = QuantMode.UnsignedMode) -> Tuple[int, np.float32]:
    """Returns (zero_point, scale)."""
    lo, hi = fixup_range(rng, mode == QuantMode.SignedSymmetricMode)
    if mode == QuantMode.UnsignedMode:
        qmin, qmax = 0.0, float((1 << bits) - 1)
    elif mode == QuantMode.SignedSymmetricMode:
        qmin, qmax = float(-(1 << (bits - 1)) + 1), float((1 << (bits - 1)) - 1)
    elif mode == QuantMode.SignedAsymmetricMode:
        qmin, qmax = float(-(1 << (bits - 1))), float((1 << (bits - 1)) - 1)
    else:
        raise ValueError("Invalid QuantMode")
    span = np.float64(f32(hi - lo))
    scale = span / (qmax - qmin)
    bias = np.round(np.float64(lo) * (qmin - qmax) / span) + qmin  # np.round: half to even, like Math.Round
    return int(bias), f32(scale)


def range_of(x: np.ndarray) -> Tuple[np.float32, np.float32]:
    """Finite min/max, with the evaluator's initial values when nothing is finite."""
    x = np.asarray(x, np.float32)
    fin = x[np.isfinite(x)]
    if fin.size == 0:
        return f32(np.finfo(np.float32).max), f32(np.finfo(np.float32).min)
    return f32(fin.min()), f32(fin.max())


def union(a: Tuple[float, float], b: Tuple[float, float]) -> Tuple[np.float32, np.float32]:
    return f32(min(a[0], b[0])), f32(max(a[1], b[1]))


def calibrate_range(samples: Iterable[np.ndarray]) -> Tuple[np.float32, np.float32]:
    """NoClip calibration: union of per-sample finite ranges, then the calibrator's FixUpRange."""
    rng = None
    for s in samples:
        r = range_of(s)
        rng = r if rng is None else union(rng, r)
    if rng is None:
        raise ValueError("no calibration samples")
    return calib_fixup_range(rng)


def quantize_weights(w: np.ndarray, bits: int = 8) -> Tuple[np.ndarray, int, np.float32]:
    """Per-tensor asymmetric u8 weights: GetQuantParam on (min(0,wmin), max(0,wmax)), then the
    native quantize formula on the host (constants are folded at compile time in the reference)."""
    w = np.asarray(w, np.float32)
    zp, scale = get_quant_param((w.min(), w.max()), bits, QuantMode.UnsignedMode)
    q = np.clip(np.rint(w / scale + f32(zp)), 0, 255).astype(np.uint8)
    return q, zp, scale
