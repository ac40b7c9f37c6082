"""Shared helpers of the test-suite: seeded synthetic inputs and error metrics."""
from __future__ import annotations

from fractions import Fraction

import numpy as np

SEED = 2024


def rng_for(cfg: int, tensor: int, field: int) -> np.random.Generator:
    """One independent stream per (configuration, tensor, field) so tensors can be generated
    separately: field 0 = g, 1 = w, 2 = m, 3 = v."""
    return np.random.default_rng([SEED, cfg, tensor, field])


def lans_inputs(sizes, cfg=0, g16=False, zero_state=False, loss_scale=1024.0):
    """``g16``: False -> fp32 gradients; True or "float16" -> loss-scaled float16; "bfloat16" ->
    loss-scaled bfloat16 carried as uint16 bit patterns."""
    g, w, m, v = [], [], [], []
    for t, n in enumerate(sizes):
        gt = rng_for(cfg, t, 0).normal(0.0, 1e-3, n)
        if g16 == "bfloat16":
            from oracle.halfs import f32_to_bf16_bits

            g.append(f32_to_bf16_bits((gt * loss_scale).astype(np.float32)))
        else:
            g.append((gt * loss_scale).astype(np.float16) if g16 else gt.astype(np.float32))
        w.append(rng_for(cfg, t, 1).normal(0.0, 0.02, n).astype(np.float32))
        if zero_state:
            m.append(np.zeros(n, np.float32))
            v.append(np.zeros(n, np.float32))
        else:
            m.append(rng_for(cfg, t, 2).normal(0.0, 1e-4, n).astype(np.float32))
            v.append(np.abs(rng_for(cfg, t, 3).normal(0.0, 1e-6, n)).astype(np.float32))
    return g, w, m, v


def max_rel_err(got, want) -> float:
    """Strict per-element relative error max |got-want| / |want| (0 where both agree exactly)."""
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    if got.size == 0:
        return 0.0
    d = np.abs(got - want)
    with np.errstate(divide="ignore", invalid="ignore"):
        r = np.where(d == 0.0, 0.0, d / np.abs(want))
    return float(np.max(r))


def round_to_format(x: Fraction, mantissa_bits: int, emin: int) -> Fraction:
    """Exact round-to-nearest-even of a rational to a binary floating-point grid with
    `mantissa_bits` explicit fraction bits and least normal exponent `emin` (normals and
    subnormals; no overflow handling: callers stay far below the format's maximum)."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    a = abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    elif Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, emin)
    quantum = Fraction(2) ** (e - mantissa_bits)
    q = round(a / quantum)  # Fraction.__round__ rounds half to even
    return sign * q * quantum


def round_to_f32(x: Fraction) -> Fraction:
    return round_to_format(x, 23, -126)


FORMATS = {"float16": (10, -14), "bfloat16": (7, -126), "float32": (23, -126), "float64": (52, -1022)}


def f32_to_fraction(x) -> Fraction:
    return Fraction(float(np.float32(x)))
