"""16-bit float conversions of the mixed-precision LANS path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

The reference trains half-precision models with fp32 master weights: half gradients are widened
with ``_op.group_cast(g_list, "float32")`` before ``raf.op.lans`` (python/raf/optim/lans.py:261-265)
and the updated fp32 weight is narrowed with ``_op.cast(new_w, self.dtype)`` and written over the
model's parameter (lans.py:289-291, :303-305).  Widening is exact; narrowing is a conversion with
round-to-nearest-even (an LLVM ``fptrunc`` for float16; add-and-shift rounding for bfloat16).

NumPy has no bfloat16, so bfloat16 arrays are carried as ``uint16`` bit patterns.

Parity status: pinned (tests/test_oracle_halfs.py) by exhaustive round trips over all 65536
patterns, hand-picked ties, and ``torch``'s own conversions as an independent routine.
"""
from __future__ import annotations

import numpy as np


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """bfloat16 bit patterns (uint16) -> fp32: the pattern is the upper half of the fp32 word."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bfloat16 bit patterns, round to nearest even; NaNs become quiet NaNs with the sign kept."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = ((u.astype(np.uint64) + np.uint64(0x7FFF) + lsb.astype(np.uint64)) >> np.uint64(16)).astype(np.uint16)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    quiet = ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16)
    return np.where(nan, quiet, rounded)


def widen_grad(g: np.ndarray) -> np.ndarray:
    """What ``group_cast(..., "float32")`` does to one gradient: float16 and bfloat16 (as uint16
    patterns) widen exactly, float32 passes through."""
    g = np.asarray(g)
    if g.dtype == np.uint16:
        return bf16_bits_to_f32(g)
    if g.dtype in (np.float16, np.float32):
        return g.astype(np.float32)
    raise TypeError(f"gradient dtype {g.dtype}: expected float32, float16 or uint16 (bfloat16 bits)")


def narrow_weight(w32: np.ndarray, dtype: str) -> np.ndarray:
    """``cast(new_w, dtype)`` of the fp32 weight: ``"float16"`` -> np.float16 array,
    ``"bfloat16"`` -> uint16 bit patterns."""
    w32 = np.asarray(w32, dtype=np.float32)
    if dtype == "float16":
        with np.errstate(over="ignore"):
            return w32.astype(np.float16)
    if dtype == "bfloat16":
        return f32_to_bf16_bits(w32)
    raise TypeError(f"model dtype {dtype!r}: expected 'float16' or 'bfloat16'")
