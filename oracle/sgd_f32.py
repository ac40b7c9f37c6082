"""CPU oracle for ``raf.op.sgd`` -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

The reference computes the momentum-SGD step with a two-stage TVM tensor
expression (python/raf/_tvm_op/sgd.py:13-30):

    v1 = mu * v0 + dx            (:21-24)
    x1 = x0 - learning_rate * v1 (:26-29)

where ``mu`` and ``learning_rate`` are the schema's doubles
(scripts/src_codegen/def_schema.py:675-676) turned into constants of the
tensor dtype by ``tir.const(..., dtype=x0.dtype)`` (sgd.py:18-19), and the
outputs come back as the tuple ``(v1, x1)`` (src/op/declare/optimizer.cc:34-42).
The CPU build target is plain ``llvm`` with no ``-mcpu``
(include/raf/device.h:97-104), i.e. generic x86-64 without FMA, so each of the
four fp32 operations is rounded on its own:

    t  = fl32(mu32 * v0)     v1 = fl32(t + dx)
    s  = fl32(lr32 * v1)     x1 = fl32(x0 - s)

The arithmetic itself lives in TVM (dmlc/tvm, an un-vendored submodule with no
pinned revision), which is absent here, so the no-contraction property cannot
be confirmed by running the reference; it is pinned instead
(tests/test_oracle_sgd.py) by exact rational arithmetic with explicit
roundings, vectors on which a fused multiply-add gives a different bit
pattern, the reference's own float64 closed-form test
(tests/python/op/tvm/test_tvm_loss.py:158-176) and ``torch.optim.SGD``.

Only tests, the smoke check and the benchmark's CPU baseline leg may import
this module.
"""
from __future__ import annotations

import numpy as np


def sgd_step(x0, dx, v0, learning_rate: float, mu: float):
    """Returns ``(v1, x1)`` as new fp32 arrays; inputs are not modified."""
    x0 = np.asarray(x0, dtype=np.float32)
    dx = np.asarray(dx, dtype=np.float32)
    v0 = np.asarray(v0, dtype=np.float32)
    assert x0.shape == dx.shape == v0.shape  # declare/optimizer.cc:29-33
    lr32 = np.float32(learning_rate)
    mu32 = np.float32(mu)
    with np.errstate(all="ignore"):
        t = np.multiply(mu32, v0, dtype=np.float32)
        v1 = np.add(t, dx, dtype=np.float32)
        s = np.multiply(lr32, v1, dtype=np.float32)
        x1 = np.subtract(x0, s, dtype=np.float32)
    return v1, x1


def sgd_step_typed(x0, dx, v0, learning_rate: float, mu: float, dtype: str):
    """The same step in another element type, which is how the reference's compute is written
    (``tir.const(value, dtype=x0.dtype)``, sgd.py:18-19): ``"float64"``, ``"float16"`` or
    ``"bfloat16"`` (arrays of uint16 bit patterns).  The constants are rounded once from double to
    the element type and each of the four operations is rounded to the element type on its own;
    for the 16-bit types through fp32 (widen, operate, round back), as a CPU without half
    arithmetic evaluates them -- with 24 >= 2p + 2 bits in between that equals the correctly
    rounded 16-bit operation.  **Parity unpinned by the reference**: its tests run the op in fp32
    only; pinned here against exact rational arithmetic (tests/test_oracle_sgd.py)."""
    from oracle.halfs import bf16_bits_to_f32, f32_to_bf16_bits

    if dtype == "float64":
        x0, dx, v0 = (np.asarray(a, dtype=np.float64) for a in (x0, dx, v0))
        with np.errstate(all="ignore"):
            v1 = np.float64(mu) * v0 + dx
            x1 = x0 - np.float64(learning_rate) * v1
        return v1, x1
    if dtype == "float16":
        x0, dx, v0 = (np.asarray(a, dtype=np.float16) for a in (x0, dx, v0))
        op = lambda f, a, b: f(a.astype(np.float32), b.astype(np.float32), dtype=np.float32).astype(np.float16)
        lr, m = np.float16(learning_rate), np.float16(mu)  # double -> half, one rounding
        with np.errstate(all="ignore"):
            v1 = op(np.add, op(np.multiply, np.full_like(v0, m), v0), dx)
            x1 = op(np.subtract, x0, op(np.multiply, np.full_like(v1, lr), v1))
        return v1, x1
    if dtype == "bfloat16":
        x0, dx, v0 = (np.asarray(a, dtype=np.uint16) for a in (x0, dx, v0))
        op = lambda f, a, b: f32_to_bf16_bits(f(bf16_bits_to_f32(a), bf16_bits_to_f32(b), dtype=np.float32))
        lr, m = bf16_from_double(learning_rate), bf16_from_double(mu)
        with np.errstate(all="ignore"):
            v1 = op(np.add, op(np.multiply, np.full_like(v0, m), v0), dx)
            x1 = op(np.subtract, x0, op(np.multiply, np.full_like(v1, lr), v1))
        return v1, x1
    raise TypeError(f"dtype {dtype!r}: expected 'float64', 'float16' or 'bfloat16'")


def bf16_from_double(x: float) -> np.uint16:
    """double -> bfloat16 bit pattern with ONE rounding to nearest even (going through fp32 first
    could round twice): the two neighbouring bfloat16 values are compared exactly."""
    from fractions import Fraction

    from oracle.halfs import bf16_bits_to_f32

    lo = int(np.asarray(np.float32(x)).view(np.uint32)) & 0xFFFF0000
    # candidates around the fp32 neighbour: one step of the bfloat16 grid either side
    best = None
    for bits in (lo - 0x10000, lo, lo + 0x10000):
        value = Fraction(float(bf16_bits_to_f32(np.uint16((bits >> 16) & 0xFFFF))))
        err = abs(value - Fraction(x))
        key = (err, (bits >> 16) & 1)  # nearest; ties to the even pattern
        if best is None or key < best[0]:
            best = (key, bits)
    return np.uint16((best[1] >> 16) & 0xFFFF)


def sgd_list_step(x_list, dx_list, v_list, learning_rate: float, mu: float, model_dtype=None):
    """What the reference's traced optimizer computes per parameter (python/raf/optim/
    sgd.py:187-215): ``dx`` widened to fp32 (``cast(dxi, "float32")``, exact), then

        v <- fl32(fl32(momentum * v) + dx)           add(multiply(momentum, v), dx, out=v)
        w <- fl32(w - fl32(learning_rate * v))       subtract(w, multiply(lr, v), out=w)

    -- the same four roundings as ``raf.op.sgd``, ``momentum`` and ``learning_rate`` being fp32
    arrays (sgd.py:106-107) -- and, for a half-precision model, the parameter as
    ``cast(new_w, dtype)``.  Gradients may be float32, float16 or bfloat16 bit patterns
    (uint16).  Returns ``(xs, vs, ps)`` as new arrays; ``ps`` is None without ``model_dtype``."""
    from oracle.halfs import narrow_weight, widen_grad

    xs, vs = [], []
    for x0, dx, v0 in zip(x_list, dx_list, v_list):
        g = widen_grad(dx).reshape(np.asarray(x0).shape)
        v1, x1 = sgd_step(x0, g, v0, learning_rate, mu)
        xs.append(x1)
        vs.append(v1)
    ps = [narrow_weight(x, model_dtype) for x in xs] if model_dtype else None
    return xs, vs, ps
