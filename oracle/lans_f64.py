"""CPU oracle for ``raf.op.lans`` -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A float64 NumPy transcription of the LANS update rule that the reference
implements in fp32 CUDA.  Only tests, the smoke check and the benchmark's CPU
baseline leg may import this module; the product path never does.

What is transcribed, and from where (paths relative to the reference tree):

* host scalars ``step``, ``bias_correction{1,2}``, ``beta3``:
  src/op/dialect/cuda/lans.cc:94-109
* hyper-parameters arrive as C ``float``/``int``/``bool`` schema fields, so
  they are rounded to fp32 before any arithmetic:
  scripts/src_codegen/def_schema.py:678-694
* per-tensor L2 norm = sqrt(sum of squares): multi_tensor_lans.cu:95-185
* stage 1 (moments and the two update directions), both weight-decay modes:
  src/op/dialect/cuda/kernels/multi_tensor_lans.cu:283-307 (and :264-269 for
  the ``weight_decay == 0`` case where the weight is treated as 0)
* stage 2 (trust ratios and the weight update): multi_tensor_lans.cu:346-352,
  :386
* phase order (norm g, norm w, stage 1, norm u_m, norm u_g, stage 2):
  multi_tensor_lans.cu:420-447
* tensor list layout ``[g..., w..., m..., v...]``: python/raf/optim/lans.py:89

Deliberate, documented differences from the reference *behaviour* (not from
its rule): the reference writes ``u_m`` over the gradient and keeps ``u_g`` in
a scratch buffer whose per-tensor regions overlap for three or more tensors
(lans.cc:116-119); the oracle follows the rule, keeps ``g`` intact and gives
every tensor its own ``u_g``.

Arithmetic: every operation after the fp32 rounding of the scalars is float64.
``(1 - beta2)`` and ``beta3 = 1 - beta1`` are fp32 subtractions exactly as in
the reference (both are exact by Sterbenz' lemma for the usual betas).

Parity status: pinned (tests/test_oracle_lans.py) by the step-1 closed form,
``torch.optim.Adam`` moments/direction, an independent scalar brute force,
exact-arithmetic known answers, and invariants (tensor independence,
||dw|| bound, power-of-two gradient scaling, zero-norm special cases).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence, Tuple

import math

import numpy as np

from oracle.halfs import narrow_weight, widen_grad


def f32(x) -> float:
    """Round a Python number to fp32 and return it as a Python float."""
    return float(np.float32(x))


@dataclass(frozen=True)
class LansHParams:
    """Schema fields of ``raf.op.lans`` (def_schema.py:685-693) with the
    defaults of ``raf.optim.LANS`` (python/raf/optim/lans.py:44-55)."""

    learning_rate: float = 1e-3
    beta1: float = 0.9
    beta2: float = 0.999
    eps: float = 1e-6
    bias_correction: int = 1
    weight_decay: float = 0.01
    grad_averaging: int = 1
    mode: int = 1  # 1 = decoupled weight decay, 0 = L2 on the scaled gradient
    normalize_grad: bool = True
    # Extension used by the fp16-gradient configuration: the gradient is
    # multiplied by this fp32 factor (e.g. 1/1024) before anything else.
    grad_unscale: float = 1.0


@dataclass(frozen=True)
class LansScalars:
    lr: float
    beta1: float
    beta2: float
    one_minus_beta2: float
    beta3: float
    eps: float
    wd: float
    bc1: float
    bc2: float


def lans_scalars(hp: LansHParams, step) -> LansScalars:
    """Host-side scalars, lans.cc:94-109.  ``step`` is the value held by the
    0-d fp32 step tensor; it is truncated to int as ``(int)fstep`` does."""
    lr, b1, b2 = f32(hp.learning_rate), f32(hp.beta1), f32(hp.beta2)
    eps, wd = f32(hp.eps), f32(hp.weight_decay)
    istep = int(np.float32(step))
    bc1 = bc2 = 1.0
    if int(hp.bias_correction) == 1:
        # std::pow(float, int) promotes to double; the result is stored in a float
        bc1 = f32(1.0 - b1 ** istep)
        bc2 = f32(1.0 - b2 ** istep)
    beta3 = 1.0
    if int(hp.grad_averaging) == 1:
        beta3 = float(np.float32(1.0) - np.float32(b1))
    omb2 = float(np.float32(1.0) - np.float32(b2))
    return LansScalars(lr, b1, b2, omb2, beta3, eps, wd, bc1, bc2)


def grad_to_f64(g: np.ndarray, hp: LansHParams) -> np.ndarray:
    """Gradient ingest: float32, float16 or bfloat16 (uint16 bit patterns) ->
    fp32 exactly as ``group_cast`` widens it (python/raf/optim/lans.py:261-265),
    times the fp32 unscale factor (one fp32 rounding; exact for powers of
    two), then float64."""
    g32 = widen_grad(g) * np.float32(hp.grad_unscale)
    return g32.astype(np.float64)


def l2norm(x: np.ndarray) -> float:
    x = np.asarray(x, dtype=np.float64).ravel()
    return float(np.sqrt(np.dot(x, x)))


def lans_directions(g, w, m, v, sc: LansScalars, hp: LansHParams, repeat: int = 1):
    """Stage 1 for one tensor; float64 in, float64 out.
    Returns (m1, v1, u_m, u_g, grad_norm).  ``repeat``: see lans_tensor_step."""
    gn = l2norm(g) * math.sqrt(repeat)
    with np.errstate(invalid="ignore"):  # an overflowed gradient gives inf / inf = NaN, as on the device
        sg = g / (gn + sc.eps) if (hp.normalize_grad and gn != 0.0) else g
    wp = w if sc.wd != 0.0 else np.zeros_like(w)
    if int(hp.mode) == 0:
        sg = sg + sc.wd * wp
    m1 = m * sc.beta1 + sc.beta3 * sg
    v1 = v * sc.beta2 + sc.one_minus_beta2 * sg * sg
    den = np.sqrt(v1 / sc.bc2) + sc.eps
    with np.errstate(invalid="ignore", divide="ignore"):  # 0 / 0 (eps = 0) propagates NaN, as the rule says
        if int(hp.mode) == 0:
            u_m = (m1 / sc.bc1) / den
            u_g = sg / den
        else:
            sp = sc.wd * wp
            u_m = (m1 / sc.bc1) / den + sp
            u_g = sg / den + sp
    return m1, v1, u_m, u_g, gn


def lans_tensor_step(g, w, m, v, step, hp: LansHParams, repeat: int = 1):
    """One LANS step on one tensor.  Inputs are used at float64 (g through
    ``grad_to_f64``); returns float64 ``(w1, m1, v1, norms)`` where ``norms`` =
    (||g||, ||w||, ||u_m||, ||u_g||).

    ``repeat`` = k > 1 stands for a tensor that consists of k copies of the
    given arrays back to back (a way to state what the step does to a tensor
    of billions of elements without holding it): each of its norms is sqrt(k)
    times the pattern's, and every copy gets the pattern's result."""
    sc = lans_scalars(hp, step)
    g64 = grad_to_f64(g, hp).ravel()
    w64 = np.asarray(w, dtype=np.float64).ravel()
    m64 = np.asarray(m, dtype=np.float64).ravel()
    v64 = np.asarray(v, dtype=np.float64).ravel()
    rep = math.sqrt(repeat)
    pn = l2norm(w64) * rep
    m1, v1, u_m, u_g, gn = lans_directions(g64, w64, m64, v64, sc, hp, repeat)
    un_m, un_g = l2norm(u_m) * rep, l2norm(u_g) * rep
    r_m = sc.lr * (pn / un_m) if (un_m != 0.0 and pn != 0.0) else sc.lr
    r_g = sc.lr * (pn / un_g) if (un_g != 0.0 and pn != 0.0) else sc.lr
    r_m *= sc.beta1
    r_g *= sc.beta3
    w1 = w64 - r_m * u_m - r_g * u_g
    return w1, m1, v1, (gn, pn, un_m, un_g)


def lans_step(
    g_list: Sequence[np.ndarray],
    w_list: Sequence[np.ndarray],
    m_list: Sequence[np.ndarray],
    v_list: Sequence[np.ndarray],
    step,
    hp: LansHParams = LansHParams(),
    state_dtype=np.float32,
) -> Tuple[List[np.ndarray], List[np.ndarray], List[np.ndarray], np.ndarray]:
    """One LANS step over a tensor list.  ``state_dtype=np.float32`` stores the
    new w/m/v the way the operator's fp32 tensors do (one rounding of the
    float64 result); ``np.float64`` keeps the state unrounded.  Returns new
    lists plus an ``[n, 4]`` float64 array of the per-tensor norms."""
    n = len(w_list)
    assert len(g_list) == len(m_list) == len(v_list) == n
    ws, ms, vs = [], [], []
    norms = np.zeros((n, 4), dtype=np.float64)
    for t in range(n):
        w1, m1, v1, nr = lans_tensor_step(g_list[t], w_list[t], m_list[t], v_list[t], step, hp)
        shape = np.asarray(w_list[t]).shape
        ws.append(w1.astype(state_dtype).reshape(shape))
        ms.append(m1.astype(state_dtype).reshape(shape))
        vs.append(v1.astype(state_dtype).reshape(shape))
        norms[t] = nr
    return ws, ms, vs, norms


def lans_step_dynamic_scale(g_list, w_list, m_list, v_list, step, hp: LansHParams, inv_scale, found_inf,
                            state_dtype=np.float32):
    """The step under dynamic loss scaling (an extension of this build; the
    reference unscales with graph ops in front of the optimizer and has no
    skip): the gradient is multiplied by the fp32 value ``inv_scale`` instead
    of ``hp.grad_unscale``, and a non-zero ``found_inf`` skips the step, i.e.
    w, m, v come back as they went in (norms are then reported as NaN)."""
    if float(np.float32(found_inf)) != 0.0:
        n = len(w_list)
        keep = lambda xs: [np.array(x, copy=True) for x in xs]
        return keep(w_list), keep(m_list), keep(v_list), np.full((n, 4), np.nan)
    import dataclasses

    return lans_step(g_list, w_list, m_list, v_list, step,
                     dataclasses.replace(hp, grad_unscale=float(np.float32(inv_scale))), state_dtype)


def lans_mixed_step(g_list, w_list, m_list, v_list, step, hp: LansHParams = LansHParams(),
                    model_dtype: str = "float16"):
    """The mixed-precision step of the reference's wrapper: ``lans_step`` on
    the fp32 master weights, then the model's half-precision parameters as
    ``cast(new_w, dtype)`` of the *stored fp32* weight (python/raf/optim/
    lans.py:289-291, :303-305).  Returns ``(ws, ms, vs, ps, norms)``; ``ps``
    are float16 arrays or bfloat16 bit patterns (uint16)."""
    ws, ms, vs, norms = lans_step(g_list, w_list, m_list, v_list, step, hp, np.float32)
    ps = [narrow_weight(w, model_dtype) for w in ws]
    return ws, ms, vs, ps, norms


def lans_flat_list_step(tensor_list, step, hp: LansHParams = LansHParams(), state_dtype=np.float32):
    """Same, on the operator's flat list ``[g..., w..., m..., v...]``
    (python/raf/optim/lans.py:89); returns the flat output list in the same
    order with ``g`` passed through untouched."""
    assert len(tensor_list) % 4 == 0  # declare/optimizer.cc:49
    n = len(tensor_list) // 4
    g, w, m, v = (tensor_list[i * n:(i + 1) * n] for i in range(4))
    ws, ms, vs, _ = lans_step(g, w, m, v, step, hp, state_dtype)
    return list(g) + ws + ms + vs
