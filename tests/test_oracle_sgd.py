"""Pins of the SGD oracle (oracle/sgd_f32.py and the C restatement).  Nothing here retypes the
oracle's NumPy expression: the checks are exact rational arithmetic with explicit fp32 rounding,
fused-vs-unfused discrimination, the reference's own closed-form test, and torch.optim.SGD."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import sgd_f32
from tests.helpers import f32_to_fraction, round_to_f32


def _rational_sgd(x0, dx, v0, lr, mu, fused=False):
    lr32, mu32 = f32_to_fraction(lr), f32_to_fraction(mu)
    v1, x1 = [], []
    for a, d, b in zip(x0, dx, v0):
        a, d, b = Fraction(float(a)), Fraction(float(d)), Fraction(float(b))
        if fused:
            nv = round_to_f32(mu32 * b + d)
            nx = round_to_f32(a - lr32 * nv)
        else:
            nv = round_to_f32(round_to_f32(mu32 * b) + d)
            nx = round_to_f32(a - round_to_f32(lr32 * nv))
        v1.append(float(nv))
        x1.append(float(nx))
    return np.array(v1, np.float32), np.array(x1, np.float32)


def _inputs(n, seed, scale_v=1e-3):
    r = np.random.default_rng(seed)
    return (r.normal(0, .02, n).astype(np.float32), r.normal(0, 1e-3, n).astype(np.float32),
            r.normal(0, scale_v, n).astype(np.float32))


def test_round_to_f32_helper_matches_numpy():
    r = np.random.default_rng(1)
    for x in list(r.normal(0, 1, 200)) + [1e-40, -3e-39, 2.0 ** -149 * 0.5, 2.0 ** -149 * 1.5, 1 + 2.0 ** -24]:
        assert float(round_to_f32(Fraction(float(x)))) == float(np.float32(x))


def test_oracle_equals_exact_rational_four_roundings():
    x0, dx, v0 = _inputs(400, 7)
    v1, x1 = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    ev, ex = _rational_sgd(x0, dx, v0, 0.01, 0.9)
    assert np.array_equal(v1.view(np.uint32), ev.view(np.uint32))
    assert np.array_equal(x1.view(np.uint32), ex.view(np.uint32))


def test_oracle_is_not_the_fused_evaluation():
    # a fused multiply-add rounds once; on enough random inputs it must disagree somewhere,
    # and the oracle must side with the unfused result everywhere
    x0, dx, v0 = _inputs(2000, 11)
    v1, x1 = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    fv, fx = _rational_sgd(x0, dx, v0, 0.01, 0.9, fused=True)
    uv, ux = _rational_sgd(x0, dx, v0, 0.01, 0.9, fused=False)
    assert (fv != uv).any() and (fx != ux).any(), "vectors do not discriminate fused from unfused"
    assert np.array_equal(v1, uv) and np.array_equal(x1, ux)


def test_denormals_and_specials_exact():
    tiny = np.float32(2.0 ** -140)
    x0 = np.array([tiny, -tiny, 0.0, -0.0, 1.0, 3e-39], np.float32)
    dx = np.array([tiny, 3 * tiny, 0.0, -0.0, np.float32(2.0 ** -149), -1e-39], np.float32)
    v0 = np.array([tiny, -5 * tiny, -0.0, 0.0, 7 * tiny, 2e-39], np.float32)
    v1, x1 = sgd_f32.sgd_step(x0, dx, v0, 0.5, 0.75)
    ev, ex = _rational_sgd(x0, dx, v0, 0.5, 0.75)
    assert np.array_equal(v1, ev) and np.array_equal(x1, ex)  # no flush to zero
    assert (v1 != 0).sum() >= 4
    inf = sgd_f32.sgd_step(np.array([1.0, np.inf], np.float32), np.array([np.nan, 1.0], np.float32),
                           np.array([0.0, 0.0], np.float32), 0.1, 0.9)
    assert np.isnan(inf[0][0]) and np.isnan(inf[1][0]) and np.isposinf(inf[1][1])


def test_hyperparameters_rounded_once_to_fp32():
    # mu = 0.9 is not representable: the rule uses fl32(0.9), not the double
    x0, dx, v0 = np.float32([0.0]), np.float32([0.0]), np.float32([1.0])
    v1, _ = sgd_f32.sgd_step(x0, dx, v0, 0.0, 0.9)
    assert v1[0] == np.float32(0.9) and float(v1[0]) != 0.9


def test_reference_closed_form_kat():
    # the reference's op test (tests/python/op/tvm/test_tvm_loss.py:158-176): float64 closed form,
    # rtol = atol = 1e-4, shape 4x4, random mu, lr 0.01, outputs ordered (v1, x1)
    r = np.random.default_rng(0)
    x0 = r.standard_normal((4, 4)).astype("float32")
    dx = r.standard_normal((4, 4)).astype("float32")
    v0 = r.standard_normal((4, 4)).astype("float32")
    mu = r.standard_normal(1)[0]
    n_v1 = mu * v0 + dx
    n_x1 = x0 - 0.01 * n_v1
    m_v1, m_x1 = sgd_f32.sgd_step(x0, dx, v0, 0.01, mu)
    assert m_v1.shape == (4, 4) and m_v1.dtype == np.float32
    np.testing.assert_allclose(m_v1, n_v1, 1e-4, 1e-4)
    np.testing.assert_allclose(m_x1, n_x1, 1e-4, 1e-4)


def test_against_torch_sgd_trajectory():
    # tests/python/optim/test_sgd.py:80-125 compares with torch.optim.SGD(lr=.1, momentum=.01), 1e-4
    r = np.random.default_rng(3)
    x = r.normal(0, 1, 257).astype(np.float32)
    v = np.zeros_like(x)
    p = torch.nn.Parameter(torch.from_numpy(x.copy()))
    opt = torch.optim.SGD([p], lr=0.1, momentum=0.01, dampening=0.0)
    for _ in range(10):
        g = r.normal(0, 1, 257).astype(np.float32)
        p.grad = torch.from_numpy(g.copy())
        opt.step()
        v, x = sgd_f32.sgd_step(x, g, v, 0.1, 0.01)
        np.testing.assert_allclose(x, p.detach().numpy(), rtol=2e-6, atol=1e-7)


def test_inputs_untouched_and_shape_check():
    x0, dx, v0 = _inputs(16, 5)
    keep = (x0.copy(), dx.copy(), v0.copy())
    sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    assert all(np.array_equal(a, b) for a, b in zip((x0, dx, v0), keep))
    with pytest.raises(AssertionError):
        sgd_f32.sgd_step(x0, dx[:8], v0, 0.01, 0.9)


@pytest.mark.parametrize("n", [0, 1, 3, 1000, 70001])
def test_c_restatement_bit_equal(c_oracle, n):
    x0, dx, v0 = _inputs(n, 13 + n)
    a = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    for threads in (1, 4):
        b = c_oracle.sgd_step(x0, dx, v0, 0.01, 0.9, threads=threads)
        assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32))
        assert np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))


def test_list_step_is_the_op_per_parameter_with_exact_widening_and_rne_copies():
    """The traced optimizer's per-parameter sequence (python/raf/optim/sgd.py:187-215): the same
    four roundings as the op on the widened gradient, then cast(new_w, dtype)."""
    import torch
    from oracle import halfs

    rng = np.random.default_rng(9)
    xs = [rng.normal(0, 0.02, n).astype(np.float32) for n in (7, 1000)]
    vs = [rng.normal(0, 1e-3, n).astype(np.float32) for n in (7, 1000)]
    d32 = [rng.normal(0, 1e-3, n).astype(np.float32) for n in (7, 1000)]
    for name, tdt, grads in (("float16", torch.float16, [d.astype(np.float16) for d in d32]),
                             ("bfloat16", torch.bfloat16, [halfs.f32_to_bf16_bits(d) for d in d32])):
        nx, nv, ps = sgd_f32.sgd_list_step(xs, grads, vs, 0.01, 0.9, name)
        for x0, g, v0, x1, v1, p in zip(xs, grads, vs, nx, nv, ps):
            wide = torch.from_numpy(g.view(np.int16)).view(tdt).float().numpy()  # torch's own widening
            ev, ex = sgd_f32.sgd_step(x0, wide, v0, 0.01, 0.9)
            assert np.array_equal(ev, v1) and np.array_equal(ex, x1)
            t = torch.from_numpy(x1).to(tdt).view(torch.int16).numpy().view(np.uint16)
            assert np.array_equal(p.view(np.uint16), t)
    nx, nv, ps = sgd_f32.sgd_list_step(xs, d32, vs, 0.01, 0.9)
    assert ps is None and np.array_equal(nx[1], sgd_f32.sgd_step(xs[1], d32[1], vs[1], 0.01, 0.9)[1])


# ------------------------------------------------------------------ other element types
@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float64"])
def test_typed_step_against_exact_rationals(dtype):
    """sgd_step_typed: constants rounded once from double, then four operations each rounded once
    to the element type -- checked with exact rational arithmetic, on values that include
    subnormals of the 16-bit formats and pairs whose sum falls between two grid points."""
    from fractions import Fraction

    from oracle.halfs import bf16_bits_to_f32, f32_to_bf16_bits
    from tests.helpers import FORMATS, round_to_format

    bits, emin = FORMATS[dtype]
    rnd = lambda q: round_to_format(q, bits, emin)
    rng = np.random.default_rng(77)
    n = 400
    raw = [rng.normal(0, s, n) for s in (0.02, 1e-3, 1e-3)]
    raw[0][:8] = [6.1e-5, -5.96e-8, 3.0e-7, 1.0, -1.0, 0.333, 65000.0 if dtype == "float16" else 1e30, 0.0]
    raw[2][:4] = [1.0009765625, 0.99951171875, 2.0**-14, -(2.0**-24)]
    if dtype == "float64":
        x, dx, v = (a.astype(np.float64) for a in raw)
        value = lambda a: [Fraction(float(t)) for t in a]
    elif dtype == "float16":
        x, dx, v = (a.astype(np.float16) for a in raw)
        value = lambda a: [Fraction(float(t)) for t in a]
    else:
        x, dx, v = (f32_to_bf16_bits(a.astype(np.float32)) for a in raw)
        value = lambda a: [Fraction(float(t)) for t in bf16_bits_to_f32(a)]
    lr, mu = 0.0123, 0.9
    v1, x1 = sgd_f32.sgd_step_typed(x, dx, v, lr, mu, dtype)
    lr_q, mu_q = rnd(Fraction(lr)), rnd(Fraction(mu))
    fx, fd, fv, got_v, got_x = value(x), value(dx), value(v), value(v1), value(x1)
    for i in range(n):
        if i == 6:
            continue  # the large entry: fine for the product, but keep the check away from overflow
        want_v = rnd(rnd(mu_q * fv[i]) + fd[i])
        want_x = rnd(fx[i] - rnd(lr_q * want_v))
        assert got_v[i] == want_v, (dtype, i, "v1")
        assert got_x[i] == want_x, (dtype, i, "x1")


def test_typed_step_reduces_to_the_fp32_rule():
    """The same construction in float32 must be sgd_step itself (a dropped rounding or a swapped
    operand in the typed path would show here too)."""
    rng = np.random.default_rng(5)
    x, dx, v = (rng.normal(0, s, 1000).astype(np.float32) for s in (0.02, 1e-3, 1e-3))
    v1, x1 = sgd_f32.sgd_step(x, dx, v, 0.01, 0.9)
    w1, y1 = sgd_f32.sgd_step_typed(x, dx, v, float(np.float32(0.01)), float(np.float32(0.9)), "float64")
    # float64 evaluation of the fp32 inputs agrees with the four-rounding fp32 result to the
    # rounding errors of its operands (an ulp of |x0| ~ 0.02 is 1.9e-9, of |v| ~ 1e-3 1.2e-10)
    assert np.max(np.abs(w1 - v1.astype(np.float64))) <= 6e-10
    assert np.max(np.abs(y1 - x1.astype(np.float64))) <= 4e-9


def test_bfloat16_constant_is_rounded_once():
    """double -> bfloat16 directly; going through fp32 first would round 1 + 2^-8 + 2^-30 down
    to a tie and then to even (1.0) instead of up."""
    from oracle.halfs import bf16_bits_to_f32

    tricky = 1.0 + 2.0**-8 + 2.0**-30
    assert float(bf16_bits_to_f32(sgd_f32.bf16_from_double(tricky))) == 1.0 + 2.0**-7
    assert float(bf16_bits_to_f32(sgd_f32.bf16_from_double(0.5))) == 0.5
    assert float(bf16_bits_to_f32(sgd_f32.bf16_from_double(-3.0))) == -3.0
