"""Pins of the LANS oracle (oracle/lans_f64.py and the C restatement).  The reference's own LANS
tests compare against apex's FusedLANS at 1e-3 on a live GPU and hold no stored vectors
(tests/python/optim/test_lans.py:94-137), so the oracle is pinned by what the mathematics fixes:
hand-computed exact cases, the step-1 closed form, torch.optim.Adam's moments and direction, an
independent scalar evaluation, and invariants -- each chosen so that a dropped term, a swapped
beta, a wrong norm or a wrong list order fails it."""
import math

import numpy as np
import pytest
import torch

from oracle import lans_f64
from oracle.lans_f64 import LansHParams, f32
from tests.helpers import lans_inputs, max_rel_err


# ------------------------------------------------------------------ hand-computed exact cases
def test_by_hand_single_element_decoupled():
    # g=3, w=4, m=v=0, no normalisation, no bias correction, beta3=1, beta1=.5, beta2=.75, eps=0:
    # m1=3, v1=.25*9=2.25, den=1.5, u_m=u_g=2, ||w||=4, ||u||=2, r_m=.5*(4/2)*.5=.5, r_g=1
    # w1 = 4 - .5*2 - 1*2 = 1
    hp = LansHParams(learning_rate=0.5, beta1=0.5, beta2=0.75, eps=0.0, bias_correction=0,
                     weight_decay=0.0, grad_averaging=0, mode=1, normalize_grad=False)
    w1, m1, v1, norms = lans_f64.lans_tensor_step(np.float32([3]), np.float32([4]), np.float32([0]),
                                                  np.float32([0]), 1, hp)
    assert w1[0] == 1.0 and m1[0] == 3.0 and v1[0] == 2.25
    assert norms == (3.0, 4.0, 2.0, 2.0)


def test_by_hand_two_elements_with_decay_and_averaging():
    # g=(3,4) normalised by ||g||=5 (eps=0): sg=(.6,.8); beta1=.5 -> beta3=.5; beta2=.75; step 1 with
    # bias correction: bc1=.5, bc2=.25.  m1=.5*sg, v1=.25*sg^2 -> m1/bc1=sg, sqrt(v1/bc2)=|sg| ->
    # adam direction = (1,1); wd=.5, w=(2,-2) -> decoupled: u = (1+1, 1-1) = (2,0) for both terms.
    # ||w||=sqrt(8), ||u||=2, ratio = lr*sqrt(8)/2; w1 = w - (beta1+beta3)*ratio*u = (2-lr*sqrt(8), -2)
    hp = LansHParams(learning_rate=0.25, beta1=0.5, beta2=0.75, eps=0.0, bias_correction=1,
                     weight_decay=0.5, grad_averaging=1, mode=1, normalize_grad=True)
    w1, m1, v1, norms = lans_f64.lans_tensor_step(np.float32([3, 4]), np.float32([2, -2]),
                                                  np.float32([0, 0]), np.float32([0, 0]), 1, hp)
    np.testing.assert_allclose(w1, [2 - 0.25 * math.sqrt(8), -2.0], rtol=1e-15)
    np.testing.assert_allclose(m1, [0.3, 0.4], rtol=1e-15)
    np.testing.assert_allclose(v1, [0.09, 0.16], rtol=1e-15)
    np.testing.assert_allclose(norms, (5.0, math.sqrt(8), 2.0, 2.0), rtol=1e-15)


def test_by_hand_l2_mode_differs_from_decoupled():
    # mode 0 adds wd*w to the scaled gradient *before* the moments: with g=0 the moments become
    # those of wd*w, while mode 1 leaves them at zero and only adds wd*w to the directions.
    hp0 = LansHParams(learning_rate=0.5, beta1=0.5, beta2=0.75, eps=0.0, bias_correction=0,
                      weight_decay=0.5, grad_averaging=0, mode=0, normalize_grad=False)
    w1, m1, v1, _ = lans_f64.lans_tensor_step(np.float32([0]), np.float32([4]), np.float32([0]),
                                              np.float32([0]), 1, hp0)
    # sg = 0 + .5*4 = 2; m1 = 2; v1 = .25*4 = 1; den = 1; u_m = 2, u_g = 2; r_m=.5*(4/2)*.5=.5, r_g=1
    assert m1[0] == 2.0 and v1[0] == 1.0 and w1[0] == 4 - 0.5 * 2 - 1 * 2
    hp1 = LansHParams(**{**hp0.__dict__, "mode": 1})
    w1b, m1b, v1b, _ = lans_f64.lans_tensor_step(np.float32([0]), np.float32([4]), np.float32([0]),
                                                 np.float32([0]), 1, hp1)
    # m1 = v1 = 0, den = 0 -> 0/0: the rule propagates NaN (multi_tensor_lans.cu:224 says so)
    assert m1b[0] == 0.0 and v1b[0] == 0.0 and np.isnan(w1b[0])


# ------------------------------------------------------------------ host scalars
def test_scalars_follow_fp32_schema_and_double_pow():
    sc = lans_f64.lans_scalars(LansHParams(), 3.0)
    b1, b2 = float(np.float32(0.9)), float(np.float32(0.999))
    assert sc.beta1 == b1 and sc.beta2 == b2 and sc.eps == float(np.float32(1e-6))
    assert sc.beta1 != 0.9  # rounded to fp32 first
    assert sc.bc1 == float(np.float32(1.0 - b1 ** 3)) and sc.bc2 == float(np.float32(1.0 - b2 ** 3))
    assert sc.beta3 == float(np.float32(1) - np.float32(0.9))
    assert sc.one_minus_beta2 == float(np.float32(1) - np.float32(0.999))
    off = lans_f64.lans_scalars(LansHParams(bias_correction=0, grad_averaging=0), 3.0)
    assert off.bc1 == 1.0 and off.bc2 == 1.0 and off.beta3 == 1.0
    # (int)fstep truncation, lans.cc:98-99
    assert lans_f64.lans_scalars(LansHParams(), 2.9).bc1 == lans_f64.lans_scalars(LansHParams(), 2.0).bc1


# ------------------------------------------------------------------ step-1 closed form
@pytest.mark.parametrize("n", [1, 5, 1000])
def test_step1_closed_form(n):
    # m=v=0, defaults: u_m == u_g == u = sg/(|sg|+eps) + wd*w and w1 = w - lr*(||w||/||u||)*u
    g, w, m, v = lans_inputs([n], cfg=11, zero_state=True)
    hp = LansHParams()
    w1, m1, v1, norms = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 1, hp)
    g64, w64 = g[0].astype(np.float64), w[0].astype(np.float64)
    eps, wd, lr = f32(1e-6), f32(0.01), f32(1e-3)
    sg = g64 / (np.linalg.norm(g64) + eps)
    u = sg / (np.abs(sg) + eps) + wd * w64
    want = w64 - lr * (np.linalg.norm(w64) / np.linalg.norm(u)) * u
    assert max_rel_err(w1, want) < 1e-11
    np.testing.assert_allclose(norms[2], np.linalg.norm(u), rtol=1e-12)
    np.testing.assert_allclose(norms[3], norms[2], rtol=1e-12)
    np.testing.assert_allclose(m1, (1 - f32(0.9)) * sg, rtol=1e-12)
    np.testing.assert_allclose(v1, (1 - f32(0.999)) * sg * sg, rtol=1e-12)


# ------------------------------------------------------------------ torch.optim.Adam cross-check
def test_moments_and_direction_match_torch_adam():
    # without gradient normalisation and weight decay the m/v recurrences are Adam's exp_avg /
    # exp_avg_sq and u_m is Adam's bias-corrected direction.  torch uses unrounded bias corrections,
    # the rule fp32-rounded ones: agreement to ~1e-7 relative, far below any structural mistake.
    n, steps = 64, 4
    r = np.random.default_rng(5)
    b1, b2, eps = f32(0.9), f32(0.999), f32(1e-6)
    hp = LansHParams(weight_decay=0.0, normalize_grad=False)
    p = torch.nn.Parameter(torch.zeros(n, dtype=torch.float64))
    opt = torch.optim.Adam([p], lr=1.0, betas=(b1, b2), eps=eps)
    m = np.zeros(n)
    v = np.zeros(n)
    w = r.normal(0, 0.02, n)
    for step in range(1, steps + 1):
        g = r.normal(0, 1e-3, n).astype(np.float32)
        before = p.detach().numpy().copy()
        p.grad = torch.from_numpy(g.astype(np.float64))
        opt.step()
        adam_dir = before - p.detach().numpy()  # lr = 1
        sc = lans_f64.lans_scalars(hp, step)
        m, v, u_m, u_g, _ = lans_f64.lans_directions(g.astype(np.float64), w, m, v, sc, hp)
        st = opt.state[p]
        np.testing.assert_allclose(m, st["exp_avg"].numpy(), rtol=1e-12)
        np.testing.assert_allclose(v, st["exp_avg_sq"].numpy(), rtol=1e-12)
        np.testing.assert_allclose(u_m, adam_dir, rtol=5e-7)
        # u_g is the same direction with the raw gradient in place of the first moment
        den = np.sqrt(v / sc.bc2) + eps
        np.testing.assert_allclose(u_g * den, g.astype(np.float64), rtol=1e-12)


# ------------------------------------------------------------------ independent scalar evaluation
def _scalar_lans(g, w, m, v, step, hp):
    """Element-by-element Python floats and math.fsum norms; written against the rule's text."""
    lr, b1, b2, eps, wd = (f32(hp.learning_rate), f32(hp.beta1), f32(hp.beta2), f32(hp.eps),
                           f32(hp.weight_decay))
    k = int(step)
    bc1 = f32(1 - b1 ** k) if hp.bias_correction == 1 else 1.0
    bc2 = f32(1 - b2 ** k) if hp.bias_correction == 1 else 1.0
    b3 = float(np.float32(1) - np.float32(b1)) if hp.grad_averaging == 1 else 1.0
    omb2 = float(np.float32(1) - np.float32(b2))
    g = [float(np.float32(np.float32(x) * np.float32(hp.grad_unscale))) for x in g]
    gn = math.sqrt(math.fsum(x * x for x in g))
    pn = math.sqrt(math.fsum(float(x) ** 2 for x in w))
    ms, vs, ums, ugs = [], [], [], []
    for gi, wi, mi, vi in zip(g, map(float, w), map(float, m), map(float, v)):
        s = gi / (gn + eps) if (hp.normalize_grad and gn != 0) else gi
        wp = wi if wd != 0 else 0.0
        if hp.mode == 0:
            s = s + wd * wp
        mn = mi * b1 + b3 * s
        vn = vi * b2 + omb2 * s * s
        den = math.sqrt(vn / bc2) + eps
        extra = wd * wp if hp.mode == 1 else 0.0
        ms.append(mn)
        vs.append(vn)
        ums.append(mn / bc1 / den + extra)
        ugs.append(s / den + extra)
    unm = math.sqrt(math.fsum(x * x for x in ums))
    ung = math.sqrt(math.fsum(x * x for x in ugs))
    rm = (lr * (pn / unm) if (unm != 0 and pn != 0) else lr) * b1
    rg = (lr * (pn / ung) if (ung != 0 and pn != 0) else lr) * b3
    wn = [wi - rm * a - rg * b for wi, a, b in zip(map(float, w), ums, ugs)]
    return wn, ms, vs, (gn, pn, unm, ung)


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("flags", [(1, 1, True), (0, 1, True), (1, 0, False), (0, 0, False)])
@pytest.mark.parametrize("wd", [0.01, 0.0])
def test_against_scalar_evaluation(mode, flags, wd):
    bias, avg, norm = flags
    hp = LansHParams(mode=mode, bias_correction=bias, grad_averaging=avg, normalize_grad=norm,
                     weight_decay=wd)
    for n, step in ((1, 1), (7, 2), (16, 5)):
        g, w, m, v = lans_inputs([n], cfg=20 + n)
        w1, m1, v1, norms = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], step, hp)
        sw, sm, sv, sn = _scalar_lans(g[0], w[0], m[0], v[0], step, hp)
        np.testing.assert_allclose(w1, sw, rtol=1e-12)
        np.testing.assert_allclose(m1, sm, rtol=1e-13)
        np.testing.assert_allclose(v1, sv, rtol=1e-13)
        np.testing.assert_allclose(norms, sn, rtol=1e-13)


def test_fp16_gradient_unscale_is_applied_first():
    g, w, m, v = lans_inputs([33], cfg=31, g16=True)
    hp = LansHParams(grad_unscale=1.0 / 1024)
    a = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 2, hp)
    # same as feeding the exactly unscaled fp32 gradient with no unscale
    g32 = (g[0].astype(np.float32) / np.float32(1024)).astype(np.float32)
    b = lans_f64.lans_tensor_step(g32, w[0], m[0], v[0], 2, LansHParams())
    for x, y in zip(a[:3], b[:3]):
        assert np.array_equal(x, y)
    sw, *_ = _scalar_lans(g[0], w[0], m[0], v[0], 2, hp)
    np.testing.assert_allclose(a[0], sw, rtol=1e-12)


def test_dynamic_scale_is_an_exact_unscale_or_no_step_at_all():
    """The dynamic-loss-scaling form (an extension with no counterpart in the reference): with a
    power-of-two scale it is the plain step on the exactly unscaled gradients, bit for bit; a set
    overflow flag returns w, m, v untouched, whatever the gradients hold; a scale that is not a
    power of two is rounded to fp32 once, like a device word would hold it."""
    sizes = [7, 130]
    g, w, m, v = lans_inputs(sizes, cfg=33)
    g512 = [(x * np.float32(512)).astype(np.float32) for x in g]
    a = lans_f64.lans_step_dynamic_scale(g512, w, m, v, 3, LansHParams(), 1.0 / 512, 0.0)
    b = lans_f64.lans_step(g, w, m, v, 3, LansHParams())
    for xs, ys in zip(a[:3], b[:3]):
        for x, y in zip(xs, ys):
            assert np.array_equal(x, y)
    np.testing.assert_array_equal(a[3], b[3])
    poisoned = [np.full_like(x, np.inf) for x in g]
    sw, sm, sv, sn = lans_f64.lans_step_dynamic_scale(poisoned, w, m, v, 3, LansHParams(), 1.0 / 512, 1.0)
    for xs, ys in zip((sw, sm, sv), (w, m, v)):
        for x, y in zip(xs, ys):
            assert np.array_equal(x, y) and x is not y
    assert np.isnan(sn).all()
    third = lans_f64.lans_step_dynamic_scale(g, w, m, v, 3, LansHParams(), 1.0 / 3.0, 0.0)
    same = lans_f64.lans_step(g, w, m, v, 3, LansHParams(grad_unscale=float(np.float32(1.0 / 3.0))))
    assert all(np.array_equal(x, y) for x, y in zip(third[0], same[0]))
    assert np.array_equal(third[3], same[3])
    assert not np.array_equal(third[3], b[3])  # and the scale is applied at all


def test_repeat_stands_for_a_tensor_of_back_to_back_copies():
    """lans_tensor_step(..., repeat=k) against the step on the pattern tiled k times explicitly: the
    norms are sqrt(k) times the pattern's and every copy gets the same result (to the rounding of the
    differently ordered sums); repeat=1 changes no bit."""
    g, w, m, v = lans_inputs([257], cfg=34)
    hp = LansHParams()
    for k in (2, 3, 7):
        tiled = [np.tile(a[0], k) for a in (g, w, m, v)]
        w1, m1, v1, n1 = lans_f64.lans_tensor_step(*tiled, 4, hp)
        wr, mr, vr, nr = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 4, hp, repeat=k)
        np.testing.assert_allclose(nr, n1, rtol=1e-13)
        for big, pat in ((w1, wr), (m1, mr), (v1, vr)):
            for j in range(k):
                np.testing.assert_allclose(big[j * 257:(j + 1) * 257], pat, rtol=1e-12, atol=0)
        assert not np.allclose(nr, lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 4, hp)[3])
    a = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 4, hp, repeat=1)
    b = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 4, hp)
    assert all(np.array_equal(x, y) for x, y in zip(a[:3], b[:3])) and a[3] == b[3]


# ------------------------------------------------------------------ invariants and special cases
def test_tensor_independence_and_list_order():
    sizes = [5, 1, 130, 17]
    g, w, m, v = lans_inputs(sizes, cfg=40)
    ws, ms, vs, norms = lans_f64.lans_step(g, w, m, v, 3)
    perm = [2, 0, 3, 1]
    pw, pm, pv, pn = lans_f64.lans_step([g[i] for i in perm], [w[i] for i in perm],
                                        [m[i] for i in perm], [v[i] for i in perm], 3)
    for k, i in enumerate(perm):
        assert np.array_equal(pw[k], ws[i]) and np.array_equal(pm[k], ms[i])
        assert np.array_equal(pv[k], vs[i]) and np.array_equal(pn[k], norms[i])
    # the flat operator list is [g..., w..., m..., v...] and g comes back untouched
    flat = lans_f64.lans_flat_list_step(g + w + m + v, 3)
    assert all(flat[i] is g[i] for i in range(4))
    assert all(np.array_equal(flat[4 + i], ws[i]) for i in range(4))
    assert all(np.array_equal(flat[8 + i], ms[i]) for i in range(4))
    assert all(np.array_equal(flat[12 + i], vs[i]) for i in range(4))
    with pytest.raises(AssertionError):
        lans_f64.lans_flat_list_step(g + w + m + v[:3], 3)


def test_update_norm_bound_and_step1_equality():
    # ||w - w1|| <= lr*(beta1 + beta3)*||w||, with equality when u_m and u_g are parallel (step 1)
    g, w, m, v = lans_inputs([500], cfg=41)
    lr = f32(1e-3)
    for step, state in ((1, True), (4, False)):
        mm = np.zeros_like(m[0]) if state else m[0]
        vv = np.zeros_like(v[0]) if state else v[0]
        w1, _, _, norms = lans_f64.lans_tensor_step(g[0], w[0], mm, vv, step, LansHParams())
        dn = np.linalg.norm(w[0].astype(np.float64) - w1)
        bound = lr * norms[1]  # beta1 + beta3 == 1
        assert dn <= bound * (1 + 1e-12)
        if state:
            np.testing.assert_allclose(dn, bound, rtol=1e-10)
        else:
            assert dn < bound * (1 - 1e-6)  # u_m and u_g are no longer parallel


def test_power_of_two_gradient_scaling_invariance():
    g, w, m, v = lans_inputs([300], cfg=42, zero_state=True)
    hp = LansHParams(eps=0.0)
    a = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 1, hp)
    b = lans_f64.lans_tensor_step(g[0] * np.float32(64), w[0], m[0], v[0], 1, hp)
    for x, y in zip(a[:3], b[:3]):
        assert np.array_equal(x, y)
    c = lans_f64.lans_tensor_step(g[0] * np.float32(64), w[0], m[0], v[0], 1,
                                  LansHParams(eps=0.0, normalize_grad=False))
    assert not np.array_equal(a[2], c[2])  # without normalisation the second moment scales


def test_zero_norm_special_cases():
    n = 10
    g, w, m, v = lans_inputs([n], cfg=43)
    z = np.zeros(n, np.float32)
    hp = LansHParams()
    lr, b1 = f32(1e-3), f32(0.9)
    b3 = float(np.float32(1) - np.float32(0.9))
    # ||g|| == 0: no normalisation (no 0/eps blow-up); moments just decay
    w1, m1, v1, norms = lans_f64.lans_tensor_step(z, w[0], m[0], v[0], 2, hp)
    assert norms[0] == 0.0
    np.testing.assert_allclose(m1, m[0].astype(np.float64) * b1, rtol=1e-15)
    # ||w|| == 0: both ratios fall back to lr (times beta1 / beta3)
    sc = lans_f64.lans_scalars(hp, 2)
    _, _, u_m, u_g, _ = lans_f64.lans_directions(g[0].astype(np.float64), z.astype(np.float64),
                                                 m[0].astype(np.float64), v[0].astype(np.float64), sc, hp)
    w1, *_ = lans_f64.lans_tensor_step(g[0], z, m[0], v[0], 2, hp)
    np.testing.assert_allclose(w1, -(lr * b1) * u_m - (lr * b3) * u_g, rtol=1e-12)


def test_zero_weight_decay_ignores_weights_in_stage1():
    g, w, m, v = lans_inputs([50], cfg=44)
    hp = LansHParams(weight_decay=0.0)
    sc = lans_f64.lans_scalars(hp, 2)
    a = lans_f64.lans_directions(g[0].astype(np.float64), w[0].astype(np.float64),
                                 m[0].astype(np.float64), v[0].astype(np.float64), sc, hp)
    b = lans_f64.lans_directions(g[0].astype(np.float64), np.full(50, np.inf),
                                 m[0].astype(np.float64), v[0].astype(np.float64), sc, hp)
    for x, y in zip(a[:4], b[:4]):
        assert np.array_equal(x, y)


def test_state_dtype_and_shapes():
    g, w, m, v = lans_inputs([12], cfg=45)
    w2 = [w[0].reshape(3, 4)]
    ws, ms, vs, _ = lans_f64.lans_step(g, w2, m, v, 1)
    assert ws[0].shape == (3, 4) and ws[0].dtype == np.float32
    ws64, *_ = lans_f64.lans_step(g, w2, m, v, 1, state_dtype=np.float64)
    assert ws64[0].dtype == np.float64
    assert np.array_equal(ws64[0].astype(np.float32), ws[0])


# ------------------------------------------------------------------ the C restatement
@pytest.mark.parametrize("g16", [False, True, "bfloat16"])
@pytest.mark.parametrize("mode", [0, 1])
def test_c_restatement_matches_numpy_oracle(c_oracle, g16, mode):
    sizes = [1, 3, 4, 5, 511, 513, 4097, 70000, 0]
    g, w, m, v = lans_inputs(sizes, cfg=50, g16=g16)
    hp = LansHParams(mode=mode, grad_unscale=(1 / 1024 if g16 else 1.0))
    for step in (1, 3):
        ws, ms, vs, norms = lans_f64.lans_step(g, w, m, v, step, hp)
        wc, mc, vc = [a.copy() for a in w], [a.copy() for a in m], [a.copy() for a in v]
        nc = c_oracle.lans_step_inplace(g, wc, mc, vc, step, hp, threads=4)
        for a, b in zip(ws + ms + vs, wc + mc + vc):
            assert max_rel_err(b, a) <= 6e-8  # the same float64 value, rounded to fp32
        mism = sum(int((a != b).sum()) for a, b in zip(ws + ms + vs, wc + mc + vc))
        assert mism <= 2  # a rounding-boundary flip is possible, nothing more
        np.testing.assert_allclose(nc, norms, rtol=1e-13)


# ------------------------------------------------------------------ mixed precision
def test_bf16_gradient_equals_its_widened_float32(c_oracle):
    """group_cast widens exactly (python/raf/optim/lans.py:261-265): a bfloat16 gradient and the
    fp32 array holding the same values give identical results in both oracles."""
    from oracle import halfs

    g, w, m, v = lans_inputs([5000, 7], cfg=52, g16="bfloat16")
    g32 = [halfs.bf16_bits_to_f32(x) for x in g]
    # the widened values really are on the bfloat16 grid and scaled as generated (~1e-3 * 1024)
    assert all((x.view(np.uint32) & 0xFFFF == 0).all() for x in g32)
    assert 0.5 < np.std(g32[0]) < 2.0
    hp = LansHParams(grad_unscale=1 / 1024)
    a = lans_f64.lans_step(g, w, m, v, 2, hp)
    b = lans_f64.lans_step(g32, w, m, v, 2, hp)
    for x, y in zip(a[0] + a[1] + a[2], b[0] + b[1] + b[2]):
        assert np.array_equal(x, y)
    wc, mc, vc = [x.copy() for x in w], [x.copy() for x in m], [x.copy() for x in v]
    wd, md, vd = [x.copy() for x in w], [x.copy() for x in m], [x.copy() for x in v]
    c_oracle.lans_step_inplace(g, wc, mc, vc, 2, hp)
    c_oracle.lans_step_inplace(g32, wd, md, vd, 2, hp)
    for x, y in zip(wc + mc + vc, wd + md + vd):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("model_dtype", ["float16", "bfloat16"])
def test_mixed_step_copies_are_the_narrowed_stored_weights(c_oracle, model_dtype):
    """cast(new_w, dtype) acts on the fp32 weight that was stored (lans.py:289-291), not on the
    float64 value behind it; both oracles must agree on that, bit for bit given equal weights."""
    import torch
    from oracle import halfs

    g, w, m, v = lans_inputs([4097, 3, 70000], cfg=53, g16=True)
    hp = LansHParams(grad_unscale=1 / 1024)
    ws, ms, vs, ps, _ = lans_f64.lans_mixed_step(g, w, m, v, 2, hp, model_dtype)
    tdt = torch.float16 if model_dtype == "float16" else torch.bfloat16
    for w32, p in zip(ws, ps):
        t = torch.from_numpy(w32).to(tdt).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(p.view(np.uint16), t)
    wc, mc, vc = [x.copy() for x in w], [x.copy() for x in m], [x.copy() for x in v]
    pc = [np.zeros(x.size, np.uint16) for x in w]
    c_oracle.lans_step_inplace(g, wc, mc, vc, 2, hp, p_list=pc, model_dtype=model_dtype)
    for w32, p in zip(wc, pc):
        assert np.array_equal(p, halfs.narrow_weight(w32, model_dtype).view(np.uint16))


def test_c_restatement_thread_count_independent(c_oracle):
    g, w, m, v = lans_inputs([200000, 70001], cfg=51)
    outs = []
    for threads in (1, 3, 8):
        wc, mc, vc = [a.copy() for a in w], [a.copy() for a in m], [a.copy() for a in v]
        n = c_oracle.lans_step_inplace(g, wc, mc, vc, 2, LansHParams(), threads=threads)
        outs.append((wc, mc, vc, n))
    for o in outs[1:]:
        assert all(np.array_equal(a, b) for a, b in zip(outs[0][0], o[0]))
        assert np.array_equal(outs[0][3], o[3])
