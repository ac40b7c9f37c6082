"""`raf_amd.op.TensorList` through the operator front end on the GPU: a handle gives the bits a
plain list gives, is rebuilt rather than silently stale when a tensor's storage moves, and the VM's
calling pattern (a new tuple value every call, gradients at alternating addresses) reaches the same
OpEnv and the same results."""
import numpy as np
import pytest
import torch

from oracle import lans_f64, sgd_f32
from oracle.lans_f64 import LansHParams
from tests.helpers import lans_inputs, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev(arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(DEV) for a in arrs]


def _args(hp):
    return (hp.learning_rate, hp.beta1, hp.beta2, hp.eps, True, hp.weight_decay, True, True, True)


def _check(tl, n, want_w, want_m, want_v, tol=1e-5):
    for t in range(n):
        assert max_rel_err(tl[n + t].cpu().numpy(), want_w[t]) <= tol
        assert max_rel_err(tl[2 * n + t].cpu().numpy(), want_m[t]) <= tol
        assert max_rel_err(tl[3 * n + t].cpu().numpy(), want_v[t]) <= tol


SIZES = [70_001, 3, 300_000, 4096, 0, 9]


def test_handle_and_plain_list_give_the_same_bits(native_libs):
    from raf_amd import op

    hp = LansHParams()
    g, w, m, v = lans_inputs(SIZES, cfg=130)
    n = len(SIZES)
    op.clear_op_env_cache()
    plain = _dev(g) + _dev(w) + _dev(m) + _dev(v)
    held = op.TensorList(_dev(g) + _dev(w) + _dev(m) + _dev(v))
    step = torch.zeros((), device=DEV)
    ow, om, ov = w, m, v
    for s in (1, 2, 3):
        step.fill_(float(s))
        assert op.lans(plain, step, *_args(hp)) is plain
        assert op.lans(held, step, *_args(hp)) is held
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, s, hp)
    torch.cuda.synchronize()
    assert len([k for k in op._env_cache if k[0] == "lans"]) == 1  # one OpEnv serves both lists
    for a, b in zip(plain, held):
        assert torch.equal(a, b)
    _check(held, n, ow, om, ov)
    assert held.rebuilds == 0
    op.clear_op_env_cache()


def test_handle_made_before_a_storage_swap_is_rebuilt(native_libs):
    """`x.data = ...` after the handle was made: the next call must update the NEW storage (and
    leave the old one alone), not silently the old one."""
    from raf_amd import op

    hp = LansHParams()
    g, w, m, v = lans_inputs(SIZES, cfg=131)
    n = len(SIZES)
    op.clear_op_env_cache()
    tensors = _dev(g) + _dev(w) + _dev(m) + _dev(v)
    held = op.TensorList(tensors)
    step = torch.ones((), device=DEV)
    op.lans(held, step, *_args(hp))
    ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, 1, hp)
    # weight 2 moves to a new allocation (same values); a gradient too
    old_w2 = tensors[n + 2].data
    tensors[n + 2].data = old_w2.clone()
    tensors[0].data = tensors[0].data.clone()
    frozen = old_w2.clone()
    step.fill_(2.0)
    op.lans(held, step, *_args(hp))
    torch.cuda.synchronize()
    assert held.rebuilds == 1
    assert torch.equal(old_w2, frozen), "the step wrote through the stale address"
    ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, 2, hp)
    _check(held, n, ow, om, ov)
    # an untracked handle is the caller's promise, like a TupleValue: it keeps the old addresses
    untracked = op.TensorList(tensors, track=False)
    tensors[n + 2].data = tensors[n + 2].data.clone()
    assert not untracked.current()
    op.clear_op_env_cache()


def test_vm_calling_pattern(native_libs):
    """A new TupleValue over the same tensor values at every call, and gradients that alternate
    between two allocations with DIFFERENT values: same OpEnv, right table every step."""
    from raf_amd import op

    hp = LansHParams()
    g, w, m, v = lans_inputs(SIZES, cfg=132)
    g_other = lans_inputs(SIZES, cfg=133)[0]
    n = len(SIZES)
    op.clear_op_env_cache()
    op.set_executor("vm")
    try:
        first = op.TensorList(_dev(g) + _dev(w) + _dev(m) + _dev(v))
        second = first.replaced(0, _dev(g_other))
        assert second[n] is first[n]  # w, m, v are shared
        step = torch.zeros((), device=DEV)
        ow, om, ov = w, m, v
        for s in range(1, 7):
            step.fill_(float(s))
            op.lans(first if s % 2 else second, step, *_args(hp))
            ow, om, ov, _ = lans_f64.lans_step(g if s % 2 else g_other, ow, om, ov, s, hp)
        torch.cuda.synchronize()
        assert len([k for k in op._env_cache if k[0] == "lans"]) == 1
        _check(first, n, ow, om, ov, tol=1e-4)
    finally:
        op.set_executor("interpreter")
        op.clear_op_env_cache()


def test_sgd_multi_with_a_handle_and_fresh_gradient_objects(native_libs):
    """sgd_multi takes the handle too; a plain list whose gradient OBJECTS are new every step (same
    storage) shares everything else with the previous step's handle.  Bit-exact against the oracle."""
    from raf_amd import op

    sizes = [10_007, 4, 65_536]
    rng = np.random.default_rng(5)
    x = [rng.normal(0, 0.02, k).astype(np.float32) for k in sizes]
    dx = [rng.normal(0, 1e-3, k).astype(np.float32) for k in sizes]
    v = [np.zeros(k, np.float32) for k in sizes]
    op.clear_op_env_cache()
    tx, tdx, tv = _dev(x), _dev(dx), _dev(v)
    held = op.TensorList(tx + tdx + tv)
    ox, ov = x, v
    for _ in range(2):
        op.sgd_multi(held, 0.01, 0.9)
        ox, ov, _ = sgd_f32.sgd_list_step(ox, dx, ov, 0.01, 0.9)
    for _ in range(2):
        op.sgd_multi(tx + [t.detach() for t in tdx] + tv, 0.01, 0.9)
        ox, ov, _ = sgd_f32.sgd_list_step(ox, dx, ov, 0.01, 0.9)
    torch.cuda.synchronize()
    for t in range(len(sizes)):
        assert np.array_equal(tx[t].cpu().numpy(), ox[t]) and np.array_equal(tv[t].cpu().numpy(), ov[t])
    assert len([k for k in op._env_cache if k[0] == "sgd_multi"]) == 1
    op.clear_op_env_cache()


def test_gradients_allocated_anew_every_step(native_libs):
    """torch's default: `.grad` tensors are new objects at new addresses every iteration.  The
    front end has a handful of handles for recent lists; once they are taken the oldest is rebound
    to the new gradients in place.  Twelve steps with different gradient values at every step
    against the oracle, one OpEnv throughout."""
    from raf_amd import op

    hp = LansHParams()
    g0, w, m, v = lans_inputs(SIZES, cfg=131)
    n = len(SIZES)
    op.clear_op_env_cache()
    tw, tm, tv = _dev(w), _dev(m), _dev(v)
    step = torch.zeros((), device=DEV)
    ow, om, ov = w, m, v
    held = []  # keeps every step's gradients alive, so that every step's are at addresses of their own
    steps = op._recent_lists.maxlen + 4
    for s in range(1, steps + 1):
        g = [(a * np.float32(1.0 + 0.125 * s)).astype(np.float32) for a in g0]
        tg = _dev(g)
        held.append(tg)
        step.fill_(float(s))
        op.lans(tg + tw + tm + tv, step, *_args(hp))
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, s, hp)
    torch.cuda.synchronize()
    assert len({t.data_ptr() for tg in held for t in tg if t.numel()}) == steps * sum(1 for k in SIZES if k)
    assert len([k for k in op._env_cache if k[0] == "lans"]) == 1
    assert len(op._recent_lists) == op._recent_lists.maxlen
    assert sum(h.rebinds for h in op._recent_lists) == 4
    _check(tg + tw + tm + tv, n, ow, om, ov, tol=2e-5)
    op.clear_op_env_cache()


def test_gradients_that_die_with_their_step_are_not_kept_alive(native_libs):
    """The same, with the caller dropping each step's gradients after the call (what autograd with
    `zero_grad(set_to_none=True)` amounts to): one handle takes every step's gradients over in
    place and holds none of them once the call has returned; results against the oracle."""
    import gc
    import weakref

    from raf_amd import op

    hp = LansHParams()
    g0, w, m, v = lans_inputs(SIZES, cfg=132)
    n = len(SIZES)
    op.clear_op_env_cache()
    tw, tm, tv = _dev(w), _dev(m), _dev(v)
    step = torch.zeros((), device=DEV)
    ow, om, ov = w, m, v
    for s in range(1, 7):
        g = [(a * np.float32(1.0 + 0.25 * s)).astype(np.float32) for a in g0]
        tg = _dev(g)
        alive = weakref.ref(tg[0])
        step.fill_(float(s))
        op.lans(tg + tw + tm + tv, step, *_args(hp))
        del tg
        gc.collect()
        if s == 1:
            first_step = alive   # not known to be short-lived yet: kept until the next call shows it
        else:
            assert alive() is None, "the front end still holds the gradients of a finished call"
            assert first_step() is None
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, s, hp)
    torch.cuda.synchronize()
    assert len(op._recent_lists) == 1 and op._recent_lists[0].rebinds == 5
    assert len([k for k in op._env_cache if k[0] == "lans"]) == 1
    for t in range(n):
        assert max_rel_err(tw[t].cpu().numpy(), ow[t]) <= 2e-5
        assert max_rel_err(tv[t].cpu().numpy(), ov[t]) <= 2e-5
    op.clear_op_env_cache()
