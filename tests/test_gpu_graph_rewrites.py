"""GPU parity of the hip dialect's whole-graph rewrites.  The optimizer part of the functions that
the reference's traced optimizers build for a whole model (python/raf/optim/sgd.py:187-215,
python/raf/optim/lans.py:244-312) goes through the FuseDialect pass and is run through the C ABI;
the results must be, bit for bit, those of the multi-tensor ops called directly (and so the
oracle's), in place on the caller's tensors, with one launch sequence for the whole model."""
import numpy as np
import pytest
import torch

from oracle import halfs, lans_f64, sgd_f32
from oracle.lans_f64 import LansHParams
from tests.helpers import lans_inputs, max_rel_err, rng_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SHAPES = [(1024, 1024), (1024,), (30522, 7), (5, 3, 2, 7), (1,), (70001,)]


def _dev(a):
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16)
    return torch.from_numpy(a.copy()).to(DEV)


def _bits(t):
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16).ravel()
    return t.cpu().numpy().view(np.uint32).ravel()


def _sgd_inputs(cfg, grad):
    w, d, v = [], [], []
    for t, shape in enumerate(SHAPES):
        n = int(np.prod(shape))
        w.append(rng_for(cfg, t, 1).normal(0, 0.02, n).astype(np.float32).reshape(shape))
        g = rng_for(cfg, t, 0).normal(0, 1e-3, n).astype(np.float32).reshape(shape)
        d.append(g.astype(np.float16) if grad == "float16" else halfs.f32_to_bf16_bits(g) if grad == "bfloat16" else g)
        v.append(rng_for(cfg, t, 2).normal(0, 1e-3, n).astype(np.float32).reshape(shape))
    return w, d, v


@pytest.mark.parametrize("grad", ["float32", "float16", "bfloat16"])
def test_traced_sgd_optimizer_runs_as_one_multi_tensor_call(native_libs, grad):
    from raf_amd import op

    w, d, v = _sgd_inputs(310, grad)
    tw, td, tv = [_dev(a) for a in w], [_dev(a) for a in d], [_dev(a) for a in v]
    tp = None
    if grad != "float32":  # a half-precision model: the parameters the cast and the copy write
        tp = [torch.zeros(a.shape, dtype=td[0].dtype, device=DEV) for a in w]
    opt = op.TracedSgdOptimizer(tw, td, tv, 0.01, 0.9, p=tp)
    assert opt.ops == ["raf.op.hip.sgd_multi_mixed" if tp else "raf.op.hip.sgd_multi"]
    before, after = opt.ir_before, opt.ir_after
    assert before.count("raf.op.subtract(") == len(SHAPES) and "hip" not in before
    assert "raf.op.subtract(" not in after and "raf.op.cast(" not in after and "raf.op.add(" not in after
    ptrs = [t.data_ptr() for t in tw + tv]
    ow, ov = [a.ravel() for a in w], [a.ravel() for a in v]
    for _ in range(3):
        opt()
        ow, ov, _ = sgd_f32.sgd_list_step(ow, [a.ravel() for a in d], ov, 0.01, 0.9)
    torch.cuda.synchronize()
    assert ptrs == [t.data_ptr() for t in tw + tv]  # in place
    for t in range(len(SHAPES)):
        assert np.array_equal(_bits(tw[t]), ow[t].view(np.uint32)), t
        assert np.array_equal(_bits(tv[t]), ov[t].view(np.uint32)), t
        if tp:
            want = halfs.narrow_weight(ow[t], grad).view(np.uint16)
            assert np.array_equal(_bits(tp[t]), want), t


def test_traced_sgd_with_a_free_zero_tensor_keeps_cast_and_copy(native_libs):
    """As traced, the optimizer's zero tensor is an input of the function: the copy into the model's
    parameter cannot be folded away.  The updates still run as one multi-tensor call; the cast and
    the copy stay in the graph (this library has no backend for them: they are listed and skipped)."""
    from raf_amd import op
    from raf_amd._lib import RafError

    w, d, v = _sgd_inputs(311, "float16")
    tw, td, tv = [_dev(a) for a in w], [_dev(a) for a in d], [_dev(a) for a in v]
    tp = [torch.zeros(a.shape, dtype=torch.float16, device=DEV) for a in w]
    with pytest.raises(RafError, match="Cannot find a valid dispatch for op raf.op.cast"):
        op.TracedSgdOptimizer(tw, td, tv, 0.01, 0.9, p=tp, zero_is_constant=False)
    opt = op.TracedSgdOptimizer(tw, td, tv, 0.01, 0.9, p=tp, zero_is_constant=False, allow_partial=True)
    assert opt.ops[0] == "raf.op.hip.sgd_multi" and set(opt.ops[1:]) == {"!raf.op.cast"}
    assert opt.ir_after.count("raf.op.cast(") == len(SHAPES) and "zero" in opt.ir_after
    opt()
    torch.cuda.synchronize()
    ow, ov, _ = sgd_f32.sgd_list_step([a.ravel() for a in w], [a.ravel() for a in d], [a.ravel() for a in v], 0.01, 0.9)
    for t in range(len(SHAPES)):
        assert np.array_equal(_bits(tw[t]), ow[t].view(np.uint32))
        assert not tp[t].any()  # the copy did not run


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
def test_traced_lans_optimizer_runs_as_one_lans_mixed_call(native_libs, dtype):
    from raf_amd import op

    sizes = [int(np.prod(s)) for s in SHAPES]
    g, w, m, v = lans_inputs(sizes, cfg=312, g16=True if dtype == "float16" else "bfloat16", loss_scale=1.0)
    shaped = lambda arrs: [a.reshape(s) for a, s in zip(arrs, SHAPES)]
    td = torch.float16 if dtype == "float16" else torch.bfloat16

    def fresh():
        return ([_dev(a) for a in shaped(g)], [_dev(a) for a in shaped(w)], [_dev(a) for a in shaped(m)],
                [_dev(a) for a in shaped(v)], [torch.zeros(s, dtype=td, device=DEV) for s in SHAPES])

    tg, tw, tm, tv, tp = fresh()
    step = torch.ones((), device=DEV)
    opt = op.TracedLansOptimizer(tg, tw, tm, tv, tp, step)
    assert opt.ops == ["raf.op.hip.lans_mixed"]
    assert "raf.op.group_cast(" in opt.ir_before and opt.ir_before.count("raf.op.cast(") == len(SHAPES)
    for gone in ("group_cast", "raf.op.cast(", "raf.op.add(", "raf.op.lans("):
        assert gone not in opt.ir_after, gone
    # the same three steps through the extension op called directly
    rg, rw, rm, rv, rp = fresh()
    rstep = torch.ones((), device=DEV)
    hp = LansHParams()
    args = (hp.learning_rate, hp.beta1, hp.beta2, hp.eps, True, hp.weight_decay, True, True, True)
    ow, om, ov = w, m, v
    for s in (1, 2, 3):
        step.fill_(float(s))
        rstep.fill_(float(s))
        opt()
        op.lans_mixed(rg + rw + rm + rv + rp, rstep, *args)
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, s, hp)
    torch.cuda.synchronize()
    for t in range(len(SHAPES)):
        for a, b in ((tw, rw), (tm, rm), (tv, rv), (tp, rp)):
            assert np.array_equal(_bits(a[t]), _bits(b[t])), t
        assert max_rel_err(tw[t].cpu().numpy().ravel(), ow[t]) <= 1e-4
        assert np.array_equal(_bits(tg[t]), _bits(rg[t]))  # the half gradients are only read


def test_traced_lans_with_a_free_zero_tensor_folds_the_group_cast_only(native_libs):
    from raf_amd import op

    sizes = [int(np.prod(s)) for s in SHAPES]
    g, w, m, v = lans_inputs(sizes, cfg=313, g16=True, loss_scale=1.0)
    tg, tw, tm, tv = ([_dev(a) for a in x] for x in (g, w, m, v))
    tp = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in sizes]
    step = torch.full((), 2.0, device=DEV)
    opt = op.TracedLansOptimizer(tg, tw, tm, tv, tp, step, zero_is_constant=False, allow_partial=True)
    assert opt.ops[0] == "raf.op.hip.lans" and set(opt.ops[1:]) == {"!raf.op.cast"}
    assert "group_cast" not in opt.ir_after and opt.ir_after.count("raf.op.cast(") == len(SHAPES)
    opt()
    torch.cuda.synchronize()
    ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, 2, LansHParams())
    for t in range(len(sizes)):
        assert max_rel_err(tw[t].cpu().numpy(), ow[t]) <= 1e-5
        assert max_rel_err(tm[t].cpu().numpy(), om[t]) <= 1e-5
        assert max_rel_err(tv[t].cpu().numpy(), ov[t]) <= 1e-5


def test_traced_lans_optimizer_takes_the_loss_scaling_in_force(native_libs):
    """The loss scaling set for LANS calls reaches the lans_mixed call inside a traced optimizer's
    graph: a static inverse scale, then a device-resident one with an overflow flag that skips a step."""
    from raf_amd import op

    sizes = [int(np.prod(s)) for s in SHAPES]
    g, w, m, v = lans_inputs(sizes, cfg=314, g16=True, loss_scale=1024.0)
    tg, tw, tm, tv = ([_dev(a) for a in x] for x in (g, w, m, v))
    tp = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in sizes]
    step = torch.ones((), device=DEV)
    opt = op.TracedLansOptimizer(tg, tw, tm, tv, tp, step)
    hp = LansHParams(grad_unscale=1.0 / 1024)
    try:
        op.set_lans_grad_unscale(1.0 / 1024)
        opt()
        torch.cuda.synchronize()
        ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, 1, hp)
        for t in range(len(sizes)):
            assert max_rel_err(tw[t].cpu().numpy(), ow[t]) <= 1e-5
        # dynamic: the scale word says 1/1024 too, the flag skips step 2, step 3 runs as step 2 would
        op.set_lans_grad_unscale(1.0)
        inv_scale = torch.full((), 1.0 / 1024, device=DEV)
        found_inf = torch.ones((), device=DEV)
        op.set_lans_dynamic_scale(inv_scale, found_inf)
        step.fill_(2.0)
        before = [t.clone() for t in tw + tm + tv + tp]
        opt()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(before, tw + tm + tv + tp))
        found_inf.zero_()
        opt()
        torch.cuda.synchronize()
        ow2, _, _, _ = lans_f64.lans_step(g, ow, om, ov, 2, hp)
        for t in range(len(sizes)):
            assert max_rel_err(tw[t].cpu().numpy(), ow2[t]) <= 1e-5
            assert torch.equal(tp[t], tw[t].half())
    finally:
        op.set_lans_grad_unscale(1.0)
        op.set_lans_dynamic_scale(None, None)
