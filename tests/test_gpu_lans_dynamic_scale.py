"""GPU tests of dynamic loss scaling in the LANS step: the reciprocal of the loss scale and the
overflow flag are fp32 words in device memory that the kernels read when they start, so the scale
can change and a step can be skipped on one plan without a host synchronisation."""

import numpy as np
import pytest
import torch

from oracle import lans_f64
from oracle.lans_f64 import LansHParams
from tests.helpers import lans_inputs, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _to_dev(arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(DEV) for a in arrs]


def _khp(hp):
    from raf_amd import kernels

    return kernels.make_hparams(hp.learning_rate, hp.beta1, hp.beta2, hp.eps, hp.bias_correction,
                                hp.weight_decay, hp.grad_averaging, hp.mode, hp.normalize_grad, hp.grad_unscale)


@pytest.mark.parametrize("schedule", ["phased", "pipelined"])
@pytest.mark.parametrize("g16", [True, "bfloat16"])
def test_scale_changes_and_skipped_steps_on_one_plan(native_libs, schedule, g16):
    from raf_amd import kernels

    sizes = [300_001, 70_001, 17, 4096, 1_100_000]
    hp = LansHParams(grad_unscale=123.0)  # must be ignored once the device word is set
    # the same true gradient under two loss scales, then an overflowed one
    scales = [1024.0, 256.0]
    grads = [lans_inputs(sizes, cfg=70, g16=g16, loss_scale=s)[0] for s in scales]
    _, w, m, v = lans_inputs(sizes, cfg=70, g16=g16)
    dt = torch.float16 if g16 is True else torch.bfloat16
    as_dev = lambda gs: [torch.from_numpy(a).to(DEV) if g16 is True
                         else torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16) for a in gs]
    tw, tm, tv = _to_dev(w), _to_dev(m), _to_dev(v)
    tp = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in sizes]
    tg = as_dev(grads[0])
    plan = kernels.LansPlan(sizes, dt, DEV)
    plan.set_schedule(schedule)
    inv_scale = torch.zeros((), device=DEV)
    found_inf = torch.zeros((), device=DEV)
    plan.set_dynamic_scale(inv_scale, found_inf)

    ow, om, ov = w, m, v
    step = 0
    for s, g in zip(scales, grads):  # step 1 at scale 1024, step 2 at scale 256: no new plan, no sync
        step += 1
        inv_scale.fill_(1.0 / s)
        for dst, src in zip(tg, as_dev(g)):
            dst.copy_(src)
        plan.step(tg, tw, tm, tv, step, _khp(hp), p=tp)
        ow, om, ov, on = lans_f64.lans_step_dynamic_scale(g, ow, om, ov, step, hp, 1.0 / s, 0.0)
    torch.cuda.synchronize()
    for got, want, name in ((tw, ow, "w"), (tm, om, "m"), (tv, ov, "v")):
        for t in range(len(sizes)):
            e = max_rel_err(got[t].cpu().numpy(), want[t])
            assert e <= 1e-5, f"{name}[{t}] after two scales: max rel err {e:.3e}"
    norms = plan.read_norms()
    assert np.max(np.abs(norms - on) / on) < 1e-10

    # an overflowed gradient with the flag raised: the step is a no-op, bit for bit
    before = [t.clone() for t in tw + tm + tv + tp]
    tg[1].view(torch.int16)[12345] = 0x7C00 if g16 is True else 0x7F80  # +inf
    found_inf.fill_(1.0)
    plan.step(tg, tw, tm, tv, step + 1, _khp(hp), p=tp)
    torch.cuda.synchronize()
    for a, b in zip(tw + tm + tv + tp, before):
        assert torch.equal(a, b)
    sw, sm, sv, _ = lans_f64.lans_step_dynamic_scale(grads[1], ow, om, ov, step + 1, hp, 1.0 / 256, 1.0)
    assert all(np.array_equal(a, b) for a, b in zip(sw + sm + sv, ow + om + ov))

    # flag lowered again, finite gradient back: the plan carries on from the unchanged state
    found_inf.zero_()
    for dst, src in zip(tg, as_dev(grads[1])):
        dst.copy_(src)
    plan.step(tg, tw, tm, tv, step + 1, _khp(hp), p=tp)
    torch.cuda.synchronize()
    ow, om, ov, _ = lans_f64.lans_step_dynamic_scale(grads[1], ow, om, ov, step + 1, hp, 1.0 / 256, 0.0)
    for t in range(len(sizes)):
        assert max_rel_err(tw[t].cpu().numpy(), ow[t]) <= 1e-5
        assert torch.equal(tp[t], tw[t].half())

    # switched off: the host value counts again
    plan.set_dynamic_scale(None, None)
    plan.close()


def test_dynamic_scale_words_must_be_fp32_gpu_scalars(native_libs):
    from raf_amd import kernels

    plan = kernels.LansPlan([16], torch.float32, DEV)
    with pytest.raises(TypeError):
        plan.set_dynamic_scale(torch.zeros((), dtype=torch.float16, device=DEV), None)
    with pytest.raises(TypeError):
        plan.set_dynamic_scale(None, torch.zeros(()))
    plan.close()


def test_dynamic_scale_through_the_operator_front_end(native_libs):
    """raf.op.lans_mixed with the hip dialect's loss-scaling extension: the OpEnv is kept while the
    scale changes and while a step is skipped."""
    from raf_amd import op

    sizes = [70_001, 300_000, 9]
    hp = LansHParams()
    g1024, w, m, v = lans_inputs(sizes, cfg=71, g16=True, loss_scale=1024.0)
    g64 = lans_inputs(sizes, cfg=71, g16=True, loss_scale=64.0)[0]
    tg, tw, tm, tv = _to_dev(g1024), _to_dev(w), _to_dev(m), _to_dev(v)
    tp = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in sizes]
    step = torch.ones((), device=DEV)
    inv_scale = torch.full((), 1.0 / 1024, device=DEV)
    found_inf = torch.zeros((), device=DEV)
    args = (hp.learning_rate, hp.beta1, hp.beta2, hp.eps, True, hp.weight_decay, True, True, True)
    op.clear_op_env_cache()
    op.set_lans_dynamic_scale(inv_scale, found_inf)
    try:
        tl = tg + tw + tm + tv + tp
        op.lans_mixed(tl, step, *args)
        ow, om, ov, _ = lans_f64.lans_step_dynamic_scale(g1024, w, m, v, 1, hp, 1.0 / 1024, 0.0)
        envs = len(op._env_cache)
        # overflow: skipped
        found_inf.fill_(1.0)
        step.fill_(2.0)
        op.lans_mixed(tl, step, *args)
        # the scale backs off to 64, the same true gradient arrives under it
        found_inf.zero_()
        inv_scale.fill_(1.0 / 64)
        for dst, src in zip(tg, _to_dev(g64)):
            dst.copy_(src)
        op.lans_mixed(tl, step, *args)
        torch.cuda.synchronize()
        assert len(op._env_cache) == envs  # no new OpEnv for a new scale or a skipped step
        ow, om, ov, _ = lans_f64.lans_step_dynamic_scale(g64, ow, om, ov, 2, hp, 1.0 / 64, 0.0)
        for t in range(len(sizes)):
            assert max_rel_err(tw[t].cpu().numpy(), ow[t]) <= 1e-5
            assert max_rel_err(tm[t].cpu().numpy(), om[t]) <= 1e-5
            assert max_rel_err(tv[t].cpu().numpy(), ov[t]) <= 1e-5
            assert torch.equal(tp[t], tw[t].half())
    finally:
        op.set_lans_dynamic_scale(None, None)
        op.clear_op_env_cache()


def test_two_models_of_one_architecture_share_an_op_env(native_libs):
    """Two tensor lists with the same shapes (two models of one architecture) alternate through
    raf.op.lans: they are served by one OpEnv, whose plan keeps a device pointer table per recent
    list (tests/test_gpu_lans.py counts the uploads), and both follow the oracle."""
    from raf_amd import op

    sizes = [70_001, 300_000, 9]
    hp = LansHParams()
    args = (hp.learning_rate, hp.beta1, hp.beta2, hp.eps, True, hp.weight_decay, True, True, True)
    op.clear_op_env_cache()
    models = []
    for cfg in (72, 73):
        g, w, m, v = lans_inputs(sizes, cfg=cfg)
        models.append((g, w, m, v, _to_dev(g) + _to_dev(w) + _to_dev(m) + _to_dev(v)))
    step = torch.zeros((), device=DEV)
    for s in (1, 2, 3):
        step.fill_(float(s))
        for _, _, _, _, tl in models:
            op.lans(tl, step, *args)
    torch.cuda.synchronize()
    assert len([k for k in op._env_cache if k[0] == "lans"]) == 1
    n = len(sizes)
    for g, w, m, v, tl in models:
        ow, om, ov = w, m, v
        for s in (1, 2, 3):
            ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, s, hp)
        for t in range(n):
            assert max_rel_err(tl[n + t].cpu().numpy(), ow[t]) <= 1e-5
            assert max_rel_err(tl[3 * n + t].cpu().numpy(), ov[t]) <= 1e-5
    op.clear_op_env_cache()


def test_optimizer_class_does_not_count_a_skipped_step(native_libs):
    """raf_amd.optim.LANS under dynamic loss scaling: a step that the kernels skipped because of an
    overflow leaves w, m, v alone AND leaves the device-resident step counter where it was, so the
    bias corrections of the next applied step are those of step 2, not 3 (the oracle's
    lans_step_dynamic_scale with the count of applied steps)."""
    from raf_amd import op, optim

    sizes = [70_001, 9, 4096]
    hp = LansHParams()
    g, w, _, _ = lans_inputs(sizes, cfg=74)
    params = [torch.nn.Parameter(t) for t in _to_dev(w)]
    for p, gt in zip(params, _to_dev(g)):
        p.grad = gt
    inv_scale = torch.ones((), device=DEV)
    found_inf = torch.zeros((), device=DEV)
    op.clear_op_env_cache()
    op.set_lans_dynamic_scale(inv_scale, found_inf)
    try:
        opt = optim.LANS(params)
        zeros = [np.zeros_like(a) for a in w]
        opt.step()                       # applied as step 1
        ow, om, ov, _ = lans_f64.lans_step_dynamic_scale(g, w, zeros, zeros, 1, hp, 1.0, 0.0)
        found_inf.fill_(1.0)
        opt.step()                       # skipped: nothing moves, nothing is counted
        found_inf.zero_()
        opt.step()                       # applied as step 2
        ow, om, ov, _ = lans_f64.lans_step_dynamic_scale(g, ow, om, ov, 2, hp, 1.0, 0.0)
        torch.cuda.synchronize()
        assert float(opt._step_dev) == 3.0 and opt._step == 4  # applied steps + 1; calls + 1
        for t in range(len(sizes)):
            assert max_rel_err(params[t].data.cpu().numpy(), ow[t]) <= 1e-5
            assert max_rel_err(opt.params[t][2].cpu().numpy(), om[t]) <= 1e-5
            assert max_rel_err(opt.params[t][3].cpu().numpy(), ov[t]) <= 1e-5
    finally:
        op.set_lans_dynamic_scale(None, None)
        op.clear_op_env_cache()
