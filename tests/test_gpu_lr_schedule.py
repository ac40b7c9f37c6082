"""A learning-rate schedule through the operator front end: a new learning rate every step must
give exactly what a fresh OpEnv with that constant would give (the oracle's result), while the
OpEnv, its plan and its workspace are kept; other hyper-parameters still select their own OpEnv,
and the table of OpEnvs stays bounded."""
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


def test_lans_learning_rate_schedule_keeps_its_op_env(native_libs):
    from raf_amd import op

    op.clear_op_env_cache()
    sizes = [5, 4096, 10_000, 70_001]
    g, w, m, v = lans_inputs(sizes, cfg=310, g16=False)
    tg, tw, tm, tv = _dev(g), _dev(w), _dev(m), _dev(v)
    ow, om, ov = w, m, v
    lrs = [1e-3, 2e-3, 5e-4, 5e-4, 7e-3]
    for step, lr in enumerate(lrs, start=1):
        op.lans(tg + tw + tm + tv, torch.tensor(float(step), device=DEV), lr, 0.9, 0.999, 1e-6, 1, 0.01, 1, 1, True)
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, step, LansHParams(learning_rate=lr))
    torch.cuda.synchronize()
    for got, want in zip(tw + tm + tv, ow + om + ov):
        assert max_rel_err(got.cpu().numpy(), want) <= 1e-5 * len(lrs)
    assert len(op._env_cache) == 1  # five learning rates, one OpEnv
    # another weight decay is another OpEnv, as in the reference
    op.lans(tg + tw + tm + tv, torch.tensor(6.0, device=DEV), 1e-3, 0.9, 0.999, 1e-6, 1, 0.02, 1, 1, True)
    assert len(op._env_cache) == 2


def test_sgd_learning_rate_schedule_is_bit_exact(native_libs):
    from raf_amd import op

    op.clear_op_env_cache()
    rng = np.random.default_rng(5)
    x = rng.normal(0, 0.02, 5003).astype(np.float32)
    d = rng.normal(0, 1e-3, 5003).astype(np.float32)
    v = np.zeros(5003, np.float32)
    tx, td, tv = _dev([x])[0], _dev([d])[0], _dev([v])[0]
    mx, mv = tx.clone(), tv.clone()
    for lr in (0.1, 0.05, 0.025, 0.3):
        tv, tx = op.sgd(tx, td, tv, lr, 0.9)            # single-tensor op: new outputs
        op.sgd_multi([mx, td, mv], lr, 0.9)             # multi-tensor op: in place
        x, v = sgd_f32.sgd_step(x, d, v, lr, 0.9)[::-1]
    assert np.array_equal(tx.cpu().numpy().view(np.uint32), x.view(np.uint32))
    assert np.array_equal(tv.cpu().numpy().view(np.uint32), v.view(np.uint32))
    assert torch.equal(mx, tx) and torch.equal(mv, tv)
    assert len(op._env_cache) == 2  # one OpEnv per op, whatever the learning rate


def test_op_env_table_is_bounded(native_libs):
    from raf_amd import op

    op.clear_op_env_cache()
    x = torch.zeros(64, device=DEV)
    for i in range(op._env_cache.capacity + 20):
        op.sgd(x, x, x, 0.1, 0.5 + i * 1e-3)  # the momentum is part of the signature
    assert len(op._env_cache) == op._env_cache.capacity


def test_learning_rate_setter_refuses_other_op_envs(native_libs):
    from raf_amd import _lib, op

    op.clear_op_env_cache()
    x = torch.ones(100, device=DEV)
    op.l2norm(x)
    (env,) = op._env_cache.values()
    with pytest.raises(_lib.RafError, match="has no learning rate"):
        env.set_learning_rate(0.5)
