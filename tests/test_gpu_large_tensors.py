"""Tensors of more than 2^31 elements (the reference counts elements in 32 bits, lans.cc:55-64, and
cannot take them; 288 GB of HBM can).  A tensor of billions of elements is built as k copies of a
2^20-element pattern, so the CPU side only ever handles the pattern: every copy must come out with
the same bits, the first copy must match the oracle, and the norms are sqrt(k) times the pattern's.
An index that wrapped at 2^31 or 2^32 would leave copies untouched, or different."""

import numpy as np
import pytest
import torch

from oracle import lans_f64, sgd_f32
from oracle.lans_f64 import LansHParams
from tests.helpers import lans_inputs, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PATTERN = 1 << 20
COPIES = 2049  # 2^31 + 2^20 elements


def _tiled(a, copies=COPIES, extra=0):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    out = t.repeat(copies)
    if extra:
        out = torch.cat([out, t[:extra]])
    return out


def _every_copy_equals_the_first(t, copies=COPIES):
    return bool((t[:copies * PATTERN].view(copies, PATTERN) == t[:PATTERN]).all())


@pytest.mark.parametrize("schedule", ["pipelined", "phased"])
def test_lans_on_a_tensor_beyond_2_to_31_elements(native_libs, schedule):
    from raf_amd import kernels

    g, w, m, v = lans_inputs([PATTERN], cfg=120)
    hp = LansHParams()
    n = COPIES * PATTERN
    assert n > 1 << 31
    tg, tw, tm, tv = (_tiled(a[0]) for a in (g, w, m, v))
    small = [torch.from_numpy(a[0][:70001].copy()).to(DEV) for a in (g, w, m, v)]  # a second, ordinary tensor
    plan = kernels.LansPlan([n, 70001], torch.float32, DEV)
    plan.set_schedule(schedule)
    kh = kernels.make_hparams(hp.learning_rate, hp.beta1, hp.beta2, hp.eps, hp.bias_correction, hp.weight_decay,
                              hp.grad_averaging, hp.mode, hp.normalize_grad, hp.grad_unscale)
    plan.step([tg, small[0]], [tw, small[1]], [tm, small[2]], [tv, small[3]], 3, kh)
    torch.cuda.synchronize()
    norms = plan.read_norms()
    plan.close()
    ow, om, ov, on = lans_f64.lans_tensor_step(g[0], w[0], m[0], v[0], 3, hp, repeat=COPIES)
    assert np.max(np.abs(norms[0] - np.array(on)) / np.array(on)) < 1e-10
    for got, want, name in ((tw, ow, "w"), (tm, om, "m"), (tv, ov, "v")):
        assert _every_copy_equals_the_first(got), name
        e = max_rel_err(got[:PATTERN].cpu().numpy(), want.astype(np.float32))
        assert e <= 1e-5, (name, e)
    assert _every_copy_equals_the_first(tg)  # the gradient is left alone
    sw, sm, sv, _ = lans_f64.lans_step([g[0][:70001]], [w[0][:70001]], [m[0][:70001]], [v[0][:70001]], 3, hp)
    assert max_rel_err(small[1].cpu().numpy(), sw[0]) <= 1e-5


def test_sgd_on_a_tensor_beyond_2_to_31_elements(native_libs):
    from raf_amd import kernels

    rng = np.random.default_rng(121)
    x0, dx, v0 = (rng.normal(0, s, PATTERN).astype(np.float32) for s in (0.02, 1e-3, 1e-3))
    extra = 4099  # a vector part, and a tail of three elements
    tx, td, tv = (_tiled(a, extra=extra) for a in (x0, dx, v0))
    n = tx.numel()
    assert n > 1 << 31
    v1, x1 = kernels.sgd_f32(tx, td, tv, 0.01, 0.9)
    torch.cuda.synchronize()
    ov, ox = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    for got, want in ((v1, ov), (x1, ox)):
        assert _every_copy_equals_the_first(got)
        assert np.array_equal(got[:PATTERN].cpu().numpy(), want)
        assert np.array_equal(got[COPIES * PATTERN:].cpu().numpy(), want[:extra])
    del v1, x1
    # the same list through the multi-tensor step, in place, with a short tensor behind the long one
    sx, sd, sv = (torch.from_numpy(a[:5000].copy()).to(DEV) for a in (x0, dx, v0))
    plan = kernels.SgdPlan([n, 5000], torch.float32, DEV)
    plan.step([tx, sx], [td, sd], [tv, sv], 0.01, 0.9)
    torch.cuda.synchronize()
    plan.close()
    for got, want in ((tv, ov), (tx, ox)):
        assert _every_copy_equals_the_first(got)
        assert np.array_equal(got[:PATTERN].cpu().numpy(), want)
        assert np.array_equal(got[COPIES * PATTERN:].cpu().numpy(), want[:extra])
    assert np.array_equal(sx.cpu().numpy(), ox[:5000]) and np.array_equal(sv.cpu().numpy(), ov[:5000])


def test_l2norm_beyond_2_to_31_elements(native_libs):
    from raf_amd import kernels

    rng = np.random.default_rng(122)
    x = rng.normal(0, 1.0, PATTERN).astype(np.float32)
    t = _tiled(x, extra=7)
    assert t.numel() > 1 << 31
    got = float(kernels.l2norm(t).cpu())
    x64 = x.astype(np.float64)
    want = np.float32(np.sqrt(COPIES * np.dot(x64, x64) + np.dot(x64[:7], x64[:7])))
    assert abs(np.float32(got) - want) <= np.spacing(want)


def test_fuse_and_defuse_parts_beyond_2_to_32_bytes(native_libs):
    from raf_amd import kernels

    rng = np.random.default_rng(123)
    pat = rng.integers(0, 1 << 31, PATTERN, dtype=np.int64).astype(np.int32)
    big = _tiled(pat, copies=1025, extra=3)  # 2^32 + 2^22 + 12 bytes
    assert big.numel() * 4 > 1 << 32
    small = torch.arange(1001, dtype=torch.int32, device=DEV)
    plan = kernels.FusePlan([big.numel() * 4, small.numel() * 4], DEV)
    flat = torch.zeros(big.numel() + small.numel(), dtype=torch.int32, device=DEV)
    plan.fuse([big, small], flat)
    torch.cuda.synchronize()
    assert bool((flat[:1025 * PATTERN].view(1025, PATTERN) == big[:PATTERN]).all())
    assert torch.equal(flat[1025 * PATTERN:big.numel()], big[:3]) and torch.equal(flat[big.numel():], small)
    back_big, back_small = torch.zeros_like(big), torch.zeros_like(small)
    plan.defuse(flat, [back_big, back_small])
    torch.cuda.synchronize()
    plan.close()
    assert torch.equal(back_big, big) and torch.equal(back_small, small)
