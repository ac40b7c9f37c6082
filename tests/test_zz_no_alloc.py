"""GPU test of rafhip_lans_step_noalloc, the LANS step for callers that cannot allocate: it works on
the library's static device scratch array instead of a caller workspace.  Through the C ABI, its
w, m, v (and 16-bit weight copies) must be bit-identical to rafhip_lans_step_mixed's on the same
inputs -- on two calls in a row, the second over a smaller list, because every call on a GPU
shares one array that still holds the previous call's contents.  The file is named so that pytest
collects it last."""

import ctypes

import numpy as np
import pytest
import torch

from tests.helpers import lans_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# several multi-chunk tensors (chunks of 8192 and of 4096 elements), one-chunk tensors, tails that
# are not a multiple of four, an empty tensor
FIRST = [1_200_003, 70_001, 4096, 1, 0, 655_360, 33, 8191]
SECOND = [70_001, 5, 20_000]  # smaller: fewer tensors, fewer chunks


def _to_dev(arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(DEV) for a in arrs]


def _run_pair(sizes, cfg, schedule, g16, copy16, step):
    """The same step through both entry points on two copies of the same inputs."""
    from raf_amd import kernels

    g, w, m, v = lans_inputs(sizes, cfg=cfg, g16=g16)
    hp = kernels.make_hparams(grad_unscale=(1 / 1024 if g16 else 1.0))
    out = []
    for noalloc in (False, True):
        tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
        tp = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in sizes] if copy16 else None
        plan = kernels.LansPlan(sizes, tg[0].dtype, DEV)
        plan.set_schedule(schedule)
        if noalloc:
            plan.step_noalloc(tg, tw, tm, tv, step, hp, p=tp)
        else:
            plan.step(tg, tw, tm, tv, step, hp, p=tp)
        torch.cuda.synchronize()
        plan.close()
        out.append((tw, tm, tv, tp, tg))
    return out, g


def _assert_identical(pair, g_in, what):
    (w0, m0, v0, p0, _), (w1, m1, v1, p1, g1) = pair
    for name, a, b in (("w", w0, w1), ("m", m0, m1), ("v", v0, v1)):
        for t, (x, y) in enumerate(zip(a, b)):
            assert torch.equal(x, y), f"{what}: {name}[{t}] differs between the two entry points"
    if p0 is not None:
        for t, (x, y) in enumerate(zip(p0, p1)):
            assert torch.equal(x, y), f"{what}: 16-bit copy [{t}] differs between the two entry points"
    for t, (x, y) in enumerate(zip(g1, g_in)):  # the gradient is read-only
        assert np.array_equal(x.cpu().numpy(), y), f"{what}: gradient [{t}] was modified"


@pytest.mark.parametrize("schedule", ["phased", "pipelined"])
@pytest.mark.parametrize("g16,copy16", [(False, False), (True, True)])
def test_noalloc_step_equals_workspace_step_twice_in_a_row(native_libs, schedule, g16, copy16):
    first, g_first = _run_pair(FIRST, 81, schedule, g16, copy16, step=3)
    _assert_identical(first, g_first, f"first call ({schedule})")
    # something changed at all (the step is not a no-op that trivially agrees)
    w_before = lans_inputs(FIRST, cfg=81, g16=g16)[1]
    assert not np.array_equal(first[1][0][0].cpu().numpy(), w_before[0])
    second, g_second = _run_pair(SECOND, 82, schedule, g16, copy16, step=torch.tensor(7.0, device=DEV))
    _assert_identical(second, g_second, f"second, smaller call ({schedule})")


def test_noalloc_step_matches_the_oracle(native_libs):
    """Against the float64 oracle too, at the tolerance of a single step (1e-5 per element)."""
    from oracle import lans_f64
    from oracle.lans_f64 import LansHParams
    from raf_amd import kernels
    from tests.helpers import max_rel_err

    sizes = [100_003, 17, 4097]
    g, w, m, v = lans_inputs(sizes, cfg=83)
    ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, 2, LansHParams())
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.step_noalloc(tg, tw, tm, tv, 2, kernels.make_hparams())
    torch.cuda.synchronize()
    for got, want, name in ((tw, ow, "w"), (tm, om, "m"), (tv, ov, "v")):
        for t in range(len(sizes)):
            e = max_rel_err(got[t].cpu().numpy(), want[t])
            assert e <= 1e-5, f"{name}[{t}] max rel err {e:.3e}"


def test_noalloc_step_refuses_a_list_beyond_the_static_scratch(native_libs):
    from raf_amd import _lib, kernels

    lib = _lib.optim()
    n = 100_000  # 64 B of statistics + 32 B of partial sums per one-element tensor: 9.6 MB
    plan = kernels.LansPlan([1] * n, torch.float32, DEV)
    assert plan.workspace_bytes > _lib.RAFHIP_LANS_STATIC_SCRATCH_BYTES
    ptrs = (ctypes.c_void_p * n)()
    hp = kernels.make_hparams()
    st = lib.rafhip_lans_step_noalloc(plan._h, ptrs, ptrs, ptrs, ptrs, None, _lib.RAFHIP_F16, None, 1,
                                      ctypes.byref(hp), None)
    assert st == _lib.RAFHIP_ERR_WORKSPACE
    assert "static" in _lib.last_error() and str(plan.workspace_bytes) in _lib.last_error()
    plan.close()
