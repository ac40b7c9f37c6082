"""GPU parity of raf.op.lans: the HIP kernels, called through the C ABI, against the float64
oracle.  Tolerances are the stated ones -- max relative error per element 1e-5 after one step and
1e-4 after 100 steps -- on w, m and v; norms must agree to 1e-10."""

import numpy as np
import pytest
import torch

from oracle import lans_f64
from oracle.lans_f64 import LansHParams
from tests.golden import make_fixtures as mf
from tests.helpers import lans_inputs, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL_1 = 1e-5
TOL_100 = 1e-4


def _to_dev(arrs):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(DEV) for a in arrs]


def _khp(hp: LansHParams):
    from raf_amd import kernels

    return kernels.make_hparams(hp.learning_rate, hp.beta1, hp.beta2, hp.eps, hp.bias_correction,
                                hp.weight_decay, hp.grad_averaging, hp.mode, hp.normalize_grad,
                                hp.grad_unscale)


def _gpu_steps(g, w, m, v, hp, first_step, steps=1, step_on_device=True):
    from raf_amd import kernels

    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan([a.size for a in w], tg[0].dtype if tg else torch.float32, DEV)
    for s in range(steps):
        step = first_step + s
        arg = torch.tensor(float(step), dtype=torch.float32, device=DEV) if step_on_device else step
        plan.step(tg, tw, tm, tv, arg, _khp(hp))
    torch.cuda.synchronize()
    norms = plan.read_norms()
    plan.close()
    back = lambda ts: [t.cpu().numpy() for t in ts]
    return back(tw), back(tm), back(tv), norms, back(tg)


def _assert_close(got, want, tol, what):
    for t, (a, b) in enumerate(zip(got, want)):
        e = max_rel_err(a, b)
        assert e <= tol, f"{what}[{t}] max rel err {e:.3e} > {tol}"


def _assert_norms(got, want):
    nz = want != 0
    assert np.array_equal(got[~nz], want[~nz])
    if nz.any():
        assert np.max(np.abs(got[nz] - want[nz]) / want[nz]) < 1e-10


# ------------------------------------------------------------------ committed fixtures
@pytest.mark.parametrize("name", list(mf.LANS_CASES))
def test_golden_fixture(native_libs, name):
    z = np.load(mf.HERE / "lans_kat.npz")
    kw, g16, first_step = mf.LANS_CASES[name]
    hp = LansHParams(**kw)
    nt = len(mf.LANS_SIZES)
    g, w, m, v = ([z[f"{name}/{q}{t}"] for t in range(nt)] for q in "gwmv")
    for steps in mf.LANS_STORED:
        gw, gm, gv, norms, _ = _gpu_steps(g, w, m, v, hp, first_step, steps)
        tol = TOL_1 if steps == 1 else TOL_100
        for q, got in (("w", gw), ("m", gm), ("v", gv)):
            _assert_close(got, [z[f"{name}/{q}{t}_after{steps}"] for t in range(nt)], tol, f"{name}/{q}")
        _assert_norms(norms, z[f"{name}/norms_after{steps}"])


# ------------------------------------------------------------------ edge sizes, flags, paths
EDGE_SIZES = [1, 3, 4, 5, 0, 255, 256, 257, 1023, 1024, 1025, 16383, 16384, 16385, 65537, 100003]


@pytest.mark.parametrize("g16", [False, True])
@pytest.mark.parametrize("mode", [0, 1])
def test_edge_sizes_against_oracle(native_libs, g16, mode):
    hp = LansHParams(mode=mode, grad_unscale=(1 / 1024 if g16 else 1.0))
    g, w, m, v = lans_inputs(EDGE_SIZES, cfg=60 + mode, g16=g16)
    ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 2, hp)
    gw, gm, gv, gn, gg = _gpu_steps(g, w, m, v, hp, 2)
    _assert_close(gw, ow, TOL_1, "w")
    _assert_close(gm, om, TOL_1, "m")
    _assert_close(gv, ov, TOL_1, "v")
    _assert_norms(gn, on)
    assert all(np.array_equal(a, b) for a, b in zip(gg, g)), "gradients must stay untouched"


@pytest.mark.parametrize("flags", [
    dict(bias_correction=0), dict(grad_averaging=0), dict(normalize_grad=False),
    dict(weight_decay=0.0), dict(weight_decay=0.0, mode=0),
    dict(learning_rate=0.02, beta1=0.8, beta2=0.99, eps=1e-8, weight_decay=0.1),
])
def test_flag_combinations(native_libs, flags):
    hp = LansHParams(**flags)
    sizes = [7, 1000, 20001]
    g, w, m, v = lans_inputs(sizes, cfg=70)
    ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 5, hp)
    gw, gm, gv, gn, _ = _gpu_steps(g, w, m, v, hp, 5)
    _assert_close(gw, ow, TOL_1, "w")
    _assert_close(gm, om, TOL_1, "m")
    _assert_close(gv, ov, TOL_1, "v")
    _assert_norms(gn, on)


def test_step_from_device_tensor_equals_host_step(native_libs):
    g, w, m, v = lans_inputs([3000, 17], cfg=71)
    a = _gpu_steps(g, w, m, v, LansHParams(), 7, step_on_device=True)
    b = _gpu_steps(g, w, m, v, LansHParams(), 7, step_on_device=False)
    for x, y in zip(a[:3], b[:3]):
        assert all(np.array_equal(p, q) for p, q in zip(x, y))


def test_unaligned_tensors_take_the_scalar_path(native_libs):
    from raf_amd import kernels

    sizes = [5, 1001, 40000]
    g, w, m, v = lans_inputs(sizes, cfg=72)
    hp = LansHParams()
    ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 3, hp)

    def shifted(arrs, off):  # views that start `off` elements into a larger buffer
        out = []
        for a in arrs:
            buf = torch.zeros(a.size + 8, dtype=torch.float32, device=DEV)
            buf[off:off + a.size] = torch.from_numpy(a).to(DEV)
            out.append(buf[off:off + a.size])
        return out

    tg, tw, tm, tv = shifted(g, 1), shifted(w, 2), shifted(m, 3), shifted(v, 1)
    assert tg[1].data_ptr() % 16 != 0
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.step(tg, tw, tm, tv, 3, _khp(hp))
    torch.cuda.synchronize()
    _assert_close([t.cpu().numpy() for t in tw], ow, TOL_1, "w")
    _assert_close([t.cpu().numpy() for t in tm], om, TOL_1, "m")
    _assert_close([t.cpu().numpy() for t in tv], ov, TOL_1, "v")
    _assert_norms(plan.read_norms(), on)


def test_zero_norm_tensors(native_libs):
    sizes = [100, 100, 100]
    g, w, m, v = lans_inputs(sizes, cfg=73)
    g[0][:] = 0  # ||g|| == 0: gradient not normalised
    w[1][:] = 0  # ||w|| == 0: trust ratios fall back to lr
    g[2][:] = 0
    m[2][:] = 0
    v[2][:] = 0
    w[2][:] = 0  # everything zero: stays zero with eps > 0, is 0/0 = NaN with eps == 0
    for eps, all_zero_gives_nan in ((1e-6, False), (0.0, True)):
        hp = LansHParams(eps=eps)
        with np.errstate(all="ignore"):
            ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 2, hp)
        gw, gm, gv, gn, _ = _gpu_steps(g, w, m, v, hp, 2)
        for t in (0, 1):
            assert max_rel_err(gw[t], ow[t]) <= TOL_1 and max_rel_err(gm[t], om[t]) <= TOL_1
            assert max_rel_err(gv[t], ov[t]) <= TOL_1
        assert np.isnan(ow[2]).all() == all_zero_gives_nan  # the rule propagates NaN, so do we
        assert np.array_equal(np.isnan(gw[2]), np.isnan(ow[2]))
        assert np.array_equal(gw[2][~np.isnan(ow[2])], ow[2][~np.isnan(ow[2])])
        assert gn[0][0] == 0.0 and gn[1][1] == 0.0


def test_empty_list_and_empty_tensors(native_libs):
    from raf_amd import kernels

    plan = kernels.LansPlan([], torch.float32, DEV)
    plan.step([], [], [], [], 1, _khp(LansHParams()))  # no-op
    plan2 = kernels.LansPlan([0, 0], torch.float32, DEV)
    z = [torch.empty(0, device=DEV), torch.empty(0, device=DEV)]
    plan2.step(z, z, z, z, 1, _khp(LansHParams()))
    torch.cuda.synchronize()


# ------------------------------------------------------------------ properties
def test_bitwise_determinism_and_order_independence(native_libs):
    sizes = [40000, 3, 70001, 1 << 18]
    g, w, m, v = lans_inputs(sizes, cfg=74)
    a = _gpu_steps(g, w, m, v, LansHParams(), 2)
    b = _gpu_steps(g, w, m, v, LansHParams(), 2)
    perm = [3, 1, 0, 2]
    c = _gpu_steps(*([x[i] for i in perm] for x in (g, w, m, v)), LansHParams(), 2)
    for q in range(3):
        for t in range(4):
            assert np.array_equal(a[q][t], b[q][t])
            assert np.array_equal(a[q][perm[t]], c[q][t])  # a tensor's result ignores its neighbours
    assert np.array_equal(a[3], b[3])


def test_hundred_steps_against_oracle(native_libs, c_oracle):
    """100 consecutive steps, state carried in fp32 on both sides, gradient fixed."""
    sizes = [1, 9, 4099, 70001]
    g, w, m, v = lans_inputs(sizes, cfg=75, zero_state=True)
    hp = LansHParams()
    gw, gm, gv, gn, _ = _gpu_steps(g, w, m, v, hp, 1, steps=100)
    ow, om, ov = [a.copy() for a in w], [a.copy() for a in m], [a.copy() for a in v]
    for s in range(1, 101):
        on = c_oracle.lans_step_inplace(g, ow, om, ov, s, hp, threads=4)
    _assert_close(gw, ow, TOL_100, "w")
    _assert_close(gm, om, TOL_100, "m")
    _assert_close(gv, ov, TOL_100, "v")
    _assert_norms(gn, on)
    # and against the NumPy oracle on the small tensors (the C restatement is itself pinned to it)
    nw, nm, nv = [a.copy() for a in w[:3]], [a.copy() for a in m[:3]], [a.copy() for a in v[:3]]
    for s in range(1, 101):
        nw, nm, nv, _ = lans_f64.lans_step(g[:3], nw, nm, nv, s, hp)
    _assert_close(gw[:3], nw, TOL_100, "w(numpy)")


# ------------------------------------------------------------------ error paths (no kernel runs)
def test_workspace_and_argument_errors(native_libs):
    from raf_amd import _lib, kernels

    plan = kernels.LansPlan([1000], torch.float32, DEV)
    t = [torch.zeros(1000, device=DEV)]
    hp = _khp(LansHParams())
    with pytest.raises(_lib.RafHipError) as e:
        plan.step(t, t, t, t, 1, hp, workspace=torch.empty(64, dtype=torch.uint8, device=DEV))
    assert e.value.status == _lib.RAFHIP_ERR_WORKSPACE
    big = torch.empty(plan.workspace_bytes + 512, dtype=torch.uint8, device=DEV)
    start = (256 - big.data_ptr() % 256) % 256 + 4  # 4 bytes past a 256-byte boundary
    with pytest.raises(_lib.RafHipError, match="aligned"):
        plan.step(t, t, t, t, 1, hp, workspace=big[start:])
    bad = kernels.make_hparams(mode=2)
    with pytest.raises(_lib.RafHipError, match="mode"):
        plan.step(t, t, t, t, 1, bad)
    with pytest.raises(ValueError):
        plan.step(t + t, t, t, t, 1, hp)
    with pytest.raises(TypeError):
        plan.step([t[0].half()], t, t, t, 1, hp)
    with pytest.raises(TypeError):
        kernels.LansPlan([8], torch.float64, DEV)


# ------------------------------------------------------------------ the two schedules
def test_default_schedule_follows_list_length(native_libs, monkeypatch):
    """Lists of 64 Mi elements or more run pipelined, shorter ones phased; the environment variable
    and the per-plan setter override that."""
    from raf_amd import kernels

    monkeypatch.delenv("RAFHIP_LANS_SCHEDULE", raising=False)
    for sizes, want in (([1000, 5], "phased"), ([(1 << 26) - 1], "phased"), ([1 << 25, 1 << 25], "pipelined")):
        plan = kernels.LansPlan(sizes, torch.float32, DEV)
        assert plan.schedule == want, sizes
        plan.set_schedule("pipelined" if want == "phased" else "phased")
        assert plan.schedule != want
        plan.close()
    monkeypatch.setenv("RAFHIP_LANS_SCHEDULE", "pipelined")
    plan = kernels.LansPlan([1000, 5], torch.float32, DEV)
    assert plan.schedule == "pipelined"
    plan.close()
    # a plan option beats the environment, which beats the built-in choice
    plan = kernels.LansPlan([1000, 5], torch.float32, DEV, schedule=native_libs.RAFHIP_LANS_PHASED)
    assert plan.schedule == "phased"
    plan.close()
    with pytest.raises(TypeError, match="no plan option"):
        kernels.LansPlan([8], torch.float32, DEV, chunk=3)


@pytest.mark.parametrize("group_elems", [None, 1 << 20])
@pytest.mark.parametrize("g16", [False, True])
def test_pipelined_schedule_is_bitwise_equal_to_phased(native_libs, monkeypatch, g16, group_elems):
    """The persistent, cache-aware schedule runs the same per-chunk code and adds the same partials
    in the same order as the one-launch-per-pass schedule: every output bit must agree, and both must
    match the oracle."""
    from raf_amd import kernels, shapes

    if group_elems is not None:  # small cache groups: many rounds, three passes in flight at once
        monkeypatch.setenv("RAFHIP_LANS_GROUP_ELEMS", str(group_elems))
    cases = {
        "edge": [1, 3, 4, 5, 0, 255, 1023, 8191, 8192, 8193, 16385, 65537, 100003],
        "many small": shapes.log_uniform_numels(400, seed=3),
        "several groups": [1 << 20, 3, 5000, (1 << 22) + 7, 1 << 19, 12345, 1 << 21, 3 << 20],
    }
    hp = LansHParams(grad_unscale=(1 / 1024 if g16 else 1.0))
    for name, sizes in cases.items():
        g, w, m, v = lans_inputs(sizes, cfg=80, g16=g16)
        results = {}
        for schedule in ("phased", "pipelined"):
            tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
            plan = kernels.LansPlan(sizes, tg[0].dtype, DEV)
            plan.set_schedule(schedule)
            for step in (2, 3):
                plan.step(tg, tw, tm, tv, torch.tensor(float(step), device=DEV), _khp(hp))
            torch.cuda.synchronize()
            norms = plan.read_norms()  # also raises if a bounded wait of the pipelined kernel ran out
            results[schedule] = ([t.cpu().numpy() for t in tw + tm + tv], norms)
            plan.close()
        for a, b in zip(results["phased"][0], results["pipelined"][0]):
            assert np.array_equal(a, b), name
        assert np.array_equal(results["phased"][1], results["pipelined"][1]), name
        ow, om, ov = w, m, v
        for step in (2, 3):
            ow, om, ov, on = lans_f64.lans_step(g, ow, om, ov, step, hp)
        _assert_close(results["pipelined"][0], ow + om + ov, TOL_1, name)
        _assert_norms(results["pipelined"][1], on)


@pytest.mark.parametrize("copy16", [False, True])
def test_sliced_last_pass_of_streaming_lists_is_bitwise_equal(native_libs, monkeypatch, copy16):
    """Lists beyond the cache run the phased schedule's last pass in 1024-element slices of a chunk,
    one workgroup each.  Forced onto short ragged lists (resident limit 0), every slice size gives
    the unsliced pass's bits, which are the pipelined schedule's; unaligned tensors (scalar path)
    and the 16-bit weight copies included."""
    from raf_amd import kernels

    sizes = [1, 3, 4, 5, 0, 255, 1023, 1024, 1025, 4095, 4097, 8191, 8192, 8193, 16385, 65537, 100003,
             (1 << 20) + 1029, 12345]
    g, w, m, v = lans_inputs(sizes, cfg=81, g16=True)
    hp = LansHParams(grad_unscale=1 / 1024)
    results = {}
    for variant in ("pipelined", "0", "10", "11", "12"):
        options = {"resident_mib": 0}  # treat even these short lists as far larger than the cache
        if variant != "pipelined":
            options["apply_slice_shift"] = int(variant)
        tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
        # every third tensor starts 4 bytes off a 16-byte boundary
        backing = [torch.zeros(n + 1, device=DEV) for n in sizes]
        for i in range(0, len(sizes), 3):
            off = backing[i][1:]
            off.copy_(tw[i])
            tw[i] = off
        tp = [torch.zeros(n, dtype=torch.float16, device=DEV) for n in sizes] if copy16 else None
        plan = kernels.LansPlan(sizes, tg[0].dtype, DEV, **options)
        plan.set_schedule("pipelined" if variant == "pipelined" else "phased")
        for step in (1, 2):
            plan.step(tg, tw, tm, tv, step, _khp(hp), p=tp)
        torch.cuda.synchronize()
        plan.read_norms()
        results[variant] = [t.cpu().numpy() for t in tw + tm + tv + (tp or [])]
        plan.close()
    for variant in ("0", "10", "11", "12"):
        for i, (a, b) in enumerate(zip(results["pipelined"], results[variant])):
            assert np.array_equal(a, b), (variant, i)
    ow, om, ov = w, m, v
    for step in (1, 2):
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, step, hp)
    _assert_close(results["10"][:3 * len(sizes)], ow + om + ov, TOL_1, "sliced")


def test_random_lists_groupings_and_slicings_agree_bitwise(native_libs, monkeypatch):
    """Whatever the list looks like and however the pipelined work list is cut (cache-group size,
    slices per round, resident workgroups), the result is the phased schedule's, bit for bit, and no
    bounded wait runs out."""
    from raf_amd import kernels

    rng = np.random.default_rng(9)
    hp = LansHParams()
    for case in range(24):
        n = int(rng.integers(1, 40))
        kinds = rng.integers(0, 4, n)
        sizes = [int(x) for x in np.where(kinds == 0, rng.integers(0, 64, n),          # tiny, some empty
                                 np.where(kinds == 1, rng.integers(1000, 9000, n),      # around one chunk
                                 np.where(kinds == 2, rng.integers(20_000, 200_000, n),  # a few chunks
                                          rng.integers(500_000, 1_500_000, n))))]       # large-chunk tensors
        g, w, m, v = lans_inputs(sizes, cfg=200 + case, g16=bool(case % 2))
        hp_case = LansHParams(grad_unscale=(1 / 1024 if case % 2 else 1.0), mode=int(case % 3 == 0))
        outs = []
        for schedule in ("phased", "pipelined"):
            options = {}
            if schedule == "pipelined":
                options = dict(
                    group_elements=int(rng.choice([1, 50_000, 400_000, 3_000_000])),
                    round_slices=int(rng.choice([1, 2, 8, 64, 4096])),
                    blocks_per_cu=int(rng.choice([1, 2, 3])),
                    # tensors from this size on are treated as too large for the cache: their items
                    # are marked streaming and merged into the list of the cached groups
                    stream_from_elements=int(rng.choice([50_000, 600_000, 10**9])),
                    stream_hold_items=int(rng.choice([0, 7, 3072])))
            tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
            plan = kernels.LansPlan(sizes, tg[0].dtype, DEV, **options)
            plan.set_schedule(schedule)
            for step in (1, 2):
                plan.step(tg, tw, tm, tv, step, _khp(hp_case))
            torch.cuda.synchronize()
            norms = plan.read_norms()  # raises if a wait ran out
            outs.append(([t.cpu().numpy() for t in tw + tm + tv], norms))
            plan.close()
        for a, b in zip(outs[0][0], outs[1][0]):
            assert np.array_equal(a, b), (case, sizes)
        assert np.array_equal(outs[0][1], outs[1][1]), (case, sizes)
        if case < 6:  # and both are the oracle's
            ow, om, ov = w, m, v
            for step in (1, 2):
                ow, om, ov, on = lans_f64.lans_step(g, ow, om, ov, step, hp_case)
            _assert_close(outs[1][0], ow + om + ov, TOL_1, f"case {case}")


# ------------------------------------------------------------------ graph capture
@pytest.mark.parametrize("schedule", ["phased", "pipelined"])
def test_step_can_be_captured_in_a_hip_graph(native_libs, schedule):
    """A step enqueues kernels only (no allocation, no host synchronisation once the pointer table
    has been sent), so it can be captured; every replay, with eager work and synchronisations in
    between, must give the bits of the eager step from the same state."""
    from raf_amd import kernels

    sizes = [70001, 5, 8192, 300000, 1]
    g, w, m, v = lans_inputs(sizes, cfg=85)
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.set_schedule(schedule)
    plan.bind(tg, tw, tm, tv, _khp(LansHParams()))
    step = torch.full((), 1.0, device=DEV)

    def one_step():
        plan.step_bound(step)
        step.add_(1.0)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the side stream: the pointer table goes out here
        one_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        one_step()
    torch.cuda.synchronize()
    for _ in range(4):
        state = [t.clone() for t in tw + tm + tv] + [step.clone()]
        one_step()  # eager
        torch.cuda.synchronize()
        want = [t.clone() for t in tw + tm + tv]
        for dst, src in zip(tw + tm + tv + [step], state):
            dst.copy_(src)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(tw + tm + tv, want))
        assert plan.read_norms().shape == (len(sizes), 4)
    plan.close()


def test_a_captured_step_keeps_its_pointer_table(native_libs):
    """A graph replays kernels that read one of the plan's device tables.  The table a step was
    captured with is held: eager steps with five other gradient lists afterwards (more than the
    plan has tables) must not overwrite it, so a replay still updates the captured tensors with the
    captured gradients; a capture whose pointers are new to the plan (no warm-up with them) sends
    them inside the graph and is held likewise; and once every table is held by a graph, pointers
    the plan has never seen are refused instead of evicting one."""
    from raf_amd import kernels
    from raf_amd._lib import RAFHIP_TABLE_SLOTS

    sizes = [70001, 5, 8192, 300000, 1]
    hp = LansHParams()
    g, w, m, v = lans_inputs(sizes, cfg=87)
    others = [lans_inputs(sizes, cfg=88 + k)[0] for k in range(RAFHIP_TABLE_SLOTS + 1)]
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    tothers = [_to_dev(o) for o in others]
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    step = torch.full((), 1.0, device=DEV)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        plan.step(tg, tw, tm, tv, step, _khp(hp))  # warm-up: the table goes out, the workspace exists
        step.add_(1.0)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.step(tg, tw, tm, tv, step, _khp(hp))
        step.add_(1.0)
    torch.cuda.synchronize()
    ow, om, ov, _ = lans_f64.lans_step(g, w, m, v, 1, hp)      # the warm-up; a capture runs nothing
    n_steps = 1
    uploads = plan.table_uploads
    for k, other in enumerate(tothers):                       # five other lists: every free table is reused
        plan.step(other, tw, tm, tv, step, _khp(hp))
        step.add_(1.0)
        n_steps += 1
        ow, om, ov, _ = lans_f64.lans_step(others[k], ow, om, ov, n_steps, hp)
    assert plan.table_uploads == uploads + len(tothers)
    torch.cuda.synchronize()
    for _ in range(2):
        graph.replay()                                         # still the first gradient list
        n_steps += 1
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, n_steps, hp)
    torch.cuda.synchronize()
    plan.read_norms()
    _assert_close([t.cpu().numpy() for t in tw], ow, 1e-4, "w")
    _assert_close([t.cpu().numpy() for t in tv], ov, 1e-4, "v")

    # captures with pointers the plan has not seen: sent inside the graph, held, replayable
    graphs = [graph]
    for k in range(RAFHIP_TABLE_SLOTS - 1):
        fresh = [t.clone() for t in tothers[k]]
        tothers.append(fresh)  # keep alive
        gk = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gk):
            plan.step(fresh, tw, tm, tv, step, _khp(hp))
            step.add_(1.0)
        graphs.append((gk, k))
    torch.cuda.synchronize()
    for gk, k in graphs[1:]:
        gk.replay()
        n_steps += 1
        ow, om, ov, _ = lans_f64.lans_step(others[k], ow, om, ov, n_steps, hp)
    torch.cuda.synchronize()
    _assert_close([t.cpu().numpy() for t in tw], ow, 1e-4, "w")
    # every table is held now: a list the plan does not know is refused, a held one still runs
    with pytest.raises(RuntimeError, match="held by captured graphs"):
        plan.step(tothers[RAFHIP_TABLE_SLOTS], tw, tm, tv, step, _khp(hp))
    plan.step(tg, tw, tm, tv, step, _khp(hp))
    n_steps += 1
    ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, n_steps, hp)
    torch.cuda.synchronize()
    _assert_close([t.cpu().numpy() for t in tw], ow, 1e-4, "w")
    _assert_close([t.cpu().numpy() for t in tm], om, 1e-4, "m")
    plan.close()


def test_same_tensors_on_another_stream(native_libs):
    """The pointer table is uploaded on the first call's stream; a second call with the same tensors
    on another stream must still see it (the library orders the new stream behind the upload)."""
    from raf_amd import kernels

    sizes = [300000, 17, 70001]
    g, w, m, v = lans_inputs(sizes, cfg=86)
    hp = LansHParams()
    ow, om, ov = w, m, v
    for step in (1, 2):
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, step, hp)
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        plan.step(tg, tw, tm, tv, 1, _khp(hp))
    s2.wait_stream(s1)  # the caller orders the two steps; the table upload is the library's business
    with torch.cuda.stream(s2):
        plan.step(tg, tw, tm, tv, 2, _khp(hp))
    torch.cuda.synchronize()
    _assert_close([t.cpu().numpy() for t in tw], ow, TOL_1, "w")
    plan.close()


def test_a_wait_that_runs_out_is_reported_not_hung(native_libs, monkeypatch):
    """Every wait of the persistent kernel is bounded.  With the bound forced to zero polls from the
    host, waits give up at once: the kernel still drains, the step's results are declared invalid by
    rafhip_lans_read_norms, and the next plan (default bound) works as usual."""
    from raf_amd import kernels

    sizes = [1 << 22, 3 << 20, 70001]
    g, w, m, v = lans_inputs(sizes, cfg=87)
    hp = LansHParams()
    monkeypatch.setenv("RAFHIP_LANS_SPIN_LIMIT", "0")
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.set_schedule("pipelined")
    plan.step(tg, tw, tm, tv, 1, _khp(hp))
    torch.cuda.synchronize()  # returns: no workgroup is left waiting
    with pytest.raises(native_libs.RafHipError, match="bounded wait"):
        plan.read_norms()
    # a caller that never reads the norms learns of it from the next step on the plan, once
    plan.step(tg, tw, tm, tv, 2, _khp(hp))  # the report above cleared the flag: this one runs (and times out)
    torch.cuda.synchronize()
    with pytest.raises(native_libs.RafHipError, match="earlier pipelined step .* bounded wait"):
        plan.step(tg, tw, tm, tv, 3, _khp(hp))
    plan.set_schedule("phased")
    plan.step(tg, tw, tm, tv, 3, _khp(hp))  # reported once; the plan works on
    torch.cuda.synchronize()
    plan.close()
    monkeypatch.delenv("RAFHIP_LANS_SPIN_LIMIT")
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.set_schedule("pipelined")
    plan.step(tg, tw, tm, tv, 1, _khp(hp))
    torch.cuda.synchronize()
    ow, _, _, on = lans_f64.lans_step(g, w, m, v, 1, hp)
    _assert_norms(plan.read_norms(), on)
    _assert_close([t.cpu().numpy() for t in tw], ow, TOL_1, "w")
    plan.close()


@pytest.mark.parametrize("bad", [np.inf, np.nan])
def test_overflowed_gradient_poisons_only_its_tensor(native_libs, bad):
    """A loss-scale overflow leaves inf / NaN in a half gradient.  The rule then turns that tensor's
    w, m, v into NaN (as the reference's arithmetic would); the other tensors are untouched by it,
    both schedules agree on where the NaNs are, and the persistent kernel's waits are not confused
    by NaN partial sums (its 'not ready' pattern is itself a NaN)."""
    from raf_amd import kernels

    sizes = [30000, 70001, 9000]
    hp = LansHParams(grad_unscale=1 / 1024)
    g, w, m, v = lans_inputs(sizes, cfg=88, g16=True)
    g[1][12345] = np.float16(bad)
    ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 2, hp)
    assert np.isnan(ow[1]).all() and not np.isnan(ow[0]).any() and not np.isnan(ow[2]).any()
    outs = {}
    for schedule in ("phased", "pipelined"):
        tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
        plan = kernels.LansPlan(sizes, torch.float16, DEV)
        plan.set_schedule(schedule)
        plan.step(tg, tw, tm, tv, 2, _khp(hp))
        torch.cuda.synchronize()
        norms = plan.read_norms()
        outs[schedule] = [t.cpu().numpy() for t in tw + tm + tv]
        plan.close()
        for q, want in zip((0, 3, 6), (ow, om, ov)):
            got = outs[schedule][q:q + 3]
            assert np.array_equal(np.isnan(got[1]), np.isnan(want[1]))
            _assert_close([got[0], got[2]], [want[0], want[2]], TOL_1, schedule)
        assert np.isnan(norms[1][0]) or np.isinf(norms[1][0])
        _assert_norms(norms[[0, 2]], on[[0, 2]])
    for a, b in zip(outs["phased"], outs["pipelined"]):
        assert np.array_equal(a, b, equal_nan=True)


def test_two_persistent_kernels_side_by_side(native_libs):
    """Two plans stepping on two streams at once share the CUs.  A waiting workgroup only ever
    depends on items with earlier tickets, which running workgroups hold, so neither kernel needs
    all of its workgroups resident; both must finish and match the oracle."""
    from raf_amd import kernels

    hp = LansHParams()
    lists = [[1 << 22, 3 << 20, 70001, 1 << 21], [5 << 20, 1 << 20, 9, 1 << 22]]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    state = []
    for cfg, sizes in enumerate(lists):
        g, w, m, v = lans_inputs(sizes, cfg=89 + cfg)
        plan = kernels.LansPlan(sizes, torch.float32, DEV)
        plan.set_schedule("pipelined")
        state.append((g, w, m, v, plan, _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)))
    torch.cuda.synchronize()
    for step in (1, 2, 3):
        for (g, w, m, v, plan, tg, tw, tm, tv), s in zip(state, streams):
            with torch.cuda.stream(s):
                plan.step(tg, tw, tm, tv, step, _khp(hp))
    torch.cuda.synchronize()
    for g, w, m, v, plan, tg, tw, tm, tv in state:
        ow, om, ov = w, m, v
        for step in (1, 2, 3):
            ow, om, ov, on = lans_f64.lans_step(g, ow, om, ov, step, hp)
        _assert_norms(plan.read_norms(), on)
        _assert_close([t.cpu().numpy() for t in tw], ow, TOL_1, "w")
        plan.close()


def test_a_step_that_runs_out_of_a_wait_leaves_old_or_new_values(native_libs, monkeypatch):
    """Whatever consumes a value that never arrived passes a 'lost' marker on instead of computing
    with it, and the third pass skips the stores of an element whose parameters are lost: after a
    step that reported a time-out every element of w, m and v holds either its old value or the
    value a good step gives it -- all three of one element from the same side -- never garbage."""
    from raf_amd import kernels

    sizes = [1 << 22, 3 << 20, 70001, 5000, 1 << 21]
    g, w, m, v = lans_inputs(sizes, cfg=93)
    hp = LansHParams()
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.set_schedule("pipelined")
    plan.step(tg, tw, tm, tv, 2, _khp(hp))
    torch.cuda.synchronize()
    plan.read_norms()  # a good step: no report
    plan.close()
    new = [[t.cpu().numpy() for t in ts] for ts in (tw, tm, tv)]

    monkeypatch.setenv("RAFHIP_LANS_SPIN_LIMIT", "0")
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.set_schedule("pipelined")
    plan.step(tg, tw, tm, tv, 2, _khp(hp))
    torch.cuda.synchronize()
    monkeypatch.delenv("RAFHIP_LANS_SPIN_LIMIT")
    with pytest.raises(native_libs.RafHipError, match="bounded wait"):
        plan.read_norms()
    plan.close()
    got = [[t.cpu().numpy() for t in ts] for ts in (tw, tm, tv)]
    old = [w, m, v]
    for t in range(len(sizes)):
        is_new = [got[q][t].view(np.uint32) == new[q][t].view(np.uint32) for q in range(3)]
        is_old = [got[q][t].view(np.uint32) == old[q][t].view(np.uint32) for q in range(3)]
        for q in range(3):
            assert np.all(is_new[q] | is_old[q]), f"tensor {t}, array {'wmv'[q]}: a value that is neither old nor new"
        # an element is updated as a whole or not at all (where old and new differ, which they do
        # for m and v of every element with a non-zero gradient)
        updated = is_new[1] & ~is_old[1]
        kept = is_old[1] & ~is_new[1]
        assert not np.any(updated & ~is_new[0]) and not np.any(updated & ~is_new[2])
        assert not np.any(kept & ~is_old[0]) and not np.any(kept & ~is_old[2])


def test_workspace_needs_only_16_byte_alignment(native_libs):
    """RAF's memory pools hand out blocks aligned to 64 bytes (include/raf/memory_pool.h), not 256:
    a workspace at such an address must be accepted and give the same bits."""
    from raf_amd import kernels

    sizes = [70001, 300000, 9]
    g, w, m, v = lans_inputs(sizes, cfg=94)
    outs = []
    for offset in (0, 64, 16):
        tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
        plan = kernels.LansPlan(sizes, torch.float32, DEV)
        for schedule in ("phased", "pipelined"):
            plan.set_schedule(schedule)
            block = torch.empty(plan.workspace_bytes + 256, dtype=torch.uint8, device=DEV)
            ws = block[offset:offset + plan.workspace_bytes]
            assert ws.data_ptr() % 256 == offset
            plan.step(tg, tw, tm, tv, 1 if schedule == "phased" else 2, _khp(LansHParams()), workspace=ws)
        torch.cuda.synchronize()
        outs.append([t.cpu().numpy() for t in tw + tm + tv])
        plan.close()
    for other in outs[1:]:
        assert all(np.array_equal(a, b) for a, b in zip(outs[0], other))
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    block = torch.empty(plan.workspace_bytes + 256, dtype=torch.uint8, device=DEV)
    with pytest.raises(native_libs.RafHipError, match="16-byte aligned"):
        plan.step(tg, tw, tm, tv, 1, _khp(LansHParams()), workspace=block[8:8 + plan.workspace_bytes])
    plan.close()


@pytest.mark.parametrize("schedule", ["phased", "pipelined"])
def test_bound_form_equals_the_unbound_step(native_libs, schedule):
    """rafhip_lans_plan_bind + rafhip_lans_step_bound: same bits as rafhip_lans_step_mixed, over
    several steps, after binding other tensors, and with unbound steps on the same plan in between."""
    from raf_amd import kernels

    sizes = [70001, 5, 8192, 300000, 1, 0]
    hp = _khp(LansHParams())
    ga, wa, ma, va = lans_inputs(sizes, cfg=95)
    gb, wb, mb, vb = lans_inputs(sizes, cfg=96)

    def run(bound):
        A = [_to_dev(x) for x in (ga, wa, ma, va)]
        B = [_to_dev(x) for x in (gb, wb, mb, vb)]
        plan = kernels.LansPlan(sizes, torch.float32, DEV)
        plan.set_schedule(schedule)
        step = torch.zeros((), device=DEV)

        def do(lst, rebind):
            step.add_(1.0)
            if bound:
                if rebind:
                    plan.bind(*lst, hp)
                plan.step_bound(step)
            else:
                plan.step(*lst, step, hp)

        do(A, True)
        do(A, False)
        do(B, True)
        do(B, False)
        step.add_(1.0)
        plan.step(*A, step, hp)  # an unbound step takes the device table away from the bound tensors ...
        do(B, False)             # ... and the next bound step brings it back
        torch.cuda.synchronize()
        plan.close()
        return [t.cpu().numpy() for lst in (A, B) for ts in lst[1:] for t in ts]

    for a, b in zip(run(False), run(True)):
        assert np.array_equal(a, b)


def test_bound_step_without_binding_is_an_error(native_libs):
    from raf_amd import _lib, kernels
    import ctypes

    plan = kernels.LansPlan([100], torch.float32, DEV)
    hp = _khp(LansHParams())
    st = plan.lib.rafhip_lans_step_bound(plan._h, None, 1, ctypes.byref(hp), plan.workspace.data_ptr(),
                                         plan.workspace.numel(), None)
    assert st == _lib.RAFHIP_ERR_INVALID_ARG and "rafhip_lans_plan_bind" in _lib.last_error()
    plan.close()


def test_two_lists_alternating_on_two_streams_through_one_plan(native_libs):
    """The device pointer table is rewritten when the pointers change.  A kernel launched earlier on
    another stream may still be reading it: the library orders the new stream behind the previous
    one before it overwrites the table, so steps on one plan are serialised whatever stream they
    are issued on, and each gets its own list's pointers."""
    from raf_amd import kernels

    sizes = [3 << 20, 1 << 22, 70001, 2 << 20]
    hp = LansHParams()
    lists = []
    for cfg in (97, 98):
        g, w, m, v = lans_inputs(sizes, cfg=cfg)
        lists.append((g, w, m, v, _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)))
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.set_schedule("pipelined")
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for step in (1, 2, 3):
        for (g, w, m, v, tg, tw, tm, tv), s in zip(lists, streams):
            with torch.cuda.stream(s):
                plan.step(tg, tw, tm, tv, step, _khp(hp))
    torch.cuda.synchronize()
    for g, w, m, v, tg, tw, tm, tv in lists:
        ow, om, ov = w, m, v
        for step in (1, 2, 3):
            ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, step, hp)
        _assert_close([t.cpu().numpy() for t in tw], ow, TOL_1, "w")
        _assert_close([t.cpu().numpy() for t in tv], ov, TOL_1, "v")
    plan.close()


def test_alternating_pointer_lists_stop_uploading(native_libs):
    """A plan keeps a device pointer table per recent pointer list: gradients that alternate between
    two allocations (what an executor that allocates them per iteration produces) cost two uploads
    in all, a list seen before is found again after others were used, a fifth distinct list replaces
    the least recently used one -- and every step reads the right table (checked against the oracle
    with different gradient values in every allocation)."""
    from raf_amd import kernels

    sizes = [70001, 5, 1 << 16, 4096, 300_000]
    hp = LansHParams()
    _, w, m, v = lans_inputs(sizes, cfg=120)
    grads = [lans_inputs(sizes, cfg=121 + k)[0] for k in range(5)]
    tw, tm, tv = _to_dev(w), _to_dev(m), _to_dev(v)
    tgs = [_to_dev(g) for g in grads]
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    order = [0, 1, 0, 1, 0, 1, 2, 0, 3, 4, 1, 1]
    uploads = []
    for i, k in enumerate(order):
        plan.step(tgs[k], tw, tm, tv, i + 1, _khp(hp))
        uploads.append(plan.table_uploads)
    torch.cuda.synchronize()
    plan.read_norms()
    #            0  1  0  1  0  1  2  0  3  4  1 (evicted by 4: sent again)  1
    assert uploads == [1, 2, 2, 2, 2, 2, 3, 3, 4, 5, 6, 6], uploads
    ow, om, ov = w, m, v
    for i, k in enumerate(order):
        ow, om, ov, _ = lans_f64.lans_step(grads[k], ow, om, ov, i + 1, hp)
    _assert_close([t.cpu().numpy() for t in tw], ow, 1e-4, "w")
    _assert_close([t.cpu().numpy() for t in tv], ov, 1e-4, "v")
    plan.close()


def test_per_kernel_timing_slots(native_libs):
    """rafhip_lans_timing_*: five intervals per step, zero where the schedule launches nothing."""
    from raf_amd import kernels

    hp = LansHParams()
    cases = [("pipelined", [1 << 20, 70001], [True, True, False, False, False]),
             ("phased", [1 << 20, 70001], [True] * 5),          # a long tensor: the two finish launches run
             ("phased", [70001, 5, 4096], [True, False, True, False, True])]  # short tensors: they do not
    for schedule, sizes, nonzero in cases:
        g, w, m, v = lans_inputs(sizes, cfg=95)
        tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
        plan = kernels.LansPlan(sizes, torch.float32, DEV)
        plan.set_schedule(schedule)
        plan.timing_enable(2)
        with pytest.raises(native_libs.RafHipError, match="holds no step"):
            plan.timing_read(0)
        for step in (1, 2, 3):
            plan.step(tg, tw, tm, tv, step, _khp(hp))
        torch.cuda.synchronize()
        for slot in (0, 1):
            ms = plan.timing_read(slot)
            assert len(ms) == 5 and all(x >= 0.0 for x in ms)
            assert [x > 0.0 for x in ms] == nonzero, (schedule, sizes, ms)
            assert sum(ms) < 50.0
        plan.timing_enable(0)
        plan.step(tg, tw, tm, tv, 4, _khp(hp))
        torch.cuda.synchronize()
        plan.close()
