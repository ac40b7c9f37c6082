"""GPU parity of the mixed-precision LANS step (half gradients in, half weight copies out), called
through the C ABI: bfloat16 / float16 gradients against the float64 oracle (1e-5 per element), and
the 16-bit weight copies bit-exactly against the round-to-nearest-even narrowing of the fp32
weights the same step stored."""
import numpy as np
import pytest
import torch

from oracle import halfs, lans_f64
from oracle.lans_f64 import LansHParams
from tests.helpers import lans_inputs, max_rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL_1 = 1e-5
TOL_100 = 1e-4
EDGE_SIZES = [1, 3, 4, 5, 0, 255, 256, 257, 1023, 8191, 8192, 8193, 16385, 65537, 100003]
TORCH_DT = {"float16": torch.float16, "bfloat16": torch.bfloat16}


def _dev_grad(a):
    if a.dtype == np.uint16:  # bfloat16 bit patterns
        return torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16)
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _to_dev(arrs):
    return [_dev_grad(a) for a in arrs]


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _khp(hp):
    from raf_amd import kernels

    return kernels.make_hparams(hp.learning_rate, hp.beta1, hp.beta2, hp.eps, hp.bias_correction,
                                hp.weight_decay, hp.grad_averaging, hp.mode, hp.normalize_grad,
                                hp.grad_unscale)


def _run(g, w, m, v, hp, steps, model_dtype=None, schedule=None, skip=(), first_step=1):
    """Returns (w, m, v as fp32 arrays, p as uint16 bit patterns or None per tensor, norms)."""
    from raf_amd import kernels

    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    tp = None
    if model_dtype:
        tp = [None if t in skip else torch.full((a.size,), 7.0, dtype=TORCH_DT[model_dtype], device=DEV)
              for t, a in enumerate(w)]
    plan = kernels.LansPlan([a.size for a in w], tg[0].dtype, DEV)
    if schedule:
        plan.set_schedule(schedule)
    for s in range(steps):
        plan.step(tg, tw, tm, tv, torch.tensor(float(first_step + s), device=DEV), _khp(hp), p=tp)
    torch.cuda.synchronize()
    norms = plan.read_norms()
    plan.close()
    back = lambda ts: [t.cpu().numpy() for t in ts]
    ps = None if tp is None else [None if t is None else _bits(t) for t in tp]
    return back(tw), back(tm), back(tv), ps, norms


def _assert_close(got, want, tol, what):
    for t, (a, b) in enumerate(zip(got, want)):
        e = max_rel_err(a, b)
        assert e <= tol, f"{what}[{t}] max rel err {e:.3e} > {tol}"


@pytest.mark.parametrize("mode", [0, 1])
def test_bf16_gradients_against_oracle(native_libs, mode):
    hp = LansHParams(mode=mode, grad_unscale=1 / 1024)
    g, w, m, v = lans_inputs(EDGE_SIZES, cfg=90 + mode, g16="bfloat16")
    ow, om, ov, on = lans_f64.lans_step(g, w, m, v, 3, hp)
    gw, gm, gv, _, gn = _run(g, w, m, v, hp, 1, first_step=3)
    _assert_close(gw, ow, TOL_1, "w")
    _assert_close(gm, om, TOL_1, "m")
    _assert_close(gv, ov, TOL_1, "v")
    nz = on != 0
    assert np.max(np.abs(gn[nz] - on[nz]) / on[nz]) < 1e-10


def test_bf16_widening_matches_float32_gradients_bitwise(native_libs):
    """A bfloat16 gradient and the same values handed over as float32 must give identical bits:
    widening is exact, so the fused ingest equals group_cast followed by the fp32 op."""
    hp = LansHParams(grad_unscale=1 / 1024)
    g, w, m, v = lans_inputs([5000, 70001, 9], cfg=92, g16="bfloat16")
    a = _run(g, w, m, v, hp, 2)
    b = _run([halfs.bf16_bits_to_f32(x) for x in g], w, m, v, hp, 2)
    for x, y in zip(a[0] + a[1] + a[2], b[0] + b[1] + b[2]):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("g16", ["float16", "bfloat16"])
@pytest.mark.parametrize("model_dtype", ["float16", "bfloat16"])
def test_weight_copy_is_the_rounded_stored_weight(native_libs, g16, model_dtype):
    hp = LansHParams(grad_unscale=1 / 1024)
    g, w, m, v = lans_inputs(EDGE_SIZES, cfg=93, g16=g16)
    plain = _run(g, w, m, v, hp, 2)
    mixed = _run(g, w, m, v, hp, 2, model_dtype=model_dtype)
    for x, y in zip(plain[0] + plain[1] + plain[2], mixed[0] + mixed[1] + mixed[2]):
        assert np.array_equal(x, y), "writing the copies must not change w, m, v"
    assert np.array_equal(plain[4], mixed[4])
    for t, (w32, p) in enumerate(zip(mixed[0], mixed[3])):
        want = halfs.narrow_weight(w32, model_dtype).view(np.uint16)
        assert np.array_equal(p, want), f"tensor {t}"
    # and against the oracle's own mixed step: at most one 16-bit ulp where the fp32 weights differ
    ow, om, ov, op, _ = lans_f64.lans_mixed_step(g, w, m, v, 1, hp, model_dtype)
    ow, om, ov, op, _ = lans_f64.lans_mixed_step(g, ow, om, ov, 2, hp, model_dtype)
    _assert_close(mixed[0], ow, TOL_1, "w")
    for p, o in zip(mixed[3], op):
        d = np.abs(p.astype(np.int32) - o.view(np.uint16).astype(np.int32))
        assert d.max(initial=0) <= 1
        assert (d != 0).mean() < 1e-3 if d.size > 1000 else True


def test_special_values_in_the_copy(native_libs):
    """Overflow to infinity, binary16 subnormals and zeros through the narrowing, lr = 0 so that the
    stored weight is the input weight."""
    hp = LansHParams(learning_rate=0.0, weight_decay=0.0)
    w0 = np.array([65504.0, 65519.0, 65520.0, 1e5, -1e5, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 6e-8,
                   1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 0.0, -0.0, 3.0e38, 1e-40], np.float32)
    g = [np.full(w0.size, 1e-3, np.float32)]
    for model_dtype in ("float16", "bfloat16"):
        out = _run(g, [w0], [np.zeros_like(w0)], [np.zeros_like(w0)], hp, 1, model_dtype=model_dtype)
        assert np.array_equal(out[0][0].view(np.uint32), w0.view(np.uint32))
        assert np.array_equal(out[3][0], halfs.narrow_weight(w0, model_dtype).view(np.uint16))


def test_skipped_and_unaligned_copies(native_libs):
    """NULL entries leave that tensor without a copy; a copy that is only 2-byte aligned takes the
    element-wise path and gives the same bits."""
    from raf_amd import kernels

    hp = LansHParams()
    sizes = [4099, 20000, 8192]
    g, w, m, v = lans_inputs(sizes, cfg=94)
    ref = _run(g, w, m, v, hp, 1, model_dtype="float16")
    part = _run(g, w, m, v, hp, 1, model_dtype="float16", skip=(1,))
    assert part[3][1] is None
    assert np.array_equal(part[3][0], ref[3][0]) and np.array_equal(part[3][2], ref[3][2])
    tg, tw, tm, tv = _to_dev(g), _to_dev(w), _to_dev(m), _to_dev(v)
    backing = [torch.zeros(n + 8, dtype=torch.float16, device=DEV) for n in sizes]
    tp = [b[1:1 + n] for b, n in zip(backing, sizes)]  # 2-byte aligned views
    plan = kernels.LansPlan(sizes, torch.float32, DEV)
    plan.step(tg, tw, tm, tv, 1, _khp(hp), p=tp)
    torch.cuda.synchronize()
    for t in range(3):
        assert np.array_equal(_bits(tp[t]), ref[3][t])
        assert np.array_equal(tw[t].cpu().numpy(), ref[0][t])
        assert float(backing[t][0]) == 0.0 and float(backing[t][1 + sizes[t]:].abs().sum()) == 0.0
    plan.close()


@pytest.mark.parametrize("g16", ["float16", "bfloat16"])
def test_schedules_agree_bitwise_with_copies(native_libs, monkeypatch, g16):
    monkeypatch.setenv("RAFHIP_LANS_GROUP_ELEMS", str(1 << 20))
    hp = LansHParams(grad_unscale=1 / 1024)
    sizes = [1 << 20, 3, 5000, (1 << 21) + 7, 1 << 19, 12345, 8192, 3 << 19]
    g, w, m, v = lans_inputs(sizes, cfg=95, g16=g16)
    a = _run(g, w, m, v, hp, 2, model_dtype=g16, schedule="phased")
    b = _run(g, w, m, v, hp, 2, model_dtype=g16, schedule="pipelined")
    for x, y in zip(a[0] + a[1] + a[2] + a[3], b[0] + b[1] + b[2] + b[3]):
        assert np.array_equal(x, y)
    assert np.array_equal(a[4], b[4])
    ow, om, ov = w, m, v
    for step in (1, 2):
        ow, om, ov, _ = lans_f64.lans_step(g, ow, om, ov, step, hp)
    _assert_close(b[0], ow, TOL_1, "w")


def test_hundred_mixed_steps(native_libs, c_oracle):
    """bf16 gradients, bf16 copies, 100 steps: w, m, v within 1e-4 of the oracle, copies equal to
    the narrowing of the final fp32 weights."""
    hp = LansHParams(grad_unscale=1 / 1024)
    sizes = [30000, 77, 262144 + 5]
    g, w, m, v = lans_inputs(sizes, cfg=96, g16="bfloat16", zero_state=True)
    out = _run(g, w, m, v, hp, 100, model_dtype="bfloat16")
    ow, om, ov = [a.copy() for a in w], [a.copy() for a in m], [a.copy() for a in v]
    op = [np.zeros(a.size, np.uint16) for a in w]
    for step in range(1, 101):
        c_oracle.lans_step_inplace(g, ow, om, ov, step, hp, p_list=op, model_dtype="bfloat16")
    _assert_close(out[0], ow, TOL_100, "w")
    _assert_close(out[1], om, TOL_100, "m")
    _assert_close(out[2], ov, TOL_100, "v")
    for t in range(len(sizes)):
        assert np.array_equal(out[3][t], halfs.f32_to_bf16_bits(out[0][t]))
        d = np.abs(out[3][t].astype(np.int32) - op[t].astype(np.int32))
        assert d.max() <= 1


def test_mixed_argument_errors(native_libs):
    from raf_amd import kernels

    plan = kernels.LansPlan([16], torch.bfloat16, DEV)
    hp = kernels.make_hparams()
    f = [torch.zeros(16, device=DEV)]
    gb = [torch.zeros(16, device=DEV, dtype=torch.bfloat16)]
    with pytest.raises(TypeError):
        plan.step([f[0].half()], f, f, f, 1, hp)  # plan was made for bfloat16 gradients
    with pytest.raises(TypeError):
        plan.step(gb, f, f, f, 1, hp, p=[torch.zeros(16, device=DEV)])  # fp32 is not a 16-bit copy
    with pytest.raises(TypeError):
        plan.step(gb, f, f, f, 1, hp, p=[torch.zeros(8, device=DEV, dtype=torch.float16)])
    import ctypes

    lib = native_libs.optim()
    ptr = (ctypes.c_void_p * 1)(f[0].data_ptr())
    gp = (ctypes.c_void_p * 1)(gb[0].data_ptr())
    st = lib.rafhip_lans_step_mixed(plan._h, gp, ptr, ptr, ptr, ptr, 0, None, 1, ctypes.byref(hp),
                                    plan.workspace.data_ptr(), plan.workspace.numel(), None)
    assert st == native_libs.RAFHIP_ERR_UNSUPPORTED and b"weight-copy dtype" in lib.rafhip_last_error()
    plan.close()


# ------------------------------------------------------------------ committed fixtures
@pytest.mark.parametrize("name", ["f16_f16", "bf16_bf16", "bf16_f16"])
def test_mixed_golden_fixture(native_libs, name):
    """Mixed-precision LANS, multi-tensor SGD with half gradients and copies, against the stored
    vectors: LANS weights within 1e-5, their 16-bit copies equal to the narrowing of what was
    stored; SGD bit-exact on x, v and the copies."""
    from raf_amd import kernels
    from tests.golden import make_fixtures as mf

    z = np.load(mf.HERE / "mixed_kat.npz")
    gdt, mdt = mf.MIXED_CASES[name]
    nt = len(mf.MIXED_SIZES)
    g, w, m, v = ([z[f"lans/{name}/{q}{t}"] for t in range(nt)] for q in "gwmv")
    out = _run(g, w, m, v, LansHParams(grad_unscale=1 / 1024), 2, model_dtype=mdt, first_step=2)
    for t in range(nt):
        assert max_rel_err(out[0][t], z[f"lans/{name}/w{t}_after2"]) <= TOL_1
        assert np.array_equal(out[3][t], halfs.narrow_weight(out[0][t], mdt).view(np.uint16))
        d = np.abs(out[3][t].astype(np.int32) - z[f"lans/{name}/p{t}_after2"].astype(np.int32))
        assert d.max(initial=0) <= 1
    tx, td, tv = _to_dev(w), _to_dev(g), _to_dev(m)
    tp = [torch.zeros(a.size, dtype=TORCH_DT[mdt], device=DEV) for a in w]
    plan = kernels.SgdPlan([a.size for a in w], td[0].dtype, DEV)
    for _ in range(2):
        plan.step(tx, td, tv, 0.01, 0.9, p=tp)
    torch.cuda.synchronize()
    for t in range(nt):
        assert np.array_equal(tx[t].cpu().numpy().view(np.uint32), z[f"sgd/{name}/x{t}_after2"])
        assert np.array_equal(tv[t].cpu().numpy().view(np.uint32), z[f"sgd/{name}/v{t}_after2"])
        assert np.array_equal(_bits(tp[t]), z[f"sgd/{name}/p{t}_after2"])
    plan.close()
