"""The committed fixtures against the oracle (CPU): a change in the oracle's results, or a stale
fixture, fails here before it can mislead a GPU parity run."""
import numpy as np

from oracle import halfs, lans_f64, sgd_f32, tensor_ops
from tests.golden import make_fixtures as mf
from tests.helpers import max_rel_err

GOLDEN = mf.HERE


def test_sgd_fixture_matches_oracle_bitwise(c_oracle):
    z = np.load(GOLDEN / "sgd_kat.npz")
    v1, x1 = sgd_f32.sgd_step(z["x0"], z["dx"], z["v0"], float(z["learning_rate"]), float(z["mu"]))
    cv1, cx1 = c_oracle.sgd_step(z["x0"], z["dx"], z["v0"], float(z["learning_rate"]), float(z["mu"]))
    for got_v, got_x in ((v1, x1), (cv1, cx1)):
        nan_v = np.isnan(got_v)
        nan_x = np.isnan(got_x)
        # NaN payloads are not part of the contract; everything else is bit-exact
        assert np.array_equal(nan_v, np.isnan(z["v1_bits"].view(np.float32)))
        assert np.array_equal(nan_x, np.isnan(z["x1_bits"].view(np.float32)))
        assert np.array_equal(got_v.view(np.uint32)[~nan_v], z["v1_bits"][~nan_v])
        assert np.array_equal(got_x.view(np.uint32)[~nan_x], z["x1_bits"][~nan_x])
    assert nan_v.sum() >= 1 and np.isinf(v1).sum() >= 2  # the special lanes are really there


def test_lans_fixture_matches_oracle(c_oracle):
    z = np.load(GOLDEN / "lans_kat.npz")
    nt = len(mf.LANS_SIZES)
    for name, (kw, g16, first_step) in mf.LANS_CASES.items():
        hp = lans_f64.LansHParams(**kw)
        g = [z[f"{name}/g{t}"] for t in range(nt)]
        assert g[0].dtype == (np.float16 if g16 else np.float32)
        w = [z[f"{name}/w{t}"] for t in range(nt)]
        m = [z[f"{name}/m{t}"] for t in range(nt)]
        v = [z[f"{name}/v{t}"] for t in range(nt)]
        cw, cm, cv = [a.copy() for a in w], [a.copy() for a in m], [a.copy() for a in v]
        for s in range(mf.LANS_STEPS):
            w, m, v, norms = lans_f64.lans_step(g, w, m, v, first_step + s, hp)
            cn = c_oracle.lans_step_inplace(g, cw, cm, cv, first_step + s, hp, threads=2)
            if s + 1 not in mf.LANS_STORED:
                continue
            np.testing.assert_allclose(norms, z[f"{name}/norms_after{s + 1}"], rtol=1e-14)
            np.testing.assert_allclose(cn, z[f"{name}/norms_after{s + 1}"], rtol=1e-12)
            for t in range(nt):
                for q, arrs, carrs in (("w", w, cw), ("m", m, cm), ("v", v, cv)):
                    want = z[f"{name}/{q}{t}_after{s + 1}"]
                    assert np.array_equal(arrs[t], want), (name, q, t, s)
                    assert max_rel_err(carrs[t], want) <= 1.2e-7, (name, q, t, s)


def test_mixed_fixture_matches_oracle(c_oracle):
    z = np.load(GOLDEN / "mixed_kat.npz")
    nt = len(mf.MIXED_SIZES)
    hp = lans_f64.LansHParams(grad_unscale=1.0 / 1024)
    for name, (gdt, mdt) in mf.MIXED_CASES.items():
        g, w, m, v = ([z[f"lans/{name}/{q}{t}"] for t in range(nt)] for q in "gwmv")
        assert g[0].dtype == (np.float16 if gdt == "float16" else np.uint16)
        cw, cm, cv = [a.copy() for a in w], [a.copy() for a in m], [a.copy() for a in v]
        cp = [np.zeros(a.size, np.uint16) for a in w]
        x, vel = w, m
        for s in range(2):
            w, m, v, p, _ = lans_f64.lans_mixed_step(g, w, m, v, 2 + s, hp, mdt)
            c_oracle.lans_step_inplace(g, cw, cm, cv, 2 + s, hp, p_list=cp, model_dtype=mdt)
            x, vel, sp = sgd_f32.sgd_list_step(x, g, vel, 0.01, 0.9, mdt)
        for t in range(nt):
            assert np.array_equal(w[t], z[f"lans/{name}/w{t}_after2"])
            assert np.array_equal(p[t].view(np.uint16), z[f"lans/{name}/p{t}_after2"])
            assert max_rel_err(cw[t], w[t]) <= 1.2e-7
            assert np.array_equal(cp[t], halfs.narrow_weight(cw[t], mdt).view(np.uint16))
            assert np.array_equal(x[t].view(np.uint32), z[f"sgd/{name}/x{t}_after2"])
            assert np.array_equal(vel[t].view(np.uint32), z[f"sgd/{name}/v{t}_after2"])
            assert np.array_equal(sp[t].view(np.uint16), z[f"sgd/{name}/p{t}_after2"])
    for dt in mf.NORM_DTYPES:
        for k, n in enumerate(mf.NORM_SIZES):
            r = tensor_ops.l2norm(mf.norm_input(n, dt, k))
            assert np.array_equal(np.frombuffer(r.tobytes(), dtype=np.uint8), z[f"l2norm/{dt}/{n}"])
