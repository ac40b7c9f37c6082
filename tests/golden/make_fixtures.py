"""Writes the committed fixtures of this directory from the CPU oracle.

    python tests/golden/make_fixtures.py

The reference holds no stored vectors for either operator and can be neither built nor imported
here (its arithmetic needs TVM / CUDA), so these vectors come from the oracle under oracle/, which
tests/test_oracle_*.py pin independently.  They serve two purposes: the GPU parity tests compare
the HIP kernels with them on the GPU box (where only committed files exist), and the CPU suite
re-derives them so that a change of the oracle's results cannot pass unnoticed.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

from oracle import halfs, lans_f64, sgd_f32, tensor_ops  # noqa: E402
from tests.helpers import lans_inputs  # noqa: E402

LANS_SIZES = [1, 3, 4, 5, 63, 65, 512, 513]
LANS_CASES = {
    # name: (hparams kwargs, fp16 gradients, first step number)
    "default": (dict(), False, 1),
    "l2_mode": (dict(mode=0), False, 2),
    "fp16_grad": (dict(grad_unscale=1.0 / 1024), True, 1),
    "plain": (dict(bias_correction=0, grad_averaging=0, normalize_grad=False, weight_decay=0.0), False, 3),
}
LANS_STEPS = 3
LANS_STORED = (1, 3)  # results kept after these many steps


def sgd_fixture():
    r = np.random.default_rng([2024, 1])
    n = 1531
    x0 = r.normal(0, 0.02, n).astype(np.float32)
    dx = r.normal(0, 1e-3, n).astype(np.float32)
    v0 = r.normal(0, 1e-3, n).astype(np.float32)
    tiny = np.float32(2.0 ** -140)
    special = np.array([0.0, -0.0, tiny, -tiny, 3e-39, np.inf, -np.inf, np.nan, 1.0, -1.0], np.float32)
    x0[: special.size] = special
    dx[special.size: 2 * special.size] = special
    v0[2 * special.size: 3 * special.size] = special
    v1, x1 = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    np.savez_compressed(HERE / "sgd_kat.npz", x0=x0, dx=dx, v0=v0, learning_rate=0.01, mu=0.9,
                        v1_bits=v1.view(np.uint32), x1_bits=x1.view(np.uint32))


def lans_fixture():
    out = {}
    for name, (kw, g16, first_step) in LANS_CASES.items():
        hp = lans_f64.LansHParams(**kw)
        g, w, m, v = lans_inputs(LANS_SIZES, cfg=100 + len(name), g16=g16, zero_state=(first_step == 1))
        for t in range(len(LANS_SIZES)):
            out[f"{name}/g{t}"], out[f"{name}/w{t}"] = g[t], w[t]
            out[f"{name}/m{t}"], out[f"{name}/v{t}"] = m[t], v[t]
        for s in range(LANS_STEPS):
            w, m, v, norms = lans_f64.lans_step(g, w, m, v, first_step + s, hp)
            if s + 1 not in LANS_STORED:
                continue
            out[f"{name}/norms_after{s + 1}"] = norms
            for t in range(len(LANS_SIZES)):
                out[f"{name}/w{t}_after{s + 1}"] = w[t]
                out[f"{name}/m{t}_after{s + 1}"] = m[t]
                out[f"{name}/v{t}_after{s + 1}"] = v[t]
    np.savez_compressed(HERE / "lans_kat.npz", **out)


MIXED_SIZES = [1, 4, 5, 257, 1027]
MIXED_CASES = {
    # name: (gradient dtype, model dtype)
    "f16_f16": ("float16", "float16"),
    "bf16_bf16": ("bfloat16", "bfloat16"),
    "bf16_f16": ("bfloat16", "float16"),
}
NORM_SIZES = [1, 5, 1000, 70001]
NORM_DTYPES = ("float32", "float64", "float16", "bfloat16")


def norm_input(n, dtype, k):
    x = np.random.default_rng([2024, 7, k]).normal(0, 0.02, n)
    if dtype == "bfloat16":
        return halfs.f32_to_bf16_bits(x.astype(np.float32))
    return x.astype(dtype)


def mixed_fixture():
    """The mixed-precision LANS step (half gradients in, 16-bit weight copies out), the
    multi-tensor SGD step with half gradients and copies, and l2norm in its four dtypes."""
    out = {}
    hp = lans_f64.LansHParams(grad_unscale=1.0 / 1024)
    for name, (gdt, mdt) in MIXED_CASES.items():
        g, w, m, v = lans_inputs(MIXED_SIZES, cfg=120 + len(name), g16=gdt)
        for t in range(len(MIXED_SIZES)):
            out[f"lans/{name}/g{t}"], out[f"lans/{name}/w{t}"] = g[t], w[t]
            out[f"lans/{name}/m{t}"], out[f"lans/{name}/v{t}"] = m[t], v[t]
        for s in range(2):
            w, m, v, p, _ = lans_f64.lans_mixed_step(g, w, m, v, 2 + s, hp, mdt)
        for t in range(len(MIXED_SIZES)):
            out[f"lans/{name}/w{t}_after2"] = w[t]
            out[f"lans/{name}/p{t}_after2"] = p[t].view(np.uint16)
        # SGD on the same tensors: x = w, dx = g (not unscaled), v = m
        g, x, vel, _ = lans_inputs(MIXED_SIZES, cfg=120 + len(name), g16=gdt)
        for s in range(2):
            x, vel, p = sgd_f32.sgd_list_step(x, g, vel, 0.01, 0.9, mdt)
        for t in range(len(MIXED_SIZES)):
            out[f"sgd/{name}/x{t}_after2"] = x[t].view(np.uint32)
            out[f"sgd/{name}/v{t}_after2"] = vel[t].view(np.uint32)
            out[f"sgd/{name}/p{t}_after2"] = p[t].view(np.uint16)
    for dt in NORM_DTYPES:
        for k, n in enumerate(NORM_SIZES):
            r = tensor_ops.l2norm(norm_input(n, dt, k))
            out[f"l2norm/{dt}/{n}"] = np.frombuffer(r.tobytes(), dtype=np.uint8)
    np.savez_compressed(HERE / "mixed_kat.npz", **out)


FIXTURES = {"sgd_kat.npz": sgd_fixture, "lans_kat.npz": lans_fixture, "mixed_kat.npz": mixed_fixture}

if __name__ == "__main__":
    # no arguments: every fixture; otherwise the named files only
    for f in sys.argv[1:] or FIXTURES:
        FIXTURES[f]()
        print(f, (HERE / f).stat().st_size, "bytes")
