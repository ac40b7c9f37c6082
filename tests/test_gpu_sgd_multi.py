"""GPU parity of the multi-tensor, in-place momentum-SGD step, called through the C ABI: bit-exact
against the fp32 oracle on every element of x and v (four separately rounded operations), for
fp32, float16 and bfloat16 gradients, with and without 16-bit copies of the new weights."""
import numpy as np
import pytest
import torch

from oracle import halfs, sgd_f32
from tests.helpers import rng_for

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SIZES = [1, 3, 4, 5, 0, 255, 1023, 4095, 4096, 4097, 8193, 65537, 100003]


def _inputs(sizes, cfg, grad):
    xs, ds, vs = [], [], []
    for t, n in enumerate(sizes):
        xs.append(rng_for(cfg, t, 1).normal(0, 0.02, n).astype(np.float32))
        d = rng_for(cfg, t, 0).normal(0, 1e-3, n).astype(np.float32)
        ds.append(d.astype(np.float16) if grad == "float16" else halfs.f32_to_bf16_bits(d) if grad == "bfloat16" else d)
        vs.append(rng_for(cfg, t, 2).normal(0, 1e-3, n).astype(np.float32))
    return xs, ds, vs


def _dev(a):
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16)
    return torch.from_numpy(a.copy()).to(DEV)


def _bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("grad", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("model_dtype", [None, "float16", "bfloat16"])
def test_multi_tensor_sgd_is_bit_exact(native_libs, grad, model_dtype):
    from raf_amd import kernels

    xs, ds, vs = _inputs(SIZES, 200, grad)
    tx, td, tv = [_dev(a) for a in xs], [_dev(a) for a in ds], [_dev(a) for a in vs]
    tdt = {"float16": torch.float16, "bfloat16": torch.bfloat16}
    tp = [torch.full((a.size,), 3.0, dtype=tdt[model_dtype], device=DEV) for a in xs] if model_dtype else None
    plan = kernels.SgdPlan(SIZES, td[0].dtype, DEV)
    ox, ov = xs, vs
    for step in range(3):
        plan.step(tx, td, tv, 0.01, 0.9, p=tp)
        ox, ov, op = sgd_f32.sgd_list_step(ox, ds, ov, 0.01, 0.9, model_dtype)
    torch.cuda.synchronize()
    for t in range(len(SIZES)):
        assert np.array_equal(tx[t].cpu().numpy().view(np.uint32), ox[t].view(np.uint32)), f"x[{t}]"
        assert np.array_equal(tv[t].cpu().numpy().view(np.uint32), ov[t].view(np.uint32)), f"v[{t}]"
        assert np.array_equal(_bits(td[t]) if grad != "float32" else td[t].cpu().numpy(),
                              ds[t].view(np.uint16) if grad != "float32" else ds[t]), "gradients must stay untouched"
        if model_dtype:
            assert np.array_equal(_bits(tp[t]), op[t].view(np.uint16)), f"p[{t}]"
    plan.close()


def test_multi_tensor_sgd_equals_the_single_tensor_op(native_libs):
    """Same bits as raf.op.sgd applied parameter by parameter, including on inputs where a fused
    multiply-add would round differently and on unaligned views."""
    from raf_amd import kernels

    sizes = [4099, 70001, 17]
    xs, ds, vs = _inputs(sizes, 201, "float32")
    backing = [torch.zeros(3 * (n + 8), device=DEV) for n in sizes]
    tx = [b[1:1 + n] for b, n in zip(backing, sizes)]                      # 4-byte aligned views
    td = [b[n + 9:2 * n + 9] for b, n in zip(backing, sizes)]
    tv = [b[2 * n + 14:3 * n + 14] for b, n in zip(backing, sizes)]
    for dst, src in zip(tx + td + tv, xs + ds + vs):
        dst.copy_(torch.from_numpy(src))
    want = [kernels.sgd_f32(x.clone(), d.clone(), v.clone(), 0.0625, 0.875) for x, d, v in zip(tx, td, tv)]
    plan = kernels.SgdPlan(sizes, torch.float32, DEV)
    plan.step(tx, td, tv, 0.0625, 0.875)
    for t in range(3):
        assert torch.equal(tv[t], want[t][0]) and torch.equal(tx[t], want[t][1])
    plan.close()


def test_multi_tensor_sgd_large_list_streams(native_libs, c_oracle):
    """A BERT-base-sized list (1.3 GB of x, dx, v: the non-temporal path) against the C oracle."""
    from raf_amd import kernels, shapes

    sizes = shapes.numels(shapes.bert_base_shapes())
    gen = torch.Generator(DEV).manual_seed(5)
    tx = [torch.randn(n, device=DEV, generator=gen) * 0.02 for n in sizes]
    td = [torch.randn(n, device=DEV, generator=gen) * 1e-3 for n in sizes]
    tv = [torch.randn(n, device=DEV, generator=gen) * 1e-3 for n in sizes]
    x0, d0, v0 = torch.cat(tx).cpu().numpy(), torch.cat(td).cpu().numpy(), torch.cat(tv).cpu().numpy()
    plan = kernels.SgdPlan(sizes, torch.float32, DEV)
    plan.step(tx, td, tv, 0.01, 0.9)
    v1, x1 = c_oracle.sgd_step(x0, d0, v0, 0.01, 0.9, threads=8)
    assert np.array_equal(torch.cat(tx).cpu().numpy().view(np.uint32), x1.view(np.uint32))
    assert np.array_equal(torch.cat(tv).cpu().numpy().view(np.uint32), v1.view(np.uint32))
    plan.close()


def test_multi_tensor_sgd_errors_and_empty(native_libs):
    from raf_amd import kernels

    kernels.SgdPlan([], torch.float32, DEV).step([], [], [], 0.1, 0.9)
    z = torch.zeros(0, device=DEV)
    kernels.SgdPlan([0], torch.float32, DEV).step([z], [z], [z], 0.1, 0.9)
    plan = kernels.SgdPlan([8], torch.float16, DEV)
    f = [torch.zeros(8, device=DEV)]
    with pytest.raises(TypeError):
        plan.step(f, f, f, 0.1, 0.9)  # gradients must be float16 for this plan
    with pytest.raises(TypeError):
        plan.step(f, [f[0].half()], f, 0.1, 0.9, p=[torch.zeros(8, device=DEV)])
    with pytest.raises(TypeError):
        kernels.SgdPlan([8], torch.float64, DEV)
    with pytest.raises(ValueError):
        plan.step(f + f, [f[0].half()], f, 0.1, 0.9)


def test_sgd_multi_ops_through_dialect_dispatch(native_libs):
    """raf_amd.op.sgd_multi / sgd_multi_mixed: declare -> dispatch to the hip dialect -> OpEnv."""
    from raf_amd import op

    sizes = [(3, 5), (7,), (4100,)]
    xs = [rng_for(210, t, 1).normal(0, 0.02, s).astype(np.float32) for t, s in enumerate(sizes)]
    ds = [rng_for(210, t, 0).normal(0, 1e-3, s).astype(np.float32) for t, s in enumerate(sizes)]
    vs = [rng_for(210, t, 2).normal(0, 1e-3, s).astype(np.float32) for t, s in enumerate(sizes)]
    tl = [_dev(a) for a in xs + ds + vs]
    out = op.sgd_multi(tl, 0.01, 0.9)
    assert out[0] is tl[0] and len(out) == 9
    ox, ov, _ = sgd_f32.sgd_list_step(xs, ds, vs, 0.01, 0.9)
    for t in range(3):
        assert np.array_equal(tl[t].cpu().numpy(), ox[t]) and np.array_equal(tl[6 + t].cpu().numpy(), ov[t])
    d16 = [d.astype(np.float16) for d in ds]
    tl = [_dev(a) for a in xs + d16 + vs] + [torch.zeros(s, dtype=torch.float16, device=DEV) for s in sizes]
    op.sgd_multi_mixed(tl, 0.01, 0.9)
    ox, ov, opp = sgd_f32.sgd_list_step(xs, d16, vs, 0.01, 0.9, "float16")
    for t in range(3):
        assert np.array_equal(tl[t].cpu().numpy(), ox[t]) and np.array_equal(tl[6 + t].cpu().numpy(), ov[t])
        assert np.array_equal(tl[9 + t].cpu().numpy(), opp[t])
    with pytest.raises(native_libs.RafError, match="float16 or bfloat16"):
        op.sgd_multi_mixed(tl[:9] + [t.float() for t in tl[9:]], 0.01, 0.9)
