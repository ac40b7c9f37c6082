"""GPU parity of raf.op.sgd: the HIP kernel, called through the C ABI, against the fp32 oracle --
bit for bit (NaN lanes compared as NaN masks; payloads are not part of the contract)."""
import numpy as np
import pytest
import torch

from oracle import sgd_f32
from tests.golden import make_fixtures as mf

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _bits_equal(got: torch.Tensor, want: np.ndarray):
    g = got.detach().cpu().numpy().ravel()
    w = np.ascontiguousarray(want).ravel()
    nan = np.isnan(w)
    assert np.array_equal(np.isnan(g), nan)
    assert np.array_equal(g.view(np.uint32)[~nan], w.view(np.uint32)[~nan])


def _rand(n, seed):
    r = np.random.default_rng([2024, 1, seed])
    return (r.normal(0, .02, n).astype(np.float32), r.normal(0, 1e-3, n).astype(np.float32),
            r.normal(0, 1e-3, n).astype(np.float32))


def test_golden_fixture_bitwise(native_libs):
    from raf_amd import kernels

    z = np.load(mf.HERE / "sgd_kat.npz")
    x, dx, v = (torch.from_numpy(z[k]).to(DEV) for k in ("x0", "dx", "v0"))
    v1, x1 = kernels.sgd_f32(x, dx, v, float(z["learning_rate"]), float(z["mu"]))
    _bits_equal(v1, z["v1_bits"].view(np.float32))
    _bits_equal(x1, z["x1_bits"].view(np.float32))
    # inputs untouched (out-of-place op, src/op/declare/optimizer.cc:34-42)
    assert np.array_equal(x.cpu().numpy().view(np.uint32), z["x0"].view(np.uint32))
    assert np.array_equal(v.cpu().numpy().view(np.uint32), z["v0"].view(np.uint32))


@pytest.mark.parametrize("n", [0, 1, 2, 3, 4, 5, 7, 255, 256, 257, 1023, 1025, 2048 * 3 + 1, 1 << 20])
def test_sizes_and_tails(native_libs, n):
    from raf_amd import kernels

    x0, dx, v0 = _rand(n, n)
    v1, x1 = kernels.sgd_f32(torch.from_numpy(x0).to(DEV), torch.from_numpy(dx).to(DEV),
                             torch.from_numpy(v0).to(DEV), 0.01, 0.9)
    ov, ox = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    _bits_equal(v1, ov)
    _bits_equal(x1, ox)


@pytest.mark.parametrize("offset", [1, 2, 3])
def test_unaligned_views_take_the_scalar_path(native_libs, offset):
    from raf_amd import kernels

    n = 10001
    x0, dx, v0 = _rand(n + 8, 77 + offset)
    tx, tdx, tv = (torch.from_numpy(a).to(DEV)[offset:offset + n] for a in (x0, dx, v0))
    assert tx.data_ptr() % 16 != 0
    v1, x1 = kernels.sgd_f32(tx, tdx, tv, 0.05, 0.5)
    ov, ox = sgd_f32.sgd_step(x0[offset:offset + n], dx[offset:offset + n], v0[offset:offset + n], 0.05, 0.5)
    _bits_equal(v1, ov)
    _bits_equal(x1, ox)


def test_outputs_may_alias_inputs(native_libs):
    from raf_amd import kernels

    x0, dx, v0 = _rand(100003, 5)
    tx, tdx, tv = (torch.from_numpy(a).to(DEV) for a in (x0, dx, v0))
    kernels.sgd_f32(tx, tdx, tv, 0.01, 0.9, v_out=tv, x_out=tx)
    ov, ox = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    _bits_equal(tv, ov)
    _bits_equal(tx, ox)


def test_config1_full_size_bitwise(native_libs, c_oracle):
    """Benchmark configuration 1: one fp32 tensor of 4,194,304 elements, w~N(0,.02), grad~N(0,1e-3),
    velocity 0, lr .01, momentum .9 -- every element compared."""
    from raf_amd import kernels

    n = 4_194_304
    r = np.random.default_rng([2024, 1, 0])
    x0 = r.normal(0, .02, n).astype(np.float32)
    dx = r.normal(0, 1e-3, n).astype(np.float32)
    v0 = np.zeros(n, np.float32)
    tx, tdx, tv = (torch.from_numpy(a).to(DEV) for a in (x0, dx, v0))
    for _ in range(3):  # three consecutive steps, state carried on both sides
        tv, tx = kernels.sgd_f32(tx, tdx, tv, 0.01, 0.9)
        v0, x0 = c_oracle.sgd_step(x0, dx, v0, 0.01, 0.9, threads=8)
        _bits_equal(tv, v0)
        _bits_equal(tx, x0)


def test_2d_shape_and_shape_mismatch(native_libs):
    from raf_amd import kernels

    x0, dx, v0 = (a.reshape(37, 29) for a in _rand(37 * 29, 9))
    v1, x1 = kernels.sgd_f32(torch.from_numpy(x0).to(DEV), torch.from_numpy(dx).to(DEV),
                             torch.from_numpy(v0).to(DEV), 0.01, 0.9)
    assert v1.shape == (37, 29)
    ov, ox = sgd_f32.sgd_step(x0, dx, v0, 0.01, 0.9)
    _bits_equal(v1.reshape(-1), ov.reshape(-1))
    with pytest.raises(ValueError):
        kernels.sgd_f32(torch.zeros(4, device=DEV), torch.zeros(5, device=DEV), torch.zeros(4, device=DEV), .1, .9)
    with pytest.raises(TypeError):
        kernels.sgd_f32(*(torch.zeros(4, device=DEV, dtype=torch.float16),) * 3, .1, .9)


@pytest.mark.parametrize("shape", [[4, 4]])
@pytest.mark.parametrize("seed", range(6))
def test_reference_style_closed_form(native_libs, shape, seed):
    """The reference's own operator test (tests/python/op/tvm/test_tvm_loss.py:158-176), through the
    operator front end: standard-normal inputs, a standard-normal momentum (negative ones included),
    learning rate 0.01, checked as there against the float64 closed form at 1e-4 -- and, beyond the
    reference, bit for bit against the fp32 oracle."""
    from raf_amd import op

    rng = np.random.default_rng(seed)
    x0 = rng.standard_normal(shape).astype("float32")
    dx = rng.standard_normal(shape).astype("float32")
    v0 = rng.standard_normal(shape).astype("float32")
    mu = float(rng.standard_normal(1)[0])
    learning_rate = 0.01
    n_v1 = mu * v0 + dx
    n_x1 = x0 - learning_rate * n_v1
    m_v1, m_x1 = op.sgd(torch.from_numpy(x0).to(DEV), torch.from_numpy(dx).to(DEV),
                        torch.from_numpy(v0).to(DEV), learning_rate, mu)
    np.testing.assert_allclose(m_v1.cpu().numpy(), n_v1, 1e-4, 1e-4)
    np.testing.assert_allclose(m_x1.cpu().numpy(), n_x1, 1e-4, 1e-4)
    ov, ox = sgd_f32.sgd_step(x0, dx, v0, learning_rate, mu)
    assert m_v1.shape == tuple(shape) and m_x1.shape == tuple(shape)
    _bits_equal(m_v1.reshape(-1), ov.reshape(-1))
    _bits_equal(m_x1.reshape(-1), ox.reshape(-1))


@pytest.mark.parametrize("dtype", ["float16", "bfloat16", "float64"])
def test_sgd_in_other_element_types_is_bit_exact(native_libs, dtype):
    """raf.op.sgd is written in the dtype of x (python/raf/_tvm_op/sgd.py:18-19): float64 and the
    16-bit types, through the C ABI and through the operator front end, bit for bit against the
    oracle (itself pinned by exact rational arithmetic; the reference's tests run fp32 only), on
    sizes that exercise the 16-byte path, its tail and the unaligned path."""
    from oracle.halfs import f32_to_bf16_bits
    from raf_amd import kernels, op

    rng = np.random.default_rng(11)
    tdt = {"float16": torch.float16, "bfloat16": torch.bfloat16, "float64": torch.float64}[dtype]
    for n, offset in ((100_003, 0), (8, 0), (5, 0), (70_001, 1), (1 << 20, 0)):
        raw = [rng.normal(0, s, n + offset) for s in (0.02, 1e-3, 1e-3)]
        raw[0][:4] = [6.1e-5, -5.96e-8, 1.0, 0.0]  # 16-bit subnormals among them
        if dtype == "bfloat16":
            host = [f32_to_bf16_bits(a.astype(np.float32)) for a in raw]
            dev = [torch.from_numpy(a.view(np.int16).copy()).to(DEV).view(torch.bfloat16)[offset:] for a in host]
            back = lambda t: t.view(torch.int16).cpu().numpy().view(np.uint16)
        else:
            npdt = np.float16 if dtype == "float16" else np.float64
            host = [a.astype(npdt) for a in raw]
            dev = [torch.from_numpy(a).to(DEV)[offset:] for a in host]
            back = lambda t: t.cpu().numpy()
        want_v, want_x = sgd_f32.sgd_step_typed(*[a[offset:] for a in host], 0.0123, 0.9, dtype)
        for call in (kernels.sgd, op.sgd):
            v1, x1 = call(*dev, 0.0123, 0.9)
            assert v1.dtype == tdt and x1.dtype == tdt
            assert np.array_equal(back(v1), want_v, equal_nan=False), (dtype, n, call.__module__, "v1")
            assert np.array_equal(back(x1), want_x, equal_nan=False), (dtype, n, call.__module__, "x1")
    with pytest.raises(TypeError):
        kernels.sgd(torch.zeros(4, device=DEV), torch.zeros(4, device=DEV).half(), torch.zeros(4, device=DEV), 0.1, 0.9)
