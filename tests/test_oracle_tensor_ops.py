"""Pins of the l2norm / fuse_tensor / defuse_tensor oracle (no GPU)."""
import math
from fractions import Fraction

import numpy as np
import pytest

from oracle import halfs, tensor_ops


def test_l2norm_exact_rational_sum_on_small_inputs():
    rng = np.random.default_rng(11)
    for dtype in (np.float32, np.float64, np.float16):
        x = rng.standard_normal(37).astype(dtype)
        exact = sum(Fraction(float(v)) ** 2 for v in x)
        got = tensor_ops.l2norm_f64(x)
        # |got^2 - exact| within a few float64 ulps of the exact sum
        assert abs(Fraction(got) ** 2 - exact) <= exact * Fraction(1, 2 ** 50)


def test_l2norm_closed_forms():
    assert tensor_ops.l2norm_f64(np.array([3.0, 4.0], np.float32)) == 5.0
    assert tensor_ops.l2norm_f64(np.array([[1, 2], [2, 4]], np.float32)) == 5.0
    assert tensor_ops.l2norm_f64(np.full(1 << 20, 0.5, np.float32)) == 512.0
    assert tensor_ops.l2norm_f64(np.zeros(0, np.float32)) == 0.0
    # fp32 values whose squares overflow fp32 do not overflow the float64 accumulation
    assert tensor_ops.l2norm_f64(np.array([3e30, 4e30], np.float32)) == pytest.approx(5e30, rel=1e-7)
    out = tensor_ops.l2norm(np.array([3e30, 4e30], np.float32))
    assert out.dtype == np.float32 and out.shape == ()
    assert tensor_ops.l2norm(np.array([300.0, 400.0], np.float16)) == np.float16(500.0)
    assert np.isinf(tensor_ops.l2norm(np.array([60000.0, 60000.0], np.float16)))  # 84852 > 65504


def test_l2norm_against_fsum_and_homogeneity():
    rng = np.random.default_rng(12)
    x = (rng.standard_normal(200001) * 1e-3).astype(np.float32)
    ref = math.sqrt(math.fsum(float(v) * float(v) for v in x))
    assert tensor_ops.l2norm_f64(x) == pytest.approx(ref, rel=1e-14)
    assert tensor_ops.l2norm_f64(x * np.float32(1024)) == pytest.approx(1024 * ref, rel=1e-14)
    # the reference test's own check (tests/python/op/tvm/test_tvm_reduce.py:186-206)
    import torch
    t = torch.from_numpy(x.reshape(-1)[:24].reshape(2, 3, 4))
    assert float(tensor_ops.l2norm(t.numpy())) == pytest.approx(float(torch.sqrt(torch.sum(t * t))), rel=1e-6)


def test_l2norm_bfloat16_bits():
    bits = halfs.f32_to_bf16_bits(np.array([3.0, 4.0], np.float32))
    out = tensor_ops.l2norm(bits)
    assert out.dtype == np.uint16 and halfs.bf16_bits_to_f32(out) == 5.0


def test_fuse_is_elements_back_to_back():
    rng = np.random.default_rng(13)
    data = [rng.standard_normal(s).astype(np.float32) for s in [(3, 5), (7,), (0,), (2, 2, 2), ()]]
    flat = tensor_ops.fuse_tensor(data)
    assert flat.shape == (3 * 5 + 7 + 0 + 8 + 1,) and flat.dtype == np.float32
    k = 0
    for a in data:  # element by element, independent of numpy's concatenate
        for v in a.ravel():
            assert flat[k] == v
            k += 1
    assert k == flat.size


def test_defuse_inverts_fuse_and_checks_the_size():
    rng = np.random.default_rng(14)
    data = [rng.integers(0, 255, s).astype(np.uint8) for s in [(3, 5), (7,), (0,), (2, 2, 2), (1,)]]
    sizes, shapes, idx = tensor_ops.defuse_args(data)
    assert sizes == [15, 7, 0, 8, 1] and shapes == [3, 5, 7, 0, 2, 2, 2, 1] and idx == [2, 3, 4, 7, 8]
    back = tensor_ops.defuse_tensor(tensor_ops.fuse_tensor(data), sizes, shapes, idx)
    assert all(a.shape == b.shape and np.array_equal(a, b) for a, b in zip(data, back))
    with pytest.raises(AssertionError, match="Input tensor size should be 31"):
        tensor_ops.defuse_tensor(np.zeros(30, np.uint8), sizes, shapes, idx)
