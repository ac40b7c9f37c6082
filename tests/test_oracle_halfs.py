"""Pins of the 16-bit conversions used by the mixed-precision LANS path (no GPU): widening of
half gradients is exact, narrowing of the fp32 weight rounds to nearest even.  Checked against the
exhaustive set of 65536 patterns, hand-computed ties and torch's own conversions."""
import numpy as np
import pytest
import torch

from oracle import c_oracle, halfs


def _f32(bits):
    return np.array(bits, dtype=np.uint32).view(np.float32)


def _interesting_f32(n=1 << 20, seed=5):
    rng = np.random.default_rng(seed)
    any_bits = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)
    weights = (rng.standard_normal(n) * 0.02).astype(np.float32)
    tiny = (rng.standard_normal(n) * 1e-6).astype(np.float32)  # binary16 subnormal range
    # every binary16 and bfloat16 value, and the exact midpoints between neighbouring binary16 values
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    b = halfs.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16))
    hp = np.arange(0x7BFF, dtype=np.uint16)
    mid = ((hp.view(np.float16).astype(np.float64) + (hp + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2)
    return np.concatenate([any_bits, weights, tiny, h, b, mid.astype(np.float32), -mid.astype(np.float32)])


def test_bf16_widening_is_the_upper_half_of_the_word():
    bits = np.arange(65536, dtype=np.uint16)
    got = halfs.bf16_bits_to_f32(bits)
    want = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # 0x3F80 is 1.0, 0xC000 is -2.0, 0x0001 is the smallest subnormal 2^-133
    assert halfs.bf16_bits_to_f32(np.array([0x3F80, 0xC000, 0x0001], np.uint16)).tolist() == [1.0, -2.0, 2.0 ** -133]


def test_bf16_narrowing_known_answers():
    # 1 + 2^-8 is the midpoint of 1 and 1 + 2^-7: ties to even (1.0); 1 + 3*2^-8 ties up to 1 + 2^-6
    x = _f32([0x3F808000, 0x3F818000, 0x3F808001, 0x3F807FFF, 0x7F7FFFFF, 0xFF800000, 0x00000000, 0x80000000])
    want = [0x3F80, 0x3F82, 0x3F81, 0x3F80, 0x7F80, 0xFF80, 0x0000, 0x8000]
    assert halfs.f32_to_bf16_bits(x).tolist() == want
    assert c_oracle.narrow_bits(x, "bfloat16").tolist() == want


def test_f16_narrowing_known_answers():
    # 65504 max; 65519.99 -> 65504; 65520 -> inf; 2^-24 min subnormal; 2^-25 ties to zero; just above -> 2^-24
    x = np.array([65504.0, 65519.996, 65520.0, 2.0 ** -24, 2.0 ** -25, np.nextafter(np.float32(2.0 ** -25), np.float32(1)),
                  1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, -0.0, 6.1035156e-05], dtype=np.float32)
    want = [0x7BFF, 0x7BFF, 0x7C00, 0x0001, 0x0000, 0x0001, 0x3C00, 0x3C02, 0x8000, 0x0400]
    assert halfs.narrow_weight(x, "float16").view(np.uint16).tolist() == want
    assert c_oracle.narrow_bits(x, "float16").tolist() == want


@pytest.mark.parametrize("dtype,tdtype", [("float16", torch.float16), ("bfloat16", torch.bfloat16)])
def test_narrowing_agrees_with_torch_and_between_the_two_oracles(dtype, tdtype):
    x = _interesting_f32()
    ours = halfs.narrow_weight(x, dtype)
    ours = ours.view(np.uint16)
    c = c_oracle.narrow_bits(x, dtype)
    t = torch.from_numpy(x).to(tdtype).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(ours[~nan], t[~nan])
    assert np.array_equal(c[~nan], t[~nan])
    # NaNs stay NaNs in every implementation
    is_nan16 = (lambda b: ((b & 0x7C00) == 0x7C00) & ((b & 0x03FF) != 0)) if dtype == "float16" else \
               (lambda b: ((b & 0x7F80) == 0x7F80) & ((b & 0x007F) != 0))
    assert is_nan16(ours[nan]).all() and is_nan16(c[nan]).all()


def test_round_trip_of_every_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    for dtype, widen in (("float16", lambda b: b.view(np.float16).astype(np.float32)),
                         ("bfloat16", halfs.bf16_bits_to_f32)):
        f = widen(bits)
        ok = ~np.isnan(f)
        assert np.array_equal(halfs.narrow_weight(f, dtype).view(np.uint16)[ok], bits[ok])
        assert np.array_equal(c_oracle.narrow_bits(f, dtype)[ok], bits[ok])


def test_widen_grad_dispatch():
    g16 = np.array([1.5, -2.0], np.float16)
    assert halfs.widen_grad(g16).dtype == np.float32 and halfs.widen_grad(g16).tolist() == [1.5, -2.0]
    assert halfs.widen_grad(np.array([0x3FC0], np.uint16)).tolist() == [1.5]
    with pytest.raises(TypeError):
        halfs.widen_grad(np.array([1], np.int32))
