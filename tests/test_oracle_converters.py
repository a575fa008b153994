"""Pins the oracle's 16-bit converters against torch (exhaustively where finite)."""
import numpy as np
import torch

import oracle
from conftest import bits16, from_bits16, f32_bits


def test_half_to_float_all_patterns():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.half_to_float(bits)
    want = from_bits16(bits, torch.float16).float().numpy()
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(f32_bits(got)[~nan], f32_bits(want)[~nan])


def test_bf16_to_float_all_patterns():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = oracle.bf16_to_float(bits)
    want = from_bits16(bits, torch.bfloat16).float().numpy()
    nan = np.isnan(want)
    assert np.array_equal(f32_bits(got)[~nan], f32_bits(want)[~nan])


def _interesting_floats():
    rng = np.random.default_rng(7)
    parts = [
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(200000) * 1e-5).astype(np.float32),       # fp16 subnormal range
        (rng.standard_normal(100000) * 6e4).astype(np.float32),        # around fp16 max
        rng.integers(0, 2**32, 400000, dtype=np.uint64).astype(np.uint32).view(np.float32),  # any bit pattern
    ]
    # every fp16 value, and the midpoint between each pair of neighbours (exact ties)
    h = from_bits16(np.arange(0x7C01, dtype=np.uint32).astype(np.uint16), torch.float16).float().numpy()
    ties = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    parts += [h, -h, ties, -ties, np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf))]
    parts.append(np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.99, 65520.0, 2.0**-24, 2.0**-25,
                           np.nextafter(np.float32(2.0**-25), np.float32(1))], dtype=np.float32))
    return np.concatenate(parts)


def test_fp32_to_fp16_is_round_to_nearest_even():
    x = _interesting_floats()
    got = oracle.to_fp16_from_fp32(x)
    want = bits16(torch.from_numpy(x).half())
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x03FF) != 0)


def test_fp32_to_bf16_truncation_and_rne():
    x = _interesting_floats()
    nan = np.isnan(x)
    assert np.array_equal(oracle.to_bf16_from_fp32(x), (f32_bits(x) >> 16).astype(np.uint16))   # adam_cpu.hpp:135-137
    got = oracle.to_bf16_from_fp32(x, rne=True)
    want = bits16(torch.from_numpy(x).bfloat16())
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7F80) == 0x7F80) and np.all((got[nan] & 0x007F) != 0)
