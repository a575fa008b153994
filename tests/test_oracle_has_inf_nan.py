"""Pins the oracle's has_inf_nan: every 16-bit pattern against torch.isinf | torch.isnan,
the sticky flag, n <= 0, and a sweep shaped like the reference's tests/test_has_inf_nan.py."""
import random

import numpy as np
import pytest
import torch

import oracle
from conftest import bits16, from_bits16

DTYPES = [("fp16", torch.float16), ("bf16", torch.bfloat16)]


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_every_pattern(name, dtype):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    t = from_bits16(bits, dtype)
    want = (torch.isinf(t) | torch.isnan(t)).numpy()
    for b, w in zip(bits, want):
        out = np.zeros(1, np.uint8)
        oracle.has_inf_nan(np.array([b], np.uint16), out, name)
        assert out[0] == int(w), hex(b)
    finite = bits[~want]
    out = np.zeros(1, np.uint8)
    oracle.has_inf_nan(finite, out, name)
    assert out[0] == 0


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_flag_is_sticky_and_empty_is_noop(name, dtype):
    out = np.array([1], np.uint8)
    oracle.has_inf_nan(bits16(torch.ones(10).to(dtype)), out, name)
    assert out[0] == 1                       # has_inf_nan.cu:64-66: never cleared
    out = np.array([7], np.uint8)
    oracle.has_inf_nan(np.zeros(0, np.uint16), out, name)
    assert out[0] == 7                       # n <= 0 returns early (:108,:128)


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_reference_style_sweep(name, dtype):
    rnd = random.Random(0)
    torch.manual_seed(0)

    def check(x, v):
        out = np.zeros(1, np.uint8)
        oracle.has_inf_nan(bits16(x), out, name)
        assert out[0] == v

    for n in list(range(1, 100)) + [1000, 10000, 100000]:
        x = torch.rand(n).to(dtype)
        check(x, 0)
        p = rnd.randint(0, n - 1)
        x[p] = float("inf")
        check(x, 1)
        x[p] = 2
        check(x, 0)
        x[rnd.randint(0, n - 1)] = float("nan")
        check(x, 1)
        x[rnd.randint(0, n - 1)] = float("-inf")
        check(x, 1)


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_grad_sumsq_against_torch(name, dtype):
    """sum of squares in double = (g.double().norm(2)) ** 2, the quantity optim_manager.py:186-190 accumulates."""
    gen = torch.Generator().manual_seed(3)
    for n in (1, 7, 1000, 100003):
        g = (torch.randn(n, generator=gen) * 3).to(dtype)
        want = (g.double().norm(2) ** 2).item()
        got = oracle.grad_sumsq(bits16(g), name)
        assert abs(got - want) <= 1e-12 * max(1.0, want)
    assert oracle.grad_sumsq(bits16(torch.tensor([3.0, 4.0]).to(dtype)), name) == 25.0
