"""The library's host-memory Adam (adam_cpu_*_launcher, to_*_from_fp32) against the committed
vectors of the reference's compiled adam_cpu.hpp and against the oracle.  Runs on the CPU."""
import os

import numpy as np
import pytest
import torch

import oracle
import bmtrain_amd.C as C
from bmtrain_amd.optim import _function as F
from conftest import bits16, f32_bits, from_bits16, load_golden

CASES = ["adam_cpu_fp16_t8", "adam_cpu_fp16_t3_delta", "adam_cpu_fp16_t1", "adam_cpu_bf16_t8", "adam_cpu_bf16_t2_delta"]


def _host_level():
    have = set()
    with open("/proc/cpuinfo") as f:
        for line in f:
            if line.startswith("flags"):
                have = set(line.split(":", 1)[1].split())
                break
    narrow = {"avx", "fma", "f16c"} <= have
    return 2 if ("avx512f" in have and narrow) else (1 if narrow else 0)


class affinity:
    """Runs the body with exactly `threads` CPUs in the affinity mask (the library sizes its
    thread fan-out from it, like the reference: adam_cpu.hpp:54-58)."""
    def __init__(self, threads):
        self.threads = threads
    def __enter__(self):
        self.saved = os.sched_getaffinity(0)
        if len(self.saved) < self.threads:
            pytest.skip(f"needs {self.threads} CPUs")
        os.sched_setaffinity(0, set(sorted(self.saved)[:self.threads]))
    def __exit__(self, *exc):
        os.sched_setaffinity(0, self.saved)


@pytest.mark.parametrize("case", CASES)
def test_matches_compiled_reference_vectors(case):
    g = load_golden(case)
    dtype, n, threads, level = str(g["dtype"]), int(g["n"]), int(g["threads"]), int(g["level"])
    if dtype == "fp16" and _host_level() != level:
        pytest.skip("vector recorded at another SIMD level; covered by the oracle comparison below")
    tdtype = torch.float16 if dtype == "fp16" else torch.bfloat16
    b1, b2, eps, lr, wd, scale = (float(g[k]) for k in ("beta1", "beta2", "eps", "lr", "weight_decay", "scale"))
    p = torch.from_numpy(g["p0"].copy())
    m = torch.zeros(n); v = torch.zeros(n)
    h = torch.zeros(n, dtype=tdtype)
    with affinity(threads):
        for s in range(1, int(g["steps"]) + 1):
            delta = torch.zeros(4) if bool(g["record_delta"]) else None
            F.adam_cpu(p, h, delta, from_bits16(g[f"g{s}"], tdtype), m, v, b1, b2, eps, lr, scale, wd, s)
            assert np.array_equal(f32_bits(p.numpy()), f32_bits(g[f"p{s}"])), (case, s)
            assert np.array_equal(f32_bits(m.numpy()), f32_bits(g[f"m{s}"])), (case, s)
            assert np.array_equal(f32_bits(v.numpy()), f32_bits(g[f"v{s}"])), (case, s)
            assert np.array_equal(bits16(h), g[f"h{s}"]), (case, s)
            if delta is not None:
                np.testing.assert_allclose(delta.numpy(), g[f"d{s}"], rtol=2e-4, atol=1e-6)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("n", [1, 15, 16, 17, 1000, 65537])
def test_matches_oracle_bit_for_bit(dtype, n):
    tdtype = torch.float16 if dtype == "fp16" else torch.bfloat16
    gen = torch.Generator().manual_seed(n)
    p = torch.randn(n, generator=gen) * 0.02
    m = torch.randn(n, generator=gen) * 1e-4
    v = (torch.randn(n, generator=gen) * 1e-6).abs()
    h = torch.zeros(n, dtype=tdtype)
    po, mo, vo, ho = p.numpy().copy(), m.numpy().copy(), v.numpy().copy(), np.zeros(n, np.uint16)
    threads = len(os.sched_getaffinity(0))
    for step, scale in ((1, 1.0), (5, 1024.0), (100, 7.0)):
        g = (torch.randn(n, generator=gen) * 1e-3 * scale).to(tdtype)
        delta = torch.zeros(4)
        delta_o = np.zeros(4, np.float32)
        F.adam_cpu(p, h, delta, g, m, v, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, step)
        bc1, bc2 = oracle.bias_corrections(0.9, 0.999, step)
        if dtype == "fp16":
            oracle.adam_cpu_fp16(po, ho, delta_o, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2,
                                 _host_level(), threads)
        else:
            oracle.adam_cpu_bf16(po, ho, delta_o, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2, threads)
        assert np.array_equal(f32_bits(p.numpy()), f32_bits(po))
        assert np.array_equal(f32_bits(m.numpy()), f32_bits(mo))
        assert np.array_equal(f32_bits(v.numpy()), f32_bits(vo))
        assert np.array_equal(bits16(h), ho)
        np.testing.assert_allclose(delta.numpy(), delta_o, rtol=1e-3, atol=1e-6)


def test_host_converters():
    gen = torch.Generator().manual_seed(0)
    x = torch.cat([torch.randn(100001, generator=gen), torch.randn(1000, generator=gen) * 1e-6,
                   torch.tensor([0.0, -0.0, 65504.0, 65520.0, 1e-8, float("inf"), -float("inf")])])
    assert np.array_equal(bits16(F.fp16_from_fp32(x)), oracle.to_fp16_from_fp32(x.numpy()))
    assert np.array_equal(bits16(F.fp16_from_fp32(x)), bits16(x.half()))
    assert np.array_equal(bits16(F.bf16_from_fp32(x)), oracle.to_bf16_from_fp32(x.numpy()))


def test_adam_cpu_rejects_bad_arguments():
    n = 8
    p = torch.zeros(n); m = torch.zeros(n); v = torch.zeros(n)
    h = torch.zeros(n, dtype=torch.float16); g = torch.zeros(n, dtype=torch.float16)
    args = (0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 1)
    with pytest.raises(AssertionError, match="same number of elements"):
        F.adam_cpu(p, h, None, g[:4], m, v, *args)
    with pytest.raises(AssertionError, match="float32"):
        F.adam_cpu(p.double(), h, None, g, m, v, *args)
    with pytest.raises(AssertionError, match="contiguous"):
        F.adam_cpu(torch.zeros(2 * n)[::2], h, None, g, m, v, *args)
    with pytest.raises(AssertionError, match="length of 4"):
        F.adam_cpu(p, h, torch.zeros(3), g, m, v, *args)


def test_worker_pool_survives_many_calls_affinity_changes_and_fork():
    """The host Adam keeps its helper threads between calls: many small calls, a change of the thread count,
    and use in a forked child must all keep working and keep matching the oracle."""
    import multiprocessing as mp

    def one_round(n, seed):
        gen = torch.Generator().manual_seed(seed)
        p = torch.randn(n, generator=gen) * 0.02
        m = torch.zeros(n); v = torch.zeros(n); h = torch.zeros(n, dtype=torch.bfloat16)
        g = torch.randn(n, generator=gen).bfloat16()
        po, mo, vo, ho = p.numpy().copy(), m.numpy().copy(), v.numpy().copy(), np.zeros(n, np.uint16)
        F.adam_cpu(p, h, None, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 1)
        bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 1)
        oracle.adam_cpu_bf16(po, ho, None, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
        return np.array_equal(f32_bits(p.numpy()), f32_bits(po)) and np.array_equal(bits16(h), ho)

    for k in range(200):
        assert one_round(1 + 37 * k, k)
    cpus = len(os.sched_getaffinity(0))
    for threads in (2, 1, 3, cpus):
        if threads <= cpus:
            with affinity(threads):
                assert one_round(10007, threads)
    ctx = mp.get_context("fork")
    q = ctx.Queue()
    child = ctx.Process(target=lambda: q.put(one_round(5003, 99)))
    child.start()
    child.join(60)
    assert child.exitcode == 0 and q.get(timeout=5) is True
    assert one_round(4099, 7)
