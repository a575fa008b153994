"""Pins the oracle's Adam restatements.

* CPU offload trees: bit-for-bit against vectors produced by the reference's own compiled
  adam_cpu.hpp (tests/golden/adam_cpu_*.npz) and, when oracle/_ref is built and this CPU
  can run it, against that module live on fresh random inputs.
* GPU bf16 tree: it is the same expression as the reference's scalar CPU bf16 loop, so the
  same vectors pin its fp32 state bit-for-bit; the bf16 copy is torch's RNE cast.
* GPU fp16 tree (no compiled reference exists): exact power-of-two scaling identity against
  the bf16 tree, float64 AdamW, lr = 0.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from conftest import bits16, f32_bits, load_golden

GOLDEN_CASES = ["adam_cpu_fp16_t8", "adam_cpu_fp16_t3_delta", "adam_cpu_fp16_t1", "adam_cpu_bf16_t8",
                "adam_cpu_bf16_t2_delta"]


def _hyper(g):
    return [float(g[k]) for k in ("beta1", "beta2", "eps", "lr")], float(g["scale"]), float(g["weight_decay"])


@pytest.mark.parametrize("case", GOLDEN_CASES)
def test_cpu_trees_match_compiled_reference_vectors(case):
    g = load_golden(case)
    (b1, b2, eps, lr), scale, wd = _hyper(g)
    dtype, n, threads, level = str(g["dtype"]), int(g["n"]), int(g["threads"]), int(g["level"])
    p = g["p0"].copy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    h = np.zeros(n, np.uint16)
    for s in range(1, int(g["steps"]) + 1):
        bc1, bc2 = oracle.bias_corrections(b1, b2, s)
        delta = np.zeros(4, np.float32) if bool(g["record_delta"]) else None
        if dtype == "fp16":
            oracle.adam_cpu_fp16(p, h, delta, g[f"g{s}"], m, v, b1, b2, eps, lr, scale, wd, bc1, bc2, level, threads)
        else:
            oracle.adam_cpu_bf16(p, h, delta, g[f"g{s}"], m, v, b1, b2, eps, lr, scale, wd, bc1, bc2, threads)
        assert np.array_equal(f32_bits(p), f32_bits(g[f"p{s}"])), (case, s, "p")
        assert np.array_equal(f32_bits(m), f32_bits(g[f"m{s}"])), (case, s, "m")
        assert np.array_equal(f32_bits(v), f32_bits(g[f"v{s}"])), (case, s, "v")
        assert np.array_equal(h, g[f"h{s}"]), (case, s, "p16")
        if delta is not None:   # float accumulation order is not fixed by the threaded reference
            np.testing.assert_allclose(delta, g[f"d{s}"], rtol=2e-4, atol=1e-6)


def test_golden_vectors_tell_the_trees_apart():
    """The vectors must be able to fail.  Continuing from the stored state after step 1 (non-zero
    moments), the un-contracted tree, and the scalar tree applied where the reference used the
    vector tree, must both disagree with the stored step 2."""
    g = load_golden("adam_cpu_bf16_t8")
    (b1, b2, eps, lr), scale, wd = _hyper(g)
    n = int(g["n"])
    bc1, bc2 = oracle.bias_corrections(b1, b2, 2)
    for tree, same in ((oracle.TREE_FMA_MVP, True), (oracle.TREE_PLAIN, False)):
        p, m, v, h = g["p1"].copy(), g["m1"].copy(), g["v1"].copy(), np.zeros(n, np.uint16)
        oracle.adam_cpu_bf16(p, h, None, g["g2"], m, v, b1, b2, eps, lr, scale, wd, bc1, bc2, 8, tree)
        agree = all(np.array_equal(f32_bits(a), f32_bits(g[k])) for a, k in ((p, "p2"), (m, "m2"), (v, "v2")))
        assert agree == same, tree
    g = load_golden("adam_cpu_fp16_t8")
    (b1, b2, eps, lr), scale, wd = _hyper(g)
    n = int(g["n"])
    for level, same in ((2, True), (0, False)):
        p, m, v, h = g["p1"].copy(), g["m1"].copy(), g["v1"].copy(), np.zeros(n, np.uint16)
        oracle.adam_cpu_fp16(p, h, None, g["g2"], m, v, b1, b2, eps, lr, scale, wd, bc1, bc2, level, 8)
        agree = all(np.array_equal(f32_bits(a), f32_bits(g[k])) for a, k in ((p, "p2"), (m, "m2"), (v, "v2")))
        assert agree == same, level


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_cpu_trees_match_compiled_reference_live(dtype):
    ref = oracle.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref/refadam.so not built here (or CPU without AVX-512F)")
    threads = len(os.sched_getaffinity(0))
    level = ref.get_cpu_level()
    gen = torch.Generator().manual_seed(5)
    for n, scale in ((1, 1.0), (17, 8.0), (4099, 1024.0), (100003, 3.0)):
        p = (torch.randn(n, generator=gen) * 0.02).numpy().copy()
        m = (torch.randn(n, generator=gen) * 1e-4).numpy().copy()
        v = (torch.randn(n, generator=gen) * 1e-6).abs().numpy().copy()
        h = np.zeros(n, np.uint16)
        po, mo, vo, ho = p.copy(), m.copy(), v.copy(), h.copy()
        for step in (1, 2, 100):
            gt = torch.randn(n, generator=gen) * 1e-3 * scale
            g16 = bits16(gt.half() if dtype == "fp16" else gt.bfloat16())
            bc1, bc2 = oracle.bias_corrections(0.9, 0.999, step)
            hyp = (0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
            if dtype == "fp16":
                ref.adam_cpu_fp16_launcher(n, p.ctypes.data, h.ctypes.data, 0, g16.ctypes.data, m.ctypes.data,
                                           v.ctypes.data, *hyp)
                oracle.adam_cpu_fp16(po, ho, None, g16, mo, vo, *hyp, level, threads)
            else:
                ref.adam_cpu_bf16_launcher(n, p.ctypes.data, h.ctypes.data, 0, g16.ctypes.data, m.ctypes.data,
                                           v.ctypes.data, *hyp)
                oracle.adam_cpu_bf16(po, ho, None, g16, mo, vo, *hyp, threads)
            for a, b in ((p, po), (m, mo), (v, vo)):
                assert np.array_equal(f32_bits(a), f32_bits(b)), (dtype, n, step)
            assert np.array_equal(h, ho)


def test_gpu_bf16_tree_is_the_compiled_scalar_cpu_tree():
    """adam_cuda.cu:60-64 and adam_cpu.hpp:265-276 are one expression; the oracle's GPU bf16
    function must reproduce the compiled reference's fp32 state, and its 16-bit copy must be
    the round-to-nearest-even cast where the CPU path truncates."""
    g = load_golden("adam_cpu_bf16_t8")
    (b1, b2, eps, lr), scale, wd = _hyper(g)
    n = int(g["n"])
    p = g["p0"].copy(); m = np.zeros(n, np.float32); v = np.zeros(n, np.float32); h = np.zeros(n, np.uint16)
    for s in range(1, int(g["steps"]) + 1):
        bc1, bc2 = oracle.bias_corrections(b1, b2, s)
        oracle.adam_gpu_bf16(p, h, g[f"g{s}"], m, v, b1, b2, eps, lr, scale, wd, bc1, bc2)
        assert np.array_equal(f32_bits(p), f32_bits(g[f"p{s}"]))
        assert np.array_equal(f32_bits(m), f32_bits(g[f"m{s}"]))
        assert np.array_equal(f32_bits(v), f32_bits(g[f"v{s}"]))
        assert np.array_equal(h, bits16(torch.from_numpy(p).bfloat16()))
        assert np.all(h.astype(np.int32) - g[f"h{s}"].astype(np.int32) >= 0)   # RNE never below truncation
        assert np.all(h.astype(np.int32) - g[f"h{s}"].astype(np.int32) <= 1)


def _adamw_float64(p, g, m, v, b1, b2, eps, lr, wd, step):
    """Textbook decoupled-decay Adam in float64 with the float32-rounded hyper-parameters."""
    f = lambda x: float(np.float32(x))
    b1, b2, eps, lr, wd = map(f, (b1, b2, eps, lr, wd))
    bc1, bc2 = (f(c) for c in oracle.bias_corrections(b1, b2, step))
    omb1, omb2 = f(np.float32(1) - np.float32(b1)), f(np.float32(1) - np.float32(b2))
    m = b1 * m + omb1 * g
    v = b2 * v + omb2 * g * g
    p = p - lr * (m / bc1) / (np.sqrt(v / bc2) + eps) - lr * wd * p
    return p, m, v


def test_gpu_bf16_tree_against_float64_and_torch_adamw():
    gen = torch.Generator().manual_seed(3)
    n = 20000
    p0 = (torch.randn(n, generator=gen) * 0.02)
    g = (torch.randn(n, generator=gen) * 1e-3).bfloat16()
    hyp = dict(b1=0.9, b2=0.999, eps=1e-8, lr=1e-3, wd=0.01)
    # oracle, three steps from zero moments
    p = p0.numpy().copy(); m = np.zeros(n, np.float32); v = np.zeros(n, np.float32); h = np.zeros(n, np.uint16)
    p64, m64, v64 = p0.double().numpy(), np.zeros(n), np.zeros(n)
    # torch AdamW (decoupled decay) in float64 — a library routine this special case must reduce to
    tp = torch.nn.Parameter(p0.double().clone())
    opt = torch.optim.AdamW([tp], lr=float(np.float32(1e-3)), betas=(float(np.float32(0.9)), float(np.float32(0.999))),
                            eps=float(np.float32(1e-8)), weight_decay=float(np.float32(0.01)))
    for step in (1, 2, 3):
        bc1, bc2 = oracle.bias_corrections(0.9, 0.999, step)
        oracle.adam_gpu_bf16(p, h, bits16(g), m, v, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
        p64, m64, v64 = _adamw_float64(p64, g.double().numpy(), m64, v64, step=step, **hyp)
        tp.grad = g.double()
        opt.step()
    assert np.abs(p - p64).max() <= 1e-6 * np.abs(p64).max()
    assert np.abs(m - m64).max() <= 1e-6 * np.abs(m64).max()
    assert np.abs(v - v64).max() <= 1e-6 * np.abs(v64).max()
    # torch's AdamW places eps outside the bias-corrected sqrt in the same way; it differs from the
    # float64 restatement only by float64 rounding and by the exactly representable hyper-parameters.
    np.testing.assert_allclose(tp.detach().numpy(), p64, rtol=0, atol=5e-9)


def test_gpu_fp16_tree_scaling_identity():
    """With scale = 2^k, gradients and first moment representable in both formats and no
    under/overflow, every intermediate of the fp16 tree is exactly 2^k (or 2^2k under the sqrt)
    times the bf16 tree's, so p' is identical bit for bit, v' = scale * v'_bf16 and the
    un-rounded m' = scale * m'_bf16."""
    gen = torch.Generator().manual_seed(9)
    n = 50000
    scale = 1024.0
    p0 = (torch.randn(n, generator=gen) * 0.02).numpy()
    def away_from_zero(t, floor):   # keeps value * scale inside fp16's normal range
        return torch.where(t >= 0, t + floor, t - floor)
    real_g = away_from_zero(torch.randn(n, generator=gen) * 1e-3, 1e-5).bfloat16()   # 8 significant bits
    real_m = away_from_zero(torch.randn(n, generator=gen) * 1e-4, 1e-6).bfloat16()
    real_v = (torch.randn(n, generator=gen) * 1e-6).abs().float()
    g_fp16 = (real_g.float() * scale).half()
    m_fp16 = (real_m.float() * scale).half()
    assert torch.equal(g_fp16.float(), real_g.float() * scale) and torch.equal(m_fp16.float(), real_m.float() * scale)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 7)
    # bf16 tree on the real quantities (scale 1)
    pa = p0.copy(); ma = real_m.float().numpy().copy(); va = real_v.numpy().copy(); ha = np.zeros(n, np.uint16)
    oracle.adam_gpu_bf16(pa, ha, bits16(real_g), ma, va, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
    # fp16 tree on the scaled quantities
    pb = p0.copy(); mb = bits16(m_fp16); vb = (real_v * scale).numpy().copy(); hb = np.zeros(n, np.uint16)
    oracle.adam_gpu_fp16(pb, hb, bits16(g_fp16), mb, vb, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
    assert np.array_equal(f32_bits(pa), f32_bits(pb))
    assert np.array_equal(f32_bits(va * np.float32(scale)), f32_bits(vb))
    assert np.array_equal(mb, bits16(torch.from_numpy(ma * np.float32(scale)).half()))
    assert np.array_equal(hb, bits16(torch.from_numpy(pb).half()))


def test_gpu_fp16_tree_against_float64():
    gen = torch.Generator().manual_seed(4)
    n = 20000
    scale = 1000.0      # not a power of two
    p0 = (torch.randn(n, generator=gen) * 0.02)
    g16 = (torch.randn(n, generator=gen) * 1e-3 * scale).half()
    p = p0.numpy().copy(); m16 = np.zeros(n, np.uint16); v = np.zeros(n, np.float32); h = np.zeros(n, np.uint16)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 1)
    oracle.adam_gpu_fp16(p, h, bits16(g16), m16, v, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
    g_real = g16.double().numpy() / float(np.float32(scale))
    p64, m64, v64 = _adamw_float64(p0.double().numpy(), g_real, np.zeros(n), np.zeros(n), 0.9, 0.999, 1e-8, 1e-3, 0.01, 1)
    assert np.abs(p - p64).max() <= 1e-6 * np.abs(p64).max()
    assert np.abs(v / np.float32(scale) - v64).max() <= 1e-6 * np.abs(v64).max()
    m_real = oracle.half_to_float(m16) / np.float32(scale)
    assert np.abs(m_real - m64).max() <= 2.0 ** -11 * np.abs(m64).max() + 6e-8 / scale   # fp16 rounding of m*scale


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_lr_zero_freezes_parameters_but_not_moments(flavour):
    """hold_steps passes lr = 0 (adam.py:155): p' = fma(-0, p, p - 0) = p exactly."""
    gen = torch.Generator().manual_seed(6)
    n = 1000
    p0 = (torch.randn(n, generator=gen) * 0.02).numpy()
    p = p0.copy(); v = np.zeros(n, np.float32); h = np.zeros(n, np.uint16)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 1)
    gt = torch.randn(n, generator=gen)
    if flavour == "bf16":
        m = np.zeros(n, np.float32)
        oracle.adam_gpu_bf16(p, h, bits16(gt.bfloat16()), m, v, 0.9, 0.999, 1e-8, 0.0, 1.0, 0.01, bc1, bc2)
        assert np.all(m != 0)
    else:
        m = np.zeros(n, np.uint16)
        oracle.adam_gpu_fp16(p, h, bits16(gt.half()), m, v, 0.9, 0.999, 1e-8, 0.0, 4.0, 0.01, bc1, bc2)
        assert np.all(m != 0)
    assert np.array_equal(f32_bits(p), f32_bits(p0))
    assert np.all(v > 0)
