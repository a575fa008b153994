"""Seeded random shapes, base offsets and hyper-parameters through the C ABI against the oracle:
the cases nobody thought of writing down."""
import numpy as np
import pytest
import torch

import oracle
from bmtrain_amd.loss import _function as LF
from bmtrain_amd.optim import _function as OF
from conftest import bits16, f32_bits, ulp_distance16

pytestmark = pytest.mark.gpu


def _offset_view(t, off, pad=16):
    buf = torch.zeros(t.numel() + pad, dtype=t.dtype, device="cuda")
    buf[off:off + t.numel()] = t.reshape(-1).cuda()
    return buf, buf[off:off + t.numel()].view(t.shape)


@pytest.mark.parametrize("seed", range(24))
def test_cross_entropy_random_case(seed):
    rnd = np.random.default_rng(1000 + seed)
    name, dtype = [("fp16", torch.float16), ("bf16", torch.bfloat16)][seed % 2]
    n = int(rnd.choice([rnd.integers(1, 40), rnd.integers(40, 3000), rnd.integers(3000, 40000), rnd.integers(40000, 140000)]))
    m = int(rnd.integers(1, max(2, min(40, 400000 // n))))
    off = int(rnd.integers(0, 8))
    std = float(rnd.choice([0.1, 1.0, 4.0, 20.0]))
    ignore = int(rnd.choice([-100, 0, n - 1]))
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, n, generator=gen) * std + float(rnd.normal() * 5)).to(dtype)
    t = torch.randint(0, n, (m,), generator=gen, dtype=torch.int32)
    t[torch.rand(m, generator=gen) < 0.2] = ignore
    want_soft, want_loss = oracle.ce_forward(bits16(x), t.numpy(), ignore, name)
    _, xg = _offset_view(x, off)
    soft_buf, soft = _offset_view(torch.zeros_like(x), off)
    out = torch.empty(m, dtype=torch.float32, device="cuda")
    LF.cross_entropy_forward(m, n, xg, t.cuda(), soft, out, ignore)
    case = (name, m, n, off, std, ignore)
    assert ulp_distance16(bits16(soft), want_soft).max() <= 1, case
    np.testing.assert_allclose(out.cpu().numpy(), want_loss, rtol=3e-6, atol=3e-6, err_msg=str(case))
    v = (torch.rand(m, generator=gen) * float(rnd.choice([1.0, 1024.0]))).float()
    want = bits16(soft)
    oracle.ce_backward_inplace(v.numpy(), t.numpy(), want, ignore, name)
    LF.cross_entropy_backward_inplace(m, n, v.cuda(), t.cuda(), soft, ignore)
    assert np.array_equal(bits16(soft), want), case
    assert soft_buf[:off].count_nonzero() == 0 and soft_buf[off + m * n:].count_nonzero() == 0, case


@pytest.mark.parametrize("seed", range(24))
def test_adam_random_case(seed):
    rnd = np.random.default_rng(2000 + seed)
    flavour = ["bf16", "fp16"][seed % 2]
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    mdt = torch.float16 if flavour == "fp16" else torch.float32
    n = int(rnd.choice([rnd.integers(1, 64), rnd.integers(64, 10000), rnd.integers(10000, 600000)]))
    off = int(rnd.integers(0, 4))
    scale = float(rnd.choice([1.0, 128.0, 1000.0, 65536.0])) if flavour == "fp16" else float(rnd.choice([1.0, 3.0, 1024.0]))
    lr = float(rnd.choice([0.0, 1e-4, 1e-2]))
    wd = float(rnd.choice([0.0, 0.01, 0.3]))
    b1, b2 = float(rnd.choice([0.0, 0.9, 0.99])), float(rnd.choice([0.9, 0.999]))
    eps = float(rnd.choice([1e-8, 1e-5]))
    step = int(rnd.integers(1, 5000))
    gen = torch.Generator().manual_seed(seed)
    p = torch.randn(n, generator=gen) * 0.05
    g = (torch.randn(n, generator=gen) * 1e-3 * min(scale, 1024.0)).to(dt16)
    m = (torch.randn(n, generator=gen) * 1e-4 * (scale if flavour == "fp16" else 1.0)).clamp(-6e4, 6e4).to(mdt)
    v = (torch.randn(n, generator=gen) * 1e-6 * (scale if flavour == "fp16" else 1.0)).abs()
    (_, pg), (_, gg), (_, mg), (_, vg) = (_offset_view(t, off) for t in (p, g, m, v))
    h_buf, hg = _offset_view(torch.zeros(n, dtype=dt16), off)
    fn = OF.adam_fp16 if flavour == "fp16" else OF.adam_bf16
    fn(pg, hg, gg, mg, vg, b1, b2, eps, lr, scale, wd, step)
    bc1, bc2 = oracle.bias_corrections(b1, b2, step)
    po, vo, ho = p.numpy().copy(), v.numpy().copy(), np.zeros(n, np.uint16)
    case = (flavour, n, off, scale, lr, wd, b1, b2, eps, step)
    if flavour == "fp16":
        mo = bits16(m)
        oracle.adam_gpu_fp16(po, ho, bits16(g), mo, vo, b1, b2, eps, lr, scale, wd, bc1, bc2)
        assert np.array_equal(bits16(mg), mo), case
    else:
        mo = m.numpy().copy()
        oracle.adam_gpu_bf16(po, ho, bits16(g), mo, vo, b1, b2, eps, lr, scale, wd, bc1, bc2)
        assert np.array_equal(f32_bits(mg.cpu().numpy()), f32_bits(mo)), case
    assert np.array_equal(f32_bits(pg.cpu().numpy()), f32_bits(po)), case
    assert np.array_equal(f32_bits(vg.cpu().numpy()), f32_bits(vo)), case
    assert np.array_equal(bits16(hg), ho), case
    assert h_buf[:off].count_nonzero() == 0 and h_buf[off + n:].count_nonzero() == 0, case
