"""Fused Adam on the GPU, through the C ABI, against the oracle.

The kernels implement one fixed expression tree with correctly rounded division and square
root, so the bar here is tighter than the stated tolerance (fp32 state <= 1e-6 relative,
16-bit copy <= 1 ulp): every output must equal the oracle's bit for bit.  The oracle's tree is
itself pinned to the reference's compiled CPU Adam (tests/test_oracle_adam.py)."""
import numpy as np
import pytest
import torch

import oracle
from bmtrain_amd.optim import _function as F
from conftest import bits16, f32_bits, from_bits16, load_golden

pytestmark = pytest.mark.gpu
HYP = dict(beta1=0.9, beta2=0.999, eps=1e-8, lr=1e-3, weight_decay=0.01)


def _state(n, gen, flavour):
    p = torch.randn(n, generator=gen) * 0.02
    m = torch.randn(n, generator=gen) * 1e-4
    v = (torch.randn(n, generator=gen) * 1e-6).abs()
    if flavour == "fp16":
        m = m.half()
    return p, m, v


def _run_both(flavour, p, m, v, g, scale, step, lr=HYP["lr"], wd=HYP["weight_decay"], offset=0):
    """Steps GPU copies (placed `offset` elements into larger buffers) and oracle copies."""
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    n = p.numel()

    def place(t):
        buf = torch.zeros(n + offset + 8, dtype=t.dtype, device="cuda")
        buf[offset:offset + n] = t.cuda()
        return buf, buf[offset:offset + n]

    (pb, pg), (mb, mg), (vb, vg), (gb, gg) = place(p), place(m), place(v), place(g)
    hb, hg = place(torch.zeros(n, dtype=dt16))
    fn = F.adam_fp16 if flavour == "fp16" else F.adam_bf16
    fn(pg, hg, gg, mg, vg, HYP["beta1"], HYP["beta2"], HYP["eps"], lr, scale, wd, step)
    torch.cuda.synchronize()
    # nothing outside the view may change
    for buf in (pb, mb, vb, hb):
        assert torch.count_nonzero(buf[:offset]) == 0 and torch.count_nonzero(buf[offset + n:]) == 0

    po, vo, ho = p.numpy().copy(), v.numpy().copy(), np.zeros(n, np.uint16)
    bc1, bc2 = oracle.bias_corrections(HYP["beta1"], HYP["beta2"], step)
    if flavour == "fp16":
        mo = bits16(m)
        oracle.adam_gpu_fp16(po, ho, bits16(g), mo, vo, HYP["beta1"], HYP["beta2"], HYP["eps"], lr, scale, wd, bc1, bc2)
        m_equal = np.array_equal(bits16(mg), mo)
    else:
        mo = m.numpy().copy()
        oracle.adam_gpu_bf16(po, ho, bits16(g), mo, vo, HYP["beta1"], HYP["beta2"], HYP["eps"], lr, scale, wd, bc1, bc2)
        m_equal = np.array_equal(f32_bits(mg.cpu().numpy()), f32_bits(mo))
    assert np.array_equal(f32_bits(pg.cpu().numpy()), f32_bits(po)), "fp32 master"
    assert np.array_equal(f32_bits(vg.cpu().numpy()), f32_bits(vo)), "second moment"
    assert m_equal, "first moment"
    assert np.array_equal(bits16(hg), ho), "16-bit copy"
    return pg.cpu(), mg.cpu(), vg.cpu()


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 8, 63, 1023, 1024, 1025, 2047, 2048, 2049, 4099, (1 << 20) + 3])
def test_bit_exact_against_oracle(flavour, n):
    gen = torch.Generator().manual_seed(n)
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    p, m, v = _state(n, gen, flavour)
    for step, scale in ((1, 1.0), (2, 1024.0), (100, 3.0)):
        g = (torch.randn(n, generator=gen) * 1e-3 * scale).to(dt16)
        p, m, v = _run_both(flavour, p, m, v, g, scale, step)


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
@pytest.mark.parametrize("offset", [1, 2, 3, 4, 5, 6, 7])
def test_views_at_any_element_offset(flavour, offset):
    """Parameters are often slices of one flat buffer.  All arrays offset alike: vector body with
    scalar head/tail; the guard elements around the views must stay untouched."""
    gen = torch.Generator().manual_seed(offset)
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    for n in (1, 3, 6, 1000, 5001):
        p, m, v = _state(n, gen, flavour)
        g = (torch.randn(n, generator=gen) * 1e-3).to(dt16)
        _run_both(flavour, p, m, v, g, 1.0, 3, offset=offset)


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_arrays_with_different_alignment_phases(flavour):
    """fp32 master at offset 1, gradient at offset 2, ...: no common vector phase, element path."""
    gen = torch.Generator().manual_seed(77)
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    n = 3001
    p, m, v = _state(n, gen, flavour)
    g = (torch.randn(n, generator=gen) * 1e-3).to(dt16)
    bufs = {}
    for k, (name, t) in enumerate((("p", p), ("m", m), ("v", v), ("g", g), ("h", torch.zeros(n, dtype=dt16)))):
        b = torch.zeros(n + 16, dtype=t.dtype, device="cuda")
        b[k + 1:k + 1 + n] = t.cuda()
        bufs[name] = b[k + 1:k + 1 + n]
    fn = F.adam_fp16 if flavour == "fp16" else F.adam_bf16
    fn(bufs["p"], bufs["h"], bufs["g"], bufs["m"], bufs["v"], 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 5)
    po, vo, ho = p.numpy().copy(), v.numpy().copy(), np.zeros(n, np.uint16)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 5)
    if flavour == "fp16":
        mo = bits16(m)
        oracle.adam_gpu_fp16(po, ho, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
    else:
        mo = m.numpy().copy()
        oracle.adam_gpu_bf16(po, ho, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
    assert np.array_equal(f32_bits(bufs["p"].cpu().numpy()), f32_bits(po))
    assert np.array_equal(bits16(bufs["h"]), ho)


def test_bf16_kernel_reproduces_the_reference_compiled_cpu_adam():
    """Vectors written by the reference's own adam_cpu.hpp (bf16 path): the GPU kernel's fp32
    parameters and moments are identical bit for bit; the bf16 copy is the round-to-nearest-even
    neighbour of the reference CPU path's truncated copy (0 or 1 ulp above it)."""
    g = load_golden("adam_cpu_bf16_t8")
    n = int(g["n"])
    p = torch.from_numpy(g["p0"].copy()).cuda()
    m = torch.zeros(n, device="cuda"); v = torch.zeros(n, device="cuda")
    h = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    for s in range(1, int(g["steps"]) + 1):
        grad = from_bits16(g[f"g{s}"], torch.bfloat16).cuda()
        F.adam_bf16(p, h, grad, m, v, float(g["beta1"]), float(g["beta2"]), float(g["eps"]), float(g["lr"]),
                    float(g["scale"]), float(g["weight_decay"]), s)
        assert np.array_equal(f32_bits(p.cpu().numpy()), f32_bits(g[f"p{s}"]))
        assert np.array_equal(f32_bits(m.cpu().numpy()), f32_bits(g[f"m{s}"]))
        assert np.array_equal(f32_bits(v.cpu().numpy()), f32_bits(g[f"v{s}"]))
        d = bits16(h).astype(np.int32) - g[f"h{s}"].astype(np.int32)
        assert d.min() >= 0 and d.max() <= 1


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_tolerances_against_float64(flavour):
    """The stated bars, against a float64 evaluation: fp32 state <= 1e-6 relative (norm-wise),
    16-bit copy <= 1 ulp of the float64 result."""
    from conftest import ulp_distance16
    gen = torch.Generator().manual_seed(21)
    n = 200000
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    scale = 1024.0 if flavour == "fp16" else 1.0
    p = torch.randn(n, generator=gen) * 0.02
    m_real = torch.randn(n, generator=gen) * 1e-4
    v_real = (torch.randn(n, generator=gen) * 1e-6).abs()
    g = (torch.randn(n, generator=gen) * 1e-3 * scale).to(dt16)
    step = 100
    pg, vg, gg = p.cuda(), (v_real * scale).cuda() if flavour == "fp16" else v_real.cuda(), g.cuda()
    hg = torch.zeros(n, dtype=dt16, device="cuda")
    if flavour == "fp16":
        mg = (m_real * scale).half().cuda()
        m_in = mg.double().cpu() / scale
        F.adam_fp16(pg, hg, gg, mg, vg, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, step)
    else:
        mg = m_real.cuda()
        m_in = m_real.double()
        F.adam_bf16(pg, hg, gg, mg, vg, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, step)
    f = lambda x: float(np.float32(x))
    b1, b2, eps, lr, wd = f(0.9), f(0.999), f(1e-8), f(1e-3), f(0.01)
    bc1, bc2 = (f(c) for c in oracle.bias_corrections(0.9, 0.999, step))
    greal = g.double() / scale
    m64 = b1 * m_in + f(np.float32(1) - np.float32(0.9)) * greal
    v64 = b2 * v_real.double() + f(np.float32(1) - np.float32(0.999)) * greal * greal
    p64 = p.double() - lr * (m64 / bc1) / (torch.sqrt(v64 / bc2) + eps) - lr * wd * p.double()
    rel = lambda a, b: ((a - b).abs().max() / b.abs().max()).item()
    assert rel(pg.double().cpu(), p64) <= 1e-6
    assert rel(vg.double().cpu() / (scale if flavour == "fp16" else 1.0), v64) <= 1e-6
    if flavour == "bf16":
        assert rel(mg.double().cpu(), m64) <= 1e-6
    assert ulp_distance16(bits16(hg), bits16(p64.to(dt16))).max() <= 1


def test_lr_zero_holds_parameters():
    n = 10000
    gen = torch.Generator().manual_seed(8)
    p = (torch.randn(n, generator=gen) * 0.02).cuda()
    p0 = p.clone()
    h = p.bfloat16()
    m = torch.zeros(n, device="cuda"); v = torch.zeros(n, device="cuda")
    g = torch.randn(n, generator=gen).bfloat16().cuda()
    F.adam_bf16(p, h, g, m, v, 0.9, 0.999, 1e-8, 0.0, 1.0, 0.01, 1)
    assert torch.equal(p, p0) and torch.count_nonzero(m) == n and torch.count_nonzero(v) == n


def test_argument_checks():
    n = 16
    p = torch.zeros(n, device="cuda"); m = torch.zeros(n, device="cuda"); v = torch.zeros(n, device="cuda")
    h = torch.zeros(n, dtype=torch.bfloat16, device="cuda"); g = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    a = (0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 1)
    with pytest.raises(AssertionError, match="same number"):
        F.adam_bf16(p, h, g[:8], m, v, *a)
    with pytest.raises(AssertionError, match="bfloat16"):
        F.adam_bf16(p, h.half(), g, m, v, *a)
    with pytest.raises(AssertionError, match="cuda"):
        F.adam_bf16(p.cpu(), h, g, m, v, *a)
    with pytest.raises(AssertionError, match="float16"):
        F.adam_fp16(p, h, g, m.half(), v, *a)
    # the 16-bit parameter is output only (long launches keep their tile counters there): a launch whose
    # 16-bit output shares memory with the gradient or the state is refused
    both = torch.zeros(2 * n, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="overlaps"):
        F.adam_bf16(p, both[4:4 + n], both[:n], m, v, *a)
    with pytest.raises(RuntimeError, match="overlaps"):
        F.adam_bf16(p, p.view(torch.bfloat16)[:n], g, m, v, *a)
    F.adam_bf16(p, both[n:], both[:n], m, v, *a)          # adjacent is fine


def test_a_bad_entry_anywhere_in_a_multi_tensor_table_means_nothing_was_stepped():
    """The multi-tensor launcher checks its whole table before the first launch: 70 tensors (three launches' worth)
    with the last one's 16-bit output overlapping its gradient are refused, and no tensor — not even those of the
    first two launches — has been touched."""
    gen = torch.Generator(device="cuda").manual_seed(5)
    rows, originals = [], []
    for k in range(70):
        n = 5000 + 4 * k
        p = torch.randn(n, generator=gen, device="cuda") * 0.02
        g = (torch.randn(n, generator=gen, device="cuda") * 1e-3).bfloat16()
        rows.append((p, torch.full((n,), -1, dtype=torch.bfloat16, device="cuda"), g, torch.zeros(n, device="cuda"),
                     torch.zeros(n, device="cuda")))
        originals.append(p.clone())
    p, h, g, m, v = rows[-1]
    rows[-1] = (p, g.view(torch.bfloat16), g, m, v)              # 16-bit output == gradient
    with pytest.raises(RuntimeError, match="overlaps"):
        F.adam_multi(rows, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 3)
    torch.cuda.synchronize()
    for (p, h, g, m, v), p0 in zip(rows[:-1], originals):
        assert torch.equal(p, p0) and torch.count_nonzero(m) == 0 and torch.count_nonzero(v) == 0
        assert torch.equal(h.view(torch.int16), torch.full_like(h, -1).view(torch.int16))


def test_a_long_batch_whose_counter_host_is_shared_takes_the_kernel_without_counters():
    """A long batch keeps its tile counters in the tail of the largest tensor's 16-bit output.  When another entry
    of the table shares that memory (here: a second tensor whose 16-bit output is a view into the large tensor's
    output tail — its values are overwritten by whichever store comes last, as in any table that names memory
    twice), the batch must not keep counters there: the large tensor's fp32 state, which nothing else touches,
    comes out exactly as from a launch of its own."""
    n = (3 << 22) + 4096
    gen = torch.Generator(device="cuda").manual_seed(9)
    p = torch.randn(n, generator=gen, device="cuda") * 0.02
    g = (torch.randn(n, generator=gen, device="cuda") * 1e-3).bfloat16()
    alone = (p.clone(), torch.zeros(n, dtype=torch.bfloat16, device="cuda"), g, torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"))
    F.adam_bf16(*alone, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 3)
    big = (p.clone(), torch.zeros(n, dtype=torch.bfloat16, device="cuda"), g, torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"))
    k = 4096
    small = (torch.zeros(k, device="cuda"), big[1][n - k:], torch.zeros(k, dtype=torch.bfloat16, device="cuda"),
             torch.zeros(k, device="cuda"), torch.zeros(k, device="cuda"))
    F.adam_multi([big, small], 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 3)
    torch.cuda.synchronize()
    for a, b in zip((alone[0], alone[3], alone[4]), (big[0], big[3], big[4])):
        assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert torch.equal(alone[1][:n - k].view(torch.int16), big[1][:n - k].view(torch.int16))
    assert torch.count_nonzero(small[0]) == 0                     # zero gradient, zero state: the small tensor stays zero


def _fill_(x, std, gen, absolute=False, chunk=1 << 27):
    for lo in range(0, x.numel(), chunk):
        part = x[lo:lo + chunk]
        r = torch.randn(part.numel(), generator=gen, device="cuda", dtype=torch.float32).mul_(std)
        part.copy_(r.abs_() if absolute else r)


def _check_slices(n, slices, before, after, step, scale):
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, step)
    for lo, hi in slices:
        po, mo, vo = (before[k][lo:hi].cpu().numpy().copy() for k in ("p", "m", "v"))
        ho = np.zeros(hi - lo, np.uint16)
        oracle.adam_gpu_bf16(po, ho, bits16(before["g"][lo:hi]), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
        assert np.array_equal(f32_bits(after["p"][lo:hi].cpu().numpy()), f32_bits(po)), (lo, hi)
        assert np.array_equal(f32_bits(after["m"][lo:hi].cpu().numpy()), f32_bits(mo)), (lo, hi)
        assert np.array_equal(f32_bits(after["v"][lo:hi].cpu().numpy()), f32_bits(vo)), (lo, hi)
        assert np.array_equal(bits16(after["h"][lo:hi]), ho), (lo, hi)


def test_one_transformer_block_flat_buffer():
    """202,383,360 elements (4*4096^2 + 3*4096*11008), step 100, scale 1.  Seeded slices are checked
    against the oracle bit for bit; the whole buffer is checked by stepping a second copy in
    three separately launched pieces (different tile-to-workgroup mapping) and comparing all of it."""
    n = 202_383_360
    gen = torch.Generator(device="cuda").manual_seed(1)
    before = {"p": torch.empty(n, device="cuda"), "m": torch.empty(n, device="cuda"), "v": torch.empty(n, device="cuda"),
              "g": torch.empty(n, dtype=torch.bfloat16, device="cuda")}
    _fill_(before["p"], 0.02, gen); _fill_(before["m"], 1e-4, gen); _fill_(before["v"], 1e-6, gen, absolute=True)
    _fill_(before["g"], 1e-3, gen)
    after = {k: before[k].clone() for k in ("p", "m", "v")}
    after["h"] = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    F.adam_bf16(after["p"], after["h"], before["g"], after["m"], after["v"], 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100)
    rnd = np.random.default_rng(1)
    starts = [0, n - 70000] + [int(s) for s in rnd.integers(0, n - 70000, 6)]
    _check_slices(n, [(s, s + 65536 + 11) for s in starts], before, after, 100, 1.0)
    pieces = {k: before[k].clone() for k in ("p", "m", "v")}
    pieces["h"] = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    cuts = [0, 50_000_003, 120_000_001, n]
    for lo, hi in zip(cuts[:-1], cuts[1:]):
        F.adam_bf16(pieces["p"][lo:hi], pieces["h"][lo:hi], before["g"][lo:hi], pieces["m"][lo:hi], pieces["v"][lo:hi],
                    0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100)
    for k in ("p", "m", "v", "h"):
        assert torch.equal(pieces[k].view(torch.int32 if k != "h" else torch.int16),
                           after[k].view(torch.int32 if k != "h" else torch.int16)), k


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
@pytest.mark.parametrize("n,off", [((3 << 22) - 1, 0), ((3 << 22) + 2, 2), ((3 << 22) + 1024 * 7 + 5, 1), ((3 << 22) + 12, 3),
                                   ((1 << 24) - 1, 0), ((1 << 24) + 2, 2), ((1 << 24) + 1024 * 7 + 5, 1), ((1 << 24) + 4 * 2048 + 3, 0),
                                   ((1 << 25) + 12345, 0), ((1 << 25) + 4096 * 3 + 1, 2), (3 * (1 << 24) + 4 * 1537, 3),
                                   ((1 << 24) + 77, 8), ((3 << 22) + 5000, 256), ((1 << 25) + 1, 1000), ((3 << 22) + 1023, 1),
                                   ((3 << 22) + 1020, 4), ((5 << 21) - 1, 0), ((5 << 21) + 2, 2), ((5 << 21) + 1023, 1),
                                   ((3 << 23) - 1, 0), ((3 << 23) + 1024 * 7 + 5, 1), ((3 << 23) + 1020, 4)])
def test_around_the_launch_size_where_the_resident_grid_takes_over(flavour, n, off):
    """From 10,485,760 (bf16) or 25,165,824 (fp16) elements on, a resident grid draws tiles of 256 groups from four
    counters: a slot of the library's own array when the stream has one (here), else places in the 16-bit output
    (word 0 of the vectors nvec-1, nvec-513, nvec-1025, nvec-1537; covered under graph capture in
    test_gpu_streams_graphs.py).  Whole-buffer comparison with the oracle just below and above both sizes, with
    unaligned heads and partial last tiles: every tile stepped exactly once, every 16-bit value in place.  A resident launch starts its tiles at the fp32 parameters' next 4 KiB boundary and leaves
    the up to 1,023 elements in front of it to the element kernel (offsets 1 to 1,000 below), unless that would take
    the call below the size of a resident launch (the last two cases)."""
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    mdt = torch.float16 if flavour == "fp16" else torch.float32
    scale = 4.0 if flavour == "fp16" else 1.0
    gen = torch.Generator().manual_seed(n)
    p = torch.randn(n, generator=gen) * 0.02
    m = (torch.randn(n, generator=gen) * 1e-4 * scale).to(mdt)
    v = (torch.randn(n, generator=gen) * 1e-6 * scale).abs()
    g = (torch.randn(n, generator=gen) * 1e-3 * scale).to(dt16)
    def place(t, fill=0):
        buf = torch.full((n + 1032,), fill, dtype=t.dtype, device="cuda")
        buf[off:off + n] = t.cuda()
        return buf[off:off + n]
    pg, mg, vg, gg = place(p), place(m), place(v), place(g)
    hg = place(torch.zeros(n, dtype=dt16), fill=-1)        # a non-zero pattern where the counter will live
    fn = F.adam_fp16 if flavour == "fp16" else F.adam_bf16
    fn(pg, hg, gg, mg, vg, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 7)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 7)
    po, vo = p.numpy().copy(), v.numpy().copy()
    ho = np.zeros(n, np.uint16)
    if flavour == "fp16":
        mo = bits16(m)
        oracle.adam_gpu_fp16(po, ho, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
        assert np.array_equal(bits16(mg), mo)
    else:
        mo = m.numpy().copy()
        oracle.adam_gpu_bf16(po, ho, bits16(g), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
        assert np.array_equal(f32_bits(mg.cpu().numpy()), f32_bits(mo))
    assert np.array_equal(f32_bits(pg.cpu().numpy()), f32_bits(po))
    assert np.array_equal(f32_bits(vg.cpu().numpy()), f32_bits(vo))
    assert np.array_equal(bits16(hg), ho)


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_more_than_2_to_the_31_elements(flavour):
    """Element counts beyond int32 (the reference's launchers take `int n`, adam_cuda.cu:76,103): the last stretch of a
    2^31 + 12345 element buffer must be stepped, and stepped correctly, in both flavours."""
    n = (1 << 31) + 12345
    fp16 = flavour == "fp16"
    dt16 = torch.float16 if fp16 else torch.bfloat16
    scale = 8.0 if fp16 else 1.0
    gen = torch.Generator(device="cuda").manual_seed(31)
    before = {"p": torch.empty(n, device="cuda"), "m": torch.zeros(n, dtype=torch.float16 if fp16 else torch.float32, device="cuda"),
              "v": torch.zeros(n, device="cuda"), "g": torch.empty(n, dtype=dt16, device="cuda")}
    _fill_(before["p"], 0.02, gen); _fill_(before["g"], 1e-3 * scale, gen)
    slices = [(0, 4096), ((1 << 31) - 2048, (1 << 31) + 2048), (n - 12345, n)]
    snap = {k: {s: before[k][s[0]:s[1]].clone() for s in slices} for k in ("p", "m", "v", "g")}
    h = torch.zeros(n, dtype=dt16, device="cuda")
    fn = F.adam_fp16 if fp16 else F.adam_bf16
    fn(before["p"], h, before["g"], before["m"], before["v"], 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 1)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 1)
    for s in slices:
        po, vo = (snap[k][s].cpu().numpy().copy() for k in ("p", "v"))
        ho = np.zeros(s[1] - s[0], np.uint16)
        if fp16:
            mo = bits16(snap["m"][s])
            oracle.adam_gpu_fp16(po, ho, bits16(snap["g"][s]), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
            assert np.array_equal(bits16(before["m"][s[0]:s[1]]), mo), s
        else:
            mo = snap["m"][s].cpu().numpy().copy()
            oracle.adam_gpu_bf16(po, ho, bits16(snap["g"][s]), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
            assert np.array_equal(f32_bits(before["m"][s[0]:s[1]].cpu().numpy()), f32_bits(mo)), s
        assert np.array_equal(f32_bits(before["p"][s[0]:s[1]].cpu().numpy()), f32_bits(po)), s
        assert np.array_equal(f32_bits(before["v"][s[0]:s[1]].cpu().numpy()), f32_bits(vo)), s
        assert np.array_equal(bits16(h[s[0]:s[1]]), ho), s
    # every element of the last stretch was stepped (a gradient that rounded to zero leaves v at zero)
    assert torch.count_nonzero(before["v"][-(1 << 20):]) == torch.count_nonzero(before["g"][-(1 << 20):]) > (1 << 20) - 64
    del before, h, snap
    torch.cuda.empty_cache()


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_multi_tensor_launch_equals_per_tensor_launches(flavour):
    """adam_multi: many tensors per launch, bit for bit what one launch per tensor produces (and hence the
    oracle), including sizes that are not multiples of 4, more tensors than one batch holds, and a tensor
    whose views are not vector-aligned (stepped alone)."""
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    mdt = torch.float16 if flavour == "fp16" else torch.float32
    gen = torch.Generator().manual_seed(12)
    sizes = [1, 2, 3, 4, 5, 1023, 1024, 4096, 4097, 4099, 128 * 128, 1237, 65536 + 3, 7, 300001] + [257] * 40
    single, multi = [], []
    for k, n in enumerate(sizes):
        p = torch.randn(n, generator=gen) * 0.02
        m = (torch.randn(n, generator=gen) * 1e-4).to(mdt)
        v = (torch.randn(n, generator=gen) * 1e-6).abs()
        g = (torch.randn(n, generator=gen) * 1e-3 * 8).to(dt16)
        def place(t, off):
            buf = torch.zeros(t.numel() + 8, dtype=t.dtype, device="cuda")
            buf[off:off + t.numel()] = t.cuda()
            return buf[off:off + t.numel()]
        off = 1 if k == 9 else 0          # one unaligned tensor
        for dest in (single, multi):
            dest.append((place(p, off), place(torch.zeros(n, dtype=dt16), off), place(g, off), place(m, off), place(v, off)))
    fn = F.adam_fp16 if flavour == "fp16" else F.adam_bf16
    for step in (1, 2):
        for p32, p16, g, m, v in single:
            fn(p32, p16, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 8.0, 0.01, step)
        F.adam_multi(multi, 0.9, 0.999, 1e-8, 1e-3, 8.0, 0.01, step)
    for a, b in zip(single, multi):
        for x, y in zip(a, b):
            assert torch.equal(x.view(torch.int16 if x.element_size() == 2 else torch.int32),
                               y.view(torch.int16 if y.element_size() == 2 else torch.int32))
    F.adam_multi([], 0.9, 0.999, 1e-8, 1e-3, 8.0, 0.01, 1)
    with pytest.raises(AssertionError):
        F.adam_multi([(single[0][0], single[0][1].float(), single[0][2], single[0][3], single[0][4])], 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 1)


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_long_multi_tensor_launch_runs_as_one_resident_grid(flavour):
    """Batches of 3 * 2^22 (bf16) or 3 * 2^23 (fp16) elements or more run as one resident grid over all their tensors: tiles of 256 groups numbered
    through the tensors, drawn by ticket from four counters kept in the 16-bit output of the largest tensor; leftover
    elements and the counters' places are finished by a small kernel.  40 tensors (two launches, the second a short
    one), 33 equal tensors, and a mix of sizes from 3 to 2^24 + 5 elements with every leftover count — bit for bit
    against one launch per tensor."""
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    mdt = torch.float16 if flavour == "fp16" else torch.float32
    fn = F.adam_fp16 if flavour == "fp16" else F.adam_bf16
    for sizes in ([1_200_001 + 4 * k for k in range(39)] + [2_000_003], [1_200_000] * 32 + [4096 * 300 + 3],
                  [(1 << 24) + 5, 77, 4096, (1 << 22) + 2, 3, 1_000_001, 255, 1024, 1023, 6, (1 << 23) + 3],
                  [(1 << 22) + 1, (1 << 23) + 2, 4099, 255],          # 12.6 M elements: resident for bf16, short kernel for fp16
                  [(3 << 22) - 8192, 4096, 4097],                      # just above the bf16 size, the largest tensor just below it
                  [(3 << 23) - 8192, 4096, 4097]):                     # the same at the fp16 size
        gen = torch.Generator(device="cuda").manual_seed(len(sizes))
        single, multi = [], []
        for n in sizes:
            p = torch.randn(n, generator=gen, device="cuda") * 0.02
            m = (torch.randn(n, generator=gen, device="cuda") * 1e-4).to(mdt)
            v = (torch.randn(n, generator=gen, device="cuda") * 1e-6).abs()
            g = (torch.randn(n, generator=gen, device="cuda") * 1e-3).to(dt16)
            for dest in (single, multi):
                dest.append((p.clone(), torch.full((n,), -1, dtype=dt16, device="cuda"), g, m.clone(), v.clone()))
        for p32, p16, g, m, v in single:
            fn(p32, p16, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 2.0, 0.01, 5)
        F.adam_multi(multi, 0.9, 0.999, 1e-8, 1e-3, 2.0, 0.01, 5)
        for a, b in zip(single, multi):
            for x, y in zip(a, b):
                assert torch.equal(x.view(torch.int16 if x.element_size() == 2 else torch.int32),
                                   y.view(torch.int16 if y.element_size() == 2 else torch.int32))


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_multi_tensor_launch_of_more_than_2_to_the_31_elements(flavour):
    """A batch of 2^31 elements or more takes its tiles from the four counters in turn, and a workgroup's tiles may then
    step back over a tensor boundary.  Five tensors of 3 to 1.2 B elements (2.4 B in all, every leftover count, the
    largest one - which hosts the counters - in the middle) in one multi-tensor launch against one launch per tensor,
    by checksum of every array and bit for bit on a slice around every tensor's end."""
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    mdt = torch.float16 if flavour == "fp16" else torch.float32
    fn = F.adam_fp16 if flavour == "fp16" else F.adam_bf16
    sizes = [900_000_001, 3, 1_200_000_002, 4099, 300_000_003]
    assert sum(sizes) >= 1 << 31
    gen = torch.Generator(device="cuda").manual_seed(9)

    def filled(n, std, dtype, absolute=False):
        x = torch.empty(n, dtype=dtype, device="cuda")
        for lo in range(0, n, 1 << 27):
            part = x[lo:lo + (1 << 27)]
            r = torch.randn(part.numel(), generator=gen, device="cuda") * std
            part.copy_(r.abs() if absolute else r)
        return x
    single, multi = [], []
    for n in sizes:
        p, m = filled(n, 0.02, torch.float32), filled(n, 1e-4, mdt)
        v, g = filled(n, 1e-6, torch.float32, absolute=True), filled(n, 1e-3, dt16)
        single.append((p, torch.full((n,), -1, dtype=dt16, device="cuda"), g, m, v))
        multi.append((p.clone(), torch.full((n,), -1, dtype=dt16, device="cuda"), g, m.clone(), v.clone()))
    for p32, p16, g, m, v in single:
        fn(p32, p16, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 2.0, 0.01, 5)
    F.adam_multi(multi, 0.9, 0.999, 1e-8, 1e-3, 2.0, 0.01, 5)
    torch.cuda.synchronize()
    for a, b in zip(single, multi):
        for k in (0, 1, 3, 4):
            x, y = a[k], b[k]
            assert _checksum(x) == _checksum(y), k
            kind = torch.int16 if x.element_size() == 2 else torch.int32
            assert torch.equal(x[-70_000:].view(kind), y[-70_000:].view(kind)) and torch.equal(x[:70_000].view(kind), y[:70_000].view(kind))
    del single, multi
    torch.cuda.empty_cache()


def _checksum(t, chunk=1 << 28):
    """Order-independent 64-bit checksum of a tensor's bit patterns."""
    view = t.view(torch.int32 if t.element_size() == 4 else torch.int16)
    total = 0
    for lo in range(0, view.numel(), chunk):
        total += int(view[lo:lo + chunk].to(torch.int64).sum().item())
    return total & ((1 << 64) - 1)


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_whole_model_flat_buffer_equals_tensor_list(flavour):
    """6,738,415,616 elements (a 7B-parameter model's state, 108 GB; 94 GB in the fp16 flavour): one launch over the
    flat buffers.  Seeded slices — the first and last elements, and a stretch across element 2^32 — are checked
    against the oracle bit for bit; then the identical inputs are stepped tensor by tensor (291 tensors of the
    Llama-7B shapes, one launch each) and every output buffer must have the same checksum."""
    fp16 = flavour == "fp16"
    dt16 = torch.float16 if fp16 else torch.bfloat16
    scale = 64.0 if fp16 else 1.0
    fn = F.adam_fp16 if fp16 else F.adam_bf16
    layer = [4096 * 4096] * 4 + [4096 * 11008] * 3 + [4096] * 2
    shapes = [32000 * 4096] + layer * 32 + [4096, 32000 * 4096]
    n = sum(shapes)
    assert n == 6_738_415_616 and len(shapes) == 291
    bufs = {"h": torch.empty(n, dtype=dt16, device="cuda"), "g": torch.empty(n, dtype=dt16, device="cuda"),
            "p": torch.empty(n, device="cuda"), "m": torch.empty(n, dtype=torch.float16 if fp16 else torch.float32, device="cuda"),
            "v": torch.empty(n, device="cuda")}

    def fill():
        gen = torch.Generator(device="cuda").manual_seed(4)
        _fill_(bufs["p"], 0.02, gen); _fill_(bufs["m"], 1e-4 * scale, gen); _fill_(bufs["v"], 1e-6 * scale, gen, absolute=True)
        _fill_(bufs["g"], 1e-3 * scale, gen)
        bufs["h"].zero_()

    fill()
    rnd = np.random.default_rng(4)
    starts = [0, n - 70000, (1 << 32) - 30000] + [int(s) for s in rnd.integers(0, n - 70000, 5)]
    slices = [(s, s + 65536 + 7) for s in starts]
    snap = {k: {s: bufs[k][s[0]:s[1]].clone() for s in slices} for k in ("p", "m", "v", "g")}
    fn(bufs["p"], bufs["h"], bufs["g"], bufs["m"], bufs["v"], 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 100)
    bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 100)
    for s in slices:
        po, vo = (snap[k][s].cpu().numpy().copy() for k in ("p", "v"))
        ho = np.zeros(s[1] - s[0], np.uint16)
        if fp16:
            mo = bits16(snap["m"][s])
            oracle.adam_gpu_fp16(po, ho, bits16(snap["g"][s]), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
            assert np.array_equal(bits16(bufs["m"][s[0]:s[1]]), mo), s
        else:
            mo = snap["m"][s].cpu().numpy().copy()
            oracle.adam_gpu_bf16(po, ho, bits16(snap["g"][s]), mo, vo, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
            assert np.array_equal(f32_bits(bufs["m"][s[0]:s[1]].cpu().numpy()), f32_bits(mo)), s
        assert np.array_equal(f32_bits(bufs["p"][s[0]:s[1]].cpu().numpy()), f32_bits(po)), s
        assert np.array_equal(f32_bits(bufs["v"][s[0]:s[1]].cpu().numpy()), f32_bits(vo)), s
        assert np.array_equal(bits16(bufs["h"][s[0]:s[1]]), ho), s
    flat = {k: _checksum(bufs[k]) for k in ("p", "m", "v", "h")}

    fill()
    lo = 0
    for size in shapes:
        hi = lo + size
        fn(bufs["p"][lo:hi], bufs["h"][lo:hi], bufs["g"][lo:hi], bufs["m"][lo:hi], bufs["v"][lo:hi],
           0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 100)
        lo = hi
    assert {k: _checksum(bufs[k]) for k in ("p", "m", "v", "h")} == flat
    del snap
    bufs.clear()
    torch.cuda.empty_cache()
