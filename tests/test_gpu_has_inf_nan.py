"""has_inf_nan on the GPU, through the C ABI, against the oracle: bit-exact 0/1."""
import random

import numpy as np
import pytest
import torch

import oracle
from bmtrain_amd.loss import _function as F
from bmtrain_amd import C
from conftest import bits16, from_bits16

pytestmark = pytest.mark.gpu
DTYPES = [("fp16", torch.float16), ("bf16", torch.bfloat16)]


def gpu_flag(x, start=0):
    out = torch.full((1,), start, dtype=torch.uint8, device="cuda")[0]
    F.has_inf_nan(x, out)
    return int(out.item())


def oracle_flag(x, name, start=0):
    out = np.array([start], np.uint8)
    oracle.has_inf_nan(bits16(x), out, name)
    return int(out[0])


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_every_bit_pattern(name, dtype):
    """One launch per pattern, each on a one-element tensor, each with its own flag byte."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = from_bits16(bits, dtype).cuda()
    flags = torch.zeros(65536, dtype=torch.uint8, device="cuda")
    launcher = C.has_nan_inf_fp16_launcher if name == "fp16" else C.has_nan_inf_bf16_launcher
    stream = torch.cuda.current_stream().cuda_stream
    for i in range(65536):
        launcher(1, x.data_ptr() + 2 * i, 0, flags.data_ptr() + i, stream)
    got = flags.cpu().numpy()
    want = np.zeros(65536, np.uint8)
    for i in range(65536):
        oracle.has_inf_nan(bits[i:i + 1], want[i:i + 1], name)
    assert np.array_equal(got, want)
    # and all the finite patterns together raise nothing
    finite = from_bits16(bits[want == 0], dtype).cuda()
    assert gpu_flag(finite) == 0


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_reference_style_sweep(name, dtype):
    rnd = random.Random(1)
    torch.manual_seed(1)
    for n in list(range(1, 100)) + [1000] * 3 + [10000] * 3 + [100000] * 3 + [1000000] * 3:
        x = torch.rand(n).to(dtype).cuda()
        assert gpu_flag(x) == 0 == oracle_flag(x, name)
        p = rnd.randint(0, n - 1)
        x[p] = float("inf")
        assert gpu_flag(x) == 1 == oracle_flag(x, name)
        x[p] = 2
        assert gpu_flag(x) == 0
        x[rnd.randint(0, n - 1)] = float("nan")
        assert gpu_flag(x) == 1
        x[rnd.randint(0, n - 1)] = float("-inf")
        x[rnd.randint(0, n - 1)] = float("inf")
        assert gpu_flag(x) == 1 == oracle_flag(x, name)


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_unaligned_views_see_exactly_their_elements(name, dtype):
    """A hit just outside the view must not count; a hit on its first or last element must."""
    base = torch.ones(4096 + 64, dtype=dtype, device="cuda")
    for off in range(0, 17):
        for n in (1, 2, 7, 8, 9, 15, 16, 17, 255, 1024, 4000):
            view = base[off:off + n]
            base.fill_(1)
            if off > 0:
                base[off - 1] = float("inf")
            base[off + n] = float("nan")
            assert gpu_flag(view) == 0, (off, n)
            base[off] = float("inf")
            assert gpu_flag(view) == 1, (off, n)
            base[off] = 1
            base[off + n - 1] = float("nan")
            assert gpu_flag(view) == 1, (off, n)


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_sticky_flag_and_empty_input(name, dtype):
    x = torch.ones(1000, dtype=dtype, device="cuda")
    assert gpu_flag(x, start=1) == 1           # never cleared
    assert gpu_flag(x[:0], start=0) == 0       # n == 0 is a no-op
    flag = torch.zeros(1, dtype=torch.uint8, device="cuda")[0]
    bad = x.clone(); bad[123] = float("nan")
    for t in (x, bad, x, x):                   # accumulated over tensors, as check_overflow does
        F.has_inf_nan(t, flag)
    assert flag.item() == 1


def test_dtype_and_layout_errors():
    out = torch.zeros(1, dtype=torch.uint8, device="cuda")[0]
    with pytest.raises(ValueError):
        F.has_inf_nan(torch.ones(4, device="cuda"), out)
    with pytest.raises(AssertionError):
        F.has_inf_nan(torch.ones(4, dtype=torch.float16), out)
    with pytest.raises(AssertionError):
        F.has_inf_nan(torch.ones(8, dtype=torch.float16, device="cuda")[::2], out)
    with pytest.raises(AssertionError):
        F.has_inf_nan(torch.ones(4, dtype=torch.float16, device="cuda"), torch.zeros(1, device="cuda"))


def _fill_normal_(x, std, seed, chunk=1 << 28):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    for lo in range(0, x.numel(), chunk):
        part = x[lo:lo + chunk]
        part.copy_(torch.randn(part.numel(), generator=gen, device="cuda", dtype=torch.float32).mul_(std))


@pytest.mark.parametrize("name,dtype,n", [("bf16", torch.bfloat16, 6_738_415_616), ("fp16", torch.float16, 1 << 30)])
def test_full_size_buffers(name, dtype, n):
    """The gradient-buffer sizes of a 7B-parameter model: all finite -> 0; one +inf and one NaN
    at seeded offsets (beyond 2^32 bytes for bf16) -> 1; each alone -> 1."""
    x = torch.empty(n, dtype=dtype, device="cuda")
    _fill_normal_(x, 1e-3, seed=2)
    assert gpu_flag(x) == 0
    rnd = random.Random(2)
    a, b = rnd.randrange(n), rnd.randrange(n)
    keep_a, keep_b = x[a].clone(), x[b].clone()
    x[a] = float("inf")
    assert gpu_flag(x) == 1
    x[b] = float("nan")
    assert gpu_flag(x) == 1
    x[a] = keep_a
    assert gpu_flag(x) == 1
    x[b] = keep_b
    assert gpu_flag(x) == 0
    x[n - 1] = float("-inf")                    # very last element
    assert gpu_flag(x) == 1
    # a strided sample agrees with the oracle
    sample = x[:: max(1, n // (1 << 20))].contiguous()
    assert gpu_flag(sample) == oracle_flag(sample, name)
    if name == "bf16":
        # the same buffer handed over as the 291 gradient tensors of the model (five launches of up to 64 tensors):
        # the flag follows an inf / NaN at the seeded offsets, in a 4,096-element tensor and in the last element; the sum
        # of squares equals the single-buffer pass to 1e-8 (the tiles, and so the fp32 partial sums, start elsewhere)
        from bmtrain_amd.optim import _function as OF
        x[n - 1] = keep_last = 0.0
        layer = [4096 * 4096] * 4 + [11008 * 4096] * 3 + [4096] * 2
        sizes = [32000 * 4096] + layer * 32 + [4096, 32000 * 4096]
        assert sum(sizes) == n
        pieces, lo = [], 0
        for size in sizes:
            pieces.append(x[lo:lo + size])
            lo += size
        flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
        whole, listed = torch.zeros(1, dtype=torch.float64, device="cuda"), torch.zeros(1, dtype=torch.float64, device="cuda")
        OF.grad_stats(x, whole, flag)
        OF.grad_stats_multi(pieces, listed, flag)
        OF.grad_stats_multi(pieces, None, flag)
        assert flag.item() == 0
        assert abs(whole.item() - listed.item()) <= 1e-8 * whole.item() and whole.item() > 0
        small = next(k for k, size in enumerate(sizes) if size == 4096)
        for piece, at in ((None, a), (None, b), (pieces[small], 4095), (pieces[-1], sizes[-1] - 1), (pieces[0], 0)):
            target = x if piece is None else piece
            keep = target[at].clone()
            for bad in (float("inf"), float("nan")):
                target[at] = bad
                for with_sum in (False, True):
                    flag.zero_()
                    OF.grad_stats_multi(pieces, torch.zeros(1, dtype=torch.float64, device="cuda") if with_sum else None, flag)
                    assert flag.item() == 1, (at, bad, with_sum)
            target[at] = keep
        flag.zero_()
        OF.grad_stats_multi(pieces, None, flag)
        assert flag.item() == 0
    del x
    torch.cuda.empty_cache()


# ---- gradient statistics: overflow flag + sum of squares in one pass --------------------------
def _stats(x, sumsq_start=0.0, flag_start=0):
    from bmtrain_amd.optim import _function as OF
    sumsq = torch.full((1,), sumsq_start, dtype=torch.float64, device="cuda")
    flag = torch.full((1,), flag_start, dtype=torch.uint8, device="cuda")
    OF.grad_stats(x, sumsq, flag)
    return sumsq.item(), int(flag.item())


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_grad_stats_against_oracle(name, dtype):
    gen = torch.Generator().manual_seed(5)
    base = torch.zeros(3_000_064, dtype=dtype, device="cuda")
    for n in (1, 2, 7, 8, 9, 1000, 16384, 16385, 100003, 3_000_000):
        for off in (0, 1, 5):
            x = (torch.randn(n, generator=gen) * 2).to(dtype)
            view = base[off:off + n]
            view.copy_(x)
            got, flag = _stats(view)
            want = oracle.grad_sumsq(bits16(x), name)
            assert flag == 0 and abs(got - want) <= 1e-6 * want, (n, off, got, want)
            # identical input, identical bits; accumulation into a running total
            again, _ = _stats(view)
            assert again == got
            total, _ = _stats(view, sumsq_start=10.0)
            assert abs(total - (10.0 + got)) <= 1e-9 * (10.0 + got)
    x = torch.ones(5000, dtype=dtype, device="cuda")
    assert _stats(x) == (5000.0, 0)
    x[4321] = float("inf")
    s, flag = _stats(x)
    assert flag == 1 and s == float("inf")
    assert _stats(torch.ones(10, dtype=dtype, device="cuda"), flag_start=1)[1] == 1      # sticky
    assert _stats(x[:0], sumsq_start=2.5) == (2.5, 0)                                    # empty: no-op


@pytest.mark.parametrize("name,dtype", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_grad_stats_counts_tiny_gradients(name, dtype):
    """Subnormal fp16 gradients (unscaled gradients below 6e-5 are) must enter the sum of squares, and so
    must the smallest normal values of either type, alone and mixed with ordinary values."""
    gen = torch.Generator().manual_seed(6)
    n = 200_003
    if dtype == torch.float16:
        tiny = from_bits16(torch.randint(1, 0x0400, (n,), generator=gen).numpy().astype(np.uint16), dtype)   # all subnormal
    else:
        tiny = (torch.randn(n, generator=gen) * 1e-18).to(dtype)     # squares near the bottom of fp32's normal range
    for x in (tiny, torch.where(torch.arange(n) % 3 == 0, (torch.randn(n, generator=gen) * 1e-3).to(dtype), tiny)):
        got, flag = _stats(x.cuda())
        want = oracle.grad_sumsq(bits16(x), name)
        assert want > 0 and flag == 0 and abs(got - want) <= 1e-6 * want, (got, want)


def test_clip_grad_norm_uses_one_pass_and_matches_torch():
    import bmtrain_amd as bmt
    torch.manual_seed(9)
    ps = [torch.nn.Parameter(torch.randn(s, device="cuda").to(d))
          for s, d in ((100003, torch.bfloat16), (4096, torch.bfloat16), (77, torch.float16), (50, torch.float32))]
    manager = bmt.optim.OptimManager(loss_scale=64)
    for p in ps:
        p.grad = (torch.randn_like(p.float()) * 64).to(p.dtype)
    want = torch.cat([p.grad.float().flatten() for p in ps]).norm() / 64
    before = [p.grad.clone() for p in ps]
    got = manager.clip_grad_norm([{"params": ps}], max_norm=1.0)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=0)
    coef = 64.0 / (want * 64 + 1e-6)
    for p, b in zip(ps, before):
        torch.testing.assert_close(p.grad.float(), (b.float() * coef).to(p.dtype).float(), rtol=2e-2, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_several_tensors_in_one_launch(dtype):
    """grad_stats_multi_launcher: the overflow scan and the scan with the sum of squares over 150 tensors of 1 to
    1.3 M elements at every 2-byte alignment (three launches of up to 64 tensors).  The flag equals the tensor-by-tensor
    scan for a clean set and for an inf / NaN planted in turn in the first element, the last element, the unaligned
    head and tail and the middle of several tensors; the sum of squares equals float64 arithmetic to 1e-6 and is the
    same bits run after run."""
    from bmtrain_amd.optim import _function as OF
    from bmtrain_amd.loss import _function as LF
    rnd = np.random.default_rng(5)
    sizes = [1, 2, 7, 8, 9, 15, 16, 17, 1023, 8192, 8193, 65536 + 3] + [int(x) for x in rnd.integers(1, 1_300_000, 138)]
    pool = torch.empty(sum(sizes) + 16 * len(sizes), dtype=dtype, device="cuda").normal_(0, 2.0)
    grads, at = [], 0
    for k, n in enumerate(sizes):
        at += k % 8                                   # every 2-byte phase of a 16-byte vector
        grads.append(pool[at:at + n])
        at += n + (8 - at % 8) % 8 + 8
    flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
    OF.grad_stats_multi(grads, None, flag)
    assert flag.item() == 0
    sums = []
    for _ in range(2):
        sumsq = torch.zeros(1, dtype=torch.float64, device="cuda")
        OF.grad_stats_multi(grads, sumsq, flag)
        sums.append(sumsq.view(torch.int64).item())
        assert flag.item() == 0
    assert sums[0] == sums[1]
    exact = sum(g.double().pow(2).sum().item() for g in grads)
    assert abs(torch.tensor(sums[0]).view(torch.float64).item() - exact) <= 1e-6 * exact
    for k, where in ((0, 0), (3, -1), (11, 2), (11, -3), (40, 5), (70, -1), (149, 0), (100, None)):
        g = grads[k]
        i = g.numel() // 2 if where is None else (where if where >= 0 else g.numel() + where)
        i = min(max(i, 0), g.numel() - 1)
        keep = g[i].item()
        for bad in (float("inf"), float("nan")):
            g[i] = bad
            for with_sum in (False, True):
                flag.zero_()
                OF.grad_stats_multi(grads, torch.zeros(1, dtype=torch.float64, device="cuda") if with_sum else None, flag)
                single = torch.zeros(1, dtype=torch.uint8, device="cuda")
                for t in grads:
                    LF.has_inf_nan(t, single)
                assert flag.item() == single.item() == 1, (k, i, bad, with_sum)
        g[i] = keep
    flag.zero_()
    OF.grad_stats_multi(grads, None, flag)
    assert flag.item() == 0
    # nothing is launched for a table with a bad entry
    from bmtrain_amd import C
    with pytest.raises(RuntimeError, match="null pointer"):
        C.grad_stats_multi_launcher([(grads[0].data_ptr(), 8), (0, 8)], 1, 0, flag.data_ptr(), 0, 0)
