"""Fused cross-entropy on the GPU, through the C ABI, against the oracle.

Bars: loss <= 1e-3 relative to an fp32 reference (met with a wide margin: the test uses 2e-6);
stored softmax and gradients <= 1 ulp of the 16-bit type against the oracle's restatement of the
reference expressions.  The backward kernel alone is exact arithmetic on its 16-bit input, so
on identical input it must match the oracle bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from bmtrain_amd.loss import _function as F
from bmtrain_amd.loss import FusedCrossEntropy, OpFusedCrossEntropy
from conftest import bits16, from_bits16, ulp_distance16

pytestmark = pytest.mark.gpu
DTYPES = [("fp16", torch.float16), ("bf16", torch.bfloat16)]


def _case(m, n, dtype, seed, std=2.0, ignore_frac=0.1):
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, n, generator=gen) * std).to(dtype)
    t = torch.randint(0, n, (m,), generator=gen, dtype=torch.int32)
    t[torch.rand(m, generator=gen) < ignore_frac] = -100
    return x, t


def _forward_gpu(x, t, ignore=-100):
    xg, tg = x.cuda(), t.cuda()
    softmax = torch.empty_like(xg)
    out = torch.empty(x.size(0), dtype=torch.float32, device="cuda")
    F.cross_entropy_forward(x.size(0), x.size(1), xg, tg, softmax, out, ignore)
    return softmax, out


# every launch shape of the forward: one wave per row, 256 / 512 / 1024 lanes per row with 1..4 vectors per
# lane in registers, registers + LDS with and without a re-read part of any length; row lengths that
# are not multiples of 8 (rows then start at every 2-byte offset in turn) in each of them
WIDTHS = [1, 2, 3, 7, 8, 9, 10, 15, 16, 17, 90, 100, 512, 513, 520, 1000, 1001, 1024, 1500, 2048, 2056, 4096, 4097, 6100,
          8192, 8200, 10240, 12288, 12295, 16384, 20001, 30000, 32000, 32001, 32768, 32775, 49151, 50257, 50264, 65535,
          65536, 65544, 81920, 81928, 90001, 98304, 100000, 100003, 128256, 128257, 131072, 131079, 131080, 151936, 151937, 256000, 300001]


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("n", WIDTHS)
def test_forward_against_oracle(name, dtype, n):
    m = max(5, min(2000, 1_000_000 // n))          # about a million elements per case
    x, t = _case(m, n, dtype, seed=n)
    softmax, loss = _forward_gpu(x, t)
    want_soft, want_loss = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    assert ulp_distance16(bits16(softmax), want_soft).max() <= 1
    # rarely off by its one ulp: more often for fp16 values in the normal range, whose ulp is 2^-11 of the value,
    # than for bf16 (2^-8) or the subnormal fp16 values of long rows.  Measured over 3 M elements per width: fp16
    # 1.6e-4 to 2.5e-4 up to 512 classes, 1e-4 at 4,096, 4e-5 at 32,000, 1e-5 beyond 100,000; bf16 1e-5 to 6e-5 at
    # every width; two-class rows 5e-4 in both types.  The bounds leave a factor of 1.5 to 2 for the sample of about a
    # million elements (the differing elements of a row move together with its sum); the benchmark shapes have a test
    # of their own.
    if n <= 2:
        allowed = 1e-3
    elif name == "fp16":
        allowed = 4e-4 if n <= 8192 else 1.5e-4
    else:
        allowed = 1.5e-4
    # The differing elements of a row move together with its sum: when the sum lands on the other side of an fp32
    # rounding than the oracle's, the row's quotients that sit next to a 16-bit rounding boundary all flip.  Over 240
    # rows per width and type the worst single row differs on 1.4e-3 of its elements (bf16; fp16 4e-4) while the mean
    # stays at 1e-5 to 4e-5, so a sample of only nine long rows needs room for one such row on top of the rate.
    one_unlucky_row = (1.5e-3 if name == "bf16" else 5e-4) * n
    assert (bits16(softmax) != want_soft).sum() <= 3 + allowed * m * n + one_unlucky_row
    np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=2e-6, atol=2e-6)
    ref32 = torch.nn.functional.cross_entropy(x.float(), t.long(), ignore_index=-100, reduction="none").numpy()
    np.testing.assert_allclose(loss.cpu().numpy(), ref32, rtol=1e-3, atol=1e-6)
    assert np.all(loss.cpu().numpy()[t.numpy() == -100] == 0)


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 5, 7, 8, 9, 15, 100, 1000, 1001, 4096, 32000, 50001, 50257, 128256, 128257])
def test_backward_bit_exact_on_identical_input(name, dtype, n):
    m = 11
    x, t = _case(m, n, dtype, seed=n + 1)
    soft, _ = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    gen = torch.Generator().manual_seed(n)
    for upstream in (1.0, 32768.0, 2.0 ** 20):
        v = (torch.rand(m, generator=gen) * upstream / m).float()
        v[t == -100] = 0
        want = soft.copy()
        oracle.ce_backward_inplace(v.numpy(), t.numpy(), want, -100, name)
        xg = from_bits16(soft, dtype).reshape(m, n).cuda()
        F.cross_entropy_backward_inplace(m, n, v.cuda(), t.cuda(), xg, -100)
        assert np.array_equal(bits16(xg).reshape(m, n), want), upstream
    # an ignored row with a non-zero grad_output is scaled, not zeroed (cross_entropy.cu:46-60)
    v = torch.ones(m)
    want = soft.copy()
    oracle.ce_backward_inplace(v.numpy(), t.numpy(), want, -100, name)
    xg = from_bits16(soft, dtype).reshape(m, n).cuda()
    F.cross_entropy_backward_inplace(m, n, v.cuda(), t.cuda(), xg, -100)
    assert np.array_equal(bits16(xg).reshape(m, n), want)


def _value16(bits, dtype):
    return from_bits16(bits, dtype).double().numpy()


def _ulp_size16(bits, dtype):
    """Spacing of the 16-bit format at each value (subnormal spacing below the normal range)."""
    v = np.abs(_value16(bits, dtype))
    mant, emin = (10, -14) if dtype == torch.float16 else (7, -126)
    e = np.floor(np.log2(np.maximum(v, 2.0 ** emin)))
    return 2.0 ** (e - mant)


def check_gradient_end_to_end(got_soft, got_grad, want_soft, v, t, name, dtype):
    """The chain forward -> backward against the oracle's chain.

    1. backward is exact arithmetic on the stored softmax: the GPU gradient must equal the oracle's
       backward applied to the GPU's own stored softmax, bit for bit;
    2. hence the GPU gradient can differ from the oracle's end-to-end gradient only where the stored
       softmax differs (<= 1 ulp, rare), and there by no more than that one softmax step times
       |grad_output| plus the final rounding.  (An fp16 softmax of a 32,000-class row is mostly
       subnormal, so one step of it can be several ulps of the scaled-up gradient.)"""
    same_input = got_soft.copy()
    oracle.ce_backward_inplace(v, t, same_input, -100, name)
    assert np.array_equal(got_grad, same_input)
    end_to_end = want_soft.copy()
    oracle.ce_backward_inplace(v, t, end_to_end, -100, name)
    differs = got_grad != end_to_end
    assert not np.any(differs & (got_soft == want_soft))
    assert differs.mean() < 1e-3
    if differs.any():
        err = np.abs(_value16(got_grad, dtype) - _value16(end_to_end, dtype))
        bound = _ulp_size16(want_soft, dtype) * np.abs(v.astype(np.float64))[:, None] + _ulp_size16(end_to_end, dtype)
        assert np.all(err[differs] <= bound[differs])
    return differs.mean()


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("n", [1000, 32000, 128256])
def test_forward_backward_chain(name, dtype, n):
    """Gradients through both kernels vs the oracle through both restatements, at the upstream scales
    training uses (at 1.0 most fp16 gradients of a 16k-row mean are below the subnormal range)."""
    m = 9
    x, t = _case(m, n, dtype, seed=n + 2, ignore_frac=0.3)
    valid = (t != -100).float()
    want_soft, _ = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    for upstream in (1.0, 32768.0, 2.0 ** 20):
        v = (valid / valid.sum() * upstream / 1024).float()      # mean over a 1024x larger batch
        softmax, _ = _forward_gpu(x, t)
        got_soft = bits16(softmax)
        assert ulp_distance16(got_soft, want_soft).max() <= 1
        F.cross_entropy_backward_inplace(m, n, v.cuda(), t.cuda(), softmax, -100)
        got = bits16(softmax)
        check_gradient_end_to_end(got_soft, got, want_soft, v.numpy(), t.numpy(), name, dtype)
        assert np.all(got[t.numpy() == -100] == 0)


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("n", [64, 1000, 4096, 32000, 50264, 128256, 151936, 100003])   # one width per forward kernel
def test_special_rows(name, dtype, n):
    huge = 60000.0 if dtype == torch.float16 else 3e38
    rows = [
        torch.full((n,), float("-inf")),                 # M clamps to -1e6, S = 1e-10
        torch.full((n,), 0.5),                           # uniform
        torch.cat([torch.tensor([huge]), torch.zeros(n - 1)]),
        torch.cat([torch.tensor([float("nan")]), torch.ones(n - 1)]),
        torch.cat([torch.tensor([float("inf")]), torch.ones(n - 1)]),
        torch.linspace(-30, 30, n),
        torch.cat([torch.zeros(n - 3), torch.tensor([huge, -huge, huge])]),   # equal huge values: e^0 each
        torch.full((n,), -huge),                         # below the clamp: all exponentials 0
        torch.linspace(-200, 0, n),                      # results down to the subnormals of the 16-bit type
    ]
    x = torch.stack(rows).to(dtype)
    t = torch.tensor([0, 5, 0, 3, 0, n - 1, n - 1, 1, n - 2], dtype=torch.int32)
    softmax, loss = _forward_gpu(x, t)
    want_soft, want_loss = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    got = from_bits16(bits16(softmax), dtype).float().numpy()
    want = from_bits16(want_soft, dtype).float().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert ulp_distance16(bits16(softmax)[~np.isnan(got)], want_soft[~np.isnan(want)]).max() <= 1
    np.testing.assert_allclose(loss.cpu().numpy(), want_loss, rtol=2e-6, atol=1e-6, equal_nan=True)
    # out-of-range target that is not ignore_index: NaN loss instead of an out-of-bounds read
    _, loss = _forward_gpu(x[:2], torch.tensor([n, -7], dtype=torch.int32))
    assert torch.isnan(loss).all()


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("m,n", [(6, 1024), (5, 1001), (3, 50257), (2, 131075), (3, 20488), (4, 86583), (40, 5), (9, 8)])
def test_unaligned_bases(name, dtype, m, n):
    """Arrays that start at any 2-byte offset: logits and softmax at the same offset from a 128-byte line (long rows:
    vectors placed from each row's first line boundary), at the same offset from a 16-byte boundary only (vectors
    placed from the first 16-byte boundary) and at different ones (element loads); nothing outside is written."""
    x, t = _case(m, n, dtype, seed=n + m)
    want_soft, want_loss = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    buf = torch.zeros(m * n + 80, dtype=dtype, device="cuda")
    for off, soft_off in ((1, 1), (4, 4), (7, 7), (63, 63), (0, 64), (9, 73), (3, 11), (0, 8), (24, 40), (2, 5), (0, 1)):
        xg = buf[off:off + m * n].view(m, n)
        xg.copy_(x)
        soft_buf = torch.zeros(m * n + 80, dtype=dtype, device="cuda")
        soft = soft_buf[soft_off:soft_off + m * n].view(m, n)
        out = torch.empty(m, dtype=torch.float32, device="cuda")
        F.cross_entropy_forward(m, n, xg, t.cuda(), soft, out, -100)
        assert ulp_distance16(bits16(soft), want_soft).max() <= 1, (off, soft_off)
        np.testing.assert_allclose(out.cpu().numpy(), want_loss, rtol=2e-6, atol=2e-6)
        assert soft_buf[:soft_off].count_nonzero() == 0 and soft_buf[soft_off + m * n:].count_nonzero() == 0
        v = torch.rand(m)
        want = bits16(soft)
        oracle.ce_backward_inplace(v.numpy(), t.numpy(), want, -100, name)
        F.cross_entropy_backward_inplace(m, n, v.cuda(), t.cuda(), soft, -100)
        assert np.array_equal(bits16(soft), want), (off, soft_off)
        assert soft_buf[:soft_off].count_nonzero() == 0 and soft_buf[soft_off + m * n:].count_nonzero() == 0


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_sumexp_and_softmax_inplace(name, dtype):
    for m, n, off in ((5, 1000, 0), (3, 32000, 0), (4, 777, 0), (7, 50257, 3), (33, 5, 1), (2, 9, 7)):
        x, _ = _case(m, n, dtype, seed=n)
        xg = torch.zeros(m * n + 8, dtype=dtype, device="cuda")[off:off + m * n].view(m, n)
        xg.copy_(x)
        mx = xg.float().max(-1).values.contiguous()
        se = F.fused_sumexp(xg, mx)
        want_se = oracle.fused_sumexp(bits16(x), mx.cpu().numpy(), name)
        np.testing.assert_allclose(se.cpu().numpy(), want_se, rtol=2e-6)
        want = bits16(x)
        oracle.fused_softmax_inplace(want, mx.cpu().numpy(), want_se, name)
        F.fused_softmax_inplace(xg, mx, torch.from_numpy(want_se).cuda())
        assert ulp_distance16(bits16(xg), want).max() <= 1


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("m,n,off", [(4197, 32008, 0), (4200, 32001, 0), (4197, 32008, 3), (2700, 50257, 5), (1560, 86583, 0),
                                     (16800, 32001, 5)])      # 2^29 elements or more: the counters are taken in turn
def test_elementwise_kernels_on_a_large_array(name, dtype, m, n, off):
    """Arrays of 2^27 elements or more with rows of 8,192 or more run as a resident grid whose tiles (8,192
    elements) straddle rows and whose last tile is ragged: 4,197 rows of 32,008; and, with vectors that hold the end
    of one row and the start of the next and a few elements in front of the first vector and behind the last one, rows
    whose length is not a multiple of 8 (32,001; 50,257; 86,583) and arrays that start `off` elements behind a 16-byte
    boundary.  Backward is bit-exact on identical input, the in-place softmax within one unit in the last place; two
    launches on two streams at once use separate ticket counters; the words in front of and behind the array stay
    as they were."""
    assert m * n >= 1 << 27 and (m * n // 8) % 1024 != 0 and n % 8192 != 0
    from bmtrain_amd import C
    x, t = _case(m, n, dtype, seed=77)
    soft, _ = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    v = (torch.rand(m, generator=torch.Generator().manual_seed(5)) * 32768.0 / m).float()
    v[t == -100] = 0
    want = soft.copy()
    oracle.ce_backward_inplace(v.numpy(), t.numpy(), want, -100, name)
    guard = 4096
    side = torch.cuda.Stream()
    bufs = []
    for _ in range(2):
        buf = torch.full((off + m * n + guard,), 1.0, dtype=dtype, device="cuda")
        buf[off:off + m * n].view(m, n).copy_(from_bits16(soft, dtype).reshape(m, n))
        bufs.append(buf)
    vg, tg = v.cuda(), t.cuda()
    torch.cuda.synchronize()
    before = C.bmt_hip_flat_stream_stats()
    F.cross_entropy_backward_inplace(m, n, vg, tg, bufs[0][off:off + m * n].view(m, n), -100)
    with torch.cuda.stream(side):
        F.cross_entropy_backward_inplace(m, n, vg, tg, bufs[1][off:off + m * n].view(m, n), -100)
    torch.cuda.synchronize()
    assert C.bmt_hip_flat_stream_stats()["resident"] == before["resident"] + 2      # both ran as the resident grid
    for buf in bufs:
        assert np.array_equal(bits16(buf[off:off + m * n]).reshape(m, n), want)
        assert bool((buf[off + m * n:] == 1.0).all()) and bool((buf[:off] == 1.0).all())

    buf = bufs[0]
    xg = buf[off:off + m * n].view(m, n)
    xg.copy_(x)
    mx = xg.float().max(-1).values.contiguous()
    want_se = oracle.fused_sumexp(bits16(x), mx.cpu().numpy(), name)
    want = bits16(x)
    oracle.fused_softmax_inplace(want, mx.cpu().numpy(), want_se, name)
    F.fused_softmax_inplace(xg, mx, torch.from_numpy(want_se).cuda())
    assert ulp_distance16(bits16(xg), want).max() <= 1
    assert bool((buf[off + m * n:] == 1.0).all()) and bool((buf[:off] == 1.0).all())


def test_elementwise_kernels_on_more_streams_than_the_library_keeps_counters_for():
    """The resident grid keeps its ticket counters per stream, for up to 256 streams of a device; a launch on a further
    stream gets the table entry of a stream whose last launch has completed, or takes the kernel that needs no
    counters.  260 streams, one launch each, same bits everywhere."""
    m, n = 4197, 32008
    x, t = _case(m, n, torch.bfloat16, seed=78)
    soft, _ = oracle.ce_forward(bits16(x), t.numpy(), -100, "bf16")
    v = torch.full((m,), 1.0 / m)
    want = soft.copy()
    oracle.ce_backward_inplace(v.numpy(), t.numpy(), want, -100, "bf16")
    start = from_bits16(soft, torch.bfloat16).reshape(m, n).cuda()
    vg, tg = v.cuda(), t.cuda()
    work = torch.empty_like(start)
    # torch hands out streams from a pool of 32, so the streams are created through the runtime itself
    # (looked up through the library under test, so that it is the runtime instance the library and torch share)
    import ctypes
    from bmtrain_amd import C
    hip = C._lib
    hip.hipStreamCreate.argtypes, hip.hipStreamCreate.restype = [ctypes.POINTER(ctypes.c_void_p)], ctypes.c_int
    hip.hipStreamDestroy.argtypes, hip.hipStreamDestroy.restype = [ctypes.c_void_p], ctypes.c_int
    handles = []
    try:
        for _ in range(260):
            handle = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(handle)) == 0
            handles.append(handle)
        torch.cuda.synchronize()
        for i, handle in enumerate(handles):
            stream = torch.cuda.ExternalStream(handle.value)
            with torch.cuda.stream(stream):
                work.copy_(start, non_blocking=True)
                F.cross_entropy_backward_inplace(m, n, vg, tg, work, -100)
            stream.synchronize()
            if i in (0, 1, 254, 255, 256, 257, 259):
                assert np.array_equal(bits16(work).reshape(m, n), want), i
    finally:
        torch.cuda.synchronize()
        for handle in handles:
            hip.hipStreamDestroy(handle)


# ---- module level, shaped like the reference's tests/test_loss_func.py -----------------------
def _run(x, tgt, loss_func, scale=32768, use_float=False):
    x = x.clone().detach()
    if use_float:
        x = x.float()
    x = x.requires_grad_()
    loss = loss_func(x, tgt)
    (loss * scale).backward()
    return loss, x.grad


def _check(x, tgt, fused, plain):
    loss_1, grad_1 = _run(x, tgt, fused)
    loss_2, grad_2 = _run(x, tgt, plain, use_float=True)
    assert grad_1.isnan().sum() == 0 and grad_2.isnan().sum() == 0
    assert (loss_1 - loss_2).abs().item() < 1e-5          # tests/test_loss_func.py:31
    assert (grad_1 - grad_2).abs().max().item() < 1e-1    # tests/test_loss_func.py:32


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_module_against_torch_cross_entropy(dtype):
    torch.manual_seed(0)
    N = 32 * 512
    for C in [10, 50, 90, 100, 500, 900, 1000, 5000, 16000, 30000]:
        x = torch.randn(N, C).cuda().to(dtype)
        tgt = torch.randint(0, C, (N,)).cuda().long()
        _check(x, tgt, FusedCrossEntropy(), torch.nn.CrossEntropyLoss())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_module_with_class_weights_and_ignored_targets(dtype):
    torch.manual_seed(1)
    N = 32 * 512
    for C in (10, 50, 100):
        weight = (torch.randperm(C) + 1).cuda()
        x = torch.randn(N, C).cuda().to(dtype)
        tgt = torch.randint(0, C, (N,)).cuda().long()
        tgt[torch.randint(0, 2, (N,)).cuda().bool()] = -100
        _check(x, tgt, FusedCrossEntropy(weight=weight.clone().to(dtype)),
               torch.nn.CrossEntropyLoss(weight=weight.clone().float()))
        for reduction in ("none", "sum"):
            a = FusedCrossEntropy(reduction=reduction)(x, tgt)
            b = torch.nn.functional.cross_entropy(x.float(), tgt, reduction=reduction)
            torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-4 if reduction == "none" else 1.0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_reduction_against_the_torch_expressions(dtype):
    """FusedCrossEntropy reduces the per-row losses with one launch each way (OpLossReduce) where
    bmtrain/loss/cross_entropy.py:243-260 uses torch operations; with `fused_reduction = False` the module runs those
    operations.  Same rows, same targets: the loss agrees to 1e-6 relative (only the order of the additions differs, torch adds in fp32;
    the fused sums are checked against float64 arithmetic below), the logits' gradient is bit-identical - except under
    `mean` with class weights, where the divisor is a rounded sum of weights that may differ in its last bit and the
    gradient then differs by one step of the 16-bit type on a few elements - for sum and mean, with and without class
    weights (fp32 and 16-bit), with no, some and all rows ignored, for row counts around the kernel's strides, and with
    an upstream factor as a loss scale gives."""
    torch.manual_seed(11)
    for m, C in ((1, 17), (7, 100), (1000, 257), (1023, 64), (1025, 64), (4097, 1000), (16384, 512)):
        x = (torch.randn(m, C, device="cuda") * 2).to(dtype)
        for ignored in ("none", "some", "all"):
            tgt = torch.randint(0, C, (m,), device="cuda")
            if ignored == "some":
                tgt[torch.rand(m, device="cuda") < 0.3] = -100
            elif ignored == "all":
                tgt[:] = -100
            for weight in (None, torch.rand(C, device="cuda") + 0.5, (torch.rand(C, device="cuda") + 0.5).to(dtype)):
                for reduction in ("mean", "sum"):
                    for scale in (1.0, 32768.0):
                        results = []
                        for fused in (True, False):
                            module = FusedCrossEntropy(weight=weight, reduction=reduction)
                            module.fused_reduction = fused
                            xi = x.clone().requires_grad_()
                            loss = module(xi, tgt)
                            (loss * scale).backward()
                            results.append((loss.detach(), xi.grad))
                        (la, ga), (lb, gb) = results
                        assert la.dtype == lb.dtype == torch.float32 and la.shape == lb.shape == ()
                        case = (m, C, ignored, None if weight is None else weight.dtype, reduction, scale)
                        if ignored == "all" and reduction == "mean":
                            assert torch.isnan(la) and torch.isnan(lb), case          # 0 / 0, as in the reference
                            assert torch.isnan(ga).all() and torch.isnan(gb).all(), case
                            continue
                        assert abs(la.item() - lb.item()) <= 1e-6 * abs(lb.item()) + 1e-30, case
                        if weight is not None and reduction == "mean":
                            # the divisor is itself a rounded sum of weights here: it may differ in its last bit
                            steps = (ga.view(torch.int16).int() - gb.view(torch.int16).int()).abs()
                            assert steps.max().item() <= 1 and (steps > 0).float().mean().item() < 0.02, case
                        else:
                            assert torch.equal(ga.view(torch.int16), gb.view(torch.int16)), case
    # the launchers by themselves against float64 arithmetic, also beyond the 4 x 1024 rows of one pass of the loop
    from bmtrain_amd.loss import _function as LF
    for m in (0, 1, 4095, 4096, 4097, 100_000):
        losses = torch.rand(m, device="cuda") * 12
        tgt = torch.randint(0, 50, (m,), device="cuda", dtype=torch.int32)
        tgt[::7] = -1
        weight = torch.rand(50, device="cuda") + 0.1
        for w in (None, weight):
            for mean in (False, True):
                result, wsum = torch.empty((), device="cuda"), torch.empty((), device="cuda")
                LF.loss_reduce_forward(losses, tgt, w, 50, -1, mean, result, wsum)
                wr = ((tgt != -1).float() if w is None else torch.where(tgt != -1, weight[tgt.clamp(min=0).long()], 0.0))
                exact_s = (wr * losses).double().sum().item()
                exact_w = wr.double().sum().item()
                assert abs(wsum.item() - exact_w) <= 6e-8 * exact_w
                if exact_w == 0 and mean:            # no row counts: 0 / 0, as in the reference
                    assert torch.isnan(result)
                    continue
                want = exact_s / exact_w if mean else exact_s
                assert abs(result.item() - want) <= 2e-7 * abs(want), (m, mean)
                up = torch.full((), 3.0, device="cuda")
                rows = torch.empty(m, device="cuda")
                LF.loss_reduce_backward(tgt, w, 50, -1, mean, wsum, up, rows)
                assert torch.equal(rows, (up / wsum if mean else up) * wr)
    # a class outside the weight table weighs nothing instead of being read
    tgt = torch.tensor([3, 50, -7, 2], device="cuda", dtype=torch.int32)
    result, wsum = torch.empty((), device="cuda"), torch.empty((), device="cuda")
    LF.loss_reduce_forward(torch.ones(4, device="cuda"), tgt, weight, 50, -100, False, result, wsum)
    assert wsum.item() == (weight[3] + weight[2]).item()


def test_module_contract():
    x = torch.randn(8, 16, device="cuda")
    tgt = torch.randint(0, 16, (8,), device="cuda")
    # fp32 input is torch's own cross entropy, label smoothing included
    a = FusedCrossEntropy(label_smoothing=0.1)(x, tgt)
    b = torch.nn.functional.cross_entropy(x, tgt, label_smoothing=0.1)
    assert torch.equal(a, b)
    with pytest.raises(ValueError):
        FusedCrossEntropy(weight=torch.ones(3, device="cuda"))(x.half(), tgt)
    with pytest.raises(AssertionError):
        OpFusedCrossEntropy.apply(x.half()[0], tgt.int(), -100)
    import bmtrain_amd
    bmtrain_amd.config["tp_size"] = 2
    try:
        with pytest.raises(NotImplementedError):
            FusedCrossEntropy(parallel=True)(x.half(), tgt)
    finally:
        del bmtrain_amd.config["tp_size"]
    # backward hands back the softmax buffer itself as the gradient
    xh = x.half().requires_grad_()
    out = OpFusedCrossEntropy.apply(xh, tgt.int(), -100)
    out.sum().backward()
    assert xh.grad.dtype == torch.float16 and xh.grad.shape == xh.shape
    # all targets ignored: 0 / 0
    assert torch.isnan(FusedCrossEntropy()(x.half(), torch.full((8,), -100, device="cuda")))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_vocab_parallel_loss_with_one_rank(dtype):
    """bmtrain/loss/cross_entropy.py:38-106 with a tensor-parallel group of one: same loss and
    gradient as the fused non-parallel path and as torch in fp32 (ignored targets included)."""
    torch.manual_seed(7)
    N, C = 4096, 8000
    x = torch.randn(N, C).cuda().to(dtype)
    tgt = torch.randint(0, C, (N,)).cuda().long()
    tgt[::7] = -100
    vp, fused, plain = FusedCrossEntropy(parallel=True), FusedCrossEntropy(), torch.nn.CrossEntropyLoss()
    loss_v, grad_v = _run(x, tgt, vp)
    loss_f, grad_f = _run(x, tgt, fused)
    loss_p, grad_p = _run(x, tgt, plain, use_float=True)
    assert (loss_v - loss_p).abs().item() < 1e-5 and (loss_v - loss_f).abs().item() < 1e-5
    assert (grad_v.float() - grad_p).abs().max().item() < 1e-1
    assert grad_v[tgt == -100].count_nonzero() == 0
    ulp = 2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7
    assert ((grad_v.float() - grad_f.float()).abs() <= ulp * grad_f.float().abs() + 1e-3).all()


LM_HEADS = [(16384, 32000, "fp16", torch.float16, 2.0, 10, 3), (8192, 128256, "bf16", torch.bfloat16, 3.0, 20, 4)]


def _lm_head_case(m, n, dtype, std, every, seed):
    """The benchmark inputs: logits ~ N(0, std) rounded to the 16-bit type, uniform targets, one row in `every`
    ignored (seeded permutation)."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.empty(m, n, dtype=dtype, device="cuda")
    for lo in range(0, m, 1024):
        x[lo:lo + 1024] = (torch.randn(1024, n, generator=gen, device="cuda") * std).to(dtype)
    t = torch.randint(0, n, (m,), generator=gen, device="cuda", dtype=torch.int32)
    t[torch.randperm(m, generator=gen, device="cuda")[: m // every]] = -100
    return x, t


@pytest.mark.parametrize("m,n,name,dtype,std,every,seed", LM_HEADS)
def test_language_model_head_shape(m, n, name, dtype, std, every, seed):
    """16,384 rows x 32,000 classes fp16 (logits N(0,2), 10 % ignored) and 8,192 rows x 128,256 classes bf16
    (N(0,3), 5 % ignored), mean reduction.  Seeded rows are checked against the oracle; all rows are checked
    through row sums, the loss against torch in fp32 on the GPU, and sign / zero structure of the gradient."""
    x, t = _lm_head_case(m, n, dtype, std, every, seed)
    softmax = torch.empty_like(x)
    out = torch.empty(m, dtype=torch.float32, device="cuda")
    F.cross_entropy_forward(m, n, x, t, softmax, out, -100)
    rows = [0, 1, m - 1] + [int(r) for r in np.random.default_rng(3).integers(0, m, 13)]
    idx = torch.tensor(rows, device="cuda")
    want_soft, want_loss = oracle.ce_forward(bits16(x[idx]), t[idx].cpu().numpy(), -100, name)
    assert ulp_distance16(bits16(softmax[idx]), want_soft).max() <= 1
    np.testing.assert_allclose(out[idx].cpu().numpy(), want_loss, rtol=2e-6, atol=2e-6)
    sums = torch.zeros(m, device="cuda")
    ref = torch.zeros(m, device="cuda")
    for lo in range(0, m, 2048):
        sums[lo:lo + 2048] = softmax[lo:lo + 2048].float().sum(-1)
        ref[lo:lo + 2048] = torch.nn.functional.cross_entropy(x[lo:lo + 2048].float(), t[lo:lo + 2048].long(),
                                                              ignore_index=-100, reduction="none")
    assert (sums - 1).abs().max().item() < 2e-2            # 16-bit rounding of n tiny terms
    torch.testing.assert_close(out, ref, rtol=1e-3, atol=1e-5)
    valid = (t != -100)
    scale = 2.0 ** 20
    v = (valid.float() / valid.sum() * scale)
    got_soft = bits16(softmax[idx])
    F.cross_entropy_backward_inplace(m, n, v, t, softmax, -100)
    assert softmax[~valid].count_nonzero() == 0
    check_gradient_end_to_end(got_soft, bits16(softmax[idx]), want_soft, v[idx].cpu().numpy(), t[idx].cpu().numpy(),
                              name, dtype)
    tv = t[valid].long()
    at_target = softmax[valid].gather(1, tv[:, None])
    assert (at_target < 0).all()
    del x, softmax
    torch.cuda.empty_cache()


@pytest.mark.parametrize("m,n,name,dtype,std,every,seed", LM_HEADS)
def test_gradient_parity_at_the_benchmark_shapes(m, n, name, dtype, std, every, seed, capsys):
    """How far the two kernels are from the oracle's chain (libm expf, IEEE division, two roundings to 16 bits) on
    the benchmark inputs, in units of the types involved, at upstream scales 1, 32768 and 2^20.  The kernels run on
    the full shape; a seeded sample of rows (24 M elements) is compared.

    Stored softmax: never more than 1 ulp off, and different on fewer than 1 element in 10,000.
    Gradient, in ulps of the gradient's own 16-bit value: identical wherever the stored softmax is; bf16: never
    more than 1 ulp off.  fp16 at 32,000 classes: the stored softmax is mostly *subnormal* (p ~ 3e-5 < 6.1e-5), so
    one step of it is 2^-24 whatever the value, while the gradient p * grad_output * scale is a normal number whose
    ulp can be far smaller than 2^-24 * grad_output * scale: a softmax off by its one ulp can be several gradient
    ulps off (the same holds between any two evaluations of the reference's expression with different expf
    implementations).  Those elements are bounded by that one softmax step, and counted."""
    x, t = _lm_head_case(m, n, dtype, std, every, seed)
    sample = 768 if n == 32000 else 192
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(seed))[:sample].sort().values.cuda()
    softmax = torch.empty_like(x)
    out = torch.empty(m, dtype=torch.float32, device="cuda")
    F.cross_entropy_forward(m, n, x, t, softmax, out, -100)
    ts = t[rows].cpu().numpy()
    want_soft, want_loss = oracle.ce_forward(bits16(x[rows]), ts, -100, name)
    want_soft = want_soft.reshape(sample, n)
    got_soft = bits16(softmax[rows]).reshape(sample, n)
    dist = ulp_distance16(got_soft, want_soft)
    report = [f"{name} {m}x{n}: stored softmax differs on {np.mean(dist != 0):.2e} of {dist.size} elements, max {dist.max()} ulp"]
    assert dist.max() <= 1 and np.mean(dist != 0) < 1e-4
    np.testing.assert_allclose(out[rows].cpu().numpy(), want_loss, rtol=2e-6, atol=2e-6)
    valid = (t != -100).float()
    for upstream in (1.0, 32768.0, 2.0 ** 20):
        v = (valid / valid.sum() * upstream).contiguous()
        grad = softmax.clone()
        F.cross_entropy_backward_inplace(m, n, v, t, grad, -100)
        got = bits16(grad[rows]).reshape(sample, n)
        del grad
        vs = v[rows].cpu().numpy()
        want = np.ascontiguousarray(want_soft.copy())
        oracle.ce_backward_inplace(vs, ts, want, -100, name)
        same_input = np.ascontiguousarray(got_soft.copy())
        oracle.ce_backward_inplace(vs, ts, same_input, -100, name)
        assert np.array_equal(got, same_input)                       # the backward kernel itself is exact
        err = np.abs(_value16(got.reshape(-1), dtype) - _value16(want.reshape(-1), dtype))
        ulps = (err / _ulp_size16(want.reshape(-1), dtype)).reshape(sample, n)
        assert not np.any((ulps != 0) & (dist == 0))                 # differences only where the softmax differs
        report.append(f"  grad_output scale {upstream:g}: gradient differs on {np.mean(ulps != 0):.2e}, by more than 1 ulp on "
                      f"{np.mean(ulps > 1):.2e}, max {ulps.max():.0f} ulp")
        assert np.mean(ulps != 0) < 1e-4
        if dtype == torch.bfloat16:
            assert ulps.max() <= 1
        else:
            assert np.mean(ulps > 1) < 5e-5
            step = _ulp_size16(want_soft.reshape(-1), dtype).reshape(sample, n) * np.abs(vs.astype(np.float64))[:, None]
            bound = step + _ulp_size16(want.reshape(-1), dtype).reshape(sample, n)
            assert np.all(err.reshape(sample, n) <= bound)
    with capsys.disabled():
        print("\n" + "\n".join(report))
    del x, softmax
    torch.cuda.empty_cache()


def test_more_than_2_to_the_31_logits():
    """20,000 rows x 128,257 classes (2.57e9 elements, odd row length): rows whose element offsets lie beyond
    2^31 and 2^32 bytes are checked against the oracle, forward and backward."""
    m, n = 20000, 128257
    gen = torch.Generator(device="cuda").manual_seed(11)
    x = torch.empty(m, n, dtype=torch.bfloat16, device="cuda")
    for lo in range(0, m, 2000):
        x[lo:lo + 2000] = (torch.randn(2000, n, generator=gen, device="cuda") * 2).bfloat16()
    t = torch.randint(0, n, (m,), generator=gen, device="cuda", dtype=torch.int32)
    softmax = torch.empty_like(x)
    out = torch.empty(m, dtype=torch.float32, device="cuda")
    F.cross_entropy_forward(m, n, x, t, softmax, out, -100)
    rows = [0, 1, 8371, 8372, 16743, 16744, 16745, m - 2, m - 1]       # near 2^30 and 2^31 elements, and the end
    idx = torch.tensor(rows, device="cuda")
    want_soft, want_loss = oracle.ce_forward(bits16(x[idx]), t[idx].cpu().numpy(), -100, "bf16")
    assert ulp_distance16(bits16(softmax[idx]), want_soft).max() <= 1
    np.testing.assert_allclose(out[idx].cpu().numpy(), want_loss, rtol=2e-6, atol=2e-6)
    assert torch.isfinite(out).all()
    v = torch.rand(m, generator=gen, device="cuda")
    want = bits16(softmax[idx])
    oracle.ce_backward_inplace(v[idx].cpu().numpy(), t[idx].cpu().numpy(), want, -100, "bf16")
    F.cross_entropy_backward_inplace(m, n, v, t, softmax, -100)
    assert np.array_equal(bits16(softmax[idx]), want)
    del x, softmax
    torch.cuda.empty_cache()
