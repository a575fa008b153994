"""The launchers are asynchronous on the caller's stream, allocate nothing and synchronise nothing, so a
whole step can run on a side stream or be captured into a HIP graph and replayed."""
import numpy as np
import pytest
import torch

import oracle
from bmtrain_amd.loss import _function as LF
from bmtrain_amd.optim import _function as OF
from conftest import bits16, f32_bits

pytestmark = pytest.mark.gpu


def _state(n, seed, device="cuda"):
    gen = torch.Generator().manual_seed(seed)
    p = (torch.randn(n, generator=gen) * 0.02).to(device)
    m = (torch.randn(n, generator=gen) * 1e-4).to(device)
    v = (torch.randn(n, generator=gen) * 1e-6).abs().to(device)
    g = (torch.randn(n, generator=gen) * 1e-3).bfloat16().to(device)
    return p, torch.zeros(n, dtype=torch.bfloat16, device=device), g, m, v


def _step(p, h, g, m, v, flag, x, t, soft, loss, go, step):
    LF.has_inf_nan(g, flag)
    OF.adam_bf16(p, h, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, step)
    LF.cross_entropy_forward(x.size(0), x.size(1), x, t, soft, loss, -100)
    LF.cross_entropy_backward_inplace(x.size(0), x.size(1), go, t, soft, -100)


def _ce_inputs(rows, classes, seed):
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, classes, generator=gen) * 2).bfloat16().cuda()
    t = torch.randint(0, classes, (rows,), generator=gen, dtype=torch.int32).cuda()
    return x, t, torch.empty_like(x), torch.empty(rows, device="cuda"), torch.full((rows,), 1.0 / rows, device="cuda")


@pytest.mark.parametrize("n", [100_003, (1 << 25) + 5])       # below and above the size where Adam tiles go by ticket
def test_step_on_a_side_stream_equals_the_default_stream(n):
    a, b = _state(n, 1), _state(n, 1)
    ce_a, ce_b = _ce_inputs(64, 50257, 2), _ce_inputs(64, 50257, 2)
    flag_a, flag_b = (torch.zeros(1, dtype=torch.uint8, device="cuda")[0] for _ in range(2))
    _step(*a, flag_a, *ce_a, 3)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _step(*b, flag_b, *ce_b, 3)
    side.synchronize()
    torch.cuda.synchronize()
    for x, y in zip(a + ce_a, b + ce_b):
        assert torch.equal(x.view(torch.uint8), y.view(torch.uint8))
    assert flag_a.item() == flag_b.item() == 0


@pytest.mark.parametrize("n", [100_003, (1 << 25) + 5])
def test_step_captured_in_a_graph_replays_like_eager(n):
    """Four replays with eager work and synchronisation between them; every replay is compared with the same
    step run eagerly on a twin state (and the first one with the oracle)."""
    eager, graphed = _state(n, 7), _state(n, 7)
    ce_e, ce_g = _ce_inputs(32, 32000, 8), _ce_inputs(32, 32000, 8)
    flag_e, flag_g = (torch.zeros(1, dtype=torch.uint8, device="cuda")[0] for _ in range(2))
    logits_static = ce_g[0]
    before = [t.cpu().numpy().copy() if t.dtype == torch.float32 else bits16(t) for t in eager]

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                         # warm-up outside capture, on a scratch copy
        scratch = tuple(t.clone() for t in graphed)
        _step(*scratch, flag_g.clone(), *tuple(t.clone() for t in ce_g), 1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _step(*graphed, flag_g, *ce_g, 1)               # the step number is baked into the captured arguments
    # capture executes nothing: state is untouched
    assert np.array_equal(f32_bits(graphed[0].cpu().numpy()), f32_bits(before[0]))

    for replay in range(4):
        new_logits = (torch.randn(32, 32000, device="cuda") * 2).bfloat16()     # eager work between replays
        logits_static.copy_(new_logits); ce_e[0].copy_(new_logits)
        graph.replay()
        _step(*eager, flag_e, *ce_e, 1)
        torch.cuda.synchronize()
        for x, y in zip(eager + ce_e, graphed + ce_g):
            assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), replay
        if replay == 0:
            p, h, g, m, v = before
            bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 1)
            oracle.adam_gpu_bf16(p, h, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
            assert np.array_equal(f32_bits(graphed[0].cpu().numpy()), f32_bits(p))
            assert np.array_equal(bits16(graphed[1]), h)
    assert flag_g.item() == 0
    graphed[2][17] = float("inf")                         # the captured scan sees the new gradient contents
    graph.replay()
    torch.cuda.synchronize()
    assert flag_g.item() == 1


def test_large_in_place_cross_entropy_kernels_captured_in_a_graph():
    """On a capturing stream the element-wise cross-entropy kernels of large arrays do without the library's ticket
    counters (a graph may be replayed on any stream, also on two at once); eager launches and replays give the same
    bits, replay after replay, with eager launches between them."""
    rows, classes = 4197, 32008                         # 2^27 elements or more: the resident grid when launched eagerly
    x, t, soft, loss, go = _ce_inputs(rows, classes, 9)
    LF.cross_entropy_forward(rows, classes, x, t, soft, loss, -100)
    eager = soft.clone()
    LF.cross_entropy_backward_inplace(rows, classes, go, t, eager, -100)
    work = soft.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        LF.cross_entropy_backward_inplace(rows, classes, go, t, work, -100)        # warm-up outside the capture
        side.synchronize()
        work.copy_(soft)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            LF.cross_entropy_backward_inplace(rows, classes, go, t, work, -100)
    torch.cuda.synchronize()
    for _ in range(3):
        work.copy_(soft)
        again = soft.clone()
        LF.cross_entropy_backward_inplace(rows, classes, go, t, again, -100)        # eager, same counters as before
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(work.view(torch.int16), eager.view(torch.int16))
        assert torch.equal(again.view(torch.int16), eager.view(torch.int16))


def _runtime():
    """hipStreamCreate / hipStreamDestroy of the runtime instance the library and torch share (torch itself hands
    out streams from a pool of 32 and never destroys one)."""
    import ctypes
    from bmtrain_amd import C
    hip = C._lib
    hip.hipStreamCreate.argtypes, hip.hipStreamCreate.restype = [ctypes.POINTER(ctypes.c_void_p)], ctypes.c_int
    hip.hipStreamDestroy.argtypes, hip.hipStreamDestroy.restype = [ctypes.c_void_p], ctypes.c_int
    return hip, ctypes


def test_a_process_that_recycles_streams_keeps_the_resident_kernel():
    """The resident in-place kernel keeps eight ticket counters per stream in a table of 256 streams per device.
    700 streams are created through the runtime, used for one large in-place launch each and destroyed (300 are alive
    at any time — the runtime reuses the addresses of destroyed streams, so only streams that are alive together have
    different handles): every launch must still run as the resident grid — the table entry of a
    stream whose last launch has completed is handed on — and every checked result equals the first one."""
    from bmtrain_amd import C
    hip, ctypes = _runtime()
    rows, classes = 4197, 32008
    x, t, soft, loss, go = _ce_inputs(rows, classes, 11)
    LF.cross_entropy_forward(rows, classes, x, t, soft, loss, -100)
    expect = soft.clone()
    LF.cross_entropy_backward_inplace(rows, classes, go, t, expect, -100)
    torch.cuda.synchronize()
    before = C.bmt_hip_flat_stream_stats()
    work = [soft.clone() for _ in range(4)]
    alive, seen = [], set()
    try:
        for k in range(700):
            handle = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(handle)) == 0
            alive.append(handle)
            seen.add(handle.value)
            if len(alive) > 300:
                torch.cuda.synchronize()
                assert hip.hipStreamDestroy(alive.pop(0)) == 0
            buf = work[k % 4]
            side = torch.cuda.ExternalStream(handle.value)
            with torch.cuda.stream(side):
                buf.copy_(soft, non_blocking=True)
                LF.cross_entropy_backward_inplace(rows, classes, go, t, buf, -100)
            side.synchronize()
            if k % 50 == 49 or k >= 696:
                assert torch.equal(buf.view(torch.int16), expect.view(torch.int16)), k
    finally:
        torch.cuda.synchronize()
        for handle in alive:
            hip.hipStreamDestroy(handle)
    after = C.bmt_hip_flat_stream_stats()
    assert len(seen) > 256                                # more distinct handles than the table has entries
    assert after["resident"] - before["resident"] == 700
    assert after["fallback"] == before["fallback"]
    assert after["evictions"] - before["evictions"] >= len(seen) - 256


def test_entries_of_streams_with_work_in_flight_are_not_handed_on():
    """300 runtime streams, each with its own buffer, all launched without waiting in between, three rounds: whatever
    the table does for the streams beyond its 256 entries (hand on an entry whose launch has completed, or take the
    kernel without counters), no two running launches may share counters — every buffer comes out exact."""
    from bmtrain_amd import C
    hip, ctypes = _runtime()
    rows, classes = 4197, 32008
    x, t, soft, loss, go = _ce_inputs(rows, classes, 12)
    LF.cross_entropy_forward(rows, classes, x, t, soft, loss, -100)
    expect = soft.clone()
    LF.cross_entropy_backward_inplace(rows, classes, go, t, expect, -100)
    torch.cuda.synchronize()
    handles = []
    try:
        for _ in range(300):
            handle = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(handle)) == 0
            handles.append(handle)
        bufs = [torch.empty_like(soft) for _ in handles]
        before = C.bmt_hip_flat_stream_stats()
        for rnd in range(3):
            for handle, buf in zip(handles, bufs):
                with torch.cuda.stream(torch.cuda.ExternalStream(handle.value)):
                    buf.copy_(soft, non_blocking=True)
                    LF.cross_entropy_backward_inplace(rows, classes, go, t, buf, -100)
            torch.cuda.synchronize()
            for k, buf in enumerate(bufs):
                assert torch.equal(buf.view(torch.int16), expect.view(torch.int16)), (rnd, k)
        after = C.bmt_hip_flat_stream_stats()
        assert after["resident"] + after["fallback"] - before["resident"] - before["fallback"] == 900
    finally:
        torch.cuda.synchronize()
        for handle in handles:
            hip.hipStreamDestroy(handle)


def test_host_threads_launching_at_once_on_their_own_streams():
    """Six host threads (ctypes releases the interpreter lock for the call), each with a stream, buffers and state of
    its own, run 12 whole steps at the same time: has_inf_nan, a resident-grid Adam launch, the long-row forward and
    the resident in-place backward.  The library's only shared host state on this path is the per-device stream table
    behind its mutex and a few cached device properties; every thread's result equals the one a single thread gets."""
    import threading
    n, rows, classes = (1 << 24) + 9, 1100, 128256
    x, t, soft0, loss0, go = _ce_inputs(rows, classes, 21)
    want_state = _state(n, 5)
    want_soft, want_loss = torch.empty_like(soft0), torch.empty_like(loss0)
    want_flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
    for step in range(1, 13):
        _step(*want_state, want_flag, x, t, want_soft, want_loss, go, step)
    torch.cuda.synchronize()
    threads, failures = [], []

    def work(k):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                state = _state(n, 5)
                soft, loss = torch.empty_like(soft0), torch.empty_like(loss0)
                flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
                for step in range(1, 13):
                    _step(*state, flag, x, t, soft, loss, go, step)
                stream.synchronize()
                same = [torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(state, want_state)]
                same += [torch.equal(soft.view(torch.int16), want_soft.view(torch.int16)), torch.equal(loss, want_loss),
                         int(flag.item()) == 0]
                if not all(same):
                    failures.append((k, same))
        except Exception as exc:                      # reported by the main thread
            failures.append((k, repr(exc)))

    for k in range(6):
        threads.append(threading.Thread(target=work, args=(k,)))
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not any(th.is_alive() for th in threads)
    assert failures == []


@pytest.mark.parametrize("flavour", ["bf16", "fp16"])
def test_long_adam_launch_with_and_without_the_library_s_counters(flavour):
    """A resident Adam launch draws its tiles from counters: a slot of the library's own array when the stream has
    one, else (here: under graph capture) four places in the 16-bit output that a kernel in front zeroes and a kernel
    behind overwrites with the real values.  Three steps each way on twin states, from views 5 elements into their
    buffers: same bits after every step, and the first step equal to the oracle."""
    n, off = (1 << 25) + 4 * 2048 + 3, 5                  # resident size for both flavours
    dt16 = torch.float16 if flavour == "fp16" else torch.bfloat16
    mdt = torch.float16 if flavour == "fp16" else torch.float32
    scale = 16.0 if flavour == "fp16" else 1.0
    fn = OF.adam_fp16 if flavour == "fp16" else OF.adam_bf16
    gen = torch.Generator().manual_seed(31)
    host = [torch.randn(n, generator=gen) * 0.02, torch.zeros(n, dtype=dt16), (torch.randn(n, generator=gen) * 1e-3 * scale).to(dt16),
            (torch.randn(n, generator=gen) * 1e-4 * scale).to(mdt), (torch.randn(n, generator=gen) * 1e-6 * scale).abs()]

    def place():
        views = []
        for t in host:
            buf = torch.full((n + 64,), -1, dtype=t.dtype, device="cuda")
            buf[off:off + n] = t.cuda()
            views.append(buf[off:off + n])
        return views
    eager, graphed = place(), place()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                         # warm-up outside capture, on a scratch copy
        fn(*[t.clone() for t in graphed], 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 1)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn(*graphed, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 1)
    for replay in range(3):
        fn(*eager, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, 1)
        graph.replay()
        torch.cuda.synchronize()
        for x, y in zip(eager, graphed):
            assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), replay
        if replay == 0:
            p, v = host[0].numpy().copy(), host[4].numpy().copy()
            h = np.zeros(n, np.uint16)
            bc1, bc2 = oracle.bias_corrections(0.9, 0.999, 1)
            if flavour == "fp16":
                m = bits16(host[3])
                oracle.adam_gpu_fp16(p, h, bits16(host[2]), m, v, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
                assert np.array_equal(bits16(graphed[3]), m)
            else:
                m = host[3].numpy().copy()
                oracle.adam_gpu_bf16(p, h, bits16(host[2]), m, v, 0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
                assert np.array_equal(f32_bits(graphed[3].cpu().numpy()), f32_bits(m))
            assert np.array_equal(f32_bits(graphed[0].cpu().numpy()), f32_bits(p))
            assert np.array_equal(f32_bits(graphed[4].cpu().numpy()), f32_bits(v))
            assert np.array_equal(bits16(graphed[1]), h)


def test_long_adam_launches_on_more_streams_than_the_library_keeps_counters_for():
    """264 runtime streams, each stepping a state of its own (same contents) by one resident-size launch, all in flight
    together: the streams beyond the table's 256 entries get an entry whose launch has completed or fall back to the
    counters in the 16-bit output; no two running launches may share counters — every state comes out like the first,
    and the first like a launch made alone."""
    hip, ctypes = _runtime()
    n = (3 << 22) + 4 * 300 + 1
    proto = _state(n, 41)
    alone = [t.clone() for t in proto]
    OF.adam_bf16(*alone, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 3)
    torch.cuda.synchronize()
    handles = []
    try:
        for _ in range(264):
            handle = ctypes.c_void_p()
            assert hip.hipStreamCreate(ctypes.byref(handle)) == 0
            handles.append(handle)
        states = [[proto[0].clone(), torch.zeros_like(proto[1]), proto[2], proto[3].clone(), proto[4].clone()] for _ in handles]
        torch.cuda.synchronize()
        for rnd in range(2):
            for handle, st in zip(handles, states):
                with torch.cuda.stream(torch.cuda.ExternalStream(handle.value)):
                    OF.adam_bf16(*st, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 3 + rnd)
            torch.cuda.synchronize()
            if rnd == 0:
                for k, st in enumerate(states):
                    for x, y in zip(st, alone):
                        assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), k
        for k, st in enumerate(states[1:]):
            for x, y in zip(st, states[0]):
                assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), k
    finally:
        torch.cuda.synchronize()
        for handle in handles:
            hip.hipStreamDestroy(handle)
