"""The entry point that allocates nothing: grad_stats_noalloc_launcher against grad_stats_{fp16,bf16}_launcher."""
import ctypes

import pytest
import torch

from bmtrain_amd import C

pytestmark = pytest.mark.gpu


def _both(g, is_bf16):
    """(sumsq, flag) from the workspace form and from the allocation-free form, through the C ABI."""
    stream = torch.cuda.current_stream().cuda_stream
    n = g.numel()
    out = []
    work = torch.empty(C.grad_stats_workspace_floats(n), dtype=torch.float32, device="cuda")
    for form in ("workspace", "noalloc"):
        sumsq = torch.full((1,), 0.5, dtype=torch.float64, device="cuda")       # accumulated into: start off zero
        flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
        if form == "workspace":
            fn = C.grad_stats_bf16_launcher if is_bf16 else C.grad_stats_fp16_launcher
            fn(n, g.data_ptr(), sumsq.data_ptr(), flag.data_ptr(), work.data_ptr(), stream)
        else:
            C.grad_stats_noalloc_launcher(n, g.data_ptr(), 1 if is_bf16 else 0, sumsq.data_ptr(), flag.data_ptr(), stream)
        out.append((sumsq.cpu().view(torch.int64).item(), int(flag.item())))
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_two_calls_in_a_row_the_second_smaller(dtype):
    """Bit-identical sum of squares and the same flag as the workspace form, on two consecutive calls that share
    the library's fixed array: a large gradient first (many partial sums), then a smaller one whose launch must
    not see what the first call left behind; then one with an inf and an unaligned base."""
    torch.manual_seed(5)
    big = (torch.randn((1 << 25) + 12345, device="cuda") * 3).to(dtype)
    small = (torch.randn(70001, device="cuda") * 3).to(dtype)
    for g in (big, small):
        want, got = _both(g, dtype == torch.bfloat16)
        assert want == got and want[1] == 0
        exact = g.double().pow(2).sum().item() + 0.5
        assert abs(torch.tensor(want[0]).view(torch.float64).item() - exact) <= 1e-6 * exact
    odd = small[3:60000].clone()[1:]            # 2-byte aligned only
    odd[12345] = float("inf")
    want, got = _both(odd, dtype == torch.bfloat16)
    assert want[1] == 1 and got[1] == 1


def test_nothing_is_allocated_and_too_large_is_refused():
    g = torch.zeros(1 << 20, dtype=torch.bfloat16, device="cuda")
    sumsq = torch.zeros(1, dtype=torch.float64, device="cuda")
    flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    C.grad_stats_noalloc_launcher(g.numel(), g.data_ptr(), 1, sumsq.data_ptr(), flag.data_ptr(), stream)   # first use
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(5):
        C.grad_stats_noalloc_launcher(g.numel(), g.data_ptr(), 1, sumsq.data_ptr(), flag.data_ptr(), stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    with pytest.raises(RuntimeError, match="2\\^36"):
        C.grad_stats_noalloc_launcher((1 << 36) + (1 << 20), g.data_ptr(), 1, sumsq.data_ptr(), flag.data_ptr(), stream)
    C.grad_stats_noalloc_launcher(0, 0, 1, 0, 0, stream)       # n <= 0: no-op


def test_captured_in_a_graph_and_replayed():
    """The call is meant for code under graph capture.  Captured on a side stream (after one eager call on the same
    device, so that the array's address has been looked up outside the capture), then replayed five times on that
    stream with new gradient contents and eager work in between: every replay gives the bits of the workspace form,
    and no device memory is taken by capture or replay."""
    n = (1 << 22) + 777
    g = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
    sumsq = torch.zeros(1, dtype=torch.float64, device="cuda")
    flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
    work = torch.empty(C.grad_stats_workspace_floats(n), dtype=torch.float32, device="cuda")
    want_sumsq = torch.zeros(1, dtype=torch.float64, device="cuda")
    want_flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        C.grad_stats_noalloc_launcher(n, g.data_ptr(), 1, sumsq.data_ptr(), flag.data_ptr(), side.cuda_stream)   # warm-up
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            sumsq.zero_()                                   # a fill kernel, not a memset node
            flag.zero_()
            C.grad_stats_noalloc_launcher(n, g.data_ptr(), 1, sumsq.data_ptr(), flag.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    gen = torch.Generator(device="cuda").manual_seed(8)
    for replay in range(5):
        g.copy_((torch.randn(n, generator=gen, device="cuda") * (replay + 1)).bfloat16())     # eager work between replays
        if replay == 3:
            g[n - 5] = float("nan")
        want_sumsq.zero_(); want_flag.zero_()
        C.grad_stats_bf16_launcher(n, g.data_ptr(), want_sumsq.data_ptr(), want_flag.data_ptr(), work.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(flag.item()) == int(want_flag.item()) == (1 if replay == 3 else 0), replay
        if replay != 3:
            assert sumsq.view(torch.int64).item() == want_sumsq.view(torch.int64).item(), replay
    del gen
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before - (64 << 20)      # torch's generator may cache a block; no growth per replay
