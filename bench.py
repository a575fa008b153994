#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A "step" is one pass of the per-GPU optimizer hot path of a 7B-parameter (Llama-7B shaped) model:

    has_inf_nan over all bf16 gradients        (6,738,415,616 elements, 13.5 GB read)
    fused Adam (bf16) over the flat state      (same count; 28 B / element = 188.7 GB of traffic)
    FusedCrossEntropy forward + backward bf16  (8,192 rows x 128,256 classes, 5 % ignored)

with all inputs resident in HBM before the timed region.  Every kernel is bracketed by HIP events on
the launch stream inside the timed steps; the headline value is the Adam kernel's algorithmic HBM
throughput, and the other kernels are reported next to it.  The CPU baseline (the reference's own
compiled AVX Adam when oracle/_ref is present and runnable, else this repository's restatement) is
timed on the host cores in the same run.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--small]

prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published peak
ADAM_BF16_BYTES = 28            # per element: read p32 4 + m 4 + v 4 + g 2, write p32 4 + m 4 + v 4 + p16 2
SCAN_BYTES = 2                  # per element

LLAMA7B_ELEMENTS = 32 * (4 * 4096 * 4096 + 3 * 4096 * 11008 + 2 * 4096) + 2 * 32000 * 4096 + 4096
assert LLAMA7B_ELEMENTS == 6_738_415_616


def ce_bytes_per_row(classes: int) -> int:
    """forward: read x 2C, write softmax 2C, target 4, loss 4; backward: read 2C, write 2C, target 4,
    grad_output 4."""
    return 8 * classes + 16


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--small", action="store_true",
                    help="one transformer block (202,383,360 elements) and 2,048 rows: a quick functional run, "
                         "not the headline workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the side measurements (other configurations, optimizer-level step); for profiler runs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="after the timed steps, run one plain device-to-device copy of the logits buffer "
                         "(rows * classes * 2 bytes read and written) so that rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE readings can be scaled by a transfer of known size")
    return ap.parse_args()


def fill_normal_(x, std, gen, absolute=False, chunk=1 << 27):
    import torch
    for lo in range(0, x.numel(), chunk):
        part = x[lo:lo + chunk]
        r = torch.randn(part.numel(), generator=gen, device=x.device, dtype=torch.float32).mul_(std)
        part.copy_(r.abs_() if absolute else r)


def cpu_baseline():
    """Reference CPU path on the host cores: AdamOffloadOptimizer's kernel (adam_cpu, fp16 gradients) on
    N = 2^24, lr 1e-3, betas (0.9, 0.999), eps 1e-8, wd 0.01, loss scale 1024, rounds of 10 steps for about 10 s; and
    torch's CPU cross_entropy forward + backward on a row sample of the benchmark's shape."""
    import numpy as np
    import torch
    import oracle

    cores = len(os.sched_getaffinity(0))
    n = 1 << 24
    gen = torch.Generator().manual_seed(0)
    p = (torch.randn(n, generator=gen) * 0.02).numpy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    h = np.zeros(n, np.uint16)
    grads = [(torch.randn(n, generator=gen) * 1e-3 * 1024).half().view(torch.int16).numpy().view(np.uint16).copy()
             for _ in range(2)]
    ref = oracle.load_ref()
    times = []
    step = 0
    t_start = time.perf_counter()
    rounds = 0
    while rounds < 1 or (time.perf_counter() - t_start < 10.0 and rounds < 500):
        for _ in range(10):
            step += 1
            g = grads[step % 2]
            bc1, bc2 = oracle.bias_corrections(0.9, 0.999, step)
            t0 = time.perf_counter()
            if ref is not None:
                ref.adam_cpu_fp16_launcher(n, p.ctypes.data, h.ctypes.data, 0, g.ctypes.data, m.ctypes.data,
                                           v.ctypes.data, 0.9, 0.999, 1e-8, 1e-3, 1024.0, 0.01, bc1, bc2)
            else:
                oracle.adam_cpu_fp16(p, h, None, g, m, v, 0.9, 0.999, 1e-8, 1e-3, 1024.0, 0.01, bc1, bc2, 0, 1)
            times.append(time.perf_counter() - t0)
        rounds += 1
    times.sort()
    median = times[len(times) // 2]
    out = {
        "value": round(ADAM_BF16_BYTES * n / median / 1e9, 3),
        "unit": "GB/s",
        "cores": cores if ref is not None else 1,
        "kind": "reference" if ref is not None else "port",
        "sample": f"adam_cpu fp16 grads, N=2^24, {len(times)} steps timed, median {median * 1e3:.2f} ms/step"
                  + (f", SIMD level {ref.get_cpu_level()}" if ref is not None else ", scalar restatement"),
        "ms_per_step": round(median * 1e3, 3),
        "elements_per_s": round(n / median, 1),
    }
    # the reference's bf16 host path (a scalar loop per thread), same inputs, 10 steps
    gb = [(torch.randn(n, generator=gen) * 1e-3).bfloat16().view(torch.int16).numpy().view(np.uint16).copy()]
    if ref is not None:
        bf_times = []
        for k in range(10):
            bc1, bc2 = oracle.bias_corrections(0.9, 0.999, k + 1)
            t0 = time.perf_counter()
            ref.adam_cpu_bf16_launcher(n, p.ctypes.data, h.ctypes.data, 0, gb[0].ctypes.data, m.ctypes.data,
                                       v.ctypes.data, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, bc1, bc2)
            bf_times.append(time.perf_counter() - t0)
        bf_times.sort()
        out["adam_bf16_GBps"] = round(ADAM_BF16_BYTES * n / bf_times[5] / 1e9, 3)
        out["adam_bf16_sample"] = f"adam_cpu bf16 grads, N=2^24, 10 steps, median {bf_times[5] * 1e3:.2f} ms/step"
    # this repository's own host Adam (the offload optimizer's kernel) on the same inputs and cores, beside it
    try:
        from bmtrain_amd import C
        prod = {}
        for label, launcher, grad_bits, scale in (("fp16", C.adam_cpu_fp16_launcher, grads[0], 1024.0),
                                                  ("bf16", C.adam_cpu_bf16_launcher, gb[0], 1.0)):
            ts = []
            for k in range(20):
                bc1, bc2 = oracle.bias_corrections(0.9, 0.999, k + 1)
                t0 = time.perf_counter()
                launcher(n, p.ctypes.data, h.ctypes.data, 0, grad_bits.ctypes.data, m.ctypes.data, v.ctypes.data,
                         0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
                ts.append(time.perf_counter() - t0)
            ts.sort()
            prod[label] = {"GBps_median": round(ADAM_BF16_BYTES * n / ts[len(ts) // 2] / 1e9, 1),
                           "GBps_best": round(ADAM_BF16_BYTES * n / ts[0] / 1e9, 1),
                           "ms_median": round(ts[len(ts) // 2] * 1e3, 3), "ms_min": round(ts[0] * 1e3, 3)}
        out["product_host_adam"] = dict(prod, cores=cores, sample="adam_cpu_{fp16,bf16}_launcher of libbmt_hip.so, N=2^24, "
                                        "20 steps back to back, same buffers and cores as the reference's kernel above")
    except Exception as exc:                      # the baseline must not sink the GPU numbers
        out["product_host_adam"] = {"error": repr(exc)}
    # The same kernels on a working set no cache holds (N = 2^27: 1.9 GB of state and gradients, 3.76 GB moved per
    # step).  At N = 2^24 the 235 MB working set fits the last-level caches of large hosts, and the figures above then
    # say more about the cache than about the kernel: they have read 350 to 1,400 GB/s for the same code on
    # different boxes of this pool.
    try:
        nb = 1 << 27
        pb = np.full(nb, 0.01, np.float32); mb = np.zeros(nb, np.float32); vb = np.zeros(nb, np.float32)
        hb = np.zeros(nb, np.uint16)
        gbig = np.tile(grads[0], nb // n)
        big = {}
        from bmtrain_amd import C as _C
        runs = [("product_fp16", _C.adam_cpu_fp16_launcher, 1024.0)]
        if ref is not None:
            runs.insert(0, ("reference_fp16", ref.adam_cpu_fp16_launcher, 1024.0))
        for label, launcher, scale in runs:
            ts = []
            for k in range(6):
                bc1, bc2 = oracle.bias_corrections(0.9, 0.999, k + 1)
                t0 = time.perf_counter()
                launcher(nb, pb.ctypes.data, hb.ctypes.data, 0, gbig.ctypes.data, mb.ctypes.data, vb.ctypes.data,
                         0.9, 0.999, 1e-8, 1e-3, scale, 0.01, bc1, bc2)
                ts.append(time.perf_counter() - t0)
            ts = sorted(ts[1:])
            big[label] = {"GBps_median": round(ADAM_BF16_BYTES * nb / ts[len(ts) // 2] / 1e9, 1), "ms_median": round(ts[len(ts) // 2] * 1e3, 2)}
        out["adam_cpu_N_2^27_beyond_cache"] = dict(big, cores=cores, sample="adam_cpu fp16 grads, N=2^27, 5 steps timed after one warm-up")
        del pb, mb, vb, hb, gbig
    except Exception as exc:
        out["adam_cpu_N_2^27_beyond_cache"] = {"error": repr(exc)}
    # CPU cross-entropy (torch), fp32 as FusedCrossEntropy itself does for fp32 input
    torch.set_num_threads(cores)
    for key, rows, classes, std, every in (("ce", 256, 128256, 3.0, 20), ("ce_32000", 1024, 32000, 2.0, 10)):
        x = (torch.randn(rows, classes, generator=gen) * std).requires_grad_()
        t = torch.randint(0, classes, (rows,), generator=gen)
        t[::every] = -100
        best = float("inf")
        for _ in range(3):
            x.grad = None
            t0 = time.perf_counter()
            loss = torch.nn.functional.cross_entropy(x, t, ignore_index=-100)
            loss.backward()
            best = min(best, time.perf_counter() - t0)
        out[key + "_rows_per_s"] = round(rows / best, 1)
        out[key + "_sample"] = (f"torch CPU cross_entropy fwd+bwd fp32, {rows} rows x {classes} classes, "
                                f"{cores} threads, best of 3")
    return out


def timed_batches(torch, fn, iters=20, per_batch=4):
    """(mean, median, min) of the time per call in ms.  The calls run back to back in batches of `per_batch`, each
    batch bracketed by one pair of events (an event between every two short launches would add its own gap to
    each of them); mean over all batches, median and minimum over the batches."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    batches = max(iters // per_batch, 3)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
    for a, b in evs:
        a.record()
        for _ in range(per_batch):
            fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) / per_batch for a, b in evs)
    return sum(ts) / len(ts), ts[len(ts) // 2], ts[0]


def other_workloads(torch, dev, LF, OF, iters=20):
    """The other configurations the targets are stated on (not the headline line): one transformer block's
    flat Adam step (202,383,360 elements, bf16, t = 100; also fp16 and the gradient statistics pass over the
    same gradients), the fp16 overflow scan over 2^30 elements, and the fp16 language-model head
    cross-entropy (16,384 rows x 32,000 classes, 10 % ignored)."""
    def timed(fn):
        return timed_batches(torch, fn, iters)

    def entry(stats, nbytes, **more):
        mean, median, low = stats
        gbps = nbytes / (mean * 1e-3) / 1e9
        return dict({"ms": round(mean, 4), "ms_median": round(median, 4), "ms_min": round(low, 4),
                     "achieved_GBps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}, **more)

    out = {}
    gen = torch.Generator(device=dev).manual_seed(1)
    n = 202_383_360
    p16 = torch.empty(n, dtype=torch.bfloat16, device=dev)
    grad = torch.empty(n, dtype=torch.bfloat16, device=dev)
    p32, mom, var = (torch.empty(n, device=dev) for _ in range(3))
    fill_normal_(p32, 0.02, gen); fill_normal_(mom, 1e-4, gen); fill_normal_(var, 1e-6, gen, absolute=True)
    fill_normal_(grad, 1e-3, gen)
    out["adam_bf16_one_block_202M"] = entry(
        timed(lambda: OF.adam_bf16(p32, p16, grad, mom, var, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100)), ADAM_BF16_BYTES * n,
        buffers="five separate allocations made for this measurement")
    sumsq = torch.zeros(1, dtype=torch.float64, device=dev)
    flag = torch.zeros(1, dtype=torch.uint8, device=dev)
    out["grad_stats_bf16_202M"] = entry(timed(lambda: OF.grad_stats(grad, sumsq, flag)), 2 * n)
    # single mid-size tensors, as per-tensor stepping of a model meets them: below 10,485,760 elements a bf16 launch is
    # one workgroup per tile, from there on the resident grid (launches back to back, so each figure holds one launch gap)
    for label, k in (("adam_bf16_one_tensor_2^22", 1 << 22), ("adam_bf16_one_tensor_2^23", 1 << 23),
                     ("adam_bf16_one_tensor_12.6M", 3 << 22), ("adam_bf16_one_tensor_4096x4096", 1 << 24),
                     ("adam_bf16_one_tensor_11008x4096", 11008 * 4096)):
        out[label] = entry(timed_batches(torch, lambda: OF.adam_bf16(p32[:k], p16[:k], grad[:k], mom[:k], var[:k], 0.9, 0.999, 1e-8, 1e-3,
                                                                     1.0, 0.01, 100), 64, per_batch=16), ADAM_BF16_BYTES * k, elements=k)
    # the same through views that start off every grid (parameters anywhere inside a flat buffer): 1,001 elements in
    for label, k in (("adam_bf16_one_tensor_2^23_view_1001_elements_in", 1 << 23),
                     ("adam_bf16_one_tensor_45M_view_1001_elements_in", 11008 * 4096)):
        lo = 1001
        out[label] = entry(timed_batches(torch, lambda: OF.adam_bf16(p32[lo:lo + k], p16[lo:lo + k], grad[lo:lo + k], mom[lo:lo + k],
                                                                     var[lo:lo + k], 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100),
                                         64, per_batch=16), ADAM_BF16_BYTES * k, elements=k)
    del p16, grad, p32, mom, var
    torch.cuda.empty_cache()
    # the fp16 flavour (24 B / element: the first moment is a 16-bit array, kept multiplied by the loss scale), on buffers of its own
    p32, var = torch.empty(n, device=dev), torch.empty(n, device=dev)
    h16, g16, m16 = (torch.empty(n, dtype=torch.float16, device=dev) for _ in range(3))
    fill_normal_(p32, 0.02, gen); fill_normal_(var, 1e-3, gen, absolute=True); fill_normal_(g16, 1.0, gen); m16.zero_()
    out["adam_fp16_one_block_202M"] = entry(
        timed(lambda: OF.adam_fp16(p32, h16, g16, m16, var, 0.9, 0.999, 1e-8, 1e-3, 1024.0, 0.01, 100)), 24 * n,
        bytes_per_element=24)
    del p32, var, h16, g16, m16
    torch.cuda.empty_cache()
    nf = LLAMA7B_ELEMENTS
    p32, var = torch.empty(nf, device=dev), torch.empty(nf, device=dev)
    h16, g16, m16 = (torch.empty(nf, dtype=torch.float16, device=dev) for _ in range(3))
    fill_normal_(p32, 0.02, gen); fill_normal_(var, 1e-3, gen, absolute=True); fill_normal_(g16, 1.0, gen); m16.zero_()
    out["adam_fp16_6.74B"] = entry(
        timed_batches(torch, lambda: OF.adam_fp16(p32, h16, g16, m16, var, 0.9, 0.999, 1e-8, 1e-3, 1024.0, 0.01, 100), 6, per_batch=1),
        24 * nf, bytes_per_element=24, elements=nf)
    del p32, var, h16, g16, m16
    torch.cuda.empty_cache()

    n16 = 1 << 30
    g = torch.empty(n16, dtype=torch.float16, device=dev)
    fill_normal_(g, 1e-3, gen)
    flag = torch.zeros(1, dtype=torch.uint8, device=dev)[0]
    out["has_inf_nan_fp16_2^30"] = entry(timed(lambda: LF.has_inf_nan(g, flag)), SCAN_BYTES * n16)
    del g
    torch.cuda.empty_cache()

    gen = torch.Generator(device=dev).manual_seed(3)
    rows, classes = 16384, 32000
    x = torch.empty(rows, classes, dtype=torch.float16, device=dev)
    fill_normal_(x.view(-1), 2.0, gen)
    t = torch.randint(0, classes, (rows,), generator=gen, device=dev, dtype=torch.int32)
    t[torch.randperm(rows, generator=gen, device=dev)[: rows // 10]] = -100
    soft = torch.empty_like(x)
    loss = torch.empty(rows, dtype=torch.float32, device=dev)
    valid = (t != -100).float()
    go = (valid / valid.sum()).contiguous()

    def fwd_bwd():
        LF.cross_entropy_forward(rows, classes, x, t, soft, loss, -100)
        LF.cross_entropy_backward_inplace(rows, classes, go, t, soft, -100)
    stats = timed(fwd_bwd)
    out["ce_fp16_16384x32000_fwd_bwd"] = entry(stats, ce_bytes_per_row(classes) * rows, rows_per_s=round(rows / (stats[0] * 1e-3), 1))
    out["ce_fp16_16384x32000_forward"] = entry(
        timed(lambda: LF.cross_entropy_forward(rows, classes, x, t, soft, loss, -100)), (4 * classes + 8) * rows)
    del soft

    # the loss module around the kernels (bmtrain/loss/cross_entropy.py:216-260): output allocations, the ignore mask,
    # the mean over valid rows and autograd, on top of the two launches; reported beside the kernels, outside the roofline
    import bmtrain_amd as bmt
    loss_fn = bmt.loss.FusedCrossEntropy(ignore_index=-100)

    def module_step(logits, targets):
        logits.grad = None
        loss_fn(logits, targets).backward()

    t64 = t.long()
    x.requires_grad_(True)
    stats = timed(lambda: module_step(x, t64))
    out["ce_fp16_16384x32000_module_fwd_bwd"] = {
        "ms": round(stats[0], 4), "ms_median": round(stats[1], 4), "ms_min": round(stats[2], 4),
        "rows_per_s": round(rows / (stats[0] * 1e-3), 1),
        "what": "FusedCrossEntropy(ignore_index=-100)(x, t).backward(): the two kernels plus allocation of the 1 GB softmax / "
                "gradient tensor, the int32 cast of the targets, the mean over the rows that are not ignored (one launch each way) and autograd"}
    x.grad = None
    del x, t64
    torch.cuda.empty_cache()

    # a vocabulary that is not a multiple of 64 (86,583 classes): every row starts at another offset from the 128-byte lines
    # (the forward only: the backward works on the flat array and never sees rows)
    rows, classes = 6144, 86583
    x = torch.empty(rows, classes, dtype=torch.bfloat16, device=dev)
    fill_normal_(x.view(-1), 3.0, gen)
    t = torch.randint(0, classes, (rows,), generator=gen, device=dev, dtype=torch.int32)
    soft = torch.empty_like(x)
    loss = torch.empty(rows, dtype=torch.float32, device=dev)
    out["ce_bf16_6144x86583_forward"] = entry(
        timed(lambda: LF.cross_entropy_forward(rows, classes, x, t, soft, loss, -100)), (4 * classes + 8) * rows)
    del x, soft, t
    torch.cuda.empty_cache()

    # the two row helpers of the vocabulary-parallel loss, bf16, 8,192 rows x 128,256 classes
    rows, classes = 8192, 128256
    x = torch.empty(rows, classes, dtype=torch.bfloat16, device=dev)
    fill_normal_(x.view(-1), 3.0, gen)
    t64 = torch.randint(0, classes, (rows,), generator=gen, device=dev)
    t64[::20] = -100
    x.requires_grad_(True)
    stats = timed(lambda: module_step(x, t64))
    out["ce_bf16_8192x128256_module_fwd_bwd"] = {
        "ms": round(stats[0], 4), "ms_median": round(stats[1], 4), "ms_min": round(stats[2], 4),
        "rows_per_s": round(rows / (stats[0] * 1e-3), 1), "what": "as above, 2.1 GB softmax / gradient tensor"}
    x.grad = None
    x.requires_grad_(False)
    del t64
    row_max = torch.full((rows,), 14.0, dtype=torch.float32, device=dev)
    row_sum = torch.full((rows,), 5e4, dtype=torch.float32, device=dev)
    out["fused_sumexp_bf16_8192x128256"] = entry(timed(lambda: LF.fused_sumexp(x, row_max)), (2 * classes + 8) * rows)
    out["fused_softmax_inplace_bf16_8192x128256"] = entry(timed(lambda: LF.fused_softmax_inplace(x, row_max, row_sum)),
                                                          (4 * classes + 8) * rows)
    del x
    torch.cuda.empty_cache()

    # many small tensors through one multi-tensor launch: 300 vectors of 4,096 elements
    small = [(torch.zeros(4096, device=dev), torch.zeros(4096, dtype=torch.bfloat16, device=dev),
              torch.zeros(4096, dtype=torch.bfloat16, device=dev), torch.zeros(4096, device=dev), torch.zeros(4096, device=dev))
             for _ in range(300)]
    stats = timed(lambda: OF.adam_multi(small, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100))
    out["adam_multi_bf16_300x4096"] = {"ms": round(stats[0], 4), "ms_median": round(stats[1], 4), "ms_min": round(stats[2], 4),
                                       "what": "300 tensors of 4,096 elements, 32 per launch (launch-bound, not a bandwidth figure)"}
    del small

    # the offload optimizer on one block: gradients device -> host, host Adam, 16-bit parameters host -> device
    import bmtrain_amd as bmt
    n = 202_383_360
    param = torch.nn.Parameter(torch.zeros(n, dtype=torch.bfloat16, device=dev))
    offload = bmt.optim.AdamOffloadOptimizer([param], lr=1e-3, weight_decay=0.01)
    g = torch.empty(n, dtype=torch.bfloat16, device=dev)
    fill_normal_(g, 1e-3, gen)
    walls = []
    for k in range(6):
        param.grad = g
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        offload.step()
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t0) * 1e3)
    walls = sorted(walls[1:])                 # the first step allocates and pins the host state
    out["adam_offload_step_bf16_202M"] = {
        "ms_wall_median": round(walls[len(walls) // 2], 2), "ms_wall_min": round(walls[0], 2), "steps": len(walls),
        "elements_per_s": round(n / (walls[len(walls) // 2] * 1e-3), 1),
        "what": "AdamOffloadOptimizer.step(): D2H of gradients, host Adam, H2D of the 16-bit copy, pieces pipelined (PCIe both ways)"}
    return out


def tensor_list_step(torch, p16, grad, p32, mom, var, merge, batch=True, iters=5):
    """The same 6.74 B elements stepped the way a training script does it: 291 parameter tensors of the
    Llama-7B shapes (views into the flat buffers, as ZeRO keeps them; state pre-populated at step 99) through
    `AdamOptimizer.step()`.  merge = True: the optimizer finds the tensors back to back and steps them as one
    run; merge = False: up to 32 tensors per launch, tiles handed out by ticket; batch = False as well: one
    launch per tensor."""
    import bmtrain_amd as bmt
    layer = [(4096, 4096)] * 4 + [(11008, 4096)] * 2 + [(4096, 11008)] + [(4096,)] * 2
    shapes = [(32000, 4096)] + layer * 32 + [(4096,), (32000, 4096)]
    params, lo = [], 0
    for shape in shapes:
        size = 1
        for d in shape:
            size *= d
        param = torch.nn.Parameter(p16[lo:lo + size].view(shape), requires_grad=True)
        param.grad = grad[lo:lo + size].view(shape)
        params.append((param, lo, size, shape))
        lo += size
    assert lo == p16.numel()
    opt = bmt.optim.AdamOptimizer([q[0] for q in params], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    opt.merge_adjacent = merge
    opt.batch_launches = batch
    for param, lo, size, shape in params:
        opt.state[param] = {"step": 99, "exp_avg": mom[lo:lo + size].view(shape),
                            "exp_avg_sq": var[lo:lo + size].view(shape), "_param_fp32": p32[lo:lo + size].view(shape)}
    for _ in range(2):
        opt.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        opt.step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / iters * 1e3
    gbps = ADAM_BF16_BYTES * p16.numel() / (ms * 1e-3) / 1e9
    return {"tensors": len(shapes), "ms_wall": round(ms, 3), "achieved_GBps": round(gbps, 1),
            "frac": round(gbps / HBM_PEAK_GBPS, 4)}


def full_model_side_measurements(torch, OF, p16, grad, p32, mom, var, iters=5):
    """On the resident 6.74 B-element state: the one-pass gradient statistics, and `clip_grad_norm` + `step()`
    through OptimManager with clipping active — eager (the gradients are scaled in place, then stepped) and
    deferred (the step's kernels apply the factor; one pass less over the gradients)."""
    import bmtrain_amd as bmt
    n = grad.numel()
    out = {}
    sumsq = torch.zeros(1, dtype=torch.float64, device=grad.device)
    flag = torch.zeros(1, dtype=torch.uint8, device=grad.device)
    OF.grad_stats(grad, sumsq, flag)
    torch.cuda.synchronize()
    mean, median, low = timed_batches(torch, lambda: OF.grad_stats(grad, sumsq, flag), 12)
    out["grad_stats_bf16_6.74B"] = {"ms": round(mean, 4), "ms_median": round(median, 4), "ms_min": round(low, 4),
                                    "achieved_GBps": round(2 * n / (mean * 1e-3) / 1e9, 1),
                                    "frac": round(2 * n / (mean * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    layer = [(4096, 4096)] * 4 + [(11008, 4096)] * 2 + [(4096, 11008)] + [(4096,)] * 2
    shapes = [(32000, 4096)] + layer * 32 + [(4096,), (32000, 4096)]
    # the same gradients as the 291 tensors of the model, handed over as a list (as separately allocated
    # gradients are): one launch per 64 tensors against one or two launches per tensor
    from bmtrain_amd.loss import _function as LF
    pieces, lo = [], 0
    for shape in shapes:
        size = 1
        for d in shape:
            size *= d
        pieces.append(grad[lo:lo + size])
        lo += size

    def per_tensor(with_sum):
        for g in pieces:
            if with_sum:
                OF.grad_stats(g, sumsq, flag)
            else:
                LF.has_inf_nan(g, flag)
    for label, fn in (("has_inf_nan_291_tensors_multi_launch", lambda: OF.grad_stats_multi(pieces, None, flag)),
                      ("has_inf_nan_291_tensors_launch_per_tensor", lambda: per_tensor(False)),
                      ("grad_stats_291_tensors_multi_launch", lambda: OF.grad_stats_multi(pieces, sumsq, flag)),
                      ("grad_stats_291_tensors_launch_per_tensor", lambda: per_tensor(True))):
        fn()
        torch.cuda.synchronize()
        mean, median, low = timed_batches(torch, fn, 8, 1)
        out[label] = {"ms": round(mean, 4), "ms_median": round(median, 4), "ms_min": round(low, 4),
                      "achieved_GBps": round(2 * n / (mean * 1e-3) / 1e9, 1),
                      "frac": round(2 * n / (mean * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
    gen = torch.Generator(device=grad.device).manual_seed(44)
    for label, defer in (("eager", False), ("deferred", True)):
        params, lo = [], 0
        for shape in shapes:
            size = 1
            for d in shape:
                size *= d
            q = torch.nn.Parameter(p16[lo:lo + size].view(shape))
            q.grad = grad[lo:lo + size].view(shape)
            params.append((q, lo, size, shape))
            lo += size
        opt = bmt.optim.AdamOptimizer([q[0] for q in params], lr=1e-3, weight_decay=0.01)
        for q, lo, size, shape in params:
            opt.state[q] = {"step": 99, "exp_avg": mom[lo:lo + size].view(shape), "exp_avg_sq": var[lo:lo + size].view(shape),
                            "_param_fp32": p32[lo:lo + size].view(shape)}
        manager = bmt.optim.OptimManager(loss_scale=1.0, defer_clip=defer, loss_scale_steps=10 ** 9)
        manager.add_optimizer(opt)
        walls = []
        for k in range(iters + 1):
            fill_normal_(grad, 1e-3, gen)                 # eager clipping shrinks the gradients in place: refill
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            manager.clip_grad_norm(opt.param_groups, max_norm=1e-3)
            manager.step()
            torch.cuda.synchronize()
            walls.append((time.perf_counter() - t0) * 1e3)
        walls = sorted(walls[1:])
        out["clip_grad_norm_plus_step_6.74B_" + label] = {"ms_wall_median": round(walls[len(walls) // 2], 3),
                                                          "ms_wall_min": round(walls[0], 3), "steps": len(walls)}
    return out


KERNEL_SOURCES = ("adam.hip", "cross_entropy.hip", "has_inf_nan.hip", "loss_reduce.hip", "bmt_device.h", "bmt_host.h")


def kernel_sources_digest():
    """sha256 over the device sources: the measured traffic in profiles/ is tied to the kernels it was taken on."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "bmtrain_amd", "csrc", name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def load_measured_traffic():
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE); see profiles/.  The file
    records the digest of the kernel sources it was measured on; figures taken on other sources are not
    reported (second element: where the figures come from, or why there are none)."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if not os.path.exists(path):
        return {}, "profiles/hbm_traffic.json is missing: traffic not reported"
    with open(path) as f:
        measured = json.load(f)
    have, want = measured.get("_kernel_sources_sha256"), kernel_sources_digest()
    if have != want:
        return {}, ("profiles/hbm_traffic.json was measured on kernel sources with digest %s, the sources here have %s: "
                    "traffic not reported" % (have, want))
    return measured, ("rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this command on these kernel sources "
                      "(digest %s), read from profiles/hbm_traffic.json (not measured by this run)" % want)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures the single-GPU hot path only: run it with --gpus 1 "
              "(the path uses no collectives; nothing is sharded across GPUs).", file=sys.stderr)
        sys.exit(2)

    import torch
    import bmtrain_amd  # noqa: F401  (fails loudly when libbmt_hip.so is missing)
    from bmtrain_amd.loss import _function as LF
    from bmtrain_amd.optim import _function as OF

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")

    if args.small:
        n, rows, classes, workload = 202_383_360, 2048, 128256, "one_block_202M_plus_ce_2048x128256_bf16"
    else:
        n, rows, classes = LLAMA7B_ELEMENTS, 8192, 128256
        workload = "llama7b_full_step: has_inf_nan + adam_bf16 over 6,738,415,616 elements, ce bf16 8192x128256"

    # Allocation order of a training process: 16-bit parameters first, their gradients after the first
    # backward pass, the activations of the loss (logits, softmax) with them, and the optimizer's fp32 state
    # last, because AdamOptimizer creates it lazily inside the first step().
    gen = torch.Generator(device=dev).manual_seed(4)
    p16 = torch.empty(n, dtype=torch.bfloat16, device=dev)
    grad = torch.empty(n, dtype=torch.bfloat16, device=dev)
    logits = torch.empty(rows, classes, dtype=torch.bfloat16, device=dev)
    softmax = torch.empty_like(logits)
    p32 = torch.empty(n, device=dev)
    mom = torch.empty(n, device=dev)
    var = torch.empty(n, device=dev)
    fill_normal_(p32, 0.02, gen)
    fill_normal_(mom, 1e-4, gen)
    fill_normal_(var, 1e-6, gen, absolute=True)
    fill_normal_(grad, 1e-3, gen)
    for lo in range(0, n, 1 << 28):
        p16[lo:lo + (1 << 28)].copy_(p32[lo:lo + (1 << 28)])
    fill_normal_(logits.view(-1), 3.0, gen)
    target = torch.randint(0, classes, (rows,), generator=gen, device=dev, dtype=torch.int32)
    target[torch.randperm(rows, generator=gen, device=dev)[: rows // 20]] = -100
    row_loss = torch.empty(rows, dtype=torch.float32, device=dev)
    valid = (target != -100).float()
    grad_output = (valid / valid.sum()).contiguous()
    flag = torch.zeros(1, dtype=torch.uint8, device=dev)[0]
    torch.cuda.synchronize()

    names = ["has_inf_nan", "adam", "ce_forward", "ce_backward"]

    def one_step(step_index, events=None):
        def mark(k):
            if events is not None:
                events[k].record()
        flag.zero_()
        mark(0)
        LF.has_inf_nan(grad, flag)
        mark(1)
        OF.adam_bf16(p32, p16, grad, mom, var, 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100 + step_index)
        mark(2)
        LF.cross_entropy_forward(rows, classes, logits, target, softmax, row_loss, -100)
        mark(3)
        LF.cross_entropy_backward_inplace(rows, classes, grad_output, target, softmax, -100)
        mark(4)

    for w in range(args.warmup):
        one_step(w)
    torch.cuda.synchronize()

    all_events = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        one_step(args.warmup + k, all_events[k])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    assert flag.item() == 0, "synthetic gradients are finite"
    assert torch.isfinite(row_loss).all()

    # The cross-entropy kernels once more, outside the step: the forward launched four times per event pair (one pair
    # around a single sub-millisecond launch also holds the gap to the launch before it), and the backward "cold":
    # between forward and backward a scan over the 13.5 GB of gradients sweeps the caches, where the step's own
    # backward starts right after the forward that wrote its input.
    ce_side = None
    if not args.small:
        fwd = timed_batches(torch, lambda: LF.cross_entropy_forward(rows, classes, logits, target, softmax, row_loss, -100), 24)
        cold = []
        for _ in range(8):
            LF.cross_entropy_forward(rows, classes, logits, target, softmax, row_loss, -100)
            LF.has_inf_nan(grad, flag)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            LF.cross_entropy_backward_inplace(rows, classes, grad_output, target, softmax, -100)
            b.record()
            b.synchronize()
            cold.append(a.elapsed_time(b))
        cold.sort()
        fb = (4 * classes + 8) * rows
        ce_side = {"ce_forward_back_to_back": {"ms": round(fwd[0], 4), "ms_median": round(fwd[1], 4), "ms_min": round(fwd[2], 4),
                                               "frac": round(fb / (fwd[0] * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
                   "ce_backward_cold": {"ms": round(sum(cold) / len(cold), 4), "ms_median": round(cold[len(cold) // 2], 4),
                                        "ms_min": round(cold[0], 4),
                                        "frac": round(fb / (sum(cold) / len(cold) * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}}

    if args.calibrate_copy:
        softmax.copy_(logits)
        torch.cuda.synchronize()

    per_step = {name: sorted(ev[i].elapsed_time(ev[i + 1]) for ev in all_events) for i, name in enumerate(names)}
    ms = {name: sum(ts) / len(ts) for name, ts in per_step.items()}

    def spread(name):
        ts = per_step[name]
        return {"ms_median": round(ts[len(ts) // 2], 4), "ms_min": round(ts[0], 4), "ms_max": round(ts[-1], 4)}
    adam_gbps = ADAM_BF16_BYTES * n / (ms["adam"] * 1e-3) / 1e9
    scan_gbps = SCAN_BYTES * n / (ms["has_inf_nan"] * 1e-3) / 1e9
    ce_ms = ms["ce_forward"] + ms["ce_backward"]
    ce_rows_per_s = rows / (ce_ms * 1e-3)
    ce_gbps = ce_bytes_per_row(classes) * rows / (ce_ms * 1e-3) / 1e9
    ce_fwd_gbps = (4 * classes + 8) * rows / (ms["ce_forward"] * 1e-3) / 1e9
    ce_bwd_gbps = (4 * classes + 8) * rows / (ms["ce_backward"] * 1e-3) / 1e9
    traffic, traffic_source = load_measured_traffic()

    result = {
        "metric": "fused_adam_hbm_gbps_at_6.7b_params",
        "value": round(adam_gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": workload, "elements": n, "ce_rows": rows, "ce_classes": classes,
                   "grad_dtype": "bf16", "adam_step": "t=100+k, lr 1e-3, betas (0.9,0.999), eps 1e-8, wd 0.01, scale 1"},
        "roofline": {
            "kernel": "adam_stream_kernel<bf16>" if n >= (1 << 24) else "adam_bf16_vec_kernel",
            "bound": "hbm",
            "achieved": round(adam_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(adam_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic.get("adam_stream_kernel", {}).get("bytes_per_launch") if not args.small else None,
            "traffic_source": traffic_source,
            "algorithmic_bytes_per_launch": ADAM_BF16_BYTES * n,
            "ms_per_launch": round(ms["adam"], 4),
            **spread("adam"),
            # every timed launch in step order (the mean above is what `value` uses)
            "ms_each_step": [round(ev[1].elapsed_time(ev[2]), 3) for ev in all_events],
        },
        "ce_fwd_bwd_rows_per_s": round(ce_rows_per_s, 1),
        "other_kernels": {
            "has_inf_nan": {"ms": round(ms["has_inf_nan"], 4), **spread("has_inf_nan"), "achieved_GBps": round(scan_gbps, 1),
                            "frac": round(scan_gbps / HBM_PEAK_GBPS, 4), "algorithmic_bytes": SCAN_BYTES * n},
            "ce_forward": {"ms": round(ms["ce_forward"], 4), **spread("ce_forward"), "achieved_GBps": round(ce_fwd_gbps, 1),
                           "frac": round(ce_fwd_gbps / HBM_PEAK_GBPS, 4)},
            "ce_backward": {"ms": round(ms["ce_backward"], 4), **spread("ce_backward"), "achieved_GBps": round(ce_bwd_gbps, 1),
                            "frac": round(ce_bwd_gbps / HBM_PEAK_GBPS, 4)},
            "ce_fwd_bwd": {"ms": round(ce_ms, 4), "achieved_GBps": round(ce_gbps, 1),
                           "frac": round(ce_gbps / HBM_PEAK_GBPS, 4), "bytes_per_row": ce_bytes_per_row(classes)},
        },
    }
    if ce_side:
        result["other_kernels"].update(ce_side)
    side = not (args.small or args.no_other_workloads)
    block_in_place = model_side = None
    if side:
        # one transformer block's worth of the resident model state (what a training process steps when it steps
        # one block): the first 202,383,360 elements of the five 6.74 B-element arrays
        nb = 202_383_360
        step_block = lambda: OF.adam_bf16(p32[:nb], p16[:nb], grad[:nb], mom[:nb], var[:nb], 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.01, 100)
        mean, median, low = timed_batches(torch, step_block, 40)
        block_in_place = {"ms": round(mean, 4), "ms_median": round(median, 4), "ms_min": round(low, 4),
                          "achieved_GBps": round(ADAM_BF16_BYTES * nb / (mean * 1e-3) / 1e9, 1),
                          "frac": round(ADAM_BF16_BYTES * nb / (mean * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                          "buffers": "the first block's slice of the resident 6.74 B-element state"}
        model_side = full_model_side_measurements(torch, OF, p16, grad, p32, mom, var)
    tensor_list = None if not side else {
        "adjacent_tensors_merged": tensor_list_step(torch, p16, grad, p32, mom, var, True),
        "32_tensors_per_launch": tensor_list_step(torch, p16, grad, p32, mom, var, False),
        "one_launch_per_tensor": tensor_list_step(torch, p16, grad, p32, mom, var, False, batch=False)}
    # free the device before the side measurements and the host baseline
    del p32, mom, var, grad, p16, logits, softmax
    torch.cuda.empty_cache()
    if side:
        result["other_workloads"] = other_workloads(torch, dev, LF, OF)
        result["other_workloads"]["adam_bf16_llama7b_291_tensors_via_optimizer_step"] = tensor_list
        result["other_workloads"]["adam_bf16_one_block_202M_in_model_state"] = block_in_place
        result["other_workloads"].update(model_side)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
