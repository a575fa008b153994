"""Writes tests/golden/adam_cpu_*.npz: input/output vectors of the reference's own CPU
Adam, produced by running oracle/_ref/refadam.so (the reference's adam_cpu.hpp compiled
as it lies in the reference checkout; build it with `make -C oracle ref`).

Only data is stored: inputs (initial fp32 parameters, per-step 16-bit gradients as bit
patterns, hyper-parameters) and the outputs the compiled reference produced for them
(fp32 parameters, moments, 16-bit copy, delta_info after every step), together with the
SIMD level and thread count in effect, because those decide which elements take the
vector or the scalar expression tree.

    python tests/golden/make_adam_cpu_vectors.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
HYPER = dict(beta1=0.9, beta2=0.999, eps=1e-8, lr=1e-3, weight_decay=0.01)


def bits16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def make(ref, dtype: str, n: int, threads: int, scale: float, steps: int, seed: int, record_delta: bool):
    os.sched_setaffinity(0, set(sorted(os.sched_getaffinity(0))[:threads]))
    assert len(os.sched_getaffinity(0)) == threads
    gen = torch.Generator().manual_seed(seed)
    p = (torch.randn(n, generator=gen) * 0.02).numpy().copy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    p16 = np.zeros(n, np.uint16)
    out = dict(p0=p.copy(), dtype=dtype, n=n, threads=threads, level=ref.get_cpu_level(), scale=scale, steps=steps,
               record_delta=record_delta, **HYPER)
    launcher = ref.adam_cpu_fp16_launcher if dtype == "fp16" else ref.adam_cpu_bf16_launcher
    for s in range(1, steps + 1):
        g = torch.randn(n, generator=gen) * 1e-3 * scale
        g16 = bits16(g.half() if dtype == "fp16" else g.bfloat16())
        delta = np.zeros(4, np.float32)
        bc1, bc2 = oracle.bias_corrections(HYPER["beta1"], HYPER["beta2"], s)
        launcher(n, p.ctypes.data, p16.ctypes.data, delta.ctypes.data if record_delta else 0, g16.ctypes.data,
                 m.ctypes.data, v.ctypes.data, HYPER["beta1"], HYPER["beta2"], HYPER["eps"], HYPER["lr"], scale,
                 HYPER["weight_decay"], bc1, bc2)
        out[f"g{s}"] = g16
        out[f"p{s}"] = p.copy()
        out[f"m{s}"] = m.copy()
        out[f"v{s}"] = v.copy()
        out[f"h{s}"] = p16.copy()
        out[f"d{s}"] = delta
    return out


def main():
    ref = oracle.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/refadam.so is not built (make -C oracle ref) or this CPU lacks AVX-512F")
    all_cpus = os.sched_getaffinity(0)
    cases = [
        # name, dtype, n, threads, scale, steps, seed, record_delta
        ("adam_cpu_fp16_t8", "fp16", 1031, 8, 1024.0, 3, 11, False),
        ("adam_cpu_fp16_t3_delta", "fp16", 257, 3, 4.0, 2, 12, True),
        ("adam_cpu_fp16_t1", "fp16", 45, 1, 1024.0, 2, 13, False),
        ("adam_cpu_bf16_t8", "bf16", 1031, 8, 1024.0, 3, 14, False),
        ("adam_cpu_bf16_t2_delta", "bf16", 130, 2, 3.0, 2, 15, True),
    ]
    for name, *args in cases:
        data = make(ref, *args)
        os.sched_setaffinity(0, all_cpus)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **data)
        print("wrote", name, "level", data["level"], "threads", data["threads"])


if __name__ == "__main__":
    main()
