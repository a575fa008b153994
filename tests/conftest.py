import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# ---- helpers shared by the test modules -------------------------------------------
def bits16(t: torch.Tensor) -> np.ndarray:
    """uint16 bit patterns of a fp16 / bf16 torch tensor (on any device)."""
    return t.detach().contiguous().cpu().view(torch.int16).numpy().view(np.uint16).copy()


def from_bits16(bits: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(dtype)


def f32_bits(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def ulp_distance16(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """Distance in units in the last place between two arrays of fp16 or bf16 bit patterns
    (sign-magnitude order mapped onto a line; +0 and -0 coincide)."""
    def line(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(line(a_bits) - line(b_bits))


def load_golden(name: str) -> dict:
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}
