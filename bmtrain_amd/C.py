"""Stand-in for BMTrain's compiled extension module ``bmtrain.C`` on the hot path.

The reference registers its launchers with pybind11 (csrc/bind.cpp:3-35); every
pointer crosses as a Python int and every hyper-parameter as a C float.  This
module exposes the same callables, with the same names and positional order, on
top of the C ABI of ``libbmt_hip.so`` (include/bmt_hip.h), loaded with ctypes.

There is no fallback: if the shared library has not been built, importing this
module raises ImportError; a non-zero status from a launcher raises RuntimeError.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "csrc", "libbmt_hip.so")

if not os.path.exists(LIBRARY_PATH):
    raise ImportError(
        f"{LIBRARY_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
        "(or `python -c 'import __graft_entry__ as g; g.build()'` from the repository root)"
    )

_lib = ctypes.CDLL(LIBRARY_PATH)

_i64, _i32, _f, _p = ctypes.c_int64, ctypes.c_int32, ctypes.c_float, ctypes.c_void_p
_HYPER = [_f] * 8  # beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2

# name -> argument types, in the order of include/bmt_hip.h
_SIGNATURES = {
    "has_nan_inf_fp16_launcher": [_i64, _p, _p, _p, _p],
    "has_nan_inf_bf16_launcher": [_i64, _p, _p, _p, _p],
    "adam_fp16_launcher": [_i64, _p, _p, _p, _p, _p] + _HYPER + [_p],
    "adam_bf16_launcher": [_i64, _p, _p, _p, _p, _p] + _HYPER + [_p],
    "adam_cpu_fp16_launcher": [_i64, _p, _p, _p, _p, _p, _p] + _HYPER,
    "adam_cpu_bf16_launcher": [_i64, _p, _p, _p, _p, _p, _p] + _HYPER,
    "to_fp16_from_fp32": [_i64, _p, _p],
    "to_bf16_from_fp32": [_i64, _p, _p],
    "cross_entropy_forward_fp16_launcher": [_i32, _i32, _p, _p, _p, _p, _i32, _p],
    "cross_entropy_forward_bf16_launcher": [_i32, _i32, _p, _p, _p, _p, _i32, _p],
    "cross_entropy_backward_inplace_fp16_launcher": [_i32, _i32, _p, _p, _p, _i32, _p],
    "cross_entropy_backward_inplace_bf16_launcher": [_i32, _i32, _p, _p, _p, _i32, _p],
    "fused_sumexp_fp16_launcher": [_i32, _i32, _p, _p, _p, _p],
    "fused_sumexp_bf16_launcher": [_i32, _i32, _p, _p, _p, _p],
    "fused_softmax_inplace_fp16_launcher": [_i32, _i32, _p, _p, _p, _p],
    "fused_softmax_inplace_bf16_launcher": [_i32, _i32, _p, _p, _p, _p],
    "grad_stats_fp16_launcher": [_i64, _p, _p, _p, _p, _p],
    "grad_stats_bf16_launcher": [_i64, _p, _p, _p, _p, _p],
    "grad_stats_noalloc_launcher": [_i64, _p, _i32, _p, _p, _p],
    "cross_entropy_reduce_forward_launcher": [_i64, _p, _p, _p, _i32, _i32, _i32, _p, _p, _p],
    "cross_entropy_reduce_backward_launcher": [_i64, _p, _p, _i32, _i32, _i32, _p, _p, _p, _p],
}

_lib.bmt_hip_last_error.restype = ctypes.c_char_p
_lib.bmt_hip_last_error.argtypes = []
_lib.is_bf16_supported.restype = ctypes.c_int
_lib.is_bf16_supported.argtypes = []


def last_error() -> str:
    return (_lib.bmt_hip_last_error() or b"").decode("utf-8", "replace")


def _bind(name, argtypes):
    fn = getattr(_lib, name)
    fn.argtypes = argtypes
    fn.restype = ctypes.c_int

    def call(*args):
        if len(args) != len(argtypes):
            raise TypeError(f"{name}() takes {len(argtypes)} positional arguments but {len(args)} were given")
        status = fn(*args)
        if status != 0:
            raise RuntimeError(f"{name} failed with status {status}: {last_error()}")

    call.__name__ = name
    call.__doc__ = f"ctypes binding of `{name}` (include/bmt_hip.h)."
    return call


for _name, _argtypes in _SIGNATURES.items():
    globals()[_name] = _bind(_name, _argtypes)


def is_bf16_supported() -> int:
    return int(_lib.is_bf16_supported())


_lib.grad_stats_workspace_floats.restype = ctypes.c_int64
_lib.grad_stats_workspace_floats.argtypes = [_i64]


def grad_stats_workspace_floats(n: int) -> int:
    """Number of floats of device workspace grad_stats_*_launcher needs for n elements."""
    return int(_lib.grad_stats_workspace_floats(n))


_lib.bmt_hip_flat_stream_stats.restype = ctypes.c_int
_lib.bmt_hip_flat_stream_stats.argtypes = [ctypes.POINTER(_i64)]


def bmt_hip_flat_stream_stats() -> dict:
    """Diagnostics of the in-place cross-entropy kernels on the current device: launches that ran as the resident
    grid, large launches that fell back to the workgroup-per-tile kernel, stream-table entries reassigned."""
    out = (_i64 * 3)()
    if _lib.bmt_hip_flat_stream_stats(out) != 0:
        raise RuntimeError(f"bmt_hip_flat_stream_stats failed: {last_error()}")
    return {"resident": int(out[0]), "fallback": int(out[1]), "evictions": int(out[2])}


class AdamTensor(ctypes.Structure):
    """`bmt_adam_tensor` of include/bmt_hip.h."""
    _fields_ = [("param_fp32", _p), ("param_16", _p), ("grad_16", _p), ("m", _p), ("v", _p), ("n", _i64)]


def _bind_multi(name, extra_floats=0):
    fn = getattr(_lib, name)
    fn.argtypes = [_i32, ctypes.POINTER(AdamTensor)] + _HYPER + [_f] * extra_floats + [_p]
    fn.restype = ctypes.c_int

    def call(tensors, *args):
        """tensors: sequence of (param_fp32_ptr, param_16_ptr, grad_16_ptr, m_ptr, v_ptr, n); then beta1, beta2,
        eps, lr, scale, weight_decay, bias_correction1, bias_correction2[, grad_coef], stream."""
        if len(args) != len(_HYPER) + extra_floats + 1:
            raise TypeError(f"{name}() takes {len(_HYPER) + extra_floats + 2} positional arguments")
        table = (AdamTensor * len(tensors))(*[AdamTensor(*t) for t in tensors])
        status = fn(len(tensors), table, *args)
        if status != 0:
            raise RuntimeError(f"{name} failed with status {status}: {last_error()}")

    call.__name__ = name
    return call


class ScanTensor(ctypes.Structure):
    """`bmt_scan_tensor` of include/bmt_hip.h."""
    _fields_ = [("g_16", _p), ("n", _i64)]


_lib.grad_stats_multi_launcher.argtypes = [_i32, ctypes.POINTER(ScanTensor), _i32, _p, _p, _p, _p]
_lib.grad_stats_multi_launcher.restype = ctypes.c_int


def grad_stats_multi_launcher(tensors, is_bf16, sumsq, flag, workspace, stream):
    """tensors: sequence of (grad_16_ptr, n); sumsq / workspace may be 0 (flag only)."""
    table = (ScanTensor * len(tensors))(*[ScanTensor(*t) for t in tensors])
    status = _lib.grad_stats_multi_launcher(len(tensors), table, is_bf16, sumsq, flag, workspace, stream)
    if status != 0:
        raise RuntimeError(f"grad_stats_multi_launcher failed with status {status}: {last_error()}")


adam_bf16_multi_launcher = _bind_multi("adam_bf16_multi_launcher")
adam_fp16_multi_launcher = _bind_multi("adam_fp16_multi_launcher")
adam_bf16_multi_clip_launcher = _bind_multi("adam_bf16_multi_clip_launcher", 1)
adam_fp16_multi_clip_launcher = _bind_multi("adam_fp16_multi_clip_launcher", 1)

EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + ["is_bf16_supported", "bmt_hip_last_error", "grad_stats_workspace_floats",
                                                  "bmt_hip_flat_stream_stats", "grad_stats_multi_launcher",
                                                  "adam_bf16_multi_launcher", "adam_fp16_multi_launcher",
                                                  "adam_bf16_multi_clip_launcher", "adam_fp16_multi_clip_launcher"])
