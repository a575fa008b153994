"""TEST INFRASTRUCTURE — Python face of the CPU oracle (``bmt_oracle.c``).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package, and only to check (or time) — never to
produce a result that the library returns.

All array arguments are numpy arrays; 16-bit floating point data travels as
``uint16`` bit patterns.  Functions that the reference runs in place mutate
their array arguments in place as well.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "refadam.so")

TREE_PLAIN = 0
TREE_FMA_MV = 1
TREE_FMA_MVP = 2


def build(ref: bool = True) -> None:
    """Compile the C restatement and, when the reference checkout is present, oracle/_ref."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])
    if ref:
        subprocess.check_call(["make", "-C", _HERE, "ref"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build(ref=False)
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()

_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_f = ctypes.c_float
_p = ctypes.c_void_p


def _ptr(a, dtype):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.dtype == dtype, (type(a), getattr(a, "dtype", None), dtype)
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_p)


def _sig(name, *argtypes):
    fn = getattr(_lib, name)
    fn.argtypes = list(argtypes)
    fn.restype = None
    return fn


_half_to_float = _sig("oracle_half_to_float", _i64, _p, _p)
_to_fp16 = _sig("oracle_to_fp16_from_fp32", _i64, _p, _p)
_to_bf16 = _sig("oracle_to_bf16_from_fp32", _i64, _p, _p)
_to_bf16_rne = _sig("oracle_to_bf16_from_fp32_rne", _i64, _p, _p)
_inf_fp16 = _sig("oracle_has_inf_nan_fp16", _i64, _p, _p)
_inf_bf16 = _sig("oracle_has_inf_nan_bf16", _i64, _p, _p)
_adam_gpu_bf16 = _sig("oracle_adam_gpu_bf16", _i64, _p, _p, _p, _p, _p, _f, _f, _f, _f, _f, _f, _f, _f, ctypes.c_int)
_adam_gpu_fp16 = _sig("oracle_adam_gpu_fp16", _i64, _p, _p, _p, _p, _p, _f, _f, _f, _f, _f, _f, _f, _f, ctypes.c_int)
_adam_cpu_fp16 = _sig("oracle_adam_cpu_fp16", _i64, _p, _p, _p, _p, _p, _p, _f, _f, _f, _f, _f, _f, _f, _f, ctypes.c_int, _i64, ctypes.c_int)
_adam_cpu_bf16 = _sig("oracle_adam_cpu_bf16", _i64, _p, _p, _p, _p, _p, _p, _f, _f, _f, _f, _f, _f, _f, _f, _i64, ctypes.c_int)
_ce_fwd = {
    "fp16": _sig("oracle_ce_forward_fp16", _i64, _i64, _p, _p, _p, _p, _i32),
    "bf16": _sig("oracle_ce_forward_bf16", _i64, _i64, _p, _p, _p, _p, _i32),
}
_ce_fwd_alt = {
    "fp16": _sig("oracle_ce_forward_alt_fp16", _i64, _i64, _p, _p, _p, _p, _i32, _i32, _i32),
    "bf16": _sig("oracle_ce_forward_alt_bf16", _i64, _i64, _p, _p, _p, _p, _i32, _i32, _i32),
}
_ce_bwd = {
    "fp16": _sig("oracle_ce_backward_fp16", _i64, _i64, _p, _p, _p, _i32),
    "bf16": _sig("oracle_ce_backward_bf16", _i64, _i64, _p, _p, _p, _i32),
}
_sumexp = {
    "fp16": _sig("oracle_fused_sumexp_fp16", _i64, _i64, _p, _p, _p),
    "bf16": _sig("oracle_fused_sumexp_bf16", _i64, _i64, _p, _p, _p),
}
_softmax_inplace = {
    "fp16": _sig("oracle_fused_softmax_inplace_fp16", _i64, _i64, _p, _p, _p),
    "bf16": _sig("oracle_fused_softmax_inplace_bf16", _i64, _i64, _p, _p, _p),
}

_sumsq = {"fp16": _lib.oracle_grad_sumsq_fp16, "bf16": _lib.oracle_grad_sumsq_bf16}
for _fn in _sumsq.values():
    _fn.argtypes = [_i64, _p]
    _fn.restype = ctypes.c_double

u16, f32, i32, u8 = np.uint16, np.float32, np.int32, np.uint8


def bias_corrections(beta1: float, beta2: float, step: int):
    """bc = 1 - beta**step in Python double, as optim/_function.py:76-77,139-140,197-198."""
    return 1 - beta1 ** step, 1 - beta2 ** step


def half_to_float(bits: np.ndarray) -> np.ndarray:
    out = np.empty(bits.shape, f32)
    _half_to_float(bits.size, _ptr(bits, u16), _ptr(out, f32))
    return out


def bf16_to_float(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(f32)


def to_fp16_from_fp32(src: np.ndarray) -> np.ndarray:
    out = np.empty(src.shape, u16)
    _to_fp16(src.size, _ptr(src, f32), _ptr(out, u16))
    return out


def to_bf16_from_fp32(src: np.ndarray, rne: bool = False) -> np.ndarray:
    out = np.empty(src.shape, u16)
    (_to_bf16_rne if rne else _to_bf16)(src.size, _ptr(src, f32), _ptr(out, u16))
    return out


def has_inf_nan(bits: np.ndarray, out: np.ndarray, dtype: str) -> None:
    """Sets out[0] = 1 iff any element is inf/NaN; otherwise leaves out alone."""
    fn = {"fp16": _inf_fp16, "bf16": _inf_bf16}[dtype]
    fn(bits.size, _ptr(bits, u16), _ptr(out, u8))


def grad_sumsq(bits: np.ndarray, dtype: str) -> float:
    return float(_sumsq[dtype](bits.size, _ptr(bits, u16)))


def adam_gpu_bf16(p32, p16, g16, m, v, beta1, beta2, eps, lr, scale, wd, bc1, bc2, tree=TREE_FMA_MVP):
    _adam_gpu_bf16(p32.size, _ptr(p32, f32), _ptr(p16, u16), _ptr(g16, u16), _ptr(m, f32), _ptr(v, f32),
                   beta1, beta2, eps, lr, scale, wd, bc1, bc2, tree)


def adam_gpu_fp16(p32, p16, g16, m16, v, beta1, beta2, eps, lr, scale, wd, bc1, bc2, tree=TREE_FMA_MVP):
    _adam_gpu_fp16(p32.size, _ptr(p32, f32), _ptr(p16, u16), _ptr(g16, u16), _ptr(m16, u16), _ptr(v, f32),
                   beta1, beta2, eps, lr, scale, wd, bc1, bc2, tree)


def adam_cpu_fp16(p32, p16, delta_info, g16, m, v, beta1, beta2, eps, lr, scale, wd, bc1, bc2, level, threads,
                  scalar_tree=TREE_FMA_MVP):
    _adam_cpu_fp16(p32.size, _ptr(p32, f32), _ptr(p16, u16), _ptr(delta_info, f32), _ptr(g16, u16),
                   _ptr(m, f32), _ptr(v, f32), beta1, beta2, eps, lr, scale, wd, bc1, bc2, level, threads, scalar_tree)


def adam_cpu_bf16(p32, p16, delta_info, g16, m, v, beta1, beta2, eps, lr, scale, wd, bc1, bc2, threads=1,
                  scalar_tree=TREE_FMA_MVP):
    _adam_cpu_bf16(p32.size, _ptr(p32, f32), _ptr(p16, u16), _ptr(delta_info, f32), _ptr(g16, u16),
                   _ptr(m, f32), _ptr(v, f32), beta1, beta2, eps, lr, scale, wd, bc1, bc2, threads, scalar_tree)


def ce_forward(x_bits, target, ignore_index, dtype):
    """Returns (softmax_bits[m,n], loss[m])."""
    m, n = x_bits.shape
    softmax = np.empty((m, n), u16)
    out = np.empty(m, f32)
    _ce_fwd[dtype](m, n, _ptr(x_bits, u16), _ptr(target, i32), _ptr(softmax, u16), _ptr(out, f32), ignore_index)
    return softmax, out


EXP_LIBM, EXP_DOUBLE, EXP_WITHIN_ONE_ULP, EXP_WITHIN_TWO_ULP = 0, 1, 2, 3
SUM_WARP32, SUM_WAVE64, SUM_DOUBLE = 0, 1, 2


_alt_exp = _sig("oracle_alt_exp", _i64, _p, _p, _i32)


def alt_exp(t: np.ndarray, exp_kind: int) -> np.ndarray:
    """The exponential ce_forward_alt uses for `exp_kind`, element by element (float32 in, float32 out)."""
    out = np.empty(t.size, f32)
    _alt_exp(t.size, _ptr(t, f32), _ptr(out, f32), exp_kind)
    return out


def ce_forward_alt(x_bits, target, ignore_index, dtype, exp_kind=EXP_LIBM, sum_kind=SUM_WARP32):
    """The forward expression evaluated another equally faithful way (which expf, which block-sum order); with the
    defaults it is ce_forward.  Returns (softmax_bits[m,n], loss[m])."""
    m, n = x_bits.shape
    softmax = np.empty((m, n), u16)
    out = np.empty(m, f32)
    _ce_fwd_alt[dtype](m, n, _ptr(x_bits, u16), _ptr(target, i32), _ptr(softmax, u16), _ptr(out, f32), ignore_index,
                       exp_kind, sum_kind)
    return softmax, out


def ce_backward_inplace(grad_output, target, x_bits, ignore_index, dtype):
    m, n = x_bits.shape
    _ce_bwd[dtype](m, n, _ptr(grad_output, f32), _ptr(target, i32), _ptr(x_bits, u16), ignore_index)


def fused_sumexp(x_bits, max_logits, dtype):
    m, n = x_bits.shape
    out = np.empty(m, f32)
    _sumexp[dtype](m, n, _ptr(x_bits, u16), _ptr(max_logits, f32), _ptr(out, f32))
    return out


def fused_softmax_inplace(x_bits, max_logits, sum_exp, dtype):
    m, n = x_bits.shape
    _softmax_inplace[dtype](m, n, _ptr(x_bits, u16), _ptr(max_logits, f32), _ptr(sum_exp, f32))


# --------------------------------------------------------------------------- #
# oracle/_ref: the reference's own compiled CPU Adam (when it has been built).  #
# --------------------------------------------------------------------------- #

def _host_has(*flags) -> bool:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    have = set(line.split(":", 1)[1].split())
                    return all(x in have for x in flags)
    except OSError:
        pass
    return False


def load_ref():
    """Returns the compiled reference module (oracle/_ref/refadam.so) or None.

    It is compiled with -mavx -mfma -mf16c -mavx512f like the reference's own wheel
    build, so it is only loaded on a host that has those instruction sets."""
    if not os.path.exists(_REF_PATH):
        return None
    if not _host_has("avx", "fma", "f16c", "avx512f"):
        return None
    import importlib.util
    spec = importlib.util.spec_from_file_location("refadam", _REF_PATH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod
