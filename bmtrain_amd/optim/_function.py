"""Argument checking and dispatch in front of the Adam launchers.

Same functions, argument order and failure modes as bmtrain/optim/_function.py:
AssertionError for layout / dtype / device / size mismatches, NotImplementedError
when bf16 is unavailable; the bias corrections are computed here in Python double
(``1 - beta ** step``) and cross the C ABI as floats.
"""
import torch

from .. import C

_SIXTEEN_BIT = (torch.float16, torch.bfloat16)


def _current_stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _on_gpu(t: torch.Tensor) -> bool:
    return t.is_contiguous() and t.is_cuda


def _same_numel(ref_name, ref, **others):
    for name, t in others.items():
        assert ref.numel() == t.numel(), f"{ref_name} and {name} must have the same number of elements"


def _require_bf16():
    if not C.is_bf16_supported():
        raise NotImplementedError("bfloat16 is not supported on current GPU")


def bf16_from_fp32(param_fp32: torch.Tensor) -> torch.Tensor:
    """Host conversion by truncation (bmtrain/optim/_function.py:7-12)."""
    out = torch.empty_like(param_fp32, dtype=torch.bfloat16)
    C.to_bf16_from_fp32(param_fp32.numel(), param_fp32.data_ptr(), out.data_ptr())
    return out


def fp16_from_fp32(param_fp32: torch.Tensor) -> torch.Tensor:
    """Host conversion, round to nearest even (bmtrain/optim/_function.py:15-20)."""
    out = torch.empty_like(param_fp32, dtype=torch.float16)
    C.to_fp16_from_fp32(param_fp32.numel(), param_fp32.data_ptr(), out.data_ptr())
    return out


def adam_cpu(param_fp32, param_fp16, delta_info, g_fp16, m_fp32, v_fp32,
             beta1: float, beta2: float, eps: float, lr: float, scale: float, weight_decay: float, step: int) -> None:
    """Host-memory Adam step (bmtrain/optim/_function.py:23-100)."""
    cpu = torch.device("cpu")
    named = dict(param_fp32=param_fp32, param_fp16=param_fp16, g_fp16=g_fp16, m_fp32=m_fp32, v_fp32=v_fp32)
    for name, t in named.items():
        assert t.is_contiguous(), f"{name} must be contiguous"
    for name in ("param_fp32", "m_fp32", "v_fp32"):
        assert named[name].dtype == torch.float32, f"{name} must be float32 tensor"
    for name in ("param_fp16", "g_fp16"):
        assert named[name].dtype in _SIXTEEN_BIT, f"{name} must be float16/bfloat16 tensor"
    for name, t in named.items():
        assert t.device == cpu, f"{name} must be a cpu tensor"
    _same_numel("param_fp32", param_fp32, param_fp16=param_fp16, g_fp16=g_fp16, m_fp32=m_fp32, v_fp32=v_fp32)
    if delta_info is not None:
        assert delta_info.is_contiguous(), "delta_info must be contiguous"
        assert delta_info.dtype == torch.float32, "delta_info must be float32 tensor"
        assert delta_info.device == cpu, "delta_info must be a cpu tensor"
        assert delta_info.numel() == 4, "delta_info have a length of 4"
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    if g_fp16.dtype == torch.bfloat16:
        _require_bf16()
        launcher = C.adam_cpu_bf16_launcher
    else:
        launcher = C.adam_cpu_fp16_launcher
    launcher(
        param_fp32.numel(), param_fp32.data_ptr(), param_fp16.data_ptr(),
        delta_info.data_ptr() if delta_info is not None else 0,
        g_fp16.data_ptr(), m_fp32.data_ptr(), v_fp32.data_ptr(),
        beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2,
    )


def adam_fp16(param_fp32, param_fp16, g_fp16, m_fp16, v_fp32,
              beta1: float, beta2: float, eps: float, lr: float, scale: float, weight_decay: float, step: int) -> None:
    """Fused GPU step, fp16 parameters: moments live multiplied by ``scale``
    (bmtrain/optim/_function.py:103-158)."""
    named = dict(param_fp32=param_fp32, param_fp16=param_fp16, g_fp16=g_fp16, m_fp16=m_fp16, v_fp32=v_fp32)
    for name, t in named.items():
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    for name in ("param_fp32", "v_fp32"):
        assert named[name].dtype == torch.float32, f"{name} must be float32 tensor"
    for name in ("param_fp16", "g_fp16", "m_fp16"):
        assert named[name].dtype == torch.float16, f"{name} must be float16 tensor"
    _same_numel("param_fp32", param_fp32, param_fp16=param_fp16, g_fp16=g_fp16, m_fp16=m_fp16, v_fp32=v_fp32)
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    C.adam_fp16_launcher(
        param_fp32.numel(), param_fp32.data_ptr(), param_fp16.data_ptr(), g_fp16.data_ptr(),
        m_fp16.data_ptr(), v_fp32.data_ptr(),
        beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2, _current_stream(),
    )


def adam_bf16(param_fp32, param_bf16, g_bf16, m_fp32, v_fp32,
              beta1: float, beta2: float, eps: float, lr: float, scale: float, weight_decay: float, step: int) -> None:
    """Fused GPU step, bf16 parameters: gradient is unscaled, moments are plain fp32
    (bmtrain/optim/_function.py:161-218)."""
    named = dict(param_fp32=param_fp32, param_bf16=param_bf16, g_bf16=g_bf16, m_fp32=m_fp32, v_fp32=v_fp32)
    for name, t in named.items():
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    for name in ("param_fp32", "m_fp32", "v_fp32"):
        assert named[name].dtype == torch.float32, f"{name} must be float32 tensor"
    for name in ("param_bf16", "g_bf16"):
        assert named[name].dtype == torch.bfloat16, f"{name} must be bfloat16 tensor"
    _same_numel("param_fp32", param_fp32, param_bf16=param_bf16, g_bf16=g_bf16, m_fp32=m_fp32, v_fp32=v_fp32)
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    _require_bf16()
    C.adam_bf16_launcher(
        param_fp32.numel(), param_fp32.data_ptr(), param_bf16.data_ptr(), g_bf16.data_ptr(),
        m_fp32.data_ptr(), v_fp32.data_ptr(),
        beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2, _current_stream(),
    )


def grad_stats(g_half: torch.Tensor, sumsq: torch.Tensor, flag: torch.Tensor) -> None:
    """One pass over a 16-bit gradient: ``sumsq`` (float64, 1 element) += sum of squares and ``flag``
    (uint8, 1 element) = 1 if an inf / NaN is present (left alone otherwise).  Replaces, for gradient
    clipping, the reference's ``g.float().norm(2) ** 2`` (optim_manager.py:186-190) and folds the
    overflow scan (optim_manager.py:9-21) into the same read of the gradient."""
    assert g_half.is_contiguous() and g_half.is_cuda, "g_half must be contiguous and on cuda"
    assert sumsq.is_cuda and sumsq.dtype == torch.float64 and sumsq.numel() == 1, "sumsq must be one float64 on cuda"
    assert flag.is_cuda and flag.dtype == torch.uint8 and flag.numel() == 1, "flag must be one uint8 on cuda"
    if g_half.dtype == torch.float16:
        launcher = C.grad_stats_fp16_launcher
    elif g_half.dtype == torch.bfloat16:
        _require_bf16()
        launcher = C.grad_stats_bf16_launcher
    else:
        raise ValueError(f"grad_stats not supported for dtype {g_half.dtype}")
    n = g_half.numel()
    workspace = torch.empty(C.grad_stats_workspace_floats(n), dtype=torch.float32, device=g_half.device)
    launcher(n, g_half.data_ptr(), sumsq.data_ptr(), flag.data_ptr(), workspace.data_ptr(), _current_stream())


def grad_stats_multi(grads, sumsq, flag: torch.Tensor) -> None:
    """``grad_stats`` (``sumsq`` a float64 tensor) or the overflow scan alone (``sumsq`` None) over a list of
    16-bit gradients of one dtype, in one launch per 64 tensors instead of one or two per tensor — what a model
    whose gradients are separate allocations needs (the loops of optim_manager.py:9-21 and :186-190)."""
    if not grads:
        return
    dtype = grads[0].dtype
    if dtype == torch.bfloat16:
        _require_bf16()
    elif dtype != torch.float16:
        raise ValueError(f"grad_stats not supported for dtype {dtype}")
    assert flag.is_cuda and flag.dtype == torch.uint8 and flag.numel() == 1, "flag must be one uint8 on cuda"
    rows = []
    for g in grads:
        assert g.is_contiguous() and g.is_cuda, "gradients must be contiguous and on cuda"
        assert g.dtype == dtype, "all gradients must share one 16-bit dtype"
        rows.append((g.data_ptr(), g.numel()))
    if sumsq is None:
        C.grad_stats_multi_launcher(rows, int(dtype == torch.bfloat16), 0, flag.data_ptr(), 0, _current_stream())
        return
    assert sumsq.is_cuda and sumsq.dtype == torch.float64 and sumsq.numel() == 1, "sumsq must be one float64 on cuda"
    floats = sum(C.grad_stats_workspace_floats(n) for _, n in rows)
    workspace = torch.empty(floats, dtype=torch.float32, device=flag.device)
    C.grad_stats_multi_launcher(rows, int(dtype == torch.bfloat16), sumsq.data_ptr(), flag.data_ptr(), workspace.data_ptr(),
                                _current_stream())


def adam_multi(tensors, beta1: float, beta2: float, eps: float, lr: float, scale: float, weight_decay: float,
               step: int, grad_coef: float = 1.0) -> None:
    """Fused GPU step over several parameter tensors that share hyper-parameters and step count.
    ``grad_coef`` != 1 applies gradient clipping on the fly: every gradient element enters the step as
    ``to16(float(g) * grad_coef)`` — the bits an eager ``g.mul_(coef)`` would have left — while the gradient
    tensors stay as they are.

    ``tensors`` is a list of ``(param_fp32, param_16, g_16, m, v_fp32)`` as ``adam_fp16`` / ``adam_bf16`` take
    them, all of one 16-bit flavour.  Same arithmetic per element; the tensors travel to the device in the
    kernel arguments of as few launches as possible instead of one launch each (adam.py:72-159)."""
    if not tensors:
        return
    flavour = tensors[0][1].dtype
    assert flavour in _SIXTEEN_BIT, "adam_multi takes float16 or bfloat16 parameters"
    moment_dtype = torch.float16 if flavour == torch.float16 else torch.float32
    rows = []
    for param_fp32, param_16, g_16, m, v_fp32 in tensors:
        named = dict(param_fp32=param_fp32, param_16=param_16, g_16=g_16, m=m, v_fp32=v_fp32)
        for name, t in named.items():
            assert _on_gpu(t), f"{name} must be contiguous and on cuda"
        assert param_fp32.dtype == torch.float32 and v_fp32.dtype == torch.float32, "master and v must be float32"
        assert param_16.dtype == flavour and g_16.dtype == flavour, "all tensors must share one 16-bit dtype"
        assert m.dtype == moment_dtype, "first moment must be float16 for float16 parameters, else float32"
        _same_numel("param_fp32", param_fp32, param_16=param_16, g_16=g_16, m=m, v_fp32=v_fp32)
        rows.append((param_fp32.data_ptr(), param_16.data_ptr(), g_16.data_ptr(), m.data_ptr(), v_fp32.data_ptr(),
                     param_fp32.numel()))
    bias_correction1 = 1 - beta1 ** step
    bias_correction2 = 1 - beta2 ** step
    if flavour == torch.bfloat16:
        _require_bf16()
    if grad_coef == 1.0:
        launcher = C.adam_bf16_multi_launcher if flavour == torch.bfloat16 else C.adam_fp16_multi_launcher
        launcher(rows, beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2, _current_stream())
    else:
        launcher = C.adam_bf16_multi_clip_launcher if flavour == torch.bfloat16 else C.adam_fp16_multi_clip_launcher
        launcher(rows, beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2, grad_coef,
                 _current_stream())
