"""Argument checking and dispatch in front of the overflow-check and cross-entropy
launchers.  Same functions, argument order and exception types as
bmtrain/loss/_function.py (ValueError for a dtype that is not 16-bit,
NotImplementedError when bf16 is unavailable, AssertionError for the rest).
"""
import torch

from .. import C


def _current_stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _on_gpu(t: torch.Tensor) -> bool:
    return t.is_contiguous() and t.is_cuda


def _pick(op: str, dtype: torch.dtype, fp16, bf16):
    if dtype == torch.float16:
        return fp16
    if dtype == torch.bfloat16:
        if not C.is_bf16_supported():
            raise NotImplementedError("bfloat16 is not supported on current GPU")
        return bf16
    raise ValueError(f"{op} not supported for dtype {dtype}")


def has_inf_nan(g_half: torch.Tensor, out: torch.Tensor) -> None:
    """Sets the uint8 flag ``out`` to 1 when ``g_half`` holds an inf or NaN; leaves it
    alone otherwise, so one flag can be accumulated over many tensors
    (bmtrain/loss/_function.py:7-24).  The reference allocates and zeroes a 1024-byte
    scratch tensor per call for its two-kernel reduction; the single-kernel scan here
    needs none, so none is allocated."""
    assert out.dtype == torch.uint8, "out must be a uint8 tensor"
    assert _on_gpu(g_half), "g_fp16 must be contiguous and on cuda"
    assert _on_gpu(out), "out must be contiguous and on cuda"
    launcher = _pick("has_inf_nan", g_half.dtype, C.has_nan_inf_fp16_launcher, C.has_nan_inf_bf16_launcher)
    launcher(g_half.numel(), g_half.data_ptr(), 0, out.data_ptr(), _current_stream())


def cross_entropy_forward(m: int, n: int, input: torch.Tensor, target: torch.Tensor, softmax: torch.Tensor,
                          output: torch.Tensor, ignore_index: int) -> None:
    """softmax[m, n] and per-row loss output[m] from logits input[m, n]
    (bmtrain/loss/_function.py:27-78)."""
    for name, t in (("input", input), ("target", target), ("softmax", softmax), ("output", output)):
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    assert target.dtype == torch.int32, "target must be an int tensor"
    assert output.dtype == torch.float32, "output must be a float tensor"
    assert input.numel() == softmax.numel(), "input and softmax must have the same number of elements"
    assert target.numel() == output.numel(), "target and output must have the same number of elements"
    assert softmax.dtype == input.dtype, "input and softmax must have the same dtype"
    assert input.numel() == m * n and target.numel() == m, "m, n must describe input and target"
    launcher = _pick("cross_entropy_forward", input.dtype,
                     C.cross_entropy_forward_fp16_launcher, C.cross_entropy_forward_bf16_launcher)
    launcher(m, n, input.data_ptr(), target.data_ptr(), softmax.data_ptr(), output.data_ptr(), ignore_index,
             _current_stream())


def cross_entropy_backward_inplace(m: int, n: int, grad_output: torch.Tensor, target: torch.Tensor, x: torch.Tensor,
                                   ignore_index: int) -> None:
    """Turns the stored softmax ``x`` into the logits gradient in place
    (bmtrain/loss/_function.py:81-115)."""
    for name, t in (("grad_output", grad_output), ("target", target), ("x", x)):
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    assert grad_output.dtype == torch.float32, "grad_output must be a float tensor"
    assert target.dtype == torch.int32, "target must be an int tensor"
    assert target.numel() == grad_output.numel(), "target and grad_output must have the same number of elements"
    assert x.numel() == m * n and target.numel() == m, "m, n must describe x and target"
    launcher = _pick("cross_entropy_backward", x.dtype,
                     C.cross_entropy_backward_inplace_fp16_launcher, C.cross_entropy_backward_inplace_bf16_launcher)
    launcher(m, n, grad_output.data_ptr(), target.data_ptr(), x.data_ptr(), ignore_index, _current_stream())


def fused_sumexp(logits: torch.Tensor, max_logits: torch.Tensor) -> torch.Tensor:
    """Row sums of exp(logits - max_logits[:, None]) as fp32 (bmtrain/loss/_function.py:118-147)."""
    assert _on_gpu(logits), "logits must be contiguous and on cuda"
    assert _on_gpu(max_logits), "max_logits must be contiguous and on cuda"
    assert max_logits.dtype == torch.float32, "max_logits must be float tensor"
    assert max_logits.size(0) == logits.size(0), "max_logits must have same size(0) as logits"
    m, n = logits.size(0), logits.size(1)
    sum_exp_logits = torch.empty(m, dtype=torch.float32, device=logits.device)
    launcher = _pick("fused_sumexp", logits.dtype, C.fused_sumexp_fp16_launcher, C.fused_sumexp_bf16_launcher)
    launcher(m, n, logits.data_ptr(), max_logits.data_ptr(), sum_exp_logits.data_ptr(), _current_stream())
    return sum_exp_logits


def fused_softmax_inplace(logits: torch.Tensor, max_logits: torch.Tensor, sum_exp_logits: torch.Tensor) -> None:
    """logits <- exp(logits - max) / sum, row-wise and in place (bmtrain/loss/_function.py:150-182)."""
    for name, t in (("logits", logits), ("max_logits", max_logits), ("sum_exp_logits", sum_exp_logits)):
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    assert max_logits.dtype == torch.float32, "max_logits must be float tensor"
    assert sum_exp_logits.dtype == torch.float32, "sum_exp_logits must be float tensor"
    assert max_logits.size(0) == logits.size(0), "max_logits must have same size(0) as logits"
    assert sum_exp_logits.size(0) == logits.size(0), "sum_exp_logits must have same size(0) as logits"
    m, n = logits.size(0), logits.size(1)
    launcher = _pick("fused_softmax_inplace", logits.dtype,
                     C.fused_softmax_inplace_fp16_launcher, C.fused_softmax_inplace_bf16_launcher)
    launcher(m, n, logits.data_ptr(), max_logits.data_ptr(), sum_exp_logits.data_ptr(), _current_stream())


def loss_reduce_forward(losses: torch.Tensor, target: torch.Tensor, weight, n_classes: int, ignore_index: int,
                        mean: bool, result: torch.Tensor, weight_sum: torch.Tensor) -> None:
    """``result = sum_r w_r * losses[r]`` (divided by ``weight_sum = sum_r w_r`` when ``mean``) with
    ``w_r = 0`` for ignored rows and otherwise ``weight[target[r]]`` (1 without ``weight``): the reduction that
    bmtrain/loss/cross_entropy.py:243-260 writes in torch operations, in one launch."""
    for name, t in (("losses", losses), ("target", target), ("result", result), ("weight_sum", weight_sum)):
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    assert losses.dtype == torch.float32 and result.dtype == torch.float32 and weight_sum.dtype == torch.float32
    assert target.dtype == torch.int32, "target must be an int tensor"
    assert target.numel() == losses.numel(), "target and losses must have the same number of elements"
    if weight is not None:
        assert _on_gpu(weight) and weight.dtype == torch.float32 and weight.numel() == n_classes, \
            "weight must be a contiguous float tensor of n_classes elements on cuda"
    C.cross_entropy_reduce_forward_launcher(losses.numel(), losses.data_ptr(), target.data_ptr(),
                                            weight.data_ptr() if weight is not None else 0, n_classes, ignore_index,
                                            int(mean), result.data_ptr(), weight_sum.data_ptr(), _current_stream())


def loss_reduce_backward(target: torch.Tensor, weight, n_classes: int, ignore_index: int, mean: bool,
                         weight_sum: torch.Tensor, upstream: torch.Tensor, grad_rows: torch.Tensor) -> None:
    """``grad_rows[r] = (upstream / weight_sum if mean else upstream) * w_r``: what autograd derives from the
    torch operations of bmtrain/loss/cross_entropy.py:243-260, in one launch."""
    for name, t in (("target", target), ("weight_sum", weight_sum), ("upstream", upstream), ("grad_rows", grad_rows)):
        assert _on_gpu(t), f"{name} must be contiguous and on cuda"
    assert upstream.dtype == torch.float32 and upstream.numel() == 1, "upstream must be one float"
    assert weight_sum.dtype == torch.float32 and grad_rows.dtype == torch.float32
    assert target.dtype == torch.int32 and target.numel() == grad_rows.numel()
    if weight is not None:
        assert _on_gpu(weight) and weight.dtype == torch.float32 and weight.numel() == n_classes
    C.cross_entropy_reduce_backward_launcher(target.numel(), target.data_ptr(),
                                             weight.data_ptr() if weight is not None else 0, n_classes, ignore_index,
                                             int(mean), weight_sum.data_ptr(), upstream.data_ptr(), grad_rows.data_ptr(),
                                             _current_stream())
