"""Fused cross-entropy — API of bmtrain/loss/cross_entropy.py (non-parallel part).

``OpFusedCrossEntropy`` runs the forward kernel (softmax into a scratch tensor plus the
per-row loss) and, in backward, turns that same scratch tensor into the logits gradient
in place and returns it.  ``FusedCrossEntropy`` adds what torch.nn.CrossEntropyLoss
offers around it: ``ignore_index``, class weights, ``none`` / ``sum`` / ``mean``.
"""
from typing import Optional

import torch

from . import _function as F
from ..global_var import config


class OpFusedCrossEntropy(torch.autograd.Function):
    """Cross-entropy over dim 1 of a 16-bit [N, C] tensor; returns the fp32 loss per row."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, target: torch.Tensor, ignore_index: int):
        assert x.ndim == 2
        x = x.contiguous()
        target = target.contiguous()
        softmax = torch.empty(x.size(), device=x.device, dtype=x.dtype)
        out = torch.empty(x.size(0), device=x.device, dtype=torch.float)
        F.cross_entropy_forward(x.size(0), x.size(1), x, target, softmax, out, ignore_index)
        ctx.ignore_index = ignore_index
        ctx.save_for_backward(softmax, target)
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        grad_output = grad_output.contiguous()
        softmax, target = ctx.saved_tensors
        F.cross_entropy_backward_inplace(softmax.size(0), softmax.size(1), grad_output, target, softmax,
                                         ctx.ignore_index)
        return (softmax, None, None)


class OpLossReduce(torch.autograd.Function):
    """``sum`` / ``mean`` reduction of per-row losses with ignored rows and class weights — the torch expressions
    of bmtrain/loss/cross_entropy.py:243-260 (mask or gathered weights, product, two sums, quotient; about ten
    launches forward and six backward for [N]-sized tensors) as one launch each way.  The gradient per row is the
    same two fp32 operations autograd performs; the loss differs from the torch expression only by the order in
    which the rows are added (here: in double, then rounded once)."""

    MAX_ROWS = 1 << 20      # the forward launch is one workgroup

    @staticmethod
    def forward(ctx, losses: torch.Tensor, target: torch.Tensor, weight, n_classes: int, ignore_index: int, mean: bool):
        losses = losses.contiguous()
        result = torch.empty((), device=losses.device, dtype=torch.float)
        weight_sum = torch.empty((), device=losses.device, dtype=torch.float)
        F.loss_reduce_forward(losses, target, weight, n_classes, ignore_index, mean, result, weight_sum)
        ctx.args = (n_classes, ignore_index, mean)
        ctx.save_for_backward(target, weight_sum, weight)
        return result

    @staticmethod
    def backward(ctx, upstream: torch.Tensor):
        target, weight_sum, weight = ctx.saved_tensors
        n_classes, ignore_index, mean = ctx.args
        upstream = upstream.float().contiguous()
        grad_rows = torch.empty(target.numel(), device=target.device, dtype=torch.float)
        F.loss_reduce_backward(target, weight, n_classes, ignore_index, mean, weight_sum, upstream, grad_rows)
        return (grad_rows, None, None, None, None, None)


def _tp_all_reduce(t: torch.Tensor, op: str) -> torch.Tensor:
    """All-reduce over the tensor-parallel group.  With a group of one (the only case this
    single-GPU package runs) the reduction is the identity; a larger group needs the
    distributed runtime's communicator, which is not part of this package."""
    if config.get("tp_size", 1) == 1:
        return t
    raise NotImplementedError("tensor-parallel all-reduce needs the distributed runtime (tp_size > 1)")


class VPFusedCrossEntropy(torch.autograd.Function):
    """Vocabulary-parallel cross-entropy (bmtrain/loss/cross_entropy.py:38-106): every rank holds a
    slice [rank * V, (rank + 1) * V) of the classes.  Row maximum, target logit and sum of
    exponentials are combined across ranks between the local kernels ``fused_sumexp`` and
    ``fused_softmax_inplace``; the backward pass needs no communication."""

    @staticmethod
    def forward(ctx, logits: torch.Tensor, target: torch.Tensor):
        rank = config.get("tp_rank", 0)
        part = logits.size(-1)
        first, last = rank * part, (rank + 1) * part

        max_logits = _tp_all_reduce(torch.max(logits, dim=-1)[0].float(), "max")

        outside = (target < first) | (target >= last)          # also true for ignore_index = -100
        local_target = (target - first).masked_fill(outside, 0)
        logits_2d = logits.view(-1, part)
        local_target_1d = local_target.view(-1)
        rows = torch.arange(logits_2d.size(0), device=logits_2d.device)
        picked = logits_2d[rows, local_target_1d].contiguous().view_as(target).float()
        picked = picked.masked_fill(outside, 0.0)
        picked = _tp_all_reduce(picked, "sum") - max_logits

        sum_exp = _tp_all_reduce(F.fused_sumexp(logits_2d, max_logits.view(-1)), "sum") + 1e-10
        softmax = logits_2d.clone()
        F.fused_softmax_inplace(softmax, max_logits.view(-1), sum_exp)

        loss = torch.log(sum_exp.view(picked.shape)) - picked
        ctx.save_for_backward(softmax, outside, local_target_1d)
        ctx.logits_shape = logits.shape
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        softmax, outside, local_target_1d = ctx.saved_tensors
        grad_2d = softmax                                           # the gradient is built in place
        rows = torch.arange(grad_2d.size(0), device=grad_2d.device)
        grad_2d[rows, local_target_1d] -= (1.0 - outside.view(-1).float()).to(grad_2d.dtype)
        grad_2d.mul_(grad_output.reshape(-1, 1))
        return grad_2d.view(ctx.logits_shape), None


class FusedCrossEntropy(torch.nn.Module):
    r"""Cross entropy between raw scores ``input`` of shape :math:`(N, C)` and class indices
    ``target`` of shape :math:`(N)`, like :class:`torch.nn.CrossEntropyLoss`:

    .. math::
        l_n = - w_{y_n} \log \frac{\exp(x_{n,y_n})}{\sum_{c} \exp(x_{n,c})} \cdot 1\{y_n \ne \text{ignore\_index}\}

    reduced by ``reduction``: ``'none'``, ``'sum'``, or ``'mean'`` (the sum divided by
    :math:`\sum_n w_{y_n} 1\{y_n \ne \text{ignore\_index}\}`).

    fp32 input is handed to ``torch.nn.functional.cross_entropy`` (the only path that honours
    ``label_smoothing``); fp16 / bf16 input takes the fused kernels.

    Args:
        weight: optional 1-D tensor of ``C`` class weights.
        ignore_index: target value that contributes neither loss nor gradient.
        reduction: ``'none'`` | ``'mean'`` | ``'sum'``.
        label_smoothing: only applied to fp32 input.
        parallel: vocabulary-parallel loss (``input`` holds this rank's slice of the classes).
            With one GPU the tensor-parallel group has one member and the result equals the
            non-parallel loss; larger groups need the distributed runtime.

    Example::

        >>> loss_func = bmtrain_amd.loss.FusedCrossEntropy()
        >>> logits = torch.randn(32, 100, device="cuda").half().requires_grad_()
        >>> target = torch.randint(0, 100, (32,), device="cuda")
        >>> loss_func(logits, target).backward()
    """

    def __init__(self, weight: Optional[torch.Tensor] = None, ignore_index: int = -100, reduction: str = "mean",
                 label_smoothing: float = 0.0, parallel: bool = False) -> None:
        super().__init__()
        self.weight = weight
        self.ignore_index = ignore_index
        self.reduction = reduction
        self.label_smoothing = label_smoothing
        self.parallel = parallel
        # sum / mean of the per-row losses in one launch each way (OpLossReduce); False: the reference's torch operations
        self.fused_reduction = True

    def _can_fuse(self, losses: torch.Tensor, target: torch.Tensor) -> bool:
        if not losses.is_cuda or losses.dtype != torch.float32 or losses.numel() > OpLossReduce.MAX_ROWS:
            return False
        if target.dim() != 1 or target.numel() != losses.numel():
            return False
        w = self.weight
        if w is not None and self.parallel:     # class weights are indexed by the global class, not by this rank's slice
            return False
        return w is None or (w.is_cuda and w.device == losses.device and not w.requires_grad and w.is_floating_point())

    def forward(self, input: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
        target32 = None
        if self.parallel:
            ret = VPFusedCrossEntropy.apply(input, target.long())
        elif input.dtype == torch.float32:
            return torch.nn.functional.cross_entropy(
                input, target.long(), weight=self.weight, ignore_index=self.ignore_index,
                reduction=self.reduction, label_smoothing=self.label_smoothing)
        else:
            target32 = target.int().contiguous()
            ret = OpFusedCrossEntropy.apply(input, target32, self.ignore_index)

        if self.weight is not None and (self.weight.dim() != 1 or self.weight.size(0) != input.size(1)):
            raise ValueError("weight should be a 1D tensor of size C")
        if self.fused_reduction and self.reduction in ("sum", "mean") and self._can_fuse(ret, target):
            weight = None if self.weight is None else self.weight.detach().float().contiguous()
            if target32 is None:
                target32 = target.int().contiguous()
            return OpLossReduce.apply(ret, target32, weight, input.size(1), self.ignore_index, self.reduction == "mean")

        ignored = target == self.ignore_index
        if self.weight is not None:
            w = self.weight[torch.where(ignored, 0, target)].float()
            w[ignored] = 0
        else:
            w = (~ignored).int()

        ret = w * ret
        if self.reduction == "none":
            return ret
        if self.reduction == "sum":
            return ret.sum()
        if self.reduction == "mean":
            return ret.sum() / w.sum().float()
        raise ValueError(f"{self.reduction} is not a valid value for reduction")
