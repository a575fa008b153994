"""Loss scaling, overflow skip and optimizer stepping — API of
bmtrain/optim/optim_manager.py, single GPU.

The overflow check walks the 16-bit gradients with the ``has_inf_nan`` scan (one sticky
flag for all tensors, one host read at the end).  Cross-rank reductions of the flag and
of the gradient norm belong to the distributed runtime and are not performed here.
"""
from typing import Optional

import torch

from ..global_var import config
from ..loss._function import has_inf_nan
from ._base import flat_runs
from ._function import grad_stats, grad_stats_multi


def _scanned_grads(param_groups):
    """The gradients the overflow check looks at: those of non-fp32 parameters."""
    return [p.grad for group in param_groups for p in group["params"] if p.grad is not None and p.dtype != torch.float]


def _scan(grads, sumsq, flag):
    """The overflow scan (``sumsq`` None) or the scan with the sum of squares over 16-bit gradients: gradients that lie
    back to back are read as one run, and several runs of one dtype share a launch."""
    by_dtype = {}
    for g in flat_runs(grads):
        by_dtype.setdefault(g.dtype, []).append(g)
    for dtype, runs in by_dtype.items():
        if len(runs) > 1 and dtype in (torch.float16, torch.bfloat16):
            grad_stats_multi(runs, sumsq, flag)
        else:
            for g in runs:
                if sumsq is None:
                    has_inf_nan(g, flag)
                else:
                    grad_stats(g, sumsq, flag)


def _fingerprint(g):
    """Identifies a gradient's memory and its contents' version (in-place writes bump the counter)."""
    return (g.data_ptr(), g.numel(), g.dtype, g._version)


def launch_overflow_scan(param_groups, known=None, flag=None):
    """Starts the scan of check_overflow and returns the flag it writes (None when there is nothing to scan), without
    waiting for it.  `known` may carry the verdict of an earlier pass over gradients: a pair (flag tensor,
    {fingerprint}); gradients found in it unchanged are not read again.  `flag`: a flag to go on with (it is sticky)."""
    grads = _scanned_grads(param_groups)
    if not grads:
        return flag
    if known is not None and all(_fingerprint(g) in known[1] for g in grads):
        return known[0] if flag is None else torch.maximum(flag, known[0])
    if flag is None:
        flag = torch.zeros(1, dtype=torch.uint8, device="cuda")[0]
    _scan(grads, None, flag)
    return flag


def check_overflow(param_groups, known=None):
    """Raises OverflowError when any non-fp32 gradient holds an inf or NaN
    (optim_manager.py:9-21)."""
    flag = launch_overflow_scan(param_groups, known)
    if flag is not None and flag > 0:
        raise OverflowError("Gradient overflow")


def grad_rescale(param_groups, scale):
    """`p.grad /= scale` for every parameter with a gradient (optim_manager.py:23-27), one launch per run of gradients
    that lie back to back instead of one per parameter."""
    grads = [p.grad for group in param_groups for p in group["params"] if p.grad is not None and p.requires_grad]
    for g in flat_runs(grads):
        g /= scale


class OptimManager:
    """Steps a set of optimizers (and their lr schedulers) that share one dynamic loss scale.

    >>> manager = OptimManager(loss_scale=1024)
    >>> manager.add_optimizer(optimizer, lr_scheduler)
    >>> manager.zero_grad(); manager.backward(loss); manager.step()
    """

    def __init__(self, loss_scale: Optional[float] = None, loss_scale_factor: float = 2,
                 loss_scale_steps: int = 1024, min_loss_scale=1, max_loss_scale=float("inf"),
                 grad_scale: Optional[int] = None, defer_clip: bool = False, reuse_overflow_verdict: bool = False):
        # defer_clip: clip_grad_norm only measures; the clipping factor is applied inside the optimizer's fused
        # step (same parameter update, bit for bit, one pass less over the gradients), and `p.grad` keeps its
        # unclipped values.  Taken only for a call that covers every parameter of every optimizer, all of which
        # must take `grad_coef` in step(), and that is the only call before the step; anything else clips eagerly.
        self.defer_clip = defer_clip
        self._pending_clip = None
        # reuse_overflow_verdict: step() trusts the inf / NaN verdict that clip_grad_norm's pass over the 16-bit
        # gradients produced, for gradients whose memory and autograd version counter are unchanged since.  Off
        # by default: writes through `.data`, `.detach()` views or raw pointers (what collectives do) do not
        # move the version counter, and a gradient overwritten that way between the two calls would go
        # unchecked.  Never used while a communicator or a copy stream is registered in `config`.
        self.reuse_overflow_verdict = reuse_overflow_verdict
        self.loss_scale_enabled = loss_scale is not None
        self.loss_scale = loss_scale if self.loss_scale_enabled else 1
        self.steps_since_last_scale = 0
        self.loss_scale_factor = loss_scale_factor if loss_scale_factor > 1 else 1 / loss_scale_factor
        self.loss_scale_steps = loss_scale_steps
        self.min_loss_scale = min_loss_scale
        self.max_loss_scale = max_loss_scale
        self.grad_scale = config["zero_size"] if grad_scale is None else grad_scale
        self.optimizers = []
        self.lr_schedulers = []
        self._clip_calls = 0          # clip_grad_norm calls since the last backward / zero_grad / step
        # verdict of the overflow scan that clip_grad_norm's pass over the gradients produced on the side
        self._known_overflow = None

    def add_optimizer(self, optimizer: torch.optim.Optimizer, lr_scheduler=None):
        """All optimizers of one manager share the loss scale."""
        self.optimizers.append(optimizer)
        self.lr_schedulers.append(lr_scheduler)

    def scale_loss(self, loss: torch.Tensor) -> torch.Tensor:
        return loss * (self.loss_scale / self.grad_scale)

    @staticmethod
    def _join_load_stream(after_step: bool):
        """Orders the compute stream against the runtime's copy stream when one is
        registered (optim_manager.py:103-105, :155-156)."""
        load_stream = config.get("load_stream")
        if load_stream is None:
            return
        current = torch.cuda.current_stream()
        if after_step:
            load_stream.wait_stream(current)
        else:
            current.wait_stream(load_stream)

    def backward(self, loss: torch.Tensor):
        self._known_overflow = None
        if self._pending_clip is not None:      # gradients are about to be accumulated into: clip them first
            self._scale_grads(self._pending_clip[1], self._pending_clip[0])
        self._pending_clip = None
        self._clip_calls = 0
        self.scale_loss(loss).backward()
        self._join_load_stream(after_step=False)

    def zero_grad(self):
        self._known_overflow = None
        self._pending_clip = None
        self._clip_calls = 0
        for optimizer in self.optimizers:
            optimizer.zero_grad(set_to_none=False)

    def _verdict_usable(self):
        if not self.reuse_overflow_verdict or config.get("comm") is not None or config.get("load_stream") is not None:
            return None
        return self._known_overflow

    def _overflowed(self, meanwhile=None) -> bool:
        """One sticky flag over the gradients of all optimizers, read once.  `meanwhile` is called between the
        launches and the read: host work done there runs while the GPU scans."""
        known = self._verdict_usable()
        flag = None
        for optimizer in self.optimizers:
            flag = launch_overflow_scan(optimizer.param_groups, known, flag)
        self._known_overflow = None
        if meanwhile is not None:
            meanwhile()
        return flag is not None and bool(flag > 0)

    def step(self):
        """Skips the step and lowers the scale on overflow; otherwise steps every optimizer
        and scheduler and raises the scale after ``loss_scale_steps`` clean steps."""
        pending = None if self._pending_clip is None else self._pending_clip[0]
        plans = {}

        def plan_steps():       # the optimizers' host-side preparation; under loss scaling it overlaps the overflow scan
            for optimizer in self.optimizers:
                if getattr(optimizer, "_bmtrain_optimizer", False) and hasattr(optimizer, "plan_step"):
                    plan = optimizer.plan_step(scale=self.loss_scale, grad_coef=pending, create_state=False)
                    if plan is not None:
                        plans[id(optimizer)] = plan

        if self.loss_scale_enabled and self._overflowed(meanwhile=plan_steps):
            lowered = self.loss_scale / self.loss_scale_factor
            print("Gradient overflow, change scale from %lf to %lf" % (self.loss_scale, lowered))
            with torch.no_grad():
                if self.loss_scale > self.min_loss_scale:
                    self._justify_scale(lowered)
                self.zero_grad()
            return
        self._pending_clip = None
        self._clip_calls = 0
        for optimizer, lr_scheduler in zip(self.optimizers, self.lr_schedulers):
            if id(optimizer) in plans:
                optimizer.step(scale=self.loss_scale, grad_coef=pending, _plan=plans[id(optimizer)])
            elif pending is not None:
                optimizer.step(scale=self.loss_scale, grad_coef=pending)
            elif getattr(optimizer, "_bmtrain_optimizer", False):
                optimizer.step(scale=self.loss_scale)
            else:
                if self.loss_scale_enabled:
                    grad_rescale(optimizer.param_groups, self.loss_scale)
                optimizer.step()
            if lr_scheduler is not None:
                lr_scheduler.step()
        if self.loss_scale_enabled:
            self.steps_since_last_scale += 1
            if self.steps_since_last_scale >= self.loss_scale_steps and self.loss_scale < self.max_loss_scale:
                self._justify_scale(self.loss_scale * self.loss_scale_factor)
        self._join_load_stream(after_step=True)

    def _can_defer(self, parameters) -> bool:
        """Deferred clipping hands ONE factor to every optimizer's step, which is the eager result only when
        this call saw every parameter of every optimizer and no other call precedes the step."""
        if not (self.defer_clip and self.optimizers and self._clip_calls == 1
                and all(getattr(o, "supports_grad_coef", False) for o in self.optimizers)):
            return False
        owned = {id(p) for o in self.optimizers for group in o.param_groups for p in group["params"]}
        return owned == {id(p) for p in parameters}

    @staticmethod
    def _scale_grads(parameters, clip_coef):
        """`p.grad.mul_(clip_coef)` for every parameter (optim_manager.py:196-199).  Back-to-back gradients
        are scaled by one launch.  The factor is handed over as a Python number equal to what the tensor form
        uses on the GPU — the 0-dim fp32 tensor rounded to the gradient's dtype — which takes torch's
        vectorised scalar kernel: same bits, 3x faster."""
        as_number = {}
        for g in flat_runs([p.grad.data for p in parameters if p.grad is not None]):
            if g.is_cuda and g.dtype in (torch.float16, torch.bfloat16, torch.float32):
                if g.dtype not in as_number:
                    as_number[g.dtype] = float(clip_coef.to(g.dtype))
                g.mul_(as_number[g.dtype])
            else:
                g.mul_(clip_coef)

    def clip_grad_norm(self, param_groups, max_norm, norm_type=2, eps=1e-6):
        """Clips the (still loss-scaled) gradients to ``max_norm`` in place and returns the
        unscaled total norm (optim_manager.py:158-200)."""
        scale = self.loss_scale
        scanned = None
        if self._pending_clip is not None:
            # a second call before the step: the first call's factor has to be in the gradients by now
            self._scale_grads(self._pending_clip[1], self._pending_clip[0])
            self._pending_clip = None
            self._clip_calls = 2
        else:
            self._clip_calls = getattr(self, "_clip_calls", 0) + 1
        parameters = [p for group in param_groups for p in group["params"]]
        # parameters without a gradient count as zeros (optim_manager.py:176-181): they add nothing
        with_grad = [p for p in parameters if p.grad is not None]
        grads = [p.grad.data for p in with_grad]
        device = grads[0].device if grads else (parameters[0].device if parameters else "cuda")
        if norm_type == "inf":
            total_norm = max(g.abs().max() for g in grads).detach() if grads else torch.zeros((), device=device)
        else:
            norm_type = float(norm_type)
            acc = torch.zeros(1, dtype=torch.float32, device=device)
            fused = [g for g in grads if norm_type == 2.0 and g.is_cuda and g.is_contiguous()
                     and g.dtype in (torch.float16, torch.bfloat16)]
            fused_ids = {id(g) for g in fused}
            if fused:
                # 16-bit gradients: one read of each tensor instead of an fp32 copy plus a norm
                sumsq = torch.zeros(1, dtype=torch.float64, device=device)
                flag = torch.zeros(1, dtype=torch.uint8, device=device)
                _scan(fused, sumsq, flag)
                acc += sumsq.float()
                scanned = (flag, [p.grad for p, g in zip(with_grad, grads) if id(g) in fused_ids])
            for g in grads:
                if id(g) not in fused_ids:
                    acc += g.float().norm(norm_type) ** norm_type
            total_norm = acc[0] ** (1.0 / norm_type)
        clip_coef = float(max_norm * scale) / (total_norm + eps)
        if clip_coef < 1:
            if self._can_defer(parameters):
                self._pending_clip = (clip_coef, with_grad)          # applied by the next step()
            else:
                self._scale_grads(with_grad, clip_coef)
        # The pass over the 16-bit gradients also looked for inf / NaN, and the scaling above cannot change that
        # verdict (it multiplies by a finite factor below one, or by zero when the norm itself is infinite);
        # step() reuses it for gradients that nobody has written to since.
        self._known_overflow = None
        if scanned is not None and self.reuse_overflow_verdict:
            self._known_overflow = (scanned[0][0], {_fingerprint(g) for g in scanned[1]})
        return total_norm / scale

    @torch.no_grad()
    def _justify_scale(self, scale):
        for optimizer in self.optimizers:
            if hasattr(optimizer, "_on_justify_scale"):
                optimizer._on_justify_scale(self.loss_scale, scale)
        self.loss_scale = scale
        self.steps_since_last_scale = 0

    def state_dict(self, gather_opt=False) -> dict:
        def opt_state(opt):
            try:
                return opt.state_dict(gather_opt)
            except TypeError:  # optimizers whose state_dict() takes no argument
                return opt.state_dict()
        return {
            "optimizers": [opt_state(opt) for opt in self.optimizers],
            "lr_schedulers": [s.state_dict() if s else None for s in self.lr_schedulers],
            "loss_scale": self.loss_scale,
            "loss_scale_enabled": self.loss_scale_enabled,
        }

    def load_state_dict(self, state_dict: dict) -> None:
        assert len(self.optimizers) == len(state_dict["optimizers"])
        assert len(self.lr_schedulers) == len(state_dict["lr_schedulers"])
        for opt, saved in zip(self.optimizers, state_dict["optimizers"]):
            opt.load_state_dict(saved)
        for scheduler, saved in zip(self.lr_schedulers, state_dict["lr_schedulers"]):
            if scheduler is not None:
                scheduler.load_state_dict(saved)
        self.loss_scale = state_dict["loss_scale"]
        self.loss_scale_enabled = state_dict["loss_scale_enabled"]
