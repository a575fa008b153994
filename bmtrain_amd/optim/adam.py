"""On-device Adam for fp32 / fp16 / bf16 parameters — API of bmtrain/optim/adam.py.

16-bit parameters are stepped by fused HIP launches (``_function.adam_fp16`` /
``adam_bf16``): fp32 master copy, moments and the 16-bit parameter are updated in a
single pass over memory.  Parameters that lie back to back in one buffer (the flat
per-block storage of ZeRO, whose gradients lie back to back too) get their state
allocated back to back as well and are stepped by one launch over the whole run;
small tensors elsewhere share launches; the rest take one launch per tensor.  State layout per parameter (part of the checkpoint format):
``step`` (int), ``exp_avg`` (fp16 for fp16 parameters, else fp32), ``exp_avg_sq``
(fp32), ``_param_fp32`` (fp32 master, 16-bit parameters only).  For fp16 parameters
the two moments are stored multiplied by the loss scale, which is why
``_on_justify_scale`` rescales them whenever the scale changes.
"""
import torch

from . import _function as F
from ._base import check_grad, follows, remap_loaded_state, span, span_follows, torch_adam_fp32, validate_hyper, wants_maximize


def _adjacent_runs(work):
    """Splits 16-bit work items into maximal runs in which all five arrays of an item follow those of the
    item before and step count and learning rate agree."""
    runs, last = [], None
    for item in work:
        here = [span(t) for t in item[:5]]
        prev = runs[-1][-1] if runs else None
        if (prev is not None and item[5] == prev[5] and item[6] == prev[6]
                and all(span_follows(a, b) for a, b in zip(here, last))):
            runs[-1].append(item)
        else:
            runs.append([item])
        last = here
    return runs


class AdamOptimizer(torch.optim.Optimizer):
    """Adam optimizer support fp16 and bf16."""

    _bmtrain_optimizer = True

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, hold_steps=0):
        validate_hyper(lr, betas, eps, weight_decay)
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._hold_steps = hold_steps
        # Tensors share launches, up to 32 per launch (same arithmetic per element as one launch per tensor,
        # which remains available by setting batch_launches to False); a batch of 12.6 M (bf16) or 25.2 M (fp16) elements or more runs as
        # one resident grid over all its tensors.  Tensors of `alone_from` elements or more are long launches
        # by themselves.
        self.batch_launches = True
        self.alone_from = 1 << 28
        # Parameters, gradients and state that are adjacent in memory are stepped as one flat tensor.
        self.merge_adjacent = True

    def _on_justify_scale(self, old_scale, new_scale):
        """fp16 moments are kept as moment * loss_scale (adam.py:46-55)."""
        ratio = new_scale / old_scale
        for group in self.param_groups:
            for p in group["params"]:
                state = self.state.get(p)
                if state and p.dtype == torch.float16:
                    state["exp_avg"] *= ratio
                    state["exp_avg_sq"] *= ratio

    def _init_state(self, p):
        self._init_states([p])
        return self.state[p]

    def _init_states(self, params):
        """Creates the state of `params` (in order).  16-bit parameters that follow each other in memory
        receive views into common flat buffers, so that the run can later be stepped by one launch."""
        runs = []
        for p in params:
            last = runs[-1][-1] if runs else None
            if (self.merge_adjacent and last is not None and p.dtype == last.dtype and p.dtype != torch.float32
                    and follows(p, last)):
                runs[-1].append(p)
            else:
                runs.append([p])
        for run in runs:
            first = run[0]
            total = sum(q.numel() for q in run)
            moment_dtype = torch.float16 if first.dtype == torch.float16 else torch.float32
            exp_avg = torch.zeros(total, dtype=moment_dtype, device=first.device)
            exp_avg_sq = torch.zeros(total, dtype=torch.float32, device=first.device)
            master = None if first.dtype == torch.float32 else torch.empty(total, dtype=torch.float32, device=first.device)
            lo = 0
            for q in run:
                hi = lo + q.numel()
                state = self.state[q]
                state["step"] = 0
                state["exp_avg"] = exp_avg[lo:hi].view(q.size())
                state["exp_avg_sq"] = exp_avg_sq[lo:hi].view(q.size())
                if master is not None:
                    state["_param_fp32"] = master[lo:hi].view(q.size())
                    state["_param_fp32"].copy_(q)
                lo = hi

    # step() can apply a gradient clipping factor on the fly (see OptimManager(defer_clip=True))
    supports_grad_coef = True

    @torch.no_grad()
    def step(self, closure=None, scale=1, grad_coef=None, _plan=None):
        """One optimisation step; ``scale`` is the loss scale the gradients carry.  ``grad_coef`` (a 0-dim
        tensor or float below one) clips on the fly: each gradient enters as if it had been multiplied in
        place by it — for 16-bit gradients with the factor rounded to their dtype and the product rounded
        back, as the in-place multiplication does on the GPU — but the gradient tensors are left alone.
        ``_plan``: what ``plan_step`` returned for the same arguments a moment ago (OptimManager prepares the
        step while the overflow scan is still running on the GPU)."""
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for action in (self.plan_step(scale, grad_coef) if _plan is None else _plan):
            action()
        return loss

    @torch.no_grad()
    def plan_step(self, scale=1, grad_coef=None, create_state=True):
        """The host side of a step — which tensors go into which launch, with which step count and learning
        rate — as a list of calls that ``step`` then only has to make.  Nothing of the optimizer's state changes
        here except that parameters seen for the first time get their state; with ``create_state=False`` not
        even that: None is returned instead of a plan when a parameter has no state yet (a step that may still be
        called off must not copy parameters into master weights).  A plan is only good for a step taken right
        away, before anybody touches parameters, gradients or state."""
        actions = []
        for group in self.param_groups:
            beta1, beta2 = group["betas"][0], group["betas"][1]
            eps, weight_decay = group["eps"], group["weight_decay"]
            active = [p for p in group["params"] if p.grad is not None and p.requires_grad]
            for p in active:
                check_grad(p)
            fresh = [p for p in active if len(self.state[p]) == 0]
            if fresh and not create_state:
                return None
            self._init_states(fresh)

            half = []     # 16-bit work: (param_fp32, param, grad, exp_avg, exp_avg_sq, step, lr)
            counted = []  # their states: the step count goes up when the step is taken
            for p in active:
                state = self.state[p]
                grad = -p.grad if wants_maximize(group) else p.grad
                if p.dtype == torch.float32:
                    # hold_steps is tested before the increment on this path (adam.py:137).
                    lr = 0.0 if state["step"] < self._hold_steps else group["lr"]
                    actions.append(self._fp32_action(p, grad, state, lr, scale, grad_coef, beta1, beta2, eps, weight_decay))
                else:
                    # ... and after the increment on the fused path (adam.py:145,155).
                    step = state["step"] + 1
                    lr = 0.0 if step < self._hold_steps else group["lr"]
                    half.append((state["_param_fp32"], p, grad, state["exp_avg"], state["exp_avg_sq"], step, lr))
                    counted.append(state)
            if counted:
                actions.append(self._count_action(counted))

            # 16-bit parameters that can share launches: (dtype, step, lr) -> tensors.
            batches, singles = {}, []
            coef16 = {}
            if grad_coef is not None:      # the factor as the in-place multiplication would see it, per dtype
                as_tensor = torch.as_tensor(grad_coef, dtype=torch.float32)
                coef16 = {dt: float(as_tensor.to(dt).float()) for dt in (torch.float16, torch.bfloat16)}
            for run in _adjacent_runs(half) if self.merge_adjacent else [[w] for w in half]:
                p32, p, grad, m, v, step, lr = run[0]
                if len(run) > 1:
                    total = sum(w[1].numel() for w in run)
                    p32, p, grad, m, v = (t.as_strided((total,), (1,)) for t in (p32, p, grad, m, v))
                item = (p32, p, grad, m, v, step, lr)
                if (self.batch_launches or coef16) and p.is_contiguous() and grad.is_contiguous():
                    batches.setdefault((p.dtype, step, lr), []).append(item)
                else:
                    singles.append(item)
            for key in list(batches) if not coef16 else []:     # with a clipping factor everything goes batched
                singles.extend(w for w in batches[key] if w[1].numel() >= self.alone_from)
                batches[key] = [w for w in batches[key] if w[1].numel() < self.alone_from]
            for p32, p, grad, m, v, step, lr in singles:
                actions.append(self._single_action(p32, p, grad, m, v, step, lr, scale, grad_coef if coef16 else None,
                                                   beta1, beta2, eps, weight_decay))
            for (dtype, step, lr), items in batches.items():
                if items:
                    actions.append(self._multi_action([w[:5] for w in items], step, lr, scale, coef16.get(dtype, 1.0),
                                                      beta1, beta2, eps, weight_decay))
        return actions

    @staticmethod
    def _count_action(states):
        def run():
            for state in states:
                state["step"] += 1
        return run

    @staticmethod
    def _multi_action(tensors, step, lr, scale, coef, beta1, beta2, eps, weight_decay):
        def run():
            F.adam_multi(tensors, beta1, beta2, eps, lr, scale, weight_decay, step, grad_coef=coef)
        return run

    @staticmethod
    def _fp32_action(p, grad, state, lr, scale, grad_coef, beta1, beta2, eps, weight_decay):
        def run():
            g = grad if grad_coef is None else grad * grad_coef
            torch_adam_fp32(p, g / scale, state["exp_avg"], state["exp_avg_sq"], state["step"],
                            beta1=beta1, beta2=beta2, lr=lr, weight_decay=weight_decay, eps=eps)
            state["step"] += 1
        return run

    @staticmethod
    def _single_action(p32, p, grad, m, v, step, lr, scale, grad_coef, beta1, beta2, eps, weight_decay):
        def run():
            g = grad
            if grad_coef is not None:      # not contiguous: clip a copy of the gradient eagerly
                g = grad * torch.as_tensor(grad_coef, dtype=torch.float32, device=grad.device)
            fused = F.adam_fp16 if p.dtype == torch.float16 else F.adam_bf16
            fused(p32, p, g, m, v, beta1, beta2, eps, lr, scale, weight_decay, step)
        return run

    def get_avg_delta():
        raise NotImplementedError(
            "get delta info is not supported in Adam optimizer , try bmt.optim.AdamOffloadOptimizer"
        )

    def get_var_delta():
        raise NotImplementedError(
            "get delta info is not supported in Adam optimizer , try bmt.optim.AdamOffloadOptimizer"
        )

    def load_state_dict(self, state_dict: dict) -> None:
        """Loads optimizer state, casting each tensor to the dtype / device this optimizer
        keeps it in and rebuilding a missing fp32 master copy from the parameter
        (adam.py:175-248)."""

        def convert(param, entry):
            if param.dtype != torch.float32 and "_param_fp32" not in entry:
                entry["_param_fp32"] = torch.empty(param.size(), dtype=torch.float32, device=param.device)
                entry["_param_fp32"].copy_(param)
            wanted = {
                "exp_avg": torch.float16 if param.dtype == torch.float16 else torch.float32,
                "exp_avg_sq": torch.float32,
                "_param_fp32": torch.float32,
            }
            for name, dtype in wanted.items():
                if name in entry:
                    entry[name] = entry[name].to(param.device).to(dtype)
            return entry

        remap_loaded_state(self, state_dict, convert)

    # zero_grad(set_to_none=True) breaks gradient accumulation into persistent buffers.
    def zero_grad(self, set_to_none: bool = False):
        super().zero_grad(set_to_none=set_to_none)
