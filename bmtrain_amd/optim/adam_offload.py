"""Adam with optimizer state in host memory — API of bmtrain/optim/adam_offload.py.

Per step: gradients are copied device -> pinned host memory asynchronously, each
parameter is updated on the host as soon as its copy has landed (``_function.adam_cpu``
for 16-bit parameters, torch's functional Adam for fp32), and the fresh 16-bit copy is
sent back host -> device asynchronously.  16-bit tensors larger than ``chunk_elements``
are cut into pieces with one event each, so the host step of piece k runs while piece
k+1 is still arriving and piece k-1 is already on its way back; the pieces are disjoint
element ranges, so the result is that of one call over the whole tensor whenever the
vector / scalar split inside ``adam_cpu`` falls the same way (bf16 always; fp16 to
within the two host expression trees).
"""
import torch

from . import _function as F
from ._base import check_grad, remap_loaded_state, torch_adam_fp32, validate_hyper, wants_maximize

_STATE_KEYS = ("step", "exp_avg", "exp_avg_sq", "_param_fp32")


def _pinned(size, dtype):
    return torch.empty(size, dtype=dtype, pin_memory=torch.cuda.is_available())


class AdamOffloadOptimizer(torch.optim.Optimizer):
    """Adam optimizer using optimizer offload."""

    _bmtrain_optimizer = True

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, hold_steps=0,
                 record_delta=False, chunk_elements=1 << 22):
        validate_hyper(lr, betas, eps, weight_decay)
        self.avg_delta = 0
        self.var_delta = 0
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._hold_steps = hold_steps
        self._events = []
        self.chunk_elements = int(chunk_elements)
        self.record_delta = record_delta
        if record_delta:
            for group in self.param_groups:
                for p in group["params"]:
                    p._delta_info = torch.zeros(4, dtype=torch.float32, device="cpu")

    @staticmethod
    def _staging_buffers(p, state):
        """Pinned host buffers the asynchronous copies go through."""
        if p.dtype == torch.float32:
            state["_grad_fp32"] = _pinned(p.size(), torch.float32)
        else:
            state["_param_fp16"] = _pinned(p.size(), p.dtype)
            state["_grad_fp16"] = _pinned(p.size(), p.dtype)

    def _init_state(self, p):
        state = self.state[p]
        state["step"] = 0
        state["exp_avg"] = torch.zeros(p.size(), dtype=torch.float32, device="cpu")
        state["exp_avg_sq"] = torch.zeros(p.size(), dtype=torch.float32, device="cpu")
        if p.dtype == torch.float32:
            state["_param_fp32"] = _pinned(p.size(), torch.float32)
        else:
            state["_param_fp32"] = torch.empty(p.size(), dtype=torch.float32, device="cpu")
        state["_param_fp32"].copy_(p)
        self._staging_buffers(p, state)
        return state

    @torch.no_grad()
    def step(self, closure=None, scale=1):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()

        work = []
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None or not p.requires_grad:
                    continue
                check_grad(p)
                state = self.state[p]
                if len(state) == 0:
                    state = self._init_state(p)
                work.append((p, state, group))

        # Stage every gradient on the host, piece by piece; each copy gets its own event.
        stream = torch.cuda.current_stream()
        pieces = {}
        used = 0
        for p, state, _ in work:
            if p.dtype == torch.float32:
                bounds = [(0, p.numel())]
                src, dst = p.grad, state["_grad_fp32"]
            else:
                step_size = max(self.chunk_elements, 1)
                bounds = [(lo, min(lo + step_size, p.numel())) for lo in range(0, p.numel(), step_size)] or [(0, 0)]
                src, dst = p.grad.view(-1), state["_grad_fp16"].view(-1)
            mine = []
            for lo, hi in bounds:
                if used == len(self._events):
                    self._events.append(torch.cuda.Event())
                if len(bounds) == 1:
                    dst.copy_(src, non_blocking=True)
                else:
                    dst[lo:hi].copy_(src[lo:hi], non_blocking=True)
                stream.record_event(self._events[used])
                mine.append((lo, hi, self._events[used]))
                used += 1
            pieces[p] = mine

        sum_delta = sum_sq_delta = 0.0
        total_numel = 0
        for p, state, group in work:
            beta1, beta2 = group["betas"][0], group["betas"][1]
            if p.dtype == torch.float32:
                pieces[p][0][2].synchronize()
                grad = state["_grad_fp32"].mul_(1.0 / scale)
                if wants_maximize(group):
                    grad = -grad
                lr = 0.0 if state["step"] < self._hold_steps else group["lr"]
                torch_adam_fp32(state["_param_fp32"], grad, state["exp_avg"], state["exp_avg_sq"], state["step"],
                                beta1=beta1, beta2=beta2, lr=lr, weight_decay=group["weight_decay"], eps=group["eps"])
                p.copy_(state["_param_fp32"], non_blocking=True)
                state["step"] += 1
                continue

            state["step"] += 1
            lr = 0.0 if state["step"] < self._hold_steps else group["lr"]
            p32, p16, g16 = state["_param_fp32"].view(-1), state["_param_fp16"].view(-1), state["_grad_fp16"].view(-1)
            m, v = state["exp_avg"].view(-1), state["exp_avg_sq"].view(-1)
            device_p = p.view(-1)
            part_sum = part_sq = 0.0
            for lo, hi, event in pieces[p]:
                event.synchronize()
                grad = g16[lo:hi]
                if wants_maximize(group):
                    grad = -grad
                F.adam_cpu(
                    p32[lo:hi], p16[lo:hi], p._delta_info if self.record_delta else None,
                    grad, m[lo:hi], v[lo:hi],
                    beta1, beta2, group["eps"], lr, scale, group["weight_decay"], state["step"],
                )
                if self.record_delta:
                    part_sum += p._delta_info[2].item()
                    part_sq += p._delta_info[3].item()
                device_p[lo:hi].copy_(p16[lo:hi], non_blocking=True)
            total_numel += p16.numel()
            if self.record_delta:
                if len(pieces[p]) > 1 and p16.numel() > 0:    # statistics of the whole tensor, as one call leaves them
                    mean = part_sum / p16.numel()
                    p._delta_info.copy_(torch.tensor([mean, part_sq / p16.numel() - mean * mean, part_sum, part_sq]))
                sum_delta += part_sum
                sum_sq_delta += part_sq

        if self.record_delta and total_numel > 0:
            self.avg_delta = sum_delta / total_numel
            self.var_delta = sum_sq_delta / total_numel - self.avg_delta ** 2
        return loss

    def get_avg_delta(self):
        return self.avg_delta if self.record_delta else 0

    def get_var_delta(self):
        return self.var_delta if self.record_delta else 0

    def load_state_dict(self, state_dict: dict) -> None:
        """Loads optimizer state onto the host (adam_offload.py:230-327).  A state dict saved
        with ``gather=True`` holds whole tensors: a parameter that carries a partition range
        (``_start_partition`` / ``_end_partition``) takes its slice, a parameter without one
        is left to be initialised lazily at the next step."""
        is_whole = bool(state_dict.get("is_whole", False))

        def convert(param, entry):
            start = getattr(param, "_start_partition", None)
            if is_whole:
                if start is None:
                    return None
                end = param._end_partition
                for name in ("_param_fp32", "exp_avg_sq", "exp_avg"):
                    if name in entry:
                        entry[name] = entry[name][start:end]
            if "_param_fp32" not in entry:
                with torch.no_grad():
                    entry["_param_fp32"] = torch.empty(param.size(), dtype=torch.float32, device="cpu")
                    entry["_param_fp32"].copy_(param)
            for name in ("exp_avg", "exp_avg_sq", "_param_fp32"):
                if name in entry:
                    entry[name] = entry[name].to("cpu").to(torch.float32)
            if param.dtype == torch.float32 and torch.cuda.is_available():
                entry["_param_fp32"] = entry["_param_fp32"].pin_memory()
            self._staging_buffers(param, entry)
            return entry

        remap_loaded_state(self, state_dict, convert)

    def state_dict(self, gather=False) -> dict:
        """Optimizer state with parameters replaced by their running index; only the keys of
        the checkpoint format are kept (no staging buffers).  ``is_whole`` tells the loader
        whether tensors are whole or one partition (adam_offload.py:329-382).  With a single
        GPU the local partition is the whole tensor, so ``gather=True`` involves no exchange."""
        index_of = {}
        packed_groups = []
        next_index = 0
        for group in self.param_groups:
            packed = {k: v for k, v in group.items() if k != "params"}
            for offset, p in enumerate(group["params"]):
                index_of.setdefault(id(p), next_index + offset)
            packed["params"] = [index_of[id(p)] for p in group["params"]]
            next_index += len(packed["params"])
            packed_groups.append(packed)
        packed_state = {}
        for key, entry in self.state.items():
            packed_key = index_of[id(key)] if isinstance(key, torch.Tensor) else key
            packed_state[packed_key] = {name: entry[name] for name in _STATE_KEYS}
        return {"state": packed_state, "param_groups": packed_groups, "is_whole": bool(gather)}

    def zero_grad(self, set_to_none: bool = False):
        super().zero_grad(set_to_none=set_to_none)
