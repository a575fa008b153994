"""Pieces shared by the on-device and the offloaded Adam optimizers: hyper-parameter
validation, state-dict re-keying, and the delegation of fp32 parameters to torch."""
from collections import defaultdict
from copy import deepcopy
from itertools import chain

import torch
import torch.optim._functional as _torch_functional

SUPPORTED_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def span(t):
    """(storage address, first byte, byte behind the last, dtype) of a contiguous tensor; None otherwise."""
    if not t.is_contiguous():
        return None
    begin = t.data_ptr()
    return (t.untyped_storage().data_ptr(), begin, begin + t.numel() * t.element_size(), t.dtype)


def span_follows(s, prev):
    """True if the tensor of span `s` starts where the one of span `prev` ends, inside the same storage."""
    return s is not None and prev is not None and s[1] == prev[2] and s[0] == prev[0] and s[3] == prev[3]


def follows(t, prev):
    """True if contiguous tensor `t` starts where contiguous `prev` ends, inside the same storage."""
    return span_follows(span(t), span(prev))


def flat_runs(tensors):
    """Joins tensors that lie back to back in one storage (e.g. the gradients of a ZeRO block's flat
    buffer) into flat 1-D views, in order; tensors that stand alone are passed through unchanged."""
    out, run = [], []

    def close():
        if len(run) == 1:
            out.append(run[0])
        elif run:
            out.append(run[0].as_strided((sum(t.numel() for t in run),), (1,)))
        run.clear()

    last = None
    for t in tensors:
        here = span(t)                     # every tensor is looked at once, not once from either side
        if run and not span_follows(here, last):
            close()
        run.append(t)
        last = here
    close()
    return out


def validate_hyper(lr, betas, eps, weight_decay):
    """ValueError texts follow torch.optim.Adam, as bmtrain/optim/adam.py:30-39 does."""
    if not 0.0 <= lr:
        raise ValueError("Invalid learning rate: {}".format(lr))
    if not 0.0 <= eps:
        raise ValueError("Invalid epsilon value: {}".format(eps))
    for index, beta in enumerate(betas[:2]):
        if not 0.0 <= beta < 1.0:
            raise ValueError("Invalid beta parameter at index {}: {}".format(index, beta))
    if not 0.0 <= weight_decay:
        raise ValueError("Invalid weight_decay value: {}".format(weight_decay))


def check_grad(p):
    if p.grad.is_sparse:
        raise RuntimeError("Adam does not support sparse gradients, please consider SparseAdam instead")
    if p.dtype not in SUPPORTED_DTYPES:
        raise RuntimeError("Adam only supports fp32, fp16 and bf16 gradients")


def wants_maximize(group) -> bool:
    return group.get("maximize", False) is True


def torch_adam_fp32(param, grad, exp_avg, exp_avg_sq, step, *, beta1, beta2, lr, weight_decay, eps):
    """fp32 parameters are not a kernel target: like the reference (adam.py:114-142,
    adam_offload.py:156-187) they go through torch's functional Adam — coupled L2 decay,
    bias correction at ``step + 1`` — on whatever device the tensors live."""
    _torch_functional.adam(
        [param], [grad], [exp_avg], [exp_avg_sq], [], [torch.tensor(float(step))],
        amsgrad=False, beta1=beta1, beta2=beta2, lr=lr, weight_decay=weight_decay, eps=eps, maximize=False,
    )


def remap_loaded_state(optimizer, state_dict, convert):
    """Common skeleton of ``load_state_dict``: validates group shapes, maps saved
    parameter ids onto the live parameters, lets ``convert(param, entry)`` cast /
    complete each per-parameter entry (it may return None to drop it), and installs
    the result.  Entries that belong to no live parameter are kept untouched."""
    state_dict = deepcopy(state_dict)
    groups = optimizer.param_groups
    saved_groups = state_dict["param_groups"]
    if len(groups) != len(saved_groups):
        raise ValueError("loaded state dict has a different number of parameter groups")
    for live, saved in zip(groups, saved_groups):
        if len(live["params"]) != len(saved["params"]):
            raise ValueError(
                "loaded state dict contains a parameter group that doesn't match the size of optimizer's group"
            )
    live_by_saved_id = dict(zip(
        chain.from_iterable(g["params"] for g in saved_groups),
        chain.from_iterable(g["params"] for g in groups),
    ))
    new_state = defaultdict(dict)
    for key, entry in state_dict["state"].items():
        if key not in live_by_saved_id:
            new_state[key] = entry
            continue
        param = live_by_saved_id[key]
        entry = convert(param, entry)
        if entry is not None:
            new_state[param] = entry
    new_groups = []
    for live, saved in zip(groups, saved_groups):
        saved["params"] = live["params"]
        new_groups.append(saved)
    optimizer.__setstate__({"state": new_state, "param_groups": new_groups})
    return state_dict
