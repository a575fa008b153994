"""Host-side behaviour that needs no GPU: hyper-parameter validation, state-dict re-keying,
dtype dispatch errors, the manager's scale bookkeeping."""
import pytest
import torch

import bmtrain_amd as bmt
from bmtrain_amd.loss import _function as LF
from bmtrain_amd.optim import _function as OF


def test_validation_messages():
    p = [torch.nn.Parameter(torch.zeros(1))]
    with pytest.raises(ValueError, match="Invalid learning rate"):
        bmt.optim.AdamOptimizer(p, lr=-0.1)
    with pytest.raises(ValueError, match="Invalid epsilon"):
        bmt.optim.AdamOptimizer(p, eps=-1e-8)
    with pytest.raises(ValueError, match="index 0"):
        bmt.optim.AdamOffloadOptimizer(p, betas=(1.0, 0.999))
    with pytest.raises(ValueError, match="index 1"):
        bmt.optim.AdamOffloadOptimizer(p, betas=(0.9, 1.0))
    with pytest.raises(ValueError, match="weight_decay"):
        bmt.optim.AdamOptimizer(p, weight_decay=-1)
    assert bmt.optim.AdamOptimizer._bmtrain_optimizer and bmt.optim.AdamOffloadOptimizer._bmtrain_optimizer


def test_gpu_entry_points_refuse_cpu_tensors():
    x = torch.zeros(8, dtype=torch.float16)
    with pytest.raises(AssertionError):
        LF.has_inf_nan(x, torch.zeros(1, dtype=torch.uint8))
    with pytest.raises(AssertionError):
        OF.adam_fp16(torch.zeros(8), x, x, x, torch.zeros(8), 0.9, 0.999, 1e-8, 1e-3, 1.0, 0.0, 1)
    with pytest.raises(AssertionError):
        LF.cross_entropy_forward(2, 4, x.view(2, 4), torch.zeros(2, dtype=torch.int32), x.view(2, 4).clone(),
                                 torch.zeros(2), -100)


def test_adam_load_state_dict_casts_and_rebuilds_master():
    p = torch.nn.Parameter(torch.randn(6).half())
    opt = bmt.optim.AdamOptimizer([p], lr=1e-3)
    saved = {
        "state": {0: {"step": 3, "exp_avg": torch.ones(6, dtype=torch.float32), "exp_avg_sq": torch.ones(6, dtype=torch.float64)}},
        "param_groups": [{"lr": 5e-4, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.0, "params": [0]}],
    }
    opt.load_state_dict(saved)
    st = opt.state[p]
    assert st["step"] == 3 and st["exp_avg"].dtype == torch.float16 and st["exp_avg_sq"].dtype == torch.float32
    assert torch.equal(st["_param_fp32"], p.detach().float())
    assert opt.param_groups[0]["lr"] == 5e-4 and opt.param_groups[0]["params"][0] is p
    with pytest.raises(ValueError, match="different number"):
        opt.load_state_dict({"state": {}, "param_groups": []})
    with pytest.raises(ValueError, match="doesn't match the size"):
        opt.load_state_dict({"state": {}, "param_groups": [{"params": [0, 1]}]})


def test_offload_state_dict_layout():
    p = torch.nn.Parameter(torch.randn(6).bfloat16())
    q = torch.nn.Parameter(torch.randn(3))
    opt = bmt.optim.AdamOffloadOptimizer([{"params": [p]}, {"params": [q], "lr": 0.5}], lr=1e-3)
    sd = opt.state_dict()
    assert sd["is_whole"] is False and sd["state"] == {}
    assert [g["params"] for g in sd["param_groups"]] == [[0], [1]]
    saved = {
        "state": {0: {"step": 2, "exp_avg": torch.ones(6), "exp_avg_sq": torch.ones(6)}},
        "param_groups": sd["param_groups"], "is_whole": False,
    }
    opt.load_state_dict(saved)
    st = opt.state[p]
    assert torch.equal(st["_param_fp32"], p.detach().float())
    assert st["_param_fp16"].dtype == torch.bfloat16 and st["_grad_fp16"].shape == p.shape
    out = opt.state_dict()
    assert set(out["state"][0]) == {"step", "exp_avg", "exp_avg_sq", "_param_fp32"}
    # whole-tensor checkpoints: a parameter with a partition range takes its slice,
    # one without is dropped and re-initialised lazily
    p._start_partition, p._end_partition = 2, 8
    whole = {"state": {0: {"step": 1, "exp_avg": torch.arange(10.0), "exp_avg_sq": torch.arange(10.0),
                           "_param_fp32": torch.arange(10.0)},
                       1: {"step": 1, "exp_avg": torch.zeros(3), "exp_avg_sq": torch.zeros(3)}},
             "param_groups": sd["param_groups"], "is_whole": True}
    opt.load_state_dict(whole)
    assert torch.equal(opt.state[p]["exp_avg"], torch.arange(2.0, 8.0)) and q not in opt.state


def test_manager_scale_bookkeeping():
    m = bmt.optim.OptimManager(loss_scale=1024, loss_scale_factor=0.5)
    assert m.loss_scale_factor == 2 and m.loss_scale_enabled and m.grad_scale == 1
    assert bmt.optim.OptimManager().loss_scale == 1 and not bmt.optim.OptimManager().loss_scale_enabled

    class Probe:
        calls = []
        def _on_justify_scale(self, old, new):
            self.calls.append((old, new))
    m.add_optimizer(Probe())
    m._justify_scale(512)
    assert Probe.calls == [(1024, 512)] and m.loss_scale == 512 and m.steps_since_last_scale == 0
    loss = torch.tensor(2.0)
    assert m.scale_loss(loss).item() == 1024.0
    assert bmt.optim.OptimManager(loss_scale=8, grad_scale=4).scale_loss(loss).item() == 4.0
