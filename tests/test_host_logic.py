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


def test_runs_of_adjacent_tensors():
    """Which parameters the fused optimizer steps as one flat run: all five arrays back to back in one
    storage each, same step count and learning rate."""
    from bmtrain_amd.optim.adam import _adjacent_runs
    from bmtrain_amd.optim._base import flat_runs, follows as _follows
    flat = torch.zeros(100, dtype=torch.bfloat16)
    a, b, c = flat[0:10], flat[10:40].view(5, 6), flat[41:50]
    assert _follows(b, a) and not _follows(c, b) and not _follows(a, b)
    assert not _follows(flat[10:40:2], a)                                  # not contiguous
    assert not _follows(torch.zeros(30, dtype=torch.bfloat16), a)          # another storage
    assert not _follows(flat.view(torch.float16)[10:40], a)                # another dtype
    joined = flat_runs([a, b, c, torch.zeros(3, dtype=torch.bfloat16), flat[50:60], flat[60:100]])
    assert [t.numel() for t in joined] == [40, 9, 3, 50] and joined[0].data_ptr() == flat.data_ptr()
    assert joined[1] is c and flat_runs([]) == []

    def item(lo, hi, step=3, lr=1e-3, bufs={}):
        for name, dtype in (("p32", torch.float32), ("p", torch.bfloat16), ("g", torch.bfloat16), ("m", torch.float32),
                            ("v", torch.float32)):
            bufs.setdefault(name, torch.zeros(100, dtype=dtype))
        return tuple(bufs[k][lo:hi] for k in ("p32", "p", "g", "m", "v")) + (step, lr)

    work = [item(0, 10), item(10, 30), item(30, 31), item(32, 40), item(40, 50, step=4), item(50, 60, step=4, lr=0.0),
            item(60, 70, step=4, lr=0.0)]
    runs = _adjacent_runs(work)
    assert [len(r) for r in runs] == [3, 1, 1, 2]
    # one array out of line is enough to split
    stray = list(item(70, 80, step=4, lr=0.0))
    stray[2] = torch.zeros(10, dtype=torch.bfloat16)
    assert [len(r) for r in _adjacent_runs(work + [tuple(stray)])] == [3, 1, 1, 2, 1]
    assert _adjacent_runs([]) == []


def test_a_planned_step_changes_nothing_until_it_is_taken():
    """AdamOptimizer.plan_step on fp32 parameters (the path that runs without a GPU): planning touches neither
    parameters nor state nor step counts, no plan is made for a parameter without state when told not to create it,
    and taking the plan equals step()."""
    import bmtrain_amd as bmt
    torch.manual_seed(3)

    def build():
        torch.manual_seed(3)
        ps = [torch.nn.Parameter(torch.randn(7)), torch.nn.Parameter(torch.randn(3, 4))]
        for q in ps:
            q.grad = torch.randn_like(q)
        return ps, bmt.optim.AdamOptimizer([{"params": ps[:1], "lr": 1e-2}, {"params": ps[1:], "lr": 1e-3, "weight_decay": 0.1}])
    pa, oa = build()
    pb, ob = build()
    assert oa.plan_step(scale=2.0, create_state=False) is None and all(len(oa.state[q]) == 0 for q in pa)
    oa.step(scale=2.0)
    ob.step(scale=2.0)
    before = [q.detach().clone() for q in pa]
    plan = oa.plan_step(scale=2.0, create_state=False)
    assert plan is not None
    assert all(torch.equal(q.detach(), b) for q, b in zip(pa, before)) and all(oa.state[q]["step"] == 1 for q in pa)
    oa.step(scale=2.0, _plan=plan)
    ob.step(scale=2.0)
    for q, r in zip(pa, pb):
        assert torch.equal(q.detach(), r.detach()) and oa.state[q]["step"] == ob.state[r]["step"] == 2
        assert torch.equal(oa.state[q]["exp_avg"], ob.state[r]["exp_avg"])
        assert torch.equal(oa.state[q]["exp_avg_sq"], ob.state[r]["exp_avg_sq"])


def test_manager_unscales_the_gradients_of_a_foreign_optimizer():
    """An optimizer that is not one of this package's gets its gradients divided by the loss scale before its own step
    (optim_manager.py:23-27, :141-143): gradients that are views into one buffer are divided by one launch, with the
    values of the per-parameter division; parameters that need no gradient are left alone."""
    import bmtrain_amd as bmt
    from bmtrain_amd.optim.optim_manager import grad_rescale
    flat_p, flat_g = torch.randn(30), torch.randn(30) * 64
    ps = [torch.nn.Parameter(flat_p[0:10]), torch.nn.Parameter(flat_p[10:24].view(2, 7)), torch.nn.Parameter(torch.randn(5)),
          torch.nn.Parameter(torch.randn(4), requires_grad=False)]
    ps[0].grad, ps[1].grad, ps[2].grad = flat_g[0:10], flat_g[10:24].view(2, 7), torch.randn(5) * 64
    ps[3].grad = torch.ones(4)
    want = [p.grad.clone() / 64 for p in ps[:3]]
    untouched = flat_g[24:].clone()
    grad_rescale([{"params": ps}], 64)
    assert all(torch.equal(p.grad, w) for p, w in zip(ps, want)) and torch.equal(ps[3].grad, torch.ones(4))
    assert torch.equal(flat_g[24:], untouched)
    opt = torch.optim.SGD([p for p in ps if p.requires_grad], lr=0.5)
    manager = bmt.optim.OptimManager(loss_scale=None)
    manager.add_optimizer(opt)
    before = [p.detach().clone() for p in ps[:3]]
    manager.step()                                # no loss scaling: the foreign optimizer simply steps
    assert all(torch.equal(p.detach(), b - 0.5 * w) for p, b, w in zip(ps, before, want))


def test_state_of_adjacent_parameters_is_allocated_back_to_back():
    flat = torch.zeros(64, dtype=torch.bfloat16)
    params = [torch.nn.Parameter(flat[0:16].view(4, 4)), torch.nn.Parameter(flat[16:24]), torch.nn.Parameter(flat[30:40]),
              torch.nn.Parameter(torch.zeros(5))]
    opt = bmt.optim.AdamOptimizer(params, lr=1e-3)
    opt._init_states(params)
    s = [opt.state[p] for p in params]
    assert s[0]["exp_avg"].shape == (4, 4) and s[0]["_param_fp32"].dtype == torch.float32
    for key in ("exp_avg", "exp_avg_sq", "_param_fp32"):
        assert s[1][key].data_ptr() == s[0][key].data_ptr() + 16 * 4
        assert s[2][key].untyped_storage().data_ptr() != s[0][key].untyped_storage().data_ptr()
    assert "_param_fp32" not in s[3] and s[3]["exp_avg"].dtype == torch.float32
    opt.merge_adjacent = False
    other = [torch.nn.Parameter(flat[40:48]), torch.nn.Parameter(flat[48:56])]
    opt._init_states(other)
    assert opt.state[other[1]]["exp_avg"].untyped_storage().data_ptr() != opt.state[other[0]]["exp_avg"].untyped_storage().data_ptr()
