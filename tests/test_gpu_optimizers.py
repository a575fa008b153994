"""Optimizer classes and the loss-scale manager on the GPU, shaped like the reference's
tests/test_optim.py and the overflow handling of bmtrain/optim/optim_manager.py."""
import copy

import numpy as np
import pytest
import torch

import bmtrain_amd as bmt

pytestmark = pytest.mark.gpu


class TestModule(torch.nn.Module):
    __test__ = False

    def __init__(self):
        super().__init__()
        self.fc1 = torch.nn.Linear(128, 128, bias=False)
        self.fc2 = torch.nn.Linear(128, 128)
        self.fc3 = torch.nn.Linear(128, 128)
        self.fc4 = torch.nn.Linear(128, 128)
        self.fc5 = torch.nn.Linear(128, 128)
        self.param = torch.nn.Parameter(torch.empty(1237))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_five_way_agreement(dtype):
    """tests/test_optim.py:24-85: fused (16-bit), offload (16-bit), torch Adam (fp32), fused (fp32),
    offload (fp32) on identical gradients, lr = 1, loss scale 4, 100 steps."""
    torch.manual_seed(0)
    models = [TestModule() for _ in range(5)]
    state = models[0].state_dict()
    for k in state:
        state[k] = torch.randn_like(state[k])
    for mdl in models:
        mdl.load_state_dict(state)
    model1, model2 = models[0].cuda().to(dtype), models[1].cuda().to(dtype)
    model3, model4, model5 = (mdl.cuda() for mdl in models[2:])
    opt1 = bmt.optim.AdamOptimizer(model1.parameters(), lr=1)
    opt2 = bmt.optim.AdamOffloadOptimizer(model2.parameters(), lr=1)
    opt3 = torch.optim.Adam(model3.parameters(), lr=1)
    opt4 = bmt.optim.AdamOptimizer(model4.parameters(), lr=1)
    opt5 = bmt.optim.AdamOffloadOptimizer(model5.parameters(), lr=1)
    manager = bmt.optim.OptimManager(loss_scale=4)
    for opt in (opt1, opt2, opt3, opt4, opt5):
        manager.add_optimizer(opt)
    for _ in range(100):
        manager.zero_grad()
        for p1, p2, p3, p4, p5 in zip(*(mdl.parameters() for mdl in (model1, model2, model3, model4, model5))):
            grad = torch.randn_like(p1)
            p1.grad = grad.to(dtype)
            p2.grad = grad.to(dtype)
            p3.grad = grad.float()
            p4.grad = grad.float()
            p5.grad = grad.float()
        manager.step()
        torch.cuda.synchronize()
        for p1, p2, p3, p4, p5 in zip(*(mdl.parameters() for mdl in (model1, model2, model3, model4, model5))):
            assert torch.abs(p1 - p2).max().item() < 1
            assert torch.abs(p1 - p3).max().item() < 1
            assert torch.abs(p2 - p3).max().item() < 1
            assert torch.abs(p3 - p4).max().item() == 0
            assert torch.abs(p3 - p5).max().item() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_and_offload_agree_closely(dtype):
    """Same expression on both sides (bf16: identical fp32 state, copy differs by rounding mode)."""
    torch.manual_seed(1)
    a = torch.nn.Parameter((torch.randn(10007) * 0.02).cuda().to(dtype))
    b = torch.nn.Parameter(a.detach().clone())
    opt_a = bmt.optim.AdamOptimizer([a], lr=1e-3, weight_decay=0.01)
    opt_b = bmt.optim.AdamOffloadOptimizer([b], lr=1e-3, weight_decay=0.01, record_delta=True)
    for _ in range(5):
        g = (torch.randn(10007, device="cuda") * 1e-3 * 64).to(dtype)
        a.grad = g.clone(); b.grad = g.clone()
        opt_a.step(scale=64); opt_b.step(scale=64)
        torch.cuda.synchronize()
    pa = opt_a.state[a]["_param_fp32"].cpu()
    pb = opt_b.state[b]["_param_fp32"]
    if dtype == torch.bfloat16:
        assert torch.equal(pa, pb)
        assert torch.equal(opt_a.state[a]["exp_avg_sq"].cpu(), opt_b.state[b]["exp_avg_sq"])
    else:   # the fused fp16 path keeps its first moment in fp16 (2^-11 relative rounding per step)
        assert (pa - pb).abs().max() <= 1e-4 * pb.abs().max()
    assert opt_b.get_avg_delta() != 0 and opt_b.get_var_delta() > 0
    with pytest.raises(NotImplementedError):
        bmt.optim.AdamOptimizer.get_avg_delta()


def _host_simd_level():
    have = set()
    with open("/proc/cpuinfo") as f:
        for line in f:
            if line.startswith("flags"):
                have = set(line.split(":", 1)[1].split())
                break
    narrow = {"avx", "fma", "f16c"} <= have
    return 2 if ("avx512f" in have and narrow) else (1 if narrow else 0)


def test_offload_optimizer_on_the_reference_cpu_configuration():
    """The configuration the reference's CPU path is quoted on, exactly, through AdamOffloadOptimizer on this box:
    N = 2^24 fp32 master parameters ~ N(0, 0.02), fp16 gradients ~ N(0, 1e-3) * 1024, m = v = 0, lr 1e-3, betas
    (0.9, 0.999), eps 1e-8, weight decay 0.01, loss scale 1024, 10 steps, fixed seed.  fp32 state on the host and the
    fp16 copy on the device must equal, bit for bit, the oracle's restatement of adam_cpu_fp16_launcher
    (adam_cpu.hpp:504-533) run at this host's SIMD level and thread count over the same pieces the optimizer cuts
    the tensor into (which elements fall to the vector or the scalar tree depends on both, adam_cpu.hpp:332-351)."""
    import os
    import oracle
    from conftest import bits16, f32_bits
    n = 1 << 24
    gen = torch.Generator().manual_seed(0)
    master = torch.randn(n, generator=gen) * 0.02
    param = torch.nn.Parameter(master.half().cuda())
    opt = bmt.optim.AdamOffloadOptimizer([param], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
    # the optimizer derives its fp32 master from the 16-bit parameter; the configuration states the master itself
    with torch.no_grad():
        opt._init_state(param)["_param_fp32"].copy_(master)
    po, mo, vo = master.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    ho = np.zeros(n, np.uint16)
    threads, level = len(os.sched_getaffinity(0)), _host_simd_level()
    piece = opt.chunk_elements
    for step in range(1, 11):
        g = (torch.randn(n, generator=gen) * 1e-3 * 1024).half()
        param.grad = g.cuda()
        opt.step(scale=1024)
        bc1, bc2 = oracle.bias_corrections(0.9, 0.999, step)
        gb = bits16(g)
        for lo in range(0, n, piece):
            hi = min(lo + piece, n)
            oracle.adam_cpu_fp16(po[lo:hi], ho[lo:hi], None, gb[lo:hi], mo[lo:hi], vo[lo:hi], 0.9, 0.999, 1e-8, 1e-3, 1024.0,
                                 0.01, bc1, bc2, level, threads)
    torch.cuda.synchronize()
    state = opt.state[param]
    assert state["step"] == 10
    assert np.array_equal(f32_bits(state["_param_fp32"].numpy()), f32_bits(po))
    assert np.array_equal(f32_bits(state["exp_avg"].numpy()), f32_bits(mo))
    assert np.array_equal(f32_bits(state["exp_avg_sq"].numpy()), f32_bits(vo))
    assert np.array_equal(bits16(param.detach()), ho)
    # and the update is a real one: ten steps of lr 1e-3 with random gradients move a parameter by a few 1e-3
    moved = (state["_param_fp32"] - master).abs()
    assert 1e-3 < moved.mean().item() < 1e-2


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_offload_in_pieces_equals_offload_in_one_call(dtype):
    """A tensor cut into pieces (each with its own copy event) ends in the state one host call over the
    whole tensor leaves: bit for bit for bf16; for fp16 to within the host's two expression trees
    (which elements take the vector lanes depends on where a call's range is cut)."""
    torch.manual_seed(3)
    n = 1_000_003
    whole = torch.nn.Parameter((torch.randn(n) * 0.02).cuda().to(dtype))
    cut = torch.nn.Parameter(whole.detach().clone())
    opt_w = bmt.optim.AdamOffloadOptimizer([whole], lr=1e-3, weight_decay=0.01, record_delta=True, chunk_elements=1 << 40)
    opt_c = bmt.optim.AdamOffloadOptimizer([cut], lr=1e-3, weight_decay=0.01, record_delta=True, chunk_elements=300_000)
    for _ in range(3):
        g = (torch.randn(n, device="cuda") * 1e-3 * 8).to(dtype)
        whole.grad = g.clone(); cut.grad = g.clone()
        opt_w.step(scale=8); opt_c.step(scale=8)
        torch.cuda.synchronize()
    sw, sc = opt_w.state[whole], opt_c.state[cut]
    assert sw["step"] == sc["step"] == 3
    if dtype == torch.bfloat16:
        for key in ("_param_fp32", "exp_avg", "exp_avg_sq"):
            assert torch.equal(sw[key], sc[key]), key
        assert torch.equal(whole.detach(), cut.detach())
    else:
        for key in ("_param_fp32", "exp_avg", "exp_avg_sq"):
            torch.testing.assert_close(sc[key], sw[key], rtol=1e-6, atol=1e-9)
        assert ((whole.detach().float() - cut.detach().float()).abs() <= whole.detach().float().abs() * 2.0 ** -10).all()
    assert abs(opt_c.get_avg_delta() - opt_w.get_avg_delta()) <= 1e-5 * abs(opt_w.get_avg_delta()) + 1e-9
    assert abs(opt_c.get_var_delta() - opt_w.get_var_delta()) <= 1e-4 * opt_w.get_var_delta()
    torch.testing.assert_close(cut._delta_info, whole._delta_info, rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_parameters_in_flat_storage_are_stepped_as_runs(dtype):
    """Parameters that are views into one flat buffer (with gradients in another, as ZeRO blocks keep them)
    get back-to-back state and one launch per run; results equal one launch per tensor bit for bit.  A
    parameter without a gradient splits the run; a loaded state dict (separate tensors) ends the merging
    without changing results."""
    torch.manual_seed(5)
    shapes = [(64, 4096), (4096,), (128, 128), (7,), (300001,), (33, 5)]
    sizes = [int(np.prod(sh)) for sh in shapes]
    total = sum(sizes)
    flat_p = (torch.randn(total) * 0.02).to(dtype).cuda()
    flat_g = torch.zeros(total, dtype=dtype, device="cuda")
    merged, single = [], []
    lo = 0
    for sh, size in zip(shapes, sizes):
        q = torch.nn.Parameter(flat_p[lo:lo + size].view(sh))
        q.grad = flat_g[lo:lo + size].view(sh)
        merged.append(q)
        single.append(torch.nn.Parameter(flat_p[lo:lo + size].view(sh).clone()))
        lo += size
    opt_m = bmt.optim.AdamOptimizer(merged, lr=1e-3, weight_decay=0.01)
    opt_s = bmt.optim.AdamOptimizer(single, lr=1e-3, weight_decay=0.01)
    opt_s.merge_adjacent = False

    def step(skip=None):
        g = (torch.randn(total, device="cuda") * 1e-3 * 16).to(dtype)
        flat_g.copy_(g)
        lo = 0
        for k, size in enumerate(sizes):
            single[k].grad = None if k == skip else g[lo:lo + size].view(shapes[k]).clone()
            if k == skip:
                saved, merged[k].grad = merged[k].grad, None
            lo += size
        opt_m.step(scale=16); opt_s.step(scale=16)
        if skip is not None:
            merged[skip].grad = saved

    def same():
        for a, b in zip(merged, single):
            assert torch.equal(a.detach().view(torch.int16), b.detach().view(torch.int16))
            if len(opt_s.state[b]):
                for key in ("_param_fp32", "exp_avg", "exp_avg_sq"):
                    x, y = opt_m.state[a][key], opt_s.state[b][key]
                    assert torch.equal(x.view(torch.int16 if x.element_size() == 2 else torch.int32),
                                       y.view(torch.int16 if y.element_size() == 2 else torch.int32)), key
                assert opt_m.state[a]["step"] == opt_s.state[b]["step"]

    step(); step()
    same()
    storages = {opt_m.state[q]["exp_avg_sq"].untyped_storage().data_ptr() for q in merged}
    assert len(storages) == 1                               # one flat state buffer for the whole run
    step(skip=2)                                            # steps now differ inside the run: it splits
    same()
    step()
    same()
    opt_m.load_state_dict(copy.deepcopy(opt_m.state_dict()))   # separate tensors from here on
    step(); same()


def test_overflow_check_and_grad_norm_over_flat_gradient_storage():
    """Gradients that are views into one buffer are scanned as one run: same verdicts and norm as tensor by tensor."""
    from bmtrain_amd.optim.optim_manager import check_overflow
    torch.manual_seed(6)
    sizes = [4096, 7, 100003, 64 * 64]
    flat_g = (torch.randn(sum(sizes), device="cuda") * 64).bfloat16()
    params, lo = [], 0
    for size in sizes:
        q = torch.nn.Parameter(torch.zeros(size, dtype=torch.bfloat16, device="cuda"))
        q.grad = flat_g[lo:lo + size]
        params.append(q)
        lo += size
    lone = torch.nn.Parameter(torch.zeros(33, dtype=torch.float16, device="cuda"))
    lone.grad = torch.ones(33, dtype=torch.float16, device="cuda")
    groups = [{"params": params + [lone]}]
    check_overflow(groups)                                   # finite: no exception
    manager = bmt.optim.OptimManager(loss_scale=64)
    want = torch.cat([flat_g.float(), lone.grad.float()]).norm() / 64
    got = manager.clip_grad_norm(groups, max_norm=1e9)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=0)
    before = flat_g.clone()
    got = manager.clip_grad_norm(groups, max_norm=0.25)      # clips: the whole run is scaled by one launch
    coef = (0.25 * 64) / (want * 64 + 1e-6)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=0)
    assert torch.equal(flat_g, (before.float() * coef).bfloat16()) or \
        ((flat_g.float() - before.float() * coef).abs() <= before.float().abs() * coef * 2.0 ** -7).all()
    assert torch.equal(lone.grad, (torch.ones(33, device="cuda") * coef).half())
    flat_g[4096 + 7 + 50000] = float("nan")                  # inside the third tensor of the run
    with pytest.raises(OverflowError):
        check_overflow(groups)
    flat_g[4096 + 7 + 50000] = 0
    lone.grad[32] = float("inf")
    with pytest.raises(OverflowError):
        check_overflow(groups)


def test_step_reuses_the_overflow_verdict_of_the_clipping_pass(monkeypatch):
    """reuse_overflow_verdict=True: clip_grad_norm reads the 16-bit gradients once for norm and overflow flag;
    step() does not scan gradients nobody has written to since, and does scan again after an in-place write."""
    import bmtrain_amd.optim.optim_manager as om
    calls = []
    real, real_multi = om.has_inf_nan, om.grad_stats_multi
    monkeypatch.setattr(om, "has_inf_nan", lambda g, flag: (calls.append(g.numel()), real(g, flag))[1])

    def counted_multi(grads, sumsq, flag):          # several separate gradients share one launch
        if sumsq is None:
            calls.extend(g.numel() for g in grads)
        return real_multi(grads, sumsq, flag)
    monkeypatch.setattr(om, "grad_stats_multi", counted_multi)
    torch.manual_seed(8)
    ps = [torch.nn.Parameter(torch.randn(s, device="cuda").bfloat16()) for s in (5000, 77, 4096)]
    opt = bmt.optim.AdamOptimizer(ps, lr=1e-3)
    manager = bmt.optim.OptimManager(loss_scale=64, loss_scale_steps=1000, reuse_overflow_verdict=True)
    manager.add_optimizer(opt)

    def grads():
        for p in ps:
            p.grad = (torch.randn_like(p.float()) * 64).bfloat16()

    grads()
    manager.clip_grad_norm(opt.param_groups, max_norm=0.5)          # clips: gradients are scaled in place
    manager.step()
    assert calls == [] and opt.state[ps[0]]["step"] == 1             # verdict reused, step taken
    grads()
    manager.step()
    assert len(calls) == 3                                           # no clipping pass: scanned as usual
    calls.clear(); grads()
    manager.clip_grad_norm(opt.param_groups, max_norm=1e9)
    ps[1].grad.mul_(2.0)                                             # somebody writes to a gradient
    manager.step()
    assert len(calls) == 3 and opt.state[ps[0]]["step"] == 3
    calls.clear(); grads()
    ps[2].grad[100] = float("nan")
    manager.clip_grad_norm(opt.param_groups, max_norm=1.0)
    manager.step()                                                   # overflow seen by the clipping pass
    assert calls == [] and manager.loss_scale == 32 and opt.state[ps[0]]["step"] == 3
    calls.clear(); grads()
    manager.clip_grad_norm([{"params": ps[:2]}], max_norm=1.0)      # a subset only: the rest must be scanned
    ps[2].grad[5] = float("inf")
    manager.step()
    assert len(calls) == 3 and manager.loss_scale == 16


def test_overflow_is_scanned_again_by_default_and_whenever_a_runtime_is_registered(monkeypatch):
    """A write through `.data` does not move autograd's version counter, which is how collectives and BMTrain's own
    code touch gradients.  By default step() therefore scans every gradient itself, whatever clip_grad_norm saw;
    with reuse switched on, a registered communicator or copy stream switches it off again."""
    import bmtrain_amd.optim.optim_manager as om
    torch.manual_seed(18)
    ps = [torch.nn.Parameter(torch.randn(s, device="cuda").bfloat16()) for s in (3000, 500)]
    opt = bmt.optim.AdamOptimizer(ps, lr=1e-3)

    def grads():
        for p in ps:
            p.grad = (torch.randn_like(p.float()) * 64).bfloat16()

    manager = bmt.optim.OptimManager(loss_scale=64, loss_scale_steps=1000)        # default: no reuse
    manager.add_optimizer(opt)
    grads()
    manager.clip_grad_norm(opt.param_groups, max_norm=1e9)
    version = ps[0].grad._version
    ps[0].grad.data[7] = float("inf")                                   # raw write: same version counter
    assert ps[0].grad._version == version
    manager.step()
    assert manager.loss_scale == 32 and "step" not in opt.state.get(ps[0], {})      # seen, step skipped

    trusting = bmt.optim.OptimManager(loss_scale=64, loss_scale_steps=1000, reuse_overflow_verdict=True)
    trusting.add_optimizer(opt)
    monkeypatch.setitem(om.config, "comm", object())                    # a distributed runtime is present
    grads()
    trusting.clip_grad_norm(opt.param_groups, max_norm=1e9)
    ps[1].grad.data[3] = float("nan")
    trusting.step()
    assert trusting.loss_scale == 32


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_clip_grad_norm_with_a_parameter_that_has_no_gradient(dtype):
    """Frozen or unused parameters have `grad is None`; they count as zeros for the norm (optim_manager.py:176-181)
    and are passed over by clipping, overflow check and step."""
    torch.manual_seed(19)
    ps = [torch.nn.Parameter((torch.randn(s, device="cuda") * 0.02).to(dtype)) for s in (4096, 300, 1000)]
    opt = bmt.optim.AdamOptimizer(ps, lr=1e-3)
    for reuse in (False, True):
        manager = bmt.optim.OptimManager(loss_scale=8, reuse_overflow_verdict=reuse)
        manager.add_optimizer(opt)
        ps[0].grad = (torch.randn(4096, device="cuda") * 8).to(dtype)
        ps[1].grad = None
        ps[2].grad = (torch.randn(1000, device="cuda") * 8).to(dtype)
        want = torch.sqrt(ps[0].grad.float().norm() ** 2 + ps[2].grad.float().norm() ** 2) / 8
        got = manager.clip_grad_norm(opt.param_groups, max_norm=0.1)
        assert abs(got.item() - want.item()) <= 1e-5 * want.item()
        before = ps[1].detach().clone()
        manager.step()
        assert torch.equal(ps[1].detach(), before) and len(opt.state[ps[1]]) == 0
    assert opt.state[ps[0]]["step"] == 2
    none_at_all = [torch.nn.Parameter(torch.zeros(10, device="cuda", dtype=dtype))]
    manager = bmt.optim.OptimManager(loss_scale=8)
    assert manager.clip_grad_norm([{"params": none_at_all}], max_norm=1.0).item() == 0.0
    assert manager.clip_grad_norm([{"params": none_at_all}], max_norm=1.0, norm_type="inf").item() == 0.0


def test_deferred_clipping_is_taken_only_when_one_call_covers_everything():
    """Two optimizers clipped separately (each call with its own max_norm), a subset of the parameters, two calls in
    a row, a backward pass between clipping and step: in all of these one deferred factor for every optimizer would
    be wrong, so the manager clips eagerly and the result equals that of a manager without defer_clip, bit for bit."""
    dtype = torch.bfloat16

    def build(defer):
        torch.manual_seed(21)
        a = [torch.nn.Parameter((torch.randn(s, device="cuda") * 0.02).to(dtype)) for s in (5000, 128)]
        b = [torch.nn.Parameter((torch.randn(s, device="cuda") * 0.02).to(dtype)) for s in (2048, 77)]
        oa, ob = bmt.optim.AdamOptimizer(a, lr=1e-3), bmt.optim.AdamOptimizer(b, lr=2e-3, weight_decay=0.01)
        man = bmt.optim.OptimManager(loss_scale=16, defer_clip=defer)
        man.add_optimizer(oa); man.add_optimizer(ob)
        return a, b, oa, ob, man

    def same(x, y):
        return all(torch.equal(p.detach().view(torch.int16), q.detach().view(torch.int16)) for p, q in zip(x, y))

    ea, eb, eoa, eob, eman = build(False)
    da, db, doa, dob, dman = build(True)
    scenarios = ["per optimizer", "subset", "twice", "all at once"]
    for step, scenario in enumerate(scenarios):
        torch.manual_seed(100 + step)
        for p, q in zip(ea + eb, da + db):
            g = (torch.randn(p.numel(), device="cuda") * 16).to(dtype)
            p.grad, q.grad = g.clone(), g.clone()
        for man, oa, ob, a in ((eman, eoa, eob, ea), (dman, doa, dob, da)):
            if scenario == "per optimizer":
                man.clip_grad_norm(oa.param_groups, max_norm=0.3)
                man.clip_grad_norm(ob.param_groups, max_norm=0.05)
            elif scenario == "subset":
                man.clip_grad_norm([{"params": a[:1]}], max_norm=0.2)
            elif scenario == "twice":
                man.clip_grad_norm(oa.param_groups + ob.param_groups, max_norm=0.5)
                man.clip_grad_norm(oa.param_groups + ob.param_groups, max_norm=0.1)
            else:
                man.clip_grad_norm(oa.param_groups + ob.param_groups, max_norm=0.4)
        if scenario == "all at once":          # the one case that is deferred: gradients untouched, same update
            assert dman._pending_clip is not None and not same([p.grad for p in ea], [q.grad for q in da])
        else:
            assert dman._pending_clip is None and same([p.grad for p in ea + eb], [q.grad for q in da + db]), scenario
        eman.step(); dman.step()
        assert same(ea + eb, da + db), scenario
        for p, q in zip(ea, da):
            assert torch.equal(eoa.state[p]["exp_avg_sq"], doa.state[q]["exp_avg_sq"]), scenario


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_clipping_factor_as_a_number_gives_the_bits_of_the_tensor_form(dtype):
    """The reference clips with `g.mul_(clip_coef)`, clip_coef a 0-dim fp32 tensor on the device; torch then
    rounds the factor to the gradient's dtype before multiplying.  The manager passes that rounded factor as a
    Python number (a much faster kernel): the products must be the same bits."""
    torch.manual_seed(13)
    g = (torch.randn(1 << 18, device="cuda") * 50).to(dtype)
    for value in (0.7368421173, 1.0 / 3.0, 0.001234567, 0.99999):
        coef = torch.tensor(value, device="cuda")
        assert torch.equal(g.clone().mul_(coef), g.clone().mul_(float(coef.to(dtype))))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_deferred_clipping_updates_parameters_like_eager_clipping(dtype):
    """defer_clip: the clipping factor is applied inside the fused step.  Parameters and optimizer state end up
    bit-identical to eager clipping (in-place multiplication of the gradients, then the step); the gradients
    keep their unclipped values.  Mixed model: flat storage, separate tensors, an fp32 parameter."""
    torch.manual_seed(12)
    sizes = [4096 * 8, 77, 300001]
    def build():
        flat_p = (torch.randn(sum(sizes)) * 0.02).to(dtype).cuda()
        flat_g = torch.zeros(sum(sizes), dtype=dtype, device="cuda")
        ps, lo = [], 0
        for size in sizes:
            q = torch.nn.Parameter(flat_p[lo:lo + size]); q.grad = flat_g[lo:lo + size]
            ps.append(q); lo += size
        ps.append(torch.nn.Parameter((torch.randn(5000) * 0.02).to(dtype).cuda()))
        ps.append(torch.nn.Parameter((torch.randn(300) * 0.02).cuda()))                # fp32
        opt = bmt.optim.AdamOptimizer(ps, lr=1e-3, weight_decay=0.01)
        return ps, opt
    state = torch.get_rng_state()
    ps_e, opt_e = build()
    torch.set_rng_state(state)
    ps_d, opt_d = build()
    man_e = bmt.optim.OptimManager(loss_scale=128); man_e.add_optimizer(opt_e)
    man_d = bmt.optim.OptimManager(loss_scale=128, defer_clip=True); man_d.add_optimizer(opt_d)
    for step in range(3):
        gs = [(torch.randn(p.numel(), device="cuda") * 128).to(p.dtype).view(p.shape) for p in ps_e]
        for p, q, g in zip(ps_e, ps_d, gs):
            if p.grad is None:
                p.grad, q.grad = g.clone(), g.clone()
            else:
                p.grad.copy_(g); q.grad.copy_(g)
        max_norm = 0.5 if step != 1 else 1e9                         # step 1 does not clip
        n_e = man_e.clip_grad_norm(opt_e.param_groups, max_norm)
        n_d = man_d.clip_grad_norm(opt_d.param_groups, max_norm)
        assert torch.equal(n_e, n_d)
        if step != 1:
            assert not torch.equal(ps_e[0].grad, gs[0]) and torch.equal(ps_d[0].grad, gs[0])   # eager scaled, deferred not
        man_e.step(); man_d.step()
        for p, q in zip(ps_e, ps_d):
            assert torch.equal(p.detach().view(torch.uint8), q.detach().view(torch.uint8)), step
            for key in ("exp_avg", "exp_avg_sq", "_param_fp32"):
                if key in opt_e.state[p]:
                    assert torch.equal(opt_e.state[p][key].view(torch.uint8), opt_d.state[q][key].view(torch.uint8)), (step, key)


def test_overflow_skips_the_step_and_halves_the_scale():
    torch.manual_seed(2)
    p = torch.nn.Parameter(torch.randn(1000, device="cuda").half())
    opt = bmt.optim.AdamOptimizer([p], lr=1e-2)
    manager = bmt.optim.OptimManager(loss_scale=1024, loss_scale_steps=2)
    manager.add_optimizer(opt)
    # a clean step creates state (moments stored multiplied by the scale)
    p.grad = (torch.randn(1000, device="cuda") * 1024 * 1e-3).half()
    manager.step()
    before = p.detach().clone()
    m_before = opt.state[p]["exp_avg"].clone()
    v_before = opt.state[p]["exp_avg_sq"].clone()
    assert opt.state[p]["step"] == 1
    # overflow: skipped, scale halved, fp16 moments rescaled, grads zeroed
    p.grad = (torch.randn(1000, device="cuda")).half()
    p.grad[17] = float("inf")
    manager.step()
    assert manager.loss_scale == 512 and opt.state[p]["step"] == 1
    assert torch.equal(p.detach(), before)
    assert torch.equal(opt.state[p]["exp_avg"], m_before * 0.5)
    assert torch.equal(opt.state[p]["exp_avg_sq"], v_before * 0.5)
    assert p.grad.count_nonzero() == 0
    # NaN too
    p.grad[3] = float("nan")
    manager.step()
    assert manager.loss_scale == 256
    # two clean steps grow it again
    for _ in range(2):
        p.grad = (torch.randn(1000, device="cuda") * 1e-3).half()
        manager.step()
    assert manager.loss_scale == 512 and opt.state[p]["step"] == 3
    # never below min_loss_scale
    manager2 = bmt.optim.OptimManager(loss_scale=1, min_loss_scale=1)
    manager2.add_optimizer(opt)
    p.grad = torch.full_like(p, float("nan"))
    manager2.step()
    assert manager2.loss_scale == 1
    # fp32 parameters are not scanned (optim_manager.py:15)
    q = torch.nn.Parameter(torch.randn(10, device="cuda"))
    q.grad = torch.full_like(q, float("inf"))
    bmt.optim.optim_manager.check_overflow([{"params": [q]}])
    p.grad = torch.full_like(p, float("nan"))
    with pytest.raises(OverflowError):
        bmt.optim.optim_manager.check_overflow([{"params": [p]}])


def test_step_prepared_during_the_overflow_scan_is_the_step():
    """OptimManager.step() lets the optimizers lay out their launches (plan_step) while the overflow scan runs and only
    makes the calls once the flag has been read.  Through the manager and through optimizer.step() alone: the same
    bits in parameters and state over several steps, for two parameter groups with their own hyper-parameters,
    mixed fp32 / fp16 / bf16 parameters, hold_steps and maximize.  An overflow on the very first step leaves the
    optimizer without state (no master copy of parameters that a caller may still load), and an overflow later
    changes nothing but the moments' scale."""
    def build():
        torch.manual_seed(21)
        ps = [torch.nn.Parameter(torch.randn(n, device="cuda").to(dt)) for n, dt in
              ((5000, torch.bfloat16), (77, torch.float16), (4096, torch.bfloat16), (300, torch.float32), (1 << 16, torch.float16))]
        opt = bmt.optim.AdamOptimizer([{"params": ps[:2], "lr": 1e-2, "weight_decay": 0.1, "betas": (0.8, 0.9)},
                                       {"params": ps[2:], "lr": 3e-3, "eps": 1e-6, "maximize": True}], hold_steps=2)
        return ps, opt
    pa, oa = build()
    pb, ob = build()
    manager = bmt.optim.OptimManager(loss_scale=64.0, loss_scale_steps=10 ** 9)
    manager.add_optimizer(oa)
    # first step overflows: nothing is created
    for p in pa:
        p.grad = torch.full_like(p, float("inf") if p.dtype != torch.float32 else 0.0)
    manager.step()
    assert manager.loss_scale == 32.0 and all(len(oa.state[p]) == 0 for p in pa)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for k in range(5):
        grads = [(torch.randn(p.shape, device="cuda", generator=gen) * 32.0 * 1e-2).to(p.dtype) for p in pa]
        for p, q, g in zip(pa, pb, grads):
            p.grad, q.grad = g.clone(), g.clone()
        if k == 3:          # an overflow in between: neither side steps; the moments kept in fp16 follow the new scale
            pa[1].grad[5] = float("nan")
            manager.step()
            assert manager.loss_scale == 16.0
            ob._on_justify_scale(32.0, 16.0)
            continue
        manager.step()
        ob.step(scale=manager.loss_scale)
    for p, q in zip(pa, pb):
        assert torch.equal(p.detach().view(torch.uint8), q.detach().view(torch.uint8))
        assert oa.state[p]["step"] == ob.state[q]["step"] == 4
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(oa.state[p][key].view(torch.uint8), ob.state[q][key].view(torch.uint8)), key
    # a plan is refused, not improvised, while a parameter has no state yet
    pc, oc = build()
    for p in pc:
        p.grad = torch.zeros_like(p)
    assert oc.plan_step(scale=1.0, create_state=False) is None and all(len(oc.state[p]) == 0 for p in pc)


def test_hold_steps_and_maximize():
    p = torch.nn.Parameter(torch.ones(64, device="cuda").bfloat16())
    opt = bmt.optim.AdamOptimizer([p], lr=0.1, hold_steps=3)
    for i in range(1, 5):
        p.grad = torch.ones_like(p)
        opt.step()
        # lr is 0 while step < hold_steps, tested after the increment (adam.py:145,155)
        assert (p.detach().float() == 1).all() == (i < 3)
    q = torch.nn.Parameter(torch.zeros(64, device="cuda").bfloat16())
    opt = bmt.optim.AdamOptimizer([{"params": [q], "maximize": True}], lr=0.1)
    q.grad = torch.ones_like(q)
    opt.step()
    assert (q.detach() > 0).all()


def test_state_dict_round_trip_resumes_exactly():
    """tests/test_optim_state.py: a reloaded optimizer continues bit-identically."""
    torch.manual_seed(4)
    for cls in (bmt.optim.AdamOptimizer, bmt.optim.AdamOffloadOptimizer):
        for dtype in (torch.float16, torch.bfloat16, torch.float32):
            p = torch.nn.Parameter((torch.randn(513, device="cuda") * 0.1).to(dtype))
            q = torch.nn.Parameter(p.detach().clone())
            opt_p, opt_q = cls([p], lr=1e-2, weight_decay=0.1), cls([q], lr=1e-2, weight_decay=0.1)
            mp, mq = bmt.optim.OptimManager(loss_scale=8), bmt.optim.OptimManager(loss_scale=2)
            mp.add_optimizer(opt_p); mq.add_optimizer(opt_q)
            grads = [(torch.randn(513, device="cuda") * 8).to(dtype) for _ in range(4)]
            for g in grads[:2]:
                p.grad = g.clone(); mp.step()
            saved = copy.deepcopy(mp.state_dict())
            assert set(saved["optimizers"][0]["state"][0]) >= {"step", "exp_avg", "exp_avg_sq"}
            if dtype != torch.float32 or cls is bmt.optim.AdamOffloadOptimizer:
                assert "_param_fp32" in saved["optimizers"][0]["state"][0]
            q.data.copy_(p.data)
            mq.load_state_dict(saved)
            assert mq.loss_scale == 8
            st = opt_q.state[q]
            if cls is bmt.optim.AdamOptimizer:
                assert st["exp_avg"].dtype == (torch.float16 if dtype == torch.float16 else torch.float32)
                assert st["exp_avg_sq"].dtype == torch.float32 and st["exp_avg"].is_cuda
            else:
                assert not st["exp_avg"].is_cuda
            for g in grads[2:]:
                p.grad = g.clone(); q.grad = g.clone()
                mp.step(); mq.step()
            torch.cuda.synchronize()
            assert torch.equal(p.detach(), q.detach()), (cls.__name__, dtype)


def test_clip_grad_norm():
    torch.manual_seed(5)
    ps = [torch.nn.Parameter(torch.randn(100, device="cuda").half()) for _ in range(3)]
    manager = bmt.optim.OptimManager(loss_scale=16)
    for p in ps:
        p.grad = (torch.randn(100, device="cuda") * 16).half()
    want = torch.cat([p.grad.float() for p in ps]).norm() / 16
    got = manager.clip_grad_norm([{"params": ps}], max_norm=1.0)
    torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-3)
    after = torch.cat([p.grad.float() for p in ps]).norm() / 16
    assert abs(after.item() - 1.0) < 1e-2


def test_constructor_validation():
    p = [torch.nn.Parameter(torch.zeros(1))]
    for cls in (bmt.optim.AdamOptimizer, bmt.optim.AdamOffloadOptimizer):
        for kw in (dict(lr=-1), dict(eps=-1), dict(betas=(1.0, 0.9)), dict(betas=(0.9, -0.1)), dict(weight_decay=-1)):
            with pytest.raises(ValueError):
                cls(p, **kw)
    q = torch.nn.Parameter(torch.zeros(4, device="cuda", dtype=torch.float64))
    q.grad = torch.zeros_like(q)
    with pytest.raises(RuntimeError):
        bmt.optim.AdamOptimizer([q]).step()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_batched_and_per_tensor_stepping_agree_exactly(dtype):
    torch.manual_seed(6)
    a, b = TestModule(), TestModule()
    state = {k: torch.randn_like(v) for k, v in a.state_dict().items()}
    a.load_state_dict(state); b.load_state_dict(state)
    a, b = a.cuda().to(dtype), b.cuda().to(dtype)
    opt_a = bmt.optim.AdamOptimizer(a.parameters(), lr=1e-2, weight_decay=0.1)
    opt_b = bmt.optim.AdamOptimizer(b.parameters(), lr=1e-2, weight_decay=0.1)
    opt_b.batch_launches = False
    for _ in range(5):
        for pa, pb in zip(a.parameters(), b.parameters()):
            g = torch.randn_like(pa)
            pa.grad = g.clone(); pb.grad = g.clone()
        opt_a.step(scale=2); opt_b.step(scale=2)
    for pa, pb in zip(a.parameters(), b.parameters()):
        assert torch.equal(pa, pb)
        assert torch.equal(opt_a.state[pa]["_param_fp32"], opt_b.state[pb]["_param_fp32"])
        assert torch.equal(opt_a.state[pa]["exp_avg_sq"], opt_b.state[pb]["exp_avg_sq"])
