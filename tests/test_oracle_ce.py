"""Pins the oracle's cross-entropy restatement against torch (fp32 and float64), closed
forms on tiny rows, and the special cases the reference's constants create."""
import math

import numpy as np
import pytest
import torch

import oracle
from conftest import bits16, from_bits16, ulp_distance16

DTYPES = [("fp16", torch.float16), ("bf16", torch.bfloat16)]


def _case(m, n, dtype, seed, std=2.0, ignore_frac=0.1):
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, n, generator=gen) * std).to(dtype)
    t = torch.randint(0, n, (m,), generator=gen, dtype=torch.int32)
    drop = torch.rand(m, generator=gen) < ignore_frac
    t[drop] = -100
    return x, t


@pytest.mark.parametrize("name,dtype", DTYPES)
@pytest.mark.parametrize("m,n", [(7, 10), (5, 1000), (3, 4099), (2, 32000)])
def test_forward_against_torch(name, dtype, m, n):
    x, t = _case(m, n, dtype, seed=n)
    softmax, loss = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    want_loss = torch.nn.functional.cross_entropy(x.double(), t.long(), ignore_index=-100, reduction="none")
    np.testing.assert_allclose(loss, want_loss.float().numpy(), rtol=1e-5, atol=1e-6)
    assert np.all(loss[t.numpy() == -100] == 0)
    want_soft32 = bits16(torch.softmax(x.float(), -1).to(dtype))
    want_soft64 = bits16(torch.softmax(x.double(), -1).to(dtype))
    assert ulp_distance16(softmax, want_soft32).max() <= 1
    assert ulp_distance16(softmax, want_soft64).max() <= 1
    assert (softmax != want_soft64).mean() < 0.02


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_backward_restates_the_reference_expression(name, dtype):
    """to16((s16 - onehot) * v) on the stored 16-bit softmax (cross_entropy.cu:55-59), and
    through the module's v = w_r / sum(w) it is the textbook gradient to <= 1 ulp off the target."""
    m, n = 6, 515
    x, t = _case(m, n, dtype, seed=1)
    softmax, _ = oracle.ce_forward(bits16(x), t.numpy(), -100, name)
    valid = (t != -100)
    for upstream in (1.0, 256.0, 8192.0):     # |v| stays inside fp16 range with ~5 valid rows
        v = (valid.float() / valid.sum() * upstream).numpy().astype(np.float32)
        grad = softmax.copy()
        oracle.ce_backward_inplace(v, t.numpy(), grad, -100, name)
        s = from_bits16(softmax, dtype).float()
        onehot = torch.zeros(m, n)
        rows = torch.nonzero(valid).flatten()
        onehot[rows, t[rows].long()] = 1
        want = bits16(((s - onehot) * torch.from_numpy(v)[:, None]).to(dtype))
        assert np.array_equal(grad, want)
        xf = x.double().requires_grad_()
        (torch.nn.functional.cross_entropy(xf, t.long(), ignore_index=-100) * upstream).backward()
        # Against the textbook gradient: off-target entries are s16 * v, two roundings, <= 1 ulp.
        # The target entry is (s16 - 1) * v: the rounding of s16 is amplified by the cancellation,
        # so it only agrees to the absolute size of that rounding (half an ulp of s, times v).
        # (Where the stored softmax is an fp16 subnormal its few significant bits are all that is
        # left after scaling up — the reason the reference trains with a loss scale.)
        off = onehot.numpy() == 0
        normal = s.numpy() >= (2.0 ** -14 if dtype == torch.float16 else 2.0 ** -126)
        dist = ulp_distance16(grad, bits16(xf.grad.to(dtype)))
        assert dist[off & normal].max() <= 1
        eps16 = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8
        got = from_bits16(grad, dtype).double()
        err = (got - xf.grad).abs().numpy()[~off]
        bound = (eps16 * torch.from_numpy(v).double()[rows]).numpy() * 1.01 + np.abs(xf.grad.numpy()[~off]) * eps16
        assert np.all(err <= bound)
        assert np.all(grad[~valid.numpy()] == 0)


def test_closed_forms_on_tiny_rows():
    ln = math.log
    # one class: softmax 1, loss log(1 + 1e-10) = 0 in fp32
    s, l = oracle.ce_forward(bits16(torch.tensor([[3.0]]).half()), np.array([0], np.int32), -100, "fp16")
    assert from_bits16(s, torch.float16).item() == 1.0 and abs(l[0]) < 1e-6
    # all-equal row of C classes: softmax 1/C, loss log C
    for c in (2, 3, 8, 1000):
        x = torch.full((1, c), 0.5).half()
        s, l = oracle.ce_forward(bits16(x), np.array([c - 1], np.int32), -100, "fp16")
        assert np.all(s == bits16(torch.tensor(1.0 / c).half()))
        assert abs(l[0] - ln(c)) < 1e-5 * max(1.0, ln(c))
    # two classes: loss = softplus(x1 - x0) for target 0
    x = torch.tensor([[1.5, -0.25]]).half()
    s, l = oracle.ce_forward(bits16(x), np.array([0], np.int32), -100, "fp16")
    assert abs(l[0] - ln(1 + math.exp(-1.75))) < 1e-6
    # target == argmax on a peaked row: loss ~ 0, gradient at the target ~ 0
    x = torch.tensor([[30.0, 0.0, -5.0]]).bfloat16()
    s, l = oracle.ce_forward(bits16(x), np.array([0], np.int32), -100, "bf16")
    assert 0 <= l[0] < 1e-6 and from_bits16(s, torch.bfloat16)[0, 0].item() == 1.0


def test_constants_of_the_reference():
    # all -inf row: M clamps to -1e6 (cross_entropy.cu:22), S = 1e-10, softmax 0, loss finite
    x = torch.full((1, 4), float("-inf")).half()
    s, l = oracle.ce_forward(bits16(x), np.array([-100], np.int32), -100, "fp16")
    assert np.all(s == 0) and l[0] == 0
    # NaN logits are dropped by fmaxf in the maximum but poison the sum
    x = torch.tensor([[float("nan"), 1.0, 2.0]]).half()
    s, l = oracle.ce_forward(bits16(x), np.array([1], np.int32), -100, "fp16")
    assert np.isnan(l[0]) and np.all(np.isnan(from_bits16(s, torch.float16).numpy()))
    # an ignored row still gets its softmax (backward zeroes it through grad_output = 0)
    x, _ = _case(1, 64, torch.float16, seed=2)
    s, l = oracle.ce_forward(bits16(x), np.array([-100], np.int32), -100, "fp16")
    assert l[0] == 0 and abs(from_bits16(s, torch.float16).float().sum().item() - 1) < 1e-2
    # ... and is scaled, not zeroed, if a caller passes a non-zero grad_output for it (:46-60)
    g = s.copy()
    oracle.ce_backward_inplace(np.array([2.0], np.float32), np.array([-100], np.int32), g, -100, "fp16")
    assert np.array_equal(g, bits16((from_bits16(s, torch.float16).float() * 2).half()))


@pytest.mark.parametrize("name,dtype", DTYPES)
def test_sumexp_and_softmax_inplace(name, dtype):
    m, n = 4, 777
    x, _ = _case(m, n, dtype, seed=5)
    mx = x.float().max(-1).values.numpy().astype(np.float32)
    se = oracle.fused_sumexp(bits16(x), mx, name)
    want = torch.exp(x.double() - torch.from_numpy(mx).double()[:, None]).sum(-1)
    np.testing.assert_allclose(se, want.numpy(), rtol=2e-6)
    y = bits16(x)
    oracle.fused_softmax_inplace(y, mx, se, name)
    assert ulp_distance16(y, bits16(torch.softmax(x.double(), -1).to(dtype))).max() <= 1
