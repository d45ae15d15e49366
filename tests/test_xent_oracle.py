"""Pins oracle/xent_oracle.py (CPU): against torch's own cross-entropy, closed
forms, and torch.autograd for the backward formulas."""
import math

import torch

from oracle import xent_oracle as xo


def _rand(shape, seed):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_forward_matches_torch_cross_entropy():
    x, w = _rand((37, 24), 1), _rand((53, 24), 2)
    y = torch.randint(0, 53, (37,), generator=torch.Generator().manual_seed(3))
    loss, lse = xo.linear_cross_entropy(x, w, y)
    want = torch.nn.functional.cross_entropy(x @ w.t(), y, reduction="none")
    assert torch.allclose(loss, want, atol=1e-12)
    # the reference's oracle: -log(softmax(logits)[label]) (cross_entropy.py:428-435)
    sm = torch.softmax(x @ w.t(), -1).gather(-1, y.view(-1, 1)).squeeze(-1)
    assert torch.allclose(loss, -sm.log(), atol=1e-10)
    assert torch.allclose(lse, (x @ w.t()).exp().sum(-1).log(), atol=1e-10)


def test_closed_forms():
    n = 41
    x = _rand((5, 8), 4)
    y = torch.arange(5)
    loss, lse = xo.linear_cross_entropy(x, torch.zeros(n, 8, dtype=torch.float64), y)
    assert torch.allclose(loss, torch.full((5,), math.log(n), dtype=torch.float64))
    assert torch.allclose(lse, torch.full((5,), math.log(n), dtype=torch.float64))
    # one dominant logit at the label: loss -> 0; at another row: loss -> the gap
    w = torch.zeros(n, 8, dtype=torch.float64)
    xb = torch.zeros(2, 8, dtype=torch.float64)
    xb[:, 0] = 1.0
    w[7, 0] = 60.0
    loss, _ = xo.linear_cross_entropy(xb, w, torch.tensor([7, 3]))
    assert abs(loss[0].item()) < 1e-12 and abs(loss[1].item() - 60.0) < 1e-12
    # a swapped operand (x w instead of x w^T) or a missing target term must fail this
    assert loss[0].item() != loss[1].item()


def test_backward_matches_autograd():
    x, w = _rand((19, 12), 5).requires_grad_(True), _rand((31, 12), 6).requires_grad_(True)
    y = torch.randint(0, 31, (19,), generator=torch.Generator().manual_seed(7))
    go = _rand((19,), 8)
    loss = torch.nn.functional.cross_entropy(x @ w.t(), y, reduction="none")
    loss.backward(go)
    dx, dw = xo.linear_cross_entropy_backward(go, x.detach(), w.detach(), y)
    assert torch.allclose(dx, x.grad, atol=1e-12) and torch.allclose(dw, w.grad, atol=1e-12)
    # rows of dlogits sum to zero => dx is orthogonal to nothing in particular,
    # but sum_n dlogits = 0 makes dw's column sums equal sum_t go_t (p_t - e_y)^T x = ...;
    # check the invariant directly: dlogits rows sum to 0
    p = torch.softmax(x.detach() @ w.detach().t(), -1)
    p[torch.arange(19), y] -= 1
    assert p.sum(-1).abs().max() < 1e-12
