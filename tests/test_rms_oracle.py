"""Pins oracle/rms_oracle.py (CPU only)."""
import torch

from oracle import rms_oracle as rorc


def test_forward_closed_forms():
    w = torch.tensor([1.0, 2.0, -3.0, 0.5], dtype=torch.float64)
    # constant row c: mean square c^2 -> y = w * sign(c) for eps = 0
    x = torch.full((2, 4), -2.5, dtype=torch.float64)
    assert torch.allclose(rorc.rms_norm(x, w, 0.0), -w.expand(2, 4))
    # eps = 0: invariant under scaling of x; output / w has unit mean square
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 4, generator=g, dtype=torch.float64)
    y = rorc.rms_norm(x, w, 0.0)
    assert torch.allclose(rorc.rms_norm(7.0 * x, w, 0.0), y)
    assert torch.allclose(((y / w) ** 2).mean(-1), torch.ones(5, dtype=torch.float64))
    # one row by hand: x = (3, 4), eps = 0.5 -> mean square 12.5, rms sqrt(13)
    y = rorc.rms_norm(torch.tensor([[3.0, 4.0]], dtype=torch.float64), torch.tensor([2.0, 1.0], dtype=torch.float64), 0.5)
    assert torch.allclose(y, torch.tensor([[6.0, 4.0]], dtype=torch.float64) / 13 ** 0.5)


def test_backward_matches_autograd_and_finite_differences():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 7, 255, generator=g, dtype=torch.float64, requires_grad=True)   # the reference's odd dim
    w = torch.randn(255, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(3, 7, 255, generator=g, dtype=torch.float64)
    eps = 1e-1
    rorc.rms_norm(x, w, eps).backward(dy)
    dx, dw = rorc.rms_norm_backward(dy, x.detach(), w.detach(), eps)
    assert (dx - x.grad).abs().max() < 1e-12
    assert (dw - w.grad).abs().max() < 1e-11
    # finite difference of sum(y * dy) along a random direction in x
    u = torch.randn(3, 7, 255, generator=g, dtype=torch.float64)
    h = 1e-6
    f = lambda xx: (rorc.rms_norm(xx, w.detach(), eps) * dy).sum()
    fd = (f(x.detach() + h * u) - f(x.detach() - h * u)) / (2 * h)
    assert abs(fd - (dx * u).sum()) < 1e-6 * max(1.0, abs(fd))
