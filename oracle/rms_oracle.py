"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's RMSNorm math.

Nothing in the product package (tritonops_amd) may import this module; only
tests/ and bench.py's cpu_baseline leg use it, as the checker.

rms_norm follows RMSNormTorch.forward (common/rms.py:402-417); the backward
formulas are the ones the reference's backward kernel implements
(common/rms.py:199-213).  Pinning (tests/test_rms_oracle.py): the reference's
test holds no stored vectors (it compares against RMSNormTorch on random inputs
at 1e-2, common/rms.py:420-470), so the forward is pinned by closed forms
(constant rows, scale invariance for eps = 0, unit-norm output) and the backward
against torch.autograd and a finite-difference check.
"""
import torch


def rms_norm(x, weight, eps):
    """weight * x / sqrt(mean(x^2, -1) + eps), in x's dtype like the reference module."""
    mean_square = torch.mean(x ** 2, dim=-1, keepdim=True)
    return weight * (x / torch.sqrt(mean_square + eps))


def rms_norm_backward(dy, x, weight, eps):
    """(dx, dweight) in float64:  r = (mean(x^2) + eps)^-1/2,
    dx = dy w r - x r^3 sum_d(dy w x) / D,  dw = sum_rows dy x r."""
    x, dy, w = x.double(), dy.double(), weight.double()
    d = x.shape[-1]
    r = torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    dot = (dy * w * x).sum(-1, keepdim=True)
    dx = dy * w * r - x * r ** 3 * dot / d
    dw = (dy * x * r).reshape(-1, d).sum(0)
    return dx, dw
