"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's fused linear +
cross-entropy math.

Nothing in the product package (tritonops_amd) may import this module; only
tests/ and bench.py's cpu_baseline leg use it, as the checker.

linear_cross_entropy follows the reference's own torch oracle `cross_entropy`
(cross_entropy_triton/cross_entropy.py:428-435: -log(softmax(h @ W^T)[label]))
written as logsumexp - target logit, which is what its kernels compute
(:100-183, :337-339); the backward formulas are the ones of its backward kernel
and launcher (:255-266, :369-415).  Pinning (tests/test_xent_oracle.py): the
reference's test holds no stored vectors (random inputs against
nn.CrossEntropyLoss at 1e-1, :438-513), so the forward is pinned against
torch.nn.functional.cross_entropy and closed forms (w = 0 gives log N, a
dominant logit gives ~0), the backward against torch.autograd.
"""
import torch


def linear_cross_entropy(x, w, y):
    """(loss, lse) in float64: logits = x @ w^T, lse = logsumexp(logits, -1),
    loss = lse - logits[t, y[t]]."""
    logits = x.double() @ w.double().t()
    lse = torch.logsumexp(logits, dim=-1)
    tgt = logits.gather(-1, y.reshape(-1, 1).long()).squeeze(-1)
    return lse - tgt, lse


def linear_cross_entropy_backward(grad_o, x, w, y):
    """(dx, dw) in float64: dlogits = grad_o (softmax(logits) - onehot(y)),
    dx = dlogits @ w, dw = dlogits^T @ x."""
    x, w = x.double(), w.double()
    logits = x @ w.t()
    p = torch.softmax(logits, dim=-1)
    p[torch.arange(x.shape[0]), y.reshape(-1).long()] -= 1.0
    dl = grad_o.double().reshape(-1, 1) * p
    return dl @ w, dl.t() @ x
