"""Shared helpers of the test-suite: seeded CPU inputs and the parity bar."""
import torch

# Parity bar of this path for 16-bit inputs with fp32 accumulation: max |err|
# against the reference's PyTorch softmax(q k^T scale) v math on the same
# seeded inputs.
TOL = 2e-2
# base-2 log-sum-exp is fp32 on both sides; bf16 inputs are identical, so only
# accumulation order differs
LSE_TOL = 2e-3


def randn(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def rand_lengths(batch, lo, hi, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int32)


def cu_from(lens):
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.as_tensor(lens, dtype=torch.int32), 0)
    return cu


def max_err(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def assert_close(got, want, tol=TOL, what=""):
    e = max_err(got, want)
    assert e <= tol, "%s max abs err %.4g > %.4g" % (what, e, tol)
    assert not torch.isnan(got.float()).any(), "%s has NaN" % what
