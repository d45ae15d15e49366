"""GPU parity of the fused linear + cross-entropy (through the C ABI and the
autograd Function) against the CPU oracle."""
import math

import pytest
import torch

from oracle import xent_oracle as xo

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.float32, scale=1.0):
    return (scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))).to(dtype)


def _labels(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed))


def _check_fwd(x, w, y, tol):
    import tritonops_amd as ta

    loss, lse = ta.cross_entropy_fused_fwd(x.cuda(), w.cuda(), y.cuda())
    want_loss, want_lse = xo.linear_cross_entropy(x, w, y)
    assert loss.dtype == torch.float32 and loss.shape == (x.shape[0],)
    assert (lse.cpu().double() - want_lse).abs().max() <= tol
    assert (loss.cpu().double() - want_loss).abs().max() <= tol
    return loss, lse


# the reference's own test: T 139, vocab 279, hidden 256, bf16, uniform [0, 1) inputs
# (cross_entropy.py:438-513, tolerance 1e-1 there)
def test_reference_test_shape():
    import tritonops_amd as ta

    g = torch.Generator().manual_seed(42)
    h = torch.rand((139, 256), generator=g).to(torch.bfloat16)
    w = torch.rand((279, 256), generator=g).to(torch.bfloat16)
    y = torch.randint(0, 279, (139,), generator=g)
    _check_fwd(h, w, y, 2e-2)
    hg, wg = h.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    loss = ta.cross_entropy_fused_triton(hg, wg, y.cuda().view(-1, 1))
    loss.mean().backward()
    dx, dw = xo.linear_cross_entropy_backward(torch.full((139,), 1.0 / 139), h, w, y)
    assert hg.grad.dtype == torch.bfloat16 and wg.grad.dtype == torch.bfloat16
    assert (hg.grad.cpu().double() - dx).abs().max() <= 2e-2 * max(1.0, dx.abs().max().item())
    assert (wg.grad.cpu().double() - dw).abs().max() <= 2e-2 * max(1.0, dw.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,D,N", [
    (1, 128, 1),          # one token, one class: loss 0
    (7, 128, 255),        # a single, partial vocabulary tile
    (300, 256, 1000),     # two token tiles (the second partial), ranges of one tile
    (256, 384, 4096 + 37),  # full token tile; the last vocabulary tile is partial
    (1000, 512, 5000),    # several token tiles x several ranges
    (513, 200, 777),      # hidden size padded to 256 by the host side
    (64, 128, 70000),     # many tiles per range
])
def test_forward_shapes(dtype, T, D, N):
    x = _rand((T, D), 1, dtype)
    w = _rand((N, D), 2, dtype, scale=1.0 / math.sqrt(D) * 3.0)
    y = _labels(T, N, 3)
    _check_fwd(x, w, y, 2e-2 if dtype == torch.bfloat16 else 5e-3)


def test_labels_int32_out_of_range_and_strided_rows():
    import tritonops_amd as ta

    T, D, N = 200, 256, 1500
    big = _rand((T, 2 * D), 4, torch.bfloat16)
    x = big[:, :D]                                   # row stride 2 D
    w = _rand((N, D), 5, torch.bfloat16, scale=0.2)
    y = _labels(T, N, 6)
    l64, lse64 = ta.cross_entropy_fused_fwd(x.cuda(), w.cuda(), y.cuda())
    l32, lse32 = ta.cross_entropy_fused_fwd(x.contiguous().cuda(), w.cuda(), y.to(torch.int32).cuda())
    assert torch.equal(l64, l32) and torch.equal(lse64, lse32)
    want, _ = xo.linear_cross_entropy(x, w, y)
    assert (l64.cpu().double() - want).abs().max() <= 2e-2
    y2 = y.clone()
    y2[::3] = -100                                   # no target logit: loss = lse
    l2, lse2 = ta.cross_entropy_fused_fwd(x.cuda(), w.cuda(), y2.cuda())
    assert torch.equal(lse2, lse64)
    assert torch.equal(l2[::3], lse2[::3]) and torch.equal(l2[1::3], l64[1::3])


def test_large_logits_stay_finite():
    # logits of +-200: exp overflows fp32 without the running maximum
    T, D, N = 130, 128, 600
    x = torch.zeros((T, D), dtype=torch.bfloat16)
    x[:, 0] = 10.0
    w = torch.zeros((N, D), dtype=torch.bfloat16)
    w[:, 0] = torch.linspace(-20, 20, N).to(torch.bfloat16)
    y = _labels(T, N, 7)
    loss, lse = _check_fwd(x, w, y, 5e-2)
    assert torch.isfinite(loss).all() and torch.isfinite(lse).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_backward_against_oracle(dtype):
    import tritonops_amd as ta

    T, D, N = 700, 256, 3001
    x = _rand((T, D), 8, dtype)
    w = _rand((N, D), 9, dtype, scale=0.15)
    y = _labels(T, N, 10)
    go = _rand((T,), 11)
    xg, wg = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    loss = ta.cross_entropy_fused_triton(xg, wg, y.cuda())
    loss.backward(go.cuda())
    dx, dw = xo.linear_cross_entropy_backward(go, x, w, y)
    tol = 3e-2 if dtype == torch.bfloat16 else 5e-3
    assert (xg.grad.cpu().double() - dx).abs().max() <= tol * max(1.0, dx.abs().max().item())
    assert (wg.grad.cpu().double() - dw).abs().max() <= tol * max(1.0, dw.abs().max().item())
    # several row blocks give the same gradients as one (up to the library GEMM's choice of kernel per shape)
    _, lse = ta.cross_entropy_fused_fwd(x.cuda(), w.cuda(), y.cuda())
    a = ta.cross_entropy_fused_bwd(go.cuda(), x.cuda(), w.cuda(), y.cuda(), lse)
    b = ta.cross_entropy_fused_bwd(go.cuda(), x.cuda(), w.cuda(), y.cuda(), lse, rows_per_block=256)
    assert (a[0].float() - b[0].float()).abs().max() <= tol * max(1.0, dx.abs().max().item())
    assert (a[1].float() - b[1].float()).abs().max() <= tol * max(1.0, dw.abs().max().item())


def test_dlogits_kernel_rows_and_tails():
    import tritonops_amd as ta

    rows, N = 33, 2048 + 8 + 3                       # full segment, a vector tail and a scalar tail
    logits = _rand((rows, N), 12, torch.bfloat16)
    y = _labels(rows, N, 13)
    lse = torch.logsumexp(logits.float(), -1)
    go = _rand((rows,), 14)
    want = go.view(-1, 1).double() * (torch.exp(logits.double() - lse.double().view(-1, 1))
                                      - torch.nn.functional.one_hot(y, N).double())
    got = ta.cross_entropy_dlogits_(logits.clone().cuda(), lse.cuda(), go.cuda(), y.cuda())
    assert (got.cpu().double() - want).abs().max() <= 1e-2 * max(1.0, want.abs().max().item())
    # unaligned row stride: element-wise path
    wide = torch.zeros((rows, N + 1), dtype=torch.bfloat16)
    wide[:, :N] = logits
    got2 = ta.cross_entropy_dlogits_(wide.cuda()[:, :N], lse.cuda(), go.cuda(), y.cuda())
    assert torch.equal(got2.cpu(), got.cpu())


def test_full_size_is_invariant_to_the_launch_shape():
    """Benchmark shape (8192 tokens, hidden 4096, vocabulary 128256): the loss of
    a token does not depend on how tokens and vocabulary are dealt to
    workgroups.  8192 tokens run as 32 token tiles x 8 vocabulary ranges, a
    slice of 1024 tokens as 4 x 64, a slice of 100 as 1 x 256."""
    import tritonops_amd as ta

    T, D, N = 8192, 4096, 128256
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((T, D), device="cuda", generator=g).to(torch.bfloat16)
    w = (torch.randn((N, D), device="cuda", generator=g) * D ** -0.5).to(torch.bfloat16)
    y = torch.randint(0, N, (T,), device="cuda", generator=g)
    loss, lse = ta.cross_entropy_fused_fwd(x, w, y)
    assert torch.isfinite(loss).all() and (loss > 0).all()
    # N(0,1) logits: lse = log N + 1/2 up to sampling noise
    assert abs(lse.mean().item() - (math.log(N) + 0.5)) < 0.05
    for lo, hi in ((3072, 4096), (8000, 8100)):
        l2, s2 = ta.cross_entropy_fused_fwd(x[lo:hi], w, y[lo:hi])
        assert (l2 - loss[lo:hi]).abs().max().item() <= 1e-4
        assert (s2 - lse[lo:hi]).abs().max().item() <= 1e-4
    # against fp32 torch math on a slice of tokens (same bf16 inputs, full vocabulary)
    logits = x[:64].float() @ w.float().t()
    want = torch.logsumexp(logits, -1) - logits.gather(-1, y[:64].view(-1, 1)).squeeze(-1)
    assert (loss[:64] - want).abs().max().item() <= 2e-3


@pytest.mark.parametrize("T,D,N", [(300, 256, 1000), (257, 128, 4096 + 37), (64, 384, 263)])
def test_dlogits_from_the_gemm_kernel(T, D, N):
    """The gradient epilogue against float64 math, with logits large enough
    (|logit| up to ~60) that rounding them to bf16 first would be visible:
    partial token / vocabulary tiles, N not a multiple of 8 (element-wise stores)."""
    import tritonops_amd as ta

    x = _rand((T, D), 21, torch.bfloat16)
    w = _rand((N, D), 22, torch.bfloat16, scale=1.2)
    y = _labels(T, N, 23)
    go = _rand((T,), 24)
    logits = x.double() @ w.double().t()
    lse = torch.logsumexp(logits, -1)
    want = go.double().view(-1, 1) * (torch.exp(logits - lse.view(-1, 1)) - torch.nn.functional.one_hot(y, N).double())
    got = ta.cross_entropy_dlogits(x.cuda(), w.cuda(), y.cuda(), lse.float().cuda(), go.cuda())
    assert got.shape == (T, N) and got.dtype == torch.bfloat16
    assert (got.cpu().double() - want).abs().max() <= 1e-2 * max(1.0, want.abs().max().item())
    # rows sum to zero up to the rounding of the stored values
    assert got.float().sum(-1).abs().max().item() <= 0.1 * go.abs().max().item()
