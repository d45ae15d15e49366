"""GPU parity of RMSNorm forward / backward (through the C ABI and the autograd
Function) against the CPU oracle."""
import pytest
import torch

from oracle import rms_oracle as rorc

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.float32):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


# the reference's own test: dim 255, eps 0.1, fp32, 2-D / 3-D / 4-D inputs, rtol = atol = 1e-2
# (common/rms.py:420-470)
@pytest.mark.parametrize("shape", [(1, 255), (16, 128, 255), (8, 3, 28, 255)])
def test_reference_test_shapes_fp32(shape):
    import tritonops_amd as ta

    dim, eps = 255, 1e-1
    mod = ta.RMSNormTriton(dim, eps).cuda()
    with torch.no_grad():
        mod.weight.copy_(_rand((dim,), 3))
    x = _rand(shape, 1)
    dy = _rand(shape, 2)
    xg = x.cuda().requires_grad_(True)
    y = mod(xg)
    want = rorc.rms_norm(x.double(), mod.weight.detach().cpu().double(), eps)
    assert y.shape == x.shape and y.dtype == torch.float32
    assert (y.detach().cpu().double() - want).abs().max() < 1e-5
    y.backward(dy.cuda())
    wdx, wdw = rorc.rms_norm_backward(dy, x, mod.weight.detach().cpu(), eps)
    assert (xg.grad.cpu().double() - wdx).abs().max() < 1e-5
    assert (mod.weight.grad.cpu().double() - wdw).abs().max() < 1e-4 * max(1.0, wdw.abs().max().item())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,dim,wdtype", [(37, 4096, None), (1000, 1024, torch.float32), (5, 8192, None),
                                             (64, 264, None), (3, 16384, None), (129, 100, torch.float32),
                                             (9000, 64, None), (5000, 128, torch.float32), (2500, 2048, None),
                                             (2, 32768, None), (1, 40000, None)])
def test_sixteen_bit_inputs(dtype, rows, dim, wdtype):
    """Every shape of the 16-byte path (a wavefront per row with 1 or 2 chunks
    per lane, a workgroup per row with 1 to 16 chunks per thread; more rows
    than owners, so that owners walk several rows) and the element-wise path
    (dim 100, dim 40000, the backward pass of dim 32768), weight in the
    activation dtype or fp32."""
    import tritonops_amd as ta

    eps = 1e-6
    x, dy = _rand((rows, dim), 4, dtype), _rand((rows, dim), 5, dtype)
    w = (1.0 + 0.1 * _rand((dim,), 6)).to(wdtype or dtype)
    y, rs = ta.rmsnorm_fwd(x.cuda(), w.cuda(), eps)
    want = rorc.rms_norm(x.double(), w.double(), eps)
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    assert y.dtype == dtype
    assert (y.cpu().double() - want).abs().max() <= tol * max(1.0, want.abs().max().item())
    want_r = torch.rsqrt((x.double() ** 2).mean(-1) + eps)
    assert (rs.cpu().double() - want_r).abs().max() <= 1e-5 * want_r.abs().max()
    dx, dw = ta.rmsnorm_bwd(dy.cuda(), x.cuda(), w.cuda(), rs, eps)
    wdx, wdw = rorc.rms_norm_backward(dy, x, w, eps)
    assert dx.dtype == dtype and dw.dtype == w.dtype
    assert (dx.cpu().double() - wdx).abs().max() <= tol * max(1.0, wdx.abs().max().item())
    assert (dw.cpu().double() - wdw).abs().max() <= tol * max(1.0, wdw.abs().max().item())


@pytest.mark.parametrize("rows,dim", [(3000, 512), (7, 4096), (3, 16384), (1300, 1000)])
def test_fp32_inputs(rows, dim):
    import tritonops_amd as ta

    eps = 1e-5
    x, dy = _rand((rows, dim), 14), _rand((rows, dim), 15)
    w = 1.0 + 0.1 * _rand((dim,), 16)
    y, rs = ta.rmsnorm_fwd(x.cuda(), w.cuda(), eps)
    want = rorc.rms_norm(x.double(), w.double(), eps)
    assert (y.cpu().double() - want).abs().max() <= 1e-5 * max(1.0, want.abs().max().item())
    dx, dw = ta.rmsnorm_bwd(dy.cuda(), x.cuda(), w.cuda(), rs, eps)
    wdx, wdw = rorc.rms_norm_backward(dy, x, w, eps)
    assert (dx.cpu().double() - wdx).abs().max() <= 1e-5 * max(1.0, wdx.abs().max().item())
    assert (dw.cpu().double() - wdw).abs().max() <= 1e-4 * max(1.0, wdw.abs().max().item())


def test_strided_rows_and_determinism():
    import tritonops_amd as ta

    big = _rand((200, 3, 512), 7, torch.bfloat16).cuda()
    x = big[:, 1]                                # row stride 1536
    w = torch.ones(512, dtype=torch.bfloat16).cuda()
    y, rs = ta.rmsnorm_fwd(x, w, 1e-6)
    y2, _ = ta.rmsnorm_fwd(x.contiguous(), w, 1e-6)
    assert torch.equal(y, y2)
    dy = _rand((200, 512), 8, torch.bfloat16).cuda()
    a = ta.rmsnorm_bwd(dy, x, w, rs, 1e-6)
    b = ta.rmsnorm_bwd(dy, x, w, rs, 1e-6)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])   # no atomics: bit-reproducible


def test_full_size_properties():
    """Benchmark shape [32768, 4096] bf16: unit RMS of y / w, invariance of y to
    a power-of-two scaling of x (eps = 0), dx orthogonal to x when w = 1."""
    import tritonops_amd as ta

    T, D = 32768, 4096
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn((T, D), device="cuda", generator=g).to(torch.bfloat16)
    dy = torch.randn((T, D), device="cuda", generator=g).to(torch.bfloat16)
    w = torch.ones(D, device="cuda", dtype=torch.float32)
    y, rs = ta.rmsnorm_fwd(x, w, 0.0)
    rms = y.float().pow(2).mean(-1).sqrt()
    assert (rms - 1).abs().max().item() < 3e-3            # bf16 rounding of 4096 outputs
    y4, rs4 = ta.rmsnorm_fwd(x * 4, w, 0.0)
    assert torch.equal(y4, y)                              # exact: scaling by 4 only moves exponents
    assert torch.allclose(rs4 * 4, rs, rtol=1e-6, atol=0)
    dx, dw = ta.rmsnorm_bwd(dy, x, w, rs, 0.0)
    # d/dx of a scale-invariant function is orthogonal to x
    dots = (dx.float() * x.float()).sum(-1)
    scale = (dx.float().norm(dim=-1) * x.float().norm(dim=-1))
    assert (dots.abs() / scale).max().item() < 2e-3
    want_dw = (dy.float() * x.float() * rs.view(-1, 1)).sum(0)
    assert (dw - want_dw).abs().max().item() <= 2e-2 * want_dw.abs().max().item()
