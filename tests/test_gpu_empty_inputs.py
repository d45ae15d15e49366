"""Empty inputs through every Python entry point on the GPU: nothing is
launched, shapes and dtypes of the results are still right."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_rmsnorm_and_cross_entropy_with_no_rows():
    import tritonops_amd as ta

    x = torch.empty((0, 256), device="cuda", dtype=torch.bfloat16)
    w = torch.ones(256, device="cuda", dtype=torch.bfloat16)
    y, rs = ta.rmsnorm_fwd(x, w, 1e-6)
    assert y.shape == (0, 256) and rs.shape == (0,)
    dx, dw = ta.rmsnorm_bwd(x, x, w, rs, 1e-6)
    assert dx.shape == (0, 256) and dw.shape == (256,) and torch.count_nonzero(dw) == 0

    wl = torch.randn((100, 256), device="cuda").to(torch.bfloat16)
    labels = torch.empty((0,), device="cuda", dtype=torch.int64)
    loss, lse = ta.cross_entropy_fused_fwd(x, wl, labels)
    assert loss.shape == (0,) and lse.shape == (0,) and loss.dtype == torch.float32
    gx, gw = ta.cross_entropy_fused_bwd(torch.empty((0,), device="cuda"), x, wl, labels, lse)
    assert gx.shape == (0, 256) and gw.shape == (100, 256) and torch.count_nonzero(gw) == 0


def test_attention_with_empty_sequences_only():
    import tritonops_amd as ta

    q = torch.zeros((1, 0, 4, 64), device="cuda", dtype=torch.bfloat16)
    k = torch.zeros((1, 0, 2, 64), device="cuda", dtype=torch.bfloat16)
    cu = torch.zeros(3, device="cuda", dtype=torch.int32)          # two sequences of length 0
    o, lse = ta.flash_attention(q, k, k, cu, return_lse=True, max_seq_len=0)
    assert o.shape == q.shape and lse.shape == (1, 0, 4)
    qd = torch.randn((2, 4, 64), device="cuda").to(torch.bfloat16)
    kd = torch.zeros((2, 64, 2, 64), device="cuda", dtype=torch.bfloat16)
    od = ta.flash_attention_decoding(qd, kd, kd, cu)
    assert od.shape == qd.shape and torch.count_nonzero(od) == 0
