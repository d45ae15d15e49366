"""Head dims the kernels are not built for (the reference pads any head_dim to
the next power of two, flash_attn_triton.py:612; its tutorials run d = 16 and
32, tutorial/4.3.multi_head_attention.py:157-158): the Python side pads with
zero columns and the results must still match the oracle."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import TOL, assert_close, cu_from, randn

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("D", [16, 32, 80, 120])
@pytest.mark.parametrize("causal", [False, True])
def test_batched_forward(D, causal):
    import tritonops_amd as ta

    shape = (2, 3, 150, D)
    q, k, v = (randn(shape, s) for s in (1, 2, 3))
    want = (orc.causal_attention if causal else orc.full_attention)(q.float(), k.float(), v.float())
    got, lse = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
    assert got.shape == shape and got.is_contiguous() and lse.shape == shape[:3]
    assert_close(got, want, TOL, "o")


@pytest.mark.parametrize("D", [32, 80])
def test_packed_forward_backward_and_decode(D):
    import tritonops_amd as ta

    lens = [70, 1, 130]
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v, do = randn((1, T, 4, D), 4), randn((1, T, 2, D), 5), randn((1, T, 2, D), 6), randn((1, T, 4, D), 7)
    want = orc.flash_attn_torch(q, k, v, cu, faithful=False)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    got = ta.flash_attn_triton.apply(qg, kg, vg, cu.cuda())
    assert got.shape == q.shape
    assert_close(got.detach(), want, TOL, "o")
    got.backward(do.cuda())
    dq, dk, dv = orc.varlen_masked_attention_backward(q, k, v, do, cu, orc.causal_mask)
    for name, g, w in (("dq", qg.grad, dq), ("dk", kg.grad, dk), ("dv", vg.grad, dv)):
        assert g.shape == w.shape
        assert_close(g, w, 3e-2 * max(1.0, w.abs().max().item()), name)

    qd = randn((3, 4, D), 8)
    kd, vd = randn((3, 130, 2, D), 9), randn((3, 130, 2, D), 10)
    want = orc.flash_attn_decoding_torch(qd, kd, vd, torch.tensor(lens, dtype=torch.int32), faithful=False)
    got = ta.flash_attention_decoding(qd.cuda(), kd.cuda(), vd.cuda(), cu.cuda())
    assert got.shape == qd.shape
    assert_close(got, want, TOL, "decode o")


def test_sparse_window_forward():
    import tritonops_amd as ta

    D = 32
    lens = [200, 90]
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = randn((1, T, 2, D), 11), randn((1, T, 2, D), 12), randn((1, T, 2, D), 13)
    want = orc.flash_attn_sparse_torch(q, k, v, cu, None, 64, 16, faithful=False)
    got, _ = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, 64, 16)
    assert got.shape == q.shape
    assert_close(got, want, 3e-2, "sparse o")


def test_head_dim_beyond_128_is_refused():
    import tritonops_amd as ta

    q = randn((1, 2, 64, 160), 14).cuda()
    with pytest.raises(ValueError):
        ta.flash_attention(q, q, q, causal=True)
