"""GPU parity of the dense backward (through the C ABI and through the
autograd Function) against the CPU oracle's closed-form gradients on the same
seeded inputs."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import cu_from, randn

pytestmark = pytest.mark.gpu

# gradients are O(1); bf16 rounding of P, dS and of the results bounds the error
GRAD_TOL = 3e-2


def _check(got, want, name, tol=GRAD_TOL):
    got, want = got.float().cpu(), want.float()
    assert torch.isfinite(got).all(), name
    err = (got - want).abs().max().item()
    ref = max(want.abs().max().item(), 1.0)
    assert err <= tol * ref, "%s: max abs err %.4g (scale %.3g)" % (name, err, ref)


# (lengths, Hq, Hkv, D, dtype): the reference's own fwd+bwd test shape is
# ragged, GQA, D in {96, 128} (flash_attn_triton/flash_attn_triton.py:1005-1009,1086-1089)
CASES = [
    ([128, 77, 1, 0, 300], 2, 2, 96, torch.bfloat16),
    ([256, 255, 257, 64], 8, 4, 128, torch.bfloat16),
    ([513, 1024, 31], 4, 1, 128, torch.float16),
    ([700], 6, 2, 96, torch.float16),
    ([512, 100, 65], 4, 1, 64, torch.bfloat16),
    # lengths on either side of every tile boundary of the two kernels (64-row
    # streamed tiles, 128 / 256 resident rows): the masked and the unmasked
    # steps of an item are walked by separate loops
    ([63, 64, 65, 127, 129, 191, 192, 193, 320, 384, 385], 4, 1, 128, torch.bfloat16),
]


@pytest.mark.parametrize("lens,Hq,Hkv,D,dtype", CASES)
def test_packed_causal_backward_matches_oracle(lens, Hq, Hkv, D, dtype):
    import tritonops_amd as ta

    lens = torch.tensor(lens, dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = randn((1, T, Hq, D), 1, dtype), randn((1, T, Hkv, D), 2, dtype), randn((1, T, Hkv, D), 3, dtype)
    do = randn((1, T, Hq, D), 4, dtype)
    wq, wk, wv = orc.varlen_masked_attention_backward(q, k, v, do, cu, orc.causal_mask)
    sm = D ** -0.5 * ta.LOG2E
    o, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), sm)
    dq, dk, dv = ta.flash_attn_triton_bwd(q.cuda(), k.cuda(), v.cuda(), o, do.cuda(), lse, cu.cuda(), sm)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape and dq.dtype == dtype
    _check(dq, wq, "dq")
    _check(dk, wk, "dk")
    _check(dv, wv, "dv")


def test_autograd_function_backward():
    """flash_attn_triton.apply(...).backward(): the reference's public training
    entry (flash_attn_triton.py:816-874)."""
    import tritonops_amd as ta

    lens = torch.tensor([200, 333, 64], dtype=torch.int32)
    cu = cu_from(lens)
    T, Hq, Hkv, D = int(cu[-1]), 8, 2, 128
    q, k, v = randn((1, T, Hq, D), 11), randn((1, T, Hkv, D), 12), randn((1, T, Hkv, D), 13)
    do = randn((1, T, Hq, D), 14)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = ta.flash_attn_triton.apply(qg, kg, vg, cu.cuda())
    o.backward(do.cuda())
    wq, wk, wv = orc.varlen_masked_attention_backward(q, k, v, do, cu, orc.causal_mask)
    _check(qg.grad, wq, "dq")
    _check(kg.grad, wk, "dk")
    _check(vg.grad, wv, "dv")


@pytest.mark.parametrize("causal", [True, False])
def test_batched_backward_through_the_c_abi(causal):
    """[B,S,H,D] batched addressing (no cu_seqlens), S not a multiple of the
    tile sizes, non-causal as well."""
    import ctypes as C

    import tritonops_amd as ta
    from tritonops_amd import _lib, ops

    B, S, Hq, Hkv, D = 2, 330, 4, 2, 128
    q, k, v = randn((B, S, Hq, D), 21), randn((B, S, Hkv, D), 22), randn((B, S, Hkv, D), 23)
    do = randn((B, S, Hq, D), 24)
    sm = D ** -0.5 * ta.LOG2E
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), do.cuda()
    o, lse = ops._dense_fwd(qc, kc, vc, None, sm, causal, None)
    dq, dk, dv = ops._dense_bwd(qc, kc, vc, o, dc, lse, None, sm, causal, None)
    mask = orc.causal_mask if causal else (lambda L: torch.ones(L, L, dtype=torch.bool))
    for b in range(B):
        cu = torch.tensor([0, S], dtype=torch.int32)
        wq, wk, wv = orc.varlen_masked_attention_backward(q[b:b + 1], k[b:b + 1], v[b:b + 1], do[b:b + 1], cu, mask)
        _check(dq[b:b + 1], wq, "dq[%d]" % b)
        _check(dk[b:b + 1], wk, "dk[%d]" % b)
        _check(dv[b:b + 1], wv, "dv[%d]" % b)


@pytest.mark.parametrize("causal", [True, False])
def test_flash_attention_is_differentiable(causal):
    """flash_attention (the README's name for flash_attn_triton.apply) records
    itself for autograd in both layouts; batched [B,H,S,D] with a custom
    softmax_scale against autograd through fp32 torch math."""
    import tritonops_amd as ta

    B, H, S, D = 2, 3, 150, 64
    q, k, v, do = (randn((B, H, S, D), s) for s in (31, 32, 33, 34))
    scale = 0.2
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o, lse = ta.flash_attention(qg, kg, vg, causal=causal, softmax_scale=scale, return_lse=True)
    assert o.requires_grad and not lse.requires_grad
    o.backward(do.cuda())
    qr, kr, vr = (t.float().requires_grad_(True) for t in (q, k, v))
    s = torch.einsum("bhid,bhjd->bhij", qr, kr) * scale
    if causal:
        s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
    ref = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, -1), vr)
    ref.backward(do.float())
    assert (o.detach().float().cpu() - ref.detach()).abs().max() <= 2e-2
    for name, g, w in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        assert g.shape == w.shape
        _check(g, w, name)
    # packed form
    lens = torch.tensor([90, 40], dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    qp, kp, vp, dop = randn((1, T, 4, D), 35), randn((1, T, 2, D), 36), randn((1, T, 2, D), 37), randn((1, T, 4, D), 38)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (qp, kp, vp))
    ta.flash_attention(qg, kg, vg, cu.cuda()).backward(dop.cuda())
    wq, wk, wv = orc.varlen_masked_attention_backward(qp, kp, vp, dop, cu, orc.causal_mask)
    _check(qg.grad, wq, "packed dq")
    _check(kg.grad, wk, "packed dk")
    _check(vg.grad, wv, "packed dv")
    # no gradient requested: no graph
    with torch.no_grad():
        assert not ta.flash_attention(qg, kg, vg, cu.cuda()).requires_grad
