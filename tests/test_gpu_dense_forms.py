"""The two forms of the dense forward at head_dim 64: launches of at most one
128-row work item per CU and launches of eight rounds or more run the short
form (4-wave workgroups, three to a CU); everything in between runs the
8-wave kernel that also serves head_dim 96 and 128.  Both against the oracle,
and against each other bit for bit: a row's keys are met in the same order,
32 at a time, in either form."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, randn

pytestmark = pytest.mark.gpu

SHORT_ROWS, SHORT_PER_CU, ROUNDS = 128, 3, 8


def _items(batch, heads, max_len):
    return batch * heads * ((max_len + SHORT_ROWS - 1) // SHORT_ROWS)


def _cus():
    from tritonops_amd import _lib
    return _lib.load().mi_device_cu_count()


def _runs_short_form(batch, heads, max_len):
    n, cus = _items(batch, heads, max_len), _cus()
    return n <= cus or n >= ROUNDS * SHORT_PER_CU * cus


LENS = [0, 1, 300, 257, 2049, 511, 0, 1500, 31, 1024, 513, 2500, 255, 256, 1000, 2047, 64, 700, 1, 1280, 129, 127, 128,
        33, 2304, 96]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("heads_q,short_form", [(16, True), (4, False)])
def test_ragged_packed_batch_in_either_form(heads_q, short_form, dtype):
    import tritonops_amd as ta

    lens = torch.tensor(LENS, dtype=torch.int32)
    assert _runs_short_form(len(LENS), heads_q, int(lens.max())) == short_form, "sizes no longer select the intended form"
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = randn((1, T, heads_q, 64), 4, dtype), randn((1, T, 2, 64), 5, dtype), randn((1, T, 2, 64), 6, dtype)
    want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
    got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), 64 ** -0.5 * ta.LOG2E)
    assert_close(got, want, TOL)
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max().item() <= LSE_TOL
    nc = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), causal=False)
    want_nc = orc.varlen_masked_attention(q, k, v, cu, lambda L: torch.ones(L, L, dtype=torch.bool), faithful=False)
    assert_close(nc, want_nc, TOL)


@pytest.mark.parametrize("causal", [True, False])
def test_the_two_forms_agree_bit_for_bit(causal):
    """48 sequences of 512 tokens (6144 work items: short form) and the first 8
    of them on their own (1024 items: the 8-wave kernel)."""
    import tritonops_amd as ta

    B, H, S, D = 48, 32, 512, 64
    assert _runs_short_form(B, H, S) and not _runs_short_form(8, H, S), "sizes no longer select the intended forms"
    g = torch.Generator(device="cuda").manual_seed(7)
    q, k, v = (torch.randn((B, H, S, D), device="cuda", generator=g, dtype=torch.float32).to(torch.bfloat16)
               for _ in range(3))
    o_all, lse_all = ta.flash_attention(q, k, v, causal=causal, return_lse=True)
    o_8, lse_8 = ta.flash_attention(q[:8].contiguous(), k[:8].contiguous(), v[:8].contiguous(), causal=causal,
                                    return_lse=True)
    assert torch.equal(o_all[:8], o_8)
    assert torch.equal(lse_all[:8], lse_8)
    # and the oracle on a few (sequence, head) units of the large launch
    for b, h in ((0, 0), (17, 5), (47, 31)):
        ref = orc.causal_attention if causal else orc.full_attention
        want = ref(q[b:b + 1, h:h + 1].float().cpu(), k[b:b + 1, h:h + 1].float().cpu(), v[b:b + 1, h:h + 1].float().cpu())
        assert_close(o_all[b:b + 1, h:h + 1], want, TOL)


def test_tiny_launches_run_the_short_form_and_match():
    """One work item per workgroup and fewer workgroups than CUs: the reference's
    own head_dim-64 test shape (flash_attn_triton.py:1008) and lengths around the
    edges of the 32-key tiles and the 128-row items."""
    import tritonops_amd as ta

    for lens in ([512, 300, 1, 77], [33], [128, 129, 127, 31, 32, 0, 161]):
        assert _runs_short_form(len(lens), 4, max(lens))
        cu = cu_from(torch.tensor(lens, dtype=torch.int32))
        T = int(cu[-1])
        q, k, v = randn((1, T, 4, 64), 1), randn((1, T, 1, 64), 2), randn((1, T, 1, 64), 3)
        want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
        got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), 0.125 * ta.LOG2E)
        assert_close(got, want, TOL)
        assert (lse.cpu() - want_lse).abs().max().item() <= LSE_TOL
