"""The two forms of the dense forward at head_dim 64: the short form (4-wave
workgroups of 128 rows, three to a CU) and the 8-wave kernel that also serves
head_dim 96 and 128; the launcher picks one per launch from the number of work
items (prefill.hip, short_form_pays).  Both against the oracle, and against
each other bit for bit: a row's keys are met in the same order, 32 at a time,
in either form."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, randn

pytestmark = pytest.mark.gpu


def _cus():
    from tritonops_amd import _lib
    return _lib.load().mi_device_cu_count()


def _runs_short_form(batch, heads, max_len):
    """The launcher's choice, restated (prefill.hip: short_form_cost / short_form_pays)."""
    cus = _cus()
    n128 = batch * heads * ((max_len + 127) // 128)
    n256 = batch * heads * ((max_len + 255) // 256)
    if n128 <= cus:
        return True
    grid = 3 * cus
    q, r = divmod(n128, grid)
    rate = {1: 0.4, 2: 0.7, 3: 1.0}
    worst = 0.0
    for c in (0, cus - 1):
        items = [q + (1 if c + k * cus < r else 0) for k in range(3)]
        t, done = 0.0, 0
        for live in (3, 2, 1):
            upto = items[live - 1]
            if upto > done:
                t += (upto - done) * live / rate[live]
                done = upto
        worst = max(worst, t)
    return worst < 2.3 * ((n256 + cus - 1) // cus)


LENS_LONG = [0, 1, 300, 257, 2049, 511, 0, 1500, 31, 1024, 513, 2500, 255, 256, 1000, 2047, 64, 700, 1, 1280, 129, 127,
             128, 33, 2304, 96]
LENS_SHORT = [512, 0, 1, 300, 257, 511, 31, 500, 255, 256, 64, 129, 127, 128, 33, 96, 385, 383, 200, 77, 5, 450, 321, 100,
              160, 192, 224, 288, 352, 416, 480, 17]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lens,heads_q,short_form", [(LENS_LONG, 16, True), (LENS_SHORT, 8, False)])
def test_ragged_packed_batch_in_either_form(lens, heads_q, short_form, dtype):
    """26 sequences of up to 2500 tokens x 16 heads (8320 work items of 128 rows: ten full rounds and most of an
    eleventh); 32 sequences of up to 512 tokens x 8 heads (1024 items of 128 rows are one round and a third, 512 items of
    256 rows two even rounds: the 8-wave kernel)."""
    import tritonops_amd as ta

    lens = torch.tensor(lens, dtype=torch.int32)
    if _runs_short_form(len(lens), heads_q, int(lens.max())) != short_form:
        pytest.skip("with this device's CU count these sizes select the other form")
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
    """48 sequences of 512 tokens (6144 work items of 128 rows, eight even rounds: short form) and the first 8
    of them on their own (1024 items, a round and a third, against two even rounds of 256-row items: the 8-wave
    kernel)."""
    import tritonops_amd as ta

    B, H, S, D = 48, 32, 512, 64
    if not (_runs_short_form(B, H, S) and not _runs_short_form(8, H, S)):
        pytest.skip("with this device's CU count these sizes do not select the two forms")
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
        cu = cu_from(torch.tensor(lens, dtype=torch.int32))
        T = int(cu[-1])
        q, k, v = randn((1, T, 4, 64), 1), randn((1, T, 1, 64), 2), randn((1, T, 1, 64), 3)
        want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
        got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), 0.125 * ta.LOG2E)
        assert_close(got, want, TOL)
        assert (lse.cpu() - want_lse).abs().max().item() <= LSE_TOL
