"""The two forms of the dense forward: work items of 256 query rows on 8-wave
workgroups (dense_kernel) and of 128 rows on 4-wave workgroups
(dense_short_kernel).  The library picks one per launch (prefill.hip,
launch_one / short_form_pays); `ta.dense_form(...)` pins it.  Each form runs the
parity cases of the prefill suite, and the two must agree bit for bit: a row's
keys are met in the same order, 32 at a time, in either form."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests import test_gpu_call_forms as tc
from tests import test_gpu_prefill as tp
from tests import test_gpu_random_shapes as tr
from tests.util import LSE_TOL, TOL, assert_close, cu_from, randn

pytestmark = pytest.mark.gpu

FORMS = ["256", "128"]
LENS = [0, 1, 300, 257, 2049, 511, 0, 1500, 31, 1024, 513, 2500, 255, 256, 1000, 2047, 64, 700, 1, 1280, 129, 127, 128,
        33, 2304, 96]


def _cus():
    from tritonops_amd import _lib
    return _lib.load().mi_device_cu_count()


def _auto_runs_short_form(batch, heads, max_len, head_dim):
    """The launcher's own choice, restated (prefill.hip: launch_one, short_form_cost, short_form_pays)."""
    cus = _cus()
    n128 = batch * heads * ((max_len + 127) // 128)
    n256 = batch * heads * ((max_len + 255) // 256)
    if n128 <= cus:
        return True
    if head_dim != 64:
        return False
    q, r = divmod(n128, 3 * cus)
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


@pytest.mark.parametrize("form", FORMS)
@pytest.mark.parametrize("D,dtype", [(64, torch.bfloat16), (96, torch.float16), (128, torch.bfloat16)])
def test_ragged_packed_batch(D, dtype, form):
    """26 sequences of 0 to 2500 tokens, 16 query heads on 2 kv-heads: several work items per workgroup in either
    form, empty sequences, lengths on either side of every tile and item edge; causal and not."""
    import tritonops_amd as ta

    lens = torch.tensor(LENS, dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = randn((1, T, 16, D), 4, dtype), randn((1, T, 2, D), 5, dtype), randn((1, T, 2, D), 6, dtype)
    want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
    want_nc = orc.varlen_masked_attention(q, k, v, cu, lambda L: torch.ones(L, L, dtype=torch.bool), faithful=False)
    with ta.dense_form(form):
        got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), D ** -0.5 * ta.LOG2E)
        nc = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), causal=False)
    assert_close(got, want, TOL)
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max().item() <= LSE_TOL
    assert_close(nc, want_nc, TOL)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("D", [64, 96, 128])
def test_the_two_forms_agree_bit_for_bit(D, causal):
    import tritonops_amd as ta

    B, H, S = 6, 8, 1408        # 5.5 items of 256 rows, 11 of 128 per (sequence, head)
    g = torch.Generator(device="cuda").manual_seed(7)
    q, k, v = (torch.randn((B, H, S, D), device="cuda", generator=g, dtype=torch.float32).to(torch.bfloat16)
               for _ in range(3))
    outs = {}
    for form in FORMS + ["auto"]:
        with ta.dense_form(form):
            outs[form] = ta.flash_attention(q, k, v, causal=causal, return_lse=True)
    for form in ("128", "auto"):
        assert torch.equal(outs[form][0], outs["256"][0])
        assert torch.equal(outs[form][1], outs["256"][1])
    ref = orc.causal_attention if causal else orc.full_attention
    want = ref(q[1:2, 3:4].float().cpu(), k[1:2, 3:4].float().cpu(), v[1:2, 3:4].float().cpu())
    assert_close(outs["256"][0][1:2, 3:4], want, TOL)


def test_the_library_picks_both_forms_at_head_dim_64():
    """48 sequences of 512 tokens x 32 heads (6144 work items of 128 rows, eight even rounds of three workgroups per
    CU: the short form) and the first 8 of them on their own (1024 items are a round and a third, against two even
    rounds of 256-row items: the long form): the same bits for those 8, whatever ran."""
    import tritonops_amd as ta

    B, H, S, D = 48, 32, 512, 64
    if not (_auto_runs_short_form(B, H, S, D) and not _auto_runs_short_form(8, H, S, D)):
        pytest.skip("with this device's CU count these sizes do not select the two forms")
    g = torch.Generator(device="cuda").manual_seed(7)
    q, k, v = (torch.randn((B, H, S, D), device="cuda", generator=g, dtype=torch.float32).to(torch.bfloat16)
               for _ in range(3))
    o_all, lse_all = ta.flash_attention(q, k, v, causal=True, return_lse=True)
    o_8, lse_8 = ta.flash_attention(q[:8].contiguous(), k[:8].contiguous(), v[:8].contiguous(), causal=True,
                                    return_lse=True)
    assert torch.equal(o_all[:8], o_8) and torch.equal(lse_all[:8], lse_8)
    for b, h in ((0, 0), (17, 5), (47, 31)):
        want = orc.causal_attention(q[b:b + 1, h:h + 1].float().cpu(), k[b:b + 1, h:h + 1].float().cpu(),
                                    v[b:b + 1, h:h + 1].float().cpu())
        assert_close(o_all[b:b + 1, h:h + 1], want, TOL)


@pytest.mark.parametrize("form", FORMS)
def test_prefill_suite_in_each_form(form):
    """The parity cases of the prefill, random-shape and call-form suites with the form pinned (left to itself the
    library runs their small launches in the short form and the large ones in the long form)."""
    import tritonops_amd as ta

    with ta.dense_form(form):
        for case in tp.VARLEN_CASES:
            for dtype in (torch.bfloat16, torch.float16):
                tp.test_varlen_causal_matches_oracle(case, dtype)
        tp.test_uniform_inputs_like_reference_generator()
        for shape in [(1, 4, 256, 64), (2, 3, 200, 128), (1, 2, 77, 96), (2, 2, 1024, 128)]:
            for causal in (False, True):
                tp.test_batched_bhsd(shape, causal)
        tp.test_gqa_batched_and_strided_views()
        tp.test_closed_forms_on_device()
        tp.test_softmax_scale_and_extreme_scores()
        for slope in (0.5, 16.0, -16.0):
            for causal in (True, False):
                tp.test_scores_that_keep_growing_along_the_keys(slope, causal)
        tp.test_long_ragged_batch_with_many_tiles()
        for D, dtype in [(64, torch.float16), (96, torch.bfloat16), (128, torch.float16)]:
            tp.test_many_work_items_per_workgroup(D, dtype)
        tp.test_rows_outside_every_sequence_are_zero()
        for seed in range(8):
            tr.test_dense_forward_random_ragged_batches(seed)
        tc.test_max_seqlen_below_the_longest_sequence_cuts_it()
        tc.test_python_forms_return_zero_rows_outside_the_sequences()


def test_dense_form_rejects_other_values():
    import tritonops_amd as ta

    with pytest.raises(ValueError):
        with ta.dense_form("64"):
            pass
