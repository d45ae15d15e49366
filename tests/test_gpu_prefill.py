"""GPU parity of the dense prefill kernel (through the C ABI) against the CPU
oracle on the same seeded inputs."""
import math

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, rand_lengths, randn

pytestmark = pytest.mark.gpu


def _lse_close(got, want, valid=None):
    got, want = got.float().cpu(), want.float().cpu()
    if valid is not None:
        got, want = got[valid], want[valid]
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), fin)
    assert (got[fin] - want[fin]).abs().max().item() <= LSE_TOL


# (batch, max_len, Hq, Hkv, D): the reference's own test shapes
# (flash_attn_triton/flash_attn_triton.py:1005-1009) plus ragged edges
VARLEN_CASES = [
    (3, 128, 2, 2, 96),
    (2, 256, 8, 4, 128),
    (4, 512, 4, 1, 64),
    (5, 200, 4, 2, 128),
    (1, 1, 2, 1, 64),
]


@pytest.mark.parametrize("case", VARLEN_CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_varlen_causal_matches_oracle(case, dtype):
    import tritonops_amd as ta

    B, maxlen, Hq, Hkv, D = case
    lens = rand_lengths(B, 1, maxlen, seed=11 + B)
    cu = cu_from(lens)
    T = int(cu[-1])
    q = randn((1, T, Hq, D), 1, dtype)
    k = randn((1, T, Hkv, D), 2, dtype)
    v = randn((1, T, Hkv, D), 3, dtype)
    want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=True, return_lse=True)
    got, got_lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), D ** -0.5 * ta.LOG2E)
    torch.cuda.synchronize()
    assert got.shape == (1, T, Hq, D) and got.dtype == dtype
    assert got_lse.shape == (1, T, Hq) and got_lse.dtype == torch.float32
    assert_close(got, want, TOL, "o")
    exact = orc.flash_attn_torch(q, k, v, cu, faithful=False)
    assert_close(got, exact, TOL, "o vs fp32 math")
    _lse_close(got_lse, want_lse)
    # the autograd entry and the README entry return the same tensor
    got2 = ta.flash_attn_triton.apply(q.cuda(), k.cuda(), v.cuda(), cu.cuda())
    got3 = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda())
    assert torch.equal(got2, got) and torch.equal(got3, got)


def test_uniform_inputs_like_reference_generator():
    """The reference draws q/k/v from U[0,1) (flash_attn_triton.py:930-936)."""
    import tritonops_amd as ta

    g = torch.Generator().manual_seed(42)
    lens = torch.randint(1, 257, (2,), generator=g, dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = (torch.rand((1, T, h, 128), generator=g).to(torch.bfloat16) for h in (8, 4, 4))
    want = orc.flash_attn_torch(q, k, v, cu)
    got = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda())
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 4, 256, 64), (2, 3, 200, 128), (1, 2, 77, 96), (2, 2, 1024, 128)])
def test_batched_bhsd(shape, causal):
    import tritonops_amd as ta

    B, H, S, D = shape
    q, k, v = (randn(shape, s) for s in (5, 6, 7))
    ref = (orc.causal_attention if causal else orc.full_attention)(q, k, v)
    ref32 = (orc.causal_attention if causal else orc.full_attention)(q.float(), k.float(), v.float())
    got, lse = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
    assert got.shape == shape and got.is_contiguous() and lse.shape == (B, H, S)
    assert_close(got, ref32, TOL, "o vs fp32 math")
    assert_close(got, ref, 3e-2, "o vs input-dtype oracle")  # that oracle rounds p and o to bf16 itself
    s = torch.einsum("bhid,bhjd->bhij", q.float(), k.float()) / math.sqrt(D)
    if causal:
        s = s.masked_fill(~torch.ones(S, S, dtype=torch.bool).tril(), float("-inf"))
    _lse_close(lse, torch.logsumexp(s, -1) * orc.LOG2E)


def test_gqa_batched_and_strided_views():
    import tritonops_amd as ta

    B, Hq, Hkv, S, D = 2, 8, 2, 300, 128
    q = randn((B, Hq, S, D), 1)
    k = randn((B, Hkv, S, D), 2)
    v = randn((B, Hkv, S, D), 3)
    ke, ve = k.repeat_interleave(Hq // Hkv, 1), v.repeat_interleave(Hq // Hkv, 1)
    ref = orc.causal_attention(q.float(), ke.float(), ve.float())
    got = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=True)
    assert_close(got, ref, TOL)
    # [B,S,H,D] memory viewed as [B,H,S,D]
    qs = q.transpose(1, 2).contiguous().cuda().transpose(1, 2)
    got2 = ta.flash_attention(qs, k.cuda(), v.cuda(), causal=True)
    assert torch.equal(got2, got)


def test_closed_forms_on_device():
    import tritonops_amd as ta

    B, H, S, D = 1, 2, 192, 64
    v = randn((B, H, S, D), 9)
    k = randn((B, H, S, D), 8)
    q = torch.zeros((B, H, S, D), dtype=torch.bfloat16)
    # zero queries: uniform weights -> running mean (causal) / mean (full)
    got, lse = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=True, return_lse=True)
    run_mean = torch.cumsum(v.float(), 2) / torch.arange(1, S + 1)[None, None, :, None]
    assert_close(got, run_mean, TOL)
    want_lse = torch.log2(torch.arange(1, S + 1).float())[None, None].expand(B, H, S)
    assert (lse.cpu() - want_lse).abs().max() < 1e-4
    got = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=False)
    assert_close(got, v.float().mean(2, keepdim=True).expand_as(v), TOL)


def test_softmax_scale_and_extreme_scores():
    import tritonops_amd as ta

    B, H, S, D = 1, 2, 130, 128
    q, k, v = (randn((B, H, S, D), s) for s in (1, 2, 3))
    q = q * 8  # |scores| in the hundreds
    for sc in (0.5, 0.02):
        s = torch.einsum("bhid,bhjd->bhij", q.float(), k.float()) * sc
        ref = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, -1), v.float())
        got = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=False, softmax_scale=sc)
        assert_close(got, ref, TOL)


@pytest.mark.parametrize("slope", [0.5, 16.0, -16.0])
@pytest.mark.parametrize("causal", [True, False])
def test_scores_that_keep_growing_along_the_keys(slope, causal):
    """s_ij = c * slope * j: every later half-tile beats the running reference
    point of the row, mildly (slope 0.5: a few binades per 32 keys) or by more
    than the fp32 exponent range (slope 16: exp2 overflows unless the reference
    point is moved first); slope -16 is the mirror image (everything after the
    first keys underflows).  Checked against fp32 softmax on the same inputs."""
    import tritonops_amd as ta

    B, H, S, D = 1, 2, 1100, 128
    u = torch.full((D,), 0.125)
    j = torch.arange(S, dtype=torch.float32)
    k = (u[None, :] * (slope * j)[:, None]).to(torch.bfloat16)[None, None].expand(B, H, S, D).contiguous()
    q = u.to(torch.bfloat16)[None, None, None, :].expand(B, H, S, D).contiguous()
    v = randn((B, H, S, D), 5)
    s = torch.einsum("bhid,bhjd->bhij", q.double(), k.double()) / math.sqrt(D)
    if causal:
        s = s.masked_fill(torch.arange(S)[None, :] > torch.arange(S)[:, None], float("-inf"))
    ref = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, -1), v.double()).float()
    got, lse = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
    assert torch.isfinite(got.float()).all()
    assert_close(got, ref, TOL)
    want_lse = (torch.logsumexp(s, -1) * orc.LOG2E).float()
    rel = ((lse.cpu() - want_lse).abs() / want_lse.abs().clamp_min(1.0)).max().item()
    assert rel <= 1e-3, rel


def test_full_size_properties():
    """Size-independent checks at the benchmark shape B4 H32 S8192 D128: row 0
    equals v[0]; lse of zero-query rows; a head slice matches the oracle on a
    prefix (causality makes the prefix self-contained)."""
    import tritonops_amd as ta

    B, H, S, D = 4, 32, 8192, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn((B, H, S, D), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
               for _ in range(3))
    o, lse = ta.flash_attention(q, k, v, causal=True, return_lse=True)
    torch.cuda.synchronize()
    assert not torch.isnan(o.float()).any() and torch.isfinite(lse).all()
    assert torch.equal(o[:, :, 0], v[:, :, 0])
    P = 512
    for (b, h) in ((0, 0), (3, 31), (1, 17)):
        ref = orc.causal_attention(q[b:b + 1, h:h + 1, :P].cpu().float(), k[b:b + 1, h:h + 1, :P].cpu().float(),
                                   v[b:b + 1, h:h + 1, :P].cpu().float())
        assert_close(o[b:b + 1, h:h + 1, :P], ref, TOL)
    # last rows against a chunked fp32 evaluation on the device
    rows = slice(S - 64, S)
    s = torch.einsum("bhid,bhjd->bhij", q[:, :, rows].float(), k.float()) / math.sqrt(D)
    i = torch.arange(S - 64, S, device="cuda")[:, None]
    s = s.masked_fill(torch.arange(S, device="cuda")[None, :] > i, float("-inf"))
    ref = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, -1), v.float())
    assert_close(o[:, :, rows], ref, TOL)
    assert (lse[:, :, rows] - torch.logsumexp(s, -1) * orc.LOG2E).abs().max().item() <= LSE_TOL


def test_long_ragged_batch_with_many_tiles():
    """Several hundred KV tiles per sequence, lengths straddling every tile and
    workgroup edge (63/64/65, 255/256/257 ...), packed layout, GQA 4."""
    import tritonops_amd as ta

    lens = torch.tensor([63, 64, 65, 255, 256, 257, 1023, 1025, 2048, 3000], dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = randn((1, T, 8, 128), 1), randn((1, T, 2, 128), 2), randn((1, T, 2, 128), 3)
    want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
    got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), 128 ** -0.5 * ta.LOG2E,
                                        max_seq_len=3000)
    assert_close(got, want, TOL)
    _lse_close(lse, want_lse)
    nc = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), causal=False)
    want_nc = orc.varlen_masked_attention(q, k, v, cu, lambda L: torch.ones(L, L, dtype=torch.bool), faithful=False)
    assert_close(nc, want_nc, TOL)


@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (96, torch.bfloat16), (128, torch.float16)])
def test_many_work_items_per_workgroup(D, dtype):
    """A packed batch whose q tiles outnumber the CUs several times over, with
    empty sequences, sequences of one token and q tiles that do not exist for
    the shorter sequences: every workgroup walks a dozen work items, skips
    some, and overlaps the write-out of one with the loads of the next."""
    import tritonops_amd as ta

    lens = torch.tensor([0, 1, 300, 257, 2049, 511, 0, 1500, 31, 1024, 513, 2500, 255, 256, 1000, 2047, 64, 700, 1,
                         1280], dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    Hq, Hkv = 16, 4
    q, k, v = randn((1, T, Hq, D), 4, dtype), randn((1, T, Hkv, D), 5, dtype), randn((1, T, Hkv, D), 6, dtype)
    want, want_lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
    got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), D ** -0.5 * ta.LOG2E)
    assert_close(got, want, TOL)
    _lse_close(lse, want_lse)
    again, lse2 = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), D ** -0.5 * ta.LOG2E)
    assert torch.equal(again, got) and torch.equal(lse2, lse)


def test_rows_outside_every_sequence_are_zero():
    """Packed buffers longer than cu_seq_lens[-1]: rows that belong to no
    sequence come back as zeros in o and lse, as from the reference's
    zero-filled outputs (flash_attn_triton.py:608-609)."""
    import tritonops_amd as ta

    lens = torch.tensor([70, 130], dtype=torch.int32)
    cu = cu_from(lens)
    T, pad, Hq, Hkv, D = int(cu[-1]), 56, 4, 2, 128
    q, k, v = randn((1, T + pad, Hq, D), 1), randn((1, T + pad, Hkv, D), 2), randn((1, T + pad, Hkv, D), 3)
    sm = D ** -0.5 * ta.LOG2E
    o, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), sm)
    want, want_lse = orc.flash_attn_torch(q[:, :T], k[:, :T], v[:, :T], cu, faithful=False, return_lse=True)
    assert_close(o[:, :T], want, TOL)
    assert (lse[:, :T].cpu() - want_lse).abs().max() <= LSE_TOL
    assert torch.count_nonzero(o[:, T:]) == 0 and torch.count_nonzero(lse[:, T:]) == 0
    so, slse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, 64, 64)
    assert torch.count_nonzero(so[:, T:]) == 0 and torch.count_nonzero(slse[:, T:]) == 0
