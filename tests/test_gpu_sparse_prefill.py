"""GPU parity of the block-sparse / window-sparse prefill kernel."""
import numpy as np
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, rand_lengths, randn

pytestmark = pytest.mark.gpu


def _inputs(B, maxlen, Hq, Hkv, D, dtype=torch.bfloat16, lo=1):
    lens = rand_lengths(B, lo, maxlen, seed=3)
    cu = cu_from(lens)
    T = int(cu[-1])
    return (randn((1, T, Hq, D), 1, dtype), randn((1, T, Hkv, D), 2, dtype), randn((1, T, Hkv, D), 3, dtype), cu)


# (4, 2048, 4, 96) with LW=128, GW=0 is the reference's (disabled) test,
# flash_attn_triton/flash_attn_sparse_attn_triton.py:445-503
@pytest.mark.parametrize("lw,gw", [(128, 0), (128, 256), (100, 70), (1, 0), (64, 64), (5000, 0), (0, 5000), (0, 64), (2 ** 40, 2 ** 40)])
def test_window_sparse_matches_oracle(lw, gw):
    import tritonops_amd as ta

    q, k, v, cu = _inputs(4, 2048 if (lw, gw) == (128, 0) else 700, 4, 2, 96)
    want, want_lse = orc.flash_attn_sparse_torch(q, k, v, cu, None, lw, gw, faithful=False, return_lse=True)
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, lw, gw)
    assert_close(got, want, TOL)
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max() <= LSE_TOL
    if lw >= 5000 or gw >= 5000:       # window covers everything -> dense causal
        dense = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda())
        assert_close(got, dense, 1e-2)   # two kernels, two summation orders: one bf16 ulp of |o| < 2
    if (lw, gw) == (1, 0):             # only the diagonal -> o = v
        G = q.shape[2] // v.shape[2]
        assert_close(got, v.repeat_interleave(G, 2), 1e-6)


def test_window_sparse_in_reference_dtype_mode():
    import tritonops_amd as ta

    q, k, v, cu = _inputs(2, 300, 4, 4, 128)
    want = orc.flash_attn_sparse_torch(q, k, v, cu, None, 128, 64, faithful=True)
    got, _ = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, 128, 64)
    assert_close(got, want, 3e-2)      # that oracle also rounds the softmax itself to bf16


def test_no_window_gives_zero_rows():
    import tritonops_amd as ta

    q, k, v, cu = _inputs(2, 100, 2, 2, 64)
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda())   # LW = GW = 0
    assert torch.count_nonzero(got) == 0 and torch.isinf(lse).all()


@pytest.mark.parametrize("per_head", [False, True])
def test_block_mask_matches_oracle(per_head):
    import tritonops_amd as ta
    from tritonops_amd import masks

    B, maxlen, Hq, Hkv, D = 2, 1000, 4, 2, 128
    q, k, v, cu = _inputs(B, maxlen, Hq, Hkv, D, lo=500)
    nqb = (maxlen + 63) // 64
    if per_head:
        ms = np.stack([masks.synthetic_block_mask(nqb, band=2, sink=1, frac=0.2, seed=s) for s in range(Hq)])
        got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), block_mask=ms)
        for h in range(Hq):
            hk = h // (Hq // Hkv)
            want = orc.block_sparse_attention(q[:, :, h:h + 1], k[:, :, hk:hk + 1], v[:, :, hk:hk + 1], cu, ms[h],
                                              faithful=False)
            assert_close(got[:, :, h:h + 1], want, TOL)
    else:
        m = masks.synthetic_block_mask(nqb, band=3, sink=2, frac=0.1, seed=2)
        want, want_lse = orc.block_sparse_attention(q, k, v, cu, m, faithful=False, return_lse=True)
        got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), block_mask=m)
        assert_close(got, want, TOL)
        assert (lse.cpu() - want_lse).abs().max() <= LSE_TOL
        faithful = orc.block_sparse_attention(q, k, v, cu, m, faithful=True)
        assert_close(got, faithful, TOL)


def test_full_lower_triangle_equals_dense():
    import tritonops_amd as ta

    q, k, v, cu = _inputs(3, 520, 8, 2, 64)
    m = np.tril(np.ones((9, 9), dtype=bool))
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), block_mask=m)
    dense, dlse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), 64 ** -0.5 * ta.LOG2E)
    assert_close(got, dense, 1e-2)   # one bf16 ulp of |o| < 2
    assert (lse - dlse).abs().max().item() <= LSE_TOL


def test_listed_blocks_past_the_sequence_end_and_above_the_diagonal():
    """A mask shared by sequences of different lengths names blocks that lie
    past the end of the shorter ones, and a full (not lower-triangular) mask
    names blocks above the diagonal: both are masked per token.  Lengths that
    are multiples of the block size take the kernel's unmasked-load loop only
    when every listed block ends inside the sequence."""
    import tritonops_amd as ta

    Hq, Hkv, D = 4, 2, 128
    lens = torch.tensor([64, 256, 128, 320, 192], dtype=torch.int32)
    cu = cu_from(lens)
    T = int(cu[-1])
    q, k, v = randn((1, T, Hq, D), 1), randn((1, T, Hkv, D), 2), randn((1, T, Hkv, D), 3)
    nqb = 5
    tril = np.tril(np.ones((nqb, nqb), dtype=bool))
    want, want_lse = orc.block_sparse_attention(q, k, v, cu, tril, faithful=False, return_lse=True)
    # the lower triangle through the mask form (its lists reach past the shorter sequences)
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), block_mask=tril)
    assert_close(got, want, TOL)
    assert (lse.cpu() - want_lse).abs().max() <= LSE_TOL
    # every block listed for every row, as a hand-made CSR (the mask form refuses blocks above the diagonal)
    row_ptr = torch.arange(0, nqb * nqb + 1, nqb, dtype=torch.int32).cuda()
    col_idx = torch.arange(nqb, dtype=torch.int32).repeat(nqb).cuda()
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), row_ptr=row_ptr, col_idx=col_idx,
                                           csr_strides=(0, 0, 0, 0))
    assert_close(got, want, TOL)
    assert (lse.cpu() - want_lse).abs().max() <= LSE_TOL


def test_batched_layout_full_size_mask():
    """Benchmark-shaped mask (256x256 blocks, band 8 + 4 sinks + 10 %) on a
    reduced batch/head count, [B,H,S,D] layout; checked on sampled query blocks
    against the oracle restricted to those rows."""
    import tritonops_amd as ta
    from tritonops_amd import masks

    B, H, S, D = 1, 2, 16384, 128
    m = masks.synthetic_block_mask(S // 64, 8, 4, 0.10, seed=2)
    assert int(m.sum()) == 5995
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn((B, H, S, D), generator=g, device="cuda").to(torch.bfloat16) for _ in range(3))
    o, lse = ta.flash_attn_sparse_triton(q, k, v, None, block_mask=m)
    assert o.shape == (B, H, S, D) and lse.shape == (B, H, S)
    bm = torch.from_numpy(m).cuda()
    for qb in (0, 7, 100, 255):
        rows = torch.arange(qb * 64, qb * 64 + 64, device="cuda")
        keys = torch.arange(S, device="cuda")
        allow = bm[qb][keys // 64][None, :] & (keys[None, :] <= rows[:, None])
        s = torch.einsum("bhid,bhjd->bhij", q[:, :, rows].float(), k.float()) * D ** -0.5
        s = s.masked_fill(~allow, float("-inf"))
        ref = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, -1), v.float())
        assert_close(o[:, :, rows], ref, TOL)
        assert (lse[:, :, rows] - torch.logsumexp(s, -1) * orc.LOG2E).abs().max().item() <= LSE_TOL


@pytest.mark.parametrize("D,dtype", [(64, torch.float16), (128, torch.float16), (64, torch.bfloat16)])
def test_sparse_other_dtypes_and_head_dims(D, dtype):
    import tritonops_amd as ta
    from tritonops_amd import masks

    q, k, v, cu = _inputs(3, 400, 6, 3, D, dtype)
    want = orc.flash_attn_sparse_torch(q, k, v, cu, None, 96, 64, faithful=False)
    got, _ = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, 96, 64)
    assert got.dtype == dtype
    assert_close(got, want, TOL)
    m = masks.synthetic_block_mask(7, band=2, sink=1, frac=0.3, seed=4)
    want = orc.block_sparse_attention(q, k, v, cu, m, faithful=False)
    got, _ = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), block_mask=m)
    assert_close(got, want, TOL)
