"""GPU parity of the decoding kernels (dense / window / block-index) through
the C ABI against the CPU oracle."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, randn

pytestmark = pytest.mark.gpu


def _kv(B, L, Hkv, D, dtype, seed):
    return randn((B, L, Hkv, D), seed, dtype), randn((B, L, Hkv, D), seed + 1, dtype)


# lengths of the reference's test (flash_attn_triton/flash_attn_decoding.py:383)
# and its head_dim / dtype (D=96, fp16, :378-403), plus GQA and bf16 D=128
@pytest.mark.parametrize("Hq,Hkv,D,dtype", [
    (2, 2, 96, torch.float16),
    (32, 8, 128, torch.bfloat16),
    (8, 1, 64, torch.bfloat16),
    (6, 2, 128, torch.float16),
])
def test_dense_decode_matches_oracle(Hq, Hkv, D, dtype):
    import tritonops_amd as ta

    lens = torch.tensor([512, 2049, 8192, 0, 1, 63, 64, 65], dtype=torch.int32)
    B, L = len(lens), int(lens.max())
    q = randn((B, Hq, D), 1, dtype)
    k, v = _kv(B, L, Hkv, D, dtype, 2)
    want, want_lse = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=True, return_lse=True)
    exact = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)
    cu = cu_from(lens)
    got, lse = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), return_lse=True)
    assert got.shape == (B, Hq, D) and got.dtype == dtype
    assert_close(got, exact, TOL, "o vs fp32 math")
    assert_close(got, want, TOL, "o vs reference-dtype oracle")
    assert torch.equal(got[3].cpu(), torch.zeros(Hq, D, dtype=dtype))       # len 0 -> zeros
    assert_close(got[4], v[4, 0].repeat_interleave(Hq // Hkv, 0), 1e-6)     # len 1 -> v[0]
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max() <= LSE_TOL
    # split invariance: any chunking gives the same answer up to fp32 rounding
    for st in (64, 256, 8192):
        alt = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(), split_tokens=st)
        assert_close(alt, got, 4e-3, "split_tokens=%d" % st)


def test_decode_on_transposed_cache_and_scale():
    """KV memory [B,Hkv,L,D] passed as a [B,L,Hkv,D] view, explicit qk_scale."""
    import tritonops_amd as ta

    B, Hq, Hkv, L, D = 3, 16, 4, 1000, 128
    lens = torch.tensor([1000, 333, 17], dtype=torch.int32)
    q = randn((B, Hq, D), 4)
    kc, vc = randn((B, Hkv, L, D), 5), randn((B, Hkv, L, D), 6)
    k, v = kc.transpose(1, 2), vc.transpose(1, 2)
    want = orc.flash_attn_decoding_torch(q, k, v, lens, qk_scale=0.05, faithful=False)
    got = ta.flash_attention_decoding(q.cuda(), kc.cuda().transpose(1, 2), vc.cuda().transpose(1, 2),
                                      cu_from(lens).cuda(), 0.05)
    assert_close(got, want, TOL)


# shapes of flash_attn_triton/flash_attn_decoding_sparse.py:409-503 and windows
# from its sweep (:506-630)
@pytest.mark.parametrize("gw,lw", [(256, 4096), (64, 1024), (128, 128), (64, 0), (64, 100)])
def test_window_sparse_decode(gw, lw):
    import tritonops_amd as ta

    Hq, Hkv, D, dtype = 24, 4, 128, torch.float16
    lens = torch.tensor([512, 2561, 8192, 0, 1, 3, 64, 200], dtype=torch.int32)
    B, L = len(lens), int(lens.max())
    q = randn((B, Hq, D), 1, dtype)
    k, v = _kv(B, L, Hkv, D, dtype, 2)
    want = orc.flash_attn_sparse_decoding_torch(q, k, v, lens, gw, lw, faithful=False)
    got = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), cu_from(lens).cuda(), gw, lw)
    assert_close(got, want, TOL)
    faithful = orc.flash_attn_sparse_decoding_torch(q, k, v, lens, gw, lw, faithful=True)
    assert_close(got, faithful, TOL)


def test_window_sparse_decode_rejects_bad_global_window():
    import tritonops_amd as ta

    q = randn((1, 2, 64), 1).cuda()
    k = randn((1, 64, 2, 64), 2).cuda()
    with pytest.raises(AssertionError):
        ta.flash_attention_sparse_decoding(q, k, k, torch.tensor([0, 64], dtype=torch.int32).cuda(), 512, 512)


@pytest.mark.parametrize("top_k", [1, 7, 32])
def test_block_index_decode(top_k):
    import tritonops_amd as ta

    B, Hq, Hkv, D = 3, 8, 2, 128
    lens = torch.tensor([4096, 4000, 2049], dtype=torch.int32)
    L = 4096
    q = randn((B, Hq, D), 1)
    k, v = _kv(B, L, Hkv, D, torch.bfloat16, 2)
    g = torch.Generator().manual_seed(5)
    idx = torch.empty(B, Hkv, top_k, dtype=torch.int32)
    for b in range(B):
        nblk = (int(lens[b]) + 63) // 64
        for h in range(Hkv):
            idx[b, h] = torch.sort(torch.randperm(nblk, generator=g)[:top_k]).values
    want = orc.block_sparse_decoding(q, k, v, lens, idx, faithful=False)
    got = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                             block_indices=idx.cuda())
    assert_close(got, want, TOL)
    # all blocks listed == dense decoding
    if top_k == 32:
        full = torch.arange(64, dtype=torch.int32).expand(B, Hkv, 64).contiguous()
        cnt = ((lens + 63) // 64)[:, None].expand(B, Hkv).contiguous()
        dense = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda())
        got_all = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                                     block_indices=full.cuda(), block_counts=cnt.cuda(),
                                                     include_last_block=False)
        assert_close(got_all, dense, 4e-3)


def test_full_size_decode_properties():
    """Benchmark shape B64 Hq32 Hkv8 L<=32768 D128: a few sequences against the
    oracle, and constant-V invariance (softmax weights sum to one)."""
    import tritonops_amd as ta

    B, Hq, Hkv, L, D = 64, 32, 8, 32768, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    kc = torch.randn((B, Hkv, L, D), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    vc = torch.randn((B, Hkv, L, D), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    q = torch.randn((B, Hq, D), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    lens = torch.randint(16384, 32769, (B,), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    got = ta.flash_attention_decoding(q, kc.transpose(1, 2), vc.transpose(1, 2), None, seq_lens=lens.cuda())
    for b in (0, 31, 63):
        want = orc.flash_attn_decoding_torch(q[b:b + 1].cpu(), kc[b:b + 1].transpose(1, 2).cpu(),
                                             vc[b:b + 1].transpose(1, 2).cpu(), lens[b:b + 1], faithful=False)
        assert_close(got[b:b + 1], want, TOL)
    vc.fill_(0.5)
    got = ta.flash_attention_decoding(q, kc.transpose(1, 2), vc.transpose(1, 2), None, seq_lens=lens.cuda())
    assert (got.float() - 0.5).abs().max().item() <= 4e-3


def test_last_block_listed_and_implicit_counts_once():
    """include_last_block with the last block already in the list (and a ragged
    count) must equal the oracle, which attends each token at most once."""
    import tritonops_amd as ta

    B, Hq, Hkv, D, L = 2, 8, 2, 64, 1000
    lens = torch.tensor([1000, 515], dtype=torch.int32)      # last blocks 15 and 8 (partial)
    q = randn((B, Hq, D), 1)
    k, v = _kv(B, L, Hkv, D, torch.bfloat16, 2)
    idx = torch.tensor([[[3, 15, 0], [15, 0, 0]], [[8, 2, 0], [1, 8, 4]]], dtype=torch.int32)
    cnt = torch.tensor([[2, 1], [2, 3]], dtype=torch.int32)
    want = orc.block_sparse_decoding(q, k, v, lens, idx, cnt, include_last_block=True, faithful=False)
    for sb in (1, 2, 8):
        got = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                                 block_indices=idx.cuda(), block_counts=cnt.cuda(), split_blocks=sb)
        assert_close(got, want, TOL, "split_blocks=%d" % sb)
    no_last = orc.block_sparse_decoding(q, k, v, lens, idx, cnt, include_last_block=False, faithful=False)
    got = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                             block_indices=idx.cuda(), block_counts=cnt.cuda(),
                                             include_last_block=False)
    assert_close(got, no_last, TOL)


def _paginate(k, v, lens, page_size, seed):
    """Scatter a [B,L,Hkv,D] cache into a shuffled page pool; returns pools and
    the page table (unused entries point at a poisoned page)."""
    B, L, Hkv, D = k.shape
    pages_per_seq = (L + page_size - 1) // page_size
    need = [(int(n) + page_size - 1) // page_size for n in lens]
    total = sum(need) + 1
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(total - 1, generator=g) + 1          # page 0 stays poisoned
    kp = torch.full((total, page_size, Hkv, D), float("nan"), dtype=k.dtype)
    vp = torch.full((total, page_size, Hkv, D), float("nan"), dtype=v.dtype)
    table = torch.zeros((B, pages_per_seq), dtype=torch.int32)
    nxt = 0
    for b in range(B):
        for p in range(need[b]):
            phys = int(perm[nxt]); nxt += 1
            table[b, p] = phys
            rows = slice(p * page_size, min((p + 1) * page_size, L))
            n = rows.stop - rows.start
            kp[phys, :n] = k[b, rows]
            vp[phys, :n] = v[b, rows]
            # rows of the last page beyond the sequence hold finite junk (they are masked, not skipped)
            kp[phys, n:] = 7.0
            vp[phys, n:] = -7.0
    return kp, vp, table


@pytest.mark.parametrize("page_size", [32, 64, 256])
def test_paged_cache_is_bit_identical_to_batched(page_size):
    """The page table only changes where a tile is fetched from: same kernel,
    same order of operations, so the outputs must be equal bit for bit."""
    import tritonops_amd as ta

    lens = torch.tensor([777, 2049, 64, 0, 1, 33, 4096], dtype=torch.int32)
    B, Hq, Hkv, D = len(lens), 8, 2, 128
    L = int(lens.max())
    q = randn((B, Hq, D), 21)
    k, v = _kv(B, L, Hkv, D, torch.bfloat16, 22)
    ref, ref_lse = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                               split_tokens=256, return_lse=True)
    kp, vp, table = _paginate(k, v, lens, page_size, 5)
    got, lse = ta.flash_attention_decoding(q.cuda(), kp.cuda(), vp.cuda(), None, seq_lens=lens.cuda(),
                                           split_tokens=256, return_lse=True, kv_layout="paged",
                                           page_table=table.cuda(), max_seq_len=L)
    assert torch.equal(got, ref) and torch.equal(lse, ref_lse)
    want = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)
    assert_close(got, want, TOL)
    # block-list form over the same pages
    idx = torch.zeros((B, Hkv, 6), dtype=torch.int32)
    cnt = torch.zeros((B, Hkv), dtype=torch.int32)
    for b, n in enumerate(lens):
        nblk = (int(n) + 63) // 64
        for h in range(Hkv):
            c = min(6, nblk)
            pick = torch.randperm(max(nblk, 1), generator=torch.Generator().manual_seed(b * 7 + h))[:c]
            idx[b, h, :c] = torch.sort(pick).values.to(torch.int32)
            cnt[b, h] = c
    a = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                           block_indices=idx.cuda(), block_counts=cnt.cuda())
    b_ = ta.flash_attention_sparse_decoding(q.cuda(), kp.cuda(), vp.cuda(), None, seq_lens=lens.cuda(),
                                            block_indices=idx.cuda(), block_counts=cnt.cuda(),
                                            kv_layout="paged", page_table=table.cuda())
    assert torch.equal(a, b_)
    assert torch.isfinite(a.float()).all()


def test_packed_cache_matches_batched_and_reference_oracle_layout():
    """k, v as one [1,T,Hkv,D] buffer addressed through cu_seq_lens — the layout
    the reference's decode oracle takes (flash_attn_decoding.py:357-359)."""
    import tritonops_amd as ta

    lens = torch.tensor([512, 2049, 1, 0, 65, 300], dtype=torch.int32)
    B, Hq, Hkv, D = len(lens), 6, 2, 96
    L = int(lens.max())
    q = randn((B, Hq, D), 31, torch.float16)
    k, v = _kv(B, L, Hkv, D, torch.float16, 32)
    cu = cu_from(lens)
    kpk = torch.cat([k[b, :int(n)] for b, n in enumerate(lens)])[None]
    vpk = torch.cat([v[b, :int(n)] for b, n in enumerate(lens)])[None]
    ref = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), split_tokens=128)
    got = ta.flash_attention_decoding(q.cuda(), kpk.cuda(), vpk.cuda(), cu.cuda(), split_tokens=128,
                                      kv_layout="packed", max_seq_len=L)
    assert torch.equal(got, ref)
    want = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)
    assert_close(got, want, TOL)


@pytest.mark.parametrize("split_tokens", [64, 256, None])
def test_large_ragged_batch_is_dealt_to_the_resident_waves(split_tokens):
    """More sequences than a wavefront has lanes (the chunk-to-sequence search
    walks the batch 64 sequences at a time), many empty ones, and far more live
    chunks than resident waves at the small chunk sizes."""
    import tritonops_amd as ta

    B, Hq, Hkv, D = 150, 4, 2, 64
    g = torch.Generator().manual_seed(5)
    lens = torch.randint(0, 700, (B,), generator=g, dtype=torch.int32)
    lens[::7] = 0
    lens[64] = 699
    lens[149] = 1
    L = int(lens.max())
    q = randn((B, Hq, D), 41)
    k, v = _kv(B, L, Hkv, D, torch.bfloat16, 42)
    want = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)
    got, lse = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                           split_tokens=split_tokens, return_lse=True)
    assert_close(got, want, TOL, "o")
    assert torch.count_nonzero(got[::7]) == 0
    assert torch.isinf(lse[::7]).all() and torch.isfinite(lse[lens.cuda() > 0]).all()


def test_empty_block_list_attends_the_last_block_only():
    """block_indices [B, Hkv, 0] with include_last_block: the list is empty and
    the block holding the newest token is the only one attended."""
    import tritonops_amd as ta

    B, Hq, Hkv, D, L = 3, 4, 2, 128, 300
    lens = torch.tensor([300, 64, 0], dtype=torch.int32)
    q = randn((B, Hq, D), 1)
    k, v = _kv(B, L, Hkv, D, torch.bfloat16, 2)
    idx = torch.zeros((B, Hkv, 0), dtype=torch.int32)
    want = orc.block_sparse_decoding(q, k, v, lens, idx, include_last_block=True, faithful=False)
    got = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                             block_indices=idx.cuda())
    assert_close(got, want, TOL)
    assert torch.count_nonzero(got[2]) == 0
