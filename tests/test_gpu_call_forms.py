"""GPU parity of the call forms around the kernels: rows of packed tensors that
belong to no sequence (the library zeroes them, the caller hands in
uninitialised outputs), a `max_seq_len` hint below the longest sequence, the
window form of sparse decoding (block list derived inside the kernel) and GQA
groups of more than 32 query heads in decoding."""
import ctypes as C

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, randn

pytestmark = pytest.mark.gpu

SENTINEL = 12345.0


def _fwd_args(q, k, v, o, lse, cu, max_seqlen, total_rows):
    import tritonops_amd as ta
    from tritonops_amd import _lib

    a = _lib.AttnFwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = (t.data_ptr() for t in (q, k, v, o, lse))
    for n, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, n + "_stride_s", t.stride(1))
        setattr(a, n + "_stride_h", t.stride(2))
    a.lse_stride_s, a.lse_stride_h = lse.stride(1), lse.stride(2)
    a.cu_seqlens = cu.data_ptr()
    a.batch, a.heads_q, a.heads_kv = cu.numel() - 1, q.shape[2], k.shape[2]
    a.max_seqlen, a.head_dim, a.causal = max_seqlen, q.shape[3], 1
    a.scale_log2 = q.shape[3] ** -0.5 * ta.LOG2E
    a.total_rows = total_rows
    return a


@pytest.mark.parametrize("pad", [0, 1, 70, 300])
def test_rows_outside_every_sequence_are_zeroed_by_the_library(pad):
    """Packed forward on outputs full of a sentinel: rows of a sequence are
    computed, the `pad` rows behind cu_seqlens[-1] are zero (the reference
    zero-fills both outputs, flash_attn_triton.py:608-609), and with
    total_rows = 0 the same rows are left alone."""
    from tritonops_amd import _lib

    lib = _lib.load()
    lens = [100, 0, 37, 200]
    cu = cu_from(lens)
    used = int(cu[-1])
    T, Hq, Hkv, D = used + pad, 4, 2, 128
    q, k, v = randn((1, T, Hq, D), 1), randn((1, T, Hkv, D), 2), randn((1, T, Hkv, D), 3)
    want, want_lse = orc.flash_attn_torch(q[:, :used], k[:, :used], v[:, :used], cu, faithful=False, return_lse=True)
    qd, kd, vd, cud = q.cuda(), k.cuda(), v.cuda(), cu.cuda()
    for total_rows in (T, 0):
        o = torch.full((1, T, Hq, D), SENTINEL, device="cuda", dtype=torch.bfloat16)
        lse = torch.full((1, T, Hq), SENTINEL, device="cuda", dtype=torch.float32)
        a = _fwd_args(qd, kd, vd, o, lse, cud, max(lens), total_rows)
        _lib.check(lib.mi_attn_fwd(C.byref(a), None))
        torch.cuda.synchronize()
        assert_close(o[:, :used], want, TOL, "o")
        assert_close(lse[:, :used], want_lse, LSE_TOL, "lse")
        tail_o, tail_l = o[:, used:].float().cpu(), lse[:, used:].cpu()
        fill = 0.0 if total_rows else SENTINEL
        assert (tail_o == torch.tensor(fill).bfloat16().float()).all() and (tail_l == fill).all()


def test_python_forms_return_zero_rows_outside_the_sequences():
    """The three packed Python entry points allocate uninitialised outputs and
    still return zeros for the padding rows, forward and backward."""
    import tritonops_amd as ta

    lens = [130, 64, 1]
    cu = cu_from(lens)
    used, pad = int(cu[-1]), 93
    T, Hq, Hkv, D = used + pad, 4, 2, 64
    q, k, v, do = (randn((1, T, h, D), s) for s, h in ((1, Hq), (2, Hkv), (3, Hkv), (4, Hq)))
    # dirty the caching allocator's free blocks so that torch.empty is not accidentally zero
    for _ in range(4):
        junk = torch.full((T * Hq * D,), SENTINEL, device="cuda", dtype=torch.float32)
        del junk
    sm = D ** -0.5 * ta.LOG2E
    o, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), sm)
    assert (o[:, used:] == 0).all() and (lse[:, used:] == 0).all()
    dq, dk, dv = ta.flash_attn_triton_bwd(q.cuda(), k.cuda(), v.cuda(), o, do.cuda(), lse, cu.cuda(), sm)
    for g in (dq, dk, dv):
        assert (g[:, used:] == 0).all() and torch.isfinite(g.float()).all()
    wq, wk, wv = orc.varlen_masked_attention_backward(q[:, :used], k[:, :used], v[:, :used], do[:, :used], cu,
                                                      orc.causal_mask)
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        assert (got[:, :used].float().cpu() - want.float()).abs().max() <= 3e-2 * max(1.0, want.abs().max().item())
    os_, ls = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, 64, 64)
    assert (os_[:, used:] == 0).all() and (ls[:, used:] == 0).all()
    want = orc.flash_attn_sparse_torch(q[:, :used], k[:, :used], v[:, :used], cu, None, 64, 64, faithful=False)
    assert_close(os_[:, :used], want, TOL, "window-sparse o")


def test_zeroing_follows_what_the_host_knows_about_cu_seq_lens():
    """When the host has read a cu_seq_lens tensor and its sequences tile the whole
    buffer, the drop-ins skip the launch that zeroes rows outside the sequences;
    an in-place change of that tensor, a max_seq_len below the longest sequence,
    or a first entry above 0 must bring it back."""
    import tritonops_amd as ta
    from tritonops_amd import ops

    T, Hq, Hkv, D = 512, 4, 2, 64
    q, k, v = (randn((1, T, h, D), s).cuda() for s, h in ((1, Hq), (2, Hkv), (3, Hkv)))
    cu = torch.tensor([0, 200, 512], dtype=torch.int32, device="cuda")

    def dirty():
        for _ in range(4):
            junk = torch.full((T * Hq * D,), SENTINEL, device="cuda", dtype=torch.float32)
            del junk

    dirty()
    o, lse = ta.flash_attention(q, k, v, cu, return_lse=True)          # reads the lengths on the host
    assert ops._rows_to_cover(cu, 312, T) == 0 and ops._rows_to_cover(cu, 311, T) == T
    want = orc.flash_attn_torch(q.cpu(), k.cpu(), v.cpu(), cu.cpu(), faithful=False)
    assert_close(o, want, TOL, "o, every row inside a sequence")
    o2 = ta.flash_attention(q, k, v, cu, max_seq_len=100)             # both sequences cut: rows behind token 100 are zero
    assert (o2[:, 100:200] == 0).all() and (o2[:, 300:] == 0).all()
    assert_close(o2[:, :100], want[:, :100], TOL, "kept rows")
    cu[2] = 400                                                        # in place: the version counter moves
    dirty()
    o3, lse3 = ta.flash_attention(q, k, v, cu, return_lse=True)
    assert (o3[:, 400:] == 0).all() and (lse3[:, 400:] == 0).all()
    assert ops._rows_to_cover(cu, 512, T) == T
    cu2 = torch.tensor([64, 200, 512], dtype=torch.int32, device="cuda")   # rows in front of the first sequence
    dirty()
    o4 = ta.flash_attention(q, k, v, cu2)
    assert (o4[:, :64] == 0).all()
    os_, ls = ta.flash_attn_sparse_triton(q, k, v, cu, None, 64, 64)
    assert (os_[:, 400:] == 0).all() and (ls[:, 400:] == 0).all()


def test_max_seqlen_below_the_longest_sequence_cuts_it():
    """A bound smaller than a real length must not write outside what was sized
    for it: the long sequence is cut at the bound (for a causal forward the kept
    rows are unchanged), later rows come back as zeros, and the backward's Delta
    workspace - sized [batch, heads, max_seqlen] - is not overrun (guard words
    behind it stay intact)."""
    import tritonops_amd as ta
    from tritonops_amd import _lib

    lib = _lib.load()
    lens, bound = [300, 700, 64], 320
    cu = cu_from(lens)
    T, Hq, Hkv, D = int(cu[-1]), 4, 2, 128
    q, k, v, do = (randn((1, T, h, D), s) for s, h in ((1, Hq), (2, Hkv), (3, Hkv), (4, Hq)))
    # what a caller who really had sequences of min(len, bound) tokens would get
    keep = torch.cat([torch.arange(int(cu[i]), int(cu[i]) + min(n, bound)) for i, n in enumerate(lens)])
    cut = torch.ones(T, dtype=torch.bool)
    cut[keep] = False
    cu_cut = cu_from([min(n, bound) for n in lens])
    qc, kc, vc, doc = (t[:, keep] for t in (q, k, v, do))
    want, want_lse = orc.flash_attn_torch(qc, kc, vc, cu_cut, faithful=False, return_lse=True)
    wq, wk, wv = orc.varlen_masked_attention_backward(qc, kc, vc, doc, cu_cut, orc.causal_mask)

    sm = D ** -0.5 * ta.LOG2E
    qd, kd, vd, dod, cud = q.cuda(), k.cuda(), v.cuda(), do.cuda(), cu.cuda()
    o, lse = ta.flash_attn_triton_fwd(qd, kd, vd, cud, sm, max_seq_len=bound)
    assert_close(o[:, keep], want, TOL, "o")
    assert_close(lse[:, keep], want_lse, LSE_TOL, "lse")
    assert (o[:, cut] == 0).all() and (lse[:, cut] == 0).all()

    a = _lib.AttnBwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    dq, dk, dv = (torch.full_like(t, SENTINEL) for t in (qd, kd, vd))
    for n, t in (("q", qd), ("k", kd), ("v", vd), ("o", o), ("dout", dod), ("dq", dq), ("dk", dk), ("dv", dv),
                 ("lse", lse)):
        setattr(a, n, t.data_ptr())
        setattr(a, n + "_stride_s", t.stride(1))
        setattr(a, n + "_stride_h", t.stride(2))
    a.cu_seqlens = cud.data_ptr()
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim, a.causal = len(lens), Hq, Hkv, bound, D, 1
    a.scale_log2 = sm
    a.total_rows = T
    nb = lib.mi_attn_bwd_workspace_bytes(C.byref(a))
    assert nb == len(lens) * Hq * bound * 4
    guard = 4096
    ws = torch.full((nb // 4 + guard,), SENTINEL, device="cuda", dtype=torch.float32)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    _lib.check(lib.mi_attn_bwd(C.byref(a), None))
    torch.cuda.synchronize()
    assert (ws[nb // 4:] == SENTINEL).all(), "the backward wrote behind its workspace"
    for got, w, name in ((dq, wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        g = got[:, keep].float().cpu()
        assert (g - w.float()).abs().max() <= 3e-2 * max(1.0, w.abs().max().item()), name
        assert (got[:, cut] == 0).all(), name


def _explicit_window_list(lens, gw, lw, Hkv):
    """The window form as an explicit block list (what the Python wrapper used
    to build on the device): sink blocks, then the blocks of the last lw tokens."""
    B = lens.numel()
    n_sink, n_tail = gw // 64, (lw + 63) // 64 + 1
    nblk = (lens + 63) // 64
    tail0 = torch.maximum(torch.clamp(lens - lw, min=0) // 64, torch.full_like(lens, n_sink))
    cand = torch.cat([torch.arange(n_sink, dtype=torch.int32).expand(B, n_sink),
                      tail0[:, None] + torch.arange(n_tail, dtype=torch.int32)[None, :]], 1)
    valid = cand < nblk[:, None]
    key = torch.where(valid, cand, torch.full_like(cand, 2 ** 30))
    idx = torch.sort(key, 1).values.to(torch.int32)
    idx = torch.where(idx >= 2 ** 30, torch.zeros_like(idx), idx).contiguous()
    cnt = valid.sum(1).to(torch.int32)[:, None].expand(B, Hkv).contiguous()
    return idx, cnt, n_sink + n_tail


@pytest.mark.parametrize("gw,lw", [(64, 64), (256, 4096), (128, 0), (256, 100), (64, 1000)])
def test_window_form_decode_is_the_explicit_list_bit_for_bit(gw, lw):
    """flash_attention_sparse_decoding(q, k, v, cu, gw, lw) derives its blocks
    in the kernel; an explicit list of the same blocks with the same windows
    must give the same bits, and both match the oracle
    (flash_attn_decoding_sparse.py:391-396)."""
    import tritonops_amd as ta
    from tritonops_amd import ops

    lens = torch.tensor([0, 1, 63, 64, 65, 300, 4095, 4096, 4097, 5000, 8192, 129], dtype=torch.int32)
    B, Hq, Hkv, D, L = lens.numel(), 8, 2, 128, 8192
    q, k, v = randn((B, Hq, D), 1), randn((B, L, Hkv, D), 2), randn((B, L, Hkv, D), 3)
    cu = cu_from(lens)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    got, got_lse = ta.flash_attention_sparse_decoding(qd, kd, vd, cu.cuda(), gw, lw, return_lse=True, split_blocks=3)
    idx, cnt, cap = _explicit_window_list(lens, gw, lw, Hkv)
    ref, ref_lse = ops._decode(qd, kd, vd, None, lens.cuda(), D ** -0.5, None, None, True, block_idx=idx.cuda(),
                               block_cnt=cnt.cuda(), bi_strides=(cap, 0), max_blocks=cap, split_blocks=3,
                               window=(lw, gw))
    assert torch.equal(got, ref) and torch.equal(got_lse, ref_lse)
    want = orc.flash_attn_sparse_decoding_torch(q, k, v, lens, gw, lw, faithful=False)
    assert_close(got, want, TOL, "window-form decode")
    # the heuristic chunking (no split_blocks given) agrees as well
    assert_close(ta.flash_attention_sparse_decoding(qd, kd, vd, cu.cuda(), gw, lw), want, TOL, "default chunks")


@pytest.mark.parametrize("Hq,Hkv,D", [(64, 1, 128), (80, 2, 64), (33, 1, 96), (96, 1, 128)])
def test_decode_with_more_than_32_query_heads_per_kv_head(Hq, Hkv, D):
    """The reference decodes any Hq / Hkv (one program per query head,
    flash_attn_decoding.py:42-45,264-268); here the group is walked in slices
    of 32 query heads."""
    import tritonops_amd as ta

    lens = torch.tensor([1000, 1, 0, 2049, 333], dtype=torch.int32)
    B, L = lens.numel(), 2112
    q, k, v = randn((B, Hq, D), 1), randn((B, L, Hkv, D), 2), randn((B, L, Hkv, D), 3)
    want = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)
    got, lse = ta.flash_attention_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(), return_lse=True)
    assert_close(got, want, TOL, "MQA/GQA decode")
    assert (got[2] == 0).all() and torch.isinf(lse[2]).all()
    # block-list form with the same group sizes
    idx = torch.tensor([0, 3, 7], dtype=torch.int32).expand(B, Hkv, 3).contiguous()
    cnt = torch.tensor([3, 0, 0, 3, 3], dtype=torch.int32)[:, None].expand(B, Hkv).contiguous()
    got = ta.flash_attention_sparse_decoding(q.cuda(), k.cuda(), v.cuda(), None, seq_lens=lens.cuda(),
                                             block_indices=idx.cuda(), block_counts=cnt.cuda())
    want = orc.block_sparse_decoding(q, k, v, lens, idx, cnt, faithful=False)
    assert_close(got, want, TOL, "MQA/GQA block-list decode")
