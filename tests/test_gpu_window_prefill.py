"""GPU parity of the window form of the sparse prefill WITHOUT block lists.

flash_attn_sparse_triton(q, k, v, cu, None, local, global) can run on block lists
built on the host (tests/test_gpu_sparse_prefill.py) or hand the two windows to the
library, which then walks each 128-row item's sink tiles and band with the dense
kernel's pipeline (mi_attn_fwd_blocksparse with row_ptr = col_idx = NULL).  The
drop-in picks one per call; here the second is forced and checked against the
oracle's masked softmax (flash_attn_triton/flash_attn_sparse_attn_triton.py:391-442)
and against the first.
"""
import ctypes as C

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from, rand_lengths, randn

pytestmark = pytest.mark.gpu


@pytest.fixture
def no_lists():
    from tritonops_amd import ops
    old = ops.WINDOW_PREFILL_LISTS
    ops.WINDOW_PREFILL_LISTS = False
    yield ops
    ops.WINDOW_PREFILL_LISTS = old


def _inputs(lens, Hq, Hkv, D, dtype=torch.bfloat16):
    cu = cu_from(lens)
    T = int(cu[-1])
    return (randn((1, T, Hq, D), 1, dtype), randn((1, T, Hkv, D), 2, dtype), randn((1, T, Hkv, D), 3, dtype), cu)


def _check(q, k, v, cu, lw, gw, tol=TOL):
    import tritonops_amd as ta

    want, want_lse = orc.flash_attn_sparse_torch(q, k, v, cu, None, lw, gw, faithful=False, return_lse=True)
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, lw, gw)
    assert_close(got, want, tol)
    fin = torch.isfinite(want_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max() <= LSE_TOL
    return got, lse


# windows shorter than a tile, ending inside tiles, longer than every sequence; no global
# window (rows whose first tiles hold no visible key), a global window that meets the band
@pytest.mark.parametrize("lw,gw", [(128, 0), (128, 256), (100, 70), (1, 0), (17, 0), (64, 64), (300, 0), (129, 65),
                                   (5000, 0), (64, 5000), (1, 5000), (2 ** 40, 2 ** 40)])
@pytest.mark.parametrize("D,dtype", [(96, torch.bfloat16), (128, torch.bfloat16), (64, torch.float16)])
def test_window_walk_matches_oracle(no_lists, lw, gw, D, dtype):
    import tritonops_amd as ta

    lens = rand_lengths(4, 1, 700, seed=3)
    q, k, v, cu = _inputs(lens, 4, 2, D, dtype)
    got, _ = _check(q, k, v, cu, lw, gw)
    if lw >= 5000 or gw >= 5000:       # window covers everything -> dense causal
        dense = ta.flash_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda())
        assert_close(got, dense, 1e-2)
    if (lw, gw) == (1, 0):             # only the diagonal -> o = v
        assert_close(got, v.repeat_interleave(2, 2), 1e-6)


@pytest.mark.parametrize("lens,lw,gw", [([2048], 128, 0),              # the reference's own test, :445-503
                                        ([1, 129, 128, 127, 257], 64, 32),
                                        ([1500, 0, 3], 1024, 128),
                                        ([2600], 2048, 100)])
def test_window_walk_on_ragged_batches(no_lists, lens, lw, gw):
    q, k, v, cu = _inputs(lens, 4, 4, 128)
    _check(q, k, v, cu, lw, gw)


def test_the_two_window_paths_agree(no_lists):
    import tritonops_amd as ta

    q, k, v, cu = _inputs([3000, 1700], 8, 2, 128)
    args = (q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, 2048, 128)
    o_walk, lse_walk = ta.flash_attn_sparse_triton(*args)
    no_lists.WINDOW_PREFILL_LISTS = True
    o_list, lse_list = ta.flash_attn_sparse_triton(*args)
    assert_close(o_walk, o_list, 1e-2)       # two kernels, two summation orders
    assert (lse_walk - lse_list).abs().max().item() <= LSE_TOL


def test_window_walk_batched_layout(no_lists):
    import tritonops_amd as ta

    B, Hq, Hkv, S, D, lw, gw = 2, 4, 2, 500, 128, 200, 40
    q, k, v = randn((B, Hq, S, D), 1), randn((B, Hkv, S, D), 2), randn((B, Hkv, S, D), 3)
    o, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), None, None, lw, gw)
    cu = cu_from([S])
    for b in range(B):
        pk = lambda t: t[b].transpose(0, 1).unsqueeze(0).contiguous()
        want, want_lse = orc.flash_attn_sparse_torch(pk(q), pk(k), pk(v), cu, None, lw, gw, faithful=False, return_lse=True)
        assert_close(o[b].transpose(0, 1).unsqueeze(0), want, TOL)
        assert (lse[b].transpose(0, 1).unsqueeze(0).cpu() - want_lse).abs().max() <= LSE_TOL


def test_the_drop_in_picks_a_path_per_call(monkeypatch):
    """Lists for short windows and head_dim 64, the walk for local windows of 2048 tokens or
    more at head_dim 96 / 128; a local window of 0 always takes lists."""
    import tritonops_amd as ta
    from tritonops_amd import masks, ops

    built = []
    real = masks.window_csr
    monkeypatch.setattr(ops._masks, "window_csr", lambda *a, **kw: (built.append(a[1:3]), real(*a, **kw))[1])
    assert ops.WINDOW_PREFILL_LISTS is None
    for D, lw, lists in ((128, 2048, False), (96, 4096, False), (128, 2047, True), (64, 4096, True), (128, 0, True)):
        q, k, v, cu = _inputs([300], 2, 2, D)
        del built[:]
        ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, lw, 64)
        assert bool(built) == lists, (D, lw, built)


def test_no_lists_through_the_c_abi_and_its_refusals():
    """mi_attn_fwd_blocksparse with row_ptr = col_idx = NULL: needs both windows, and gives the
    result of the same call with the window's lists."""
    from tritonops_amd import _lib, masks

    lib = _lib.load()
    S, H, D, lw, gw = 1000, 2, 128, 256, 64
    q, k, v = (randn((1, S, H, D), s).cuda() for s in (1, 2, 3))
    cu = cu_from([S]).cuda()
    outs = []
    for lists in (None, masks.window_csr((S + 63) // 64, lw, gw, "cuda")):
        o = torch.empty_like(q)
        lse = torch.empty((1, S, H), device="cuda", dtype=torch.float32)
        a = _lib.AttnSparseArgs()
        a.struct_size = C.sizeof(a)
        a.dtype = _lib.MI_DTYPE_BF16
        a.q, a.k, a.v, a.o, a.lse = (t.data_ptr() for t in (q, k, v, o, lse))
        for n, t in (("q", q), ("k", k), ("v", v), ("o", o)):
            setattr(a, n + "_stride_s", t.stride(1))
            setattr(a, n + "_stride_h", t.stride(2))
        a.lse_stride_s, a.lse_stride_h = lse.stride(1), lse.stride(2)
        a.cu_seqlens = cu.data_ptr()
        a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = 1, H, H, S, D
        a.block_size, a.window_local, a.window_global = 64, lw, gw
        a.scale_log2 = D ** -0.5 * orc.LOG2E
        if lists is not None:
            a.row_ptr, a.col_idx = lists[0].data_ptr(), lists[1].data_ptr()
            a.row_ptr_stride_b, a.row_ptr_stride_h, a.col_idx_stride_b, a.col_idx_stride_h = lists[2]
        else:
            for wl_, wg_ in ((-1, -1), (0, 64)):
                a.window_local, a.window_global = wl_, wg_
                assert lib.mi_attn_fwd_blocksparse(C.byref(a), None) == -1   # MI_ERR_NULL_POINTER
                assert b"window_local >= 1" in lib.mi_last_error()
            a.window_local, a.window_global = lw, gw
        _lib.check(lib.mi_attn_fwd_blocksparse(C.byref(a), None))
        torch.cuda.synchronize()
        outs.append((o, lse))
    assert_close(outs[0][0], outs[1][0], 1e-2)
    assert (outs[0][1] - outs[1][1]).abs().max().item() <= LSE_TOL
