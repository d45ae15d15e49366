"""mi_decode_noalloc - the decode entry point that allocates nothing - against
mi_decode on the same arguments, through the C ABI.  Both run the same two
kernels; only the home of the split-KV partials differs (a buffer the library
holds in device memory instead of a caller workspace), so the outputs must be
equal bit for bit.  Two calls in a row, the second on a smaller input, show
that partials left behind by the first call are not picked up by the second."""
import ctypes as C

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import TOL, assert_close, randn

pytestmark = pytest.mark.gpu


def _args(q, k, v, o, lse, lens, split_tokens, block_idx=None, split_blocks=0):
    from tritonops_amd import _lib

    B, Hq, D = q.shape
    a = _lib.DecodeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr()
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_b, a.k_stride_s, a.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
    a.v_stride_b, a.v_stride_s, a.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
    a.o_stride_b, a.o_stride_h = o.stride(0), o.stride(1)
    a.seq_lens, a.cu_seqlens = lens.data_ptr(), None
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, Hq, k.shape[2], k.shape[1], D
    a.scale_log2 = D ** -0.5 * 1.4426950408889634
    a.split_tokens = split_tokens
    a.window_local = a.window_global = -1
    if block_idx is not None:
        a.block_idx = block_idx.data_ptr()
        a.block_idx_stride_b, a.block_idx_stride_h = block_idx.stride(0), block_idx.stride(1)
        a.max_blocks, a.block_size, a.split_blocks, a.include_last_block = block_idx.shape[2], 64, split_blocks, 1
    return a


def _both(lib, a, q):
    """(o, lse) of mi_decode with a caller workspace and of mi_decode_noalloc."""
    from tritonops_amd import _lib

    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    B, Hq, D = q.shape
    outs = []
    for noalloc in (False, True):
        o = torch.full((B, Hq, D), float("nan"), device="cuda", dtype=torch.bfloat16)
        lse = torch.full((B, Hq), float("nan"), device="cuda", dtype=torch.float32)
        a.o, a.lse = o.data_ptr(), lse.data_ptr()
        if noalloc:
            a.workspace, a.workspace_bytes = None, 0
            _lib.check(lib.mi_decode_noalloc(C.byref(a), st))
        else:
            nbytes = lib.mi_decode_workspace_bytes(C.byref(a))
            assert 0 < nbytes <= _lib.MI_DECODE_STATIC_SCRATCH_BYTES
            ws = torch.empty(nbytes, device="cuda", dtype=torch.uint8)
            a.workspace, a.workspace_bytes = ws.data_ptr(), nbytes
            _lib.check(lib.mi_decode(C.byref(a), st))
        torch.cuda.synchronize()
        outs.append((o, lse))
    return outs


def test_noalloc_decode_equals_workspace_decode_on_two_calls_in_a_row():
    from tritonops_amd import _lib

    lib = _lib.load()
    # first call: 6 sequences, many chunks per sequence; second call: fewer, shorter
    # sequences and fewer chunks, so most slots of the buffer keep the first call's partials
    for B, Hq, Hkv, L, lens, split in ((6, 16, 4, 4096, [4096, 3000, 1, 0, 2049, 777], 256),
                                       (2, 8, 2, 700, [700, 130], 512)):
        D = 128
        q = randn((B, Hq, D), 1 + B).cuda()
        k, v = randn((B, L, Hkv, D), 2 + B).cuda(), randn((B, L, Hkv, D), 3 + B).cuda()
        lens_t = torch.tensor(lens, dtype=torch.int32)
        lens_d = lens_t.cuda()                       # the struct holds raw addresses: keep every tensor alive
        a = _args(q, k, v, q, q, lens_d, split)
        (o_ws, lse_ws), (o_na, lse_na) = _both(lib, a, q)
        assert torch.equal(o_na, o_ws), "B=%d: outputs differ" % B
        assert torch.equal(lse_na, lse_ws)
        want = orc.flash_attn_decoding_torch(q.cpu(), k.cpu(), v.cpu(), lens_t, faithful=False)
        assert_close(o_na, want, TOL, "B=%d vs oracle" % B)


def test_noalloc_block_list_form_and_size_limit():
    from tritonops_amd import _lib

    lib = _lib.load()
    B, Hq, Hkv, L, D = 3, 8, 2, 2048, 128
    q = randn((B, Hq, D), 11).cuda()
    k, v = randn((B, L, Hkv, D), 12).cuda(), randn((B, L, Hkv, D), 13).cuda()
    lens = torch.tensor([2048, 1000, 65], dtype=torch.int32)
    idx = torch.tensor([[[0, 5, 31], [2, 3, 30]], [[0, 1, 15], [7, 8, 9]], [[0, 1, 0], [1, 0, 0]]], dtype=torch.int32)
    cnt = torch.tensor([[3, 3], [3, 3], [2, 1]], dtype=torch.int32).cuda()
    idx_d, lens_d = idx.cuda(), lens.cuda()          # the struct holds raw addresses: keep every tensor alive
    a = _args(q, k, v, q, q, lens_d, 64, idx_d, 2)
    a.block_cnt = cnt.data_ptr()
    (o_ws, lse_ws), (o_na, lse_na) = _both(lib, a, q)
    assert torch.equal(o_na, o_ws) and torch.equal(lse_na, lse_ws)
    want = orc.block_sparse_decoding(q.cpu(), k.cpu(), v.cpu(), lens, idx, cnt.cpu(), faithful=False)
    assert_close(o_na, want, TOL)
    # partials beyond the static buffer: refused before anything is launched
    big = _args(q, k, v, q, q, lens_d, 64)
    big.batch, big.max_seqlen = 4096, 1 << 20
    rc = lib.mi_decode_noalloc(C.byref(big), None)
    assert lib.mi_status_name(rc).decode() == "MI_ERR_WORKSPACE"


def test_noalloc_decode_recorded_into_a_graph_replays_like_mi_decode():
    """The callers the entry point is for include code under HIP graph
    capture.  After one call outside capture (which looks up the device address
    of the static buffer) a captured call records two kernel launches; every
    replay, over changed inputs and lengths, equals mi_decode bit for bit."""
    from tritonops_amd import _lib

    lib = _lib.load()
    B, Hq, Hkv, L, D = 4, 16, 4, 3000, 128
    q = torch.empty((B, Hq, D), device="cuda", dtype=torch.bfloat16)
    k = torch.empty((B, L, Hkv, D), device="cuda", dtype=torch.bfloat16)
    v = torch.empty_like(k)
    lens = torch.tensor([3000, 1777, 1, 640], device="cuda", dtype=torch.int32)
    o_g = torch.empty_like(q)
    lse_g = torch.empty((B, Hq), device="cuda", dtype=torch.float32)

    def fill(seed):
        g = torch.Generator(device="cuda").manual_seed(seed)
        for t in (q, k, v):
            t.copy_(torch.randn(t.shape, generator=g, device="cuda", dtype=torch.float32).to(t.dtype))

    a = _args(q, k, v, o_g, lse_g, lens, 512)
    fill(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    st = C.c_void_p(side.cuda_stream)
    _lib.check(lib.mi_decode_noalloc(C.byref(a), st))      # first call on this device: outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _lib.check(lib.mi_decode_noalloc(C.byref(a), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    for rep in range(4):
        fill(10 + rep)
        if rep == 2:
            lens.copy_(torch.tensor([5, 2999, 0, 64], device="cuda", dtype=torch.int32))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_lse = o_g.clone(), lse_g.clone()
        o = torch.full_like(q, float("nan"))
        lse = torch.full_like(lse_g, float("nan"))
        b = _lib.DecodeArgs.from_buffer_copy(a)
        b.o, b.lse = o.data_ptr(), lse.data_ptr()
        nbytes = lib.mi_decode_workspace_bytes(C.byref(b))
        ws = torch.empty(nbytes, device="cuda", dtype=torch.uint8)
        b.workspace, b.workspace_bytes = ws.data_ptr(), nbytes
        _lib.check(lib.mi_decode(C.byref(b), None))
        torch.cuda.synchronize()
        assert torch.equal(got_o, o) and torch.equal(got_lse, lse), rep
