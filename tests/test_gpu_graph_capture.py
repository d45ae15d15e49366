"""The entry points allocate nothing, copy nothing and clear nothing on their own
(workspaces come from the caller), so a caller can record them into a HIP graph.
A graph is captured once and replayed several times over changing inputs, with
eager work and synchronisations between the replays; every replay is compared
with the eager result on the same inputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _fill(dst, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    dst.copy_(torch.randn(dst.shape, generator=g, device="cuda", dtype=torch.float32).to(dst.dtype))


def test_forward_decode_rmsnorm_xent_replay_like_eager():
    import tritonops_amd as ta

    B, H, Hkv, S, D = 2, 8, 2, 1024, 128
    q = torch.empty((B, H, S, D), device="cuda", dtype=torch.bfloat16)
    k = torch.empty((B, Hkv, S, D), device="cuda", dtype=torch.bfloat16)
    v = torch.empty_like(k)
    qd = torch.empty((B, H, D), device="cuda", dtype=torch.bfloat16)
    kd = torch.empty((B, 3000, Hkv, D), device="cuda", dtype=torch.bfloat16)
    vd = torch.empty_like(kd)
    lens = torch.tensor([3000, 1777], device="cuda", dtype=torch.int32)
    x = torch.empty((512, 1024), device="cuda", dtype=torch.bfloat16)
    wn = torch.ones(1024, device="cuda", dtype=torch.bfloat16)
    wv = torch.empty((4096, 1024), device="cuda", dtype=torch.bfloat16)
    y = torch.randint(0, 4096, (512,), device="cuda")
    inputs = (q, k, v, qd, kd, vd, x, wv)

    def run():
        o, lse = ta.flash_attention(q, k, v, causal=True, return_lse=True)
        od = ta.flash_attention_decoding(qd, kd, vd, None, seq_lens=lens)
        yn, _ = ta.rmsnorm_fwd(x, wn, 1e-6)
        loss, _ = ta.cross_entropy_fused_fwd(yn, wv, y)
        return o, lse, od, yn, loss

    for i, t in enumerate(inputs):
        _fill(t, 100 + i)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                  # loads the library, sets kernel attributes: not capturable work
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = run()
    for rep in range(4):
        for i, t in enumerate(inputs):
            _fill(t, 1000 * (rep + 1) + i)
        if rep == 2:
            lens.copy_(torch.tensor([5, 2999], device="cuda", dtype=torch.int32))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run()                           # eager, same inputs
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w), rep


def test_packed_forward_and_backward_replay_like_eager():
    import tritonops_amd as ta

    lens = [700, 1, 300, 1023]
    cu = torch.tensor([0, 700, 701, 1001, 2024], device="cuda", dtype=torch.int32)
    T, Hq, Hkv, D = 2024, 8, 4, 128
    q = torch.empty((1, T, Hq, D), device="cuda", dtype=torch.bfloat16)
    k = torch.empty((1, T, Hkv, D), device="cuda", dtype=torch.bfloat16)
    v = torch.empty_like(k)
    do = torch.empty_like(q)
    inputs = (q, k, v, do)
    sm = D ** -0.5 * ta.LOG2E

    def run():
        o, lse = ta.flash_attn_triton_fwd(q, k, v, cu, sm, max_seq_len=max(lens))
        dq, dk, dv = ta.flash_attn_triton_bwd(q, k, v, o, do, lse, cu, sm, max_seq_len=max(lens))
        return o, lse, dq, dk, dv

    for i, t in enumerate(inputs):
        _fill(t, 7 + i)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = run()
    for rep in range(3):
        for i, t in enumerate(inputs):
            _fill(t, 50 * (rep + 1) + i)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run()
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w), rep


def test_sparse_prefill_forms_replay_like_eager():
    """The sparse prefill under capture: a block mask through a prebuilt CSR, and the two-window form both
    ways the drop-in can run it (block lists, which are built once per window pair and kept on the host
    side, and no lists at all).  Packed tensors with rows that belong to no sequence, so the launch that
    zeroes them is part of the graph as well."""
    import tritonops_amd as ta
    from tritonops_amd import masks, ops

    Hq, Hkv, D, lw, gw = 4, 2, 128, 300, 70
    lens = [700, 0, 333]
    T = sum(lens) + 40                                  # 40 rows behind the last sequence
    cu = torch.tensor([0, 700, 700, 1033], device="cuda", dtype=torch.int32)
    q = torch.empty((1, T, Hq, D), device="cuda", dtype=torch.bfloat16)
    k = torch.empty((1, T, Hkv, D), device="cuda", dtype=torch.bfloat16)
    v = torch.empty_like(k)
    inputs = (q, k, v)
    csr = masks.block_mask_to_csr(masks.synthetic_block_mask(11, band=2, sink=1, frac=0.3, seed=5), "cuda")

    def run():
        out = []
        old = ops.WINDOW_PREFILL_LISTS
        try:
            for lists in (True, False):
                ops.WINDOW_PREFILL_LISTS = lists
                out += ta.flash_attn_sparse_triton(q, k, v, cu, None, lw, gw, max_seq_len=700)
        finally:
            ops.WINDOW_PREFILL_LISTS = old
        out += ta.flash_attn_sparse_triton(q, k, v, cu, row_ptr=csr[0], col_idx=csr[1], csr_strides=csr[2], max_seq_len=700)
        return out

    for i, t in enumerate(inputs):
        _fill(t, 300 + i)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                  # loads the library, sets kernel attributes, builds the window's lists
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = run()
    for rep in range(3):
        for i, t in enumerate(inputs):
            _fill(t, 3000 * (rep + 1) + i)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run()
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w), rep
        assert torch.count_nonzero(got[0][0, 1033:]) == 0 and torch.count_nonzero(got[2][0, 1033:]) == 0
