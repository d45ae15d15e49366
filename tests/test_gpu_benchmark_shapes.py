"""GPU parity at the full benchmark shapes that the other test files reach only
in reduced form: block-sparse prefill at B2 H16 S16384, block-list decoding at
B32 Hkv8 KV131072 with 128 listed blocks + the last one, the dense backward
at B4 H32 S8192, and the window prefill without block lists on 32768 tokens.  Inputs of these sizes are drawn on the device; the checks
are the CPU oracle on slices that it finishes in seconds, fp32 torch math on
the device for sampled heads, and size-independent properties."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close

pytestmark = pytest.mark.gpu


def _randn_dev(shape, seed, dtype=torch.bfloat16):
    g = torch.Generator(device="cuda").manual_seed(seed)
    out = torch.empty(shape, device="cuda", dtype=dtype)
    flat = out.view(-1)
    step = 1 << 28
    for s in range(0, flat.numel(), step):
        n = min(step, flat.numel() - s)
        flat[s:s + n] = torch.randn(n, generator=g, device="cuda", dtype=torch.float32).to(dtype)
    return out


def test_block_sparse_prefill_at_the_benchmark_shape():
    """All 32 (batch, head) units of B2 H16 S16384 with the benchmark mask (so
    the launch takes the XCD-aware item mapping at its real size): sampled
    query blocks of every unit against masked fp32 math on the device, and two
    (b, h) units of the first 2048 tokens against the CPU oracle."""
    import tritonops_amd as ta
    from tritonops_amd import masks

    B, H, S, D = 2, 16, 16384, 128
    m = masks.synthetic_block_mask(S // 64, 8, 4, 0.10, seed=2)
    assert int(m.sum()) == 5995
    q, k, v = (_randn_dev((B, H, S, D), s) for s in (0, 1, 2))
    o, lse = ta.flash_attn_sparse_triton(q, k, v, None, block_mask=m)
    assert o.shape == (B, H, S, D) and lse.shape == (B, H, S)
    bm = torch.from_numpy(m).cuda()
    keys = torch.arange(S, device="cuda")
    for qb in (0, 3, 64, 129, 255):
        rows = torch.arange(qb * 64, qb * 64 + 64, device="cuda")
        allow = bm[qb][keys // 64][None, :] & (keys[None, :] <= rows[:, None])
        s = torch.einsum("bhid,bhjd->bhij", q[:, :, rows].float(), k.float()) * D ** -0.5
        s = s.masked_fill(~allow, float("-inf"))
        ref = torch.einsum("bhij,bhjd->bhid", torch.softmax(s, -1), v.float())
        assert_close(o[:, :, rows], ref, TOL, "query block %d" % qb)
        assert (lse[:, :, rows] - torch.logsumexp(s, -1) * orc.LOG2E).abs().max().item() <= LSE_TOL
    # rows of the first 32 blocks only see keys of the first 32 blocks: the CPU
    # oracle on that prefix with the mask's top-left corner
    n = 2048
    cu = torch.tensor([0, n], dtype=torch.int32)
    for b, h in ((0, 0), (1, 15)):
        sl = lambda t: t[b, h, :n].cpu()[None, :, None, :]
        want, want_lse = orc.block_sparse_attention(sl(q), sl(k), sl(v), cu, m[:32, :32], faithful=False,
                                                    return_lse=True)
        assert_close(o[b, h, :n].cpu()[None, :, None, :], want, TOL, "oracle b%d h%d" % (b, h))
        assert (lse[b, h, :n].cpu()[None, :, None] - want_lse).abs().max().item() <= LSE_TOL


def test_block_list_decode_at_the_benchmark_shape():
    """B32 Hq32 Hkv8 KV131072 D128: 128 sorted block indices per (sequence,
    kv-head) + the block of the newest token (partial: len = 131072 - r).  Some
    lists also NAME the last block, which must still count once, in the chunk
    of the implicit entry as well as in another chunk.  Four sequences against
    the CPU oracle, the chunking against itself, constant V over the batch."""
    import tritonops_amd as ta
    from tritonops_amd import masks

    B, Hq, Hkv, L, D = 32, 32, 8, 131072, 128
    lens = (L - torch.randint(0, 64, (B,), generator=torch.Generator().manual_seed(1))).to(torch.int32)
    lens[5] = L                                        # a full last block
    lens[9] = L - 63                                   # one token in the last block
    idx = masks.synthetic_decode_blocks(B, Hkv, L // 64, 128, seed=2)
    assert int(idx.max()) < L // 64 - 1 and bool((idx[..., 1:] > idx[..., :-1]).all())
    idx[3, :, -1] = L // 64 - 1                        # last block listed as well as implicit
    idx[17, 2, -1] = L // 64 - 1
    q = _randn_dev((B, Hq, D), 0)
    kc, vc = _randn_dev((B, Hkv, L, D), 1), _randn_dev((B, Hkv, L, D), 2)
    k, v = kc.transpose(1, 2), vc.transpose(1, 2)
    lens_d, idx_d = lens.cuda(), idx.cuda()
    got, lse = ta.flash_attention_sparse_decoding(q, k, v, None, seq_lens=lens_d, block_indices=idx_d,
                                                  return_lse=True)
    assert got.shape == (B, Hq, D) and torch.isfinite(got.float()).all() and torch.isfinite(lse).all()
    for b in (0, 3, 9, 17):
        want, want_lse = orc.block_sparse_decoding(q[b:b + 1].cpu(), k[b:b + 1].cpu(), v[b:b + 1].cpu(),
                                                   lens[b:b + 1], idx[b:b + 1], faithful=False, return_lse=True)
        assert_close(got[b:b + 1], want, TOL, "sequence %d" % b)
        assert (lse[b:b + 1].cpu() - want_lse).abs().max().item() <= LSE_TOL
    # the default is 8 chunks of 17 entries; 16 puts the listed last block (entry 127) and
    # the implicit one (entry 128) into different chunks; 129 is a single chunk
    for sb in (16, 129, 1):
        alt = ta.flash_attention_sparse_decoding(q, k, v, None, seq_lens=lens_d, block_indices=idx_d, split_blocks=sb)
        assert_close(alt, got, 4e-3, "split_blocks=%d" % sb)
    vc.fill_(0.25)
    flat = ta.flash_attention_sparse_decoding(q, k, v, None, seq_lens=lens_d, block_indices=idx_d)
    assert (flat.float() - 0.25).abs().max().item() <= 2e-3        # softmax weights sum to one


def test_dense_backward_at_the_benchmark_shape():
    """B4 H32 S8192 D128 causal: dq, dk, dv of three (batch, head) units against
    autograd through fp32 softmax(q k^T scale) v on the device, and
    d(sum o)/dv summing to the number of queries that see each key."""
    import tritonops_amd as ta
    from tritonops_amd import ops

    B, H, S, D = 4, 32, 8192, 128
    q, k, v, do = (_randn_dev((B, H, S, D), s) for s in (0, 1, 2, 3))
    qs, ks, vs, ds = (t.transpose(1, 2) for t in (q, k, v, do))
    sm = D ** -0.5 * ta.LOG2E
    o, lse = ops._dense_fwd(qs, ks, vs, None, sm, True, None, bhsd=True)
    dq, dk, dv = ops._dense_bwd(qs, ks, vs, o, ds, lse, None, sm, True, None)
    assert dq.shape == qs.shape and dk.shape == ks.shape and dv.shape == vs.shape
    tril = torch.ones(S, S, dtype=torch.bool, device="cuda").tril()
    for b, h in ((0, 0), (2, 17), (3, 31)):
        qr, kr, vr = (t[b, h].float().requires_grad_(True) for t in (q, k, v))
        s = (qr @ kr.T) * D ** -0.5
        ref = torch.softmax(s.masked_fill(~tril, float("-inf")), -1) @ vr
        assert_close(o[b, :, h], ref.detach(), TOL, "o b%d h%d" % (b, h))
        ref.backward(do[b, h].float())
        for name, g, w in (("dq", dq, qr.grad), ("dk", dk, kr.grad), ("dv", dv, vr.grad)):
            err = (g[b, :, h].float() - w).abs().max().item()
            bound = 3e-2 * max(1.0, w.abs().max().item())
            assert err <= bound, "%s b%d h%d: max abs err %.4g > %.4g" % (name, b, h, err, bound)
        del qr, kr, vr, s, ref
    # do = 1 everywhere: dv[j] = sum_i P[i, j], and summed over j each query row gives 1
    ds1 = torch.ones_like(do).transpose(1, 2)
    _, _, dv1 = ops._dense_bwd(qs, ks, vs, o, ds1, lse, None, sm, True, None)
    col = dv1.float().mean(-1)                                     # [B, S, H]: every column of dv[j] equals sum_i P[i, j]
    assert (col.sum(1) - S).abs().max().item() <= 1e-3 * S


def test_window_prefill_without_lists_at_the_benchmark_shape():
    """One packed sequence of 32768 tokens, 16 heads, local window 4096 / global 128 (bench.py's
    window_long_prefill), through the call without block lists: sampled blocks of query rows of every
    head against masked fp32 math on the device, the same call through the window's block lists, and
    the size-independent property that a local window as long as the sequence is dense causal attention."""
    import tritonops_amd as ta
    from tritonops_amd import ops

    S, H, D, LW, GW = 32768, 16, 128, 4096, 128
    q, k, v = (_randn_dev((1, S, H, D), s) for s in (11, 12, 13))
    cu = torch.tensor([0, S], dtype=torch.int32, device="cuda")
    assert ops.WINDOW_PREFILL_LISTS is None            # the drop-in's own choice: no lists at this window
    o, lse = ta.flash_attn_sparse_triton(q, k, v, cu, None, LW, GW)
    keys = torch.arange(S, device="cuda")
    qh, kh, vh = (t[0].transpose(0, 1).float() for t in (q, k, v))      # [H, S, D]
    for r0 in (0, 64, 4032, 4096, 4160, 20000, S - 64):
        rows = torch.arange(r0, r0 + 64, device="cuda")
        allow = (keys[None, :] <= rows[:, None]) & ((rows[:, None] - keys[None, :] < LW) | (keys[None, :] < GW))
        s = torch.einsum("hqd,hkd->hqk", qh[:, rows], kh) * D ** -0.5
        s = s.masked_fill(~allow[None], float("-inf"))
        want = torch.einsum("hqk,hkd->hqd", torch.softmax(s, -1), vh)
        assert_close(o[0, rows].transpose(0, 1), want, TOL)
        assert (lse[0, rows].transpose(0, 1) - torch.logsumexp(s, -1) * orc.LOG2E).abs().max().item() <= LSE_TOL
    old = ops.WINDOW_PREFILL_LISTS
    try:
        ops.WINDOW_PREFILL_LISTS = True
        o_l, lse_l = ta.flash_attn_sparse_triton(q, k, v, cu, None, LW, GW)
        assert_close(o, o_l, 1e-2)                     # two kernels, two summation orders
        assert (lse - lse_l).abs().max().item() <= LSE_TOL
        del o_l, lse_l
        ops.WINDOW_PREFILL_LISTS = False
        o_full, lse_full = ta.flash_attn_sparse_triton(q, k, v, cu, None, S, 0)
    finally:
        ops.WINDOW_PREFILL_LISTS = old
    o_dense, lse_dense = ta.flash_attn_triton_fwd(q, k, v, cu, D ** -0.5 * orc.LOG2E)
    assert_close(o_full, o_dense, 1e-2)
    assert (lse_full - lse_dense).abs().max().item() <= LSE_TOL
