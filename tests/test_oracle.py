"""Pins the CPU oracle (oracle/attention_oracle.py) without a GPU.

The reference holds no golden vectors for attention, so each oracle function
is checked against (a) an independent float64 loop evaluation, (b) torch's
scaled_dot_product_attention where its masks can express the case, and (c)
closed forms / invariants that a dropped scale, a wrong mask edge, a wrong
head mapping or a transposed operand would break."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attention_oracle as orc
from tests.util import cu_from, randn


def f32(shape, seed):
    return randn(shape, seed, torch.float32)


# ---------------------------------------------------------------- dense [B,H,N,D]
def test_config1_dense_noncausal_fp32_cpu():
    """The CPU-runnable benchmark configuration: B=1, H=4, S=256, D=64 fp32, scale 1/8, non-causal."""
    q, k, v = (f32((1, 4, 256, 64), s) for s in (0, 1, 2))
    o = orc.full_attention(q, k, v)
    assert o.shape == (1, 4, 256, 64) and o.dtype == torch.float32
    ref = F.scaled_dot_product_attention(q, k, v)
    assert (o - ref).abs().max() < 2e-6
    for h in (0, 3):
        bf, _ = orc.brute_force_rows(q[0, h, :5], k[0, h], v[0, h], [[True] * 256] * 5, 1 / 8)
        assert np.abs(o[0, h, :5].numpy() - bf).max() < 2e-6


@pytest.mark.parametrize("causal", [False, True])
def test_dense_against_float64_loops(causal):
    q, k, v = (f32((1, 2, 8, 4), s) for s in (3, 4, 5))
    o = (orc.causal_attention if causal else orc.full_attention)(q.double(), k.double(), v.double())
    allowed = [[(j <= i) or not causal for j in range(8)] for i in range(8)]
    for h in range(2):
        bf, _ = orc.brute_force_rows(q[0, h], k[0, h], v[0, h], allowed, 0.5)
        assert np.abs(o[0, h].numpy() - bf).max() < 1e-12
    ref = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=causal)
    assert (o - ref).abs().max() < 1e-12


def test_dense_closed_forms():
    B, H, N, D = 1, 2, 33, 16
    k, v = f32((B, H, N, D), 1), f32((B, H, N, D), 2)
    z = torch.zeros(B, H, N, D)
    assert (orc.full_attention(z, k, v) - v.mean(2, keepdim=True)).abs().max() < 1e-6
    run = torch.cumsum(v, 2) / torch.arange(1, N + 1)[None, None, :, None]
    assert (orc.causal_attention(z, k, v) - run).abs().max() < 1e-6
    q = f32((B, H, N, D), 3)
    assert (orc.causal_attention(q, k, v)[:, :, 0] - v[:, :, 0]).abs().max() < 1e-6
    # a query aligned with one key and scaled up selects that key's value row
    qsel = (k[:, :, 7] * 1e4)[:, :, None].expand(B, H, N, D)
    assert (orc.full_attention(qsel, k, v) - v[:, :, 7:8]).abs().max() < 1e-5


# ---------------------------------------------------------------- var-len GQA causal
def test_varlen_gqa_equals_per_sequence_dense_with_repeated_heads():
    lens = [5, 17, 1, 33]
    cu = cu_from(lens)
    T, Hq, Hkv, D = sum(lens), 6, 2, 16
    q, k, v = f32((1, T, Hq, D), 1), f32((1, T, Hkv, D), 2), f32((1, T, Hkv, D), 3)
    o, lse = orc.flash_attn_torch(q, k, v, cu, faithful=True, return_lse=True)
    for i, L in enumerate(lens):
        s, e = int(cu[i]), int(cu[i + 1])
        for h in range(Hq):
            hk = h // 3                                  # AABB grouping
            allowed = [[j <= r for j in range(L)] for r in range(L)]
            bf, bl = orc.brute_force_rows(q[0, s:e, h], k[0, s:e, hk], v[0, s:e, hk], allowed, D ** -0.5)
            assert np.abs(o[0, s:e, h].numpy() - bf).max() < 2e-6
            assert np.abs(lse[0, s:e, h].numpy() - bl).max() < 1e-5
    # wrong grouping (ABAB) must NOT match: guards the head map
    bf_wrong, _ = orc.brute_force_rows(q[0, :5, 1], k[0, :5, 1], v[0, :5, 1],
                                       [[j <= r for j in range(5)] for r in range(5)], D ** -0.5)
    assert np.abs(o[0, :5, 1].numpy() - bf_wrong).max() > 1e-3


def test_varlen_concatenation_and_permutation_invariance():
    lens = [9, 4, 12]
    Hq, Hkv, D = 4, 2, 8
    seqs = [(f32((1, L, Hq, D), 10 + i), f32((1, L, Hkv, D), 20 + i), f32((1, L, Hkv, D), 30 + i))
            for i, L in enumerate(lens)]
    alone = [orc.flash_attn_torch(q, k, v, cu_from([q.shape[1]])) for q, k, v in seqs]
    for order in ([0, 1, 2], [2, 0, 1]):
        q = torch.cat([seqs[i][0] for i in order], 1)
        k = torch.cat([seqs[i][1] for i in order], 1)
        v = torch.cat([seqs[i][2] for i in order], 1)
        o = orc.flash_attn_torch(q, k, v, cu_from([lens[i] for i in order]))
        assert torch.equal(o, torch.cat([alone[i] for i in order], 1))


def test_lse_is_base2_logsumexp_and_normalises():
    cu = cu_from([20])
    q, k, v = f32((1, 20, 2, 8), 1), f32((1, 20, 2, 8), 2), f32((1, 20, 2, 8), 3)
    _, lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
    s2 = torch.einsum("qhd,khd->hqk", q[0], k[0]) * 8 ** -0.5 * orc.LOG2E
    s2 = s2.masked_fill(~orc.causal_mask(20)[None], float("-inf"))
    tot = torch.exp2(s2 - lse[0].T[:, :, None]).sum(-1)
    assert (tot - 1).abs().max() < 1e-5
    assert abs(float(lse[0, 0, 0]) - float(s2[0, 0, 0])) < 1e-6       # single key: lse = score


def test_faithful_mode_rounds_like_the_reference_but_stays_close():
    cu = cu_from([64, 40])
    q, k, v = randn((1, 104, 4, 32), 1), randn((1, 104, 2, 32), 2), randn((1, 104, 2, 32), 3)
    a = orc.flash_attn_torch(q, k, v, cu, faithful=True)
    b = orc.flash_attn_torch(q, k, v, cu, faithful=False)
    assert a.dtype == torch.bfloat16 and (a.float() - b.float()).abs().max() < 2e-2
    assert not torch.equal(a, b)


# ---------------------------------------------------------------- window / block sparse
@pytest.mark.parametrize("lw,gw", [(3, 0), (4, 2), (0, 3), (1, 0), (100, 0), (0, 100), (0, 0)])
def test_window_sparse_against_loops(lw, gw):
    L, D = 13, 4
    cu = cu_from([L, 6])
    q, k, v = f32((1, L + 6, 2, D), 1), f32((1, L + 6, 1, D), 2), f32((1, L + 6, 1, D), 3)
    o, lse = orc.flash_attn_sparse_torch(q, k, v, cu, None, lw, gw, faithful=False, return_lse=True)
    allowed = [[(j <= i) and ((i - j < lw) or (j < gw)) for j in range(L)] for i in range(L)]
    for h in range(2):
        bf, bl = orc.brute_force_rows(q[0, :L, h], k[0, :L, 0], v[0, :L, 0], allowed, D ** -0.5)
        assert np.abs(o[0, :L, h].numpy() - bf).max() < 2e-6
        fin = np.isfinite(bl)
        assert np.array_equal(np.isfinite(lse[0, :L, h].numpy()), fin)
        if fin.any():
            assert np.abs(lse[0, :L, h].numpy()[fin] - bl[fin]).max() < 1e-5
    dense = orc.flash_attn_torch(q, k, v, cu, faithful=False)
    if lw >= 100 or gw >= 100:
        assert (o - dense).abs().max() < 1e-6
    if (lw, gw) == (1, 0):
        assert (o - v.expand(1, L + 6, 2, D)).abs().max() < 1e-6
    if (lw, gw) == (0, 0):
        assert torch.count_nonzero(o) == 0 and torch.isinf(lse).all()
    # the reference-dtype form agrees with the fp32 form on fp32 inputs
    o2 = orc.flash_attn_sparse_torch(q, k, v, cu, None, lw, gw, faithful=True)
    assert (o - o2).abs().max() < 1e-5


def test_block_mask_oracle():
    L = 200
    cu = cu_from([L])
    q, k, v = f32((1, L, 2, 8), 1), f32((1, L, 2, 8), 2), f32((1, L, 2, 8), 3)
    full = np.tril(np.ones((4, 4), dtype=bool))
    assert (orc.block_sparse_attention(q, k, v, cu, full, faithful=False)
            - orc.flash_attn_torch(q, k, v, cu, faithful=False)).abs().max() < 1e-6
    m = np.array([[1, 0, 0, 0], [0, 1, 0, 0], [1, 0, 1, 0], [0, 1, 1, 1]], dtype=bool)
    o = orc.block_sparse_attention(q, k, v, cu, m, faithful=False)
    allowed = [[bool(m[i // 64, j // 64]) and j <= i for j in range(L)] for i in range(L)]
    bf, _ = orc.brute_force_rows(q[0, :, 1], k[0, :, 1], v[0, :, 1], allowed, 8 ** -0.5)
    assert np.abs(o[0, :, 1].numpy() - bf).max() < 2e-6
    # a band of whole blocks differs from the token window only inside the oldest block
    band = np.array([[i - j in (0, 1) for j in range(4)] for i in range(4)])
    ob = orc.block_sparse_attention(q, k, v, cu, band, faithful=False)
    ow = orc.flash_attn_sparse_torch(q, k, v, cu, None, 64, 0, faithful=False)
    assert (ob[0, :64] - ow[0, :64]).abs().max() < 1e-6          # first block: identical key sets
    assert (ob[0, 64:] - ow[0, 64:]).abs().max() > 1e-3


# ---------------------------------------------------------------- decoding
def test_decode_is_last_row_of_noncausal_attention():
    B, Hq, Hkv, D, Lmax = 4, 4, 2, 8, 40
    lens = torch.tensor([40, 7, 1, 0], dtype=torch.int32)
    q, k, v = f32((B, Hq, D), 1), f32((B, Lmax, Hkv, D), 2), f32((B, Lmax, Hkv, D), 3)
    o, lse = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False, return_lse=True)
    for b in range(B):
        L = int(lens[b])
        for h in range(Hq):
            if L == 0:
                assert torch.count_nonzero(o[b, h]) == 0
                continue
            bf, bl = orc.brute_force_rows(q[b, h][None], k[b, :L, h // 2], v[b, :L, h // 2], [[True] * L], D ** -0.5)
            assert np.abs(o[b, h].numpy() - bf[0]).max() < 2e-6
            assert abs(float(lse[b, h]) - bl[0]) < 1e-5
    assert (o[2] - v[2, 0].repeat_interleave(2, 0)).abs().max() < 1e-6          # one key -> its value
    sd = F.scaled_dot_product_attention(q[0][:, None], k[0, :40].transpose(0, 1).repeat_interleave(2, 0),
                                        v[0, :40].transpose(0, 1).repeat_interleave(2, 0))
    assert (o[0] - sd[:, 0]).abs().max() < 2e-6
    # explicit scale is honoured
    o2 = orc.flash_attn_decoding_torch(q, k, v, lens, qk_scale=0.0, faithful=False)
    assert (o2[0] - v[0, :40].mean(0).repeat_interleave(2, 0)).abs().max() < 1e-6


@pytest.mark.parametrize("chunk", [1, 5, 16, 64])
def test_split_kv_merge_is_exact(chunk):
    """Any chunking + the merge formula reproduces the unsplit result."""
    L, H, D = 37, 3, 8
    q, k, v = f32((1, H, D), 1).double(), f32((1, L, H, D), 2).double(), f32((1, L, H, D), 3).double()
    want, want_lse = orc.decode_attention(q, k, v, [L], faithful=True, return_lse=True)
    parts, lses = [], []
    for s in range(0, L, chunk):
        o_c, l_c = orc.decode_attention(q, k[:, s:s + chunk], v[:, s:s + chunk], [min(chunk, L - s)],
                                        faithful=True, return_lse=True)
        parts.append(o_c[0])
        lses.append(l_c[0].double())
    o, lse = orc.merge_partials(torch.stack(parts), torch.stack(lses))
    assert (o - want[0]).abs().max() < 1e-6     # lse partials are fp32
    assert (lse - want_lse[0]).abs().max() < 1e-5


def test_merge_identities():
    o = f32((3, 2, 4), 1)
    l = f32((3, 2), 2)
    one, l1 = orc.merge_partials(o[:1], l[:1])
    assert torch.equal(one, o[0]) and (l1 - l[0]).abs().max() < 1e-6
    ab, lab = orc.merge_partials(o[:2], l[:2])
    abc1, _ = orc.merge_partials(torch.stack([ab, o[2]]), torch.stack([lab, l[2]]))
    abc2, _ = orc.merge_partials(o[[2, 0, 1]], l[[2, 0, 1]])
    assert (abc1 - abc2).abs().max() < 1e-6
    empty = torch.full((2,), float("-inf"))
    m, lm = orc.merge_partials(torch.stack([o[0], torch.zeros(2, 4)]), torch.stack([l[0], empty]))
    assert (m - o[0]).abs().max() < 1e-6 and (lm - l[0]).abs().max() < 1e-6
    # base 2 vs natural log
    assert abs(float(orc.merge_partials(torch.zeros(4, 1, 1), torch.zeros(4, 1))[1]) - 2.0) < 1e-6


@pytest.mark.parametrize("gw,lw", [(2, 3), (4, 0), (64, 64), (2, 100)])
def test_window_decode_against_loops(gw, lw):
    lens = torch.tensor([30, 4, 0, 1], dtype=torch.int32)
    B, H, D = 4, 2, 4
    q, k, v = f32((B, H, D), 1), f32((B, 30, 1, D), 2), f32((B, 30, 1, D), 3)
    o = orc.flash_attn_sparse_decoding_torch(q, k, v, lens, gw, lw, faithful=False)
    dense = orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)
    for b in range(B):
        L = int(lens[b])
        if L == 0:
            continue
        allowed = [[(j < gw) or (j >= L - lw) for j in range(L)]]
        bf, _ = orc.brute_force_rows(q[b, 1][None], k[b, :L, 0], v[b, :L, 0], allowed, D ** -0.5)
        assert np.abs(o[b, 1].numpy() - bf[0]).max() < 2e-6
        if gw + lw >= L:
            assert (o[b] - dense[b]).abs().max() < 1e-6


def test_block_index_decode_oracle():
    B, Hq, Hkv, D, L = 2, 4, 2, 8, 300
    lens = torch.tensor([300, 130], dtype=torch.int32)
    q, k, v = f32((B, Hq, D), 1), f32((B, L, Hkv, D), 2), f32((B, L, Hkv, D), 3)
    allb = torch.arange(5, dtype=torch.int32).expand(B, Hkv, 5).contiguous()
    cnt = torch.tensor([[5, 5], [3, 3]], dtype=torch.int32)
    assert (orc.block_sparse_decoding(q, k, v, lens, allb, cnt, include_last_block=False, faithful=False)
            - orc.flash_attn_decoding_torch(q, k, v, lens, faithful=False)).abs().max() < 1e-6
    idx = torch.tensor([[[0], [2]], [[1], [0]]], dtype=torch.int32)
    o = orc.block_sparse_decoding(q, k, v, lens, idx, faithful=False)
    keep = [j < 64 or j >= 256 for j in range(300)]              # b=0, kv-head 0: block 0 + last block (4)
    bf, _ = orc.brute_force_rows(q[0, 1][None], k[0, :, 0], v[0, :, 0], [keep], D ** -0.5)
    assert np.abs(o[0, 1].numpy() - bf[0]).max() < 2e-6
    keep = [j < 64 or j >= 128 for j in range(130)]              # b=1, kv-head 1: block 0 + last block (2, partial)
    bf, _ = orc.brute_force_rows(q[1, 3][None], k[1, :130, 1], v[1, :130, 1], [keep], D ** -0.5)
    assert np.abs(o[1, 3].numpy() - bf[0]).max() < 2e-6


@pytest.mark.parametrize("causal", [True, False])
def test_backward_formulas_match_autograd(causal):
    """The closed-form gradients against torch.autograd through an independent
    float64 evaluation of the forward (plain softmax over masked scores), GQA 2,
    ragged packed batch incl. a length-0 and a length-1 sequence."""
    torch.manual_seed(0)
    lens = torch.tensor([5, 0, 1, 37, 64], dtype=torch.int32)
    cu = torch.cat([torch.zeros(1, dtype=torch.int32), torch.cumsum(lens, 0).to(torch.int32)])
    T, Hq, Hkv, D = int(cu[-1]), 4, 2, 16
    q = torch.randn(1, T, Hq, D, dtype=torch.float64, requires_grad=True)
    k = torch.randn(1, T, Hkv, D, dtype=torch.float64, requires_grad=True)
    v = torch.randn(1, T, Hkv, D, dtype=torch.float64, requires_grad=True)
    do = torch.randn(1, T, Hq, D, dtype=torch.float64)
    mask_fn = orc.causal_mask if causal else (lambda L: torch.ones(L, L, dtype=torch.bool))
    outs = []
    for b in range(len(lens)):
        s, e = int(cu[b]), int(cu[b + 1])
        if e == s:
            continue
        kk = k[0, s:e].repeat_interleave(Hq // Hkv, dim=1)
        vv = v[0, s:e].repeat_interleave(Hq // Hkv, dim=1)
        sc = torch.einsum("qhd,khd->hqk", q[0, s:e], kk) / math.sqrt(D)
        sc = sc.masked_fill(~mask_fn(e - s)[None], float("-inf"))
        outs.append(torch.einsum("hqk,khd->qhd", torch.softmax(sc, -1), vv))
    o = torch.cat(outs)
    (o * do[0]).sum().backward()
    dq, dk, dv = orc.varlen_masked_attention_backward(q.detach(), k.detach(), v.detach(), do, cu, mask_fn)
    assert (dq - q.grad).abs().max() < 1e-10
    assert (dk - k.grad).abs().max() < 1e-10
    assert (dv - v.grad).abs().max() < 1e-10
    # a dropped term must fail: without Delta the q gradient is wrong
    assert (dq - q.grad).abs().max() < 1e-10 < q.grad.abs().max()
