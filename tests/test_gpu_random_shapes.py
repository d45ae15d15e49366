"""Seeded random shapes for the kernels whose tile loops are split into masked
and unmasked steps (dense backward, block-sparse prefill): ragged lengths on
either side of the tile sizes, every head_dim, both dtypes, GQA groups, random
block masks - each case against the CPU oracle."""
import random

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import cu_from, randn

pytestmark = pytest.mark.gpu

LENGTHS = [0, 1, 31, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 383, 385, 511, 513, 700]


def _rel(got, want):
    got, want = got.float().cpu(), want.float()
    assert torch.isfinite(got).all()
    return (got - want).abs().max().item() / max(want.abs().max().item(), 1.0)


@pytest.mark.parametrize("seed", range(8))
def test_backward_random_ragged_batches(seed):
    import tritonops_amd as ta

    rnd = random.Random(seed)
    lens = [rnd.choice(LENGTHS) for _ in range(rnd.randint(1, 4))]
    if sum(lens) == 0:
        lens[0] = 77
    Hkv = rnd.choice([1, 2, 4])
    Hq = Hkv * rnd.choice([1, 2, 4])
    D = rnd.choice([64, 96, 128])
    dt = rnd.choice([torch.bfloat16, torch.float16])
    cu = cu_from(torch.tensor(lens, dtype=torch.int32))
    T = int(cu[-1])
    q, k, v = randn((1, T, Hq, D), 1 + seed, dt), randn((1, T, Hkv, D), 2 + seed, dt), randn((1, T, Hkv, D), 3 + seed, dt)
    do = randn((1, T, Hq, D), 4 + seed, dt)
    want = orc.varlen_masked_attention_backward(q, k, v, do, cu, orc.causal_mask)
    sm = D ** -0.5 * ta.LOG2E
    o, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), sm)
    got = ta.flash_attn_triton_bwd(q.cuda(), k.cuda(), v.cuda(), o, do.cuda(), lse, cu.cuda(), sm)
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert _rel(a, b) <= 3e-2, (name, lens, Hq, Hkv, D, dt)


@pytest.mark.parametrize("seed", range(6))
def test_block_sparse_prefill_random_masks(seed):
    import tritonops_amd as ta

    rnd = random.Random(100 + seed)
    S = rnd.choice([64, 100, 257, 512, 1000, 2048])
    H = rnd.choice([1, 2, 4])
    Hkv = rnd.choice([h for h in (1, 2, 4) if H % h == 0])
    D = rnd.choice([64, 96, 128])
    dt = rnd.choice([torch.bfloat16, torch.float16])
    nb = (S + 63) // 64
    m = torch.rand(nb, nb, generator=torch.Generator().manual_seed(seed)) < rnd.choice([0.1, 0.5, 1.0])
    m = m.tril() | torch.eye(nb, dtype=torch.bool)
    cu = cu_from(torch.tensor([S], dtype=torch.int32))
    q, k, v = randn((1, S, H, D), 10 + seed, dt), randn((1, S, Hkv, D), 11 + seed, dt), randn((1, S, Hkv, D), 12 + seed, dt)
    want = orc.block_sparse_attention(q, k, v, cu, m)
    got, _ = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, block_mask=m)
    assert _rel(got, want) <= 2e-2, (S, H, Hkv, D, dt)


WINDOW_LENGTHS = [1, 31, 33, 64, 65, 127, 128, 192, 200, 257, 320, 384, 513, 700, 1000]


@pytest.mark.parametrize("lists", [True, False], ids=["lists", "no-lists"])
@pytest.mark.parametrize("seed", range(8))
def test_window_sparse_prefill_random_windows(seed, lists, monkeypatch):
    """Ragged batches through the window form with windows small enough that a
    row's first listed tile can lie wholly outside its window (the row then has
    no reference point for its probabilities yet) and with large scores (the
    reference point has to move).  Output and LSE against the oracle; rows
    without any visible key must come back as o = 0, lse = -inf.  Both ways the
    drop-in can run the form: block lists built on the host, and no lists."""
    import tritonops_amd as ta
    from tritonops_amd import ops

    monkeypatch.setattr(ops, "WINDOW_PREFILL_LISTS", lists)
    rnd = random.Random(200 + seed)
    lens = [rnd.choice(WINDOW_LENGTHS) for _ in range(rnd.randint(1, 4))]
    Hkv = rnd.choice([1, 2, 4])
    Hq = Hkv * rnd.choice([1, 2, 4])
    D = rnd.choice([64, 96, 128])
    dt = rnd.choice([torch.bfloat16, torch.float16])
    lw = rnd.choice([1, 16, 32, 33, 64, 100, 128, 200, 512])
    gw = rnd.choice([0, 0, 1, 16, 64, 65, 128, 300])
    amp = rnd.choice([1.0, 1.0, 4.0, 12.0])
    cu = cu_from(torch.tensor(lens, dtype=torch.int32))
    T = int(cu[-1])
    q = randn((1, T, Hq, D), 1 + seed, dt) * amp
    k, v = randn((1, T, Hkv, D), 2 + seed, dt), randn((1, T, Hkv, D), 3 + seed, dt)
    want, want_lse = orc.flash_attn_sparse_torch(q, k, v, cu, None, lw, gw, faithful=False, return_lse=True)
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), None, lw, gw)
    case = (lens, Hq, Hkv, D, dt, lw, gw, amp)
    assert _rel(got, want) <= 2e-2, case
    lse = lse.cpu()
    fin = torch.isfinite(want_lse)
    assert (torch.isfinite(lse) == fin).all(), case
    if fin.any():
        assert (lse[fin] - want_lse[fin]).abs().max().item() <= 2e-2, case


def test_block_list_longer_than_the_list_registers():
    """More than 128 listed blocks per row: the 64-entry list registers are
    reloaded twice along the walk.  A full lower triangle must give the dense
    kernel's result."""
    import tritonops_amd as ta

    S, H, D = 9000, 1, 64
    nb = (S + 63) // 64
    m = torch.ones(nb, nb, dtype=torch.bool).tril()
    cu = cu_from(torch.tensor([S], dtype=torch.int32))
    q, k, v = (randn((1, S, H, D), s) for s in (5, 6, 7))
    got, lse = ta.flash_attn_sparse_triton(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), block_mask=m)
    dense, dlse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), D ** -0.5 * ta.LOG2E)
    assert _rel(got, dense.cpu()) <= 1e-2
    assert (lse - dlse).abs().max().item() <= 2e-2


DENSE_LENGTHS = [0, 1, 2, 31, 33, 64, 65, 128, 129, 192, 255, 256, 257, 300, 384, 385, 511, 513, 640, 769, 1024, 1100]


@pytest.mark.parametrize("seed", range(8))
def test_dense_forward_random_ragged_batches(seed):
    """Up to six sequences per batch, lengths on either side of the 64-key tile
    and the 256-row work item, so that consecutive work items of a workgroup
    have zero to five tiles (the requests of the next item's tiles are counted
    against the output stores of the one before)."""
    import tritonops_amd as ta

    rnd = random.Random(300 + seed)
    lens = [rnd.choice(DENSE_LENGTHS) for _ in range(rnd.randint(1, 6))]
    if sum(lens) == 0:
        lens[0] = 5
    Hkv = rnd.choice([1, 2, 4])
    Hq = Hkv * rnd.choice([1, 2, 4])
    D = rnd.choice([64, 96, 128])
    dt = rnd.choice([torch.bfloat16, torch.float16])
    amp = rnd.choice([1.0, 1.0, 5.0])
    cu = cu_from(torch.tensor(lens, dtype=torch.int32))
    T = int(cu[-1])
    q = randn((1, T, Hq, D), 1 + seed, dt) * amp
    k, v = randn((1, T, Hkv, D), 2 + seed, dt), randn((1, T, Hkv, D), 3 + seed, dt)
    want, want_lse = orc.varlen_masked_attention(q, k, v, cu, orc.causal_mask, None, False, True)
    got, lse = ta.flash_attn_triton_fwd(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), D ** -0.5 * ta.LOG2E)
    case = (lens, Hq, Hkv, D, dt, amp)
    assert _rel(got, want) <= 2e-2, case
    fin = torch.isfinite(want_lse)
    assert (lse.cpu()[fin] - want_lse[fin]).abs().max().item() <= 2e-2, case
