"""Host-side block layouts (CPU)."""
import numpy as np
import pytest
import torch

from tritonops_amd import masks


@pytest.mark.parametrize("lw,gw", [(0, 0), (1, 0), (64, 0), (65, 0), (128, 256), (100, 70), (1000, 1)])
def test_window_block_mask_is_exactly_the_blocks_with_an_allowed_pair(lw, gw):
    n = 7
    L = n * 64
    i = np.arange(L)
    tok = (i[None, :] <= i[:, None]) & ((i[:, None] - i[None, :] < lw) | (i[None, :] < gw))
    want = tok.reshape(n, 64, n, 64).any(axis=(1, 3))
    assert np.array_equal(masks.window_block_mask(n, lw, gw), want)


def test_csr_round_trip_and_broadcast_strides():
    m = masks.synthetic_block_mask(12, band=2, sink=1, frac=0.3, seed=1)
    rp, ci, st = masks.block_mask_to_csr(m, "cpu")
    assert st == (0, 0, 0, 0) and rp.dtype == torch.int32 and rp.shape == (1, 1, 13)
    back = np.zeros_like(m)
    for r in range(12):
        cols = ci[0, 0, rp[0, 0, r]:rp[0, 0, r + 1]].numpy()
        assert np.all(np.diff(cols) > 0)
        back[r, cols] = True
    assert np.array_equal(back, m)
    ms = np.stack([masks.synthetic_block_mask(12, 2, 1, 0.3, seed=s) for s in range(3)])
    rp, ci, st = masks.block_mask_to_csr(ms, "cpu")
    assert st[0] == 0 and st[1] == 13 and st[3] == ci.shape[-1]
    with pytest.raises(ValueError):
        masks.block_mask_to_csr(np.ones((4, 4), dtype=bool), "cpu")


def test_benchmark_mask_has_the_stated_block_count():
    m = masks.synthetic_block_mask(256, 8, 4, 0.10, seed=2)
    assert int(m.sum()) == 5995 and not np.triu(m, 1).any() and m.diagonal().all()


def test_synthetic_decode_blocks():
    idx = masks.synthetic_decode_blocks(2, 3, 2048, 128, seed=2)
    assert idx.shape == (2, 3, 128) and idx.dtype == torch.int32
    assert (idx[..., 1:] > idx[..., :-1]).all() and idx.max() < 2047 and idx.min() >= 0
