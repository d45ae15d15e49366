"""Block layouts for the sparse kernels: window -> block list, block mask -> CSR,
and the seeded synthetic layouts used by the benchmark configurations.

Block edge is 64 tokens everywhere (MI_ATTN_BLOCK).  All builders run on the
host with numpy (the layouts are tiny) and return int32 torch tensors on the
requested device.
"""
import numpy as np
import torch

BLOCK = 64


def window_block_mask(n_blocks, local_window, global_window):
    """Boolean [n_blocks, n_blocks] mask of 64x64 blocks that contain at least
    one allowed (q, k) pair of the reference's window rule
    (flash_attn_triton/flash_attn_sparse_attn_triton.py:422-433):
        k <= q and (q - k < local_window or k < global_window).
    """
    i = np.arange(n_blocks)[:, None]
    j = np.arange(n_blocks)[None, :]
    causal = j <= i
    sink = (j * BLOCK) < global_window
    # closest pair of block i (queries) and block j <= i (keys): distance
    # 64*(i-j) - 63 for j < i, 0 on the diagonal
    mind = np.where(i == j, 0, BLOCK * (i - j) - (BLOCK - 1))
    local = mind < local_window
    return causal & (sink | local)


_WINDOW_CSR = {}


def window_csr(n_blocks, local_window, global_window, device):
    """CSR (row_ptr, col_idx, strides) of window_block_mask on `device`, built
    once per (n_blocks, windows, device) and kept: a layer calls with the same
    windows every step, so nothing is rebuilt or copied to the device per call."""
    key = (int(n_blocks), int(local_window), int(global_window), str(torch.device(device)))
    hit = _WINDOW_CSR.get(key)
    if hit is None:
        if len(_WINDOW_CSR) >= 64:
            _WINDOW_CSR.clear()
        hit = block_mask_to_csr(window_block_mask(*key[:3]), device)
        _WINDOW_CSR[key] = hit
    return hit


def block_mask_to_csr(mask, device):
    """mask: bool array/tensor [..., nq, nk] with up to two leading (batch,
    head) axes.  Returns (row_ptr, col_idx, strides) where strides =
    (row_ptr_stride_b, row_ptr_stride_h, col_idx_stride_b, col_idx_stride_h);
    axes of extent 1 broadcast (stride 0).  Only blocks on or below the
    diagonal may be set."""
    m = np.asarray(mask.cpu() if isinstance(mask, torch.Tensor) else mask).astype(bool)
    if m.ndim == 2:
        m = m[None, None]
    elif m.ndim == 3:
        m = m[None]
    if m.ndim != 4 or m.shape[-1] != m.shape[-2]:
        raise ValueError("block mask must be [nq, nq], [H, nq, nq] or [B, H, nq, nq]")
    B, H, nq, _ = m.shape
    if np.triu(m, 1).any():
        raise ValueError("block mask has live blocks above the diagonal (the kernel is causal)")
    counts = m.sum(-1)                                   # [B, H, nq]
    row_ptr = np.zeros((B, H, nq + 1), dtype=np.int32)
    row_ptr[..., 1:] = np.cumsum(counts, -1)
    cap = max(int(row_ptr[..., -1].max()), 1)
    col_idx = np.zeros((B * H, cap), dtype=np.int32)
    unit, _, cols = np.nonzero(m.reshape(B * H, nq, nq))  # row-major => ascending per row
    first = np.concatenate(([0], np.cumsum(row_ptr[..., -1].reshape(-1))[:-1]))
    col_idx[unit, np.arange(unit.size) - first[unit]] = cols
    col_idx = col_idx.reshape(B, H, cap)
    strides = (
        0 if B == 1 else H * (nq + 1), 0 if H == 1 else (nq + 1),
        0 if B == 1 else H * cap, 0 if H == 1 else cap,
    )
    return (torch.from_numpy(row_ptr).to(device), torch.from_numpy(col_idx).to(device), strides)


def synthetic_block_mask(n_blocks, band=8, sink=4, frac=0.10, seed=2):
    """Causal diagonal band of `band` blocks + `sink` leading blocks + a seeded
    uniform sample (without replacement) of `frac` of the remaining lower-
    triangular blocks."""
    i = np.arange(n_blocks)[:, None]
    j = np.arange(n_blocks)[None, :]
    base = (j <= i) & ((i - j < band) | (j < sink))
    rest = np.argwhere((j <= i) & ~base)
    g = torch.Generator().manual_seed(seed)
    n_take = int(round(frac * len(rest)))
    pick = torch.randperm(len(rest), generator=g)[:n_take].numpy()
    m = base.copy()
    m[rest[pick, 0], rest[pick, 1]] = True
    return m


def synthetic_decode_blocks(batch, heads_kv, n_blocks_total, top_k=128, seed=2):
    """Per (batch, kv-head): `top_k` sorted unique block indices drawn from
    blocks [0, n_blocks_total - 1) (the final block is added by the caller)."""
    g = torch.Generator().manual_seed(seed)
    out = torch.empty(batch, heads_kv, top_k, dtype=torch.int32)
    for b in range(batch):
        for h in range(heads_kv):
            out[b, h] = torch.sort(torch.randperm(n_blocks_total - 1, generator=g)[:top_k]).values.to(torch.int32)
    return out
