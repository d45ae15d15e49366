"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's PyTorch attention math.

Nothing in the product package (tritonops_amd) may import this module; only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it, as the
checker.  Each function restates one of the reference's in-file torch oracles
(paths relative to the reference checkout) and keeps that oracle's precision
choices when `faithful=True` (which matmul runs in the storage dtype, where
the cast to fp32 happens); `faithful=False` does the same mathematics in fp32
or fp64 throughout.

Pinning (tests/test_oracle.py): the reference ships no golden vectors for this
path, so every function here is pinned against an independent float64 numpy
triple-loop evaluation of softmax(q.k*scale + mask).v, against
torch.nn.functional.scaled_dot_product_attention where the mask is expressible,
and against closed forms (zero queries -> running mean of v, a single key ->
v itself, one-hot huge queries -> row selection, split invariance of the
merge); the backward formulas against torch.autograd through the forward.  Parity against the third-party `flash_attn` wheel, which the reference
uses as a second oracle (flash_attn_triton/flash_attn_triton.py:965-975), is
UNPINNED: that wheel is not installed and is not vendored by the reference.
"""
import math

import numpy as np
import torch

LOG2E = 1.4426950408889634
BLOCK = 64


# --------------------------------------------------------------------------
# dense [B, H, N, D]
# --------------------------------------------------------------------------
def full_attention(q, k, v):
    """Non-causal softmax(q k^T / sqrt(d)) v on [B,H,N,D], everything in the
    input dtype - tutorial/4.3.multi_head_attention.py:11-19."""
    d = q.shape[-1]
    w = torch.einsum("bhid,bhjd->bhij", q, k) / math.sqrt(d)
    w = torch.softmax(w, dim=-1)
    return torch.einsum("bhij,bhjd->bhid", w, v)


def causal_attention(q, k, v):
    """Causal variant: keys j > i are filled with -inf before the softmax -
    tutorial/4.4.causal_attention.py:22-32."""
    n, d = q.shape[-2], q.shape[-1]
    w = torch.einsum("bhid,bhjd->bhij", q, k) / math.sqrt(d)
    keep = torch.ones(n, n, dtype=torch.bool).tril()
    w = w.masked_fill(~keep, float("-inf"))
    w = torch.softmax(w, dim=-1)
    return torch.einsum("bhij,bhjd->bhid", w, v)


# --------------------------------------------------------------------------
# packed var-len GQA, generic mask
# --------------------------------------------------------------------------
def _lengths(cu):
    cu = [int(x) for x in cu]
    return [(cu[i], cu[i + 1]) for i in range(len(cu) - 1)]


def _expand_kv(x, hq):
    """AABB head sharing: q-head h reads kv-head h // (hq // hkv)
    (flash_attn_triton/flash_attn_triton.py:885-886, kernel :86-87)."""
    hkv = x.shape[2]
    return x.repeat_interleave(hq // hkv, dim=2)


def varlen_masked_attention(q, k, v, cu_seq_lens, mask_fn, scale=None, faithful=True, return_lse=False):
    """softmax over the keys allowed by mask_fn(seq_len) -> bool [L, L] for
    every sequence of a packed batch; q [1,T,Hq,D], k/v [1,T,Hkv,D].

    faithful=True follows flash_attn_torch
    (flash_attn_triton/flash_attn_triton.py:877-915): q.k^T and the scale in the
    storage dtype, cast to fp32, fp32 softmax, probabilities cast back to the
    storage dtype, p.v in the storage dtype.  Rows with no allowed key give 0
    (and lse = -inf) instead of the NaN a softmax over all -inf would give.
    lse (optional) is log2 sum 2^(s*log2e) over the allowed keys, from fp32
    scores (kernel definition, flash_attn_triton.py:163,170,180).
    """
    _, T, H, D = q.shape
    kk, vv = _expand_kv(k, H), _expand_kv(v, H)
    if scale is None:
        scale = (1 / D) ** 0.5
    work = q.dtype if faithful else torch.float32
    o = torch.zeros(1, T, H, v.shape[-1], dtype=q.dtype)
    lse = torch.full((1, T, H), float("-inf"), dtype=torch.float32)
    for s, e in _lengths(cu_seq_lens):
        L = e - s
        if L == 0:
            continue
        keep = mask_fn(L)
        sc = torch.einsum("qhd,khd->hqk", q[0, s:e].to(work), kk[0, s:e].to(work)) * scale
        sc = sc.masked_fill(~keep[None], float("-inf")).to(torch.float32)
        dead = ~keep.any(-1)                                    # rows with no key
        sc_safe = sc.masked_fill(dead[None, :, None], 0.0)
        p = torch.softmax(sc_safe, dim=-1, dtype=torch.float32)
        p = p.masked_fill(dead[None, :, None], 0.0)
        o[0, s:e] = torch.einsum("hqk,khd->qhd", p.to(work), vv[0, s:e].to(work)).to(q.dtype)
        if return_lse:
            sc32 = torch.einsum("qhd,khd->hqk", q[0, s:e].float(), kk[0, s:e].float()) * scale
            sc32 = sc32.masked_fill(~keep[None], float("-inf"))
            l2 = torch.logsumexp(sc32, dim=-1) * LOG2E            # [H, L]
            l2 = l2.masked_fill(dead[None], float("-inf"))
            lse[0, s:e] = l2.transpose(0, 1)
    return (o, lse) if return_lse else o


def varlen_masked_attention_backward(q, k, v, do, cu_seq_lens, mask_fn, scale=None):
    """Gradients of varlen_masked_attention(faithful=False) with respect to q, k
    and v for an upstream gradient `do`, by the closed formulas the reference's
    backward kernels implement (flash_attn_triton/flash_attn_triton.py:183-593;
    its test compares them with autograd through the torch path, :1086-1089):
        P = softmax(S),  dV = P^T dO,  dP = dO V^T,  Delta = rowsum(dO o O),
        dS = P o (dP - Delta),  dQ = dS K scale,  dK = dS^T Q scale,
    in float64, the gradients of the query heads sharing a kv-head summed
    (:687-692,813).  q/do [1,T,Hq,D], k/v [1,T,Hkv,D]; returns float64
    (dq, dk, dv) of the same shapes.  Pinned against torch.autograd in
    tests/test_oracle.py."""
    _, T, H, D = q.shape
    hkv = k.shape[2]
    g = H // hkv
    if scale is None:
        scale = (1 / D) ** 0.5
    dq = torch.zeros(1, T, H, D, dtype=torch.float64)
    dk = torch.zeros(1, T, hkv, D, dtype=torch.float64)
    dv = torch.zeros(1, T, hkv, D, dtype=torch.float64)
    for s, e in _lengths(cu_seq_lens):
        L = e - s
        if L == 0:
            continue
        keep = mask_fn(L)
        qq, dd = q[0, s:e].double(), do[0, s:e].double()            # [L, H, D]
        kk = k[0, s:e].double().repeat_interleave(g, dim=1)
        vv = v[0, s:e].double().repeat_interleave(g, dim=1)
        sc = torch.einsum("qhd,khd->hqk", qq, kk) * scale
        sc = sc.masked_fill(~keep[None], float("-inf"))
        dead = ~keep.any(-1)
        p = torch.softmax(sc.masked_fill(dead[None, :, None], 0.0), dim=-1).masked_fill(dead[None, :, None], 0.0)
        o = torch.einsum("hqk,khd->qhd", p, vv)
        delta = (o * dd).sum(-1).transpose(0, 1)                    # [H, L]
        dp = torch.einsum("qhd,khd->hqk", dd, vv)
        ds = p * (dp - delta[:, :, None])
        dq[0, s:e] = torch.einsum("hqk,khd->qhd", ds, kk) * scale
        dk_h = torch.einsum("hqk,qhd->khd", ds, qq) * scale          # per q-head
        dv_h = torch.einsum("hqk,qhd->khd", p, dd)
        dk[0, s:e] = dk_h.reshape(L, hkv, g, D).sum(2)
        dv[0, s:e] = dv_h.reshape(L, hkv, g, D).sum(2)
    return dq, dk, dv


def causal_mask(L):
    i = torch.arange(L)
    return i[:, None] >= i[None, :]


def flash_attn_torch(q, k, v, cu_seq_lens, faithful=True, return_lse=False):
    """Causal var-len GQA attention, scale D^-0.5 -
    flash_attn_triton/flash_attn_triton.py:877-915."""
    return varlen_masked_attention(q, k, v, cu_seq_lens, causal_mask, None, faithful, return_lse)


def window_mask(local_window, global_window):
    """allowed(q, k) = k <= q and (q < k + local or k < global) -
    flash_attn_triton/flash_attn_sparse_attn_triton.py:422-433."""
    def fn(L):
        i = torch.arange(L)
        qi, kj = i[:, None], i[None, :]
        return (qi >= kj) & ((qi < kj + local_window) | (kj < global_window))
    return fn


def flash_attn_sparse_torch(q, k, v, cu_seqlens, softmax_scale=None, local_window_size=0,
                            global_window_size=0, faithful=True, return_lse=False):
    """Window-sparse causal attention.  The reference oracle
    (flash_attn_triton/flash_attn_sparse_attn_triton.py:391-442) does q.k^T, the
    scale, the softmax and p.v all in the storage dtype; with faithful=True the
    softmax here is also taken in the storage dtype to match (:437)."""
    _, T, H, D = q.shape
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if not faithful:
        return varlen_masked_attention(q, k, v, cu_seqlens, window_mask(local_window_size, global_window_size),
                                       softmax_scale, False, return_lse)
    G = H // k.shape[2]
    o = torch.zeros_like(q)
    fn = window_mask(local_window_size, global_window_size)
    for s, e in _lengths(cu_seqlens):
        L = e - s
        if L == 0:
            continue
        keep = fn(L)
        dead = ~keep.any(-1)
        for h in range(H):
            sc = q[0, s:e, h] @ k[0, s:e, h // G].T
            sc = torch.where(keep, sc, torch.full_like(sc, float("-inf"))) * softmax_scale
            sc = sc.masked_fill(dead[:, None], 0.0)
            p = sc.softmax(dim=-1).masked_fill(dead[:, None], 0.0)
            o[0, s:e, h] = p @ v[0, s:e, h // G]
    if return_lse:
        _, lse = varlen_masked_attention(q, k, v, cu_seqlens, fn, softmax_scale, False, True)
        return o, lse
    return o


def block_mask_token_mask(block_mask):
    """Token mask of a causal 64x64 block layout: block (i, j) live and k <= q.
    block_mask: bool [nq, nq] numpy/torch."""
    bm = torch.as_tensor(np.asarray(block_mask)).bool()

    def fn(L):
        i = torch.arange(L)
        bi = i // BLOCK
        return bm[bi[:, None], bi[None, :]] & (i[:, None] >= i[None, :])
    return fn


def block_sparse_attention(q, k, v, cu_seqlens, block_mask, softmax_scale=None, faithful=True, return_lse=False):
    """Generalisation of the window oracle to an arbitrary causal block mask
    (one mask for all heads): same arithmetic as flash_attn_torch under the
    token mask of block_mask_token_mask()."""
    return varlen_masked_attention(q, k, v, cu_seqlens, block_mask_token_mask(block_mask), softmax_scale,
                                   faithful, return_lse)


# --------------------------------------------------------------------------
# decoding
# --------------------------------------------------------------------------
def decode_attention(q, k, v, seq_lens, key_mask_fn=None, qk_scale=None, faithful=True, return_lse=False):
    """Single-query attention.  q [B,Hq,D]; k, v padded [B,maxL,Hkv,D]; only the
    first seq_lens[b] tokens count; key_mask_fn(b, kv_head, L) -> bool [L]
    restricts the keys further (None = all).

    faithful=True follows flash_attn_decoding_torch
    (flash_attn_triton/flash_attn_decoding.py:339-368): q.k in the storage
    dtype, scale, softmax in the storage dtype, p.v in the storage dtype.  (That
    oracle takes packed KV already expanded to Hq heads, :357-359 and
    flash_attn_decoding_sparse.py:479-488; the padded GQA form here is what the
    launcher takes, flash_attn_decoding.py:213-219.)  Length 0, or no allowed
    key, gives a zero row.
    """
    B, H, D = q.shape
    Hkv = k.shape[2]
    G = H // Hkv
    if qk_scale is None:
        qk_scale = D ** -0.5
    work = q.dtype if faithful else torch.float32
    o = torch.zeros(B, H, v.shape[-1], dtype=q.dtype)
    lse = torch.full((B, H), float("-inf"), dtype=torch.float32)
    for b in range(B):
        L = int(seq_lens[b])
        if L == 0:
            continue
        for hk in range(Hkv):
            keep = torch.ones(L, dtype=torch.bool) if key_mask_fn is None else key_mask_fn(b, hk, L)
            if not keep.any():
                continue
            qb = q[b, hk * G:(hk + 1) * G].to(work)                 # [G, D]
            kb = k[b, :L, hk].to(work)[keep]                        # [L', D]
            vb = v[b, :L, hk].to(work)[keep]
            sc = (qb @ kb.T).to(work) * qk_scale
            p = sc.softmax(dim=-1)
            o[b, hk * G:(hk + 1) * G] = (p.to(work) @ vb).to(q.dtype)
            if return_lse:
                s32 = (q[b, hk * G:(hk + 1) * G].float() @ k[b, :L, hk].float()[keep].T) * qk_scale
                lse[b, hk * G:(hk + 1) * G] = torch.logsumexp(s32, dim=-1) * LOG2E
    return (o, lse) if return_lse else o


def flash_attn_decoding_torch(q, k, v, seq_lens, qk_scale=None, faithful=True, return_lse=False):
    """Dense decoding - flash_attn_triton/flash_attn_decoding.py:339-368."""
    return decode_attention(q, k, v, seq_lens, None, qk_scale, faithful, return_lse)


def flash_attn_sparse_decoding_torch(q, k, v, seq_lens, global_window_size=64, local_window_size=64,
                                     faithful=True, return_lse=False):
    """Window decoding: keys k < global or k >= len - local -
    flash_attn_triton/flash_attn_decoding_sparse.py:368-406 (mask :391-396)."""
    def fn(b, hk, L):
        i = torch.arange(L)
        return (L <= i + local_window_size) | (i < global_window_size)
    return decode_attention(q, k, v, seq_lens, fn, None, faithful, return_lse)


def block_sparse_decoding(q, k, v, seq_lens, block_indices, block_counts=None, include_last_block=True,
                          faithful=True, return_lse=False):
    """Block-index decoding: kv-head hk of sequence b attends the 64-token blocks
    block_indices[b, hk, :count] (+ the block of the newest token)."""
    def fn(b, hk, L):
        n = block_indices.shape[2] if block_counts is None else int(block_counts[b, hk])
        keep = torch.zeros(L, dtype=torch.bool)
        blocks = [int(x) for x in block_indices[b, hk, :n]]
        if include_last_block:
            blocks.append((L - 1) // BLOCK)
        for j in blocks:
            keep[j * BLOCK:min((j + 1) * BLOCK, L)] = True
        return keep
    return decode_attention(q, k, v, seq_lens, fn, None, faithful, return_lse)


def merge_partials(o_parts, lse2_parts):
    """LSE merge of split-KV partials, fp32 -
    flash_attn_triton/flash_attn_decoding.py:171-208:
    lse = log2 sum_c 2^lse_c ;  o = sum_c o_c 2^(lse_c - lse).
    o_parts [C, ..., D], lse2_parts [C, ...]."""
    m = lse2_parts.max(dim=0).values
    m_safe = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    w = torch.exp2(lse2_parts - m_safe)
    den = w.sum(0)
    lse = m_safe + torch.log2(den)
    lse = torch.where(den > 0, lse, torch.full_like(lse, float("-inf")))
    o = (o_parts * w[..., None]).sum(0) / torch.where(den > 0, den, torch.ones_like(den))[..., None]
    return o, lse


# --------------------------------------------------------------------------
# independent float64 evaluation used to pin the functions above
# --------------------------------------------------------------------------
def brute_force_rows(q, k, v, allowed, scale):
    """Pure-Python/numpy float64 loops: q [Nq,D], k/v [Nk,D], allowed [Nq,Nk].
    Returns (o [Nq,Dv], lse2 [Nq]); rows with no key -> 0, -inf."""
    q, k, v = (np.asarray(x, dtype=np.float64) for x in (q, k, v))
    nq, nk = q.shape[0], k.shape[0]
    o = np.zeros((nq, v.shape[1]))
    lse = np.full(nq, -np.inf)
    for i in range(nq):
        js = [j for j in range(nk) if allowed[i][j]]
        if not js:
            continue
        s = [sum(q[i, d] * k[j, d] for d in range(q.shape[1])) * scale for j in js]
        mx = max(s)
        w = [math.exp(x - mx) for x in s]
        z = sum(w)
        for t, j in enumerate(js):
            o[i] += (w[t] / z) * v[j]
        lse[i] = (mx + math.log(z)) * LOG2E
    return o, lse
