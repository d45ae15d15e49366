"""Writes tests/golden/attention_golden.pt: small seeded inputs and the outputs
of THIS repository's CPU oracle (oracle/attention_oracle.py, fp32 mode) for one
case per entry point.  The reference itself is never imported: it ships no
vectors for this path, and every oracle function is pinned independently in
tests/test_oracle.py.  The fixtures freeze the oracle (a later edit that changes
its results fails tests/test_golden.py on the CPU) and give the GPU tests a
second, file-based target.

    python tests/golden/make_golden.py
"""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attention_oracle as orc  # noqa: E402
from tritonops_amd import masks  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attention_golden.pt")


def randn(shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(torch.bfloat16)


def main():
    fx = {}
    lens = torch.tensor([70, 1, 129, 64], dtype=torch.int32)
    cu = torch.zeros(5, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    T = int(cu[-1])
    q, k, v = randn((1, T, 4, 64), 1), randn((1, T, 2, 64), 2), randn((1, T, 2, 64), 3)
    o, lse = orc.flash_attn_torch(q, k, v, cu, faithful=False, return_lse=True)
    fx["varlen_causal"] = dict(q=q, k=k, v=v, cu=cu, o=o.float(), lse=lse)

    o, lse = orc.flash_attn_sparse_torch(q, k, v, cu, None, 40, 70, faithful=False, return_lse=True)
    fx["window_sparse"] = dict(q=q, k=k, v=v, cu=cu, local=40, glob=70, o=o.float(), lse=lse)

    m = masks.synthetic_block_mask(3, band=1, sink=1, frac=0.5, seed=3)
    o, lse = orc.block_sparse_attention(q, k, v, cu, m, faithful=False, return_lse=True)
    fx["block_sparse"] = dict(q=q, k=k, v=v, cu=cu, mask=torch.from_numpy(m), o=o.float(), lse=lse)

    qb, kb, vb = randn((2, 2, 100, 128), 4), randn((2, 2, 100, 128), 5), randn((2, 2, 100, 128), 6)
    fx["dense_noncausal"] = dict(q=qb, k=kb, v=vb, o=orc.full_attention(qb.float(), kb.float(), vb.float()))

    dl = torch.tensor([300, 0, 65, 1], dtype=torch.int32)
    qd, kd, vd = randn((4, 8, 128), 7), randn((4, 300, 2, 128), 8), randn((4, 300, 2, 128), 9)
    o, lse = orc.flash_attn_decoding_torch(qd, kd, vd, dl, faithful=False, return_lse=True)
    fx["decode"] = dict(q=qd, k=kd, v=vd, lens=dl, o=o.float(), lse=lse)
    o = orc.flash_attn_sparse_decoding_torch(qd, kd, vd, dl, 64, 100, faithful=False)
    fx["window_decode"] = dict(q=qd, k=kd, v=vd, lens=dl, glob=64, local=100, o=o.float())
    idx = torch.tensor([[[0, 2], [1, 4]], [[0, 0], [0, 0]], [[0, 1], [1, 0]], [[0, 0], [0, 0]]], dtype=torch.int32)
    cnt = torch.tensor([[2, 2], [0, 0], [2, 1], [1, 1]], dtype=torch.int32)
    o = orc.block_sparse_decoding(qd, kd, vd, dl, idx, cnt, include_last_block=True, faithful=False)
    fx["block_decode"] = dict(q=qd, k=kd, v=vd, lens=dl, idx=idx, cnt=cnt, o=o.float())
    torch.save(fx, OUT)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
