"""Writes tests/golden/neighbours_golden.pt: small seeded inputs and the outputs
of THIS repository's CPU oracles for the operators built around the attention
forward: the dense backward (oracle/attention_oracle.py), RMSNorm
(oracle/rms_oracle.py) and the fused linear + cross-entropy
(oracle/xent_oracle.py).  The reference is never imported: it ships no vectors
for these operators (its tests draw random inputs), and every oracle function
is pinned independently in tests/test_oracle.py, tests/test_rms_oracle.py and
tests/test_xent_oracle.py.  The fixtures freeze the oracles and give the GPU
tests a file-based target.

    python tests/golden/make_golden_neighbours.py
"""
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attention_oracle as orc  # noqa: E402
from oracle import rms_oracle as rorc  # noqa: E402
from oracle import xent_oracle as xo  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "neighbours_golden.pt")


def randn(shape, seed, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype)


def main():
    fx = {}
    lens = torch.tensor([70, 1, 129], dtype=torch.int32)
    cu = torch.zeros(4, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    T = int(cu[-1])
    q, k, v, do = randn((1, T, 4, 64), 1), randn((1, T, 2, 64), 2), randn((1, T, 2, 64), 3), randn((1, T, 4, 64), 4)
    dq, dk, dv = orc.varlen_masked_attention_backward(q, k, v, do, cu, orc.causal_mask)
    fx["attn_backward"] = dict(q=q, k=k, v=v, do=do, cu=cu, dq=dq.float(), dk=dk.float(), dv=dv.float())

    # the reference's RMSNorm test shape: dim 255, eps 0.1, fp32 (common/rms.py:420-470)
    x, dy, w = randn((16, 7, 255), 5, torch.float32), randn((16, 7, 255), 6, torch.float32), randn((255,), 7, torch.float32)
    y = rorc.rms_norm(x.double(), w.double(), 0.1)
    dx, dw = rorc.rms_norm_backward(dy, x, w, 0.1)
    fx["rmsnorm_fp32"] = dict(x=x, dy=dy, w=w, eps=0.1, y=y.float(), dx=dx.float(), dw=dw.float())
    xb, dyb = randn((33, 512), 8), randn((33, 512), 9)
    wb = (1.0 + 0.1 * randn((512,), 10, torch.float32)).to(torch.bfloat16)
    y = rorc.rms_norm(xb.double(), wb.double(), 1e-6)
    dx, dw = rorc.rms_norm_backward(dyb, xb, wb, 1e-6)
    fx["rmsnorm_bf16"] = dict(x=xb, dy=dyb, w=wb, eps=1e-6, y=y.float(), dx=dx.float(), dw=dw.float())

    # the reference's cross-entropy test shape: 139 tokens, hidden 256, vocabulary 279, uniform inputs
    # (cross_entropy_triton/cross_entropy.py:438-470)
    g = torch.Generator().manual_seed(11)
    h = torch.rand((139, 256), generator=g).to(torch.bfloat16)
    wl = torch.rand((279, 256), generator=g).to(torch.bfloat16)
    yl = torch.randint(0, 279, (139,), generator=g)
    go = randn((139,), 12, torch.float32)
    loss, lse = xo.linear_cross_entropy(h, wl, yl)
    dxl, dwl = xo.linear_cross_entropy_backward(go, h, wl, yl)
    fx["fused_xent"] = dict(x=h, w=wl, y=yl, go=go, loss=loss.float(), lse=lse.float(), dx=dxl.float(), dw=dwl.float())
    torch.save(fx, OUT)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
