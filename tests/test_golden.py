"""Golden fixtures (tests/golden/attention_golden.pt, written by
tests/golden/make_golden.py from this repository's oracle): the CPU oracle must
keep reproducing them, and every GPU entry point must match them through the
C ABI."""
import os

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_golden.pt")


@pytest.fixture(scope="module")
def fx():
    return torch.load(PATH, weights_only=True)


def _lse_ok(got, want):
    got, want = got.float().cpu(), want.float()
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), fin)
    if fin.any():
        assert (got[fin] - want[fin]).abs().max() <= LSE_TOL


def test_oracle_reproduces_fixtures(fx):
    c = fx["varlen_causal"]
    o, lse = orc.flash_attn_torch(c["q"], c["k"], c["v"], c["cu"], faithful=False, return_lse=True)
    assert torch.equal(o.float(), c["o"]) and torch.equal(lse, c["lse"])
    c = fx["window_sparse"]
    o = orc.flash_attn_sparse_torch(c["q"], c["k"], c["v"], c["cu"], None, c["local"], c["glob"], faithful=False)
    assert torch.equal(o.float(), c["o"])
    c = fx["block_sparse"]
    o = orc.block_sparse_attention(c["q"], c["k"], c["v"], c["cu"], c["mask"].numpy(), faithful=False)
    assert torch.equal(o.float(), c["o"])
    c = fx["decode"]
    o = orc.flash_attn_decoding_torch(c["q"], c["k"], c["v"], c["lens"], faithful=False)
    assert torch.equal(o.float(), c["o"])
    c = fx["block_decode"]
    o = orc.block_sparse_decoding(c["q"], c["k"], c["v"], c["lens"], c["idx"], c["cnt"], faithful=False)
    assert torch.equal(o.float(), c["o"])
    # the zero-length and single-token rows are what the reference defines them to be
    assert torch.count_nonzero(fx["decode"]["o"][1]) == 0
    assert torch.equal(fx["decode"]["o"][3], fx["decode"]["v"][3, 0].float().repeat_interleave(4, 0))


@pytest.mark.gpu
def test_gpu_matches_fixtures(fx):
    import tritonops_amd as ta

    d = lambda t: t.cuda()
    c = fx["varlen_causal"]
    o, lse = ta.flash_attn_triton_fwd(d(c["q"]), d(c["k"]), d(c["v"]), d(c["cu"]), 64 ** -0.5 * ta.LOG2E)
    assert_close(o, c["o"], TOL, "varlen")
    _lse_ok(lse, c["lse"])
    c = fx["window_sparse"]
    o, lse = ta.flash_attn_sparse_triton(d(c["q"]), d(c["k"]), d(c["v"]), d(c["cu"]), None, c["local"], c["glob"])
    assert_close(o, c["o"], TOL, "window")
    _lse_ok(lse, c["lse"])
    c = fx["block_sparse"]
    o, lse = ta.flash_attn_sparse_triton(d(c["q"]), d(c["k"]), d(c["v"]), d(c["cu"]), block_mask=c["mask"])
    assert_close(o, c["o"], TOL, "block mask")
    _lse_ok(lse, c["lse"])
    c = fx["dense_noncausal"]
    assert_close(ta.flash_attention(d(c["q"]), d(c["k"]), d(c["v"]), causal=False), c["o"], TOL, "non-causal")
    c = fx["decode"]
    o, lse = ta.flash_attention_decoding(d(c["q"]), d(c["k"]), d(c["v"]), d(cu_from(c["lens"])), return_lse=True)
    assert_close(o, c["o"], TOL, "decode")
    _lse_ok(lse, c["lse"])
    c = fx["window_decode"]
    o = ta.flash_attention_sparse_decoding(d(c["q"]), d(c["k"]), d(c["v"]), d(cu_from(c["lens"])), c["glob"], c["local"])
    assert_close(o, c["o"], TOL, "window decode")
    c = fx["block_decode"]
    o = ta.flash_attention_sparse_decoding(d(c["q"]), d(c["k"]), d(c["v"]), None, seq_lens=d(c["lens"]),
                                           block_indices=d(c["idx"]), block_counts=d(c["cnt"]))
    assert_close(o, c["o"], TOL, "block decode")
