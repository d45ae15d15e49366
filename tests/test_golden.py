"""Golden fixtures (tests/golden/attention_golden.pt and neighbours_golden.pt,
written by tests/golden/make_golden.py and make_golden_neighbours.py from this
repository's oracles): the CPU oracles must keep reproducing them, and every GPU
entry point must match them through the C ABI."""
import os

import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import LSE_TOL, TOL, assert_close, cu_from

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_golden.pt")
PATH2 = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "neighbours_golden.pt")


@pytest.fixture(scope="module")
def fx():
    return torch.load(PATH, weights_only=True)


def _same(a, b, tol=2e-5):
    """Fixture reproduced up to the floating-point summation order of the host's
    BLAS (the fixtures were written on one machine, the suite runs on others)."""
    a, b = a.double(), b.double()
    if a.shape != b.shape:
        return False
    fin = torch.isfinite(b)
    return bool(torch.equal(a[~fin], b[~fin]) and ((a[fin] - b[fin]).abs() <= tol * (1.0 + b[fin].abs())).all())


def _lse_ok(got, want):
    got, want = got.float().cpu(), want.float()
    fin = torch.isfinite(want)
    assert torch.equal(torch.isfinite(got), fin)
    if fin.any():
        assert (got[fin] - want[fin]).abs().max() <= LSE_TOL


def test_oracle_reproduces_fixtures(fx):
    c = fx["varlen_causal"]
    o, lse = orc.flash_attn_torch(c["q"], c["k"], c["v"], c["cu"], faithful=False, return_lse=True)
    assert _same(o, c["o"]) and _same(lse, c["lse"])
    c = fx["window_sparse"]
    o = orc.flash_attn_sparse_torch(c["q"], c["k"], c["v"], c["cu"], None, c["local"], c["glob"], faithful=False)
    assert _same(o, c["o"])
    c = fx["block_sparse"]
    o = orc.block_sparse_attention(c["q"], c["k"], c["v"], c["cu"], c["mask"].numpy(), faithful=False)
    assert _same(o, c["o"])
    c = fx["decode"]
    o = orc.flash_attn_decoding_torch(c["q"], c["k"], c["v"], c["lens"], faithful=False)
    assert _same(o, c["o"])
    c = fx["block_decode"]
    o = orc.block_sparse_decoding(c["q"], c["k"], c["v"], c["lens"], c["idx"], c["cnt"], faithful=False)
    assert _same(o, c["o"])
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


@pytest.fixture(scope="module")
def nb():
    return torch.load(PATH2, weights_only=True)


def test_neighbour_oracles_reproduce_fixtures(nb):
    from oracle import rms_oracle as rorc
    from oracle import xent_oracle as xo

    c = nb["attn_backward"]
    dq, dk, dv = orc.varlen_masked_attention_backward(c["q"], c["k"], c["v"], c["do"], c["cu"], orc.causal_mask)
    assert _same(dq, c["dq"]) and _same(dk, c["dk"]) and _same(dv, c["dv"])
    for name in ("rmsnorm_fp32", "rmsnorm_bf16"):
        c = nb[name]
        y = rorc.rms_norm(c["x"].double(), c["w"].double(), c["eps"])
        dx, dw = rorc.rms_norm_backward(c["dy"], c["x"], c["w"], c["eps"])
        assert _same(y, c["y"]) and _same(dx, c["dx"]) and _same(dw, c["dw"])
    c = nb["fused_xent"]
    loss, lse = xo.linear_cross_entropy(c["x"], c["w"], c["y"])
    dx, dw = xo.linear_cross_entropy_backward(c["go"], c["x"], c["w"], c["y"])
    assert _same(loss, c["loss"]) and _same(lse, c["lse"])
    assert _same(dx, c["dx"]) and _same(dw, c["dw"])
    # a cross-entropy is positive, and lse bounds every logit from above
    assert (c["loss"] > 0).all()
    assert (c["lse"].double() >= (c["x"].double() @ c["w"].double().t()).max(-1).values).all()


@pytest.mark.gpu
def test_gpu_matches_neighbour_fixtures(nb):
    import tritonops_amd as ta

    d = lambda t: t.cuda()
    c = nb["attn_backward"]
    o, lse = ta.flash_attn_triton_fwd(d(c["q"]), d(c["k"]), d(c["v"]), d(c["cu"]), 64 ** -0.5 * ta.LOG2E)
    dq, dk, dv = ta.flash_attn_triton_bwd(d(c["q"]), d(c["k"]), d(c["v"]), o, d(c["do"]), lse, d(c["cu"]),
                                          64 ** -0.5 * ta.LOG2E)
    for name, g in (("dq", dq), ("dk", dk), ("dv", dv)):
        assert_close(g, c[name], 3e-2 * max(1.0, c[name].abs().max().item()), name)
    c = nb["rmsnorm_fp32"]
    y, rs = ta.rmsnorm_fwd(d(c["x"]), d(c["w"]), c["eps"])
    dx, dw = ta.rmsnorm_bwd(d(c["dy"]), d(c["x"]), d(c["w"]), rs, c["eps"])
    assert_close(y, c["y"], 1e-5, "rms y")
    assert_close(dx, c["dx"], 1e-5, "rms dx")
    assert_close(dw, c["dw"], 1e-4 * max(1.0, c["dw"].abs().max().item()), "rms dw")
    c = nb["rmsnorm_bf16"]
    y, rs = ta.rmsnorm_fwd(d(c["x"]), d(c["w"]), c["eps"])
    dx, dw = ta.rmsnorm_bwd(d(c["dy"]), d(c["x"]), d(c["w"]), rs, c["eps"])
    assert_close(y, c["y"], TOL * max(1.0, c["y"].abs().max().item()), "rms bf16 y")
    assert_close(dx, c["dx"], TOL * max(1.0, c["dx"].abs().max().item()), "rms bf16 dx")
    assert_close(dw, c["dw"], TOL * max(1.0, c["dw"].abs().max().item()), "rms bf16 dw")
    c = nb["fused_xent"]
    loss, lse = ta.cross_entropy_fused_fwd(d(c["x"]), d(c["w"]), d(c["y"]))
    assert_close(loss, c["loss"], TOL, "xent loss")
    assert_close(lse, c["lse"], TOL, "xent lse")
    dx, dw = ta.cross_entropy_fused_bwd(d(c["go"]), d(c["x"]), d(c["w"]), d(c["y"]), lse)
    assert_close(dx, c["dx"], 3e-2 * max(1.0, c["dx"].abs().max().item()), "xent dx")
    assert_close(dw, c["dw"], 3e-2 * max(1.0, c["dw"].abs().max().item()), "xent dw")
