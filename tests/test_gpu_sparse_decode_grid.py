"""The reference's own sweep of window-sparse decoding
(flash_attn_triton/flash_attn_decoding_sparse.py:506-630): 3 sequences of
lengths [0, 512, 2049] / [1, 2, 4] / [512, 2049, 8192], heads {4, 8, 16} x
kv-heads {1, 2, 4}, head_dim {32, 64, 96}, inputs scaled by {1, 10, 50, 100},
windows (64, 1024), (128, 128) and (512, 512).  The reference only looks for
NaN / inf / all-zero outputs there; here every case is compared with the
oracle."""
import pytest
import torch

from oracle import attention_oracle as orc
from tests.util import cu_from, randn

pytestmark = pytest.mark.gpu

SEQ_LENS = [[0, 512, 2049], [1, 2, 4], [512, 2049, 8192]]     # seq_lens_options[:batch_size], batch_size 3


def _sensitivity(q, k, v, lens, want, gw, lw, eps_rel):
    """Per output element: how far a softmax output can move when every score is
    perturbed by at most eps = eps_rel * max_j sum_d |q_d k_jd| * scale (the
    rounding of an fp32 dot product):  (e^(2 eps) - 1) * sum_j w_j |v_j - o|.
    With inputs scaled by 100 the scores reach 1e4..1e5, their fp32 rounding
    is no longer small against 1, and rows whose two best keys nearly tie
    legitimately differ between any two fp32 evaluations."""
    B, Hq, D = q.shape
    G = Hq // k.shape[2]
    out = torch.zeros(B, Hq, D, dtype=torch.float64)
    for b in range(B):
        L = int(lens[b])
        if L == 0:
            continue
        i = torch.arange(L)
        keep = (L <= i + lw) | (i < gw)
        for h in range(Hq):
            kk = k[b, :L, h // G].double()[keep]
            vv = v[b, :L, h // G].double()[keep]
            qq = q[b, h].double()
            s = (kk @ qq) * D ** -0.5
            eps = eps_rel * float((kk.abs() @ qq.abs()).max()) * D ** -0.5
            w = torch.softmax(s, 0)
            out[b, h] = torch.expm1(torch.tensor(2 * eps)) * (w[:, None] * (vv - want[b, h].double()).abs()).sum(0)
    return out


@pytest.mark.parametrize("num_heads", [4, 8, 16])
@pytest.mark.parametrize("seq_lens", SEQ_LENS, ids=lambda s: "lens" + "_".join(map(str, s)))
def test_reference_sweep_grid_against_the_oracle(seq_lens, num_heads):
    import tritonops_amd as ta

    lens = torch.tensor(seq_lens, dtype=torch.int32)
    cu = cu_from(lens).cuda()
    total = int(lens.sum())                    # the reference pads every sequence to the total length (:566-590)
    n = 0
    for num_kv_heads in (1, 2, 4):
        for D in (32, 64, 96):
            q1 = randn((3, num_heads, D), 1)
            k1, v1 = randn((3, total, num_kv_heads, D), 2), randn((3, total, num_kv_heads, D), 3)
            for scale in (1.0, 10.0, 50.0, 100.0):
                q, k, v = q1 * scale, k1 * scale, v1 * scale           # bf16 products, as in the reference (:566-590)
                qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
                for gw, lw in ((64, 1024), (128, 128), (512, 512)):
                    if gw == 512:
                        # not one of 64 / 128 / 256: the launcher asserts (:249-253)
                        with pytest.raises(AssertionError):
                            ta.flash_attention_sparse_decoding(qd, kd, vd, cu, global_window_size=gw,
                                                               local_window_size=lw)
                        continue
                    got = ta.flash_attention_sparse_decoding(qd, kd, vd, cu, global_window_size=gw,
                                                             local_window_size=lw).float().cpu()
                    want = orc.flash_attn_sparse_decoding_torch(q, k, v, lens, gw, lw, faithful=False).float()
                    assert got.shape == (3, num_heads, D) and torch.isfinite(got).all()
                    for b, L in enumerate(seq_lens):
                        if L == 0:
                            assert torch.count_nonzero(got[b]) == 0
                    # v and o scale with the inputs: the 2e-2 bar is relative to that; two fp32
                    # evaluations of the scores (the oracle's and the kernel's) each round them
                    tol = 2e-2 * scale + _sensitivity(q, k, v, lens, want, gw, lw, 2 * 2.0 ** -22).float()
                    bad = (got - want).abs() > tol
                    assert not bad.any(), "Hkv %d D %d scale %g window (%d, %d): max err %.4g" % (
                        num_kv_heads, D, scale, gw, lw, (got - want).abs().max().item())
                    n += 1
    assert n == 3 * 3 * 4 * 2
