#!/usr/bin/env python3
"""Benchmark of the attention forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints ONE JSON line.  The headline workload is the dense causal bf16 forward
B=4, H=32, S=8192, D=128 ("dense_causal"); the other benchmark configurations
(GQA decode at 32k KV, block-sparse forward, block-sparse decode) are measured
in the same run and reported under "other_workloads", each with its own
roofline object.  --workload picks a single one as the headline instead.

A step is one pass of the path over one batch of synthetic inputs that are
already resident in HBM.  `value` comes from wall-clock around K steps
bracketed by device synchronisation; `roofline.achieved` comes from HIP events
recorded on the launch stream around the same kernels (mi_time_launches).
`max_abs_err` is the largest |kernel - fp32 torch math| over a stated sample of
the benchmark tensors themselves (rows / heads / sequences), computed on the
device.  The CPU baseline is the reference's PyTorch attention math (oracle/)
timed on this host's cores on a stated slice of the same workload.
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# Device symbols of the kernels each workload's roofline figure is about, as
# rocprofv3 prints them (it leaves names with a bf16 template argument mangled).
# tests/test_abi.py checks that the built library contains every one of them.
_NS = "_ZN2mi12_GLOBAL__N_1"
KERNELS = {
    "dense_causal": _NS + "12dense_kernelIDF16bLi128EEEvNS_13PrefillParamsE",
    "c1_dense_noncausal_small": _NS + "18dense_short_kernelIDF16bLi64ELb0EEEvNS_13PrefillParamsE",
    "gqa_decode": _NS + "21decode_splitkv_kernelIDF16bLi128EEEvNS_12DecodeParamsE",
    "block_sparse": _NS + "13sparse_kernelIDF16bLi128EEEvNS_13PrefillParamsE",
    "sparse_decode": _NS + "21decode_splitkv_kernelIDF16bLi128EEEvNS_12DecodeParamsE",
    "dense_causal_bwd": " + ".join(_NS + n for n in (
        "13bwd_dq_kernelIDF16bLi128EEEvNS_9BwdParamsEi",
        "15bwd_dkdv_kernelIDF16bLi128EEEvNS_9BwdParamsEii")),
    "rmsnorm": " + ".join(_NS + n for n in (
        "18rms_fwd_vec_kernelIDF16bfLi2ELi4EEEvNS_9RmsParamsE", "18rms_bwd_vec_kernelIDF16bfLi2ELi4EEEvNS_9RmsParamsE",
        "19rms_dw_stage_kernelILi4EEEvPKfPfii", "20rms_dw_reduce_kernelIfEEvPKfPT_ii")),
    "fused_xent": _NS + "16xent_gemm_kernelIDF16bLb0EEEvNS_10XentParamsE",
}
# the reference's own call forms run on the kernels of the configurations above
KERNELS["dense_causal_packed"] = KERNELS["dense_causal"]
KERNELS["window_sparse_prefill"] = KERNELS["block_sparse"]
KERNELS["window_sparse_decode"] = KERNELS["sparse_decode"]
KERNELS["window_long_prefill"] = _NS + "18dense_short_kernelIDF16bLi128ELb1EEEvNS_13PrefillParamsE"   # the dense walk over a window's tiles


def _sync():
    torch.cuda.synchronize()


def _randn(shape, seed, device="cuda"):
    """Seeded N(0,1) -> bf16.  Big tensors are drawn on the device in chunks
    (parity tests use CPU-drawn inputs; here only the distribution matters)."""
    g = torch.Generator(device=device).manual_seed(seed)
    out = torch.empty(shape, device=device, dtype=torch.bfloat16)
    flat = out.view(-1)
    step = 1 << 28
    for s in range(0, flat.numel(), step):
        n = min(step, flat.numel() - s)
        flat[s:s + n] = torch.randn(n, generator=g, device=device, dtype=torch.float32).to(torch.bfloat16)
    return out


def _time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    _sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    _sync()
    return (time.perf_counter() - t0) / steps * 1e3   # ms per step


def _event_ms(kind, args, steps, warmup):
    """Average launch duration from HIP events on the current stream.  `args` is
    one argument struct or a list of them (launch i uses struct i % len)."""
    from tritonops_amd import _lib
    lib = _lib.load()
    ms = C.c_float(0)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    if not isinstance(args, (list, tuple)):
        args = [args]
    arr = (type(args[0]) * len(args))(*args)
    _lib.check(lib.mi_time_launches(kind, C.cast(arr, C.c_void_p), len(args), C.sizeof(args[0]), st, warmup, steps,
                                    C.byref(ms)))
    return ms.value


def _ref_rows(q, k, v, rows, scale, allow):
    """fp32 softmax(q k^T scale) v and base-2 LSE on the device: q [..., S, D]
    restricted to `rows`, k / v [..., S, D], allow bool [len(rows), S]."""
    s = torch.einsum("...id,...jd->...ij", q[..., rows, :].float(), k.float()) * scale
    s = s.masked_fill(~allow, float("-inf"))
    return torch.einsum("...ij,...jd->...id", torch.softmax(s, -1), v.float()), torch.logsumexp(s, -1) * LOG2E


def _err(got, want):
    return float((got.float() - want.float()).abs().max().item())


LOG2E = 1.4426950408889634


# ----------------------------------------------------------------------------
# workloads: each returns dict(ms_per_step, kernel_ms, work, unit-specific...)
# ----------------------------------------------------------------------------
def _fwd_args(q, k, v, o, lse, causal):
    """mi_attn_fwd_args for contiguous [B,H,S,D] tensors."""
    from tritonops_amd import _lib
    B, H, S, D = q.shape
    a = _lib.AttnFwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = (t.data_ptr() for t in (q, k, v, o, lse))
    for n, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, n + "_stride_b", t.stride(0))
        setattr(a, n + "_stride_h", t.stride(1))
        setattr(a, n + "_stride_s", t.stride(2))
    a.lse_stride_b, a.lse_stride_h, a.lse_stride_s = lse.stride(0), lse.stride(1), lse.stride(2)
    a.cu_seqlens = None
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, H, k.shape[1], S, D
    a.causal = 1 if causal else 0
    a.scale_log2 = D ** -0.5 * 1.4426950408889634
    return a


# (batch, heads, sequence length) of the dense causal workload; --dense-shape replaces it for profiling other
# shapes (the headline line of the default run is always the benchmark's own configuration)
DENSE_SHAPE = (4, 32, 8192, 128)


DENSE_FORM = "auto"   # --dense-form: pin one of the two forms of the dense kernel (for profiling)


def _dense_kernel_name(D):
    long_form = _NS + "12dense_kernelIDF16bLi%dEEEvNS_13PrefillParamsE" % D
    short_form = _NS + "18dense_short_kernelIDF16bLi%dELb0EEEvNS_13PrefillParamsE" % D
    if DENSE_FORM == "256" or (DENSE_FORM == "auto" and DENSE_SHAPE == (4, 32, 8192, 128)):
        return long_form
    if DENSE_FORM == "128":
        return short_form
    return long_form + " or " + short_form   # the launcher picks the form from the number of work items


def run_dense_causal(steps, warmup):
    import tritonops_amd as ta
    B, H, S, D = DENSE_SHAPE
    q, k, v = (_randn((B, H, S, D), s) for s in (0, 1, 2))
    fn = lambda: ta.flash_attention(q, k, v, causal=True, return_lse=True)
    with ta.dense_form(DENSE_FORM):
        ms = _time_steps(fn, steps, warmup)
    o = torch.empty_like(q)
    lse = torch.empty((B, H, S), device="cuda", dtype=torch.float32)
    args = _fwd_args(q, k, v, o, lse, True)
    args.dense_form = {"auto": 0, "256": 1, "128": 2}[DENSE_FORM]
    kms = _event_ms(0, args, steps, warmup)
    flop = 2.0 * B * H * S * (S + 1) * D            # 4*D per unmasked (q, k) pair
    # parity on the benchmark tensors: three (batch, head) units x four 64-row blocks
    err = err_lse = 0.0
    keys = torch.arange(S, device="cuda")
    for b, h in ((0, 0), (min(1, B - 1), 13 % H), (B - 1, H - 1)):
        for r0 in sorted({0, (S // 4 - 64) // 64 * 64, S // 2, S - 64}):
            rows = torch.arange(r0, r0 + 64, device="cuda")
            want, want_lse = _ref_rows(q[b, h], k[b, h], v[b, h], rows, D ** -0.5, keys[None, :] <= rows[:, None])
            err = max(err, _err(o[b, h, rows], want))
            err_lse = max(err_lse, _err(lse[b, h, rows], want_lse))
    return {
        "name": "dense_causal", "ms_per_step": ms, "kernel_ms": kms,
        "metric": "attn_fwd_tflops", "unit": "TFLOP/s", "value": flop / (ms * 1e-3) / 1e12,
        "max_abs_err": err, "max_abs_err_lse2": err_lse,
        "err_sample": "o and lse of 3 (batch, head) units x 4 blocks of 64 query rows against fp32 torch math on the device",
        "roofline": {"bound": "mfma", "achieved": flop / (kms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": _dense_kernel_name(D)},
        "config": {"workload": "dense causal flash-attention fwd bf16 B=%d H=%d S=%d D=%d, o bf16 + lse fp32%s"
                               % (B, H, S, D, "" if DENSE_FORM == "auto" else ", %s-row work items" % DENSE_FORM),
                   "flop_per_step": flop, "flop_reference_convention_4BHS2D": 4.0 * B * H * S * S * D},
    }


def run_c1_small(steps, warmup):
    """The reference's CPU-runnable case: dense non-causal B=1 H=4 S=256 D=64, q/k/v drawn in fp32 on the CPU
    from seed 0.  The GPU path runs it on the bf16 cast; the parity figure is against fp32 math on the fp32
    inputs, so it includes the rounding of the inputs."""
    import tritonops_amd as ta
    B, H, S, D = 1, 4, 256, 64
    g = torch.Generator().manual_seed(0)
    q32, k32, v32 = (torch.randn((B, H, S, D), generator=g) for _ in range(3))
    q, k, v = (t.to(torch.bfloat16).cuda() for t in (q32, k32, v32))
    fn = lambda: ta.flash_attention(q, k, v, causal=False, return_lse=True)
    ms = _time_steps(fn, steps, warmup)
    o, lse = fn()
    kms = _event_ms(0, _fwd_args(q, k, v, torch.empty_like(q), torch.empty_like(lse), False), steps, warmup)
    want = torch.softmax(torch.einsum("bhid,bhjd->bhij", q32, k32) / 8.0, -1) @ v32
    flop = 4.0 * B * H * S * S * D
    return {
        "name": "c1_dense_noncausal_small", "ms_per_step": ms, "kernel_ms": kms,
        "metric": "attn_fwd_tflops", "unit": "TFLOP/s", "value": flop / (ms * 1e-3) / 1e12,
        "max_abs_err": _err(o.cpu(), want),
        "err_sample": "all of o against fp32 softmax(q k^T / 8) v on the fp32 inputs (the kernel sees their bf16 cast)",
        "roofline": {"bound": "mfma", "achieved": flop / (kms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": KERNELS["c1_dense_noncausal_small"]},
        "config": {"workload": "dense non-causal attention fwd B=1 H=4 S=256 D=64 (the reference's CPU case; 8 work items, "
                               "launch-latency bound on a GPU), bf16 cast of fp32 N(0,1) inputs from seed 0",
                   "flop_per_step": flop},
    }


def run_dense_bwd(steps, warmup):
    """Backward of the headline configuration (dq, dk, dv from q, k, v, o, lse, do)."""
    import tritonops_amd as ta
    from tritonops_amd import _lib, ops
    B, H, S, D = 4, 32, 8192, 128
    q, k, v, do = (_randn((B, H, S, D), s) for s in (0, 1, 2, 3))
    qs, ks, vs, ds = (t.transpose(1, 2) for t in (q, k, v, do))      # [B,S,H,D] views
    sm = D ** -0.5 * ta.LOG2E
    o, lse = ops._dense_fwd(qs, ks, vs, None, sm, True, None, bhsd=True)
    steps, warmup = max(4, steps // 4), max(2, warmup // 4)         # a step is ~5x the forward
    fn = lambda: ops._dense_bwd(qs, ks, vs, o, ds, lse, None, sm, True, None)
    ms = _time_steps(fn, steps, warmup)
    dq, dk, dv = fn()
    a = _lib.AttnBwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    for n, t in (("q", qs), ("k", ks), ("v", vs), ("o", o), ("dout", ds), ("dq", dq), ("dk", dk), ("dv", dv),
                 ("lse", lse)):
        setattr(a, n, t.data_ptr())
        setattr(a, n + "_stride_b", t.stride(0))
        setattr(a, n + "_stride_s", t.stride(1))
        setattr(a, n + "_stride_h", t.stride(2))
    a.cu_seqlens = None
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim, a.causal = B, H, H, S, D, 1
    a.scale_log2 = sm
    nb = _lib.load().mi_attn_bwd_workspace_bytes(C.byref(a))
    ws = torch.empty(nb, device="cuda", dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    kms = _event_ms(5, a, steps, warmup)
    flop = 2.5 * 2.0 * B * H * S * (S + 1) * D       # 10*D per unmasked (q, k) pair: S, dP, dV, dQ, dK
    # parity on the benchmark tensors: one (batch, head) unit through autograd in fp32 on the device
    b, h = 2, 17
    qr, kr, vr = (t[b, h].float().requires_grad_(True) for t in (q, k, v))
    sc = (qr @ kr.T) * D ** -0.5
    sc = sc.masked_fill(~torch.ones(S, S, dtype=torch.bool, device="cuda").tril(), float("-inf"))
    (torch.softmax(sc, -1) @ vr).backward(do[b, h].float())
    err = max(_err(dq[b, :, h], qr.grad), _err(dk[b, :, h], kr.grad), _err(dv[b, :, h], vr.grad))
    del qr, kr, vr, sc
    return {
        "name": "dense_causal_bwd", "ms_per_step": ms, "kernel_ms": kms,
        "metric": "attn_bwd_tflops", "unit": "TFLOP/s", "value": flop / (ms * 1e-3) / 1e12,
        "max_abs_err": err,
        "err_sample": "dq, dk, dv of one (batch, head) unit against autograd through fp32 torch math on the device (bar 3e-2)",
        "roofline": {"bound": "mfma", "achieved": flop / (kms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": KERNELS["dense_causal_bwd"]},
        "config": {"workload": "dense causal attention bwd bf16 B=4 H=32 S=8192 D=128: dq, dk, dv from q, k, v, o, lse, do",
                   "flop_per_step": flop,
                   "note": "a dq kernel (which also forms delta) and a fused dk + dv kernel execute 14*D FLOP per pair (S and dP twice); the figure "
                           "counts the 10*D of a single-pass backward"},
    }


def run_decode(steps, warmup):
    import tritonops_amd as ta
    B, Hq, Hkv, L, D = 64, 32, 8, 32768, 128
    lens = torch.randint(16384, L + 1, (B,), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    lens_d = lens.cuda()
    q = _randn((B, Hq, D), 0)
    # two KV sets, alternated, so no step finds its KV in the 256 MB last-level cache
    caches = [(_randn((B, Hkv, L, D), 10 + 2 * i), _randn((B, Hkv, L, D), 11 + 2 * i)) for i in range(2)]
    state = {"i": 0}

    def fn():
        kc, vc = caches[state["i"] & 1]
        state["i"] += 1
        return ta.flash_attention_decoding(q, kc.transpose(1, 2), vc.transpose(1, 2), None, seq_lens=lens_d)
    ms = _time_steps(fn, steps, warmup)
    # event timing of the two kernels on one cache (8.6 GB >> cache, no reuse between launches)
    from tritonops_amd import _lib
    lib = _lib.load()
    kc, vc = caches[0]
    k, v = kc.transpose(1, 2), vc.transpose(1, 2)
    o = torch.empty((B, Hq, D), device="cuda", dtype=torch.bfloat16)
    a = _lib.DecodeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_b, a.k_stride_s, a.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
    a.v_stride_b, a.v_stride_s, a.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
    a.o_stride_b, a.o_stride_h = o.stride(0), o.stride(1)
    a.seq_lens, a.cu_seqlens = lens_d.data_ptr(), None
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, Hq, Hkv, L, D
    a.scale_log2 = D ** -0.5 * 1.4426950408889634
    a.split_tokens = lib.mi_decode_choose_split_tokens(B, Hkv, L, lib.mi_device_cu_count())
    nbytes = lib.mi_decode_workspace_bytes(C.byref(a))
    ws = torch.empty(nbytes, device="cuda", dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nbytes
    # launches alternate the two caches, like the wall-clock leg
    a2 = _lib.DecodeArgs.from_buffer_copy(a)
    a2.k, a2.v = caches[1][0].data_ptr(), caches[1][1].data_ptr()
    k_split = _event_ms(3, [a, a2], steps, warmup)
    k_merge = _event_ms(4, a, steps, warmup)
    # parity on the benchmark tensors: three sequences against fp32 torch math on the device
    got = ta.flash_attention_decoding(q, k, v, None, seq_lens=lens_d)
    err = 0.0
    for b in (0, 31, 63):
        n = int(lens[b])
        sc = torch.einsum("gid,gld->gil", q[b].view(Hkv, Hq // Hkv, D).float(), kc[b, :, :n].float()) * D ** -0.5
        want = torch.einsum("gil,gld->gid", torch.softmax(sc, -1), vc[b, :, :n].float()).reshape(Hq, D)
        err = max(err, _err(got[b], want))
    # same cache as a pool of shuffled 64-token pages [pages, Hkv, 64, D] behind a page table
    ps = 64
    npg = L // ps
    perm = torch.randperm(B * npg, generator=torch.Generator().manual_seed(3)).cuda()
    table = perm.view(B, npg).to(torch.int32)
    pools = []
    for t in (kc, vc):
        pool = torch.empty((B * npg, Hkv, ps, D), device="cuda", dtype=t.dtype)
        pool[perm] = t.view(B, Hkv, npg, ps, D).permute(0, 2, 1, 3, 4).reshape(B * npg, Hkv, ps, D)
        pools.append(pool.transpose(1, 2))
    kp, vp = pools
    a.k, a.v = kp.data_ptr(), vp.data_ptr()
    a.k_stride_b, a.k_stride_s, a.k_stride_h = kp.stride(0), kp.stride(1), kp.stride(2)
    a.v_stride_b, a.v_stride_s, a.v_stride_h = vp.stride(0), vp.stride(1), vp.stride(2)
    a.kv_layout, a.page_size = _lib.MI_KV_PAGED, ps
    a.page_table, a.page_table_stride_b = table.data_ptr(), table.stride(0)
    k_paged = _event_ms(3, a, steps, warmup)
    del pools, kp, vp
    nbytes_alg = float(lens.sum().item()) * Hkv * 2 * D * 2 + B * Hq * D * 2 * 2
    return {
        "name": "gqa_decode", "ms_per_step": ms, "kernel_ms": k_split, "merge_kernel_ms": k_merge,
        "metric": "decode_hbm_gbs", "unit": "GB/s", "value": nbytes_alg / (ms * 1e-3) / 1e9,
        "max_abs_err": err,
        "err_sample": "3 of the 64 sequences (all heads) against fp32 torch math on the device",
        "roofline": {"bound": "hbm", "achieved": nbytes_alg / (k_split * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "kernel": KERNELS["gqa_decode"]},
        "config": {"workload": "GQA decode bf16 B=64 Hq=32 Hkv=8 KV<=32768 (lens U[16384,32768]) D=128, split-KV + LSE merge",
                   "bytes_per_step": nbytes_alg, "split_tokens": int(a.split_tokens),
                   "paged_cache_kernel_ms": k_paged,
                   "paged_cache_note": "same launch over a pool of shuffled 64-token pages behind a page table"},
    }


def run_block_sparse(steps, warmup):
    import tritonops_amd as ta
    from tritonops_amd import masks
    B, H, S, D = 2, 16, 16384, 128
    nb = S // 64
    m = masks.synthetic_block_mask(nb, 8, 4, 0.10, seed=2)
    live = int(m.sum())
    row_ptr, col_idx, strides = masks.block_mask_to_csr(m, "cuda")
    q, k, v = (_randn((B, H, S, D), s) for s in (0, 1, 2))
    fn = lambda: ta.flash_attn_sparse_triton(q, k, v, None, row_ptr=row_ptr, col_idx=col_idx, csr_strides=strides)
    ms = _time_steps(fn, steps, warmup)
    from tritonops_amd import _lib
    o = torch.empty_like(q)
    lse = torch.empty((B, H, S), device="cuda", dtype=torch.float32)
    a = _lib.AttnSparseArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = (t.data_ptr() for t in (q, k, v, o, lse))
    for n, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, n + "_stride_b", t.stride(0))
        setattr(a, n + "_stride_h", t.stride(1))
        setattr(a, n + "_stride_s", t.stride(2))
    a.lse_stride_b, a.lse_stride_h, a.lse_stride_s = lse.stride(0), lse.stride(1), lse.stride(2)
    a.cu_seqlens = None
    a.row_ptr, a.col_idx = row_ptr.data_ptr(), col_idx.data_ptr()
    a.row_ptr_stride_b, a.row_ptr_stride_h, a.col_idx_stride_b, a.col_idx_stride_h = strides
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, H, H, S, D
    a.block_size, a.window_local, a.window_global = 64, -1, -1
    a.scale_log2 = D ** -0.5 * 1.4426950408889634
    kms = _event_ms(1, a, steps, warmup)
    flop = 4.0 * D * ((live - nb) * 64 * 64 + nb * 64 * 65 / 2) * B * H
    # parity on the benchmark tensors: five query blocks of every (batch, head) unit
    bm = torch.from_numpy(m).cuda()
    keys = torch.arange(S, device="cuda")
    err = err_lse = 0.0
    for qb in (0, 3, 64, 129, 255):
        rows = torch.arange(qb * 64, qb * 64 + 64, device="cuda")
        want, want_lse = _ref_rows(q, k, v, rows, D ** -0.5, bm[qb][keys // 64][None, :] & (keys[None, :] <= rows[:, None]))
        err = max(err, _err(o[:, :, rows], want))
        err_lse = max(err_lse, _err(lse[:, :, rows], want_lse))
    return {
        "name": "block_sparse", "ms_per_step": ms, "kernel_ms": kms,
        "metric": "sparse_attn_fwd_tflops", "unit": "TFLOP/s", "value": flop / (ms * 1e-3) / 1e12,
        "max_abs_err": err, "max_abs_err_lse2": err_lse,
        "err_sample": "5 of the 256 query blocks of all 32 (batch, head) units against masked fp32 torch math on the device",
        "roofline": {"bound": "mfma", "achieved": flop / (kms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": KERNELS["block_sparse"]},
        "config": {"workload": "block-sparse causal fwd bf16 B=2 H=16 S=16384 D=128, 64x64 blocks, band 8 + 4 sink + 10%% (%d live blocks)" % live,
                   "flop_per_step": flop,
                   "kv_tile_bytes_per_step": float(live * 64 * D * 2 * 2 * B * H),
                   "note": "every live 64x64 block re-reads its 32 KiB of K/V from L2 / last-level cache: 64 FLOP per "
                           "byte moved, so this workload is bound by cache bandwidth well before the MFMA peak"},
    }


def run_sparse_decode(steps, warmup):
    import tritonops_amd as ta
    from tritonops_amd import masks
    B, Hq, Hkv, L, D = 32, 32, 8, 131072, 128
    g = torch.Generator().manual_seed(1)
    lens = (L - torch.randint(0, 64, (B,), generator=g)).to(torch.int32)
    # Six seeded index lists, rotated: six steps read 6 x 1.08 GB of different blocks, so no step
    # finds the blocks of an earlier one in the 256 MB last-level cache.
    lists = [masks.synthetic_decode_blocks(B, Hkv, L // 64, 128, seed=2 + i).cuda() for i in range(6)]
    idx = lists[0]
    lens_d = lens.cuda()
    q = _randn((B, Hq, D), 0)
    kc, vc = _randn((B, Hkv, L, D), 1), _randn((B, Hkv, L, D), 2)
    state = {"i": 0}

    def fn():
        state["i"] += 1
        return ta.flash_attention_sparse_decoding(q, kc.transpose(1, 2), vc.transpose(1, 2), None,
                                                  seq_lens=lens_d, block_indices=lists[state["i"] % len(lists)])
    ms = _time_steps(fn, steps, warmup)
    from tritonops_amd import _lib
    lib = _lib.load()
    k, v = kc.transpose(1, 2), vc.transpose(1, 2)
    o = torch.empty((B, Hq, D), device="cuda", dtype=torch.bfloat16)
    a = _lib.DecodeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_b, a.k_stride_s, a.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
    a.v_stride_b, a.v_stride_s, a.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
    a.o_stride_b, a.o_stride_h = o.stride(0), o.stride(1)
    a.seq_lens, a.cu_seqlens = lens_d.data_ptr(), None
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, Hq, Hkv, L, D
    a.scale_log2 = D ** -0.5 * 1.4426950408889634
    a.split_tokens = 64
    a.block_idx, a.block_cnt = idx.data_ptr(), None
    a.block_idx_stride_b, a.block_idx_stride_h = Hkv * 128, 128
    a.max_blocks, a.block_size = 128, 64
    a.split_blocks = lib.mi_decode_choose_split_blocks(B, Hkv, 129, lib.mi_device_cu_count())
    a.window_local = a.window_global = -1
    a.include_last_block = 1
    nb = lib.mi_decode_workspace_bytes(C.byref(a))
    ws = torch.empty(nb, device="cuda", dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    rot = []
    for l in lists:
        ai = _lib.DecodeArgs.from_buffer_copy(a)
        ai.block_idx = l.data_ptr()
        rot.append(ai)
    kms = _event_ms(3, rot, steps, warmup)
    kms_one_list = _event_ms(3, a, steps, warmup)
    nbytes_alg = float(B * Hkv * 129 * 64 * D * 2 * 2)
    # parity on the benchmark tensors: three sequences (first list) against fp32 torch math on the device
    got = ta.flash_attention_sparse_decoding(q, k, v, None, seq_lens=lens_d, block_indices=idx)
    err = 0.0
    for b in (0, 15, 31):
        n = int(lens[b])
        blocks = torch.cat([idx[b].long(), torch.full((Hkv, 1), (n - 1) // 64, device="cuda")], 1)      # [Hkv, 129]
        tok = (blocks[:, :, None] * 64 + torch.arange(64, device="cuda")).reshape(Hkv, -1)             # [Hkv, 129*64]
        live = tok < n
        tok = tok.clamp(max=n - 1)
        kk = torch.gather(kc[b], 1, tok[:, :, None].expand(-1, -1, D)).float()
        vv = torch.gather(vc[b], 1, tok[:, :, None].expand(-1, -1, D)).float()
        sc = torch.einsum("gid,gld->gil", q[b].view(Hkv, Hq // Hkv, D).float(), kk) * D ** -0.5
        sc = sc.masked_fill(~live[:, None, :], float("-inf"))
        want = torch.einsum("gil,gld->gid", torch.softmax(sc, -1), vv).reshape(Hq, D)
        err = max(err, _err(got[b], want))
    return {
        "name": "sparse_decode", "ms_per_step": ms, "kernel_ms": kms,
        "metric": "sparse_decode_hbm_gbs", "unit": "GB/s", "value": nbytes_alg / (ms * 1e-3) / 1e9,
        "max_abs_err": err,
        "err_sample": "3 of the 32 sequences (all heads, first index list) against fp32 torch math on the device",
        "roofline": {"bound": "hbm", "achieved": nbytes_alg / (kms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "kernel": KERNELS["sparse_decode"]},
        "config": {"workload": "block-sparse decode bf16 B=32 Hq=32 Hkv=8 KV=131072 D=128, top-128 of 64-token blocks + last block",
                   "bytes_per_step": nbytes_alg, "split_blocks": int(a.split_blocks),
                   "index_lists_rotated": len(lists), "kernel_ms_same_list_every_launch": kms_one_list},
    }


def run_rmsnorm(steps, warmup):
    """RMSNorm forward + backward over [32768, 4096] bf16 activations, fp32 weight."""
    import tritonops_amd as ta
    from tritonops_amd import _lib
    T, D, eps = 32768, 4096, 1e-6
    x, dy = _randn((T, D), 0), _randn((T, D), 1)
    w = torch.ones(D, device="cuda", dtype=torch.float32)

    def fn():
        y, rs = ta.rmsnorm_fwd(x, w, eps)
        return ta.rmsnorm_bwd(dy, x, w, rs, eps)
    ms = _time_steps(fn, steps, warmup)
    y, rs = ta.rmsnorm_fwd(x, w, eps)
    dx, dw = ta.rmsnorm_bwd(dy, x, w, rs, eps)
    a = _lib.RmsNormArgs()
    a.struct_size = C.sizeof(a)
    a.x_dtype, a.w_dtype, a.dim, a.rows = _lib.MI_DTYPE_BF16, _lib.MI_DTYPE_F32, D, T
    a.x, a.w, a.y, a.rsqrt = x.data_ptr(), w.data_ptr(), y.data_ptr(), rs.data_ptr()
    a.dy, a.dx, a.dw = dy.data_ptr(), dx.data_ptr(), dw.data_ptr()
    a.x_stride = a.y_stride = a.dy_stride = a.dx_stride = D
    a.eps = eps
    nb = _lib.load().mi_rmsnorm_bwd_workspace_bytes(C.byref(a))
    ws = torch.empty(nb, device="cuda", dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    k_fwd = _event_ms(6, a, steps, warmup)
    k_bwd = _event_ms(7, a, steps, warmup)
    b_fwd = 2.0 * T * D * 2 + T * 4                 # x read, y written, rsqrt written
    b_bwd = 3.0 * T * D * 2 + T * 4                 # x, dy read, dx written, rsqrt read
    # parity on the benchmark tensors: 512 rows of y and dx, and dw over all rows, against fp32 torch math
    rows = torch.arange(0, T, T // 512, device="cuda")
    xf, dyf = x[rows].float(), dy[rows].float()
    r = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    want_dx = dyf * w * r - xf * r.pow(3) * (dyf * w * xf).sum(-1, keepdim=True) / D
    r_all = torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + eps)
    want_dw = (dy.float() * x.float() * r_all).sum(0)
    err = max(_err(y[rows], xf * r * w), _err(dx[rows], want_dx))
    err_dw = float(((dw.float() - want_dw).abs() / want_dw.abs().clamp(min=1.0)).max().item())
    del r_all, want_dw
    return {
        "name": "rmsnorm", "ms_per_step": ms, "kernel_ms": k_fwd + k_bwd,
        "metric": "rmsnorm_fwd_bwd_hbm_gbs", "unit": "GB/s", "value": (b_fwd + b_bwd) / (ms * 1e-3) / 1e9,
        "max_abs_err": err, "max_rel_err_dw": err_dw,
        "err_sample": "y and dx of 512 of the 32768 rows, dw over all rows (relative), against fp32 torch math on the device",
        "roofline": {"bound": "hbm", "achieved": (b_fwd + b_bwd) / ((k_fwd + k_bwd) * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "kernel": KERNELS["rmsnorm"]},
        "config": {"workload": "RMSNorm fwd + bwd, x [32768, 4096] bf16, weight fp32, eps 1e-6",
                   "bytes_per_step": b_fwd + b_bwd, "fwd_kernel_ms": k_fwd, "bwd_kernel_ms": k_bwd,
                   "fwd_gbs": b_fwd / (k_fwd * 1e-3) / 1e9, "bwd_gbs": b_bwd / (k_bwd * 1e-3) / 1e9},
    }


def run_fused_xent(steps, warmup):
    """Fused linear + cross-entropy, Llama-3-sized head: 8192 tokens, hidden 4096, vocabulary 128256."""
    import tritonops_amd as ta
    from tritonops_amd import _lib
    T, D, N = 8192, 4096, 128256
    x = _randn((T, D), 0)
    w = (_randn((N, D), 1).float() * (D ** -0.5)).to(torch.bfloat16)
    y = torch.randint(0, N, (T,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(2))
    steps, warmup = max(steps // 4, 3), max(warmup // 4, 2)
    ms = _time_steps(lambda: ta.cross_entropy_fused_fwd(x, w, y), steps, warmup)
    loss, lse = ta.cross_entropy_fused_fwd(x, w, y)
    go = torch.full((T,), 1.0 / T, device="cuda")
    ms_bwd = _time_steps(lambda: ta.cross_entropy_fused_bwd(go, x, w, y, lse), max(steps // 2, 2), 1)
    a = _lib.XentArgs()
    a.struct_size = C.sizeof(a)
    a.dtype, a.tokens, a.dim, a.vocab, a.labels_i64 = _lib.MI_DTYPE_BF16, T, D, N, 1
    a.x, a.w, a.y, a.lse, a.loss = x.data_ptr(), w.data_ptr(), y.data_ptr(), lse.data_ptr(), loss.data_ptr()
    a.x_stride = a.w_stride = D
    nb = _lib.load().mi_xent_fwd_workspace_bytes(C.byref(a))
    ws = torch.empty(nb, device="cuda", dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    kms = _event_ms(8, a, steps, warmup)
    # the backward's first launch: the same GEMM with the gradient epilogue
    dl = torch.empty((T, N), device="cuda", dtype=torch.bfloat16)
    g = _lib.XentBwdArgs()
    g.struct_size = C.sizeof(g)
    g.dtype, g.tokens, g.dim, g.vocab, g.labels_i64 = _lib.MI_DTYPE_BF16, T, D, N, 1
    g.x, g.w, g.y, g.lse, g.dloss = x.data_ptr(), w.data_ptr(), y.data_ptr(), lse.data_ptr(), go.data_ptr()
    g.x_stride = g.w_stride = D
    g.dlogits, g.ld = dl.data_ptr(), N
    kms_grad = _event_ms(10, g, max(steps // 2, 2), 1)
    del dl
    flop = 2.0 * T * D * N
    # parity on the benchmark tensors: loss and lse of 64 tokens against fp32 torch math on the device
    rows = torch.arange(0, T, T // 64, device="cuda")
    logits = x[rows].float() @ w.float().t()
    want_lse = torch.logsumexp(logits, -1)
    want_loss = want_lse - logits.gather(-1, y[rows].view(-1, 1)).squeeze(-1)
    err = max(_err(loss[rows], want_loss), _err(lse[rows], want_lse))
    del logits
    return {
        "name": "fused_xent", "ms_per_step": ms, "kernel_ms": kms,
        "metric": "fused_linear_xent_fwd_tflops", "unit": "TFLOP/s", "value": flop / (ms * 1e-3) / 1e12,
        "max_abs_err": err,
        "err_sample": "loss and lse of 64 of the 8192 tokens against fp32 torch math on the device",
        "roofline": {"bound": "mfma", "achieved": flop / (kms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": KERNELS["fused_xent"]},
        "config": {"workload": "fused linear + cross-entropy forward bf16, T=8192 tokens, hidden 4096, vocabulary 128256",
                   "flop_per_step": flop, "bwd_ms_per_step": ms_bwd, "dlogits_kernel_ms": kms_grad,
                   "bwd_note": "backward = the same GEMM kernel with the dlogits epilogue (dlogits_kernel_ms) + two "
                               "gradient GEMMs from the BLAS library through torch.mm (6*T*D*N FLOP in all)",
                   "bwd_tflops": 3.0 * flop / (ms_bwd * 1e-3) / 1e12},
    }


def _packed_fwd_args(q, k, v, o, lse, cu, max_len, causal=True):
    """mi_attn_fwd_args for packed [1,T,H,D] tensors with cu_seqlens."""
    from tritonops_amd import _lib
    a = _lib.AttnFwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = (t.data_ptr() for t in (q, k, v, o, lse))
    for n, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, n + "_stride_s", t.stride(1))
        setattr(a, n + "_stride_h", t.stride(2))
    a.lse_stride_s, a.lse_stride_h = lse.stride(1), lse.stride(2)
    a.cu_seqlens = cu.data_ptr()
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = cu.numel() - 1, q.shape[2], k.shape[2], max_len, q.shape[3]
    a.causal = 1 if causal else 0
    a.scale_log2 = q.shape[3] ** -0.5 * LOG2E
    a.total_rows = q.shape[1]
    return a


def run_dense_packed(steps, warmup):
    """The reference's own call form of the dense forward: packed [1,T,H,D] tensors + cu_seq_lens through
    flash_attention(q, k, v, cu) (= flash_attn_triton.apply, flash_attn_triton.py:816-846), at the headline size
    (4 sequences of 8192 tokens) and on a ragged mix of the same 32768 tokens."""
    import tritonops_amd as ta
    T, H, D = 32768, 32, 128
    q, k, v = (_randn((1, T, H, D), s) for s in (0, 1, 2))
    mixes = {"4x8192": [8192] * 4, "ragged": [8192, 4096, 12288, 2048, 1024, 5120]}
    out = {}
    for name, lens in mixes.items():
        cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
        cu[1:] = torch.cumsum(torch.tensor(lens), 0)
        cu = cu.cuda()
        fn = lambda: ta.flash_attention(q, k, v, cu, return_lse=True)
        o, lse = fn()
        o2, lse2 = torch.empty_like(o), torch.empty_like(lse)
        # the device-time leg first, the wall-clock leg right behind it: both then see the clocks of a busy
        # device, and their ratio is what the Python call form costs on the host
        kms = _event_ms(0, _packed_fwd_args(q, k, v, o2, lse2, cu, max(lens)), steps, warmup)
        ms = _time_steps(fn, steps, warmup)
        flop = sum(2.0 * H * n * (n + 1) * D for n in lens)
        # parity on the benchmark tensors: two heads x three 64-row blocks of the first, a middle and the last sequence
        err = err_lse = 0.0
        for si in (0, len(lens) // 2, len(lens) - 1):
            s0, n = int(cu[si]), lens[si]
            keys = torch.arange(n, device="cuda")
            for h in (0, 21):
                for r0 in (0, n // 2, n - 64):
                    rows = torch.arange(r0, r0 + 64, device="cuda")
                    want, want_lse = _ref_rows(q[0, s0:s0 + n, h], k[0, s0:s0 + n, h], v[0, s0:s0 + n, h], rows,
                                               D ** -0.5, keys[None, :] <= rows[:, None])
                    err = max(err, _err(o[0, s0 + rows, h], want))
                    err_lse = max(err_lse, _err(lse[0, s0 + rows, h], want_lse))
        out[name] = dict(ms=ms, kms=kms, flop=flop, err=err, err_lse=err_lse)
    m = out["4x8192"]
    r = out["ragged"]
    return {
        "name": "dense_causal_packed", "ms_per_step": m["ms"], "kernel_ms": m["kms"],
        "metric": "attn_fwd_tflops", "unit": "TFLOP/s", "value": m["flop"] / (m["ms"] * 1e-3) / 1e12,
        "max_abs_err": max(m["err"], r["err"]), "max_abs_err_lse2": max(m["err_lse"], r["err_lse"]),
        "err_sample": "o and lse of 2 heads x 3 blocks of 64 query rows in 3 sequences of each mix against fp32 torch math on the device",
        "roofline": {"bound": "mfma", "achieved": m["flop"] / (m["kms"] * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": KERNELS["dense_causal_packed"]},
        "config": {"workload": "dense causal fwd bf16, packed [1,32768,32,128] + cu_seq_lens for 4 x 8192 tokens, through "
                               "flash_attention(q, k, v, cu_seq_lens) with uninitialised outputs (the library zeroes "
                               "rows outside the sequences) and the longest length cached per cu_seq_lens tensor",
                   "flop_per_step": m["flop"],
                   "wall_over_kernel": m["ms"] / m["kms"],
                   "wall_over_kernel_note": "the wall-clock leg of this workload runs right behind its device-time leg",
                   "ragged_mix": {"lens": mixes["ragged"], "ms_per_step": r["ms"], "kernel_ms": r["kms"],
                                  "flop_per_step": r["flop"], "tflops": r["flop"] / (r["kms"] * 1e-3) / 1e12,
                                  "frac": r["flop"] / (r["kms"] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                                  "wall_over_kernel": r["ms"] / r["kms"]}},
    }


def _window_pairs(n, lw, gw):
    """Allowed (q, k) pairs of one sequence of n tokens under k <= q and (q - k < lw or k < gw)."""
    import numpy as np
    qi = np.arange(n, dtype=np.int64)
    return int((np.minimum(qi + 1, lw) + np.maximum(0, np.minimum(gw, qi + 1 - lw))).sum())


def _run_window_prefill(name, B, H, S, LW, GW, lists, steps, warmup):
    """flash_attn_sparse_triton(q, k, v, cu, None, LW, GW) on B packed sequences of S tokens, head_dim 128; the
    device-time leg goes through the C ABI with the window's block lists (`lists`) or without any."""
    import tritonops_amd as ta
    from tritonops_amd import _lib, masks
    D = 128
    T = B * S
    q, k, v = (_randn((1, T, H, D), s) for s in (0, 1, 2))
    cu = (torch.arange(B + 1, dtype=torch.int32) * S).cuda()
    fn = lambda: ta.flash_attn_sparse_triton(q, k, v, cu, None, LW, GW)
    o, lse = fn()
    o2, lse2 = torch.empty_like(o), torch.empty_like(lse)
    a = _lib.AttnSparseArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = (t.data_ptr() for t in (q, k, v, o2, lse2))
    for n, t in (("q", q), ("k", k), ("v", v), ("o", o2)):
        setattr(a, n + "_stride_s", t.stride(1))
        setattr(a, n + "_stride_h", t.stride(2))
    a.lse_stride_s, a.lse_stride_h = lse2.stride(1), lse2.stride(2)
    a.cu_seqlens = cu.data_ptr()
    if lists:
        row_ptr, col_idx, strides = masks.window_csr(S // 64, LW, GW, "cuda")
        a.row_ptr, a.col_idx = row_ptr.data_ptr(), col_idx.data_ptr()
        a.row_ptr_stride_b, a.row_ptr_stride_h, a.col_idx_stride_b, a.col_idx_stride_h = strides
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, H, H, S, D
    a.block_size, a.window_local, a.window_global = 64, LW, GW
    a.scale_log2 = D ** -0.5 * LOG2E
    a.total_rows = T
    kms = _event_ms(1, a, steps, warmup)
    ms = _time_steps(fn, steps, warmup)          # behind the device-time leg (see run_dense_packed)
    flop = 4.0 * D * _window_pairs(S, LW, GW) * H * B
    err = err_lse = 0.0
    keys = torch.arange(S, device="cuda")
    for b in sorted({0, B - 1}):
        for r0 in (0, 1024, 4160, S - 64):
            rows = torch.arange(r0, r0 + 64, device="cuda")
            allow = (keys[None, :] <= rows[:, None]) & ((rows[:, None] - keys[None, :] < LW) | (keys[None, :] < GW))
            sl = slice(b * S, (b + 1) * S)
            want, want_lse = _ref_rows(q[0, sl].transpose(0, 1), k[0, sl].transpose(0, 1), v[0, sl].transpose(0, 1),
                                       rows, D ** -0.5, allow)
            err = max(err, _err(o[0, b * S + rows].transpose(0, 1), want))
            err_lse = max(err_lse, _err(lse[0, b * S + rows].transpose(0, 1), want_lse))
    return {
        "name": name, "ms_per_step": ms, "kernel_ms": kms,
        "metric": "sparse_attn_fwd_tflops", "unit": "TFLOP/s", "value": flop / (ms * 1e-3) / 1e12,
        "max_abs_err": err, "max_abs_err_lse2": err_lse,
        "err_sample": "o and lse of all heads x 4 blocks of 64 query rows in %d of the %d sequences against masked fp32 torch "
                      "math on the device" % (len({0, B - 1}), B),
        "roofline": {"bound": "mfma", "achieved": flop / (kms * 1e-3) / 1e12, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "kernel": KERNELS[name]},
        "config": {"workload": "window-sparse causal fwd bf16, packed [1,%d,%d,128] + cu_seqlens for %d x %d tokens, local "
                               "window %d, global window %d, through flash_attn_sparse_triton(q, k, v, cu, None, %d, %d)"
                               % (T, H, B, S, LW, GW, LW, GW),
                   "flop_per_step": flop, "wall_over_kernel": ms / kms,
                   "note": ("FLOP counts the allowed (q, k) pairs only; the kernel walks whole 64x64 blocks that hold one" if lists else
                            "FLOP counts the allowed (q, k) pairs only; no block lists: the library walks each 128-row item's "
                            "sink tiles and band (whole 32-key tiles)")},
    }


def run_window_sparse_prefill(steps, warmup):
    """The reference's own sparse prefill form: token windows on packed tensors
    (flash_attn_sparse_attn_triton.py:237-326), local window 1024, global window 128, 4 sequences of 8192 tokens."""
    return _run_window_prefill("window_sparse_prefill", 4, 16, 8192, 1024, 128, True, steps, warmup)


def run_window_long_prefill(steps, warmup):
    """The same call form with a long local window on a long sequence (4096 / 128, one sequence of 32768 tokens):
    the case the drop-in sends to the library without block lists."""
    return _run_window_prefill("window_long_prefill", 1, 16, 32768, 4096, 128, False, steps, warmup)


def run_window_sparse_decode(steps, warmup):
    """The reference's own sparse decoding form: flash_attention_sparse_decoding(q, k, v, cu_seq_lens, 256, 4096)
    (flash_attn_decoding_sparse.py:222-365) at the KV size of the block-list configuration."""
    import tritonops_amd as ta
    from tritonops_amd import _lib
    B, Hq, Hkv, L, D, GW, LW = 32, 32, 8, 131072, 128, 256, 4096
    g = torch.Generator().manual_seed(1)
    lens = (L - torch.randint(0, 64, (B,), generator=g)).to(torch.int32)
    cu = torch.zeros(B + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(lens, 0)
    cu_d, lens_d = cu.cuda(), lens.cuda()
    q = _randn((B, Hq, D), 0)
    kc, vc = _randn((B, Hkv, L, D), 1), _randn((B, Hkv, L, D), 2)
    k, v = kc.transpose(1, 2), vc.transpose(1, 2)
    fn = lambda: ta.flash_attention_sparse_decoding(q, k, v, cu_d, GW, LW)
    got = fn()
    lib = _lib.load()
    o = torch.empty((B, Hq, D), device="cuda", dtype=torch.bfloat16)
    a = _lib.DecodeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _lib.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_b, a.k_stride_s, a.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
    a.v_stride_b, a.v_stride_s, a.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
    a.o_stride_b, a.o_stride_h = o.stride(0), o.stride(1)
    a.seq_lens, a.cu_seqlens = None, cu_d.data_ptr()
    a.batch, a.heads_q, a.heads_kv, a.max_seqlen, a.head_dim = B, Hq, Hkv, L, D
    a.scale_log2 = D ** -0.5 * LOG2E
    a.split_tokens = 64
    a.window_form, a.window_local, a.window_global = 1, LW, GW
    a.max_blocks, a.block_size = GW // 64 + (LW + 63) // 64 + 1, 64
    a.split_blocks = lib.mi_decode_choose_split_blocks(B, Hkv, a.max_blocks, lib.mi_device_cu_count())
    nb = lib.mi_decode_workspace_bytes(C.byref(a))
    ws = torch.empty(nb, device="cuda", dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    k_split = _event_ms(3, a, steps, warmup)
    k_both = _event_ms(2, a, steps, warmup)
    ms = _time_steps(fn, steps, warmup)          # behind the device-time legs (see run_dense_packed)
    nbytes_alg = float(B * Hkv * (GW + LW) * D * 2 * 2)
    err = 0.0
    for b in (0, 15, 31):
        n = int(lens[b])
        tok = torch.cat([torch.arange(GW), torch.arange(n - LW, n)]).cuda()
        kk, vv = kc[b][:, tok].float(), vc[b][:, tok].float()
        sc = torch.einsum("gid,gld->gil", q[b].view(Hkv, Hq // Hkv, D).float(), kk) * D ** -0.5
        want = torch.einsum("gil,gld->gid", torch.softmax(sc, -1), vv).reshape(Hq, D)
        err = max(err, _err(got[b], want))
    return {
        "name": "window_sparse_decode", "ms_per_step": ms, "kernel_ms": k_both, "splitkv_kernel_ms": k_split,
        "metric": "sparse_decode_hbm_gbs", "unit": "GB/s", "value": nbytes_alg / (ms * 1e-3) / 1e9,
        "max_abs_err": err,
        "err_sample": "3 of the 32 sequences (all heads) against fp32 torch math over the attended tokens on the device",
        "roofline": {"bound": "hbm", "achieved": nbytes_alg / (k_split * 1e-3) / 1e9, "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "kernel": KERNELS["window_sparse_decode"]},
        "config": {"workload": "window-sparse decode bf16 B=32 Hq=32 Hkv=8 KV=131072 D=128, global window 256 + local window "
                               "4096, through flash_attention_sparse_decoding(q, k, v, cu_seq_lens, 256, 4096): two "
                               "launches, the block list is derived inside the kernel",
                   "bytes_per_step": nbytes_alg, "split_blocks": int(a.split_blocks),
                   "wall_over_kernel": ms / k_both,
                   "note": "kernel_ms is both launches (split-KV + merge), which is what one call costs on the device; "
                           "the roofline figure is the split-KV launch alone. 0.58 GB per step is little work for 256 "
                           "CUs: the launch is latency-bound, not bandwidth-bound"},
    }


WORKLOADS = {
    "dense_causal": run_dense_causal,
    "c1_dense_noncausal_small": run_c1_small,
    "gqa_decode": run_decode,
    "block_sparse": run_block_sparse,
    "sparse_decode": run_sparse_decode,
    "dense_causal_bwd": run_dense_bwd,
    "rmsnorm": run_rmsnorm,
    "fused_xent": run_fused_xent,
    "dense_causal_packed": run_dense_packed,
    "window_sparse_prefill": run_window_sparse_prefill,
    "window_sparse_decode": run_window_sparse_decode,
    "window_long_prefill": run_window_long_prefill,
}

# Parity bars: the largest error a workload's own check may report (its figure under "max_abs_err",
# plus the named extra ones).  A run that exceeds one, or reports a value that is not finite, prints its
# line with "parity_ok": false and exits with status 1, so that no timing is recorded for a wrong result.
PARITY_BARS = {
    "dense_causal": {"max_abs_err": 2e-2, "max_abs_err_lse2": 2e-3},
    "c1_dense_noncausal_small": {"max_abs_err": 2e-2},
    "gqa_decode": {"max_abs_err": 2e-2},
    "block_sparse": {"max_abs_err": 2e-2, "max_abs_err_lse2": 2e-3},
    "sparse_decode": {"max_abs_err": 2e-2},
    "dense_causal_bwd": {"max_abs_err": 3e-2},
    "rmsnorm": {"max_abs_err": 4e-2, "max_rel_err_dw": 1e-2},
    "fused_xent": {"max_abs_err": 2e-2},
    "dense_causal_packed": {"max_abs_err": 2e-2, "max_abs_err_lse2": 2e-3},
    "window_sparse_prefill": {"max_abs_err": 2e-2, "max_abs_err_lse2": 2e-3},
    "window_sparse_decode": {"max_abs_err": 2e-2},
    "window_long_prefill": {"max_abs_err": 2e-2, "max_abs_err_lse2": 2e-3},
}


def _parity(r):
    bars = PARITY_BARS[r["name"]]
    ok = all(k in r and math.isfinite(r[k]) and r[k] <= bar for k, bar in bars.items())
    return ok, bars


# ----------------------------------------------------------------------------
# CPU baseline: the reference's PyTorch math on this host, bounded slice
# ----------------------------------------------------------------------------
def cpu_baseline(name):
    from oracle import attention_oracle as orc
    threads = torch.get_num_threads()
    g = torch.Generator().manual_seed(0)

    def med(fn, reps=3):
        fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2]

    if name == "dense_causal":
        B, H, S, D = 1, 32, 8192, 128
        q, k, v = (torch.randn((B, H, S, D), generator=g).to(torch.bfloat16) for _ in range(3))
        t = med(lambda: orc.causal_attention(q, k, v))
        flop = 2.0 * B * H * S * (S + 1) * D
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU bf16 causal softmax(qk^T/sqrt(d))v (tutorial/4.4 oracle) on B=1 H=32 S=8192 D=128 (one of the workload's four sequences), "
                          "median of 3; same algorithmic-FLOP formula as the GPU figure",
                "seconds": t}
    if name == "c1_dense_noncausal_small":
        B, H, S, D = 1, 4, 256, 64
        q, k, v = (torch.randn((B, H, S, D), generator=g) for _ in range(3))
        t = med(lambda: orc.full_attention(q, k, v), reps=21)
        flop = 4.0 * B * H * S * S * D
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU fp32 softmax(q k^T / sqrt(d)) v (tutorial/4.3.multi_head_attention.py:11-19) on the "
                          "whole workload B=1 H=4 S=256 D=64, median of 21",
                "seconds": t}
    if name == "block_sparse":
        from tritonops_amd import masks
        B, H, S, D = 1, 2, 16384, 128
        m = masks.synthetic_block_mask(S // 64, 8, 4, 0.10, seed=2)
        live, nb = int(m.sum()), S // 64
        q, k, v = (torch.randn((1, S, H, D), generator=g).to(torch.bfloat16) for _ in range(3))
        cu = torch.tensor([0, S], dtype=torch.int32)
        t = med(lambda: orc.block_sparse_attention(q, k, v, cu, m), reps=1)
        flop = 4.0 * D * ((live - nb) * 64 * 64 + nb * 64 * 65 / 2) * B * H
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU bf16 masked softmax(q k^T scale) v under the same block mask (the math of "
                          "flash_attn_sparse_attn_triton.py:391-442; it computes the full S x S scores and masks them) "
                          "on B=1 H=2 of B=2 H=16 (1/16 of the workload), one timed run after a warm-up; same "
                          "algorithmic-FLOP formula as the GPU figure (live blocks only)",
                "seconds": t}
    if name == "sparse_decode":
        from tritonops_amd import masks
        B, Hq, Hkv, L, D = 2, 32, 8, 131072, 128
        lens = (L - torch.randint(0, 64, (B,), generator=g)).to(torch.int32)
        idx = masks.synthetic_decode_blocks(B, Hkv, L // 64, 128, seed=2)
        q = torch.randn((B, Hq, D), generator=g).to(torch.bfloat16)
        k, v = (torch.randn((B, L, Hkv, D), generator=g, dtype=torch.bfloat16) for _ in range(2))
        t = med(lambda: orc.block_sparse_decoding(q, k, v, lens, idx))
        nb = float(B * Hkv * 129 * 64 * D * 2 * 2)
        return {"value": nb / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU bf16 decode oracle (flash_attn_decoding_sparse.py:368-406 math under the block list) "
                          "on B=2 of the 32 sequences, median of 3; same algorithmic-byte formula as the GPU figure",
                "seconds": t}
    if name == "gqa_decode":
        B, Hq, Hkv, L, D = 8, 32, 8, 32768, 128
        lens = torch.randint(16384, L + 1, (B,), generator=g, dtype=torch.int32)
        q = torch.randn((B, Hq, D), generator=g).to(torch.bfloat16)
        k, v = (torch.randn((B, L, Hkv, D), generator=g).to(torch.bfloat16) for _ in range(2))
        t = med(lambda: orc.flash_attn_decoding_torch(q, k, v, lens))
        nb = float(lens.sum()) * Hkv * 2 * D * 2
        return {"value": nb / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU bf16 decode oracle (flash_attn_decoding.py:339-368) on B=8 of the 64 sequences, median of 3",
                "seconds": t}
    if name == "dense_causal_bwd":
        B, H, S, D = 1, 8, 4096, 128
        q, k, v, do = (torch.randn((B, H, S, D), generator=g).to(torch.bfloat16) for _ in range(4))
        ts = []
        for _ in range(3):
            qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
            o = orc.causal_attention(qq, kk, vv)
            t0 = time.perf_counter()
            o.backward(do)
            ts.append(time.perf_counter() - t0)
        t = sorted(ts)[1]
        flop = 2.5 * 2.0 * B * H * S * (S + 1) * D
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU autograd backward through the bf16 causal oracle (tutorial/4.4 math) on B=1 H=8 "
                          "S=4096 D=128, median of 3; same algorithmic-FLOP formula as the GPU figure",
                "seconds": t}
    if name == "rmsnorm":
        from oracle import rms_oracle as rorc
        T, D, eps = 4096, 4096, 1e-6
        x, dy = (torch.randn((T, D), generator=g).to(torch.bfloat16) for _ in range(2))
        w = torch.ones(D)

        def fn():
            rorc.rms_norm(x.float(), w, eps).to(torch.bfloat16)
            rorc.rms_norm_backward(dy.float(), x.float(), w, eps)
        t = med(fn)
        nbytes = 5.0 * T * D * 2 + 2 * T * 4
        return {"value": nbytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU RMSNorm forward (fp32 math, bf16 result) + float64 backward formulas of the oracle "
                          "(common/rms.py math) on [4096, 4096] bf16 (1/8 of the rows), median of 3; same "
                          "algorithmic-byte formula as the GPU figure",
                "seconds": t}
    if name == "dense_causal_packed":
        S, H, D = 8192, 4, 128
        q, k, v = (torch.randn((1, S, H, D), generator=g).to(torch.bfloat16) for _ in range(3))
        cu = torch.tensor([0, S], dtype=torch.int32)
        t = med(lambda: orc.flash_attn_torch(q, k, v, cu), reps=1)
        flop = 2.0 * H * S * (S + 1) * D
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU var-len causal oracle (flash_attn_triton.py:877-915 math) on one packed sequence of 8192 "
                          "tokens, 4 of the 32 heads (1/32 of the workload), one timed run after a warm-up; same "
                          "algorithmic-FLOP formula as the GPU figure",
                "seconds": t}
    if name == "window_sparse_prefill":
        S, H, D, LW, GW = 8192, 4, 128, 1024, 128
        q, k, v = (torch.randn((1, S, H, D), generator=g).to(torch.bfloat16) for _ in range(3))
        cu = torch.tensor([0, S], dtype=torch.int32)
        t = med(lambda: orc.flash_attn_sparse_torch(q, k, v, cu, None, LW, GW), reps=1)
        flop = 4.0 * D * _window_pairs(S, LW, GW) * H
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU window oracle (flash_attn_sparse_attn_triton.py:391-442: full S x S scores, then the "
                          "mask) on one sequence of 8192 tokens, 4 of the 16 heads (1/16 of the workload), one timed run "
                          "after a warm-up; same algorithmic-FLOP formula as the GPU figure (allowed pairs only)",
                "seconds": t}
    if name == "window_long_prefill":
        S, H, D, LW, GW = 8192, 4, 128, 4096, 128
        q, k, v = (torch.randn((1, S, H, D), generator=g).to(torch.bfloat16) for _ in range(3))
        cu = torch.tensor([0, S], dtype=torch.int32)
        t = med(lambda: orc.flash_attn_sparse_torch(q, k, v, cu, None, LW, GW), reps=1)
        flop = 4.0 * D * _window_pairs(S, LW, GW) * H
        return {"value": flop / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU window oracle (flash_attn_sparse_attn_triton.py:391-442: full S x S scores, then the "
                          "mask) with the same two windows on a sequence of 8192 tokens (a quarter of the workload's) and 4 "
                          "of the 16 heads, one timed run after a warm-up; same algorithmic-FLOP formula as the GPU figure "
                          "(allowed pairs only)",
                "seconds": t}
    if name == "window_sparse_decode":
        B, Hq, Hkv, L, D, GW, LW = 1, 32, 8, 131072, 128, 256, 4096
        lens = (L - torch.randint(0, 64, (B,), generator=g)).to(torch.int32)
        q = torch.randn((B, Hq, D), generator=g).to(torch.bfloat16)
        k, v = (torch.randn((B, L, Hkv, D), generator=g, dtype=torch.bfloat16) for _ in range(2))
        t = med(lambda: orc.flash_attn_sparse_decoding_torch(q, k, v, lens, GW, LW))
        nb = float(B * Hkv * (GW + LW) * D * 2 * 2)
        return {"value": nb / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU window decode oracle (flash_attn_decoding_sparse.py:368-406) on one of the 32 "
                          "sequences, median of 3; same algorithmic-byte formula as the GPU figure",
                "seconds": t}
    if name == "fused_xent":
        from oracle import xent_oracle as xo
        T, D, N = 128, 4096, 128256
        x = torch.randn((T, D), generator=g).to(torch.bfloat16)
        w = (torch.randn((N, D), generator=g) * D ** -0.5).to(torch.bfloat16)
        y = torch.randint(0, N, (T,), generator=g)

        def fn():
            logits = (x @ w.t()).float()
            return torch.logsumexp(logits, -1) - logits.gather(-1, y.view(-1, 1)).squeeze(-1)
        t = med(fn)
        return {"value": 2.0 * T * D * N / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "sample": "torch-CPU bf16 x @ w^T, fp32 logsumexp - target logit (cross_entropy.py:428-435 math) on 128 of "
                          "the 8192 tokens, median of 3; same FLOP formula as the GPU figure",
                "seconds": t}
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=40)
    ap.add_argument("--warmup", type=int, default=15)
    ap.add_argument("--workload", default="all", choices=["all"] + list(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also launch one elementwise copy of 1 GiB (2 GiB of HBM traffic) as the reference "
                         "dispatch for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    ap.add_argument("--dense-shape", default=None, metavar="B,H,S[,D]",
                    help="batch, heads, sequence length and head_dim of the dense_causal workload instead of the "
                         "benchmark's 4,32,8192,128 (S a multiple of 64, at least 256; D 64, 96 or 128; for "
                         "profiling other shapes)")
    ap.add_argument("--dense-form", default="auto", choices=["auto", "256", "128"],
                    help="pin the dense_causal workload to one form of the dense kernel (work items of 256 or of 128 "
                         "query rows) instead of the library's per-launch choice; for profiling")
    a = ap.parse_args()
    global DENSE_FORM
    DENSE_FORM = a.dense_form
    if a.dense_shape:
        global DENSE_SHAPE
        sh = tuple(int(x) for x in a.dense_shape.split(","))
        if len(sh) == 3:
            sh += (128,)
        if len(sh) != 4 or min(sh) < 1 or sh[2] % 64 or sh[2] < 256 or sh[3] not in (64, 96, 128):
            sys.exit("bench.py: --dense-shape takes B,H,S[,D] with S a multiple of 64, at least 256, and D 64, 96 or 128")
        DENSE_SHAPE = sh
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the attention path shards over batch and "
                 "heads without communication); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from tritonops_amd import _lib
    _lib.load()   # fail loudly when the HIP library is missing

    if a.traffic_probe:
        src = torch.ones(1 << 29, device="cuda", dtype=torch.bfloat16)
        dst = torch.empty_like(src)
        torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    traffic = {}
    tfile = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tfile):
        traffic = json.load(open(tfile))   # bytes per launch measured with rocprofv3 --pmc (see profiles/)
    names = list(WORKLOADS) if a.workload == "all" else [a.workload]
    results = []
    for n in names:
        r = WORKLOADS[n](a.steps, a.warmup)
        rf = r["roofline"]
        rf["frac"] = rf["achieved"] / rf["peak"]
        # HBM bytes per launch from the committed rocprofv3 counter runs; only a reading taken from the
        # kernels this workload launches today is reported
        t = traffic.get(r["name"], {})
        fresh = t.get("kernel") == rf["kernel"]
        rf["traffic"] = t.get("hbm_bytes_per_launch") if fresh else None
        rf["traffic_source"] = ("profiles/hbm_traffic.json, measured at commit %s" % t.get("commit", traffic.get("_commit", "?"))
                                if fresh else "no counter run of this kernel on file")
        r["parity_ok"], r["parity_bars"] = _parity(r)
        results.append(r)
        torch.cuda.empty_cache()
    head = results[0]
    out = {
        "metric": head["metric"], "value": head["value"], "unit": head["unit"],
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic N(0,1) inputs drawn from a seed, resident in HBM",
        "config": head["config"], "roofline": head["roofline"], "kernel_ms": head["kernel_ms"],
        "max_abs_err": head.get("max_abs_err"), "err_sample": head.get("err_sample"),
        "parity_ok": all(r["parity_ok"] for r in results), "parity_bars": head["parity_bars"],
        "device": torch.cuda.get_device_name(0),
        "compute_units": torch.cuda.get_device_properties(0).multi_processor_count,
    }
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(head["name"])
        if out["cpu_baseline"] is not None:
            out["cpu_baseline"]["host_cpus"] = os.cpu_count()
    if len(results) > 1:
        out["other_workloads"] = [
            {k: r[k] for k in ("name", "metric", "value", "unit", "ms_per_step", "kernel_ms", "max_abs_err",
                               "max_abs_err_lse2", "max_rel_err_dw", "err_sample", "parity_ok", "parity_bars",
                               "roofline", "config") if k in r}
            for r in results[1:]]
        if not a.no_cpu_baseline:
            for r in out["other_workloads"]:
                cb = cpu_baseline(r["name"])
                if cb is not None:
                    r["cpu_baseline"] = cb
    print(json.dumps(out))
    if not out["parity_ok"]:
        bad = [r["name"] for r in results if not r["parity_ok"]]
        sys.exit("bench.py: parity bar exceeded by %s; the timings above are of wrong results" % ", ".join(bad))


if __name__ == "__main__":
    main()
