"""Drop-in Python entry points of the attention forward path.

Names, positional arguments and semantics follow the reference launchers
(citations per function, paths relative to the reference checkout); the work
is done by the HIP kernels of libmi_attn.so reached through its C ABI.  There
is no fallback: without the built library every call raises.
"""
import contextlib
import ctypes as C
import math
import threading
import weakref

import torch

from . import _lib
from . import masks as _masks

LOG2E = 1.4426950408889634
# flash_attn_sparse_triton's window form runs either on block lists built on the
# host (the block-list kernel, as every other mask) or without lists: the library
# then walks each 128-row item's sink tiles and band with the dense kernel's
# pipeline.  The second is 5 to 9 % faster for local windows of 2048 tokens or more
# at head_dim 96 / 128 (B1 H16 S32768: 0.586 against 0.615 ms at 2048, 0.995 against
# 1.087 ms at 4096) and up to 11 % slower for short windows and at head_dim 64, so
# the choice is made per call.  True / False force one of the two (tests).
WINDOW_PREFILL_LISTS = None
_WINDOW_WALK_MIN_LOCAL = 2048
_CU_COUNT = {}


def _num_cus(lib):
    """Compute units of the current device, as the library's own launches see
    them (cached per device)."""
    dev = torch.cuda.current_device()
    n = _CU_COUNT.get(dev)
    if n is None:
        n = _CU_COUNT[dev] = int(lib.mi_device_cu_count())
    return n


def _dtype_tag(t):
    if t.dtype == torch.bfloat16:
        return _lib.MI_DTYPE_BF16
    if t.dtype == torch.float16:
        return _lib.MI_DTYPE_F16
    raise TypeError("attention inputs must be bfloat16 or float16, got %s" % t.dtype)


def _require_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("tritonops_amd runs on the GPU only (tensor on %s); there is no CPU path" % t.device)


# torch's raw-stream getter skips the Stream object that torch.cuda.current_stream() builds (3 to 4 us per call)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    if _raw_stream is not None:
        return C.c_void_p(_raw_stream(torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _inner_contig(t):
    return t if t.stride(-1) == 1 else t.contiguous()


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


_MAX_LEN_CACHE = {}   # id(cu tensor) -> (weak reference, version counter, longest sequence, first and last entry)


def _cu_facts(cu_seq_lens):
    """(longest sequence, cu[0], cu[-1]) of a cu_seq_lens tensor, kept per tensor
    OBJECT for as long as that object lives and its version counter (bumped by
    every in-place write) has not moved; one host round trip the first time."""
    key = id(cu_seq_lens)
    hit = _MAX_LEN_CACHE.get(key)
    if hit is not None and hit[0]() is cu_seq_lens and hit[1] == cu_seq_lens._version:
        return hit[2]
    if cu_seq_lens.numel() < 2:
        facts = (0, 0, 0)
    else:
        facts = tuple(int(x) for x in torch.stack(
            [(cu_seq_lens[1:] - cu_seq_lens[:-1]).max(), cu_seq_lens[0], cu_seq_lens[-1]]).tolist())
    if len(_MAX_LEN_CACHE) >= 256:
        _MAX_LEN_CACHE.clear()
    try:
        _MAX_LEN_CACHE[key] = (weakref.ref(cu_seq_lens), cu_seq_lens._version, facts)
    except TypeError:
        pass
    return facts


def _max_len(cu_seq_lens, max_seq_len):
    """Longest sequence of the batch, which sizes the launch.  Without a hint
    it costs the host round trip the reference launcher makes on every call
    (flash_attn_triton/flash_attn_triton.py:621); here the answer is kept per
    cu_seq_lens tensor object (_cu_facts), so the layers of a model that share
    one cu_seq_lens pay for it once per batch."""
    if max_seq_len is not None:
        return int(max_seq_len)
    return _cu_facts(cu_seq_lens)[0]


def _rows_to_cover(cu_seq_lens, max_seqlen, rows):
    """total_rows of a packed call: `rows` (the library zeroes the rows of the
    outputs that belong to no sequence), or 0 when the host already knows that
    there is no such row - the sequences tile [0, rows) and none is longer than
    the `max_seqlen` the call runs with - which saves the small launch that
    looks for them.  Known only while the lengths of this cu_seq_lens object
    are on file from an earlier host read (_cu_facts); never read here."""
    hit = _MAX_LEN_CACHE.get(id(cu_seq_lens))
    if hit is None or hit[0]() is not cu_seq_lens or hit[1] != cu_seq_lens._version:
        return rows
    longest, first, last = hit[2]
    return 0 if (first == 0 and last == rows and longest <= max_seqlen) else rows


_HEAD_DIMS = (64, 96, 128)


def _padded_head_dim(D):
    """Smallest head_dim the kernels are built for that holds D.  The reference
    pads every head_dim to the next power of two inside its kernels
    (flash_attn_triton.py:612); zero columns change neither q.k nor the first D
    columns of the output."""
    for d in _HEAD_DIMS:
        if D <= d:
            return d
    raise ValueError(
        "head_dim %d exceeds %d, the widest row the gfx950 kernels of this library are built for (rows of 64, 96 "
        "and 128 elements; smaller head_dims are zero-padded to the next of them).  The reference pads any "
        "head_dim to a power of two and tiles the value dimension by 128 (flash_attn_triton.py:612,622); nothing "
        "wider is implemented here, and no device work has been started." % (D, _HEAD_DIMS[-1]))


def _pad_last(t, Dp):
    return t if t.shape[-1] == Dp else torch.nn.functional.pad(t, (0, Dp - t.shape[-1]))


def _check_qkv(q, k, v):
    """Extents of k and v against q, all as [X, S, H, D]: the kernels take every
    extent from q, so a shorter k or v would be read past its end."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k and v must be 4-dimensional")
    if k.shape[-1] != q.shape[-1] or v.shape[-1] != q.shape[-1]:
        raise ValueError("q, k and v must share head_dim (got %d, %d, %d)" % (q.shape[-1], k.shape[-1], v.shape[-1]))
    if k.shape[:2] != q.shape[:2]:
        raise ValueError("k %s must have the batch and sequence extents of q %s" % (tuple(k.shape), tuple(q.shape)))
    if v.shape != k.shape:
        raise ValueError("v %s must have the shape of k %s" % (tuple(v.shape), tuple(k.shape)))
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k and v must share one dtype (got %s, %s, %s)" % (q.dtype, k.dtype, v.dtype))
    if k.shape[2] == 0 or q.shape[2] % max(k.shape[2], 1) != 0:
        raise ValueError("heads_q %d must be a positive multiple of heads_kv %d" % (q.shape[2], k.shape[2]))


def _fill_qkvo(a, q, k, v, o, lse, packed):
    """q/k/v/o given as [X, S, H, D] views (X = 1 packed, X = B batched)."""
    a.q, a.k, a.v, a.o, a.lse = _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse)
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o)):
        setattr(a, name + "_stride_b", 0 if packed else t.stride(0))
        setattr(a, name + "_stride_s", t.stride(1))
        setattr(a, name + "_stride_h", t.stride(2))
    if lse is not None:
        a.lse_stride_b = 0 if packed else lse.stride(0)
        a.lse_stride_s = lse.stride(1)
        a.lse_stride_h = lse.stride(2)


_DENSE_FORMS = {"auto": _lib.MI_DENSE_FORM_AUTO, "256": _lib.MI_DENSE_FORM_256_ROWS, "128": _lib.MI_DENSE_FORM_128_ROWS}
_dense_form = threading.local()


@contextlib.contextmanager
def dense_form(form):
    """Dense forward calls of this thread inside the block run in one form of
    the kernel: "256" (work items of 256 query rows, 8-wave workgroups), "128"
    (128 rows, 4-wave workgroups) or "auto" (the library picks per launch, the
    default).  The forms give the same bits; the switch is for tests and for
    callers who have timed their own shapes."""
    if form not in _DENSE_FORMS:
        raise ValueError("dense_form takes 'auto', '256' or '128', got %r" % (form,))
    before = getattr(_dense_form, "value", _lib.MI_DENSE_FORM_AUTO)
    _dense_form.value = _DENSE_FORMS[form]
    try:
        yield
    finally:
        _dense_form.value = before


def _dense_fwd(q, k, v, cu_seq_lens, scale_log2, causal, max_seq_len, want_lse=True, bhsd=False):
    """q,k,v as [X, S, H, D] (see _fill_qkvo). Returns (o, lse[X, S, H]); with
    `bhsd` the outputs own [X, H, S, D] / [X, H, S] memory and are returned as
    [X, S, H, ...] views of it."""
    _check_qkv(q, k, v)
    _require_gpu(q, k, v, cu_seq_lens)
    lib = _lib.load()
    q, k, v = _inner_contig(q), _inner_contig(k), _inner_contig(v)
    packed = cu_seq_lens is not None
    X, S, Hq, D = q.shape
    Dp = _padded_head_dim(D)
    if Dp != D:
        o, lse = _dense_fwd(_pad_last(q, Dp), _pad_last(k, Dp), _pad_last(v, Dp), cu_seq_lens, scale_log2, causal,
                            max_seq_len, want_lse, bhsd)
        if bhsd:
            return o.transpose(1, 2)[..., :D].contiguous().transpose(1, 2), lse
        return o[..., :D].contiguous(), lse
    if bhsd:
        o = torch.empty((X, Hq, S, D), device=q.device, dtype=q.dtype).transpose(1, 2)
        lse = torch.empty((X, Hq, S), device=q.device, dtype=torch.float32).transpose(1, 2) if want_lse else None
    else:
        # packed: rows outside every sequence (padding behind cu_seq_lens[-1]) are
        # zero in the reference, which zero-fills both outputs first
        # (flash_attn_triton.py:608-609); here the library zeroes just those rows
        # (total_rows below)
        o = torch.empty((X, S, Hq, D), device=q.device, dtype=q.dtype)
        lse = torch.empty((X, S, Hq), device=q.device, dtype=torch.float32) if want_lse else None
    if q.numel() == 0:
        return o, lse  # no token: nothing to launch (empty tensors have no address to pass)
    a = _lib.AttnFwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_tag(q)
    _fill_qkvo(a, q, k, v, o, lse, packed)
    if packed:
        if X != 1:
            raise ValueError("packed layout expects a leading dimension of 1")
        cu = cu_seq_lens.to(torch.int32)
        a.cu_seqlens = _ptr(cu)
        a.batch = cu.numel() - 1
        a.max_seqlen = min(_max_len(cu_seq_lens, max_seq_len), S)
        a.total_rows = _rows_to_cover(cu_seq_lens, a.max_seqlen, S)
    else:
        a.cu_seqlens = None
        a.batch = X
        a.max_seqlen = S
    a.heads_q, a.heads_kv, a.head_dim = Hq, k.shape[2], D
    a.causal = 1 if causal else 0
    a.scale_log2 = float(scale_log2)
    a.dense_form = getattr(_dense_form, "value", _lib.MI_DENSE_FORM_AUTO)
    _lib.check(lib.mi_attn_fwd(C.byref(a), _stream()))
    return o, lse


def _dense_bwd(q, k, v, o, do, lse, cu_seq_lens, scale_log2, causal, max_seq_len):
    """q, k, v, o, do as [X, S, H, D] views, lse [X, S, H] (see _fill_qkvo).
    Returns dq, dk, dv shaped and laid out like q, k, v."""
    _check_qkv(q, k, v)
    if o.shape != q.shape or do.shape != q.shape:
        raise ValueError("o %s and do %s must have the shape of q %s" % (tuple(o.shape), tuple(do.shape), tuple(q.shape)))
    if o.dtype != q.dtype or do.dtype != q.dtype:
        raise ValueError("o and do must have the dtype of q (%s), got %s and %s" % (q.dtype, o.dtype, do.dtype))
    if lse.shape != q.shape[:3] or lse.dtype != torch.float32:
        raise ValueError("lse must be float32 %s as returned by the forward, got %s %s"
                         % (tuple(q.shape[:3]), lse.dtype, tuple(lse.shape)))
    _require_gpu(q, k, v, o, do, lse, cu_seq_lens)
    lib = _lib.load()
    q, k, v, o, do = (_inner_contig(t) for t in (q, k, v, o, do))
    packed = cu_seq_lens is not None
    X, S, Hq, D = q.shape
    Dp = _padded_head_dim(D)
    if Dp != D:
        grads = _dense_bwd(*(_pad_last(t, Dp) for t in (q, k, v, o, do)), lse, cu_seq_lens,
                           scale_log2, causal, max_seq_len)
        return tuple(g[..., :D].contiguous() for g in grads)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    if q.numel() == 0:
        return dq, dk, dv
    a = _lib.AttnBwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_tag(q)
    for name, t in (("q", q), ("k", k), ("v", v), ("o", o), ("dout", do), ("dq", dq), ("dk", dk), ("dv", dv),
                    ("lse", lse)):
        setattr(a, name, _ptr(t))
        setattr(a, name + "_stride_b", 0 if packed else t.stride(0))
        setattr(a, name + "_stride_s", t.stride(1))
        setattr(a, name + "_stride_h", t.stride(2))
    if packed:
        cu = cu_seq_lens.to(torch.int32)
        a.cu_seqlens = _ptr(cu)
        a.batch = cu.numel() - 1
        a.max_seqlen = min(_max_len(cu_seq_lens, max_seq_len), S)
        a.total_rows = _rows_to_cover(cu_seq_lens, a.max_seqlen, S)  # rows outside every sequence receive zeros
    else:
        a.cu_seqlens = None
        a.batch = X
        a.max_seqlen = S
    a.heads_q, a.heads_kv, a.head_dim = Hq, k.shape[2], D
    a.causal = 1 if causal else 0
    a.scale_log2 = float(scale_log2)
    nbytes = lib.mi_attn_bwd_workspace_bytes(C.byref(a))
    ws = torch.empty(max(nbytes, 16), device=q.device, dtype=torch.uint8)
    a.workspace, a.workspace_bytes = _ptr(ws), nbytes
    _lib.check(lib.mi_attn_bwd(C.byref(a), _stream()))
    return dq, dk, dv


def flash_attn_triton_bwd(q, k, v, o, do, lse, cu_seq_lens, sm_scale, *, max_seq_len=None):
    """Causal var-len GQA backward on packed tensors: contract and argument
    order of flash_attn_triton_bwd in flash_attn_triton/flash_attn_triton.py
    :661-670 (`do` before `lse`; `sm_scale` contains log2(e), `lse` is the
    base-2 LSE the forward returned).  Returns (dq, dk, dv) with the shapes of
    q, k, v; rows outside every sequence receive zeros."""
    return _dense_bwd(q, k, v, o, do, lse, cu_seq_lens, sm_scale, True, max_seq_len)


def flash_attn_triton_fwd(q, k, v, cu_seq_lens, sm_scale, *, max_seq_len=None):
    """Causal var-len GQA forward on packed tensors.

    Same contract as flash_attn_triton_fwd in
    flash_attn_triton/flash_attn_triton.py:595-658: q [1,T,Hq,D], k/v
    [1,T,Hkv,D], cu_seq_lens [B+1]; `sm_scale` already contains log2(e)
    (:839).  Returns (o [1,T,Hq,D], lse [1,T,Hq] fp32, base 2).  Rows outside
    every sequence are zero in both, as in the reference (:608-609).
    `max_seq_len` skips the host sync that sizes the grid (:621); it must be
    an upper bound of every sequence length: a longer sequence is cut at the
    bound (its later rows are not attended and come back as zeros).
    """
    return _dense_fwd(q, k, v, cu_seq_lens, sm_scale, True, max_seq_len)


class flash_attn_triton(torch.autograd.Function):
    """`flash_attn_triton.apply(q, k, v, cu_seq_lens) -> o`, the autograd entry
    of flash_attn_triton/flash_attn_triton.py:816-874 (forward :819-846,
    backward :848-874)."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seq_lens):
        sm_scale = (1 / q.shape[-1]) ** 0.5 * LOG2E
        ctx.max_len = _max_len(cu_seq_lens, None)   # once: the backward gets the saved tensors as new objects
        o, lse = flash_attn_triton_fwd(q, k, v, cu_seq_lens, sm_scale, max_seq_len=ctx.max_len)
        ctx.save_for_backward(q, k, v, o, lse, cu_seq_lens)
        ctx.sm_scale = sm_scale
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, cu_seq_lens = ctx.saved_tensors
        dq, dk, dv = flash_attn_triton_bwd(q, k, v, o, do, lse, cu_seq_lens, ctx.sm_scale, max_seq_len=ctx.max_len)
        return dq, dk, dv, None


class _FlashAttention(torch.autograd.Function):
    """Autograd path of flash_attention(): q, k, v as [X, S, H, D] views, any
    of the forward's options; the backward is the dense backward with the same
    mask and scale."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seq_lens, scale_log2, causal, max_seq_len, bhsd):
        if cu_seq_lens is not None and max_seq_len is None:
            max_seq_len = _max_len(cu_seq_lens, None)
        o, lse = _dense_fwd(q, k, v, cu_seq_lens, scale_log2, causal, max_seq_len, True, bhsd)
        ctx.save_for_backward(q, k, v, o, lse, cu_seq_lens)
        ctx.opts = (scale_log2, causal, max_seq_len)
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, o, lse, cu_seq_lens = ctx.saved_tensors
        scale_log2, causal, max_seq_len = ctx.opts
        dq, dk, dv = _dense_bwd(q, k, v, o, do, lse, cu_seq_lens, scale_log2, causal, max_seq_len)
        return dq, dk, dv, None, None, None, None, None


def flash_attention(q, k, v, cu_seq_lens=None, *, causal=True, softmax_scale=None,
                    return_lse=False, max_seq_len=None):
    """The entry point the reference README advertises (README.md:30-31).

    Packed form (cu_seq_lens given): identical to flash_attn_triton.apply —
    q [1,T,Hq,D], k/v [1,T,Hkv,D], always per-sequence causal in the reference
    (flash_attn_triton.py:819-846); `causal=False` is an extension.
    Batched form (cu_seq_lens None): q [B,H,S,D], k/v [B,Hkv,S,D], the layout
    of tutorial/4.3.multi_head_attention.py:153-194 (non-causal) and
    tutorial/4.4.causal_attention.py (causal).
    `softmax_scale` is in the natural base; default D^-0.5.
    Returns o, or (o, lse2) with return_lse (lse2 [1,T,Hq] / [B,H,S]).
    Differentiable in q, k and v (like flash_attn_triton.apply, of which the
    README's flash_attention is an alias): when an input requires a gradient
    the call is recorded for autograd and backward runs the dense backward.
    """
    D = q.shape[-1]
    scale = (D ** -0.5 if softmax_scale is None else float(softmax_scale)) * LOG2E
    needs_grad = torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)
    if cu_seq_lens is not None:
        if needs_grad:
            o, lse = _FlashAttention.apply(q, k, v, cu_seq_lens, scale, causal, max_seq_len, False)
        else:
            o, lse = _dense_fwd(q, k, v, cu_seq_lens, scale, causal, max_seq_len, return_lse)
        return (o, lse) if return_lse else o
    if q.dim() != 4:
        raise ValueError("batched form expects [B, H, S, D] tensors")
    if needs_grad:
        o, lse = _FlashAttention.apply(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, scale, causal,
                                       None, True)
    else:
        o, lse = _dense_fwd(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, scale, causal,
                            None, return_lse, bhsd=True)
    o = o.transpose(1, 2)  # contiguous [B,H,S,D]
    if return_lse:
        return o, lse.transpose(1, 2)
    return o


def flash_attn_sparse_triton(q, k, v, cu_seqlens, softmax_scale=None, local_window_size=0,
                             global_window_size=0, *, block_mask=None, row_ptr=None, col_idx=None,
                             csr_strides=(0, 0, 0, 0), max_seq_len=None):
    """Sparse causal forward on packed tensors; returns (o, lse2).

    Window form — the launcher of
    flash_attn_triton/flash_attn_sparse_attn_triton.py:237-326 (the name is the
    one its test calls, :480): attends k <= q and (q - k < local_window_size
    or k < global_window_size), the rule of the oracle at :422-433, applied per
    token.  `softmax_scale` is in the natural base as in that oracle (:405-406).
    With cu_seqlens=None the tensors are batched [B,H,S,D] (extension).
    Block form — pass `block_mask` (bool [nq,nq] / [H,nq,nq] / [B,H,nq,nq] over
    64-token blocks, lower triangular) or a prebuilt CSR (`row_ptr`, `col_idx`,
    `csr_strides`); diagonal blocks are masked causally per token.
    A query with no allowed key gets o = 0 and lse = -inf.
    """
    if cu_seqlens is not None:
        _check_qkv(q, k, v)
    else:
        _check_qkv(*(t.transpose(1, 2) if t.dim() == 4 else t for t in (q, k, v)))
    _require_gpu(q, k, v, cu_seqlens)
    lib = _lib.load()
    D0 = q.shape[-1]
    if _padded_head_dim(D0) != D0:
        Dp = _padded_head_dim(D0)
        o, lse = flash_attn_sparse_triton(
            _pad_last(q, Dp), _pad_last(k, Dp), _pad_last(v, Dp), cu_seqlens,
            D0 ** -0.5 if softmax_scale is None else softmax_scale, local_window_size, global_window_size,
            block_mask=block_mask, row_ptr=row_ptr, col_idx=col_idx, csr_strides=csr_strides, max_seq_len=max_seq_len)
        return o[..., :D0].contiguous(), lse
    q, k, v = _inner_contig(q), _inner_contig(k), _inner_contig(v)
    packed = cu_seqlens is not None
    if packed:
        X, T, Hq, D = q.shape
        if X != 1:
            raise ValueError("packed layout expects a leading dimension of 1")
        cu = cu_seqlens.to(torch.int32)
        max_len = min(_max_len(cu_seqlens, max_seq_len), T)
        # rows outside every sequence are zero in the reference, which zero-fills
        # both outputs (flash_attn_sparse_attn_triton.py:274-275); the library
        # zeroes just those rows (total_rows below)
        o = torch.empty_like(q)
        lse = torch.empty((1, T, Hq), device=q.device, dtype=torch.float32)
        qv, kv, vv, ov, lv = q, k, v, o, lse
        batch = cu.numel() - 1
    else:
        # batched [B,H,S,D] form (extension, same layout as flash_attention)
        X, Hq, T, D = q.shape
        cu = None
        max_len = T
        o = torch.empty((X, Hq, T, D), device=q.device, dtype=q.dtype)
        lse = torch.empty((X, Hq, T), device=q.device, dtype=torch.float32)
        qv, kv, vv, ov, lv = (t.transpose(1, 2) for t in (q, k, v, o, lse))
        batch = X
    scale = (D ** -0.5 if softmax_scale is None else float(softmax_scale)) * LOG2E
    nqb = max((max_len + _masks.BLOCK - 1) // _masks.BLOCK, 1)
    wl = wg = -1
    if row_ptr is None:
        if block_mask is None:
            wl, wg = int(local_window_size), int(global_window_size)
            if wl < 0 or wg < 0:
                raise ValueError("window sizes must be >= 0")
            wl, wg = min(wl, 2 ** 31 - 1), min(wg, 2 ** 31 - 1)   # (the C ABI takes 32-bit windows; longer than any sequence either way)
            # The library works the blocks out from the two windows when it
            # gets no lists.  (local_window_size 0 hides even the diagonal; that
            # case always goes through lists.)
            use_lists = WINDOW_PREFILL_LISTS
            if use_lists is None:
                use_lists = not (D >= 96 and wl >= _WINDOW_WALK_MIN_LOCAL)
            if wl < 1 or use_lists:
                row_ptr, col_idx, csr_strides = _masks.window_csr(nqb, wl, wg, q.device)
        else:
            row_ptr, col_idx, csr_strides = _masks.block_mask_to_csr(block_mask, q.device)
        if row_ptr is not None and row_ptr.shape[-1] - 1 < nqb:
            raise ValueError("block mask covers %d query blocks, sequences need %d" % (row_ptr.shape[-1] - 1, nqb))
    if q.numel() == 0:
        return o, lse
    a = _lib.AttnSparseArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_tag(q)
    _fill_qkvo(a, qv, kv, vv, ov, lv, packed)
    a.cu_seqlens = _ptr(cu)
    a.row_ptr, a.col_idx = _ptr(row_ptr), _ptr(col_idx)
    a.row_ptr_stride_b, a.row_ptr_stride_h, a.col_idx_stride_b, a.col_idx_stride_h = csr_strides
    a.batch = batch
    a.heads_q, a.heads_kv, a.head_dim = Hq, kv.shape[2], D
    a.max_seqlen = max_len
    a.block_size = _masks.BLOCK
    a.window_local, a.window_global = wl, wg
    a.scale_log2 = scale
    a.total_rows = _rows_to_cover(cu_seqlens, max_len, T) if packed else 0
    _lib.check(lib.mi_attn_fwd_blocksparse(C.byref(a), _stream()))
    return o, lse


def _decode(q, k, v, cu_seq_lens, seq_lens, scale, max_seq_len, split_tokens, return_lse,
            block_idx=None, block_cnt=None, bi_strides=(0, 0), max_blocks=0, split_blocks=0,
            window=(-1, -1), include_last=False, kv_layout="batched", page_table=None, page_size=0,
            window_form=False):
    if q.dim() != 3 or k.dim() != 4:
        raise ValueError("decoding takes q [B, Hq, D] and k, v [B, maxL, Hkv, D] (or a packed / paged cache)")
    if v.shape != k.shape:
        raise ValueError("v %s must have the shape of k %s" % (tuple(v.shape), tuple(k.shape)))
    if k.shape[-1] != q.shape[-1]:
        raise ValueError("q, k and v must share head_dim")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k and v must share one dtype (got %s, %s, %s)" % (q.dtype, k.dtype, v.dtype))
    if k.shape[2] == 0 or q.shape[1] % k.shape[2] != 0:
        raise ValueError("heads_q %d must be a positive multiple of heads_kv %d" % (q.shape[1], k.shape[2]))
    for name, t, n in (("cu_seq_lens", cu_seq_lens, q.shape[0] + 1), ("seq_lens", seq_lens, q.shape[0])):
        if t is not None and (t.dim() != 1 or t.numel() != n or t.is_floating_point()):
            raise ValueError("%s must be an integer tensor of %d entries" % (name, n))
    if page_table is not None and page_table.is_floating_point():
        raise ValueError("page_table must be an integer tensor")
    _require_gpu(q, k, v, cu_seq_lens, seq_lens, page_table, block_idx, block_cnt)
    lib = _lib.load()
    D0 = q.shape[-1]
    if _padded_head_dim(D0) != D0:
        # zero-padded copies of the cache: correct, but a cache that is decoded from
        # repeatedly should be allocated with a head_dim the kernels are built for
        Dp = _padded_head_dim(D0)
        out = _decode(_pad_last(q, Dp), _pad_last(k, Dp), _pad_last(v, Dp), cu_seq_lens, seq_lens, scale, max_seq_len,
                      split_tokens, return_lse, block_idx, block_cnt, bi_strides, max_blocks, split_blocks, window,
                      include_last, kv_layout, page_table, page_size, window_form)
        if return_lse:
            return out[0][..., :D0].contiguous(), out[1]
        return out[..., :D0].contiguous()
    q, k, v = _inner_contig(q), _inner_contig(k), _inner_contig(v)
    B, Hq, D = q.shape
    Hkv = k.shape[2]
    o = torch.empty((B, Hq, D), device=q.device, dtype=q.dtype)
    lse = torch.empty((B, Hq), device=q.device, dtype=torch.float32) if return_lse else None
    if q.numel() == 0:
        return (o, lse) if return_lse else o
    if k.numel() == 0:  # an empty cache: every sequence has length 0
        o.zero_()
        if return_lse:
            lse.fill_(float("-inf"))
        return (o, lse) if return_lse else o
    a = _lib.DecodeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_tag(q)
    a.q, a.k, a.v, a.o, a.lse = _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse)
    a.q_stride_b, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_b, a.k_stride_s, a.k_stride_h = k.stride(0), k.stride(1), k.stride(2)
    a.v_stride_b, a.v_stride_s, a.v_stride_h = v.stride(0), v.stride(1), v.stride(2)
    a.o_stride_b, a.o_stride_h = o.stride(0), o.stride(1)
    if seq_lens is not None:
        seq_lens = seq_lens.to(torch.int32)
        a.seq_lens, a.cu_seqlens = _ptr(seq_lens), None
    else:
        cu_seq_lens = cu_seq_lens.to(torch.int32)
        a.seq_lens, a.cu_seqlens = None, _ptr(cu_seq_lens)
    a.batch, a.heads_q, a.heads_kv, a.head_dim = B, Hq, Hkv, D
    if kv_layout == "batched":
        if k.shape[0] != B:
            raise ValueError("k, v must be [B, maxL, Hkv, D] (pass kv_layout='packed' for a [1, T, Hkv, D] buffer)")
        a.kv_layout = _lib.MI_KV_BATCHED
        bound = k.shape[1]      # bounds every length, so no host sync is needed for the grid
    elif kv_layout == "packed":
        if k.shape[0] != 1 or cu_seq_lens is None:
            raise ValueError("packed KV is one [1, T, Hkv, D] buffer addressed through cu_seq_lens")
        a.kv_layout = _lib.MI_KV_PACKED
        bound = k.shape[1]
    elif kv_layout == "paged":
        # k, v: page pools [num_pages, page_size, Hkv, D]; page_table [B, max_pages] int32
        if page_table is None or page_table.dim() != 2 or page_table.shape[0] != B:
            raise ValueError("paged KV needs page_table [B, max_pages]")
        page_table = page_table.to(torch.int32)
        if page_table.stride(1) != 1:
            page_table = page_table.contiguous()
        page_size = int(page_size or k.shape[1])
        if page_size != k.shape[1] or page_size % 32 != 0:
            raise ValueError("page_size must equal k.shape[1] and be a multiple of 32")
        a.kv_layout, a.page_size = _lib.MI_KV_PAGED, page_size
        a.page_table, a.page_table_stride_b = _ptr(page_table), page_table.stride(0)
        bound = page_table.shape[1] * page_size
    else:
        raise ValueError("kv_layout must be 'batched', 'packed' or 'paged'")
    a.max_seqlen = int(bound if max_seq_len is None else min(max_seq_len, bound))
    a.scale_log2 = float(scale) * LOG2E
    gslices = (Hq // Hkv + 31) // 32   # wavefronts per (chunk, kv-head): 32 query heads each
    if block_idx is None and not window_form:
        a.split_tokens = int(split_tokens) if split_tokens else lib.mi_decode_choose_split_tokens(
            B, Hkv * gslices, a.max_seqlen, _num_cus(lib))
    else:
        a.split_tokens = 64
        a.window_form = 1 if window_form else 0
        a.block_idx, a.block_cnt = _ptr(block_idx), _ptr(block_cnt)
        a.block_idx_stride_b, a.block_idx_stride_h = bi_strides
        a.window_local, a.window_global = window
        a.include_last_block = 1 if (include_last and not window_form) else 0
        a.max_blocks, a.block_size = int(max_blocks), _masks.BLOCK
        a.split_blocks = int(split_blocks) if split_blocks else lib.mi_decode_choose_split_blocks(
            B, Hkv * gslices, a.max_blocks + a.include_last_block, _num_cus(lib))
    nbytes = lib.mi_decode_workspace_bytes(C.byref(a))
    if nbytes == 0:
        raise _lib.MiAttnError(lib.mi_decode_validate(C.byref(a)), lib.mi_last_error().decode())
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    a.workspace, a.workspace_bytes = _ptr(ws), nbytes
    _lib.check(lib.mi_decode(C.byref(a), _stream()))
    return (o, lse) if return_lse else o


def flash_attention_decoding(q, k, v, cu_seq_lens, qk_scale=None, *, seq_lens=None, max_seq_len=None,
                             split_tokens=None, return_lse=False, kv_layout="batched", page_table=None,
                             page_size=None):
    """Single-query decoding, split-KV + LSE merge.

    Contract of flash_attention_decoding in
    flash_attn_triton/flash_attn_decoding.py:213-336: q [B,Hq,D]; k, v
    [B,maxL,Hkv,D] (any strides, e.g. a transposed view of [B,Hkv,L,D]);
    cu_seq_lens [B+1] supplies only the lengths (:46-48); `qk_scale` natural
    base, default D^-0.5 (:236-237).  Returns o [B,Hq,D]; rows with length 0
    are zero.  Extensions: `seq_lens` [B] instead of cu_seq_lens, `max_seq_len`
    and `split_tokens` to size the launch, `return_lse` (base-2, [B,Hq]), and
    two more KV-cache layouts: kv_layout="packed" — k, v [1,T,Hkv,D] with
    sequence b in rows cu_seq_lens[b]:cu_seq_lens[b+1], what the reference's
    decode oracle consumes (:357-359); kv_layout="paged" — k, v are page pools
    [num_pages, page_size, Hkv, D] and page_table [B, max_pages] int32 maps a
    sequence's logical pages to pool pages (page_size a multiple of 32).
    """
    if (cu_seq_lens is None) == (seq_lens is None):
        raise ValueError("give exactly one of cu_seq_lens / seq_lens")
    scale = q.shape[-1] ** -0.5 if qk_scale is None else qk_scale
    return _decode(q, k, v, cu_seq_lens, seq_lens, scale, max_seq_len, split_tokens, return_lse,
                   kv_layout=kv_layout, page_table=page_table, page_size=page_size or 0)


def flash_attention_sparse_decoding(q, k, v, cu_seq_lens, global_window_size=64, local_window_size=64, *,
                                    seq_lens=None, block_indices=None, block_counts=None, block_size=64,
                                    include_last_block=True, split_blocks=None, return_lse=False,
                                    kv_layout="batched", page_table=None, page_size=None):
    """Sparse single-query decoding.

    Window form — contract of flash_attention_sparse_decoding in
    flash_attn_triton/flash_attn_decoding_sparse.py:222-365: attends the first
    `global_window_size` tokens and the last `local_window_size` tokens of each
    sequence (oracle :391-396); global_window_size must be 64, 128 or 256
    (:249-253); scale is D^-0.5 (:246).  The call is two kernel launches: the
    blocks a sequence attends are derived from its length inside the kernel.
    Block form — `block_indices` [B,Hkv,n] int32 (unique, ascending, each in
    [0, ceil(len/64))) lists the 64-token blocks each kv-head attends, shared
    by its query heads; `block_counts` [B,Hkv] optionally gives the number of
    valid entries; with `include_last_block` the block holding the newest
    token is added if absent.  Tokens >= len are masked.
    Both forms also read a paged cache (kv_layout="paged", page_table,
    page_size as in flash_attention_decoding).
    """
    if kv_layout not in ("batched", "paged"):
        raise ValueError("sparse decoding reads a 'batched' or a 'paged' cache")
    layout = dict(kv_layout=kv_layout, page_table=page_table, page_size=page_size or 0)
    if (cu_seq_lens is None) == (seq_lens is None):
        raise ValueError("give exactly one of cu_seq_lens / seq_lens")
    if block_size != _masks.BLOCK:
        raise ValueError("block_size must be %d" % _masks.BLOCK)
    B, Hq, D = q.shape
    Hkv = k.shape[2]
    scale = D ** -0.5
    if block_indices is None:
        gw, lw = int(global_window_size), int(local_window_size)
        assert gw in {64, 128, 256}, "global_window_size must be one of 64, 128, or 256, got %d" % gw
        if lw < 0:
            raise ValueError("local_window_size must be >= 0")
        # The blocks a sequence attends follow from (length, gw, lw) alone - the
        # first gw // 64 blocks, then the blocks from token len - lw to the last -
        # and the kernel derives them per sequence: no list is built here.
        cap = gw // _masks.BLOCK + (lw + _masks.BLOCK - 1) // _masks.BLOCK + 1
        return _decode(q, k, v, cu_seq_lens, seq_lens, scale, None, None, return_lse, max_blocks=cap,
                       split_blocks=split_blocks or 0, window=(lw, gw), window_form=True, **layout)
    lens = seq_lens if seq_lens is not None else (cu_seq_lens[1:] - cu_seq_lens[:-1])
    lens = lens.to(torch.int32)
    if block_indices.dim() != 3 or block_indices.shape[0] != B or block_indices.shape[1] != Hkv \
            or block_indices.is_floating_point():
        raise ValueError("block_indices must be an integer tensor [B, Hkv, n], got %s %s"
                         % (block_indices.dtype, tuple(block_indices.shape)))
    idx = block_indices.to(torch.int32).contiguous()
    n = idx.shape[2]
    cnt = None
    if block_counts is not None:
        if block_counts.shape != (B, Hkv) or block_counts.is_floating_point():
            raise ValueError("block_counts must be an integer tensor [B, Hkv]")
        cnt = block_counts.to(torch.int32).contiguous()
    if n == 0:
        if not include_last_block:
            raise ValueError("an empty block list needs include_last_block")
        # a non-NULL list address selects the block form even when only the implicit block is read
        idx = torch.zeros((B, Hkv, 1), device=q.device, dtype=torch.int32)
        return _decode(q, k, v, None, lens, scale, None, None, return_lse, block_idx=idx, block_cnt=None,
                       bi_strides=(Hkv, 1), max_blocks=0, split_blocks=split_blocks or 0, include_last=True, **layout)
    # the block of the newest token is appended (and de-duplicated) by the kernel
    return _decode(q, k, v, None, lens, scale, None, None, return_lse, block_idx=idx, block_cnt=cnt,
                   bi_strides=(Hkv * n, n), max_blocks=n, split_blocks=split_blocks or 0,
                   include_last=bool(include_last_block), **layout)
