"""Fused linear + cross-entropy with the names of the reference's
cross_entropy_triton/cross_entropy.py, on the HIP kernels of libmi_attn.so
(no Triton, no fallback).  The forward never materialises the logits; the
backward follows the reference's scheme in blocks of rows, with the logits GEMM
and the element-wise kernel fused into one launch (the dlogits come straight
from fp32 accumulators) and the two plain gradient GEMMs left to the BLAS
library behind torch.mm."""
import ctypes as C

import torch

from . import _lib
from .ops import _ptr, _require_gpu, _stream

_TAGS = {torch.bfloat16: _lib.MI_DTYPE_BF16, torch.float16: _lib.MI_DTYPE_F16}
# Rows of logits that the backward materialises at a time (the reference uses
# 2048, cross_entropy.py:367; a 288 GB device holds far larger blocks).
BWD_ROWS = 16384


def _tag(t):
    try:
        return _TAGS[t.dtype]
    except KeyError:
        raise TypeError("fused cross-entropy supports bfloat16 and float16 tensors, got %s" % t.dtype)


def _pad_dim(t, mult=128):
    """Rows as the kernel wants them: unit inner stride, 16-byte aligned, row
    stride a multiple of 8 and the inner size a multiple of 128 (zero columns
    do not change x @ w^T)."""
    d = t.shape[1]
    if d % mult:
        t = torch.nn.functional.pad(t, (0, mult - d % mult))
    if t.stride(1) != 1 or t.stride(0) % 8 or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def _labels(y, n):
    y = y.reshape(-1)
    if y.shape[0] != n:
        raise ValueError("Dimension mismatch: x.shape[0] (%d) != y.shape[0] (%d)" % (n, y.shape[0]))
    if y.dtype not in (torch.int32, torch.int64):
        y = y.to(torch.int64)
    return y.contiguous()


def cross_entropy_fused_fwd(x, w, y):
    """(loss, lse), both fp32 [T]: lse[t] = logsumexp_n(x[t] . w[n]),
    loss[t] = lse[t] - x[t] . w[y[t]] — forward of CrossEntropyFusedFunction
    (cross_entropy.py:276-352)."""
    _require_gpu(x, w, y)
    lib = _lib.load()
    if x.ndim != 2 or w.ndim != 2:
        raise ValueError("x and w must be 2D tensors.")
    if x.shape[1] != w.shape[1]:
        raise ValueError("x has %d columns, w has %d" % (x.shape[1], w.shape[1]))
    if w.dtype != x.dtype:
        raise TypeError("x and w must share one dtype")
    T, N = x.shape[0], w.shape[0]
    y = _labels(y, T)
    xp, wp = _pad_dim(x), _pad_dim(w)
    lse = torch.empty((T,), device=x.device, dtype=torch.float32)
    loss = torch.empty((T,), device=x.device, dtype=torch.float32)
    a = _lib.XentArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _tag(x)
    a.tokens, a.dim, a.vocab = T, xp.shape[1], N
    a.labels_i64 = 1 if y.dtype == torch.int64 else 0
    a.x, a.w, a.y = _ptr(xp), _ptr(wp), _ptr(y)
    a.x_stride = xp.stride(0) if T > 1 else xp.shape[1]
    a.w_stride = wp.stride(0) if N > 1 else wp.shape[1]
    a.lse, a.loss = _ptr(lse), _ptr(loss)
    nbytes = lib.mi_xent_fwd_workspace_bytes(C.byref(a))
    ws = torch.empty(max(nbytes, 16), device=x.device, dtype=torch.uint8)
    a.workspace, a.workspace_bytes = _ptr(ws), nbytes
    _lib.check(lib.mi_xent_fwd(C.byref(a), _stream()))
    return loss, lse


def cross_entropy_dlogits_(logits, lse, dloss, y):
    """In place: logits[t, n] <- dloss[t] (exp(logits[t, n] - lse[t]) - [n == y[t]])
    (cross_entropy_fused_bwd_kernel, cross_entropy.py:185-266)."""
    _require_gpu(logits, lse, dloss, y)
    lib = _lib.load()
    if logits.ndim != 2 or logits.stride(1) != 1:
        raise ValueError("logits must be 2-D with unit inner stride")
    a = _lib.XentGradArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _tag(logits)
    a.rows, a.vocab = logits.shape
    a.ld = logits.stride(0) if logits.shape[0] > 1 else logits.shape[1]
    a.labels_i64 = 1 if y.dtype == torch.int64 else 0
    a.logits, a.lse, a.dloss, a.y = _ptr(logits), _ptr(lse), _ptr(dloss), _ptr(y)
    _lib.check(lib.mi_xent_dlogits(C.byref(a), _stream()))
    return logits


def cross_entropy_dlogits(x, w, y, lse, dloss):
    """dlogits [T, N] in x's dtype: dloss[t] (exp(x[t] . w[n] - lse[t]) - [n == y[t]]),
    computed by the forward's GEMM kernel with the gradient epilogue on its fp32
    accumulators (replaces the logits GEMM + element-wise kernel of
    cross_entropy.py:374, :185-266, which round the logits to x's dtype first)."""
    _require_gpu(x, w, y, lse, dloss)
    lib = _lib.load()
    T, N = x.shape[0], w.shape[0]
    xp, wp = _pad_dim(x), _pad_dim(w)
    dl = torch.empty((T, N), device=x.device, dtype=x.dtype)
    a = _lib.XentBwdArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _tag(x)
    a.tokens, a.dim, a.vocab = T, xp.shape[1], N
    a.labels_i64 = 1 if y.dtype == torch.int64 else 0
    a.x, a.w, a.y = _ptr(xp), _ptr(wp), _ptr(y)
    a.x_stride = xp.stride(0) if T > 1 else xp.shape[1]
    a.w_stride = wp.stride(0) if N > 1 else wp.shape[1]
    a.lse, a.dloss = _ptr(lse), _ptr(dloss)
    a.dlogits, a.ld = _ptr(dl), N
    _lib.check(lib.mi_xent_bwd_dlogits(C.byref(a), _stream()))
    return dl


def cross_entropy_fused_bwd(grad_o, x, w, y, lse, rows_per_block=None):
    """(grad_x, grad_w) in the dtypes of x and w — backward of
    CrossEntropyFusedFunction (cross_entropy.py:355-420): per block of rows,
    dlogits from the fused GEMM kernel, then the two gradient GEMMs."""
    _require_gpu(grad_o, x, w, y, lse)
    T = x.shape[0]
    y = _labels(y, T)
    g = grad_o.reshape(-1).to(torch.float32).contiguous()
    lse = lse.contiguous()
    step = rows_per_block or BWD_ROWS
    grad_x = torch.empty_like(x)
    grad_w = None
    for s in range(0, T, step):
        e = min(s + step, T)
        xc = x[s:e]
        dl = cross_entropy_dlogits(xc, w, y[s:e], lse[s:e], g[s:e])
        torch.mm(dl, w, out=grad_x[s:e])
        if grad_w is None:
            grad_w = torch.mm(dl.t(), xc)
        else:
            grad_w.addmm_(dl.t(), xc)
    if grad_w is None:
        grad_w = torch.zeros_like(w)
    return grad_x, grad_w


class CrossEntropyFusedFunction(torch.autograd.Function):
    """Drop-in for the reference's autograd Function (cross_entropy.py:270-420)."""

    @staticmethod
    def forward(ctx, x, w, y):
        if y.ndim != 1 and y.shape[-1] != 1:
            raise ValueError("y must be a 1D tensor.")
        loss, lse = cross_entropy_fused_fwd(x, w, y)
        ctx.save_for_backward(x, w, y, lse)
        return loss

    @staticmethod
    def backward(ctx, grad_o):
        x, w, y, lse = ctx.saved_tensors
        grad_x, grad_w = cross_entropy_fused_bwd(grad_o, x, w, y, lse)
        return grad_x, grad_w, None


def cross_entropy_fused_triton(x, w, y):
    """loss [T] fp32 of softmax cross-entropy over x @ w^T (cross_entropy.py:423-425)."""
    return CrossEntropyFusedFunction.apply(x, w, y)
