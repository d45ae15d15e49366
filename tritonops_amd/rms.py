"""RMSNorm with the class names of the reference's common/rms.py, on the HIP
kernels of libmi_attn.so (no Triton, no fallback)."""
import ctypes as C

import torch
from torch import nn
from torch.autograd import Function

from . import _lib
from .ops import _ptr, _require_gpu, _stream

_TAGS = {torch.bfloat16: _lib.MI_DTYPE_BF16, torch.float16: _lib.MI_DTYPE_F16, torch.float32: _lib.MI_DTYPE_F32}


def _tag(t):
    try:
        return _TAGS[t.dtype]
    except KeyError:
        raise TypeError("RMSNorm supports bfloat16, float16 and float32 tensors, got %s" % t.dtype)


def _rows(x):
    """[..., D] -> 2-D tensor whose rows are contiguous (a view when possible)."""
    x2 = x.reshape(-1, x.shape[-1])
    return x2 if x2.stride(-1) == 1 else x2.contiguous()


def _args(x2, weight, eps):
    a = _lib.RmsNormArgs()
    a.struct_size = C.sizeof(a)
    a.x_dtype, a.w_dtype = _tag(x2), _tag(weight)
    a.rows, a.dim = x2.shape
    a.x, a.w = _ptr(x2), _ptr(weight)
    a.x_stride = x2.stride(0) if x2.shape[0] > 1 else x2.shape[1]
    a.eps = float(eps)
    return a


def rmsnorm_fwd(x, weight, eps):
    """y = x / sqrt(mean(x^2) + eps) * weight over the last dimension; returns
    (y, rsqrt) with rsqrt fp32 [rows] — forward of RMSNormTritonFunction
    (common/rms.py:223-287)."""
    _require_gpu(x, weight)
    lib = _lib.load()
    if x.shape[-1] != weight.shape[0]:
        raise ValueError("Expected weight dim %d, got %d" % (x.shape[-1], weight.shape[0]))
    if weight.dtype != x.dtype and weight.dtype != torch.float32:
        weight = weight.to(x.dtype)
    weight = weight.contiguous()
    x2 = _rows(x)
    y = torch.empty((x2.shape[0], x2.shape[1]), device=x.device, dtype=x.dtype)
    rsqrt = torch.empty((x2.shape[0],), device=x.device, dtype=torch.float32)
    a = _args(x2, weight, eps)
    a.y, a.rsqrt, a.y_stride = _ptr(y), _ptr(rsqrt), y.shape[1]
    _lib.check(lib.mi_rmsnorm_fwd(C.byref(a), _stream()))
    return y.view(x.shape), rsqrt


def rmsnorm_bwd(dy, x, weight, rsqrt, eps):
    """(dx, dweight) — backward of RMSNormTritonFunction (common/rms.py:289-355);
    dweight is reduced deterministically (the reference uses atomics, :215)."""
    _require_gpu(dy, x, weight, rsqrt)
    lib = _lib.load()
    wk = weight if (weight.dtype == x.dtype or weight.dtype == torch.float32) else weight.to(x.dtype)
    wk = wk.contiguous()
    x2, dy2 = _rows(x), _rows(dy.to(x.dtype))
    dx = torch.empty((x2.shape[0], x2.shape[1]), device=x.device, dtype=x.dtype)
    dw = torch.zeros_like(wk)
    a = _args(x2, wk, eps)
    a.rsqrt = _ptr(rsqrt)
    a.dy, a.dx, a.dw = _ptr(dy2), _ptr(dx), _ptr(dw)
    a.dy_stride = dy2.stride(0) if dy2.shape[0] > 1 else dy2.shape[1]
    a.dx_stride = dx.shape[1]
    nbytes = lib.mi_rmsnorm_bwd_workspace_bytes(C.byref(a))
    ws = torch.empty(max(nbytes, 16), device=x.device, dtype=torch.uint8)
    a.workspace, a.workspace_bytes = _ptr(ws), nbytes
    _lib.check(lib.mi_rmsnorm_bwd(C.byref(a), _stream()))
    return dx.view(x.shape), dw.to(weight.dtype)


class RMSNormTritonFunction(Function):
    """`RMSNormTritonFunction.apply(x, weight, eps)` — common/rms.py:221-355."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        y, rsqrt = rmsnorm_fwd(x, weight, eps)
        ctx.eps = eps
        ctx.save_for_backward(x, weight, rsqrt)
        return y

    @staticmethod
    def backward(ctx, grad_output):
        x, weight, rsqrt = ctx.saved_tensors
        dx, dw = rmsnorm_bwd(grad_output, x, weight, rsqrt, ctx.eps)
        return dx, dw, None


class RMSNormTriton(nn.Module):
    """Drop-in for RMSNormTriton of common/rms.py:358-383: weight initialised to
    ones, eps default 1e-6."""

    def __init__(self, dim, eps=1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        return RMSNormTritonFunction.apply(x, self.weight, self.eps)
