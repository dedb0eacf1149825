"""Host-side mirror of the reference's attention ops over the C ABI.

Names, argument meaning and error behaviour follow paperkiln's
``ops::fused_attention`` / ``ops::swa_attention`` (src/ops.cpp:863-1027,
declared include/microtorch/ops.hpp:141-150). torch tensors are used only as
handles on device memory and for the current HIP stream; all arithmetic runs
in libpaperkiln_amd.so.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import AttnShape, Tensor4

_DT = {torch.float32: _lib.PK_F32, torch.bfloat16: _lib.PK_BF16}


def _t4(x: torch.Tensor) -> Tensor4:
    if x.dim() != 4 or x.stride(3) != 1:
        raise RuntimeError("expected a [B,T,H,dk] tensor with contiguous head_dim")
    return Tensor4(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2))


def _shape(q, k, scale, causal, window, sinks, grad_dtype=None) -> AttnShape:
    B, T, Hq, dk = q.shape
    if q.dtype not in _DT:
        raise RuntimeError("dtype must be float32 or bfloat16")
    gd = _DT[grad_dtype] if grad_dtype is not None else _DT[q.dtype]
    return AttnShape(B, T, Hq, k.shape[2], dk, int(bool(causal)), int(window), int(sinks), float(scale),
                     _DT[q.dtype], gd)


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def attn_fwd(q, k, v, scale, causal=True, window=0, sinks=0):
    """q: [B,T,Hq,dk]; k, v: [B,T,Hkv,dk] (any batch/token/head strides).
    Returns (o [B,T,Hq,dk], lse [B,Hq,T] fp32). Only O and LSE are written."""
    if not q.is_cuda:
        raise RuntimeError("paperkiln_amd has no CPU path: tensors must live on the GPU")
    if k.shape != v.shape or k.shape[0] != q.shape[0] or k.shape[1] != q.shape[1] or k.shape[3] != q.shape[3]:
        raise RuntimeError("fused_attention: shape mismatch")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("fused_attention: dtype mismatch")
    B, T, Hq, dk = q.shape
    o = torch.empty((B, T, Hq, dk), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, Hq, T), dtype=torch.float32, device=q.device)
    sh = _shape(q, k, scale, causal, window, sinks)
    _lib.check(_lib.lib().pk_attn_fwd(C.byref(sh), C.byref(_t4(q)), C.byref(_t4(k)), C.byref(_t4(v)),
                                       C.byref(_t4(o)), C.c_void_p(lse.data_ptr()), _stream()))
    return o, lse


BWD_DELTA, BWD_DKDV, BWD_DQ, BWD_ALL = 1, 2, 4, 7


def bwd_workspace_bytes(q, k, grad_dtype=None, window=0, sinks=0):
    """Bytes of scratch pk_attn_bwd needs for these shapes and this mask (pk_attn_bwd_workspace_bytes):
    a band mask with sink keys needs more than the plain causal mask."""
    sh = _shape(q, k, 1.0, True, window, sinks, grad_dtype or q.dtype)
    return max(int(_lib.lib().pk_attn_bwd_workspace_bytes(C.byref(sh))), 16)


def attn_bwd(q, k, v, o, lse, d_o, scale, causal=True, window=0, sinks=0, grad_dtype=None, out=None,
             stages=BWD_ALL):
    """Recompute backward from (Q, K, V, O, LSE, dO). Returns (dq, dk, dv);
    dk/dv are summed over each GQA group. ``out`` may supply preallocated
    (dq, dk, dv, workspace) to keep a timed loop free of allocations."""
    grad_dtype = grad_dtype or q.dtype
    sh = _shape(q, k, scale, causal, window, sinks, grad_dtype)
    L = _lib.lib()
    nbytes = L.pk_attn_bwd_workspace_bytes(C.byref(sh))
    if out is None:
        dq = torch.empty(q.shape, dtype=grad_dtype, device=q.device)
        dk = torch.empty(k.shape, dtype=grad_dtype, device=q.device)
        dv = torch.empty(v.shape, dtype=grad_dtype, device=q.device)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
    else:
        dq, dk, dv, ws = out
    _lib.check(L.pk_attn_bwd_stages(C.byref(sh), C.byref(_t4(q)), C.byref(_t4(k)), C.byref(_t4(v)),
                                    C.byref(_t4(o)), C.c_void_p(lse.data_ptr()), C.byref(_t4(d_o)),
                                    C.byref(_t4(dq)), C.byref(_t4(dk)), C.byref(_t4(dv)),
                                    C.c_void_p(ws.data_ptr()), ws.numel(), stages, _stream()))
    return dq, dk, dv


def attn_bwd_static(q, k, v, o, lse, d_o, scale, causal=True, window=0, sinks=0, out=None):
    """pk_attn_bwd_static: the same backward with the library's own static scratch instead of a workspace. The
    call itself allocates nothing; ``out`` supplies (dq, dk, dv), which are allocated here only when it is None."""
    if out is None:
        out = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))
    dq, dk, dv = out
    sh = _shape(q, k, scale, causal, window, sinks, dq.dtype)
    _lib.check(_lib.lib().pk_attn_bwd_static(C.byref(sh), C.byref(_t4(q)), C.byref(_t4(k)), C.byref(_t4(v)),
                                              C.byref(_t4(o)), C.c_void_p(lse.data_ptr()), C.byref(_t4(d_o)),
                                              C.byref(_t4(dq)), C.byref(_t4(dk)), C.byref(_t4(dv)), _stream()))
    return dq, dk, dv


class _AttnFn(torch.autograd.Function):
    """Tape node that keeps O and LSE only (plus its parents Q, K, V), in place
    of the reference closure's captured [T,T] matrix A (src/ops.cpp:902)."""

    @staticmethod
    def forward(ctx, q, k, v, scale, causal, window, sinks):
        o, lse = attn_fwd(q, k, v, scale, causal, window, sinks)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.cfg = (scale, causal, window, sinks)
        return o

    @staticmethod
    def backward(ctx, d_o):
        q, k, v, o, lse = ctx.saved_tensors
        scale, causal, window, sinks = ctx.cfg
        if d_o.stride(3) != 1:
            d_o = d_o.contiguous()
        dq, dk, dv = attn_bwd(q, k, v, o, lse, d_o, scale, causal, window, sinks)
        return dq, dk, dv, None, None, None, None


def _as_heads(x: torch.Tensor, seq_len: int, who: str):
    """The reference op takes one head as a [rows, dk] matrix whose rows are
    B stacked sequences of seq_len (src/ops.cpp:869-879): view it as [B,T,1,dk]."""
    rows = x.shape[0]
    sl = rows if seq_len == 0 else seq_len
    if rows % sl != 0:
        raise RuntimeError(f"{who}: rows not a multiple of seq_len")
    return x.view(rows // sl, sl, 1, x.shape[1])


def fused_attention(q, k, v, scale, seq_len=0, causal=True):
    """ops::fused_attention(q, k, v, scale, seq_len, causal) for one head:
    q, k, v are [rows, dk]; returns y [rows, dk]. Differentiable."""
    if k.shape[0] != q.shape[0] or v.shape[0] != q.shape[0] or q.shape[1] != k.shape[1] or v.shape[1] != k.shape[1]:
        raise RuntimeError("fused_attention: shape mismatch")
    y = _AttnFn.apply(_as_heads(q, seq_len, "fused_attention"), _as_heads(k, seq_len, "fused_attention"),
                      _as_heads(v, seq_len, "fused_attention"), scale, causal, 0, 0)
    return y.view(q.shape[0], q.shape[1])


def swa_attention(q, k, v, scale, window, sinks, seq_len=0):
    """ops::swa_attention(q, k, v, scale, window, sinks, seq_len) for one head."""
    if k.shape[0] != q.shape[0] or v.shape[0] != q.shape[0] or q.shape[1] != k.shape[1] or v.shape[1] != k.shape[1]:
        raise RuntimeError("swa_attention: shape mismatch")
    if window == 0:
        raise RuntimeError("swa_attention: window must be >= 1")
    y = _AttnFn.apply(_as_heads(q, seq_len, "swa_attention"), _as_heads(k, seq_len, "swa_attention"),
                      _as_heads(v, seq_len, "swa_attention"), scale, True, window, sinks)
    return y.view(q.shape[0], q.shape[1])


def attention(q, k, v, scale, causal=True, window=0, sinks=0):
    """All heads at once on [B,T,H,dk] tensors (GQA when k/v have fewer heads). Differentiable."""
    return _AttnFn.apply(q, k, v, scale, causal, window, sinks)


class _CheckpointFn(torch.autograd.Function):
    """checkpoint(fn, x) of the reference (src/autograd.cpp:68-102): the forward runs fn with the
    tape off and keeps only its input and output; the backward re-runs fn on a detached copy of the
    input with the tape on, seeds the recomputed output with the incoming gradient and runs the inner
    tape, so parameters used inside fn receive their gradients in place and x receives the inner
    input's gradient."""

    @staticmethod
    def forward(ctx, fn, x):
        ctx.fn = fn
        ctx.save_for_backward(x)
        with torch.no_grad():
            return fn(x)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        x2 = x.detach().requires_grad_(True)
        with torch.enable_grad():
            y2 = ctx.fn(x2)
        if y2.shape != dy.shape:
            raise RuntimeError("checkpoint: recomputed output shape mismatch")
        torch.autograd.backward(y2, dy)
        return None, x2.grad


def checkpoint(fn, x):
    """y = fn(x) without keeping fn's intermediate activations; they are rebuilt in the backward.
    As in the reference, the node is only recorded when x requires a gradient (the closure hangs
    off x, src/autograd.cpp:80-83); with the tape off it is a plain call."""
    if not torch.is_grad_enabled() or not x.requires_grad:
        return fn(x)
    return _CheckpointFn.apply(fn, x)
