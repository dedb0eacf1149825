"""The operators of one Llama block on GPU tensors, through the C ABI
(`pk_op_*` in include/paperkiln_amd.h). Names, argument order and error
behaviour follow paperkiln's `microtorch::ops` (src/ops.cpp); tensors are
torch CUDA tensors, fp32 or bf16, contiguous. There is no CPU path.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import PK_BF16, PK_F32, check


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return PK_F32
    if t.dtype == torch.bfloat16:
        return PK_BF16
    raise TypeError(f"unsupported dtype {t.dtype}")


def _chk(*ts):
    for t in ts:
        if not t.is_cuda or not t.is_contiguous():
            raise ValueError("block ops take contiguous CUDA tensors")
    if any(t.dtype != ts[0].dtype or t.shape != ts[0].shape for t in ts):
        raise RuntimeError("shape mismatch")


def _s():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(t.data_ptr())


def add(a, b):
    _chk(a, b)
    y = torch.empty_like(a)
    check(_lib.lib().pk_op_add(_p(a), _p(b), _p(y), a.numel(), _dt(a), _s()))
    return y


def mul(a, b):
    _chk(a, b)
    y = torch.empty_like(a)
    check(_lib.lib().pk_op_mul(_p(a), _p(b), _p(y), a.numel(), _dt(a), _s()))
    return y


def scale(a, s):
    _chk(a)
    y = torch.empty_like(a)
    check(_lib.lib().pk_op_scale(_p(a), float(s), _p(y), a.numel(), _dt(a), _s()))
    return y


def axpy_(y, a, x):
    """y += a * x in place."""
    _chk(y, x)
    check(_lib.lib().pk_op_axpy(_p(y), float(a), _p(x), y.numel(), _dt(y), _s()))
    return y


def fill_(y, v):
    _chk(y)
    check(_lib.lib().pk_op_fill(_p(y), float(v), y.numel(), _dt(y), _s()))
    return y


def silu(x, dy=None):
    """ops::silu; with dy also the closure's dx."""
    _chk(x)
    y = torch.empty_like(x)
    check(_lib.lib().pk_op_silu_fwd(_p(x), _p(y), x.numel(), _dt(x), _s()))
    if dy is None:
        return y
    _chk(x, dy)
    dx = torch.empty_like(x)
    check(_lib.lib().pk_op_silu_bwd(_p(x), _p(dy), _p(dx), x.numel(), _dt(x), _s()))
    return y, dx


def silu_mul(gate, up, dy=None):
    """mul(silu(gate), up) in one pass; with dy also (dgate, dup)."""
    _chk(gate, up)
    y = torch.empty_like(gate)
    L = _lib.lib()
    check(L.pk_op_silu_mul_fwd(_p(gate), _p(up), _p(y), gate.numel(), _dt(gate), _s()))
    if dy is None:
        return y
    _chk(gate, dy)
    dg, du = torch.empty_like(gate), torch.empty_like(gate)
    check(L.pk_op_silu_mul_bwd(_p(gate), _p(up), _p(dy), _p(dg), _p(du), gate.numel(), _dt(gate), _s()))
    return y, dg, du


def rmsnorm(x, w, dy=None, eps=1e-5):
    """ops::rmsnorm: y (and, with dy, dx and dw). w is fp32 [cols]."""
    _chk(x)
    if x.dim() != 2 or w.numel() != x.shape[1] or w.dtype != torch.float32:
        raise RuntimeError("rmsnorm: w must be [1, cols(x)]")
    R, Cc = x.shape
    y = torch.empty_like(x)
    ri = torch.empty(R, dtype=torch.float32, device=x.device)
    L = _lib.lib()
    check(L.pk_op_rmsnorm_fwd(_p(x), _p(w), float(eps), _p(y), _p(ri), R, Cc, _dt(x), _s()))
    if dy is None:
        return y
    _chk(x, dy)
    dx = torch.empty_like(x)
    dw = torch.empty(Cc, dtype=torch.float32, device=x.device)
    check(L.pk_op_rmsnorm_bwd(_p(dy), _p(x), _p(ri), _p(w), _p(dw), _p(dx), R, Cc, _dt(x), _s()))
    return y, dx, dw


def apply_rope(qkv, pos, theta, head_dim, inverse=False, all_heads=False):
    """ops::apply_rope on a fused [T, 3d] matrix; pos: int32 CUDA tensor [T]."""
    _chk(qkv)
    if qkv.dim() != 2 or qkv.shape[1] % 3 != 0:
        raise RuntimeError("apply_rope: cols must be divisible by 3")
    d = qkv.shape[1] // 3
    if pos.dtype != torch.int32 or pos.numel() != qkv.shape[0] or not pos.is_cuda:
        raise RuntimeError("apply_rope: one int32 position per row")
    y = torch.empty_like(qkv)
    check(_lib.lib().pk_op_rope(_p(qkv), _p(pos), float(theta), qkv.shape[0], d, int(head_dim), int(all_heads),
                                int(inverse), _p(y), _dt(qkv), _s()))
    return y


def embedding(table, ids, dy=None, dtype=torch.float32):
    """ops::embedding: rows of an fp32 table; with dy also the scatter-added table gradient."""
    if table.dtype != torch.float32 or ids.dtype != torch.int32:
        raise TypeError("embedding: fp32 table, int32 ids")
    V, d = table.shape
    if ids.numel() and (int(ids.min()) < 0 or int(ids.max()) >= V):
        raise RuntimeError("embedding: id out of range")
    n = ids.numel()
    y = torch.empty((n, d), dtype=dtype, device=table.device)
    L = _lib.lib()
    check(L.pk_op_embedding_fwd(_p(table), _p(ids), _p(y), n, V, d, _dt(y), _s()))
    if dy is None:
        return y
    dt = torch.zeros_like(table)
    check(L.pk_op_embedding_bwd(_p(dy), _p(ids), _p(dt), n, V, d, _dt(dy), _s()))
    return y, dt


def cross_entropy(logits, targets):
    """ops::cross_entropy: (mean NLL, dlogits for upstream gradient 1). logits are not modified."""
    _chk(logits)
    R, V = logits.shape
    if targets.numel() != R:
        raise RuntimeError("cross_entropy: one target per row")
    if int(targets.min()) < 0 or int(targets.max()) >= V:
        raise RuntimeError("cross_entropy: target out of range")
    dl = logits.clone()
    nll = torch.empty(R, dtype=torch.float32, device=logits.device)
    loss = C.c_float()
    check(_lib.lib().pk_op_cross_entropy(_p(dl), _p(targets), R, V, 1.0, _p(nll), C.byref(loss), _dt(dl), _s()))
    return loss.value, dl


def adamw_(p, g, m, v, lr, b1=0.9, b2=0.999, eps=1e-8, wd=0.01, t=1):
    """nn::AdamW::step on one fp32 parameter, in place."""
    _chk(p, g, m, v)
    check(_lib.lib().pk_op_adamw(_p(p), _p(g), _p(m), _p(v), p.numel(), lr, b1, b2, eps, wd, int(t), _s()))
    return p


def clip_grad_norm_(grads, max_norm):
    """ops::clip_grad_norm: scales the fp32 gradients in place when their global norm exceeds max_norm."""
    sq = 0.0
    L = _lib.lib()
    for g in grads:
        _chk(g)
        out = C.c_double()
        check(L.pk_op_sumsq(_p(g), g.numel(), C.byref(out), _s()))
        sq += out.value
    total = float(torch.tensor(sq, dtype=torch.float64).sqrt().to(torch.float32))
    if total > max_norm and total > 0.0:
        s = float(torch.tensor(max_norm, dtype=torch.float32) / torch.tensor(total, dtype=torch.float32))
        for g in grads:
            check(L.pk_op_scale(_p(g), s, _p(g), g.numel(), _dt(g), _s()))
    return total


def set_head_kernel(in_product: bool) -> int:
    """How the chunked tied head forms loss and dlogits from bf16 operands (pk_set_head_kernel): True (default) =
    inside the logits product, the logits never stored; False = an fp32 logits matrix and a row kernel over it.
    Returns the previous setting."""
    return int(_lib.lib().pk_set_head_kernel(1 if in_product else 0))


def set_gemm_backend(mode: int) -> int:
    """Choose the kernel for bf16 GEMMs (pk_set_gemm_backend): 1 (default) = the library's own matrix-core kernel
    wherever it applies, in the form it picks per shape, with a backward pass's weight-gradient products multiplied
    several at a time as one grouped launch; 2 = the same with every product on its own; 0 = rocBLAS only; 3 .. 11 =
    the own kernel with one form forced (measurements; see include/paperkiln_amd.h). Returns the previous setting
    (0, 1, 2)."""
    return int(_lib.lib().pk_set_gemm_backend(int(mode)))


def matmul(a, b, trans_a=False, trans_b=False, out_dtype=None, out=None):
    """device::gemm: op(a) @ op(b), fp32 accumulate. With ``out`` the product is ADDED to it (beta = 1)."""
    _chk(a)
    _chk(b)
    if a.dtype != b.dtype:
        raise RuntimeError("gemm: operand dtypes differ")
    m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    k2, n = (b.shape[1], b.shape[0]) if trans_b else b.shape
    if k != k2:
        raise RuntimeError("gemm: inner dimensions disagree")
    c = out if out is not None else torch.empty((m, n), dtype=out_dtype or a.dtype, device=a.device)
    if out is not None and (tuple(out.shape) != (m, n) or not out.is_contiguous()):
        raise RuntimeError("gemm: output shape mismatch")
    check(_lib.lib().pk_op_gemm(_p(a), int(trans_a), _p(b), int(trans_b), _p(c), m, n, k, _dt(a), _dt(c),
                                int(out is not None), _s()))
    return c
