"""ctypes binding of libpaperkiln_amd.so (the C ABI in include/paperkiln_amd.h).

The library is built in-tree by ``__graft_entry__.build()`` (or ``make -C
paperkiln_amd/csrc``). There is no fallback: if the shared object is missing
or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpaperkiln_amd.so")

PK_F32, PK_BF16 = 0, 1


class Tensor4(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_t", C.c_int64), ("stride_h", C.c_int64)]


class AttnShape(C.Structure):
    _fields_ = [("B", C.c_int32), ("T", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("dk", C.c_int32),
                ("causal", C.c_int32), ("window", C.c_int32), ("sinks", C.c_int32), ("scale", C.c_float),
                ("dtype", C.c_int32), ("grad_dtype", C.c_int32)]


class LlamaConfig(C.Structure):
    _fields_ = [("vocab", C.c_int32), ("d", C.c_int32), ("n_layers", C.c_int32), ("n_heads", C.c_int32),
                ("d_ff", C.c_int32), ("rope_theta", C.c_float), ("tie_embeddings", C.c_int32),
                ("compute_dtype", C.c_int32), ("rope_all_heads", C.c_int32), ("window", C.c_int32),
                ("sinks", C.c_int32)]


class LlamaStats(C.Structure):
    _fields_ = [("live_vars_after_forward", C.c_int64), ("activation_bytes_after_forward", C.c_int64),
                ("peak_activation_bytes", C.c_int64)]


class PkError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"paperkiln_amd error {code}: {msg}")
        self.code = code


_lib = None

# every symbol include/paperkiln_amd.h declares
EXPORTS = ["pk_last_error", "pk_init", "pk_attn_fwd", "pk_attn_bwd_workspace_bytes", "pk_attn_bwd", "pk_attn_bwd_stages", "pk_attn_bwd_static",
           "pk_alloc", "pk_free", "pk_memcpy_h2d", "pk_memcpy_d2h", "pk_live_bytes", "pk_peak_bytes", "pk_reset_peak", "pk_trim",
           "pk_llama_create", "pk_llama_destroy", "pk_llama_num_params", "pk_llama_param_info", "pk_llama_set_param",
           "pk_llama_get_param", "pk_llama_get_grad", "pk_llama_loss_backward", "pk_llama_adamw_step",
           "pk_llama_set_head_chunk",
           "pk_op_add", "pk_op_mul", "pk_op_scale", "pk_op_axpy", "pk_op_fill", "pk_op_silu_fwd", "pk_op_silu_bwd", "pk_op_silu_mul_fwd", "pk_op_silu_mul_bwd",
           "pk_op_rmsnorm_fwd", "pk_op_rmsnorm_bwd", "pk_op_rope", "pk_op_embedding_fwd", "pk_op_embedding_bwd",
           "pk_op_cross_entropy", "pk_op_adamw", "pk_op_sumsq", "pk_op_gemm", "pk_set_gemm_backend", "pk_set_head_kernel"]


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`; "
                "paperkiln_amd has no CPU or PyTorch fallback")
        L = C.CDLL(LIB_PATH)
        T4, SH = C.POINTER(Tensor4), C.POINTER(AttnShape)
        L.pk_last_error.restype = C.c_char_p
        L.pk_init.argtypes = [C.c_int, C.c_char_p, C.c_size_t]
        L.pk_attn_fwd.argtypes = [SH, T4, T4, T4, T4, C.c_void_p, C.c_void_p]
        L.pk_attn_bwd_workspace_bytes.argtypes = [SH]
        L.pk_attn_bwd_workspace_bytes.restype = C.c_size_t
        L.pk_attn_bwd.argtypes = [SH, T4, T4, T4, T4, C.c_void_p, T4, T4, T4, T4, C.c_void_p, C.c_size_t, C.c_void_p]
        L.pk_attn_bwd_stages.argtypes = [SH, T4, T4, T4, T4, C.c_void_p, T4, T4, T4, T4, C.c_void_p, C.c_size_t,
                                         C.c_int, C.c_void_p]
        L.pk_attn_bwd_static.argtypes = [SH, T4, T4, T4, T4, C.c_void_p, T4, T4, T4, T4, C.c_void_p]
        f32p, i32p = C.POINTER(C.c_float), C.POINTER(C.c_int)
        L.pk_alloc.argtypes = [C.c_size_t, C.POINTER(C.c_void_p)]
        L.pk_free.argtypes = [C.c_void_p]
        L.pk_memcpy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.pk_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        for fn in (L.pk_live_bytes, L.pk_peak_bytes):
            fn.restype = C.c_size_t
        L.pk_reset_peak.restype = None
        L.pk_trim.restype = None
        L.pk_llama_create.argtypes = [C.POINTER(LlamaConfig), C.c_uint, C.POINTER(C.c_void_p)]
        L.pk_llama_destroy.argtypes = [C.c_void_p]
        L.pk_llama_num_params.argtypes = [C.c_void_p]
        L.pk_llama_param_info.argtypes = [C.c_void_p, C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_int64),
                                          C.POINTER(C.c_int64)]
        L.pk_llama_set_param.argtypes = [C.c_void_p, C.c_int, f32p]
        L.pk_llama_get_param.argtypes = [C.c_void_p, C.c_int, f32p]
        L.pk_llama_get_grad.argtypes = [C.c_void_p, C.c_int, f32p]
        L.pk_llama_loss_backward.argtypes = [C.c_void_p, i32p, i32p, C.c_int64, C.c_int64, C.c_int, C.c_int, C.c_int,
                                             f32p, C.POINTER(LlamaStats), C.c_void_p]
        L.pk_llama_adamw_step.argtypes = [C.c_void_p] + [C.c_float] * 6 + [f32p]
        L.pk_llama_set_head_chunk.argtypes = [C.c_void_p, C.c_int64]
        vp, i64, ci, cf = C.c_void_p, C.c_int64, C.c_int, C.c_float
        L.pk_op_add.argtypes = [vp, vp, vp, i64, ci, vp]
        L.pk_op_mul.argtypes = [vp, vp, vp, i64, ci, vp]
        L.pk_op_scale.argtypes = [vp, cf, vp, i64, ci, vp]
        L.pk_op_axpy.argtypes = [vp, cf, vp, i64, ci, vp]
        L.pk_op_fill.argtypes = [vp, cf, i64, ci, vp]
        L.pk_op_silu_fwd.argtypes = [vp, vp, i64, ci, vp]
        L.pk_op_silu_bwd.argtypes = [vp, vp, vp, i64, ci, vp]
        L.pk_op_silu_mul_fwd.argtypes = [vp, vp, vp, i64, ci, vp]
        L.pk_op_silu_mul_bwd.argtypes = [vp, vp, vp, vp, vp, i64, ci, vp]
        L.pk_op_rmsnorm_fwd.argtypes = [vp, vp, cf, vp, vp, i64, i64, ci, vp]
        L.pk_op_rmsnorm_bwd.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, ci, vp]
        L.pk_op_rope.argtypes = [vp, vp, cf, i64, i64, ci, ci, ci, vp, ci, vp]
        L.pk_op_embedding_fwd.argtypes = [vp, vp, vp, i64, i64, i64, ci, vp]
        L.pk_op_embedding_bwd.argtypes = [vp, vp, vp, i64, i64, i64, ci, vp]
        L.pk_op_cross_entropy.argtypes = [vp, vp, i64, i64, cf, vp, f32p, ci, vp]
        L.pk_op_adamw.argtypes = [vp, vp, vp, vp, i64, cf, cf, cf, cf, cf, ci, vp]
        L.pk_op_sumsq.argtypes = [vp, i64, C.POINTER(C.c_double), vp]
        L.pk_op_gemm.argtypes = [vp, ci, vp, ci, vp, i64, i64, i64, ci, ci, ci, vp]
        L.pk_set_gemm_backend.argtypes = [ci]
        L.pk_set_head_kernel.argtypes = [ci]
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise PkError(rc, lib().pk_last_error().decode())
