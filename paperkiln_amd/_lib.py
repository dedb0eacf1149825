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


class PkError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"paperkiln_amd error {code}: {msg}")
        self.code = code


_lib = None

# every symbol include/paperkiln_amd.h declares
EXPORTS = ["pk_last_error", "pk_init", "pk_attn_fwd", "pk_attn_bwd_workspace_bytes", "pk_attn_bwd", "pk_attn_bwd_stages"]


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
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise PkError(rc, lib().pk_last_error().decode())
