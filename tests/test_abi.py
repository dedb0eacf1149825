"""The C-ABI library loads and exports every symbol include/paperkiln_amd.h declares. No GPU, no compute."""
import ctypes
import os
import re

import pytest

from paperkiln_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "paperkiln_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pk_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} not built: run __graft_entry__.build()")
    L = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name


def test_argument_errors_do_not_need_a_gpu():
    """Shape/argument validation happens before any HIP call and mirrors the reference's throws."""
    L = _lib.lib()
    sh = _lib.AttnShape(1, 8, 3, 2, 4, 1, 0, 0, 0.5, _lib.PK_F32, _lib.PK_F32)  # Hq % Hkv != 0
    t = _lib.Tensor4(0, 0, 0, 0)
    rc = L.pk_attn_fwd(ctypes.byref(sh), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), None, None)
    assert rc == 1 and b"shape mismatch" in L.pk_last_error()
    sh = _lib.AttnShape(1, 8, 2, 2, 4, 0, 3, 0, 0.5, _lib.PK_F32, _lib.PK_F32)  # window without causal
    assert L.pk_attn_fwd(ctypes.byref(sh), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), None, None) == 2
    sh = _lib.AttnShape(1, 8, 2, 2, 4, 1, 0, 0, 0.5, _lib.PK_F32, _lib.PK_F32)
    assert L.pk_attn_fwd(ctypes.byref(sh), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), None, None) == 2  # null tensors
    assert L.pk_attn_bwd_workspace_bytes(ctypes.byref(sh)) == 4 * 1 * 2 * 8
