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


def test_backward_workspace_follows_the_mask():
    """pk_attn_bwd_workspace_bytes: delta [B, Hq, T] fp32 for every mask; a band mask with 1..32 sink keys on a
    sequence longer than key block 0's band adds the partial sink rows of a split sink tail
    ((chunks of 512 queries + 1) x {dK, dV} x 32 rows x head_dim fp32 per (batch, KV head), 256-byte aligned)."""
    L = _lib.lib()
    B, T, Hq, Hkv, dk = 2, 4096, 8, 4, 128
    delta = 4 * B * Hq * T

    def ws(window, sinks, t=T):
        sh = _lib.AttnShape(B, t, Hq, Hkv, dk, 1, window, sinks, 0.5, _lib.PK_BF16, _lib.PK_BF16)
        return L.pk_attn_bwd_workspace_bytes(ctypes.byref(sh))

    assert ws(0, 0) == delta
    assert ws(256, 0) == delta          # no sink keys: nothing to split
    assert ws(256, 33) == delta         # more sink keys than one wavefront owns: not split
    q0 = ((127 + 256 - 1) // 64 + 1) * 64   # first 64-query tile wholly past key block 0's band
    nch = -(-(T - q0) // 512)
    assert ws(256, 4) == delta + 4 * B * Hkv * (nch + 1) * 2 * 32 * dk
    assert ws(256, 4, t=q0) == 4 * B * Hq * q0   # the sequence ends with the band: no tail
    odd = 4 * B * Hq * 4001                      # delta not a multiple of 256 bytes: the tail starts aligned
    assert ws(256, 4, t=4001) == odd + (256 - odd % 256) % 256 + 4 * B * Hkv * (-(-(4001 - q0) // 512) + 1) * 2 * 32 * dk
