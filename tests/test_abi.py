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
    """pk_attn_bwd_workspace_bytes: delta [B, Hq, T] fp32 for every mask; without a band, query heads that share KV
    heads on a grid that would leave CUs idle add the per-split partial dK / dV; a band mask with 1..32 sink keys on a
    sequence longer than key block 0's band adds the partial sink rows of a split sink tail
    ((chunks of 512 queries + 1) x {dK, dV} x 32 rows x head_dim fp32 per (batch, KV head), 256-byte aligned)."""
    L = _lib.lib()
    B, T, Hq, Hkv, dk = 2, 4096, 8, 4, 128
    delta = 4 * B * Hq * T

    def ws(window, sinks, t=T):
        sh = _lib.AttnShape(B, t, Hq, Hkv, dk, 1, window, sinks, 0.5, _lib.PK_BF16, _lib.PK_BF16)
        return L.pk_attn_bwd_workspace_bytes(ctypes.byref(sh))

    # no band, 2 query heads per KV head, 16 paired key blocks x 8 (batch, KV head) units = 128 dK/dV workgroups for
    # 256 CUs: the heads of a group are dealt to 2 workgroups, whose fp32 partial dK and dV follow delta
    assert ws(0, 0) == delta + 4 * 2 * (B * Hkv) * 2 * T * dk
    mha = _lib.AttnShape(B, T, Hq, Hq, dk, 1, 0, 0, 0.5, _lib.PK_BF16, _lib.PK_BF16)
    assert L.pk_attn_bwd_workspace_bytes(ctypes.byref(mha)) == delta   # one query head per KV head: nothing to deal
    assert ws(256, 0) == delta          # no sink keys: nothing to split
    assert ws(256, 33) == delta         # more sink keys than one wavefront owns: not split
    q0 = ((127 + 256 - 1) // 64 + 1) * 64   # first 64-query tile wholly past key block 0's band
    nch = -(-(T - q0) // 512)
    assert ws(256, 4) == delta + 4 * B * Hkv * (nch + 1) * 2 * 32 * dk
    assert ws(256, 4, t=q0) == 4 * B * Hq * q0   # the sequence ends with the band: no tail
    odd = 4 * B * Hq * 4001                      # delta not a multiple of 256 bytes: the tail starts aligned
    assert ws(256, 4, t=4001) == odd + (256 - odd % 256) % 256 + 4 * B * Hkv * (-(-(4001 - q0) // 512) + 1) * 2 * 32 * dk


def test_a_window_that_covers_the_sequence_is_no_band():
    """The reference takes size_t window / sinks and defines window >= seq_len as plain causal attention
    (tests/test_swa.cpp:47-57), so INT32_MAX is a legal "no band": the shape is brought into range on the host,
    before any index arithmetic, and sizes its workspace as the causal mask does."""
    L = _lib.lib()
    B, T, Hq, Hkv, dk = 2, 4096, 8, 8, 128

    def ws(window, sinks):
        sh = _lib.AttnShape(B, T, Hq, Hkv, dk, 1, window, sinks, 0.5, _lib.PK_BF16, _lib.PK_BF16)
        return L.pk_attn_bwd_workspace_bytes(ctypes.byref(sh))

    causal = ws(0, 0)
    assert causal == 4 * B * Hq * T
    for window in (T, T + 1, 2**31 - 1):
        for sinks in (0, 4, 2**31 - 1):
            assert ws(window, sinks) == causal
    assert ws(T // 2, 4) > causal         # a real band with sink keys still gets its sink-tail rows
    assert ws(256, 2**31 - 1) == causal   # more sink keys than tokens: every key is a sink, nothing to split
    sh = _lib.AttnShape(1, 2**24 + 1, 1, 1, 64, 1, 0, 0, 0.5, _lib.PK_BF16, _lib.PK_BF16)
    assert L.pk_attn_bwd_workspace_bytes(ctypes.byref(sh)) == 0 and b"2^24" in L.pk_last_error()


def test_handle_and_pointer_errors_do_not_need_a_gpu():
    """A NULL model handle and a pointer pk_alloc never returned are reported, not dereferenced or ignored."""
    L = _lib.lib()
    r, c = ctypes.c_int64(), ctypes.c_int64()
    assert L.pk_llama_param_info(None, 0, None, 0, ctypes.byref(r), ctypes.byref(c)) == 2
    assert b"null model handle" in L.pk_last_error()
    assert L.pk_llama_num_params(None) == -1
    assert L.pk_llama_adamw_step(None, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0.0, None) == 2
    assert L.pk_llama_set_head_chunk(None, 128) == 2
    assert L.pk_llama_destroy(None) == 0
    buf = ctypes.create_string_buffer(64)
    assert L.pk_free(ctypes.cast(buf, ctypes.c_void_p)) == 2 and b"pk_alloc" in L.pk_last_error()
    assert L.pk_free(None) == 0
    assert L.pk_alloc(64, None) == 2
