"""Host-side handle on the device-resident Llama (nn::Llama of paperkiln,
include/microtorch/llama.hpp:14-51) behind the C ABI. Parameter names are the
reference's ("layers.N.self_attn.q_proj.weight", ...); arrays cross the
boundary as float32 numpy copies, as in python/bindings.cpp:21-37."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import LlamaConfig, LlamaStats

_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int)


class Llama:
    def __init__(self, vocab, d, n_layers, n_heads, d_ff, rope_theta=10000.0, compute_dtype="fp32",
                 rope_all_heads=False, window=0, sinks=0, seed=0):
        self.L = _lib.lib()
        _lib.check(self.L.pk_init(0, None, 0))
        dt = {"fp32": _lib.PK_F32, "bf16": _lib.PK_BF16}[compute_dtype]
        self.cfg = LlamaConfig(vocab, d, n_layers, n_heads, d_ff, rope_theta, 1, dt, int(rope_all_heads), window, sinks)
        self.h = C.c_void_p()
        _lib.check(self.L.pk_llama_create(C.byref(self.cfg), seed, C.byref(self.h)))
        self.names, self.shapes = [], []
        buf = C.create_string_buffer(256)
        for i in range(self.L.pk_llama_num_params(self.h)):
            r, c = C.c_int64(), C.c_int64()
            _lib.check(self.L.pk_llama_param_info(self.h, i, buf, 256, C.byref(r), C.byref(c)))
            self.names.append(buf.value.decode())
            self.shapes.append((r.value, c.value))

    def close(self):
        if self.h:
            self.L.pk_llama_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def parameter_count(self):
        return sum(r * c for r, c in self.shapes)

    def set_params(self, sd):
        for i, n in enumerate(self.names):
            a = np.ascontiguousarray(sd[n], np.float32).reshape(self.shapes[i])
            _lib.check(self.L.pk_llama_set_param(self.h, i, a.ctypes.data_as(_f32p)))

    def _get(self, fn):
        out = {}
        for i, (n, s) in enumerate(zip(self.names, self.shapes)):
            a = np.empty(s, np.float32)
            _lib.check(fn(self.h, i, a.ctypes.data_as(_f32p)))
            out[n] = a
        return out

    def params(self):
        return self._get(self.L.pk_llama_get_param)

    def grads(self):
        return self._get(self.L.pk_llama_get_grad)

    def set_head_chunk(self, rows):
        """Rows of the tied head evaluated at a time when fused_head=True (default 2048)."""
        _lib.check(self.L.pk_llama_set_head_chunk(self.h, int(rows)))

    def loss_backward(self, ids, targets, seq_len=0, checkpoint=False, backward=True, fused_head=True, stream=None):
        """zero_grad -> forward -> cross-entropy -> backward. Returns (loss, stats dict).
        stream: a HIP stream handle (int) the step is enqueued on; None = the default stream."""
        ids = np.ascontiguousarray(ids, np.int32)
        targets = np.ascontiguousarray(targets, np.int32)
        if len(ids) != len(targets):
            raise RuntimeError("cross_entropy: one target per row")
        loss, st = C.c_float(), LlamaStats()
        _lib.check(self.L.pk_llama_loss_backward(self.h, ids.ctypes.data_as(_i32p), targets.ctypes.data_as(_i32p),
                                                 len(ids), seq_len, int(checkpoint), int(backward), int(fused_head),
                                                 C.byref(loss), C.byref(st), C.c_void_p(stream) if stream else None))
        return loss.value, {"live_vars_after_forward": st.live_vars_after_forward,
                            "activation_bytes_after_forward": st.activation_bytes_after_forward,
                            "peak_activation_bytes": st.peak_activation_bytes}

    def adamw_step(self, lr, b1=0.9, b2=0.999, eps=1e-8, wd=0.01, max_norm=0.0):
        tn = C.c_float()
        _lib.check(self.L.pk_llama_adamw_step(self.h, lr, b1, b2, eps, wd, max_norm, C.byref(tn)))
        return tn.value
