"""ctypes bindings for the CPU oracle (libpk_oracle.so) and, where it was
built, the compiled reference (oracle/_ref/libpk_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg. Nothing under paperkiln_amd/ imports this.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _c(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Oracle:
    """The repo's own plain-C restatement (oracle/pk_oracle.c)."""

    def __init__(self, path: str | None = None):
        path = path or os.path.join(_HERE, "libpk_oracle.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} missing: run `make -C oracle libpk_oracle.so`")
        L = self.lib = C.CDLL(path)
        sz = C.c_size_t
        L.pko_attn_head_fwd.argtypes = [_f32p] * 3 + [sz, sz, sz, C.c_float, sz, C.c_int, sz, sz] + [_f32p] * 3
        L.pko_attn_head_bwd.argtypes = [_f32p] * 5 + [sz, sz, sz, C.c_float, sz, C.c_int, sz, sz] + [_f32p] * 3
        L.pko_attn_fwd.argtypes = [_f32p] * 3 + [sz] * 5 + [C.c_float, C.c_int, sz, sz] + [_f32p] * 2
        L.pko_attn_bwd.argtypes = [_f32p] * 4 + [sz] * 5 + [C.c_float, C.c_int, sz, sz] + [_f32p] * 3
        L.pko_attention_mask.argtypes = [sz, sz, C.c_int, _f32p]
        L.pko_visible_pairs.argtypes = [sz, C.c_int, sz, sz]
        L.pko_visible_pairs.restype = C.c_ulonglong
        f = C.c_float
        L.pko_rmsnorm_fwd.argtypes = [_f32p, _f32p, sz, sz, f, _f32p, _f32p]
        L.pko_rmsnorm_fwd.restype = None
        L.pko_rmsnorm_bwd.argtypes = [_f32p] * 4 + [sz, sz, _f32p, _f32p]
        L.pko_rmsnorm_bwd.restype = None
        L.pko_silu_fwd.argtypes = [_f32p, sz, _f32p]
        L.pko_silu_fwd.restype = None
        L.pko_silu_bwd.argtypes = [_f32p, _f32p, sz, _f32p]
        L.pko_silu_bwd.restype = None
        L.pko_rope.argtypes = [_f32p, _i32p, sz, sz, f, sz, C.c_int, _f32p]
        L.pko_embedding_fwd.argtypes = [_f32p, sz, sz, _i32p, sz, _f32p]
        L.pko_embedding_bwd.argtypes = [_f32p, _i32p, sz, sz, sz, _f32p]
        L.pko_cross_entropy.argtypes = [_f32p, _i32p, sz, sz, _f32p, _f32p]
        L.pko_adamw.argtypes = [_f32p, _f32p, _f32p, _f32p, sz, f, f, f, f, f, C.c_int]
        L.pko_adamw.restype = None
        L.pko_clip_grad_norm.argtypes = [C.POINTER(_f32p), C.POINTER(sz), sz, f]
        L.pko_clip_grad_norm.restype = f

    def head_fwd(self, q, k, v, scale, seq_len=0, causal=True, window=0, sinks=0):
        q, k, v = _c(q), _c(k), _c(v)
        T, dk = q.shape
        dv = v.shape[1]
        y = np.empty((T, dv), np.float32)
        lse = np.empty(T, np.float32)
        A = np.empty((T, T), np.float32)
        rc = self.lib.pko_attn_head_fwd(_fp(q), _fp(k), _fp(v), T, dk, dv, scale, seq_len,
                                        int(causal), window, sinks, _fp(y), _fp(lse), _fp(A))
        if rc:
            raise RuntimeError(f"pko_attn_head_fwd rc={rc}")
        return y, lse, A

    def head_bwd(self, q, k, v, A, dy, scale, seq_len=0, causal=True, window=0, sinks=0):
        q, k, v, A, dy = _c(q), _c(k), _c(v), _c(A), _c(dy)
        T, dk = q.shape
        dv = v.shape[1]
        dq = np.empty((T, dk), np.float32)
        dkk = np.empty((T, dk), np.float32)
        dvv = np.empty((T, dv), np.float32)
        rc = self.lib.pko_attn_head_bwd(_fp(q), _fp(k), _fp(v), _fp(A), _fp(dy), T, dk, dv, scale,
                                        seq_len, int(causal), window, sinks, _fp(dq), _fp(dkk), _fp(dvv))
        if rc:
            raise RuntimeError(f"pko_attn_head_bwd rc={rc}")
        return dq, dkk, dvv

    def attn_fwd(self, q, k, v, scale, causal=True, window=0, sinks=0):
        """q: [B,T,Hq,dk]; k,v: [B,T,Hkv,dk] -> (o [B,T,Hq,dk], lse [B,Hq,T])."""
        q, k, v = _c(q), _c(k), _c(v)
        B, T, Hq, dk = q.shape
        Hkv = k.shape[2]
        o = np.empty_like(q)
        lse = np.empty((B, Hq, T), np.float32)
        rc = self.lib.pko_attn_fwd(_fp(q), _fp(k), _fp(v), B, T, Hq, Hkv, dk, scale, int(causal),
                                   window, sinks, _fp(o), _fp(lse))
        if rc:
            raise RuntimeError(f"pko_attn_fwd rc={rc}")
        return o, lse

    def attn_bwd(self, q, k, v, d_o, scale, causal=True, window=0, sinks=0):
        q, k, v, d_o = _c(q), _c(k), _c(v), _c(d_o)
        B, T, Hq, dk = q.shape
        Hkv = k.shape[2]
        dq = np.empty_like(q)
        dkk = np.empty_like(k)
        dvv = np.empty_like(v)
        rc = self.lib.pko_attn_bwd(_fp(q), _fp(k), _fp(v), _fp(d_o), B, T, Hq, Hkv, dk, scale,
                                   int(causal), window, sinks, _fp(dq), _fp(dkk), _fp(dvv))
        if rc:
            raise RuntimeError(f"pko_attn_bwd rc={rc}")
        return dq, dkk, dvv

    def attention_mask(self, rows, seq_len, causal):
        out = np.empty((rows, rows), np.float32)
        rc = self.lib.pko_attention_mask(rows, seq_len, int(causal), _fp(out))
        if rc:
            raise RuntimeError(f"pko_attention_mask rc={rc}")
        return out

    def visible_pairs(self, T, causal=True, window=0, sinks=0):
        return int(self.lib.pko_visible_pairs(T, int(causal), window, sinks))

    # ---- Llama block ops --------------------------------------------------
    def rmsnorm(self, x, w, dy=None, eps=1e-5):
        """y, rms_inv (and dx, dw when dy is given)."""
        x, w = _c(x), _c(w).reshape(-1)
        R, Cc = x.shape
        y, ri = np.empty_like(x), np.empty(R, np.float32)
        self.lib.pko_rmsnorm_fwd(_fp(x), _fp(w), R, Cc, eps, _fp(y), _fp(ri))
        if dy is None:
            return y, ri
        dy = _c(dy)
        dx, dw = np.empty_like(x), np.empty(Cc, np.float32)
        self.lib.pko_rmsnorm_bwd(_fp(dy), _fp(x), _fp(ri), _fp(w), R, Cc, _fp(dw), _fp(dx))
        return y, ri, dx, dw

    def silu(self, x, dy=None):
        x = _c(x)
        y = np.empty_like(x)
        self.lib.pko_silu_fwd(_fp(x), x.size, _fp(y))
        if dy is None:
            return y
        dy = _c(dy)
        dx = np.empty_like(x)
        self.lib.pko_silu_bwd(_fp(x), _fp(dy), x.size, _fp(dx))
        return y, dx

    def rope(self, x, pos, theta, head_dim, inverse=False):
        x = _c(x)
        pos = np.ascontiguousarray(pos, np.int32)
        y = np.empty_like(x)
        rc = self.lib.pko_rope(_fp(x), pos.ctypes.data_as(_i32p), x.shape[0], x.shape[1], theta, head_dim,
                               int(inverse), _fp(y))
        if rc:
            raise RuntimeError("apply_rope: bad cols / head_dim")
        return y

    def embedding(self, table, ids, dy=None):
        table = _c(table)
        ids = np.ascontiguousarray(ids, np.int32)
        V, d = table.shape
        y = np.empty((len(ids), d), np.float32)
        if self.lib.pko_embedding_fwd(_fp(table), V, d, ids.ctypes.data_as(_i32p), len(ids), _fp(y)):
            raise RuntimeError("embedding: id out of range")
        if dy is None:
            return y
        dy = _c(dy)
        dt = np.empty_like(table)
        self.lib.pko_embedding_bwd(_fp(dy), ids.ctypes.data_as(_i32p), len(ids), V, d, _fp(dt))
        return y, dt

    def cross_entropy(self, logits, targets):
        logits = _c(logits)
        targets = np.ascontiguousarray(targets, np.int32)
        loss = C.c_float()
        dl = np.empty_like(logits)
        rc = self.lib.pko_cross_entropy(_fp(logits), targets.ctypes.data_as(_i32p), logits.shape[0], logits.shape[1],
                                        C.byref(loss), _fp(dl))
        if rc:
            raise RuntimeError("cross_entropy: target out of range")
        return loss.value, dl

    def adamw(self, p, g, m, v, lr, b1=0.9, b2=0.999, eps=1e-8, wd=0.01, t=1):
        """Returns updated copies (p, m, v)."""
        p, g, m, v = (_c(a).copy() for a in (p, g, m, v))
        self.lib.pko_adamw(_fp(p), _fp(g), _fp(m), _fp(v), p.size, lr, b1, b2, eps, wd, t)
        return p, m, v

    def clip_grad_norm(self, grads, max_norm):
        """Returns (total_norm, clipped copies)."""
        gs = [_c(g).copy() for g in grads]
        ptrs = (_f32p * len(gs))(*[_fp(g) for g in gs])
        sizes = (C.c_size_t * len(gs))(*[g.size for g in gs])
        total = self.lib.pko_clip_grad_norm(ptrs, sizes, len(gs), max_norm)
        return float(total), gs


class Reference:
    """The compiled reference behind oracle/ref_shim.cpp. Only present where
    `make -C oracle ref` ran with /root/reference available."""

    def __init__(self, path: str | None = None):
        path = path or os.path.join(_HERE, "_ref", "libpk_ref.so")
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        L = self.lib = C.CDLL(path)
        sz = C.c_size_t
        L.pkref_last_error.restype = C.c_char_p
        L.pkref_fused_attention.argtypes = [_f32p] * 4 + [sz, sz, sz, C.c_float, sz, C.c_int] + [_f32p] * 4
        L.pkref_swa_attention.argtypes = [_f32p] * 4 + [sz, sz, sz, C.c_float, sz, sz, sz] + [_f32p] * 4
        L.pkref_attention_mask.argtypes = [sz, sz, C.c_int, _f32p]
        L.pkref_rmsnorm.argtypes = [_f32p] * 3 + [sz, sz] + [_f32p] * 3
        L.pkref_silu.argtypes = [_f32p] * 2 + [sz, sz] + [_f32p] * 2
        L.pkref_apply_rope.argtypes = [_f32p, _i32p, _f32p, sz, sz, C.c_float, sz, _f32p, _f32p]
        L.pkref_cross_entropy.argtypes = [_f32p, _i32p, sz, sz, _f32p, _f32p]
        L.pkref_embedding.argtypes = [_f32p, _i32p, _f32p, sz, sz, sz, _f32p, _f32p]
        L.pkref_matmul.argtypes = [_f32p, _f32p, sz, sz, sz, _f32p]
        L.pkref_llama_create.argtypes = [sz] * 6 + [C.c_float, C.c_int, C.c_uint]
        L.pkref_llama_create.restype = C.c_void_p
        L.pkref_llama_destroy.argtypes = [C.c_void_p]
        L.pkref_llama_num_params.argtypes = [C.c_void_p]
        L.pkref_llama_num_params.restype = sz
        L.pkref_llama_param_name.argtypes = [C.c_void_p, sz]
        L.pkref_llama_param_name.restype = C.c_char_p
        L.pkref_llama_param_shape.argtypes = [C.c_void_p, sz, C.POINTER(sz), C.POINTER(sz)]
        L.pkref_llama_get_param.argtypes = [C.c_void_p, sz, _f32p]
        L.pkref_llama_set_param.argtypes = [C.c_void_p, sz, _f32p]
        L.pkref_llama_get_grad.argtypes = [C.c_void_p, sz, _f32p]
        L.pkref_llama_loss_backward.argtypes = [C.c_void_p, _i32p, _i32p, sz, sz, C.c_int, C.c_int,
                                                _f32p, C.POINTER(sz), _f32p]
        L.pkref_llama_adamw_step.argtypes = [C.c_void_p] + [C.c_float] * 6 + [_f32p]

    def _chk(self, rc):
        if rc:
            raise RuntimeError(self.lib.pkref_last_error().decode())

    def _attn(self, fn, q, k, v, dy, mid):
        q, k, v = _c(q), _c(k), _c(v)
        T, dk = q.shape
        dv = v.shape[1]
        y = np.empty((T, dv), np.float32)
        if dy is None:
            self._chk(fn(_fp(q), _fp(k), _fp(v), None, T, dk, dv, *mid, _fp(y), None, None, None))
            return y
        dy = _c(dy)
        dq = np.empty((T, dk), np.float32)
        dkk = np.empty((T, dk), np.float32)
        dvv = np.empty((T, dv), np.float32)
        self._chk(fn(_fp(q), _fp(k), _fp(v), _fp(dy), T, dk, dv, *mid, _fp(y), _fp(dq), _fp(dkk), _fp(dvv)))
        return y, dq, dkk, dvv

    def fused_attention(self, q, k, v, scale, seq_len=0, causal=True, dy=None):
        return self._attn(self.lib.pkref_fused_attention, q, k, v, dy, (scale, seq_len, int(causal)))

    def swa_attention(self, q, k, v, scale, window, sinks, seq_len=0, dy=None):
        return self._attn(self.lib.pkref_swa_attention, q, k, v, dy, (scale, window, sinks, seq_len))

    def weights(self, q, k, scale, seq_len=0, causal=True, window=0, sinks=0):
        """The reference's own A matrix, read back by passing V = I."""
        T = q.shape[0]
        eye = np.eye(T, dtype=np.float32)
        if window:
            return self.swa_attention(q, k, eye, scale, window, sinks, seq_len)
        return self.fused_attention(q, k, eye, scale, seq_len, causal)

    def attention_mask(self, rows, seq_len, causal):
        out = np.empty((rows, rows), np.float32)
        self._chk(self.lib.pkref_attention_mask(rows, seq_len, int(causal), _fp(out)))
        return out

    def rmsnorm(self, x, w, dy):
        x, w, dy = _c(x), _c(w), _c(dy)
        R, Cc = x.shape
        y, dx, dw = np.empty_like(x), np.empty_like(x), np.empty(Cc, np.float32)
        self._chk(self.lib.pkref_rmsnorm(_fp(x), _fp(w), _fp(dy), R, Cc, _fp(y), _fp(dx), _fp(dw)))
        return y, dx, dw

    def silu(self, x, dy):
        x, dy = _c(x), _c(dy)
        y, dx = np.empty_like(x), np.empty_like(x)
        self._chk(self.lib.pkref_silu(_fp(x), _fp(dy), x.shape[0], x.shape[1], _fp(y), _fp(dx)))
        return y, dx

    def apply_rope(self, qkv, pos, theta, head_dim, dy):
        qkv, dy = _c(qkv), _c(dy)
        pos = np.ascontiguousarray(pos, np.int32)
        y, dx = np.empty_like(qkv), np.empty_like(qkv)
        self._chk(self.lib.pkref_apply_rope(_fp(qkv), pos.ctypes.data_as(_i32p), _fp(dy), qkv.shape[0],
                                            qkv.shape[1], theta, head_dim, _fp(y), _fp(dx)))
        return y, dx

    def cross_entropy(self, logits, targets):
        logits = _c(logits)
        targets = np.ascontiguousarray(targets, np.int32)
        loss = C.c_float()
        dl = np.empty_like(logits)
        self._chk(self.lib.pkref_cross_entropy(_fp(logits), targets.ctypes.data_as(_i32p), logits.shape[0],
                                               logits.shape[1], C.byref(loss), _fp(dl)))
        return loss.value, dl

    def embedding(self, table, ids, dy):
        table, dy = _c(table), _c(dy)
        ids = np.ascontiguousarray(ids, np.int32)
        y = np.empty((len(ids), table.shape[1]), np.float32)
        dt = np.empty_like(table)
        self._chk(self.lib.pkref_embedding(_fp(table), ids.ctypes.data_as(_i32p), _fp(dy), table.shape[0],
                                           table.shape[1], len(ids), _fp(y), _fp(dt)))
        return y, dt

    def matmul(self, a, b):
        a, b = _c(a), _c(b)
        c = np.empty((a.shape[0], b.shape[1]), np.float32)
        self._chk(self.lib.pkref_matmul(_fp(a), _fp(b), a.shape[0], a.shape[1], b.shape[1], _fp(c)))
        return c


class RefLlama:
    """nn::Llama of the compiled reference (src/llama.cpp)."""

    def __init__(self, ref: Reference, vocab, d, n_layers, n_heads, d_ff, n_ctx=256, rope_theta=10000.0,
                 tie=True, seed=0):
        self.ref = ref
        self.h = ref.lib.pkref_llama_create(vocab, d, n_layers, n_heads, d_ff, n_ctx, rope_theta, int(tie), seed)
        if not self.h:
            raise RuntimeError(ref.lib.pkref_last_error().decode())
        L = ref.lib
        self.names, self.shapes = [], []
        for i in range(L.pkref_llama_num_params(self.h)):
            self.names.append(L.pkref_llama_param_name(self.h, i).decode())
            r, c = C.c_size_t(), C.c_size_t()
            L.pkref_llama_param_shape(self.h, i, C.byref(r), C.byref(c))
            self.shapes.append((r.value, c.value))

    def __del__(self):
        if getattr(self, "h", None):
            self.ref.lib.pkref_llama_destroy(self.h)
            self.h = None

    def params(self):
        out = {}
        for i, (n, s) in enumerate(zip(self.names, self.shapes)):
            a = np.empty(s, np.float32)
            self.ref.lib.pkref_llama_get_param(self.h, i, _fp(a))
            out[n] = a
        return out

    def set_params(self, sd):
        for i, n in enumerate(self.names):
            self.ref.lib.pkref_llama_set_param(self.h, i, _fp(_c(sd[n])))

    def grads(self):
        out = {}
        for i, (n, s) in enumerate(zip(self.names, self.shapes)):
            a = np.empty(s, np.float32)
            self.ref.lib.pkref_llama_get_grad(self.h, i, _fp(a))
            out[n] = a
        return out

    def loss_backward(self, ids, targets, seq_len=0, checkpoint=False, backward=True, want_logits=False):
        ids = np.ascontiguousarray(ids, np.int32)
        targets = np.ascontiguousarray(targets, np.int32)
        loss, live = C.c_float(), C.c_size_t()
        logits = None
        if want_logits:
            V = self.shapes[self.names.index("embed_tokens.weight")][0]
            logits = np.empty((len(ids), V), np.float32)
        self.ref._chk(self.ref.lib.pkref_llama_loss_backward(
            self.h, ids.ctypes.data_as(_i32p), targets.ctypes.data_as(_i32p), len(ids), seq_len,
            int(checkpoint), int(backward), C.byref(loss), C.byref(live), _fp(logits)))
        return loss.value, live.value, logits

    def adamw_step(self, lr, b1=0.9, b2=0.999, eps=1e-8, wd=0.01, max_norm=0.0):
        tn = C.c_float()
        self.ref._chk(self.ref.lib.pkref_llama_adamw_step(self.h, lr, b1, b2, eps, wd, max_norm, C.byref(tn)))
        return tn.value


def load_reference():
    """Reference() or None when oracle/_ref was not built."""
    try:
        return Reference()
    except (FileNotFoundError, OSError):
        return None
