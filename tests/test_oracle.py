"""Pins for the CPU oracle (oracle/pk_oracle.c). CPU only.

The oracle is checked against (1) vectors written by the compiled reference
(tests/golden/*.npz), (2) the compiled reference itself where oracle/_ref is
built, (3) what the mathematics fixes: closed forms, fp64 brute force, finite
differences, and the reference tests' own behavioural pins
(tests/test_gradcheck.cpp:196-238, tests/test_swa.cpp).
"""
import numpy as np
import pytest

from paperkiln_amd import synth

TOL = 2e-6  # fp32 summation-order noise between the oracle's GEMM and matmul_optimized's AVX2 lanes


def maxabs(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max())


def test_oracle_matches_reference_vectors(oracle, golden):
    g = golden
    o, lse = oracle.attn_fwd(g.q, g.k, g.v, g.scale, g.causal, g.window, g.sinks)
    dq, dk, dv = oracle.attn_bwd(g.q, g.k, g.v, g.d_o, g.scale, g.causal, g.window, g.sinks)
    tol = TOL * max(1.0, np.sqrt(g.T / 64.0)) * (g.Hq // g.Hkv)
    assert maxabs(o, g.o) < tol
    assert maxabs(lse, g.lse) < 4 * tol
    assert maxabs(dq, g.dq) < tol
    assert maxabs(dk, g.dk) < 2 * tol
    assert maxabs(dv, g.dv) < 2 * tol


@pytest.mark.parametrize("T,dk,sl,causal,window,sinks", [
    (8, 4, 0, True, 0, 0), (8, 4, 4, True, 0, 0), (8, 4, 4, False, 0, 0), (12, 4, 0, True, 4, 1),
    (24, 4, 12, True, 4, 1), (128, 32, 0, True, 0, 0), (128, 32, 64, True, 16, 4), (96, 16, 32, True, 5, 7)])
def test_oracle_matches_compiled_reference(oracle, reference, T, dk, sl, causal, window, sinks):
    """Stacked-batch (seq_len) semantics of the head functions against ops.cpp itself."""
    q, k, v, dy = (synth.randn(s, (T, dk)) for s in (1, 2, 3, 4))
    sc = float(np.float32(1 / np.sqrt(dk)))
    y, lse, A = oracle.head_fwd(q, k, v, sc, sl, causal, window, sinks)
    dq, dk_, dv = oracle.head_bwd(q, k, v, A, dy, sc, sl, causal, window, sinks)
    if window:
        ry, rdq, rdk, rdv = reference.swa_attention(q, k, v, sc, window, sinks, sl, dy=dy)
    else:
        ry, rdq, rdk, rdv = reference.fused_attention(q, k, v, sc, sl, causal, dy=dy)
    rA = reference.weights(q, k, sc, sl, causal, window, sinks)
    for a, b in ((y, ry), (dq, rdq), (dk_, rdk), (dv, rdv), (A, rA)):
        assert maxabs(a, b) < 4e-6
    assert np.array_equal(A != 0, rA != 0)  # identical hard-zero mask
    assert maxabs(oracle.attention_mask(T, sl, causal), reference.attention_mask(T, sl, causal)) == 0.0


def brute_force(q, k, v, d_o, scale, causal, window, sinks):
    """fp64 softmax attention and its analytic gradients, one head, from the definition."""
    q, k, v, d_o = (x.astype(np.float64) for x in (q, k, v, d_o))
    T = q.shape[0]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    vis = np.ones((T, T), bool)
    if causal:
        vis &= j <= i
    if window:
        vis &= (j + window > i) | (j < sinks)
    s = np.where(vis, scale * q @ k.T, -np.inf)
    m = s.max(1, keepdims=True)
    e = np.exp(s - m)
    z = e.sum(1, keepdims=True)
    P = e / z
    o = P @ v
    lse = (m + np.log(z))[:, 0]
    dP = d_o @ v.T
    dS = P * (dP - (dP * P).sum(1, keepdims=True)) * scale
    return o, lse, dS @ k, dS.T @ q, P.T @ d_o


@pytest.mark.parametrize("causal,window,sinks", [(True, 0, 0), (False, 0, 0), (True, 3, 0), (True, 4, 2), (True, 1, 0)])
def test_oracle_vs_fp64_brute_force(oracle, causal, window, sinks):
    T, dk = 16, 8
    q, k, v, d_o = (synth.randn(s, (T, dk)) for s in (11, 12, 13, 14))
    y, lse, A = oracle.head_fwd(q, k, v, 0.3, 0, causal, window, sinks)
    dq, dk_, dv = oracle.head_bwd(q, k, v, A, d_o, 0.3, 0, causal, window, sinks)
    bo, blse, bdq, bdk, bdv = brute_force(q, k, v, d_o, np.float64(np.float32(0.3)), causal, window, sinks)
    for a, b in ((y, bo), (lse, blse), (dq, bdq), (dk_, bdk), (dv, bdv)):
        assert maxabs(a, b) < 3e-6


def test_oracle_finite_differences(oracle):
    """Central differences, h=1e-2, relative error < 5e-3: tests/test_gradcheck.cpp:41-62,101."""
    T, dk, sc = 8, 4, 0.5
    q, k, v = (synth.randn(s, (T, dk), 0.5) for s in (61, 62, 63))
    d_o = np.full((T, dk), 1.0 / (T * dk), np.float32)  # d(mean(y))/dy

    def f(q, k, v):
        return float(oracle.head_fwd(q, k, v, sc, 0, True, 4, 1)[0].astype(np.float64).mean())

    y, lse, A = oracle.head_fwd(q, k, v, sc, 0, True, 4, 1)
    grads = oracle.head_bwd(q, k, v, A, d_o, sc, 0, True, 4, 1)
    h = 1e-2
    for idx, g in enumerate(grads):
        worst = 0.0
        for i in range(T):
            for j in range(dk):
                args = [q.copy(), k.copy(), v.copy()]
                args[idx][i, j] += h
                up = f(*args)
                args[idx][i, j] -= 2 * h
                dn = f(*args)
                fd = (up - dn) / (2 * h)
                worst = max(worst, abs(g[i, j] - fd) / (1 + max(abs(g[i, j]), abs(fd))))
        assert worst < 5e-3


def test_closed_forms(oracle):
    # T = 1: O = V, LSE = scale*q.k, dV = dO, dQ = dK = 0
    q, k, v, d_o = (synth.randn(s, (1, 8)) for s in (1, 2, 3, 4))
    y, lse, A = oracle.head_fwd(q, k, v, 0.7, 0, True, 0, 0)
    dq, dk, dv = oracle.head_bwd(q, k, v, A, d_o, 0.7, 0, True, 0, 0)
    assert maxabs(y, v) == 0.0 and maxabs(dv, d_o) == 0.0
    assert maxabs(lse, np.float32(0.7) * (q * k).sum()) < 1e-6
    assert maxabs(dq, 0) == 0.0 and maxabs(dk, 0) == 0.0
    # Q = 0: uniform weights on the visible set -> O_i = mean of visible V, LSE_i = log(count_i)
    T, dk_ = 40, 8
    k, v = synth.randn(5, (T, dk_)), synth.randn(6, (T, dk_))
    q = np.zeros((T, dk_), np.float32)
    for causal, window, sinks in ((True, 0, 0), (True, 6, 3), (False, 0, 0)):
        y, lse, A = oracle.head_fwd(q, k, v, 1.0, 0, causal, window, sinks)
        for i in range(T):
            js = [j for j in range(T) if (not causal or j <= i) and (not window or j + window > i or j < sinks)]
            assert abs(lse[i] - np.log(len(js))) < 1e-6
            assert maxabs(y[i], v[js].astype(np.float64).mean(0)) < 1e-6
        assert int((A != 0).sum()) == oracle.visible_pairs(T, causal, window, sinks) == \
            synth.visible_pairs(T, causal, window, sinks)


def test_invariants(oracle):
    T, dk = 64, 16
    q, k, v, d_o = (synth.randn(s, (T, dk)) for s in (21, 22, 23, 24))
    sc = 0.25
    y, lse, A = oracle.head_fwd(q, k, v, sc, 0, True, 8, 2)
    # rows of exp(scale*s - LSE) sum to one over the visible set
    s = sc * q.astype(np.float64) @ k.astype(np.float64).T
    P = np.where(A != 0, np.exp(s - lse[:, None]), 0.0)
    assert maxabs(P.sum(1), 1.0) < 1e-5
    assert maxabs(P, A) < 1e-6
    # rowsum(dO .* O) == rowsum(dP .* P): the identity the recompute backward rests on (ops.cpp:920-921)
    dP = d_o.astype(np.float64) @ v.astype(np.float64).T
    assert maxabs((d_o.astype(np.float64) * y).sum(1), (dP * A).sum(1)) < 1e-5


def test_swa_equivalence_and_locality(oracle):
    """tests/test_swa.cpp pins 1, 3, 4, 5."""
    T, dk, sc = 12, 4, 0.5
    q, k, v = (synth.randn(s, (T, dk)) for s in (1, 2, 3))
    a = oracle.head_fwd(q, k, v, sc, 0, True, 0, 0)[0]
    b = oracle.head_fwd(q, k, v, sc, 0, True, T, 0)[0]
    assert np.array_equal(a, b)  # window >= T, sinks = 0 == causal, bitwise (test_swa.cpp:47-57)
    # locality: v outside window u sinks leaves row i untouched (test_swa.cpp:92-106)
    y0 = oracle.head_fwd(q, k, v, sc, 0, True, 3, 0)[0]
    v2 = v.copy()
    v2[2, 0] += 10.0
    y1 = oracle.head_fwd(q, k, v2, sc, 0, True, 3, 0)[0]
    assert y0[9, 0] == y1[9, 0]
    v2[8, 0] += 10.0
    assert oracle.head_fwd(q, k, v2, sc, 0, True, 3, 0)[0][9, 0] != y0[9, 0]
    # sinks: token 0 visible beyond the window only with a sink (test_swa.cpp:108-122)
    v3 = v.copy()
    v3[0, 0] += 10.0
    assert oracle.head_fwd(q, k, v, sc, 0, True, 2, 0)[0][9, 0] == oracle.head_fwd(q, k, v3, sc, 0, True, 2, 0)[0][9, 0]
    assert oracle.head_fwd(q, k, v, sc, 0, True, 2, 1)[0][9, 0] != oracle.head_fwd(q, k, v3, sc, 0, True, 2, 1)[0][9, 0]
    # stacked batch == singles (test_swa.cpp:124-155); exact here, blocks never mix in the oracle's GEMM order
    q2, k2, v2 = (np.concatenate([x, synth.randn(s, (T, dk))]) for x, s in ((q, 16), (k, 17), (v, 18)))
    ys = oracle.head_fwd(q2, k2, v2, sc, T, True, 4, 1)[0]
    assert maxabs(ys[:T], oracle.head_fwd(q, k, v, sc, 0, True, 4, 1)[0]) < 1e-6
    assert maxabs(ys[T:], oracle.head_fwd(q2[T:], k2[T:], v2[T:], sc, 0, True, 4, 1)[0]) < 1e-6


def test_gqa_equals_repeated_kv(oracle):
    """GQA == MHA with each KV head repeated over its consecutive group, dK/dV summed."""
    B, T, Hq, Hkv, dk = 2, 24, 6, 2, 8
    q, d_o = synth.randn(1, (B, T, Hq, dk)), synth.randn(4, (B, T, Hq, dk))
    k, v = synth.randn(2, (B, T, Hkv, dk)), synth.randn(3, (B, T, Hkv, dk))
    kr, vr = np.repeat(k, Hq // Hkv, axis=2), np.repeat(v, Hq // Hkv, axis=2)
    o1, l1 = oracle.attn_fwd(q, k, v, 0.3)
    o2, l2 = oracle.attn_fwd(q, kr, vr, 0.3)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)
    dq1, dk1, dv1 = oracle.attn_bwd(q, k, v, d_o, 0.3)
    dq2, dk2, dv2 = oracle.attn_bwd(q, kr, vr, d_o, 0.3)
    assert np.array_equal(dq1, dq2)
    assert maxabs(dk1, dk2.reshape(B, T, Hkv, Hq // Hkv, dk).sum(3)) < 2e-6
    assert maxabs(dv1, dv2.reshape(B, T, Hkv, Hq // Hkv, dk).sum(3)) < 2e-6


def test_error_codes(oracle):
    q = np.zeros((6, 4), np.float32)
    with pytest.raises(RuntimeError):  # rows not a multiple of seq_len (ops.cpp:870)
        oracle.head_fwd(q, q, q, 1.0, 4, True, 0, 0)
    with pytest.raises(RuntimeError):  # a window without causal has no reference meaning
        oracle.head_fwd(q, q, q, 1.0, 0, False, 2, 0)
