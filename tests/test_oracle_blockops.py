"""CPU tests that pin the oracle's Llama block ops (oracle/pk_oracle.c):
against vectors the compiled reference wrote (tests/golden/blockops_fp32.npz,
llama_*.npz), against the compiled reference itself where it is present, and
against what the mathematics fixes (fp64 finite differences, closed forms,
invariants) -- each chosen so that a dropped term, a wrong sign or a wrong
index fails one of them.
"""
from __future__ import annotations

import os

import numpy as np
import pytest

from paperkiln_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# the reference build contracts a*b+c into FMAs, the oracle does not: a few ulp
TOL = 3e-6


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(GOLDEN, "blockops_fp32.npz"))


def close(a, b, tol=TOL):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    assert a.shape == b.shape
    err = np.abs(a - b).max()
    assert err <= tol * max(1.0, np.abs(b).max()), err


# ---- against the reference's vectors --------------------------------------------------------

def test_rmsnorm_vs_reference_vectors(oracle, vec):
    y, _, dx, dw = oracle.rmsnorm(vec["rms_x"], vec["rms_w"], vec["rms_dy"])
    close(y, vec["rms_y"])
    close(dx, vec["rms_dx"])
    close(dw, vec["rms_dw"], 1e-5)  # a 24-term column sum


def test_silu_vs_reference_vectors(oracle, vec):
    y, dx = oracle.silu(vec["silu_x"], vec["silu_dy"])
    close(y, vec["silu_y"])
    close(dx, vec["silu_dx"])


def test_rope_vs_reference_vectors(oracle, vec):
    th, hd = float(vec["rope_theta"]), int(vec["rope_head_dim"])
    close(oracle.rope(vec["rope_x"], vec["rope_pos"], th, hd), vec["rope_y"])
    close(oracle.rope(vec["rope_dy"], vec["rope_pos"], th, hd, inverse=True), vec["rope_dx"])


def test_cross_entropy_vs_reference_vectors(oracle, vec):
    loss, dl = oracle.cross_entropy(vec["ce_logits"], vec["ce_targets"])
    assert abs(loss - float(vec["ce_loss"])) < 2e-6 * abs(float(vec["ce_loss"]))
    close(dl, vec["ce_dlogits"])


def test_embedding_vs_reference_vectors(oracle, vec):
    y, dt = oracle.embedding(vec["emb_table"], vec["emb_ids"], vec["emb_dy"])
    assert np.array_equal(y, vec["emb_y"])
    close(dt, vec["emb_dtable"])


@pytest.mark.parametrize("name", ["llama_T16_single", "llama_T16x2_stacked"])
def test_clip_and_adamw_vs_reference_optimiser(oracle, name):
    """The reference's own clip_grad_norm + AdamW::step turned p: into a: given g:."""
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    names = [k[2:] for k in z.files if k.startswith("p:")]
    grads = [z["g:" + n] for n in names]
    total, clipped = oracle.clip_grad_norm(grads, 1.0)
    assert abs(total - float(z["total_norm"])) < 1e-6 * float(z["total_norm"])
    worst = 0.0
    for n, g in zip(names, clipped):
        p0 = z["p:" + n]
        p1, _, _ = oracle.adamw(p0, g.reshape(p0.shape), np.zeros_like(p0), np.zeros_like(p0), lr=3e-3, t=1)
        # the first Adam step is g/(|g|+eps): where |g| is within a few eps of 0 an ulp of g moves it
        ok = np.abs(g.reshape(p0.shape)) > 1e-6
        worst = max(worst, np.abs(p1 - z["a:" + n])[ok].max())
    assert worst < 1e-6, worst


# ---- against the compiled reference on other inputs -------------------------------------------

def test_block_ops_vs_compiled_reference(oracle, reference):
    if reference is None:
        pytest.skip("compiled reference not built here")
    x = synth.randn(201, (7, 33), 2.0)
    w = synth.randn(202, (33,), 1.0)
    dy = synth.randn(203, (7, 33), 1.0)
    ry, rdx, rdw = reference.rmsnorm(x, w.reshape(1, -1), dy)
    y, _, dx, dw = oracle.rmsnorm(x, w, dy)
    close(y, ry), close(dx, rdx), close(dw, rdw, 1e-5)
    ry, rdx = reference.silu(x, dy)
    y, dx = oracle.silu(x, dy)
    close(y, ry), close(dx, rdx)
    qkv = synth.randn(204, (9, 3 * 24), 1.0)
    pos = np.array([0, 1, 2, 3, 4, 0, 1, 2, 3], np.int32)
    g = synth.randn(205, (9, 72), 1.0)
    for hd, th in ((24, 10000.0), (6, 1e6), (2, 500.0)):
        ry, rdx = reference.apply_rope(qkv, pos, th, hd, g)
        close(oracle.rope(qkv, pos, th, hd), ry)
        close(oracle.rope(g, pos, th, hd, inverse=True), rdx)
    logits = synth.randn(206, (5, 17), 3.0)
    t = synth.randint(207, 5, 17)
    rl, rdl = reference.cross_entropy(logits, t)
    l, dl = oracle.cross_entropy(logits, t)
    assert abs(l - rl) < 2e-6 * abs(rl)
    close(dl, rdl)


# ---- what the mathematics fixes ----------------------------------------------------------------

def _fd(f, x, eps=1e-3):
    g = np.zeros_like(x, np.float64)
    for i in np.ndindex(x.shape):
        xp, xm = x.astype(np.float64).copy(), x.astype(np.float64).copy()
        xp[i] += eps
        xm[i] -= eps
        g[i] = (f(xp) - f(xm)) / (2 * eps)
    return g


def test_rmsnorm_backward_is_the_gradient(oracle):
    x = synth.randn(301, (3, 6), 1.0)
    w = (1.0 + 0.3 * synth.randn(302, (6,), 1.0)).astype(np.float32)
    dy = synth.randn(303, (3, 6), 1.0)

    def loss(xx, ww):
        r = 1.0 / np.sqrt((xx * xx).mean(axis=1, keepdims=True) + 1e-5)
        return float((xx * r * ww * dy).sum())

    _, _, dx, dw = oracle.rmsnorm(x, w, dy)
    assert np.abs(dx - _fd(lambda a: loss(a, w.astype(np.float64)), x)).max() < 5e-5
    assert np.abs(dw - _fd(lambda a: loss(x.astype(np.float64), a), w)).max() < 5e-5


def test_rmsnorm_unit_rows(oracle):
    """w = 1 and eps -> 0: every output row has mean square 1; scaling a row does not change it."""
    x = synth.randn(304, (4, 32), 3.0)
    y, ri = oracle.rmsnorm(x, np.ones(32, np.float32), eps=0.0)
    assert np.abs((y.astype(np.float64) ** 2).mean(axis=1) - 1.0).max() < 1e-5
    y2, _ = oracle.rmsnorm(7.0 * x, np.ones(32, np.float32), eps=0.0)
    assert np.abs(y2 - y).max() < 1e-5
    assert np.abs(ri - 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1))).max() < 1e-5


def test_silu_backward_is_the_derivative(oracle):
    x = np.linspace(-8, 8, 41, dtype=np.float32).reshape(1, -1)
    y, dx = oracle.silu(x, np.ones_like(x))
    f = lambda a: a / (1.0 + np.exp(-a))  # noqa: E731
    num = (f(x.astype(np.float64) + 1e-4) - f(x.astype(np.float64) - 1e-4)) / 2e-4
    assert np.abs(dx - num).max() < 1e-5
    assert abs(float(oracle.silu(np.zeros((1, 1), np.float32))[0, 0])) == 0.0
    assert np.abs(y[0, -1] - 8.0 / (1.0 + np.exp(-8.0))) < 1e-6


def test_rope_is_a_rotation_of_the_first_head_only(oracle):
    d, hd, T = 24, 6, 5
    x = synth.randn(311, (T, 3 * d), 1.0)
    pos = np.array([0, 1, 2, 7, 300], np.int32)
    y = oracle.rope(x, pos, 10000.0, hd)
    # position 0 is the identity; v third and heads 1.. of q and k are untouched (the reference's loop bound)
    assert np.array_equal(y[0], x[0])
    assert np.array_equal(y[:, 2 * d:], x[:, 2 * d:])
    assert np.array_equal(y[:, hd:d], x[:, hd:d]) and np.array_equal(y[:, d + hd:2 * d], x[:, d + hd:2 * d])
    # each adjacent pair keeps its norm and turns by pos * theta^(-2j/hd)
    for start in (0, d):
        for j in range(hd // 2):
            a, b = x[:, start + 2 * j].astype(np.float64), x[:, start + 2 * j + 1].astype(np.float64)
            c, s = y[:, start + 2 * j].astype(np.float64), y[:, start + 2 * j + 1].astype(np.float64)
            assert np.abs((a * a + b * b) - (c * c + s * s)).max() < 1e-5
            ang = pos.astype(np.float64) * 10000.0 ** (-2.0 * j / hd)
            assert np.abs(c - (a * np.cos(ang) - b * np.sin(ang))).max() < 2e-4  # fp32 angle at pos 300
            assert np.abs(s - (a * np.sin(ang) + b * np.cos(ang))).max() < 2e-4
    # the backward undoes the forward
    assert np.abs(oracle.rope(y, pos, 10000.0, hd, inverse=True) - x).max() < 1e-5
    with pytest.raises(RuntimeError):
        oracle.rope(x[:, :71], pos, 10000.0, hd)
    with pytest.raises(RuntimeError):
        oracle.rope(x, pos, 10000.0, 5)


def test_cross_entropy_closed_forms(oracle):
    R, Cc = 6, 11
    loss, dl = oracle.cross_entropy(np.zeros((R, Cc), np.float32), np.arange(R) % Cc)
    assert abs(loss - np.log(Cc)) < 1e-6
    assert np.abs(dl.sum(axis=1)).max() < 1e-7
    assert np.abs(dl[0, 0] - (1.0 / Cc - 1.0) / R) < 1e-7 and np.abs(dl[0, 1] - 1.0 / Cc / R) < 1e-8
    # a target with probability below 1e-12 costs exactly -log(1e-12)
    lg = np.zeros((1, 4), np.float32)
    lg[0, 1] = 60.0
    loss, _ = oracle.cross_entropy(lg, np.array([0]))
    assert abs(loss - (-np.log(np.float32(1e-12)))) < 1e-4
    # gradient against fp64 finite differences
    lg = synth.randn(321, (3, 5), 1.5)
    t = np.array([4, 0, 2])

    def f(a):
        a = a - a.max(axis=1, keepdims=True)
        lp = a - np.log(np.exp(a).sum(axis=1, keepdims=True))
        return float(-lp[np.arange(3), t].mean())

    _, dl = oracle.cross_entropy(lg, t)
    assert np.abs(dl - _fd(f, lg)).max() < 1e-5
    with pytest.raises(RuntimeError):
        oracle.cross_entropy(lg, np.array([0, 5, 1]))


def test_embedding_scatter_add(oracle):
    table = synth.randn(331, (6, 4), 1.0)
    ids = np.array([2, 2, 5, 2], np.int32)
    dy = synth.randn(332, (4, 4), 1.0)
    y, dt = oracle.embedding(table, ids, dy)
    assert np.array_equal(y, table[ids])
    want = np.zeros_like(table)
    want[2] = (dy[0] + dy[1]) + dy[3]
    want[5] = dy[2]
    assert np.array_equal(dt, want)
    with pytest.raises(RuntimeError):
        oracle.embedding(table, np.array([6], np.int32))


def test_adamw_first_steps_closed_form(oracle):
    """Step 1 with zero state: m/c1 = g, v/c2 = g^2 -> update = g/(|g|+eps) = sign(g) for |g| >> eps."""
    p = np.array([1.0, -2.0, 0.5, 3.0], np.float32)
    g = np.array([0.3, -0.7, 2.0, -1e-3], np.float32)
    p1, m1, v1 = oracle.adamw(p, g, np.zeros(4, np.float32), np.zeros(4, np.float32), lr=0.1, wd=0.01, t=1)
    want = p.astype(np.float64) - 0.1 * (np.sign(g) + 0.01 * p.astype(np.float64))
    assert np.abs(p1 - want).max() < 2e-6
    assert np.abs(m1 - 0.1 * g).max() < 1e-7 and np.abs(v1 - 0.001 * g * g).max() < 1e-7
    # wd only (g = 0): decoupled decay p *= 1 - lr*wd
    p2, _, _ = oracle.adamw(p, np.zeros(4, np.float32), np.zeros(4, np.float32), np.zeros(4, np.float32), lr=0.1,
                            wd=0.5, t=3)
    assert np.abs(p2 - p * 0.95).max() < 1e-6


def test_clip_grad_norm_scales_to_the_bound(oracle):
    gs = [np.full((2, 2), 3.0, np.float32), np.full(9, 4.0, np.float32)]
    total, clipped = oracle.clip_grad_norm(gs, 1.0)
    assert abs(total - np.sqrt(4 * 9 + 9 * 16)) < 1e-5
    assert abs(np.sqrt(sum(float((c.astype(np.float64) ** 2).sum()) for c in clipped)) - 1.0) < 1e-6
    total, same = oracle.clip_grad_norm(gs, 100.0)  # under the bound: untouched
    assert all(np.array_equal(a, b) for a, b in zip(gs, same))
