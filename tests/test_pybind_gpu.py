"""The pybind11 module paperkiln_amd._paperkiln: the additive Python surface over the C++ tape (the reference's
python/bindings.cpp binds none of fused_attention, swa_attention, checkpoint or Llama). Built by
__graft_entry__.build(). Mirrors how the reference's module is used: numpy float32 in, Variables, backward(),
numpy float32 out."""
import os

import numpy as np
import pytest

from paperkiln_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def module():
    from paperkiln_amd import _paperkiln
    return _paperkiln


def test_module_surface():
    m = module()
    for name in ("Variable", "tensor", "backward", "zero_grad", "checkpoint", "live_variables", "Llama", "init"):
        assert hasattr(m, name), name
    for name in ("fused_attention", "swa_attention", "attention_qkv", "rmsnorm", "silu", "add", "mul", "linear",
                 "cross_entropy"):
        assert hasattr(m.ops, name), name


def maxabs(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max())


@pytest.mark.gpu
@pytest.mark.parametrize("window,sinks", [(0, 0), (9, 2)])
def test_attention_ops_against_the_oracle(oracle, window, sinks):
    m = module()
    m.init(0)
    T, dk, sl = 96, 32, 48
    hq, hk, hv, hg = (synth.randn(s, (T, dk), 1.0) for s in (1, 2, 3, 4))
    q, k, v = (m.tensor(x, requires_grad=True) for x in (hq, hk, hv))
    if window:
        y = m.ops.swa_attention(q, k, v, 0.2, window, sinks, sl)
    else:
        y = m.ops.fused_attention(q, k, v, 0.2, seq_len=sl, causal=True)
    assert y.shape == (T, dk) and y.requires_grad
    # a scalar root whose gradient with respect to y is known: mean cross-entropy over the rows of y * g
    targets = [int(i * 5 % dk) for i in range(T)]
    loss = m.ops.cross_entropy(m.ops.mul(y, m.tensor(hg)), targets)
    m.backward(loss)
    want_y, _, A = oracle.head_fwd(hq, hk, hv, 0.2, sl, True, window, sinks)
    z = want_y.astype(np.float64) * hg
    p = np.exp(z - z.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    p[np.arange(T), targets] -= 1.0
    dy = (p / T * hg).astype(np.float32)
    dq, dk_, dv = oracle.head_bwd(hq, hk, hv, A, dy, 0.2, sl, True, window, sinks)
    assert maxabs(y.data, want_y) < 1e-5
    assert max(maxabs(q.grad, dq), maxabs(k.grad, dk_), maxabs(v.grad, dv)) < 1e-5
    with pytest.raises(RuntimeError, match="window must be >= 1"):
        m.ops.swa_attention(q, k, v, 0.2, 0, 0, 0)
    with pytest.raises(RuntimeError, match="not a multiple of seq_len"):
        m.ops.fused_attention(q, k, v, 0.2, seq_len=7)


@pytest.mark.gpu
def test_checkpoint_with_a_python_segment():
    """checkpoint(fn, x) with fn a Python callable: same loss and gradients as the plain tape, fewer live
    Variables after the forward (tests/test_checkpointing.cpp:46-90)."""
    m = module()
    m.init(0)
    T, d = 64, 32
    hx, hw, hg = synth.randn(11, (T, d), 1.0), synth.randn(12, (d, d), 0.2), np.ones((1, d), np.float32)
    targets = [int(i * 3 % d) for i in range(T)]

    def run(ckpt):
        base = m.live_variables()
        x = m.tensor(hx, requires_grad=True)
        w = m.tensor(hw, requires_grad=True, is_param=True)
        g = m.tensor(hg, requires_grad=True, is_param=True)

        def block(h):
            p = m.ops.linear(m.ops.rmsnorm(h, g), w)
            return m.ops.add(h, m.ops.silu(m.ops.fused_attention(p, p, p, 0.18, seq_len=32, causal=True)))

        h = x
        for _ in range(3):
            h = m.checkpoint(block, h) if ckpt else block(h)
        loss = m.ops.cross_entropy(h, targets)
        del h
        live = m.live_variables() - base
        m.backward(loss)
        return float(loss.data[0, 0]), x.grad, w.grad, g.grad, live

    plain, ck = run(False), run(True)
    assert plain[0] == ck[0]
    for a, b in zip(plain[1:4], ck[1:4]):
        assert maxabs(a, b) < 1e-6
    assert ck[4] * 2 < plain[4]


@pytest.mark.gpu
def test_llama_class_against_the_reference_vectors():
    m = module()
    m.init(0)
    z = np.load(os.path.join(GOLDEN, "llama_T16x2_stacked.npz"))
    vocab, d, L, H, dff = (int(x) for x in z["cfg"])
    model = m.Llama(vocab, d, L, H, dff)
    model.load_state_dict({k[2:]: z[k] for k in z.files if k.startswith("p:")})
    loss, stats = model.loss_backward([int(i) for i in z["ids"]], [int(t) for t in z["targets"]], int(z["seq_len"]),
                                      checkpoint_blocks=True)
    assert abs(loss - float(z["loss"])) < 1e-5
    grads = model.grads()
    assert max(maxabs(grads[k[2:]], z[k]) for k in z.files if k.startswith("g:")) < 1e-5
    assert stats["peak_activation_bytes"] > 0
    assert model.adamw_step(3e-3, max_norm=1.0) == pytest.approx(float(z["total_norm"]), abs=1e-4)


@pytest.mark.gpu
def test_bf16_llama_class_gradients_against_the_reference_vectors():
    """The bf16 model through the pybind class: loss within 2e-2 of the reference, every gradient tensor (plain and
    checkpointed) within 2e-2 of its largest reference entry."""
    m = module()
    m.init(0)
    z = np.load(os.path.join(GOLDEN, "llama_T16x2_stacked.npz"))
    vocab, d, L, H, dff = (int(x) for x in z["cfg"])
    model = m.Llama(vocab, d, L, H, dff, compute_dtype="bf16")
    model.load_state_dict({k[2:]: z[k] for k in z.files if k.startswith("p:")})
    for ckpt in (False, True):
        loss, _ = model.loss_backward([int(i) for i in z["ids"]], [int(t) for t in z["targets"]], int(z["seq_len"]),
                                      checkpoint_blocks=ckpt)
        assert abs(loss - float(z["loss"])) < 2e-2
        grads = model.grads()
        for k in z.files:
            if k.startswith("g:"):
                bar = 2e-2 * float(np.abs(z[k]).max())
                assert maxabs(grads[k[2:]], z[k]) <= bar, (k, ckpt)
