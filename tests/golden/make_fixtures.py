"""Write the golden vectors under tests/golden/ from the COMPILED REFERENCE.

Run in the build container only (needs oracle/_ref/libpk_ref.so, i.e.
/root/reference present when `make -C oracle ref` ran):

    python tests/golden/make_fixtures.py

Each .npz holds seeded inputs (paperkiln_amd.synth) and what the reference's
own ops::fused_attention / ops::swa_attention return for them, per head, plus
the logsumexp derived from the reference's own weight matrix A
(LSE_i = scale*s_ij - log A_ij at the row's largest weight; the reference never
stores LSE). The reference has no GQA tape, so GQA expectations are composed
the way its autograd would: one K/V head feeds several head nodes and their
gradients accumulate (src/autograd.cpp:16-24).
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.bindings import Reference  # noqa: E402
from paperkiln_amd import synth  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def lse_from_weights(q, k, A, scale):
    """LSE_i from the reference's A: scale*s_ij - log A_ij at j = argmax_j A_ij."""
    j = A.argmax(axis=1)
    s = (q.astype(np.float64) * k[j].astype(np.float64)).sum(axis=1) * np.float64(np.float32(scale))
    return (s - np.log(A[np.arange(len(j)), j].astype(np.float64))).astype(np.float32)


def run_case(ref, q, k, v, d_o, scale, causal, window, sinks):
    """q,d_o: [B,T,Hq,dk]; k,v: [B,T,Hkv,dk] -> reference o, lse, dq, dk, dv.
    Each head is one reference call on the stacked [B*T, dk] matrix with
    seq_len = T, which is how the reference batches (src/ops.cpp:869-879)."""
    B, T, Hq, dk = q.shape
    Hkv = k.shape[2]
    rep = Hq // Hkv
    o = np.zeros_like(q)
    lse = np.zeros((B, Hq, T), np.float32)
    dq = np.zeros_like(q)
    dkk = np.zeros_like(k)
    dvv = np.zeros_like(v)
    for h in range(Hq):
        qh = q[:, :, h, :].reshape(B * T, dk)
        kh = k[:, :, h // rep, :].reshape(B * T, dk)
        vh = v[:, :, h // rep, :].reshape(B * T, dk)
        gh = d_o[:, :, h, :].reshape(B * T, dk)
        if window:
            y, a, b, c = ref.swa_attention(qh, kh, vh, scale, window, sinks, T, dy=gh)
        else:
            y, a, b, c = ref.fused_attention(qh, kh, vh, scale, T, causal, dy=gh)
        A = ref.weights(qh, kh, scale, T, causal, window, sinks)
        o[:, :, h, :] = y.reshape(B, T, dk)
        lse[:, h, :] = lse_from_weights(qh, kh, A, scale).reshape(B, T)
        dq[:, :, h, :] = a.reshape(B, T, dk)
        dkk[:, :, h // rep, :] += b.reshape(B, T, dk)
        dvv[:, :, h // rep, :] += c.reshape(B, T, dk)
    return o, lse, dq, dkk, dvv


# name: (B, T, Hq, Hkv, dk, scale, causal, window, sinks, input std, round inputs to bf16, seed)
CASES = {
    # BASELINE config 1, in full
    "cfg1_fp32_B2_H4_T128_d32": (2, 128, 4, 4, 32, 1.0 / np.sqrt(32.0), True, 0, 0, 1.0, False, 101),
    # the reference's own gradcheck shapes (tests/test_gradcheck.cpp:197-238): T=8, dk=4, std 0.5
    "gradcheck_causal_T8_d4": (1, 8, 1, 1, 4, 0.5, True, 0, 0, 0.5, False, 61),
    "gradcheck_causal_batch_T4x2_d4": (2, 4, 1, 1, 4, 0.5, True, 0, 0, 0.5, False, 61),
    "gradcheck_bidir_batch_T4x2_d4": (2, 4, 1, 1, 4, 0.5, False, 0, 0, 0.5, False, 61),
    # the reference's own SWA shapes (tests/test_swa.cpp): T=12, dk=4, scale 0.5
    "swa_T12_w4_s1": (1, 12, 1, 1, 4, 0.5, True, 4, 1, 1.0, False, 4),
    "swa_T12_w3_s0": (1, 12, 1, 1, 4, 0.5, True, 3, 0, 1.0, False, 7),
    "swa_T12_w2_s1": (1, 12, 1, 1, 4, 0.5, True, 2, 1, 1.0, False, 10),
    "swa_T12x2_w4_s1": (2, 12, 1, 1, 4, 0.5, True, 4, 1, 1.0, False, 13),
    "swa_T12_w12_s0_equals_causal": (1, 12, 1, 1, 4, 0.5, True, 12, 0, 1.0, False, 1),
    # ragged sizes that straddle every tile edge, sinks wider than the window
    "swa_T97_w5_s7_d16": (3, 97, 2, 2, 16, 0.25, True, 5, 7, 1.0, False, 21),
    "bidir_T70_d24": (2, 70, 2, 2, 24, 0.2, False, 0, 0, 1.0, False, 22),
    # GQA: 4 query heads on 2 KV heads
    "gqa_T64_Hq4_Hkv2_d16": (2, 64, 4, 2, 16, 0.25, True, 0, 0, 1.0, False, 23),
    # bf16-rounded inputs at MFMA head sizes (fp32 reference arithmetic on them)
    "bf16in_causal_T200_H2_d64": (1, 200, 2, 2, 64, 0.125, True, 0, 0, 1.0, True, 31),
    "bf16in_swa_T300_w64_s4_Hq4_Hkv2_d128": (1, 300, 4, 2, 128, 1.0 / np.sqrt(128.0), True, 64, 4, 1.0, True, 32),
}


def make_inputs(B, T, Hq, Hkv, dk, std, bf16, seed):
    q = synth.randn(seed, (B, T, Hq, dk), std)
    k = synth.randn(seed + 1, (B, T, Hkv, dk), std)
    v = synth.randn(seed + 2, (B, T, Hkv, dk), std)
    d_o = synth.randn(seed + 3, (B, T, Hq, dk), 1.0)
    if bf16:
        q, k, v, d_o = (synth.bf16_round(x) for x in (q, k, v, d_o))
    return q, k, v, d_o


def main():
    ref = Reference()
    for name, (B, T, Hq, Hkv, dk, scale, causal, window, sinks, std, bf16, seed) in CASES.items():
        q, k, v, d_o = make_inputs(B, T, Hq, Hkv, dk, std, bf16, seed)
        scale = float(np.float32(scale))
        o, lse, dq, dkk, dvv = run_case(ref, q, k, v, d_o, scale, causal, window, sinks)
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"), q=q, k=k, v=v, d_o=d_o, o=o, lse=lse, dq=dq, dk=dkk, dv=dvv,
            meta=np.array([B, T, Hq, Hkv, dk, int(causal), window, sinks, int(bf16), seed], np.int64),
            scale=np.float32(scale), std=np.float32(std))
        print(f"{name}: |o|max={np.abs(o).max():.3f} |dq|max={np.abs(dq).max():.3f} "
              f"|dk|max={np.abs(dkk).max():.3f} |dv|max={np.abs(dvv).max():.3f}")


if __name__ == "__main__":
    main()
