"""Write tests/golden/blockops_fp32.npz from the COMPILED REFERENCE.

Run in the build container only (needs oracle/_ref/libpk_ref.so):

    python tests/golden/make_blockop_fixtures.py

Seeded inputs (paperkiln_amd.synth) and what the reference's own ops::rmsnorm,
ops::silu, ops::apply_rope, ops::cross_entropy and ops::embedding return for
them, forward and backward. The RoPE case has four heads so that the
reference's first-head-only rotation is visible in the vectors.
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


def main():
    ref = Reference()
    out = {}
    # rmsnorm: [24, 48]
    x = synth.randn(101, (24, 48), 1.3)
    w = (1.0 + 0.1 * synth.randn(102, (48,), 1.0)).astype(np.float32)
    dy = synth.randn(103, (24, 48), 1.0)
    y, dx, dw = ref.rmsnorm(x, w.reshape(1, -1), dy)
    out.update({"rms_x": x, "rms_w": w, "rms_dy": dy, "rms_y": y, "rms_dx": dx, "rms_dw": dw})
    # silu: [16, 40], values out to +-6
    x = synth.randn(111, (16, 40), 2.5)
    dy = synth.randn(112, (16, 40), 1.0)
    y, dx = ref.silu(x, dy)
    out.update({"silu_x": x, "silu_dy": dy, "silu_y": y, "silu_dx": dx})
    # rope: two stacked sequences of 8 tokens, d = 32, head_dim = 8 (4 heads)
    qkv = synth.randn(121, (16, 96), 1.0)
    pos = np.concatenate([np.arange(8), np.arange(8)]).astype(np.int32)
    dy = synth.randn(122, (16, 96), 1.0)
    y, dx = ref.apply_rope(qkv, pos, 10000.0, 8, dy)
    out.update({"rope_x": qkv, "rope_pos": pos, "rope_dy": dy, "rope_y": y, "rope_dx": dx,
                "rope_theta": np.float32(10000.0), "rope_head_dim": np.int32(8)})
    # cross entropy: [12, 40], one row pushed into the 1e-12 clamp
    logits = synth.randn(131, (12, 40), 2.0)
    targets = synth.randint(132, 12, 40).astype(np.int32)
    logits[3, :] = -40.0
    logits[3, (targets[3] + 1) % 40] = 40.0
    loss, dl = ref.cross_entropy(logits, targets)
    out.update({"ce_logits": logits, "ce_targets": targets, "ce_loss": np.float32(loss), "ce_dlogits": dl})
    # embedding: table [20, 8], ids with repeats
    table = synth.randn(141, (20, 8), 0.5)
    ids = np.array([3, 7, 3, 0, 19, 7, 3, 11], np.int32)
    dy = synth.randn(142, (8, 8), 1.0)
    y, dt = ref.embedding(table, ids, dy)
    out.update({"emb_table": table, "emb_ids": ids, "emb_dy": dy, "emb_y": y, "emb_dtable": dt})
    path = os.path.join(HERE, "blockops_fp32.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
