"""Write tests/golden/llama_cfg5_loss.json: the loss of the COMPILED REFERENCE (nn::Llama, src/llama.cpp) on
BASELINE config 5 at its full size -- 6 layers, d_model 512, 8 heads, d_ff 1376, vocab 32000 tied, B=8 x T=1024.

    python tests/golden/make_llama_cfg5_loss.py        (build container only; minutes of one CPU core)

The reference's own initial parameters (libstdc++ mt19937 + normal_distribution) are 141 MB and cannot travel, so
the parameters are set from this repository's portable generator instead: parameter i of named_parameters() is
synth.randn(1000 + i, shape, 0.02), norm weights 1.0 (the reference's own choice, src/llama.cpp:14-15,67). Token
ids are synth.randint(9, B*T + 1, vocab), the ones bench.py uses. Only the forward pass is run (checkpointed
blocks, so no [8192, 8192] attention matrix outlives its block): the file holds the scalar loss and the recipe.
"""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.bindings import Reference, RefLlama  # noqa: E402
from paperkiln_amd import synth  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
CFG = dict(vocab=32000, d=512, n_layers=6, n_heads=8, d_ff=1376)
B, T = 8, 1024


def cfg5_params(names, shapes):
    """the parameter recipe, shared with tests/test_llama_gpu.py"""
    out = {}
    for i, (n, s) in enumerate(zip(names, shapes)):
        is_norm = n.endswith("norm.weight") or n.endswith("layernorm.weight") or n == "norm.weight"
        out[n] = np.ones(s, np.float32) if is_norm else synth.randn(1000 + i, s, 0.02)
    return out


def main():
    ref = Reference()
    m = RefLlama(ref, n_ctx=T, seed=0, **CFG)
    params = cfg5_params(m.names, m.shapes)
    m.set_params(params)
    toks = synth.randint(9, B * T + 1, CFG["vocab"])
    t0 = time.time()
    loss, _, _ = m.loss_backward(toks[:-1], toks[1:], T, checkpoint=True, backward=False)
    out = {"loss": float(np.float32(loss)), "cfg": CFG, "B": B, "T": T, "ids": "synth.randint(9, B*T + 1, vocab)",
           "params": "named_parameters()[i] = synth.randn(1000 + i, shape, 0.02); norm weights 1.0",
           "names": m.names, "shapes": [list(s) for s in m.shapes], "seconds": round(time.time() - t0, 1)}
    json.dump(out, open(os.path.join(HERE, "llama_cfg5_loss.json"), "w"), indent=1)
    print("config 5 loss", loss, "in", out["seconds"], "s")


if __name__ == "__main__":
    main()
