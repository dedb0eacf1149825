import glob
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (plain-C restatement). Built on demand; test infrastructure only."""
    so = os.path.join(ROOT, "oracle", "libpk_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "libpk_oracle.so"])
    from oracle.bindings import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The compiled reference, or skip where oracle/_ref was not built."""
    from oracle.bindings import load_reference
    ref = load_reference()
    if ref is None:
        pytest.skip("oracle/_ref/libpk_ref.so not built (reference tree absent)")
    return ref


def golden_names():
    names = sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))
    # model-level and block-op vectors have their own loaders
    return [n for n in names if not n.startswith(("llama_", "blockops_"))]


class Golden:
    def __init__(self, name):
        z = np.load(os.path.join(GOLDEN, name + ".npz"))
        self.name = name
        (self.B, self.T, self.Hq, self.Hkv, self.dk, causal, self.window, self.sinks, bf16, self.seed) = \
            (int(x) for x in z["meta"])
        self.causal, self.bf16 = bool(causal), bool(bf16)
        self.scale = float(z["scale"])
        for key in ("q", "k", "v", "d_o", "o", "lse", "dq", "dk", "dv"):
            setattr(self, key, z[key])


@pytest.fixture(params=golden_names())
def golden(request):
    return Golden(request.param)
