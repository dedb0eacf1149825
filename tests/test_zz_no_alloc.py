"""pk_attn_bwd_static, the backward entry point that allocates nothing (its scratch is a device array inside the
library), through the C ABI against pk_attn_bwd with a caller workspace: same kernels, so the same bits. Each case
makes two calls in a row, the second on a smaller input, because every call on a GPU shares that GPU's array and
finds the previous call's contents in it. Run with -m gpu."""
import ctypes as C

import numpy as np
import pytest
import torch

from paperkiln_amd import _lib, ops

pytestmark = pytest.mark.gpu


def inputs(B, T, Hq, Hkv, dk, dtype, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    mk = lambda h: (torch.randn((B, T, h, dk), generator=gen, device="cuda") * 0.7).to(dtype)
    return mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)


def torch_allocations():
    return torch.cuda.memory_stats().get("allocation.all.allocated", 0)


# (element type, head_dim, window, sinks, first shape (B, T, Hq, Hkv), second and smaller shape)
CASES = [
    (torch.bfloat16, 128, 0, 0, (2, 1024, 4, 2), (1, 300, 2, 2)),     # matrix-core kernels, causal
    (torch.bfloat16, 64, 16, 3, (1, 2048, 2, 1), (1, 1100, 2, 1)),    # split sink tail: the scratch also holds partial rows
    (torch.float32, 64, 40, 2, (1, 1501, 2, 1), (1, 700, 2, 1)),      # fp32 matrix-core kernels, split sink tail
    (torch.float32, 24, 9, 2, (2, 333, 2, 1), (1, 100, 2, 1)),        # scalar kernels
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{str(c[0]).split('.')[-1]}_d{c[1]}_w{c[2]}_s{c[3]}")
def test_static_scratch_backward_equals_workspace_backward(case):
    dtype, dk, window, sinks, big, small = case
    scale = float(1 / np.sqrt(dk))
    for n, (B, T, Hq, Hkv) in enumerate((big, small)):
        q, k, v, d_o = inputs(B, T, Hq, Hkv, dk, dtype, 40 + n)
        o, lse = ops.attn_fwd(q, k, v, scale, True, window, sinks)
        want = ops.attn_bwd(q, k, v, o, lse, d_o, scale, True, window, sinks)
        out = tuple(torch.full_like(x, float("nan")) for x in (q, k, v))
        print(f"\n  static backward, call {n}: {dtype} B={B} T={T} Hq={Hq} Hkv={Hkv} dk={dk} w={window} s={sinks}", flush=True)
        # the property the entry point exists for: nothing is allocated, neither from the library's own pool
        # nor from the device (outputs are passed in, so torch allocates nothing either: its count of
        # allocation requests, which only ever grows, stands still)
        L = _lib.lib()
        torch.cuda.synchronize()
        before = (L.pk_live_bytes(), L.pk_peak_bytes(), torch.cuda.mem_get_info()[0], torch_allocations())
        got = ops.attn_bwd_static(q, k, v, o, lse, d_o, scale, True, window, sinks, out=out)
        torch.cuda.synchronize()
        after = (L.pk_live_bytes(), L.pk_peak_bytes(), torch.cuda.mem_get_info()[0], torch_allocations())
        assert after == before, f"call {n}: the static backward changed an allocation counter: {before} -> {after}"
        for name, a, b in zip(("dQ", "dK", "dV"), got, want):
            assert torch.isfinite(a.float()).all(), name
            assert torch.equal(a, b), f"call {n}: {name}"


def test_static_scratch_limit_is_enforced():
    """A shape whose workspace exceeds the array is refused with PK_ERR_WORKSPACE before anything is launched."""
    L = _lib.lib()
    B, T, H, dk = 8, 1 << 18, 8, 64          # delta alone: 8 * 8 * 2^18 * 4 bytes = 64 MiB > 32 MiB
    sh = _lib.AttnShape(B, T, H, H, dk, 1, 0, 0, 0.125, _lib.PK_BF16, _lib.PK_BF16)
    assert L.pk_attn_bwd_workspace_bytes(C.byref(sh)) > 32 << 20
    t = _lib.Tensor4(1, 0, 0, 0)
    rc = L.pk_attn_bwd_static(C.byref(sh), C.byref(t), C.byref(t), C.byref(t), C.byref(t), C.c_void_p(1), C.byref(t),
                              C.byref(t), C.byref(t), C.byref(t), None)
    assert rc == 3 and b"PK_ATTN_BWD_STATIC_MAX_WORKSPACE" in L.pk_last_error()
