"""GPU parity of the Llama block operators (pk_op_* through the C ABI) against
the vectors the compiled reference wrote (tests/golden/blockops_fp32.npz,
llama_*.npz) and against the CPU oracle on other seeded inputs.

Bars: fp32 storage max-abs 1e-5 (relative to the largest expected magnitude
where values exceed 1: row reductions run in a different order); bf16 storage
2e-2 against the oracle run on the same bf16-rounded inputs.
"""
from __future__ import annotations

import os

import numpy as np
import pytest

from paperkiln_amd import synth

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
F32_TOL = 1e-5
BF16_TOL = 2e-2


@pytest.fixture(scope="module")
def bo():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from paperkiln_amd import _lib, blockops
    _lib.check(_lib.lib().pk_init(0, None, 0))
    return blockops


@pytest.fixture(scope="module")
def vec():
    return np.load(os.path.join(GOLDEN, "blockops_fp32.npz"))


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t.to(dtype) if dtype is not None else t


def host(t):
    return t.float().cpu().numpy()


def close(got, want, tol):
    want = np.asarray(want, np.float64)
    err = np.abs(host(got).astype(np.float64) - want).max()
    assert err <= tol * max(1.0, np.abs(want).max()), err


def test_rmsnorm_fp32_vs_reference_vectors(bo, vec):
    y, dx, dw = bo.rmsnorm(dev(vec["rms_x"]), dev(vec["rms_w"]), dev(vec["rms_dy"]))
    close(y, vec["rms_y"], F32_TOL)
    close(dx, vec["rms_dx"], F32_TOL)
    close(dw, vec["rms_dw"], F32_TOL)


def test_silu_fp32_vs_reference_vectors(bo, vec):
    y, dx = bo.silu(dev(vec["silu_x"]), dev(vec["silu_dy"]))
    close(y, vec["silu_y"], F32_TOL)
    close(dx, vec["silu_dx"], F32_TOL)


def test_rope_fp32_vs_reference_vectors(bo, vec):
    th, hd = float(vec["rope_theta"]), int(vec["rope_head_dim"])
    pos = dev(vec["rope_pos"])
    close(bo.apply_rope(dev(vec["rope_x"]), pos, th, hd), vec["rope_y"], F32_TOL)
    close(bo.apply_rope(dev(vec["rope_dy"]), pos, th, hd, inverse=True), vec["rope_dx"], F32_TOL)


def test_rope_all_heads_switch(bo, oracle, vec):
    """all_heads=True rotates every head the way the first one is rotated; the default leaves them alone."""
    th, hd = float(vec["rope_theta"]), int(vec["rope_head_dim"])
    x, pos = vec["rope_x"], vec["rope_pos"]
    d = x.shape[1] // 3
    want = x.copy()
    for third in (0, 1):
        for h in range(d // hd):
            blk = np.zeros_like(x)
            c0 = third * d + h * hd
            blk[:, :hd] = x[:, c0:c0 + hd]  # put the head where the reference's loop rotates
            want[:, c0:c0 + hd] = oracle.rope(blk, pos, th, hd)[:, :hd]
    close(bo.apply_rope(dev(x), dev(pos), th, hd, all_heads=True), want, F32_TOL)


def test_cross_entropy_fp32_vs_reference_vectors(bo, vec):
    loss, dl = bo.cross_entropy(dev(vec["ce_logits"]), dev(vec["ce_targets"]))
    assert abs(loss - float(vec["ce_loss"])) < 1e-5 * abs(float(vec["ce_loss"]))
    close(dl, vec["ce_dlogits"], F32_TOL)


def test_embedding_vs_reference_vectors(bo, vec):
    y, dt = bo.embedding(dev(vec["emb_table"]), dev(vec["emb_ids"]), dev(vec["emb_dy"]))
    assert np.array_equal(host(y), vec["emb_y"])
    close(dt, vec["emb_dtable"], F32_TOL)


def test_embedding_gradient_is_summed_in_row_order(bo, oracle):
    """Heavily repeated ids (3000 rows over 7 table rows, a table far larger than the row count, and 8192 rows
    that all name one id, the longest run there can be): the scatter-add forms each table row's sum in ascending
    row order, as the reference's loop does (src/ops.cpp:338-347), so it equals the CPU restatement bit for bit
    and is the same on every run."""
    for vocab, n, d, seed in ((7, 3000, 48, 51), (40_000, 257, 48, 52), (1, 8192, 512, 53), (3, 1001, 130, 54)):
        table = synth.randn(seed, (vocab, d), 0.5)
        ids = synth.randint(seed + 100, n, vocab).astype(np.int32)
        g = synth.randn(seed + 200, (n, d), 1.0)
        _, want = oracle.embedding(table, ids, g)
        runs = [host(bo.embedding(dev(table), dev(ids), dev(g))[1]) for _ in range(3)]
        assert np.array_equal(runs[0], want)
        assert np.array_equal(runs[1], runs[0]) and np.array_equal(runs[2], runs[0])


@pytest.mark.parametrize("name", ["llama_T16_single"])
def test_clip_and_adamw_vs_reference_optimiser(bo, name):
    z = np.load(os.path.join(GOLDEN, name + ".npz"))
    names = [k[2:] for k in z.files if k.startswith("p:")]
    grads = [dev(z["g:" + n]).reshape(-1).contiguous() for n in names]
    total = bo.clip_grad_norm_(grads, 1.0)
    assert abs(total - float(z["total_norm"])) < 1e-5 * float(z["total_norm"])
    worst = 0.0
    for n, g in zip(names, grads):
        p = dev(z["p:" + n]).reshape(-1).contiguous()
        bo.adamw_(p, g, torch.zeros_like(p), torch.zeros_like(p), lr=3e-3, t=1)
        ok = np.abs(host(g)) > 1e-5  # the first Adam step is g/(|g|+eps): ill-conditioned at |g| ~ eps
        worst = max(worst, np.abs(host(p) - z["a:" + n].reshape(-1))[ok].max())
    assert worst < F32_TOL, worst


@pytest.mark.parametrize("dtype,tol", [("float32", F32_TOL), ("bfloat16", BF16_TOL)])
def test_block_ops_vs_oracle_larger(bo, oracle, dtype, tol):
    """Shapes of a real block (rows not a multiple of the kernels' row groups), both storage types."""
    td = getattr(torch, dtype)
    rnd = (lambda a: synth.bf16_round(a)) if dtype == "bfloat16" else (lambda a: a)
    R, Cc = 301, 512
    x, dy = rnd(synth.randn(401, (R, Cc), 1.5)), rnd(synth.randn(402, (R, Cc), 1.0))
    w = (1.0 + 0.2 * synth.randn(403, (Cc,), 1.0)).astype(np.float32)
    wy, _, wdx, wdw = oracle.rmsnorm(x, w, dy)
    y, dx, dw = bo.rmsnorm(dev(x, td), dev(w), dev(dy, td))
    close(y, wy, tol), close(dx, wdx, tol)
    close(dw, wdw, tol if dtype == "float32" else 5e-2)  # a 301-term column sum of bf16-rounded products
    wy, wdx = oracle.silu(x, dy)
    y, dx = bo.silu(dev(x, td), dev(dy, td))
    close(y, wy, tol), close(dx, wdx, tol)
    # silu(gate) .* up as one node: the product rule over the oracle's silu
    up = rnd(synth.randn(412, (R, Cc), 1.0))
    sy, sdx = oracle.silu(x, np.ones_like(x))  # sdx = silu'(x)
    y, dgate, dup = bo.silu_mul(dev(x, td), dev(up, td), dev(dy, td))
    close(y, sy * up, tol), close(dgate, dy * up * sdx, tol), close(dup, dy * sy, tol)
    a, b = rnd(synth.randn(404, (R, Cc), 1.0)), rnd(synth.randn(405, (R, Cc), 1.0))
    close(bo.add(dev(a, td), dev(b, td)), a + b, tol)
    close(bo.mul(dev(a, td), dev(b, td)), a * b, tol)
    close(bo.scale(dev(a, td), 0.37), a * np.float32(0.37), tol)
    close(bo.axpy_(dev(a, td), -1.5, dev(b, td)), a + np.float32(-1.5) * b, tol)
    assert float(bo.fill_(dev(a, td), 2.5).float().min()) == 2.5
    # rope on a Llama-shaped fused projection: 2 x 150 positions, d = 512, head_dim = 64
    qkv = rnd(synth.randn(406, (300, 3 * 512), 1.0))
    pos = np.concatenate([np.arange(150), np.arange(150)]).astype(np.int32)
    close(bo.apply_rope(dev(qkv, td), dev(pos), 10000.0, 64), oracle.rope(qkv, pos, 10000.0, 64), tol)
    # cross entropy over a 1000-word vocabulary
    lg = rnd(synth.randn(407, (97, 1000), 2.0))
    t = synth.randint(408, 97, 1000).astype(np.int32)
    wl, wdl = oracle.cross_entropy(lg, t)
    loss, dl = bo.cross_entropy(dev(lg, td), dev(t))
    assert abs(loss - wl) < (1e-5 if dtype == "float32" else 1e-3) * abs(wl)
    close(dl, wdl, tol if dtype == "float32" else 1e-3)  # |dlogits| <= 1/97
    # embedding into either storage type
    table = synth.randn(409, (500, 64), 0.5)
    ids = synth.randint(410, 333, 500).astype(np.int32)
    g = rnd(synth.randn(411, (333, 64), 1.0))
    wy, wdt = oracle.embedding(table, ids, g)
    y, dt = bo.embedding(dev(table), dev(ids), dev(g, td), dtype=td)
    close(y, rnd(wy), tol), close(dt, wdt, 1e-5)


def test_matmul_vs_numpy(bo):
    a, b = synth.randn(421, (65, 130), 1.0), synth.randn(422, (130, 47), 1.0)
    want = a.astype(np.float64) @ b.astype(np.float64)
    close(bo.matmul(dev(a), dev(b)), want, 2e-5)
    close(bo.matmul(dev(a.T.copy()), dev(b), trans_a=True), want, 2e-5)
    close(bo.matmul(dev(a), dev(b.T.copy()), trans_b=True), want, 2e-5)
    ab, bb = synth.bf16_round(a), synth.bf16_round(b)
    close(bo.matmul(dev(ab, torch.bfloat16), dev(bb, torch.bfloat16), out_dtype=torch.float32),
          ab.astype(np.float64) @ bb.astype(np.float64), 2e-5)
    with pytest.raises(RuntimeError):
        bo.matmul(dev(a), dev(a))


def test_weight_gradient_gemm_long_contraction(bo):
    """dW += X^T dY over 4096 tokens takes the sliced path (partial products added in slice order): same
    result as one product, and the same bits on every run."""
    import ctypes as C
    from paperkiln_amd import _lib
    x, dy = synth.bf16_round(synth.randn(441, (4096, 96), 1.0)), synth.bf16_round(synth.randn(442, (4096, 160), 1.0))
    g0 = synth.randn(443, (96, 160), 1.0)
    want = g0.astype(np.float64) + x.astype(np.float64).T @ dy.astype(np.float64)
    outs = []
    for _ in range(2):
        g = dev(g0)
        tx, tdy = dev(x, torch.bfloat16), dev(dy, torch.bfloat16)
        _lib.check(_lib.lib().pk_op_gemm(C.c_void_p(tx.data_ptr()), 1, C.c_void_p(tdy.data_ptr()), 0,
                                         C.c_void_p(g.data_ptr()), 96, 160, 4096, _lib.PK_BF16, _lib.PK_F32, 1,
                                         C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        outs.append(host(g))
    assert np.abs(outs[0] - want).max() < 2e-4 * np.abs(want).max()  # fp32 accumulation over 4096 terms
    assert np.array_equal(outs[0], outs[1])
    # the same slicing for a plain product with a long inner dimension and a bf16 result (dh = dlogits E)
    a, b = synth.bf16_round(synth.randn(444, (130, 4096), 0.1)), synth.bf16_round(synth.randn(445, (4096, 72), 1.0))
    want = a.astype(np.float64) @ b.astype(np.float64)
    got = bo.matmul(dev(a, torch.bfloat16), dev(b, torch.bfloat16))
    close(got, synth.bf16_round(want.astype(np.float32)), 1e-2)
    close(bo.matmul(dev(a, torch.bfloat16), dev(b, torch.bfloat16), out_dtype=torch.float32), want, 2e-4)


def test_error_behaviour(bo):
    x = dev(synth.randn(431, (4, 8), 1.0))
    with pytest.raises(RuntimeError):
        bo.rmsnorm(x, dev(np.ones(7, np.float32)))
    with pytest.raises(RuntimeError):
        bo.apply_rope(x, dev(np.arange(4, dtype=np.int32)), 10000.0, 2)  # 8 columns: not divisible by 3
    with pytest.raises(RuntimeError):
        bo.apply_rope(dev(synth.randn(432, (4, 12), 1.0)), dev(np.arange(4, dtype=np.int32)), 10000.0, 3)  # odd head_dim
    with pytest.raises(RuntimeError):
        bo.embedding(x, dev(np.array([4], np.int32)))
    with pytest.raises(RuntimeError):
        bo.cross_entropy(x, dev(np.array([0, 1, 8, 2], np.int32)))
    with pytest.raises(RuntimeError):
        bo.add(x, dev(synth.randn(433, (4, 9), 1.0)))


def test_allocator_recycles_a_block_behind_the_stream_that_used_it_last(bo):
    """A block from pk_alloc that a C-ABI call used on stream S is cached, once freed, for S and not for the stream of
    whoever frees it: an allocation for the null stream made while S still has work queued must not get that block
    back; once S is idle the block may be taken over. (S is kept busy with a long chain of fills on a large
    buffer; the check is skipped if the stream has drained by the time the allocation is made.)"""
    import ctypes as C
    from paperkiln_amd import _lib
    L = _lib.lib()
    n = 64 << 20
    side = torch.cuda.Stream()
    big = torch.empty(1 << 28, dtype=torch.float32, device="cuda")   # 1 GiB: each fill takes a fraction of a millisecond
    p = C.c_void_p()
    _lib.check(L.pk_alloc(n, C.byref(p)))
    first = p.value
    torch.cuda.synchronize()
    S = C.c_void_p(side.cuda_stream)
    with torch.cuda.stream(side):
        for _ in range(40):
            big.fill_(1.0)
    _lib.check(L.pk_op_fill(p, 2.0, n // 4, _lib.PK_F32, S))       # queued on S behind the fills
    _lib.check(L.pk_free(p))                                         # freed by a thread whose own stream is the null stream
    q = C.c_void_p()
    _lib.check(L.pk_alloc(n, C.byref(q)))                            # for the null stream
    still_busy = not side.query()
    if still_busy:
        assert q.value != first, "a block whose last user is still running was handed to another stream"
    torch.cuda.synchronize()
    _lib.check(L.pk_free(q))
    r = C.c_void_p()
    _lib.check(L.pk_alloc(n, C.byref(r)))                            # S is idle now: either cached block may come back
    assert r.value in (first, q.value)
    _lib.check(L.pk_free(r))
    if not still_busy:
        pytest.skip("the side stream drained before the allocation; only the take-over path was exercised")


GEMM_SHAPES = [(128, 128, 64), (560, 136, 200), (8, 8, 8), (2056, 520, 1376), (512, 1536, 4096), (264, 40, 8192),
               (1000, 2048, 512), (300, 264, 72), (8192, 2752, 72), (4096, 4096, 136)]


@pytest.mark.parametrize("mode", [3, 4, 5, 6, 8, 9, 11, 2],
                         ids=["tiles128", "tiles256", "ring128x4", "ring128x2", "ring256", "ring128_two_sets",
                              "ring128_two_sets_x4", "by_shape"])
@pytest.mark.parametrize("shape", GEMM_SHAPES, ids=lambda s: f"M{s[0]}_N{s[1]}_K{s[2]}")
def test_matrix_core_gemm_against_float64(bo, mode, shape):
    """The library's own bf16 GEMM (the counterpart of the reference's tiled kernel with transpose flags,
    src/cuda_resident.cu:141-171) in every form it has -- register-staged tiles and the persistent LDS-ring kernel,
    both tile geometries, ring depths 2 and 4, one and two wavefront sets per tile, and the form the library picks by
    shape -- all four transpose combinations, bf16 and fp32 results, overwrite and accumulate, ragged edges,
    contractions that are not a multiple of the slice, long ones that are split across workgroups, and outputs of more
    tiles than the chip holds workgroups (so that a workgroup walks several tiles with its loads running ahead across
    the tile boundary) -- against a float64 product of the same bf16 operands. The bar: the fp32 accumulation
    error of a K-term sum (a few 1e-6 relative to the largest |C|, the library kernel's own distance is printed beside
    it), plus one bf16 rounding where the result is stored in bf16. Two runs give the same bits."""
    M, N, K = shape
    gen = torch.Generator(device="cuda").manual_seed(M + 3 * N + 7 * K)
    prev = bo.set_gemm_backend(mode)
    try:
        for ta in (False, True):
            for tb in (False, True):
                a = torch.randn((K, M) if ta else (M, K), generator=gen, device="cuda").bfloat16()
                b = torch.randn((N, K) if tb else (K, N), generator=gen, device="cuda").bfloat16()
                want = (a.double().t() if ta else a.double()) @ (b.double().t() if tb else b.double())
                scale = float(want.abs().max())
                for od in (torch.float32, torch.bfloat16):
                    got = bo.matmul(a, b, ta, tb, out_dtype=od)
                    again = bo.matmul(a, b, ta, tb, out_dtype=od)
                    assert torch.equal(got, again)
                    err = float((got.double() - want).abs().max())
                    bar = scale * (2e-5 + (2.0 ** -8 if od == torch.bfloat16 else 0.0))
                    assert err <= bar, (ta, tb, od, err, bar)
                    c0 = torch.randn((M, N), generator=gen, device="cuda").to(od)
                    acc = c0.clone()
                    bo.matmul(a, b, ta, tb, out=acc)
                    want_acc = c0.double() + want
                    err = float((acc.double() - want_acc).abs().max())
                    bar = float(want_acc.abs().max()) * (2e-5 + (2.0 ** -7 if od == torch.bfloat16 else 0.0))
                    assert err <= bar, ("accumulate", ta, tb, od, err, bar)
    finally:
        bo.set_gemm_backend(prev)


def test_matrix_core_gemm_under_graph_capture(bo):
    """The persistent GEMM allocates nothing, clears nothing and keeps no state between launches, so a caller can record
    it into a HIP graph: a product of several tiles per workgroup, one of a single tile per workgroup with the two-set
    form, and an accumulating one, replayed three times with fresh operands copied into the captured tensors and eager
    products in between; every replay equals the eager product of the same operands bit for bit."""
    gen = torch.Generator(device="cuda").manual_seed(17)
    cases = [(8192, 2752, 512, False, False, torch.bfloat16), (2048, 512, 1536, False, True, torch.bfloat16),
             (1024, 768, 264, True, False, torch.float32)]
    prev = bo.set_gemm_backend(2)
    try:
        for M, N, K, ta, tb, od in cases:
            a = torch.randn((K, M) if ta else (M, K), generator=gen, device="cuda").bfloat16()
            b = torch.randn((N, K) if tb else (K, N), generator=gen, device="cuda").bfloat16()
            acc = torch.zeros((M, N), dtype=od, device="cuda")
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):  # warm-up outside the capture, as torch asks
                bo.matmul(a, b, ta, tb, out_dtype=od)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                c = bo.matmul(a, b, ta, tb, out_dtype=od)
                bo.matmul(a, b, ta, tb, out=acc)
            acc.zero_()
            total = torch.zeros_like(acc)
            for rep in range(3):
                fa, fb = torch.randn_like(a.float()).bfloat16(), torch.randn_like(b.float()).bfloat16()
                a.copy_(fa)
                b.copy_(fb)
                graph.replay()
                torch.cuda.synchronize()
                want = bo.matmul(fa, fb, ta, tb, out_dtype=od)  # eager work between replays
                bo.matmul(fa, fb, ta, tb, out=total)
                torch.cuda.synchronize()
                assert torch.equal(c, want), (M, N, K, "replay", rep)
                assert torch.equal(acc, total), (M, N, K, "accumulating replay", rep)
    finally:
        bo.set_gemm_backend(prev)


def test_gemm_dispatch_modes_agree(bo):
    """Default dispatch (per shape class), library only, and the hand-written kernel everywhere give the same
    product to fp32 accumulation accuracy on a Linear-shaped problem; operands the hand-written kernel does not take
    (a column count that is not a multiple of 8) fall through to the library without an error."""
    gen = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn((1024, 512), generator=gen, device="cuda").bfloat16()
    w = torch.randn((512, 1376), generator=gen, device="cuda").bfloat16()
    want = x.double() @ w.double()
    outs = []
    prev = bo.set_gemm_backend(1)
    try:
        for mode in (1, 0, 2):
            bo.set_gemm_backend(mode)
            outs.append(bo.matmul(x, w, out_dtype=torch.float32))
            assert float((outs[-1].double() - want).abs().max()) <= 2e-5 * float(want.abs().max())
        bo.set_gemm_backend(2)
        odd = torch.randn((512, 100), generator=gen, device="cuda").bfloat16()
        got = bo.matmul(x, odd, out_dtype=torch.float32)
        assert float((got.double() - x.double() @ odd.double()).abs().max()) <= 2e-5 * float(want.abs().max())
    finally:
        bo.set_gemm_backend(prev)
