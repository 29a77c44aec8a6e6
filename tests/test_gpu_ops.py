"""Parity of every HIP op against the CPU oracle, through the C ABI, on the same seeded
inputs.  Bar: bit-exact for token / index handling and the set of embedding rows
touched; |got - ref| <= 1e-5 + 1e-4 |ref| element-wise for FP32 results."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


@pytest.fixture(scope="module")
def ops():
    from seraph_amd import ops as o
    o.init(0)
    return o


def rng(seed):
    return np.random.default_rng(seed)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def parity(got, ref, what="", rtol=RTOL, atol=ATOL):
    got = np.asarray(host(got) if isinstance(got, torch.Tensor) else got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.abs(got - ref)
    bad = err > atol + rtol * np.abs(ref)
    rel = np.linalg.norm(got - ref) / (np.linalg.norm(ref) + 1e-30)
    if bad.any():
        i = np.unravel_index(np.argmax(err - rtol * np.abs(ref)), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside tolerance; worst at {i}: "
                             f"got {got[i]:.8g} ref {ref[i]:.8g}; rel-L2 {rel:.3e}")
    if atol > ATOL:
        # a case with a wider absolute term than the common bar: the margin goes on record (pytest -rA / -s shows it)
        print(f"[margin] {what}: atol {atol:g}: max abs err {err.max():.3e}, max err/tolerance "
              f"{(err / (atol + rtol * np.abs(ref))).max():.3f}, rel-L2 {rel:.3e}")
        assert rel <= 1e-4, f"{what}: rel-L2 {rel:.3e}"


# ------------------------------------------------------------------ element-wise
@pytest.mark.parametrize("n", [1, 3, 1023, 4096, 100003])
def test_elementwise_family(ops, orc, n):
    r = rng(n)
    a, b, g = (3 * r.standard_normal(n).astype(np.float32) for _ in range(3))
    A, B, G = dev(a), dev(b), dev(g)
    assert (host(ops.add(A, B, torch.empty_like(A))) == a + b).all()
    assert (host(ops.mul(A, B, torch.empty_like(A))) == a * b).all()
    assert (host(ops.scale_(A.clone(), 0.37)) == a * np.float32(0.37)).all()
    parity(ops.silu(A), orc.silu(a), "silu")
    parity(ops.silu_backward(A, G), orc.silu_backward(a, g), "silu_backward")
    dA, dB = ops.mul_backward(A, B, G)
    ra, rb = orc.mul_backward(a, b, g)
    assert (host(dA) == ra).all() and (host(dB) == rb).all()
    dG, dU = ops.swiglu_backward(A, B, G)
    rg, ru = orc.swiglu_backward(a, b, g)
    parity(dG, rg, "swiglu dGate"); parity(dU, ru, "swiglu dUp")
    parity(ops.swiglu(A, B), orc.silu(a) * b, "swiglu fwd")
    # in place, as src/train.c:5140 calls it (grad_input aliases grad_output)
    G2 = G.clone()
    ops.silu_backward(A, G2, out=G2)
    parity(G2, orc.silu_backward(a, g), "silu_backward in place")


def test_elementwise_unaligned_views(ops, orc):
    r = rng(7)
    base = r.standard_normal(5000).astype(np.float32)
    t = dev(base)
    a, b = t[1:3001], t[1002:4002]                      # 4-byte aligned only
    out = torch.empty(3001, dtype=torch.float32, device="cuda")[1:]
    ops.add(a, b, out)
    assert (host(out) == base[1:3001] + base[1002:4002]).all()


def test_fill_nan_reduce(ops, orc):
    t = torch.empty(1001, dtype=torch.int32, device="cuda")
    ops.fill_u32(t, 0xDEADBEEF)
    assert (host(t).view(np.uint32) == 0xDEADBEEF).all()
    flags = torch.zeros(8, dtype=torch.int32, device="cuda")
    x = dev(rng(1).standard_normal(70000).astype(np.float32))
    ops.nan_check(x, flags, 3)
    assert host(flags).sum() == 0
    x[69999] = float("inf")
    ops.nan_check(x, flags, 3)
    x[5] = float("nan")
    ops.nan_check(x, flags, 6)
    assert host(flags).tolist() == [0, 0, 0, 1, 0, 0, 1, 0]
    v = rng(2).standard_normal(1300).astype(np.float32)
    parity(ops.reduce_sum(dev(v)), orc.reduce_sum(v), "reduce_sum", atol=1e-4)


# ------------------------------------------------------------------ cross entropy
@pytest.mark.parametrize("rows,cols", [(9, 8192), (5, 1000), (4, 40000), (3, 33001), (2, 151936), (6, 4), (1030, 32772), (3, 1300000),
                                       (7, 12000), (5, 30000), (3, 32768)])    # 16 and 32 float4 per lane in one workgroup's registers
def test_cross_entropy_grad(ops, orc, rows, cols):
    r = rng(rows * 100003 + cols)
    x = (2 * r.standard_normal((rows, cols))).astype(np.float32)
    t = r.integers(0, cols, rows).astype(np.uint32)
    if rows > 2:
        t[1] = cols                                      # no supervision for this row
    rg, rl = orc.cross_entropy_grad(x, t, valid_rows=rows - 1)
    g, l = ops.cross_entropy_grad(dev(x), dev(t.view(np.int32)), rows - 1)
    parity(l, rl, "loss", atol=1e-5)
    parity(g, rg, "grad", atol=1e-7)
    if rows > 2:
        assert (host(g)[1] == 0).all() and host(l)[1] == 0
    # in place (grad aliases logits)
    X = dev(x)
    g2, l2 = ops.cross_entropy_grad(X, dev(t.view(np.int32)), rows - 1, grad=X)
    parity(g2, rg, "grad in place", atol=1e-7); parity(l2, rl, "loss in place")
    g0, _ = ops.cross_entropy_grad(dev(x), dev(t.view(np.int32)), 0)
    assert (host(g0) == 0).all()


@pytest.mark.parametrize("starts,dead", [([0, 3, 4, 20], (2, 3, 19)), ([0, 3, 3, 4, 20, 20], (2, 3, 19))])
def test_cross_entropy_grad_packed(ops, orc, starts, dead):
    """The last token of every sequence has no target; empty sequences change nothing."""
    r = rng(11)
    starts = np.array(starts, np.uint32)
    x = r.standard_normal((20, 8192)).astype(np.float32)
    t = r.integers(0, 8192, 20).astype(np.uint32)
    rg, rl = orc.cross_entropy_grad_packed(x, t, starts, 17)
    g, l = ops.cross_entropy_grad(dev(x), dev(t.view(np.int32)), 17, seq_starts=dev(starts.view(np.int32)))
    parity(g, rg, "packed grad", atol=1e-7); parity(l, rl, "packed loss")
    for last in dead:
        assert (host(g)[last] == 0).all() and host(l)[last] == 0


# ------------------------------------------------------------------ GEMM
@pytest.mark.parametrize("tA,tB", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("M,N,K", [(256, 384, 512), (67, 35, 129), (300, 16, 260), (16, 520, 300), (130, 140, 16),
                                   (1024, 2048, 96), (1, 1, 1), (260, 132, 64), (2052, 2500, 64), (2051, 2499, 32),
                                   (4, 4, 32), (2176, 2048, 160), (512, 512, 2048), (2048, 16, 2048), (16, 2048, 2048),
                                   (100, 36, 512), (8, 4, 4096)])
def test_gemm_forms(ops, orc, tA, tB, M, N, K):
    r = rng(M * 7 + N * 3 + K + 2 * tA + tB)
    A = r.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    C0 = r.standard_normal((M, N)).astype(np.float32)
    ref = orc.matmul(A, B, M, N, K, tA, tB)
    parity(ops.gemm(dev(A), dev(B), M, N, K, tA, tB), ref, f"gemm tA={tA} tB={tB}", atol=1e-4)
    out = dev(C0)
    ops.gemm(dev(A), dev(B), M, N, K, tA, tB, out=out, accumulate=True)
    parity(out, orc.matmul(A, B, M, N, K, tA, tB, C0), "gemm accumulate", atol=1e-4)


@pytest.mark.parametrize("tA,tB,M,N,K", [(0, 1, 2048, 16, 2048), (0, 0, 2048, 16, 1024), (1, 0, 2048, 16, 2048),
                                          (1, 0, 16, 2048, 2048), (1, 0, 8, 1024, 4096), (0, 1, 300, 20, 1000),
                                          (0, 1, 64, 64, 64), (1, 1, 2048, 16, 2048), (1, 1, 40, 2048, 1024)])
@pytest.mark.parametrize("scratch", [True, False])
def test_gemm_scaled(ops, orc, tA, tB, M, N, K, scratch):
    """alpha * product, also accumulated, with K cut into runs (scratch) and as product + scale (no scratch)."""
    r = rng(M + 3 * N + 5 * K + tA)
    A = r.standard_normal((K, M) if tA else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if tB else (K, N)).astype(np.float32)
    C0 = r.standard_normal((M, N)).astype(np.float32)
    ref = orc.matmul(A, B, M, N, K, tA, tB)
    got = ops.gemm_scaled(dev(A), dev(B), M, N, K, tA, tB, alpha=2.0, scratch=scratch)
    parity(got, 2.0 * ref, "gemm_scaled", atol=2e-4)
    again = ops.gemm_scaled(dev(A), dev(B), M, N, K, tA, tB, alpha=2.0, scratch=scratch)
    assert torch.equal(got, again)                                        # fixed summation order
    out = dev(C0)
    ops.gemm_scaled(dev(A), dev(B), M, N, K, tA, tB, out=out, accumulate=True, alpha=1.0, scratch=scratch)
    parity(out, orc.matmul(A, B, M, N, K, tA, tB, C0), "gemm_scaled accumulate", atol=1e-4)


@pytest.mark.parametrize("M,N,K", [(2048, 2048, 16), (2048, 1024, 16), (333, 512, 8), (4100, 260, 32), (64, 1024, 4)])
def test_gemm_small_k(ops, orc, M, N, K):
    """C (+)= A B^T with a rank-sized K: the kernel without matrix instructions."""
    r = rng(M + N + K)
    A = r.standard_normal((M, K)).astype(np.float32)
    B = r.standard_normal((N, K)).astype(np.float32)
    C0 = r.standard_normal((M, N)).astype(np.float32)
    parity(ops.gemm(dev(A), dev(B), M, N, K, 0, 1), orc.matmul(A, B, M, N, K, 0, 1), "small-K gemm")
    out = dev(C0)
    ops.gemm(dev(A), dev(B), M, N, K, 0, 1, out=out, accumulate=True)
    parity(out, orc.matmul(A, B, M, N, K, 0, 1, C0), "small-K gemm accumulate")


def test_gemm_reference_recipe_is_exact(ops):
    # tests/test_matmul.c:47-49 of the reference: 64^3, integers in [-5, 4]; exact in FP32
    r = rng(64)
    A = r.integers(-5, 5, (64, 64)).astype(np.float32)
    B = r.integers(-5, 5, (64, 64)).astype(np.float32)
    assert (host(ops.gemm(dev(A), dev(B), 64, 64, 64)) == (A.astype(np.int64) @ B.astype(np.int64))).all()
    A = r.integers(-5, 5, (300, 200)).astype(np.float32)
    B = r.integers(-5, 5, (300, 260)).astype(np.float32)      # TN, as the weight gradient uses it
    assert (host(ops.gemm(dev(A), dev(B), 200, 260, 300, 1, 0)) == (A.T.astype(np.int64) @ B.astype(np.int64))).all()


def test_gemm_wgrad_shape_long_k(ops, orc):
    r = rng(5)
    T, out_d, in_d = 4096, 192, 160
    dY = (1e-2 * r.standard_normal((T, out_d))).astype(np.float32)
    X = r.standard_normal((T, in_d)).astype(np.float32)
    G0 = (1e-2 * r.standard_normal((out_d, in_d))).astype(np.float32)
    out = dev(G0)
    ops.gemm(dev(dY), dev(X), out_d, in_d, T, 1, 0, out=out, accumulate=True)
    parity(out, orc.matmul(dY, X, out_d, in_d, T, 1, 0, G0), "wgrad")


@pytest.mark.parametrize("tA,tB", [(0, 1), (1, 0), (0, 0), (1, 1)])
@pytest.mark.parametrize("shapes,K", [
    ([(2048, 512), (2048, 512), (2048, 512)], 512),            # the 33M model's q / k / v: 64 x 64 tiles, one grid
    ([(512, 512), (512, 512), (512, 512)], 2048),              # their weight gradients: 32 x 32 tiles, waves split K
    ([(1408, 512), (1408, 512)], 2048),                        # gate / up weight gradients
    ([(4096, 2048), (4096, 1024), (4096, 1024)], 256),         # 128 x 128 tiles, unequal widths
    ([(300, 132), (77, 260), (64, 64), (129, 36)], 96),        # ragged edges, four products
    ([(100, 36), (67, 35)], 512),                              # a width that is no multiple of 4: run as single products
])
def test_gemm_grouped(ops, orc, tA, tB, shapes, K):
    """Several products in one launch: each output equals the single-product call's to the bit when the group runs the
    tile kernel the single call would pick, and matches the oracle within tolerance in any case."""
    from seraph_amd._lib import kernels
    r = rng(K + len(shapes) + 2 * tA + tB)
    probs, refs, singles = [], [], []
    for M, N in shapes:
        A = (0.5 * r.standard_normal((K, M) if tA else (M, K))).astype(np.float32)     # sums over K = 2048 stay inside
        B = (0.5 * r.standard_normal((N, K) if tB else (K, N))).astype(np.float32)     # the absolute term of the bar
        C0 = r.standard_normal((M, N)).astype(np.float32)
        probs.append((dev(A), dev(B), dev(C0), M, N))
        refs.append(orc.matmul(A, B, M, N, K, tA, tB, C0))
        singles.append(ops.gemm(dev(A), dev(B), M, N, K, tA, tB, out=dev(C0), accumulate=True))
    outs = ops.gemm_grouped(probs, K, tA, tB, accumulate=True)
    for o, ref, single, (M, N) in zip(outs, refs, singles, shapes):
        parity(o, ref, f"grouped gemm {M}x{N}x{K}", atol=1e-4)
        arr = (ops.GemmProblem * len(probs))(*[ops.GemmProblem(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, n) for a, b, c, m, n in probs])
        name = kernels().seraph_gemm_grouped_kernel_name(arr, len(probs), C.c_int64(K), tA, tB).decode()
        alone = kernels().seraph_gemm_kernel_name(C.c_int64(M), C.c_int64(N), C.c_int64(K), tA, tB).decode()
        if name.replace("_grouped", "") == alone or "single products" in name:
            assert torch.equal(o, single), (M, N, name)
    # overwrite form
    fresh = [(a, b, torch.full_like(c, float("nan")), m, n) for a, b, c, m, n in probs]
    for o, ref, (a, b, c0, m, n) in zip(ops.gemm_grouped(fresh, K, tA, tB), refs, probs):
        parity(o, orc.matmul(host(a), host(b), m, n, K, tA, tB), "grouped gemm, overwrite", atol=1e-4)


@pytest.mark.parametrize("tA,tB,shapes", [
    (0, 1, [(2048, 16, 2048), (2048, 16, 2048), (2048, 16, 2048)]),                       # x A^T of the q, k and v adapters
    (1, 0, [(2048, 16, 2048), (1024, 16, 2048), (1024, 16, 2048), (2048, 16, 2048)]),     # dY^T (x A^T): four adapters' B gradients
    (0, 0, [(2048, 16, 2048), (2048, 16, 1024), (2048, 16, 1024), (2048, 16, 2048)]),     # dY B: every product its own K
    (1, 0, [(16, 2048, 2048)] * 4),                                                       # (dY B)^T x: the A gradients
    (0, 1, [(2048, 2048, 16), (2048, 1024, 16), (2048, 1024, 16)]),                       # (x A^T) B^T onto q, k, v: rank-sized K
    (0, 1, [(300, 20, 1000), (64, 64, 64)]),                                              # shapes that share no launch: single calls
    (1, 1, [(2048, 16, 2048), (16, 1024, 2048), (512, 16, 1024)]),                        # both operands transposed (no call site in the step)
])
@pytest.mark.parametrize("accumulate,alpha", [(False, 2.0), (True, 1.0)])
def test_gemm_scaled_grouped_equals_the_single_calls(ops, orc, tA, tB, shapes, accumulate, alpha):
    """The rank-sized products of a layer's adapters in one launch each: every output has the bits of its own
    seraph_gemm_scaled call, and is the oracle's product within the bar."""
    r = rng(len(shapes) + 2 * tA + tB + int(alpha))
    probs, singles, refs = [], [], []
    for M, N, K in shapes:
        A = (0.5 * r.standard_normal((K, M) if tA else (M, K))).astype(np.float32)
        B = (0.5 * r.standard_normal((N, K) if tB else (K, N))).astype(np.float32)
        C0 = r.standard_normal((M, N)).astype(np.float32)
        probs.append((dev(A), dev(B), dev(C0), M, N, K))
        singles.append(ops.gemm_scaled(dev(A), dev(B), M, N, K, tA, tB, out=dev(C0), accumulate=accumulate, alpha=alpha))
        ref = alpha * orc.matmul(A, B, M, N, K, tA, tB).astype(np.float64)
        refs.append(ref + C0 if accumulate else ref)
    outs = ops.gemm_scaled_grouped(probs, tA, tB, accumulate=accumulate, alpha=alpha)
    for o, single, ref, shape in zip(outs, singles, refs, shapes):
        assert torch.equal(o, single), shape
        parity(o, ref, f"grouped scaled gemm {shape}", atol=2e-4)


@pytest.mark.parametrize("tA,tB", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,Ks", [(2048, 512, (1408, 1408)), (2048, 512, (512, 512, 512)), (1024, 2048, (2048, 1024, 1024)),
                                    (4100, 2048, (512, 256)),            # 128x128 tiles with a ragged edge
                                    (300, 260, (64, 32, 96)),            # edge tiles in both directions
                                    (96, 64, (2048, 1024)),              # few tiles, long K: 32x32 tiles whose waves share out K
                                    (40, 36, (96, 64, 128)),             # the same with ragged 32x32 tiles
                                    (130, 70, (36, 64)),                 # a K that is not whole stages: single products
                                    (512, 512, (128,))])
def test_gemm_chain(ops, orc, tA, tB, M, N, Ks):
    """C (+)= sum of products with different K in one launch: against the oracle's products added in double precision,
    for the overwriting and the accumulating form."""
    r = rng(M + N + sum(Ks) + 2 * tA + tB)
    terms, ref = [], np.zeros((M, N), np.float64)
    for K in Ks:
        A = (0.25 * r.standard_normal((K, M) if tA else (M, K))).astype(np.float32)     # sums of up to 4096 terms stay O(1)
        B = (0.25 * r.standard_normal((N, K) if tB else (K, N))).astype(np.float32)
        terms.append((dev(A), dev(B), K))
        ref += orc.matmul(A, B, M, N, K, tA, tB).astype(np.float64)
    out = ops.gemm_chain(terms, M, N, tA, tB, out=torch.full((M, N), float("nan"), device="cuda"))
    parity(out, ref.astype(np.float32), f"gemm chain {M}x{N}x{Ks}", atol=1e-4)
    C0 = r.standard_normal((M, N)).astype(np.float32)
    out = ops.gemm_chain(terms, M, N, tA, tB, out=dev(C0), accumulate=True)
    parity(out, (ref + C0).astype(np.float32), f"gemm chain {M}x{N}x{Ks}, accumulate", atol=1e-4)
    name = ops.gemm_chain_kernel_name(terms, out, M, N, tA, tB)
    one_launch = len(Ks) > 1 and all(K % 32 == 0 for K in Ks)
    assert ("chain_kernel" in name) == one_launch, name
    t64 = ((M + 63) // 64) * ((N + 63) // 64)                         # few 64x64 tiles and a long K: the waves share out K
    if one_launch and t64 < 256 and sum(Ks) >= 256:
        assert "splitk_chain_kernel" in name, name


# ------------------------------------------------------------------ rmsnorm
@pytest.mark.parametrize("rows,cols", [(33, 512), (17, 2048), (5, 4096), (9, 100), (4, 8192), (1, 4), (21, 1024), (11, 1408), (6, 256)])
def test_rmsnorm_forward_backward(ops, orc, rows, cols):
    r = rng(rows + cols)
    x = r.standard_normal((rows, cols)).astype(np.float32)
    s = (1 + 0.02 * r.standard_normal(cols)).astype(np.float32)
    dy = (1e-2 * r.standard_normal((rows, cols))).astype(np.float32)
    g0 = r.standard_normal(cols).astype(np.float32)
    for eps in (1e-5, 1e-6):
        parity(ops.rmsnorm(dev(x), dev(s), eps), orc.rmsnorm(x, s, eps), "rmsnorm")
        rdx, rgs = orc.rmsnorm_backward_batch(x, s, dy, eps, g0)
        dx, gs = ops.rmsnorm_backward(dev(x), dev(s), dev(dy), eps, grad_scale=dev(g0))
        parity(dx, rdx, "rmsnorm dx", atol=1e-7); parity(gs, rgs, "rmsnorm grad_scale")


@pytest.mark.parametrize("rows,cols", [(33, 512), (300, 2048), (9, 100), (17, 4096), (1, 4)])
def test_add_rmsnorm_equals_add_then_rmsnorm(ops, rows, cols):
    r = rng(rows + 7 * cols)
    x = dev(r.standard_normal((rows, cols)).astype(np.float32))
    b = dev(r.standard_normal((rows, cols)).astype(np.float32))
    s = dev((1 + 0.02 * r.standard_normal(cols)).astype(np.float32))
    total = ops.add(x, b, torch.empty_like(x))
    want = ops.rmsnorm(total, s, 1e-5)
    got_total, got = ops.add_rmsnorm(x, b, s, 1e-5)
    assert torch.equal(got_total, total) and torch.equal(got, want)


@pytest.mark.parametrize("rows,cols", [(33, 512), (300, 2048), (5, 4096), (9, 100), (700, 8192)])
def test_rmsnorm_backward_with_residual(ops, rows, cols):
    """dx = residual + input gradient in one pass: bit-identical to the separate add, also in place."""
    r = rng(rows * 3 + cols)
    x = dev(r.standard_normal((rows, cols)).astype(np.float32))
    s = dev((1 + 0.02 * r.standard_normal(cols)).astype(np.float32))
    dy = dev((1e-2 * r.standard_normal((rows, cols))).astype(np.float32))
    res = dev(r.standard_normal((rows, cols)).astype(np.float32))
    g0 = r.standard_normal(cols).astype(np.float32)
    dx, gs = ops.rmsnorm_backward(x, s, dy, 1e-5, grad_scale=dev(g0))
    want = ops.add(dx, res, torch.empty_like(dx))
    got, gs2 = ops.rmsnorm_backward(x, s, dy, 1e-5, grad_scale=dev(g0), residual=res)
    assert torch.equal(got, want) and torch.equal(gs, gs2)
    inplace = res.clone()
    ops.rmsnorm_backward(x, s, dy, 1e-5, grad_scale=dev(g0), residual=inplace, out=inplace)
    assert torch.equal(inplace, want)


@pytest.mark.parametrize("cols", [512, 2048, 100])
def test_rmsnorm_backward_rows_then_one_column_sum_for_all(ops, cols):
    """The row pass alone, several times, then one launch that folds every pass's partial rows: the same bits as the
    one-call backward, with and without a residual, for every row kernel (wave per row, block per row, generic)."""
    r = rng(cols)
    s = dev((1 + 0.02 * r.standard_normal(cols)).astype(np.float32))
    cases, jobs, want = [], [], []
    for i, rows in enumerate((300, 33, 2048, 1)):
        x = dev(r.standard_normal((rows, cols)).astype(np.float32))
        dy = dev((1e-2 * r.standard_normal((rows, cols))).astype(np.float32))
        res = dev(r.standard_normal((rows, cols)).astype(np.float32)) if i % 2 else None
        g0 = r.standard_normal(cols).astype(np.float32)
        want.append(ops.rmsnorm_backward(x, s, dy, 1e-5, grad_scale=dev(g0), residual=res))
        dx, part, nparts = ops.rmsnorm_backward_rows(x, s, dy, 1e-5, residual=res)
        assert nparts > 0
        gs = dev(g0)
        cases.append((dx, gs)); jobs.append((part, nparts, gs))
    ops.rmsnorm_colsum_multi(jobs, cols)
    for (dx, gs), (wdx, wgs) in zip(cases, want):
        assert torch.equal(dx, wdx) and torch.equal(gs, wgs)


def test_rmsnorm_colsum_multi_more_jobs_than_one_launch_holds(ops):
    cols, rows = 256, 40
    r = rng(11)
    s = dev((1 + 0.02 * r.standard_normal(cols)).astype(np.float32))
    x = dev(r.standard_normal((rows, cols)).astype(np.float32))
    jobs, want = [], []
    for i in range(70):
        dy = dev((1e-2 * r.standard_normal((rows, cols))).astype(np.float32))
        want.append(ops.rmsnorm_backward(x, s, dy, 1e-5)[1])
        _, part, nparts = ops.rmsnorm_backward_rows(x, s, dy, 1e-5)
        jobs.append((part, nparts, torch.zeros(cols, device="cuda")))
    ops.rmsnorm_colsum_multi(jobs, cols)
    for (_, _, gs), w in zip(jobs, want):
        assert torch.equal(gs, w)


def test_rmsnorm_backward_clamp_branch(ops, orc):
    r = rng(3)
    x = (1e-4 * r.standard_normal((6, 512))).astype(np.float32)       # sqrt(ms + 1e-5) < 0.01
    x[0] = 0
    s = r.standard_normal(512).astype(np.float32)
    dy = r.standard_normal((6, 512)).astype(np.float32)
    rdx, rgs = orc.rmsnorm_backward_batch(x, s, dy, 1e-5)
    dx, gs = ops.rmsnorm_backward(dev(x), dev(s), dev(dy), 1e-5)
    parity(dx, rdx, "clamped dx"); parity(gs, rgs, "clamped grad_scale")
    parity(host(dx)[0], dy[0].astype(np.float64) * s * 100.0, "x=0 row")


def test_qk_norm(ops, orc):
    r = rng(4)
    x = r.standard_normal((37, 4 * 64)).astype(np.float32)
    dy = r.standard_normal((37, 4 * 64)).astype(np.float32)
    parity(ops.qk_norm_(dev(x), 4, 64, 1e-6), orc.qk_norm(x, 4, 64, 1e-6), "qk_norm")
    assert (host(ops.qk_norm_(dev(x), 4, 64, 1e-6, use_qk_norm=0)) == x).all()     # disabled: untouched
    parity(ops.qk_norm_backward(dev(x), dev(dy), 4, 64, 1e-6), orc.qk_norm_backward(x, dy, 4, 64, 1e-6), "qk_norm bwd")


@pytest.mark.parametrize("T,heads,D", [(37, 4, 64), (300, 16, 128), (5, 3, 6), (1000, 8, 128), (64, 2, 32), (50, 4, 128), (20, 32, 128),
                                       (9, 40, 128)])           # 512, 4096 and 5120 values per token: two and sixteen float4 per lane, and the loop
def test_qk_norm_saved_pair(ops, orc, T, heads, D):
    """The pair the training step uses: the forward that also leaves each token's rms, and the backward from the
    normalised output and that rms.  Same derivative as the backward from the input (the oracle's), also in place, also
    for tokens whose norm is clamped at eps."""
    r = rng(T + heads)
    eps = 1e-3
    x = r.standard_normal((T, heads * D)).astype(np.float32)
    x[1] *= 1e-5                                                  # rms below eps: clamped
    x[3] = 0
    dy = r.standard_normal((T, heads * D)).astype(np.float32)
    y, rms = ops.qk_norm_saved_(dev(x), heads, D, eps)
    parity(y, orc.qk_norm(x, heads, D, eps), "qk_norm forward")
    parity(rms, np.sqrt((x.astype(np.float64) ** 2).mean(1)), "saved rms", atol=1e-7)
    ref = orc.qk_norm_backward(x, dy, heads, D, eps)
    parity(ops.qk_norm_backward_saved(y, rms, dev(dy), heads, D, eps), ref, "qk_norm backward from the output", atol=2e-5 if T else ATOL)
    g = dev(dy)
    parity(ops.qk_norm_backward_saved(y, rms, g, heads, D, eps, out=g), ref, "in place", atol=2e-5)


# ------------------------------------------------------------------ rope
@pytest.mark.parametrize("heads,D,theta,starts", [(8, 64, 10000.0, [0, 256, 300]), (16, 128, 1e6, [0, 4096]),
                                                  (3, 16, 10000.0, [0, 1, 2, 50]), (4, 64, 10000.0, [0, 7, 7, 40, 40])])
def test_rope_forward_backward(ops, orc, heads, D, theta, starts):
    r = rng(heads * D)
    T = starts[-1]
    x = r.standard_normal((T, heads * D)).astype(np.float32)
    su = np.array(starts, np.uint32)
    sd = dev(su.view(np.int32))
    # angles reach thousands of radians at theta = 1e6: FP32 sincos argument reduction sets the floor
    parity(ops.rope(dev(x), heads, D, theta, sd), orc.rope(x, heads, D, theta, su), "rope", atol=2e-5)
    parity(ops.rope(dev(x), heads, D, theta, sd, backward=True), orc.rope(x, heads, D, theta, su, backward=True),
           "rope backward", atol=2e-5)
    X = dev(x)
    ops.rope(X, heads, D, theta, sd, backward=True, out=X)                       # in place (src/train.c:5253)
    parity(X, orc.rope(x, heads, D, theta, su, backward=True), "rope backward in place", atol=2e-5)
    if len(starts) == 2:
        parity(ops.rope(dev(x), heads, D, theta, None), orc.rope(x, heads, D, theta, None), "rope unpacked", atol=2e-5)


# ------------------------------------------------------------------ embedding
def test_embedding_lookup_and_backward_bit_exact(ops, orc):
    r = rng(6)
    T, h, V = 3000, 512, 700
    tok = r.integers(0, V + 40, T).astype(np.uint32)
    tok[:50] = 13                                              # a heavily repeated token
    tok[77] = 4000000000
    dH = r.integers(-8, 9, (T, h)).astype(np.float32)          # integer-valued: any order sums exactly
    base = r.integers(-3, 4, (V, h)).astype(np.float32)
    ref = orc.embedding_backward(tok, dH, base)
    got = host(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)))
    assert (got == ref).all()
    touched = set(np.nonzero((got != base).any(1))[0].tolist())
    assert touched <= set(np.unique(tok[tok < V]).tolist())
    E = r.standard_normal((V, h)).astype(np.float32)
    assert (host(ops.embed_lookup(dev(tok.view(np.int32)), dev(E))) == orc.embed_lookup(tok, E)).all()


def test_embedding_backward_float_and_odd_hidden(ops, orc):
    r = rng(8)
    T, h, V = 500, 70, 90
    tok = r.integers(0, V, T).astype(np.uint32)
    dH = r.standard_normal((T, h)).astype(np.float32)
    base = r.standard_normal((V, h)).astype(np.float32)
    parity(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)), orc.embedding_backward(tok, dH, base),
           "embedding backward")
    # deterministic: two runs give identical bits
    a = host(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)))
    b = host(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)))
    assert (a == b).all()


def test_embedding_backward_vocabulary_larger_than_the_library_tables(ops, orc):
    """Vocabularies of more than 2^18 tokens do not fit the token tables that the library keeps: the table is then part of
    the caller's scratch and is cleared by a launch of its own in every call.  Twice with different tokens through the same
    scratch pattern, with repeated tokens on both sides of 2^18 and ids past the vocabulary; bit-exact (integer values)."""
    r = rng(19)
    T, V, h = 3000, 300000, 8
    base = r.integers(-3, 4, (V, h)).astype(np.float32)
    for seed in (1, 2):
        tok = rng(seed).integers(0, V + 1000, T).astype(np.uint32)
        tok[:40] = 5
        tok[40:80] = 262144 + 17
        tok[80:100] = V - 1
        dH = rng(seed + 10).integers(-8, 9, (T, h)).astype(np.float32)
        got = host(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)))
        assert (got == orc.embedding_backward(tok, dH, base)).all()


# ------------------------------------------------------------------ AdamW
@pytest.mark.parametrize("n", [1, 1000, 100003])
@pytest.mark.parametrize("clip", [0.0, 1.0])
def test_adamw(ops, orc, n, clip):
    r = rng(n)
    w = r.standard_normal(n).astype(np.float32)
    m = (1e-3 * r.standard_normal(n)).astype(np.float32)
    v = (1e-6 * r.random(n)).astype(np.float32)
    g = (1e-3 * r.standard_normal(n)).astype(np.float32)
    g[r.random(n) < 0.01] = 10.0
    for step in (1, 7):
        rw, rm, rv = orc.adamw(w, g, m, v, 3.14e-4, 0.9, 0.999, 0.01, 1e-8, step, clip)
        W, M, V = dev(w), dev(m), dev(v)
        ops.adamw_(W, dev(g), M, V, 3.14e-4, 0.9, 0.999, 0.01, 1e-8, step, clip)
        parity(W, rw, "adamw w", atol=1e-7); parity(M, rm, "adamw m", atol=1e-9); parity(V, rv, "adamw v", atol=1e-12)


# ------------------------------------------------------------------ attention
ATTN_CASES = [([0, 200], 4, 4, 64), ([0, 5, 6, 133, 300], 4, 2, 32), ([0, 257], 4, 2, 128), ([0, 128, 256], 2, 1, 64),
              ([0, 1], 2, 2, 64), ([0, 31, 64, 97, 161], 8, 2, 128),
              ([0, 40, 40, 100, 100], 4, 2, 64)]          # empty sequences in the middle and at the end


def _attn_inputs(seed, starts, H, KVH, D):
    r = rng(seed)
    T = starts[-1]
    mk = lambda w: (r.standard_normal((T, w)) / np.sqrt(np.sqrt(D))).astype(np.float32)
    return mk(H * D), mk(KVH * D), mk(KVH * D), mk(H * D)


@pytest.mark.parametrize("starts,H,KVH,D", ATTN_CASES)
def test_attention_forward(ops, orc, starts, H, KVH, D):
    Q, K, V, _ = _attn_inputs(1, starts, H, KVH, D)
    su = np.array(starts, np.uint32)
    ro, rl = orc.attention_forward(Q, K, V, H, KVH, D, su)
    o, l = ops.attention_forward(dev(Q), dev(K), dev(V), H, KVH, D, dev(su.view(np.int32)))
    parity(o, ro, "attention out"); parity(l, rl, "attention lse")
    if len(starts) == 2:
        o2, _ = ops.attention_forward(dev(Q), dev(K), dev(V), H, KVH, D, None)
        parity(o2, ro, "attention out, unpacked call")


ATTN_CASES_BWD = ATTN_CASES + [([0, 700, 731, 1500], 4, 2, 64), ([0, 513, 1030], 2, 1, 128), ([0, 90, 1000], 2, 2, 32),
                               # enough (key tile, kv head) items to fill the chip: every item keeps all of its iterations
                               ([0, 600, 1111, 1500, 2100, 2650, 3333, 4100], 16, 8, 128),
                               ([0, 600, 1111, 1500, 2100, 2650, 3333, 4100], 8, 8, 64),
                               ([0, 77, 2000, 4100], 8, 8, 32),
                               # wider query groups per kv head (4 and 8 query heads each)
                               ([0, 300, 700], 8, 2, 64), ([0, 513, 1030], 8, 1, 128), ([0, 90, 640], 4, 1, 32)]


@pytest.mark.parametrize("starts,H,KVH,D", ATTN_CASES_BWD)
@pytest.mark.parametrize("saved", [False, True])
@pytest.mark.parametrize("banded", [False, True])
def test_attention_backward(ops, orc, starts, H, KVH, D, saved, banded):
    Q, K, V, dO = _attn_inputs(2, starts, H, KVH, D)
    su = np.array(starts, np.uint32)
    sd = dev(su.view(np.int32))
    base = rng(3).standard_normal(K.shape).astype(np.float32)
    rdQ, rdK, rdV = orc.attention_backward(Q, K, V, dO, H, KVH, D, su, dK0=base, dV0=base)
    out = lse = None
    if saved:
        out, lse = ops.attention_forward(dev(Q), dev(K), dev(V), H, KVH, D, sd)
    # banded: scratch sized for the dS band of the longest sequence -> dQ from stored dS (5 products)
    msl = int(np.diff(starts).max()) if banded else None
    dQ, dK, dV = ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), H, KVH, D, sd, out=out, lse=lse,
                                        dK=dev(base), dV=dev(base), max_seq_len=msl)
    parity(dQ, rdQ, "dQ"); parity(dK, rdK, "dK"); parity(dV, rdV, "dV")


@pytest.mark.parametrize("starts,H,KVH,D", ATTN_CASES_BWD)
def test_attention_backward_assign_equals_the_adding_form_on_zeroed_buffers(ops, starts, H, KVH, D):
    """dK / dV assigned over buffers that hold NaN, the dS band sized from the host's copy of the offsets: bit-identical to
    the adding form run on zeroed dK / dV with the exact bound (which the case above holds against the oracle)."""
    Q, K, V, dO = _attn_inputs(12, starts, H, KVH, D)
    sd = dev(np.array(starts, np.int32))
    out, lse = ops.attention_forward(dev(Q), dev(K), dev(V), H, KVH, D, sd)
    ref = ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), H, KVH, D, sd, out=out, lse=lse,
                                 max_seq_len=int(np.diff(starts).max()))
    junk = np.full(K.shape, np.nan, np.float32)
    got = ops.attention_backward_assign(dev(Q), dev(K), dev(V), dev(dO), H, KVH, D, sd, starts, out=out, lse=lse,
                                        dK=dev(junk), dV=dev(junk))
    for g, r, name in zip(got, ref, ("dQ", "dK", "dV")):
        assert np.array_equal(host(g), host(r)), name


def test_attention_backward_assign_checks_the_host_offsets(ops):
    from seraph_amd._lib import SeraphError
    Q, K, V, dO = _attn_inputs(13, [0, 40, 100], 2, 2, 32)
    sd = dev(np.array([0, 40, 100], np.int32))
    for bad in ([0, 40, 90], [1, 40, 100], [0, 60, 50, 100][:3]):
        with pytest.raises(SeraphError):
            ops.attention_backward_assign(dev(Q), dev(K), dev(V), dev(dO), 2, 2, 32, sd, bad)


def test_scratch_that_is_missing_or_too_small_is_refused(ops):
    """Entry points that take caller-owned scratch return SERAPH_ERR_WORKSPACE (-3) before they touch anything when it is
    missing, misaligned or smaller than their *_ws_bytes() query says; the outputs keep what they held."""
    import ctypes as C
    from seraph_amd._lib import kernels
    k = kernels()
    k.seraph_hip_last_error.restype = C.c_char_p
    i64, sz, f32, p = C.c_int64, C.c_size_t, C.c_float, lambda t: C.c_void_p(t.data_ptr())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    T, h, V, H, D = 64, 256, 300, 2, 32
    x, dy = torch.randn(T, h, device="cuda"), torch.randn(T, h, device="cuda")
    w = torch.ones(h, device="cuda")
    dx, gs = torch.full((T, h), 5.0, device="cuda"), torch.full((h,), 5.0, device="cuda")
    small = torch.zeros(64, dtype=torch.uint8, device="cuda")
    nparts = C.c_int(0)
    tok = torch.randint(0, V, (T,), device="cuda", dtype=torch.int32)
    ge = torch.full((V, h), 5.0, device="cuda")
    q = torch.randn(T, H * D, device="cuda")
    dq, dk, dv = (torch.full((T, H * D), 5.0, device="cuda") for _ in range(3))
    calls = {
        "rmsnorm_backward": lambda ws, n: k.seraph_rmsnorm_backward(p(x), p(w), p(dy), p(dx), p(gs), i64(T), i64(h), f32(1e-5), ws, sz(n), st),
        "rmsnorm_backward_rows": lambda ws, n: k.seraph_rmsnorm_backward_rows(p(x), p(w), p(dy), None, p(dx), i64(T), i64(h), f32(1e-5), ws, sz(n),
                                                                            C.byref(nparts), st),
        "embedding_backward": lambda ws, n: k.seraph_embedding_backward(p(tok), p(dy), p(ge), i64(T), i64(h), i64(V), ws, sz(n), st),
        "attention_backward": lambda ws, n: k.seraph_attention_backward(p(q), p(q), p(q), p(q), None, None, p(dq), p(dk), p(dv), None, 1, i64(T),
                                                                      H, H, D, f32(D ** -0.5), ws, sz(n), st),
    }
    for name, call in calls.items():
        assert call(None, 0) == -3, name
        assert call(p(small), 64) == -3, name
        assert b"scratch" in k.seraph_hip_last_error(), name
    torch.cuda.synchronize()
    for t in (dx, gs, ge, dq, dk, dv):
        assert (t == 5.0).all()
    # the non-banded attention backward with scratch of the size it asks for: the sum into dK / dV, dQ overwritten
    k.seraph_attention_backward_ws_bytes.restype = C.c_size_t
    need = k.seraph_attention_backward_ws_bytes(i64(T), H, H, D)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    dk.zero_(); dv.zero_()
    assert calls["attention_backward"](p(ws), need) == 0
    ref = ops.attention_backward(q, q, q, q, H, H, D)
    for got, want in zip((dq, dk, dv), ref):
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)


def test_rope_and_cross_entropy_many_short_sequences(ops, orc):
    """Thousands of packed sequences: positions restart and the last token of each has no target."""
    n_seq = 3000
    r = rng(78)
    lens = r.integers(1, 12, n_seq)
    starts = np.concatenate([[0], np.cumsum(lens)]).astype(np.uint32)
    T = int(starts[-1])
    sd = dev(starts.view(np.int32))
    x = r.standard_normal((T, 2 * 64)).astype(np.float32)
    parity(ops.rope(dev(x), 2, 64, 10000.0, sd), orc.rope(x, 2, 64, 10000.0, starts), "rope", atol=2e-5)
    parity(ops.rope(dev(x), 2, 64, 10000.0, sd, backward=True), orc.rope(x, 2, 64, 10000.0, starts, backward=True), "rope bwd", atol=2e-5)
    V = 1000
    logits = r.standard_normal((T, V)).astype(np.float32)
    t = r.integers(0, V, T).astype(np.uint32)
    valid = T - n_seq
    rg, rl = orc.cross_entropy_grad_packed(logits, t, starts, valid)
    g, l = ops.cross_entropy_grad(dev(logits), dev(t.view(np.int32)), valid, seq_starts=sd)
    parity(g, rg, "packed grad", atol=1e-7); parity(l, rl, "packed loss")


def test_attention_many_short_sequences(ops, orc):
    """More sequences than the kernels keep offsets for in LDS, and more 128-token tiles than they rank by length:
    the offsets are searched in global memory and the tiles run in their natural order."""
    n_seq, H, KVH, D = 2800, 2, 1, 32
    r = rng(77)
    lens = r.integers(1, 100, n_seq)
    starts = np.concatenate([[0], np.cumsum(lens)]).astype(np.uint32)
    T = int(starts[-1])
    assert T > 1024 * 128 and n_seq + 1 > 1024
    Q, K, V, dO = _attn_inputs(5, [0, T], H, KVH, D)
    sd = dev(starts.view(np.int32))
    ro, rl = orc.attention_forward(Q, K, V, H, KVH, D, starts)
    o, l = ops.attention_forward(dev(Q), dev(K), dev(V), H, KVH, D, sd)
    parity(o, ro, "out"); parity(l, rl, "lse")
    rdQ, rdK, rdV = orc.attention_backward(Q, K, V, dO, H, KVH, D, starts)
    for msl in (None, int(lens.max())):
        dQ, dK, dV = ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), H, KVH, D, sd, out=o, lse=l, max_seq_len=msl)
        parity(dQ, rdQ, "dQ"); parity(dK, rdK, "dK"); parity(dV, rdV, "dV")


def test_attention_backward_is_deterministic(ops):
    Q, K, V, dO = _attn_inputs(4, [0, 300, 700], 4, 2, 64)
    sd = dev(np.array([0, 300, 700], np.int32))
    a = [host(t) for t in ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), 4, 2, 64, sd)]
    b = [host(t) for t in ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), 4, 2, 64, sd)]
    assert all((x == y).all() for x, y in zip(a, b))
    c = [host(t) for t in ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), 4, 2, 64, sd, max_seq_len=400)]
    d = [host(t) for t in ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), 4, 2, 64, sd, max_seq_len=400)]
    assert all((x == y).all() for x, y in zip(c, d))
    assert (a[1] == c[1]).all() and (a[2] == c[2]).all()      # dK, dV come from the same kernel either way


@pytest.mark.parametrize("starts,H,KVH,D,bound", [([0, 700, 731, 1500], 4, 2, 64, 100), ([0, 513, 1030], 2, 1, 128, 300),
                                                  ([0, 2100], 8, 8, 32, 64)])
def test_attention_backward_with_a_bound_that_is_too_small(ops, orc, starts, H, KVH, D, bound):
    """The caller's bound on the sequence length is shorter than a sequence: the device notices (the band of
    dS tiles cannot hold the sequence), leaves the band unread and forms dQ with the recomputing kernel."""
    Q, K, V, dO = _attn_inputs(6, starts, H, KVH, D)
    su = np.array(starts, np.uint32)
    sd = dev(su.view(np.int32)) if len(starts) > 2 else None
    rdQ, rdK, rdV = orc.attention_backward(Q, K, V, dO, H, KVH, D, su)
    assert bound < int(np.diff(starts).max())
    for _ in range(2):                                       # twice: the mark of one launch must not leak into the next
        dQ, dK, dV = ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), H, KVH, D, sd, max_seq_len=bound)
        parity(dQ, rdQ, "dQ"); parity(dK, rdK, "dK"); parity(dV, rdV, "dV")
    ok = ops.attention_backward(dev(Q), dev(K), dev(V), dev(dO), H, KVH, D, sd, max_seq_len=int(np.diff(starts).max()))
    parity(ok[0], rdQ, "dQ after an overflowing launch")


def test_attention_rejects_unsupported_head_dim(ops):
    from seraph_amd._lib import SeraphError
    Q = torch.zeros(8, 48, device="cuda")
    with pytest.raises(SeraphError):
        ops.attention_forward(Q, Q, Q, 2, 2, 24)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("D", [32, 64, 128, 6])
def test_rope_qk_equals_two_rope_calls(ops, packed, D):
    """seraph_rope_qk (query and key heads in one launch) is bit-identical to two seraph_rope calls."""
    import ctypes as C
    from seraph_amd.ops import _p, _stream, kernels
    T, H, KVH = 77, 6, 2
    st = dev(np.array([0, 30, 31, 77], np.uint32).view(np.int32)) if packed else None
    q = torch.randn(T, H * D, device="cuda")
    k = torch.randn(T, KVH * D, device="cuda")
    for backward in (False, True):
        q1 = ops.rope(q, H, D, 1e4, st, backward=backward)
        k1 = ops.rope(k, KVH, D, 1e4, st, backward=backward)
        q2, k2 = q.clone(), k.clone()
        rc = kernels().seraph_rope_qk(_p(q2), _p(q2), H, _p(k2), _p(k2), KVH, _p(st), 3 if packed else 1,
                                      C.c_int64(T), D, C.c_float(1e4), 1 if backward else 0, _stream())
        assert rc == 0
        torch.cuda.synchronize()
        assert torch.equal(q1, q2) and torch.equal(k1, k2)


@pytest.mark.parametrize("spins", [0, 3])
def test_cross_entropy_long_rows_when_partners_are_not_waited_for(ops, orc, spins):
    """Long rows are shared out between workgroups that exchange (max, sum) through device memory.  With the wait
    bounded to nothing (or next to nothing) a workgroup computes its partners' statistics itself from the logits, as it
    would for a partner that has not been scheduled: same results, also in place and with unsupervised rows."""
    from seraph_amd._lib import kernels
    r = rng(91)
    for rows, cols in ((5, 40000), (9, 151936), (1100, 36000)):
        x = (2 * r.standard_normal((rows, cols))).astype(np.float32)
        t = r.integers(0, cols, rows).astype(np.uint32)
        t[1] = cols
        starts = np.array([0, 3, rows], np.uint32)
        rg, rl = orc.cross_entropy_grad_packed(x, t, starts, rows - 3)
        sd = dev(starts.view(np.int32))
        g_waited, l_waited = ops.cross_entropy_grad(dev(x), dev(t.view(np.int32)), rows - 3, seq_starts=sd)
        try:
            kernels().seraph_cross_entropy_exchange_spins(spins)
            g, l = ops.cross_entropy_grad(dev(x), dev(t.view(np.int32)), rows - 3, seq_starts=sd)
            X = dev(x)
            g2, l2 = ops.cross_entropy_grad(X, dev(t.view(np.int32)), rows - 3, seq_starts=sd, grad=X)
            torch.cuda.synchronize()
        finally:
            kernels().seraph_cross_entropy_exchange_spins(1 << 16)
        parity(g, rg, "grad", atol=1e-7); parity(l, rl, "loss")
        parity(g2, rg, "grad in place", atol=1e-7); parity(l2, rl, "loss in place")
        # a part's statistics formed by a partner are the owner's own bits: whoever waited for whom, nothing changes
        assert torch.equal(g, g_waited) and torch.equal(l, l_waited)
        assert torch.equal(g2, g_waited) and torch.equal(l2, l_waited)


def test_cross_entropy_long_rows_in_more_than_one_launch(ops, orc):
    """Every (row, part) unit of a launch has an exchange record of its own (2^18 per launch); 140000 rows in two parts
    need two launches.  Sampled rows against the oracle, row sums, and the in-place form bit for bit."""
    rows, cols = 140000, 33792
    torch.manual_seed(5)
    x = torch.randn(rows, cols, device="cuda") * 2
    t = torch.randint(0, cols, (rows,), device="cuda", dtype=torch.int32)
    g, l = ops.cross_entropy_grad(x, t, rows)
    pick = np.array([0, 1, 131071, 131072, 131073, rows - 1])
    xs, ts = x[pick].cpu().numpy(), t[pick].cpu().numpy().astype(np.uint32)
    rg, rl = orc.cross_entropy_grad(xs, ts, len(pick))
    parity(g[pick] * (rows / len(pick)), rg, "grad of sampled rows", atol=1e-7)
    parity(l[pick], rl, "loss of sampled rows")
    assert float(g.sum(dim=1).abs().max()) < 1e-9
    g2, l2 = ops.cross_entropy_grad(x, t, rows, grad=x)
    assert torch.equal(g2, g) and torch.equal(l2, l)


@pytest.mark.parametrize("rows,cols", [(4, 40000), (3, 151936), (300, 151936), (2100, 77828), (40, 1000000)])
def test_cross_entropy_long_rows_are_deterministic_and_alias_safe(ops, rows, cols):
    """Rows shared out between workgroups: repeated runs and the in-place form (grad over logits) give identical bits."""
    torch.manual_seed(rows + cols)
    x = torch.randn(rows, cols, device="cuda") * 2
    t = torch.randint(0, cols, (rows,), device="cuda", dtype=torch.int32)
    if rows > 3:
        t[1] = cols                                       # an unsupervised row between live ones
    g_ref, l_ref = ops.cross_entropy_grad(x.clone(), t, rows)
    for _ in range(3):
        g, l = ops.cross_entropy_grad(x.clone(), t, rows)
        assert torch.equal(g, g_ref) and torch.equal(l, l_ref)
        X = x.clone()
        g2, l2 = ops.cross_entropy_grad(X, t, rows, grad=X)
        assert torch.equal(g2, g_ref) and torch.equal(l2, l_ref)
    # each live row's gradient sums to zero: softmax minus one-hot, scaled
    live = torch.ones(rows, dtype=torch.bool, device="cuda")
    if rows > 3:
        live[1] = False
    assert float(g_ref[live].double().sum(dim=1).abs().max()) < 1e-6
    assert float(g_ref[~live].abs().max()) == 0 if (~live).any() else True


@pytest.mark.parametrize("h", [256, 520, 1024, 2048, 4096])
@pytest.mark.parametrize("case", ["one token", "few tokens", "pairs", "mixed"])
def test_embedding_backward_repeated_tokens(ops, orc, case, h):
    """Groups of every size: a batch that is one token repeated (a padding-dominated batch), a handful of tokens, every
    token twice, and a mixture whose groups straddle the length from which a group is cut along the row's width (16, for
    rows of more than 256 columns: 520 has a ragged third slab, 2048 has eight; narrower rows are gathered by one
    wavefront at any length) and the batch size of the gather list (1024).  Integer-valued gradients: the sums are
    exact, so the check is bit-exact."""
    r = rng(15)
    T, V = 5000, 3000
    if case == "one token":
        tok = np.full(T, 7, np.uint32)
    elif case == "few tokens":
        tok = r.integers(0, 3, T).astype(np.uint32) * 1000
    elif case == "pairs":
        tok = np.concatenate([r.permutation(T // 2), r.permutation(T // 2)]).astype(np.uint32)
    else:
        sizes = [1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 1023, 1024, 1025]
        tok = np.concatenate([np.full(n, 10 + i, np.uint32) for i, n in enumerate(sizes)] +
                             [np.arange(100, 100 + T - sum(sizes), dtype=np.uint32)])
        tok = tok[r.permutation(T)]
        tok[::97] = V + 5                                      # skipped positions in between
    dH = r.integers(-8, 9, (T, h)).astype(np.float32)
    base = r.integers(-3, 4, (V, h)).astype(np.float32)
    ref = orc.embedding_backward(tok, dH, base)
    got = host(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)))
    assert (got == ref).all()
    # float gradients: deterministic and within tolerance
    dF = r.standard_normal((T, h)).astype(np.float32)
    a = ops.embedding_backward(dev(tok.view(np.int32)), dev(dF), dev(base))
    b = ops.embedding_backward(dev(tok.view(np.int32)), dev(dF), dev(base))
    assert torch.equal(a, b)
    # a row that collects up to 5000 N(0,1) terms has partial sums of about 70, whose float spacing is 8e-6: two orders of
    # addition differ by some 1e-4 in absolute terms wherever the total happens to land near zero
    parity(a, orc.embedding_backward(tok, dF, base), "embedding backward", atol=1e-3)


def test_embedding_backward_more_column_slabs_than_positions(ops, orc):
    """Rows of 9000 floats are 36 column slabs; a token that occurs 16 to 35 times has fewer positions than slabs, so its
    takers have to come back for more than one slab each.  Also repeated calls: the tables that the library keeps between
    calls carry the call's number, so what an earlier call left in them must count as empty."""
    r = rng(17)
    T, V, h = 700, 500, 9000
    sizes = [16, 17, 20, 35, 36, 37, 100]
    tok = np.concatenate([np.full(n, 3 + 7 * i, np.uint32) for i, n in enumerate(sizes)] +
                         [r.integers(100, V, T - sum(sizes)).astype(np.uint32)])
    tok = tok[r.permutation(T)]
    dH = r.integers(-8, 9, (T, h)).astype(np.float32)
    base = r.integers(-3, 4, (V, h)).astype(np.float32)
    ref = orc.embedding_backward(tok, dH, base)
    for _ in range(6):                                         # more calls than the library has tables
        got = host(ops.embedding_backward(dev(tok.view(np.int32)), dev(dH), dev(base)))
        assert (got == ref).all()
    tok2 = tok[::-1].copy()                                    # other owners, other chains, the same tables
    assert (host(ops.embedding_backward(dev(tok2.view(np.int32)), dev(dH), dev(base))) == orc.embedding_backward(tok2, dH, base)).all()
