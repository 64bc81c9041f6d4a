"""GPU parity of the variant trees (C++ host layer over the HIP kernels, through the planner
C ABI) against the CPU oracle's trees, variant by variant, on the same seeded inputs.
Bars: GEMM / SYRK normwise 16 k eps; TRSM against the oracle solve at 1e-9 relative."""
import itertools

import numpy as np
import pytest

from util import EPS, bits_equal, fro, gemm_bound, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112


@pytest.fixture(scope="module")
def ws():
    import torch
    return torch.full((4 << 20,), float("nan"), dtype=torch.float64, device="cuda")


@pytest.mark.parametrize("method", ["gemm", "gemm_pad", "gemm_tile"])
@pytest.mark.parametrize("ta,tb", list(itertools.product([N, T], [N, T])))
def test_gemm_variants_against_oracle_trees(handle, orc, ws, method, ta, tb):
    from rtatblas_amd import planner
    m, n, k = 170, 145, 162
    p = planner.Planner(method)
    variants = p.variants() if method != "gemm_pad" else p.variants()[::3]
    A = orc.fill(k if ta == T else m, m if ta == T else k, (k if ta == T else m) + 3, seed=1)
    B = orc.fill(n if tb == T else k, k if tb == T else n, (n if tb == T else k) + 1, seed=2)
    C0 = orc.fill(m, n, m + 3, seed=3)
    dA, dB = to_dev(A), to_dev(B)
    for v in variants:
        oracle_v = v.split("/")[0]          # the tile shape has no counterpart in the oracle
        want = C0.copy(order="F")
        assert orc.gemm_variant(oracle_v, ta, tb, m, n, k, 1.0, A, B, 0.5, want) == 0
        dC = to_dev(C0)
        ran = p.gemm(handle, v, ta, tb, m, n, k, 1.0, dA, A.shape[0], dB, B.shape[0], 0.5, dC,
                     C0.shape[0], ws, ws.numel() * 8)
        assert ran == v
        got = to_host(dC, C0.shape[0], n)
        Al, Bl = A[: (k if ta == T else m)], B[: (n if tb == T else k)]
        assert fro(got[:m] - want[:m]) <= gemm_bound(k, 1.0, Al, Bl, 0.5, C0[:m]), v
        assert bits_equal(got[m:], C0[m:])


@pytest.mark.parametrize("uplo,trans", list(itertools.product([121, 122], [N, T])))
def test_syrk_variants_against_oracle_trees(handle, orc, ws, uplo, trans):
    from rtatblas_amd import planner
    n, k = 213, 74
    p = planner.Planner("syrk")
    A = orc.fill(k if trans == T else n, n if trans == T else k, seed=4)
    C0 = orc.fill(n, n, n + 2, seed=5, kind=1)
    for v in p.variants():
        want = C0.copy(order="F")
        assert orc.syrk_variant(v, uplo, trans, n, k, -1.0, A, 1.0, want) == 0
        dC = to_dev(C0)
        p.syrk(handle, v, uplo, trans, n, k, -1.0, to_dev(A), A.shape[0], 1.0, dC, C0.shape[0], ws,
               ws.numel() * 8)
        got = to_host(dC, C0.shape[0], n)
        tri = np.tril if uplo == 122 else np.triu
        assert fro(tri(got[:n]) - tri(want[:n])) <= 16 * k * EPS * (fro(A) ** 2 + fro(C0[:n])), v
        if v[1] == "T":
            # the transposing variant rewrites the other triangle too (C = S^T + beta C over all
            # of C), exactly as the reference's tree does: same bits as the oracle's tree
            other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
            assert bits_equal(other(got[:n]), other(want[:n]))


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [121, 122], [N, T], [131, 132])))
def test_trsm_variants_against_oracle_trees(handle, orc, ws, side, uplo, trans, diag):
    from rtatblas_amd import planner
    m, n = 143, 152
    p = planner.Planner("trsm")
    na = m if side == 141 else n
    A = orc.fill(na, na, seed=6, kind=4)
    B0 = orc.fill(m, n, m + 1, seed=7)
    dA = to_dev(A)
    for v in p.variants():
        want = B0.copy(order="F")
        assert orc.trsm_variant(v, side, uplo, trans, diag, m, n, 1.0, A, want) == 0
        dB = to_dev(B0)
        p.trsm(handle, v, side, uplo, trans, diag, m, n, 1.0, dA, na, dB, m + 1, ws, ws.numel() * 8)
        got = to_host(dB, m + 1, n)
        assert np.allclose(got[:m], want[:m], rtol=1e-9, atol=1e-12), v
        assert bits_equal(got[m:], B0[m:])


def test_autotune_converges_and_reports(handle, orc, ws):
    from rtatblas_amd import planner
    m, n, k = 512, 512, 512                      # config C1: NN, alpha 1, beta 0, ld = M
    p = planner.Planner("gemm")
    p.set_refinement(0)                          # commit straight after the three passes
    A, B = orc.fill(m, k, seed=1), orc.fill(k, n, seed=2)
    dA, dB = to_dev(A), to_dev(B)
    dC = to_dev(np.full((m, n), np.nan, order="F"))
    seen = [p.gemm(handle, None, N, N, m, n, k, 1.0, dA, m, dB, k, 0.0, dC, m, ws, ws.numel() * 8)
            for _ in range(40)]
    assert seen[:24] == p.variants() * 3                              # three passes over the variants
    assert len(set(seen[24:])) == 1                                   # then one committed plan
    orc.cblas_on()
    try:
        want = np.zeros((m, n), order="F")
        orc.dgemm(N, N, m, n, k, 1.0, A, B, 0.0, want)
    finally:
        orc.cblas_off()
    assert fro(to_host(dC, m, n) - want) <= 16 * k * EPS * fro(A) * fro(B)
    stats = p.stats()
    assert stats[0]["key"] == {"transA": "N", "transB": "N", "m": m, "n": n, "k": k}
    assert sum(len(o["times"]) for o in stats[0]["options"]) == 40
    plans = p.plans()
    assert plans[0]["plan"] == {"transA": seen[-1][0], "transB": seen[-1][1], "transC": seen[-1][2]}
    q = planner.Planner("gemm")
    assert q.load_plans(plans) == 1
    assert q.gemm(handle, None, N, N, m, n, k, 1.0, dA, m, dB, k, 0.0, dC, m, ws,
                  ws.numel() * 8) == seen[-1]


def test_small_workspace_degrades_to_default(handle, orc):
    from rtatblas_amd import planner
    p = planner.Planner("gemm")
    m, n, k = 69, 123, 42
    A, B = orc.fill(m, k, seed=1), orc.fill(k, n, seed=2)
    dC = to_dev(np.zeros((m, n), order="F"))
    ran = p.gemm(handle, "TTT", N, N, m, n, k, 1.0, to_dev(A), m, to_dev(B), k, 0.0, dC, m, None, 0)
    assert ran == "NNN"
    assert fro(to_host(dC, m, n) - A @ B) <= 16 * k * EPS * fro(A) * fro(B)


# ---- fused variants: the transposition of the result absorbed by the kernel ---------------------

@pytest.mark.parametrize("ta,tb", list(itertools.product([N, T], [N, T])))
def test_gemm_fused_variants(handle, orc, ws, ta, tb):
    """gemm_fused enumerates [ta][tb][tc] with tc in N / T / X.  Every variant against the
    oracle's tree (X has the value of N there); "xyX" must need exactly the workspace of "xyN"
    (none at all for "NNX"), equal "xyN" bit for bit, and agree with the unfused tree "xyT"
    within the bar."""
    from rtatblas_amd import planner
    m, n, k = 170, 145, 162
    p = planner.Planner("gemm_fused")
    assert p.variants() == ["".join(v) for v in itertools.product("NT", "NT", "NTX")]
    A = orc.fill(k if ta == T else m, m if ta == T else k, (k if ta == T else m) + 3, seed=1)
    B = orc.fill(n if tb == T else k, k if tb == T else n, (n if tb == T else k) + 1, seed=2)
    C0 = orc.fill(m, n, m + 3, seed=3)
    dA, dB = to_dev(A), to_dev(B)
    Al, Bl = A[: (k if ta == T else m)], B[: (n if tb == T else k)]
    bar = gemm_bound(k, 1.0, Al, Bl, 0.5, C0[:m])
    got = {}
    for v in p.variants():
        want = C0.copy(order="F")
        assert orc.gemm_variant(v.replace("X", "N"), ta, tb, m, n, k, 1.0, A, B, 0.5, want) == 0
        dC = to_dev(C0)
        ran = p.gemm(handle, v, ta, tb, m, n, k, 1.0, dA, A.shape[0], dB, B.shape[0], 0.5, dC,
                     C0.shape[0], ws, ws.numel() * 8)
        assert ran == v
        got[v] = to_host(dC, C0.shape[0], n)
        assert fro(got[v][:m] - want[:m]) <= bar, v
        assert bits_equal(got[v][m:], C0[m:])
    args = (ta, tb, m, n, k, A.shape[0], B.shape[0], C0.shape[0])
    for xy in ("NN", "NT", "TN", "TT"):
        assert p.gemm_workspace(xy + "X", *args) == p.gemm_workspace(xy + "N", *args)
        assert p.gemm_workspace(xy + "X", *args) < p.gemm_workspace(xy + "T", *args)
        assert bits_equal(got[xy + "X"], got[xy + "N"])
        assert fro(got[xy + "X"][:m] - got[xy + "T"][:m]) <= bar
    assert p.gemm_workspace("NNX", *args) == 0


@pytest.mark.parametrize("uplo,trans", list(itertools.product([121, 122], [N, T])))
def test_syrk_fused_variants(handle, orc, ws, uplo, trans):
    """syrk_fused: "?X" against the oracle's "?F" tree and the unfused "?T" on the wanted
    triangle; no more workspace than "?F"; the other triangle keeps its bits (where "?T", like
    the reference's tree, scales it by beta)."""
    from rtatblas_amd import planner
    n, k = 213, 74
    p = planner.Planner("syrk_fused")
    assert p.variants() == ["FF", "FT", "FX", "TF", "TT", "TX"]
    A = orc.fill(k if trans == T else n, n if trans == T else k, seed=4)
    C0 = orc.fill(n, n, n + 2, seed=5, kind=1)
    tri = np.tril if uplo == 122 else np.triu
    other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
    bar = 16 * k * EPS * (fro(A) ** 2 + fro(C0[:n]))
    got = {}
    for v in p.variants():
        want = C0.copy(order="F")
        assert orc.syrk_variant(v.replace("X", "F"), uplo, trans, n, k, -1.0, A, 0.5, want) == 0
        dC = to_dev(C0)
        assert p.syrk(handle, v, uplo, trans, n, k, -1.0, to_dev(A), A.shape[0], 0.5, dC,
                      C0.shape[0], ws, ws.numel() * 8) == v
        got[v] = to_host(dC, C0.shape[0], n)
        assert fro(tri(got[v][:n]) - tri(want[:n])) <= bar, v
    args = (uplo, trans, n, k, A.shape[0], C0.shape[0])
    for a in "FT":
        assert p.syrk_workspace(a + "X", *args) == p.syrk_workspace(a + "F", *args)
        assert p.syrk_workspace(a + "X", *args) < p.syrk_workspace(a + "T", *args)
        assert bits_equal(got[a + "X"], got[a + "F"])
        assert bits_equal(other(got[a + "X"][:n]), other(C0[:n]))
        assert fro(tri(got[a + "X"][:n]) - tri(got[a + "T"][:n])) <= bar
    assert p.syrk_workspace("FX", *args) == 0


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [121, 122], [N, T], [131, 132])))
def test_trsm_fused_variants(handle, orc, ws, side, uplo, trans, diag):
    """trsm_fused: "X?" against the oracle's "F?" tree and the unfused "T?"; the workspace of
    "F?" (none for "XF")."""
    from rtatblas_amd import planner
    m, n = 143, 152
    p = planner.Planner("trsm_fused")
    assert p.variants() == ["FF", "FT", "TF", "TT", "XF", "XT"]
    na = m if side == 141 else n
    A = orc.fill(na, na, seed=6, kind=4)
    B0 = orc.fill(m, n, m + 1, seed=7)
    dA = to_dev(A)
    got = {}
    for v in p.variants():
        want = B0.copy(order="F")
        assert orc.trsm_variant(v.replace("X", "F"), side, uplo, trans, diag, m, n, 1.0, A, want) == 0
        dB = to_dev(B0)
        assert p.trsm(handle, v, side, uplo, trans, diag, m, n, 1.0, dA, na, dB, m + 1, ws,
                      ws.numel() * 8) == v
        got[v] = to_host(dB, m + 1, n)
        assert np.allclose(got[v][:m], want[:m], rtol=1e-9, atol=1e-12), v
        assert bits_equal(got[v][m:], B0[m:])
    args = (side, uplo, trans, diag, m, n, na, m + 1)
    for a in "FT":
        assert p.trsm_workspace("X" + a, *args) == p.trsm_workspace("F" + a, *args)
        assert p.trsm_workspace("X" + a, *args) < p.trsm_workspace("T" + a, *args)
        assert bits_equal(got["X" + a], got["F" + a])
        assert np.allclose(got["X" + a][:m], got["T" + a][:m], rtol=1e-9, atol=1e-12)
    assert p.trsm_workspace("XF", *args) == 0
