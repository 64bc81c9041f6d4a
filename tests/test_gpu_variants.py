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
    # three passes over the variants, the second backwards
    assert seen[:24] == p.variants() + p.variants()[::-1] + p.variants()
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
    """gemm_fused spells [ta][tb][tc] with tc in N / T / X.  Every variant against the
    oracle's tree (X has the value of N there); "xyX" must need exactly the workspace of "xyN"
    (none at all for "NNX"), equal "xyN" bit for bit, and agree with the unfused tree "xyT"
    within the bar."""
    from rtatblas_amd import planner
    m, n, k = 170, 145, 162
    p = planner.Planner("gemm_fused")
    # "X" can be asked for by name; it is the tree of "N", so the planner does not enumerate it
    assert p.variants() == ["".join(v) for v in itertools.product("NT", "NT", "NT")]
    names = ["".join(v) for v in itertools.product("NT", "NT", "NTX")]
    A = orc.fill(k if ta == T else m, m if ta == T else k, (k if ta == T else m) + 3, seed=1)
    B = orc.fill(n if tb == T else k, k if tb == T else n, (n if tb == T else k) + 1, seed=2)
    C0 = orc.fill(m, n, m + 3, seed=3)
    dA, dB = to_dev(A), to_dev(B)
    Al, Bl = A[: (k if ta == T else m)], B[: (n if tb == T else k)]
    bar = gemm_bound(k, 1.0, Al, Bl, 0.5, C0[:m])
    got = {}
    for v in names:
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
    assert p.variants() == ["FF", "FT", "TF", "TT"]
    names = ["FF", "FT", "FX", "TF", "TT", "TX"]
    A = orc.fill(k if trans == T else n, n if trans == T else k, seed=4)
    C0 = orc.fill(n, n, n + 2, seed=5, kind=1)
    tri = np.tril if uplo == 122 else np.triu
    other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
    bar = 16 * k * EPS * (fro(A) ** 2 + fro(C0[:n]))
    got = {}
    for v in names:
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
    assert p.variants() == ["FF", "FT", "TF", "TT"]
    names = ["FF", "FT", "TF", "TT", "XF", "XT"]
    na = m if side == 141 else n
    A = orc.fill(na, na, seed=6, kind=4)
    B0 = orc.fill(m, n, m + 1, seed=7)
    dA = to_dev(A)
    got = {}
    for v in names:
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


# ---- kernel-option families: the reference's switches x tile shape x tail mode (x panel) -------

def test_kernel_option_words_are_validated_and_reported(handle, orc):
    """The word the *_ex entry points take: fields out of range and stray bits are refused
    before anything is launched; rtat_last_launch names what a call ran on."""
    from rtatblas_amd import native
    m = n = 2048
    k = 512
    A, B = to_dev(orc.fill(m, k, seed=1)), to_dev(orc.fill(k, n, seed=2))
    C = to_dev(np.zeros((m, n), order="F"))
    for word in (5, 0x300, 0x3000, 0x10000, -1, native.kernel_options(2, 3, 0),
                 native.kernel_options(2, 0, 3)):
        assert handle.dgemm(N, N, m, n, k, 1.0, A, m, B, k, 0.0, C, m, variant=word,
                            check=False) == 3, hex(word)
        assert handle.dsyrk(122, N, n, k, 1.0, A, m, 0.0, C, m, variant=word, check=False) == 3
        assert handle.dtrsm(141, 122, N, 131, m, n, 1.0, C, m, C, m, variant=word, check=False) == 3
    # 256 tiles of 128 x 128 on 512 workgroup slots (256 CUs): the fixed rule leaves them whole
    # (half a round, k short of 128 panels), "split" cuts every one in two, "whole" never cuts
    for tail, cut in ((native.TAIL_AUTO, False), (native.TAIL_WHOLE, False), (native.TAIL_SPLIT, True)):
        handle.dgemm(N, N, m, n, k, 1.0, A, m, B, k, 0.0, C, m,
                     variant=native.kernel_options(native.GEMM_T128x128, tail))
        info = handle.last_launch()
        assert info["tile"] == "128x128" and info["tiles"] == 256
        if handle.peaks()[2] == 256:
            assert (info["split_tiles"] > 0) == cut and (info["split_slices"] >= 2) == cut, info
    handle.dgemm(N, N, m, n, k, 1.0, A, m, B, k, 0.0, C, m, variant=native.GEMM_T256x128)
    assert handle.last_launch()["tile"] == "256x128"
    handle.dgemm(N, N, 256, 256, 256, 1.0, A, m, B, k, 0.0, C, m)
    assert handle.last_launch()["tile"] == "32x32"           # the automatic choice's own shape
    L = to_dev(orc.fill(2048, 2048, seed=3, kind=4))
    Bt = to_dev(orc.fill(2048, 64, seed=4))
    for panel, rows in ((native.PANEL_512, 512), (native.PANEL_1024, 1024)):
        handle.dtrsm(141, 122, N, 131, 2048, 64, 1.0, L, 2048, Bt, 2048,
                     variant=native.kernel_options(panel=panel))
        assert handle.last_launch()["trsm_panel_rows"] == rows
    assert [native.tail_mode_name(i) for i in range(4)] == ["auto", "whole", "split", None]
    assert [native.trsm_panel_name(i) for i in range(4)] == ["auto", "512", "1024", None]


@pytest.fixture(scope="module")
def big_ws():
    import torch
    return torch.full((16 << 20,), float("nan"), dtype=torch.float64, device="cuda")


def test_gemm_pad_tile_variants_against_the_default(handle, orc, big_ws):
    """All 960 variants of gemm_pad_tile on one problem whose tiles leave a partial round for
    every shape and whose k is long enough to be cut: each against the oracle's tree of its
    letters (the kernel options have no counterpart there: they must not change the result
    beyond rounding) and against the default variant."""
    from rtatblas_amd import planner
    m, n, k = 300, 260, 530
    p = planner.Planner("gemm_pad_tile")
    names = p.variants()
    assert len(names) == 960 and names[0] == "NNNNNN/auto/auto"
    A, B = orc.fill(k, m, k + 3, seed=1), orc.fill(k, n, k + 1, seed=2)      # opA = T, opB = N
    C0 = orc.fill(m, n, m + 3, seed=3)
    dA, dB = to_dev(A), to_dev(B)
    bar = gemm_bound(k, 1.0, A[:k], B[:k], 0.5, C0[:m])
    wants, got = {}, {}
    for v in names:
        letters = v.split("/")[0]
        if letters not in wants:
            wants[letters] = C0.copy(order="F")
            assert orc.gemm_variant(letters, T, N, m, n, k, 1.0, A, B, 0.5, wants[letters]) == 0
        dC = to_dev(C0)
        assert p.gemm(handle, v, T, N, m, n, k, 1.0, dA, k + 3, dB, k + 1, 0.5, dC, m + 3, big_ws,
                      big_ws.numel() * 8) == v
        got[v] = to_host(dC, m + 3, n)
        assert fro(got[v][:m] - wants[letters][:m]) <= bar, v
        assert bits_equal(got[v][m:], C0[m:]), v
        assert fro(got[v][:m] - got[names[0]][:m]) <= 2 * bar, v
        assert p.gemm_workspace(v, T, N, m, n, k, k + 3, k + 1, m + 3) == \
            orc.gemm_workspace(letters, T, N, m, n, k, k + 3, k + 1, m + 3), v
    # nine tiles of 128 x 128 on 512 slots: the fixed rule cuts them along K as "split" does,
    # "whole" computes each in one workgroup - another order of summation, other bits
    assert bits_equal(got["NNNNNN/128x128/split"], got["NNNNNN/128x128/auto"])
    assert not bits_equal(got["NNNNNN/128x128/split"], got["NNNNNN/128x128/whole"])


@pytest.mark.parametrize("uplo,trans", [(122, N), (121, T)])
def test_syrk_tile_variants_against_the_default(handle, orc, big_ws, uplo, trans):
    """All 60 variants of syrk_tile against the oracle's tree of their letters and against the
    default variant, on a triangle that leaves every shape a partial round and a k that can
    be cut; the other triangle keeps its bits unless the tree is a "?T" one."""
    from rtatblas_amd import planner
    n, k = 700, 600
    p = planner.Planner("syrk_tile")
    names = p.variants()
    assert len(names) == 60 and names[0] == "FF/auto/auto"
    A = orc.fill(k if trans == T else n, n if trans == T else k, seed=4)
    C0 = orc.fill(n, n, n + 2, seed=5, kind=1)
    dA = to_dev(A)
    tri = np.tril if uplo == 122 else np.triu
    other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
    bar = 16 * k * EPS * (fro(A) ** 2 + fro(C0[:n]))
    wants, got = {}, {}
    for v in names:
        letters = v.split("/")[0]
        if letters not in wants:
            wants[letters] = C0.copy(order="F")
            assert orc.syrk_variant(letters, uplo, trans, n, k, -1.0, A, 0.5, wants[letters]) == 0
        dC = to_dev(C0)
        assert p.syrk(handle, v, uplo, trans, n, k, -1.0, dA, A.shape[0], 0.5, dC, n + 2, big_ws,
                      big_ws.numel() * 8) == v
        got[v] = to_host(dC, n + 2, n)
        assert fro(tri(got[v][:n]) - tri(wants[letters][:n])) <= bar, v
        assert fro(tri(got[v][:n]) - tri(got[names[0]][:n])) <= 2 * bar, v
        if letters[1] == "F":
            assert bits_equal(other(got[v][:n]), other(C0[:n])), v
        else:
            assert bits_equal(other(got[v][:n]), other(wants[letters][:n])), v
        assert bits_equal(got[v][n:], C0[n:]), v
        assert p.syrk_workspace(v, uplo, trans, n, k, A.shape[0], n + 2) == \
            orc.syrk_workspace(letters, uplo, trans, n, k, A.shape[0], n + 2), v


@pytest.mark.parametrize("side,uplo,trans,diag", [(141, 122, N, 131), (142, 121, T, 132)])
def test_trsm_tile_variants_against_the_default(handle, orc, big_ws, side, uplo, trans, diag):
    """All 180 variants of trsm_tile - tile shape and tail mode of the trailing updates, 512-
    and 1024-row panels - against the oracle's tree of their letters and against the default
    variant, on a triangle of more than one tall panel."""
    from rtatblas_amd import planner
    na, nrhs = 1100, 210
    m, n = (na, nrhs) if side == 141 else (nrhs, na)
    p = planner.Planner("trsm_tile")
    names = p.variants()
    assert len(names) == 180 and names[0] == "FF/auto/auto/auto"
    A = orc.fill(na, na, seed=6, kind=4)
    B0 = orc.fill(m, n, m + 1, seed=7)
    dA = to_dev(A)
    wants, got = {}, {}
    for v in names:
        letters = v.split("/")[0]
        if letters not in wants:
            wants[letters] = B0.copy(order="F")
            assert orc.trsm_variant(letters, side, uplo, trans, diag, m, n, 1.0, A,
                                    wants[letters]) == 0
        dB = to_dev(B0)
        assert p.trsm(handle, v, side, uplo, trans, diag, m, n, 1.0, dA, na, dB, m + 1, big_ws,
                      big_ws.numel() * 8) == v
        got[v] = to_host(dB, m + 1, n)
        assert np.allclose(got[v][:m], wants[letters][:m], rtol=1e-9, atol=1e-12), v
        assert np.allclose(got[v][:m], got[names[0]][:m], rtol=1e-9, atol=1e-12), v
        assert bits_equal(got[v][m:], B0[m:]), v
        assert p.trsm_workspace(v, side, uplo, trans, diag, m, n, na, m + 1) == \
            orc.trsm_workspace(letters, side, uplo, trans, diag, m, n, na, m + 1), v


def test_filtered_autotune_over_a_kernel_option_family(handle, orc, big_ws):
    """trsm_tile under a pattern filter: only admitted variants are explored, the plan is one
    of them, the plan file round-trips, and a filter learned from the report admits the
    plan and the default for a problem of the same class."""
    from rtatblas_amd import planner
    m, n = 1024, 512
    p = planner.Planner("trsm_tile")
    p.set_filter("FF/*/auto/*")
    admitted = p.trsm_admitted(141, 122, N, 131, m, n)
    assert len(admitted) == 15 and admitted[0] == "FF/auto/auto/auto"
    p.set_refinement(0)
    A = to_dev(orc.fill(m, m, seed=6, kind=4))
    B = to_dev(orc.fill(m, n, seed=7))
    seen = [p.trsm(handle, None, 141, 122, N, 131, m, n, 1.0, A, m, B, m, big_ws, big_ws.numel() * 8)
            for _ in range(60)]
    assert seen[:45] == admitted + admitted[::-1] + admitted
    assert len(set(seen[45:])) == 1 and seen[-1] in admitted
    plans = p.plans()
    assert "/".join([plans[0]["plan"]["swap_side"] + plans[0]["plan"]["transA"],
                     plans[0]["plan"]["tile"], plans[0]["plan"]["tail"],
                     plans[0]["plan"]["panel"]]) == seen[-1]
    q = planner.Planner("trsm_tile")
    assert q.load_plans(plans) == 1
    assert q.trsm(handle, None, 141, 122, N, 131, m, n, 1.0, A, m, B, m, big_ws,
                  big_ws.numel() * 8) == seen[-1]
    r = planner.Planner("trsm_tile")
    assert r.learn_filter(p.stats(), 0.05) == 1
    kept = r.trsm_admitted(141, 122, N, 131, m + 8, n)         # same class: flags and size bucket
    assert "FF/auto/auto/auto" in kept and len(kept) <= 15
    best = min(p.stats()[0]["options"], key=lambda o: sorted(o["times"])[len(o["times"]) // 2])
    assert "/".join([best["option"]["swap_side"] + best["option"]["transA"], best["option"]["tile"],
                     best["option"]["tail"], best["option"]["panel"]]) in kept
    assert len(r.trsm_admitted(142, 122, N, 131, m, n)) == 180  # a class nothing is known about
