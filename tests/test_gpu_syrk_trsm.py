"""GPU parity of rtat_dsyrk and rtat_dtrsm (through the C ABI) against the CPU oracle.
Bars: SYRK normwise 16 k eps on the referenced triangle, the other triangle bit-unchanged;
TRSM by backward residual ||op(A) X - alpha B||_F <= 16 M eps ||A||_F ||X||_F."""
import itertools

import numpy as np
import pytest

from util import EPS, bits_equal, fro, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112
OPS = {"N": N, "T": T}
UP, LO = 121, 122


def rnd(rng, m, n, ld=None):
    ld = max(m, 1) if ld is None else ld
    a = np.full((ld, n), np.nan, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n))
    return a


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("uplo,trans", list(itertools.product([UP, LO], "NT")))
@pytest.mark.parametrize("n,k,extra", [(72, 56, 0), (213, 74, 0), (300, 130, 3), (512, 64, 0),
                                       (330, 1100, 0), (700, 500, 1), (97, 250, 3)])
def test_syrk_against_oracle(handle, orc, uplo, trans, n, k, extra, variant):
    # (with the automatic shape, all but the fifth run as one launch of 32 x 32 tiles)
    rng = np.random.default_rng(n + k + uplo)
    ar, ac = (k, n) if trans == "T" else (n, k)
    A = rnd(rng, ar, ac, ar + extra)
    C0 = rnd(rng, n, n, n + extra)
    want = C0.copy(order="F")
    orc.dsyrk(uplo, OPS[trans], n, k, -1.0, A, 1.0, want)
    dC = to_dev(C0)
    handle.dsyrk(uplo, OPS[trans], n, k, -1.0, to_dev(A), A.shape[0], 1.0, dC, C0.shape[0],
                 variant=variant)
    got = to_host(dC, C0.shape[0], n)
    tri = np.tril if uplo == LO else np.triu
    bound = 16 * k * EPS * (fro(A[:ar]) ** 2 + fro(C0[:n]))
    assert fro(tri(got[:n]) - tri(want[:n])) <= bound
    other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
    assert bits_equal(other(got[:n]), other(C0[:n]))      # other triangle untouched
    assert bits_equal(got[n:], C0[n:])                    # padding untouched


@pytest.mark.parametrize("variant", [0, 2, 3])
@pytest.mark.parametrize("uplo,trans", list(itertools.product([UP, LO], "NT")))
def test_syrk_tail_tiles_cut_into_pieces(handle, orc, uplo, trans, variant):
    """A triangle of more tiles than one round of workgroups whose leftover is computed as
    64 x 64 pieces: pieces wholly outside the triangle are skipped, pieces on the diagonal
    mask their stores."""
    orc.cblas_on()
    try:
        n, k = 5237, 24
        rng = np.random.default_rng(n + uplo)
        ar, ac = (k, n) if trans == "T" else (n, k)
        A = rnd(rng, ar, ac, ar + 1)
        C0 = rnd(rng, n, n, n + 2)
        want = C0.copy(order="F")
        orc.dsyrk(uplo, OPS[trans], n, k, 1.0, A, -1.0, want)
        dC = to_dev(C0)
        handle.dsyrk(uplo, OPS[trans], n, k, 1.0, to_dev(A), A.shape[0], -1.0, dC, C0.shape[0],
                     variant=variant)
        got = to_host(dC, C0.shape[0], n)
        tri = np.tril if uplo == LO else np.triu
        bound = 16 * k * EPS * (fro(A[:ar]) ** 2 + fro(C0[:n]))
        assert fro(tri(got[:n]) - tri(want[:n])) <= bound
        other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
        assert bits_equal(other(got[:n]), other(C0[:n]))
        assert bits_equal(got[n:], C0[n:])
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 2, 3, 4])
@pytest.mark.parametrize("uplo,trans", list(itertools.product([UP, LO], "NT")))
def test_syrk_last_tiles_cut_along_k(handle, orc, uplo, trans, variant):
    """Triangles of a few more tiles than a multiple of the CU count (n = 2048 and 2900 on 256
    CUs, by shape): the last tiles are summed from K slices, the others are computed whole."""
    orc.cblas_on()
    try:
        for (n, k) in [(2048, 520), (2900, 300)]:
            rng = np.random.default_rng(n + uplo)
            ar, ac = (k, n) if trans == "T" else (n, k)
            A = rnd(rng, ar, ac, ar + 1)
            C0 = rnd(rng, n, n, n + 2)
            want = C0.copy(order="F")
            orc.dsyrk(uplo, OPS[trans], n, k, 1.0, A, 0.5, want)
            dC = to_dev(C0)
            handle.dsyrk(uplo, OPS[trans], n, k, 1.0, to_dev(A), A.shape[0], 0.5, dC,
                         C0.shape[0], variant=variant)
            got = to_host(dC, C0.shape[0], n)
            tri = np.tril if uplo == LO else np.triu
            bound = 16 * k * EPS * (fro(A[:ar]) ** 2 + fro(C0[:n]))
            assert fro(tri(got[:n]) - tri(want[:n])) <= bound
            other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
            assert bits_equal(other(got[:n]), other(C0[:n]))
            assert bits_equal(got[n:], C0[n:])
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 4])
@pytest.mark.parametrize("uplo,trans", list(itertools.product([UP, LO], "NT")))
def test_syrk_uneven_load_cut_along_k(handle, orc, uplo, trans, variant):
    """A triangle of 435 tiles of 64 x 64 (n = 1800) on 256 CUs, less than a round but 179 CUs
    one tile ahead of the rest: every tile is summed from K slices; with 325 tiles (n = 1600)
    only the 69 odd ones.  And triangles of at most
    one tile per CU (n = 1024, 1088), which the automatic shape choice may slice as well."""
    orc.cblas_on()
    try:
        for (n, k) in [(1800, 1000), (1600, 1000), (1024, 1024), (1088, 900)]:
            rng = np.random.default_rng(n + uplo + variant)
            ar, ac = (k, n) if trans == "T" else (n, k)
            A = rnd(rng, ar, ac, ar + 1)
            C0 = rnd(rng, n, n, n + 2)
            want = C0.copy(order="F")
            orc.dsyrk(uplo, OPS[trans], n, k, 1.0, A, 0.5, want)
            dC = to_dev(C0)
            handle.dsyrk(uplo, OPS[trans], n, k, 1.0, to_dev(A), A.shape[0], 0.5, dC, C0.shape[0],
                         variant=variant)
            got = to_host(dC, C0.shape[0], n)
            tri = np.tril if uplo == LO else np.triu
            bound = 16 * k * EPS * (fro(A[:ar]) ** 2 + fro(C0[:n]))
            assert fro(tri(got[:n]) - tri(want[:n])) <= bound
            other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
            assert bits_equal(other(got[:n]), other(C0[:n]))
            assert bits_equal(got[n:], C0[n:])
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 2])
@pytest.mark.parametrize("uplo,trans", list(itertools.product([UP, LO], "NT")))
def test_syrk_thin_edge_tiles(handle, orc, uplo, trans, variant):
    """A triangle of more than two rounds of 128 x 128 tiles (n = 5896 = 46 * 128 + 8) whose
    last tile row and column hold 8 rows / columns: those tiles skip their empty MFMA blocks."""
    orc.cblas_on()
    try:
        n, k = 5896, 40
        rng = np.random.default_rng(n + uplo + variant)
        ar, ac = (k, n) if trans == "T" else (n, k)
        A = rnd(rng, ar, ac, ar + 1)
        C0 = rnd(rng, n, n, n + 2)
        want = C0.copy(order="F")
        orc.dsyrk(uplo, OPS[trans], n, k, 1.0, A, 0.5, want)
        dC = to_dev(C0)
        handle.dsyrk(uplo, OPS[trans], n, k, 1.0, to_dev(A), A.shape[0], 0.5, dC, C0.shape[0],
                     variant=variant)
        got = to_host(dC, C0.shape[0], n)
        tri = np.tril if uplo == LO else np.triu
        bound = 16 * k * EPS * (fro(A[:ar]) ** 2 + fro(C0[:n]))
        assert fro(tri(got[:n]) - tri(want[:n])) <= bound
        other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
        assert bits_equal(other(got[:n]), other(C0[:n]))
        assert bits_equal(got[n:], C0[n:])
    finally:
        orc.cblas_off()


def test_syrk_beta_zero_and_scaling_only(handle, orc):
    rng = np.random.default_rng(9)
    n, k = 150, 40
    A = rnd(rng, n, k)
    C0 = np.full((n, n), np.nan, order="F")
    dC = to_dev(C0)
    handle.dsyrk(LO, N, n, k, 1.0, to_dev(A), n, 0.0, dC, n)
    got = to_host(dC, n, n)
    assert np.isfinite(np.tril(got)).all() and np.isnan(got[np.triu_indices(n, 1)]).all()
    assert fro(np.tril(got) - np.tril(A @ A.T)) <= 16 * k * EPS * fro(A) ** 2
    C1 = rnd(rng, n, n)
    dC = to_dev(C1)
    handle.dsyrk(UP, N, n, 0, 1.0, to_dev(A), n, 0.5, dC, n)          # k == 0: scale triangle
    got = to_host(dC, n, n)
    assert bits_equal(np.triu(got), np.triu(0.5 * C1))
    assert bits_equal(np.tril(got, -1), np.tril(C1, -1))


def make_tri(rng, n, lower, unit, scale):
    A = rng.uniform(-1, 1, (n, n)) / scale
    A = np.tril(A) if lower else np.triu(A)
    A[np.diag_indices(n)] = 1.0 + rng.uniform(0, 1, n)
    Tm = A.copy()
    if unit:
        Tm[np.diag_indices(n)] = 1.0
    stored = A.copy()
    mask = np.triu(np.ones((n, n), bool), 1) if lower else np.tril(np.ones((n, n), bool), -1)
    stored[mask] = np.nan                    # the other triangle must never be read
    if unit:
        stored[np.diag_indices(n)] = np.nan  # nor a unit diagonal
    return np.asfortranarray(stored), Tm


def check_trsm(handle, orc, side, uplo, trans, diag, m, n, alpha, scale, extra=0, variant=None):
    rng = np.random.default_rng(side * 3 + uplo * 5 + diag + m + n)
    na = m if side == 141 else n
    A, Tm = make_tri(rng, na, uplo == LO, diag == 132, scale)
    if extra:
        Ap = np.full((na + extra, na), np.nan, order="F")
        Ap[:na] = A
        A = Ap
    opT = Tm.T if trans == "T" else Tm
    B0 = rnd(rng, m, n, m + extra)
    dB = to_dev(B0)
    handle.dtrsm(side, uplo, OPS[trans], diag, m, n, alpha, to_dev(A), A.shape[0], dB,
                 B0.shape[0], variant=variant)
    got = to_host(dB, B0.shape[0], n)
    X = got[:m]
    assert np.isfinite(X).all(), "NaN leaked from the unreferenced triangle"
    resid = (opT @ X - alpha * B0[:m]) if side == 141 else (X @ opT - alpha * B0[:m])
    assert fro(resid) <= 16 * na * EPS * fro(opT) * fro(X)
    assert bits_equal(got[m:], B0[m:])
    want = B0.copy(order="F")
    orc.dtrsm(side, uplo, OPS[trans], diag, m, n, alpha, np.asfortranarray(A), want)
    assert np.allclose(X, want[:m], rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [UP, LO], "NT", [131, 132])))
def test_trsm_all_sixteen_small(handle, orc, side, uplo, trans, diag):
    check_trsm(handle, orc, side, uplo, trans, diag, 10, 12, 1.0, 1.0)        # matrixop_test.cpp:114
    check_trsm(handle, orc, side, uplo, trans, diag, 435, 527, 1.0, 435.0)    # executor_test.cpp:136
    check_trsm(handle, orc, side, uplo, trans, diag, 300, 257, -0.5, 300.0, extra=3)


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [UP, LO], "NT", [131, 132])))
def test_trsm_tall_panels(handle, orc, side, uplo, trans, diag):
    """Between 2048 and 4096 right-hand sides (half a workgroup to one workgroup per CU) the
    solve runs on 1024-row panels: two panels, the second ragged, with an odd leading
    dimension in one of the cases."""
    orc.cblas_on()
    try:
        na, nrhs = 1300, 2100
        m, n = (na, nrhs) if side == 141 else (nrhs, na)
        check_trsm(handle, orc, side, uplo, trans, diag, m, n, 1.0, float(na),
                   extra=3 if diag == 132 else 0)
    finally:
        orc.cblas_off()


PANEL_ORDERS = (600, 700, 770, 900, 1100, 1224, 1324, 1424)   # last panels of 5 .. 8, 1 .. 4 blocks


@pytest.mark.parametrize("case", list(enumerate(itertools.product([141, 142], [UP, LO], "NT",
                                                                   [131, 132]))))
def test_trsm_panel_block_counts_and_widths(handle, orc, case):
    """The panel kernel is straight-line code per block count of the panel (1 to 8), per
    orientation of the slab (left- or right-hand solve) and per width: 32 right-hand sides to
    the workgroup past 16 per CU (4200 here), 16 below (2100), 1024 rows at a time unless 512
    are asked for.  Full panels and ragged last ones of every block count in both widths, a
    last workgroup with 8 or 4 right-hand sides, an odd leading dimension in half of the cases;
    the rows and columns of B past m x n stay as they were (check_trsm)."""
    from rtatblas_amd import native
    idx, (side, uplo, trans, diag) = case
    on256 = handle.peaks()[2] == 256
    orc.cblas_on()
    try:
        for na, nrhs, panel in ((PANEL_ORDERS[(2 * idx) % 8], 4200, None),
                                (PANEL_ORDERS[(2 * idx + 1) % 8], 4200, None),
                                (PANEL_ORDERS[(idx + 3) % 8], 4200, native.PANEL_512),
                                (PANEL_ORDERS[(2 * idx + 5) % 8], 2100, None),
                                (PANEL_ORDERS[(2 * idx + 2) % 8], 2100, None),
                                (PANEL_ORDERS[(idx + 6) % 8], 2100, native.PANEL_512)):
            m, n = (na, nrhs) if side == 141 else (nrhs, na)
            variant = None if panel is None else native.kernel_options(panel=panel)
            check_trsm(handle, orc, side, uplo, trans, diag, m, n, 0.75, float(na),
                       extra=3 if uplo == UP else 0, variant=variant)
            info = handle.last_launch()
            if on256:
                assert (info["trsm_panel_rows"], info["trsm_panel_width"]) == \
                    (1024 if panel is None else 512, 32 if nrhs == 4200 else 16)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [1, 2, 3])
def test_trsm_kernel_variants(handle, orc, variant):
    check_trsm(handle, orc, 141, LO, "N", 131, 640, 384, 1.0, 640.0, variant=variant)
    check_trsm(handle, orc, 142, UP, "T", 132, 384, 640, 1.0, 640.0, variant=variant)


def test_trsm_diagonal_alpha_zero_and_errors(handle):
    import torch
    rng = np.random.default_rng(4)
    d = 1.0 + rng.uniform(0, 1, 200)
    A = np.asfortranarray(np.diag(d))
    B0 = rnd(rng, 200, 50)
    dB = to_dev(B0)
    handle.dtrsm(141, LO, N, 131, 200, 50, 1.0, to_dev(A), 200, dB, 200)
    assert np.allclose(to_host(dB, 200, 50), B0 / d[:, None], rtol=4 * EPS, atol=0)
    dB = to_dev(np.full((200, 50), np.nan, order="F"))
    handle.dtrsm(141, LO, N, 131, 200, 50, 0.0, to_dev(A), 200, dB, 200)
    assert (to_host(dB, 200, 50) == 0).all()
    x = torch.zeros(8, dtype=torch.float64, device="cuda")
    assert handle.dtrsm(141, LO, N, 131, 0, 5, 1.0, x, 1, x, 1, check=False) == 0
    assert handle.dtrsm(141, LO, N, 131, 8, 8, 1.0, x, 4, x, 8, check=False) == 3
    assert handle.dtrsm(141, 5, N, 131, 8, 8, 1.0, x, 8, x, 8, check=False) == 10


def test_trsm_caller_workspace(handle, orc):
    import torch
    from rtatblas_amd import native
    need = native.load().rtat_dtrsm_workspace_bytes(141, 300, 10)
    ws = torch.empty(need // 8, dtype=torch.float64, device="cuda")
    handle.set_workspace(ws, need)
    try:
        check_trsm(handle, orc, 141, LO, "N", 131, 300, 10, 1.0, 300.0)
        small = torch.empty(16, dtype=torch.float64, device="cuda")
        handle.set_workspace(small, 128)
        x = torch.ones(300 * 300, dtype=torch.float64, device="cuda")
        assert handle.dtrsm(141, LO, N, 131, 300, 10, 1.0, x, 300, x, 300, check=False) == 2
    finally:
        handle.set_workspace(None, 0)


def test_trsm_config_c5_reduced(handle, orc):
    """Left / lower / N / non-unit, A from the well-conditioned generator (strict upper = NaN),
    M = N = 2048: backward residual and agreement with host CBLAS."""
    import torch
    n = 2048
    orc.cblas_on()
    try:
        A = orc.fill(n, n, seed=1, kind=2)
        B0 = orc.fill(n, n, seed=2)
        dA = torch.empty(n * n, dtype=torch.float64, device="cuda")
        dB = torch.empty_like(dA)
        handle.dfill(dA, n, n, n, 1, 2)
        handle.dfill(dB, n, n, n, 2, 0)
        handle.dtrsm(141, LO, N, 131, n, n, 1.0, dA, n, dB, n)
        X = to_host(dB, n, n)
        L = np.tril(np.nan_to_num(A))
        assert fro(L @ X - B0) <= 16 * n * EPS * fro(L) * fro(X)
        want = B0.copy(order="F")
        orc.dtrsm(141, LO, N, 131, n, n, 1.0, np.asfortranarray(np.nan_to_num(A)), want)
        assert np.allclose(X, want, rtol=1e-9, atol=1e-11)
    finally:
        orc.cblas_off()


def test_full_size_syrk_and_trsm_properties(handle):
    """Config sizes (SYRK N=8192 K=2048; TRSM M=N=8192) checked through properties that need
    no CPU product: SYRK against DGEMM on the device, TRSM by its backward residual computed
    with DGEMM."""
    import torch
    n, k = 8192, 2048
    A = torch.empty(n * k, dtype=torch.float64, device="cuda")
    C = torch.empty(n * n, dtype=torch.float64, device="cuda")
    G = torch.empty_like(C)
    handle.dfill(A, n, k, n, 1)
    handle.dfill(C, n, n, n, 3, 1)
    G.copy_(C)
    handle.dsyrk(LO, N, n, k, 1.0, A, n, 1.0, C, n)
    handle.dgemm(N, T, n, n, k, 1.0, A, n, A, n, 1.0, G, n)
    Cm, Gm = C.view(n, n), G.view(n, n)          # row-major views = transposes; triu <-> lower
    diff = torch.triu(Cm - Gm)
    assert float(diff.norm()) <= 16 * k * EPS * (float(A.norm()) ** 2 + float(G.norm()))
    del A, C, G, diff
    m = 8192
    L = torch.empty(m * m, dtype=torch.float64, device="cuda")
    B = torch.empty_like(L)
    X = torch.empty_like(L)
    handle.dfill(L, m, m, m, 1, 2)
    handle.dfill(B, m, m, m, 2, 0)
    X.copy_(B)
    handle.dtrsm(141, LO, N, 131, m, m, 1.0, L, m, X, m)
    assert bool(torch.isfinite(X).all())
    Lz = torch.nan_to_num(L)                      # strict upper NaN -> 0 for the residual product
    R = B.clone()
    handle.dgemm(N, N, m, m, m, 1.0, Lz, m, X, m, -1.0, R, m)
    assert float(R.norm()) <= 16 * m * EPS * float(Lz.norm()) * float(X.norm())
