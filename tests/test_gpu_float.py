"""GPU parity of the single-precision entry points (rtat_sgemm / rtat_ssyrk / rtat_strsm /
rtat_sgeam, through the C ABI) — the float instantiations of the reference's templates
(src/matrix_ops/matrixop.h:33-43, 64-73, 96-105, 127-137).

The checker is the CPU oracle's double-precision routine on the same float inputs (exactly
representable in double); bar: ||C - C_ref||_F <= 16 k eps32 (|alpha| ||A|| ||B|| + |beta| ||C0||)
for GEMM / SYRK, backward residual 16 n eps32 ||A|| ||X|| for TRSM, bit-exact for copies."""
import itertools

import numpy as np
import pytest

from util import fro, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112
OPS = {"N": N, "T": T}
UP, LO = 121, 122
EPS32 = float(np.finfo(np.float32).eps)


def rnd32(rng, m, n, ld=None):
    ld = max(m, 1) if ld is None else ld
    a = np.full((ld, n), np.nan, dtype=np.float32, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    return a


def same_bits(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


def run_sgemm(handle, orc, ta, tb, m, n, k, alpha, beta, extra=(0, 0, 0), seed=0, variant=None):
    rng = np.random.default_rng(seed + m + 7 * n + 13 * k)
    ar, ac = (k, m) if ta == "T" else (m, k)
    br, bc = (n, k) if tb == "T" else (k, n)
    A = rnd32(rng, ar, ac, max(ar, 1) + extra[0])
    B = rnd32(rng, br, bc, max(br, 1) + extra[1])
    C0 = rnd32(rng, m, n, max(m, 1) + extra[2])
    want = np.asfortranarray(C0.astype(np.float64))
    orc.dgemm(OPS[ta], OPS[tb], m, n, k, alpha, np.asfortranarray(A.astype(np.float64)),
              np.asfortranarray(B.astype(np.float64)), beta, want)
    dC = to_dev(C0)
    handle.sgemm(OPS[ta], OPS[tb], m, n, k, alpha, to_dev(A), A.shape[0], to_dev(B), B.shape[0],
                 beta, dC, C0.shape[0], variant=variant)
    got = to_host(dC, C0.shape[0], n)
    c0 = 0.0 if beta == 0.0 else abs(beta) * fro(C0[:m].astype(np.float64))
    bound = 16 * max(k, 1) * EPS32 * (abs(alpha) * fro(A[:ar].astype(np.float64))
                                      * fro(B[:br].astype(np.float64)) + c0)
    err = fro(got[:m].astype(np.float64) - want[:m])
    assert err <= bound, (ta, tb, m, n, k, err, bound)
    assert same_bits(got[m:], C0[m:])          # padding rows of C are never written


@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
def test_sgemm_reference_shapes_and_ragged_edges(handle, orc, ta, tb):
    # tests/executor_test.cpp:15-17 (70,45,62) is the float executor test's shape
    for (m, n, k) in [(70, 45, 62), (26, 27, 34), (1, 1, 1), (17, 515, 16)]:
        run_sgemm(handle, orc, ta, tb, m, n, k, 1.0, 0.0)
    orc.cblas_on()
    try:
        for (m, n, k) in [(256, 256, 64), (512, 384, 130), (301, 203, 200), (130, 67, 161),
                          (1024, 640, 96), (300, 200, 2000)]:
            ar = k if ta == "T" else m
            br = n if tb == "T" else k
            # leading dimensions that are whole 16-byte vectors (vector loads) ...
            run_sgemm(handle, orc, ta, tb, m, n, k, 1.0, 0.5,
                      extra=((-ar) % 4, (-br) % 4, (-m) % 4))
            # ... and ones that are not (element-wise loads)
            run_sgemm(handle, orc, ta, tb, m, n, k, -0.75, 0.0,
                      extra=((-ar) % 4 + 1, (-br) % 4 + 3, 1), seed=3)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 2, 3, 4])
def test_sgemm_last_tiles_cut_along_k(handle, orc, variant):
    """Single precision through the K-sliced leftovers: a few tiles more than a multiple of the
    CU count (only those are cut), and a leftover of under half a round (cut as a whole)."""
    orc.cblas_on()
    try:
        for ta, tb in [("N", "N"), ("T", "N"), ("N", "T")]:
            run_sgemm(handle, orc, ta, tb, 1500, 1400, 1200, 1.0, 0.5, variant=variant)
            run_sgemm(handle, orc, ta, tb, 2100, 2048, 530, -0.5, 0.0, extra=(1, 3, 1),
                      variant=variant)
            run_sgemm(handle, orc, ta, tb, 2400, 2300, 800, 1.0, 1.0, variant=variant)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [1, 2, 3, 4])
def test_sgemm_every_tile_shape(handle, orc, variant):
    """The explicit tile shapes of rtat_sgemm_ex / rtat_ssyrk_ex / rtat_strsm_ex."""
    orc.cblas_on()
    try:
        for ta, tb in itertools.product("NT", "NT"):
            run_sgemm(handle, orc, ta, tb, 301, 203, 200, 1.0, 0.5, variant=variant)
            run_sgemm(handle, orc, ta, tb, 130, 515, 97, -0.5, 0.0, extra=(1, 3, 1), variant=variant)
    finally:
        orc.cblas_off()
    rng = np.random.default_rng(variant)
    n, k = 300, 130
    A = rnd32(rng, n, k)
    C0 = rnd32(rng, n, n)
    want = np.asfortranarray(C0.astype(np.float64))
    orc.dsyrk(LO, N, n, k, 1.0, np.asfortranarray(A.astype(np.float64)), 1.0, want)
    dC = to_dev(C0)
    handle.ssyrk(LO, N, n, k, 1.0, to_dev(A), n, 1.0, dC, n, variant=variant)
    got = to_host(dC, n, n)
    assert fro(np.tril(got.astype(np.float64)) - np.tril(want)) <= \
        16 * k * EPS32 * (fro(A.astype(np.float64)) ** 2 + fro(C0.astype(np.float64)))
    assert same_bits(np.triu(got, 1), np.triu(C0, 1))
    m = 1100                                    # two panels: one GEMM update with this shape
    L, Tm = make_tri32(rng, m, True, False, float(m))
    B0 = rnd32(rng, m, 70)
    dB = to_dev(B0)
    handle.strsm(141, LO, N, 131, m, 70, 1.0, to_dev(L), m, dB, m, variant=variant)
    X = to_host(dB, m, 70).astype(np.float64)
    assert fro(Tm @ X - B0.astype(np.float64)) <= 16 * m * EPS32 * fro(Tm) * fro(X)
    assert handle.sgemm(N, N, 8, 8, 8, 1.0, dB, 8, dB, 8, 0.0, dC, 8, variant=17, check=False) == 3


def test_sgemm_small_problems_on_32x32_tiles(handle, orc):
    """Small problems through the automatic choice: one launch of 32 x 32 tiles (k up to 32
    panels of 32 floats; 48 from one tile per CU on)."""
    orc.cblas_on()
    try:
        for ta, tb in itertools.product("NT", "NT"):
            for (m, n, k) in [(512, 512, 1024), (200, 300, 400), (97, 61, 1000), (33, 31, 17),
                              (512, 512, 1536), (2048, 32, 250)]:
                run_sgemm(handle, orc, ta, tb, m, n, k, 1.0, 0.5, extra=(1, 3, 1))
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [1, 2, 3, 4])
def test_sgemm_thin_edge_tiles(handle, orc, variant):
    """Two rounds of tiles or more with a last tile row of 8 rows and a last tile column of 3
    columns (24 and 40 of 64 for the smallest shape): those tiles skip the MFMA blocks that
    hold no element of C.  Same bar as everywhere; the rows behind C keep their bits."""
    orc.cblas_on()
    try:
        for ta, tb in itertools.product("NT", "NT"):
            run_sgemm(handle, orc, ta, tb, 4104, 4099, 70, 1.0, 0.5, extra=(1, 3, 2),
                      variant=variant)
    finally:
        orc.cblas_off()


def test_sgemm_beta_zero_ignores_nan_and_identity_is_exact(handle):
    rng = np.random.default_rng(11)
    n = 200
    A = rnd32(rng, n, n)
    I = np.asfortranarray(np.eye(n, dtype=np.float32))
    dC = to_dev(np.full((n, n), np.nan, dtype=np.float32, order="F"))
    handle.sgemm(N, N, n, n, n, 1.0, to_dev(A), n, to_dev(I), n, 0.0, dC, n)
    assert same_bits(to_host(dC, n, n), A)
    handle.sgemm(T, N, n, n, n, 1.0, to_dev(A), n, to_dev(I), n, 0.0, dC, n)
    assert same_bits(to_host(dC, n, n), np.asfortranarray(A.T))


@pytest.mark.parametrize("uplo,trans", list(itertools.product([UP, LO], "NT")))
@pytest.mark.parametrize("n,k,extra", [(72, 56, 0), (213, 74, 0), (300, 130, 3), (512, 64, 0)])
def test_ssyrk_against_oracle(handle, orc, uplo, trans, n, k, extra):
    rng = np.random.default_rng(n + k + uplo)
    ar, ac = (k, n) if trans == "T" else (n, k)
    A = rnd32(rng, ar, ac, ar + extra)
    C0 = rnd32(rng, n, n, n + extra)
    want = np.asfortranarray(C0.astype(np.float64))
    orc.dsyrk(uplo, OPS[trans], n, k, -1.0, np.asfortranarray(A.astype(np.float64)), 1.0, want)
    dC = to_dev(C0)
    handle.ssyrk(uplo, OPS[trans], n, k, -1.0, to_dev(A), A.shape[0], 1.0, dC, C0.shape[0])
    got = to_host(dC, C0.shape[0], n)
    tri = np.tril if uplo == LO else np.triu
    bound = 16 * k * EPS32 * (fro(A[:ar].astype(np.float64)) ** 2 + fro(C0[:n].astype(np.float64)))
    assert fro(tri(got[:n].astype(np.float64)) - tri(want[:n])) <= bound
    strict_other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
    assert same_bits(strict_other(got[:n]), strict_other(C0[:n]))   # other triangle untouched
    assert same_bits(got[n:], C0[n:])


def make_tri32(rng, n, lower, unit, scale):
    A = rng.uniform(-1, 1, (n, n)) / scale
    A = np.tril(A) if lower else np.triu(A)
    A[np.diag_indices(n)] = 1.0 + rng.uniform(0, 1, n)
    A = A.astype(np.float32)
    Tm = A.astype(np.float64)
    if unit:
        Tm[np.diag_indices(n)] = 1.0
    stored = A.copy()
    mask = np.triu(np.ones((n, n), bool), 1) if lower else np.tril(np.ones((n, n), bool), -1)
    stored[mask] = np.nan                    # the other triangle must never be read
    if unit:
        stored[np.diag_indices(n)] = np.nan  # nor a unit diagonal
    return np.asfortranarray(stored), Tm


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [UP, LO], "NT", [131, 132])))
def test_strsm_all_sixteen(handle, side, uplo, trans, diag):
    for (m, n, alpha, extra) in [(10, 12, 1.0, 0), (435, 527, 1.0, 0), (300, 257, -0.5, 3)]:
        rng = np.random.default_rng(side * 3 + uplo * 5 + diag + m + n)
        na = m if side == 141 else n
        A, Tm = make_tri32(rng, na, uplo == LO, diag == 132, float(na))
        if extra:
            Ap = np.full((na + extra, na), np.nan, dtype=np.float32, order="F")
            Ap[:na] = A
            A = Ap
        opT = Tm.T if trans == "T" else Tm
        B0 = rnd32(rng, m, n, m + extra)
        dB = to_dev(B0)
        handle.strsm(side, uplo, OPS[trans], diag, m, n, alpha, to_dev(A), A.shape[0], dB,
                     B0.shape[0])
        got = to_host(dB, B0.shape[0], n)
        X = got[:m].astype(np.float64)
        assert np.isfinite(X).all(), "NaN leaked from the unreferenced triangle"
        rhs = alpha * B0[:m].astype(np.float64)
        resid = (opT @ X - rhs) if side == 141 else (X @ opT - rhs)
        assert fro(resid) <= 16 * na * EPS32 * fro(opT) * fro(X)
        assert same_bits(got[m:], B0[m:])


@pytest.mark.parametrize("side,uplo,trans", list(itertools.product([141, 142], [UP, LO], "NT")))
def test_strsm_tall_panels(handle, side, uplo, trans):
    """More than 2048 right-hand sides: 1024-row panels in single precision."""
    rng = np.random.default_rng(side + uplo)
    na, nrhs = 1500, 2300
    m, n = (na, nrhs) if side == 141 else (nrhs, na)
    A, Tm = make_tri32(rng, na, uplo == LO, False, float(na))
    opT = Tm.T if trans == "T" else Tm
    B0 = rnd32(rng, m, n, m + 1)
    dB = to_dev(B0)
    handle.strsm(side, uplo, OPS[trans], 131, m, n, 1.0, to_dev(A), na, dB, m + 1)
    got = to_host(dB, m + 1, n)
    X = got[:m].astype(np.float64)
    assert np.isfinite(X).all()
    rhs = B0[:m].astype(np.float64)
    resid = (opT @ X - rhs) if side == 141 else (X @ opT - rhs)
    assert fro(resid) <= 16 * na * EPS32 * fro(opT) * fro(X)
    assert same_bits(got[m:], B0[m:])


@pytest.mark.parametrize("side,uplo,trans", list(itertools.product([141, 142], [UP, LO], "NT")))
def test_strsm_panels_32_wide(handle, side, uplo, trans):
    """Past 4096 right-hand sides: the 32-wide panel kernel in single precision, with 1024-row
    panels (two, the last of three blocks) and with 512-row panels asked for by option (three,
    the last of two blocks); last workgroup of 8 right-hand sides."""
    from rtatblas_amd import native
    rng = np.random.default_rng(3 * side + uplo)
    nrhs = 4200
    for na, panel in ((1290, None), (1200, native.PANEL_512)):
        m, n = (na, nrhs) if side == 141 else (nrhs, na)
        A, Tm = make_tri32(rng, na, uplo == LO, False, float(na))
        opT = Tm.T if trans == "T" else Tm
        B0 = rnd32(rng, m, n, m + 1)
        dB = to_dev(B0)
        handle.strsm(side, uplo, OPS[trans], 131, m, n, 1.0, to_dev(A), na, dB, m + 1,
                     variant=None if panel is None else native.kernel_options(panel=panel))
        info = handle.last_launch()
        assert (info["trsm_panel_rows"], info["trsm_panel_width"]) == \
            (1024 if panel is None else 512, 32)
        got = to_host(dB, m + 1, n)
        X = got[:m].astype(np.float64)
        assert np.isfinite(X).all()
        rhs = B0[:m].astype(np.float64)
        resid = (opT @ X - rhs) if side == 141 else (X @ opT - rhs)
        assert fro(resid) <= 16 * na * EPS32 * fro(opT) * fro(X)
        assert same_bits(got[m:], B0[m:])


def test_sgeam_copy_transpose_accumulate(handle):
    rng = np.random.default_rng(5)
    m, n = 301, 203
    A = rnd32(rng, n, m, n + 1)                   # to be transposed into m x n
    B0 = rnd32(rng, m, n, m + 3)
    dB = to_dev(B0)
    handle.sgeam(T, N, m, n, 1.0, to_dev(A), A.shape[0], 0.0, dB, B0.shape[0], dB, B0.shape[0])
    got = to_host(dB, B0.shape[0], n)
    assert same_bits(got[:m], np.asfortranarray(A[:n].T))
    assert same_bits(got[m:], B0[m:])
    dB = to_dev(B0)
    handle.sgeam(T, N, m, n, 2.0, to_dev(A), A.shape[0], 0.5, dB, B0.shape[0], dB, B0.shape[0])
    got = to_host(dB, B0.shape[0], n)
    assert same_bits(got[:m], (2.0 * A[:n].T + 0.5 * B0[:m]).astype(np.float32))


def test_sgeam_full_size_transpose_into_odd_ld_bit_exact(handle):
    """9001 x 8000 floats into ldc = 9003: the streaming kernel, columns that split cache lines
    (32 floats per line), ragged edges."""
    import torch
    m, n, lda, ldc = 9001, 8000, 8001, 9003
    S = torch.empty(lda * m, dtype=torch.float32, device="cuda").uniform_(-1, 1)
    At = S.view(m, lda)[:, :n].t()
    buf0 = torch.empty(ldc * n + 8, dtype=torch.float32, device="cuda").uniform_(-1, 1)
    for beta in (0.0, 0.5):
        buf = buf0.clone()
        handle.sgeam(T, N, m, n, 1.0, S, lda, beta, buf, ldc, buf, ldc)
        want = buf0.clone()
        Wm = want[:ldc * n].view(n, ldc)
        Wm[:, :m] = At + beta * Wm[:, :m] if beta else At
        assert torch.equal(buf.view(torch.int32), want.view(torch.int32)), beta


@pytest.mark.parametrize("seed", range(4))
def test_random_sgemm_ssyrk(handle, orc, seed):
    """Seeded random shapes, leading dimensions, scalars and flags (incl. long k with few tiles:
    tail splitting in single precision)."""
    rng = np.random.default_rng(4000 + seed)
    orc.cblas_on()
    try:
        for _ in range(8):
            kind = rng.integers(0, 3)
            if kind == 0:
                m, n, k = (int(rng.integers(1, 200)) for _ in range(3))
            elif kind == 1:
                m, n, k = int(rng.integers(60, 700)), int(rng.integers(60, 700)), int(rng.integers(1500, 5000))
            else:
                m, n, k = int(rng.integers(1500, 2600)), int(rng.integers(1500, 2600)), int(rng.integers(130, 400))
            ta, tb = str(rng.choice(["N", "T"])), str(rng.choice(["N", "T"]))
            run_sgemm(handle, orc, ta, tb, m, n, k, float(rng.choice([1.0, -0.5])),
                      float(rng.choice([0.0, 1.0, 0.5])),
                      extra=tuple(int(x) for x in rng.integers(0, 5, 3)), seed=seed)
            # SYRK on the same A shape
            uplo, trans = int(rng.choice([UP, LO])), str(rng.choice(["N", "T"]))
            ar, ac = (k, n) if trans == "T" else (n, k)
            A = rnd32(rng, ar, ac, ar + int(rng.integers(0, 5)))
            C0 = rnd32(rng, n, n, n + int(rng.integers(0, 5)))
            want = np.asfortranarray(C0.astype(np.float64))
            orc.dsyrk(uplo, OPS[trans], n, k, 1.0, np.asfortranarray(A.astype(np.float64)), -1.0, want)
            dC = to_dev(C0)
            handle.ssyrk(uplo, OPS[trans], n, k, 1.0, to_dev(A), A.shape[0], -1.0, dC, C0.shape[0])
            got = to_host(dC, C0.shape[0], n)
            tri = np.tril if uplo == LO else np.triu
            bound = 16 * k * EPS32 * (fro(A[:ar].astype(np.float64)) ** 2
                                      + fro(C0[:n].astype(np.float64)))
            assert fro(tri(got[:n].astype(np.float64)) - tri(want[:n])) <= bound, (seed, uplo, trans, n, k)
            other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
            assert same_bits(other(got[:n]), other(C0[:n]))
    finally:
        orc.cblas_off()
