"""Pins layer 1 of the CPU oracle (orc_dgemm / dsyrk / dtrsm / dgeam / dfill) before anything
is compared against it.  Checks are independent of the oracle's own formulae: SciPy's BLAS
(a separate library), numpy index permutations, closed forms and the self-consistency check
the reference's tests run on their host TRSM loops (tests/matrixop_test.cpp:58-109)."""
import itertools

import numpy as np
import pytest
from scipy.linalg import blas as sblas

from util import EPS, bits_equal, fro

OPS = {"N": 111, "T": 112}


def rnd(rng, m, n, ld=None):
    ld = max(m, 1) if ld is None else ld
    a = np.full((ld, n), np.nan, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n))
    return a


@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
@pytest.mark.parametrize("m,n,k,pad", [(70, 45, 62, 0), (26, 27, 34, 3), (1, 1, 1, 0),
                                        (5, 7, 0, 2), (33, 1, 17, 1)])
def test_dgemm_matches_scipy_blas(orc, ta, tb, m, n, k, pad):
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    A = rnd(rng, k if ta == "T" else m, m if ta == "T" else k, (k if ta == "T" else m) + pad)
    B = rnd(rng, n if tb == "T" else k, k if tb == "T" else n, (n if tb == "T" else k) + pad)
    C0 = rnd(rng, m, n, m + pad)
    for alpha, beta in [(1.0, 0.0), (-0.75, 0.5), (2.0, 1.0), (0.0, 0.5)]:
        C = C0.copy(order="F")
        orc.dgemm(OPS[ta], OPS[tb], m, n, k, alpha, A, B, beta, C)
        Al = A[: (k if ta == "T" else m)]
        Bl = B[: (n if tb == "T" else k)]
        if k > 0:
            ref = sblas.dgemm(alpha, Al, Bl, beta, C0[:m].copy(order="F"), trans_a=ta == "T",
                              trans_b=tb == "T")
        else:
            ref = beta * C0[:m] if beta != 0 else np.zeros((m, n))
        opA = Al.T if ta == "T" else Al
        opB = Bl.T if tb == "T" else Bl
        bound = 16 * max(k, 1) * EPS * (abs(alpha) * fro(opA) * fro(opB) + abs(beta) * fro(C0[:m]))
        assert fro(C[:m] - ref) <= bound
        if pad:  # padding rows are never written
            assert np.isnan(C[m:]).all()


def test_dgemm_beta_zero_never_reads_c(orc):
    rng = np.random.default_rng(7)
    A, B = rnd(rng, 9, 4), rnd(rng, 4, 6)
    C = np.full((9, 6), np.nan, order="F")
    orc.dgemm(111, 111, 9, 6, 4, 1.0, A, B, 0.0, C)
    assert np.isfinite(C).all()
    assert np.allclose(C, A @ B, rtol=0, atol=1e-14)


def test_dgemm_identity_and_rank_one(orc):
    rng = np.random.default_rng(3)
    B = rnd(rng, 12, 5)
    I = np.asfortranarray(np.eye(12))
    C = np.zeros((12, 5), order="F")
    orc.dgemm(111, 111, 12, 5, 12, 1.0, I, B, 0.0, C)
    assert bits_equal(C, B)            # products with 0 and 1 are exact
    u, v = rnd(rng, 8, 1), rnd(rng, 1, 6)
    C = np.zeros((8, 6), order="F")
    orc.dgemm(111, 111, 8, 6, 1, 1.0, u, v, 0.0, C)
    assert bits_equal(C, np.asfortranarray(u * v))


@pytest.mark.parametrize("uplo", [121, 122])
@pytest.mark.parametrize("trans", ["N", "T"])
@pytest.mark.parametrize("n,k", [(72, 56), (213, 74), (1, 3), (6, 0)])
def test_dsyrk_is_triangle_of_gemm(orc, uplo, trans, n, k):
    rng = np.random.default_rng(n + k)
    A = rnd(rng, k if trans == "T" else n, n if trans == "T" else k)
    C0 = rnd(rng, n, n, n + 2)
    C = C0.copy(order="F")
    orc.dsyrk(uplo, OPS[trans], n, k, -1.0, A, 1.0, C)
    Al = A[: (k if trans == "T" else n)]
    opA = Al.T if trans == "T" else Al
    full = C0[:n] - opA @ opA.T
    tri = np.tril if uplo == 122 else np.triu
    other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
    assert fro(tri(C[:n]) - tri(full)) <= 16 * max(k, 1) * EPS * (fro(opA) ** 2 + fro(C0[:n]))
    # the other triangle and the padding are bit-unchanged
    assert bits_equal(other(C[:n]), other(C0[:n]))
    assert np.isnan(C[n:]).all()
    if k > 0:
        ref = sblas.dsyrk(-1.0, Al, 1.0, C0[:n].copy(order="F"), trans=trans == "T",
                          lower=uplo == 122)
        assert fro(tri(C[:n]) - tri(ref)) <= 16 * k * EPS * (fro(opA) ** 2 + fro(C0[:n]))


def make_tri(rng, n, lower, unit, poison=True):
    A = rng.uniform(-1, 1, (n, n))
    A = np.tril(A) if lower else np.triu(A)
    A[np.diag_indices(n)] = 1.0 + rng.uniform(0, 1, n)
    T = A.copy()
    if unit:
        T[np.diag_indices(n)] = 1.0
    stored = A.copy()
    if poison:  # the other triangle (and a unit diagonal) must never be read
        mask = np.triu(np.ones((n, n), bool), 1) if lower else np.tril(np.ones((n, n), bool), -1)
        stored[mask] = np.nan
        if unit:
            stored[np.diag_indices(n)] = np.nan
    return np.asfortranarray(stored), T


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [121, 122], "NT", [131, 132])))
def test_dtrsm_all_sixteen(orc, side, uplo, trans, diag):
    m, n = 10, 12
    rng = np.random.default_rng(side + uplo + ord(trans) + diag)
    na = m if side == 141 else n
    A, T = make_tri(rng, na, uplo == 122, diag == 132)
    opT = T.T if trans == "T" else T
    B0 = rnd(rng, m, n, m + 3)
    B = B0.copy(order="F")
    alpha = -1.5
    orc.dtrsm(side, uplo, OPS[trans], diag, m, n, alpha, A, B)
    X = B[:m]
    resid = (opT @ X - alpha * B0[:m]) if side == 141 else (X @ opT - alpha * B0[:m])
    assert fro(resid) <= 16 * na * EPS * fro(opT) * fro(X)
    assert np.isnan(B[m:]).all()
    ref = sblas.dtrsm(alpha, np.nan_to_num(A), B0[:m].copy(order="F"), side=side == 142,
                      lower=uplo == 122, trans_a=trans == "T", diag=diag == 132)
    assert np.allclose(X, ref, rtol=1e-11, atol=1e-12)


def test_dtrsm_reference_self_check(orc):
    """tests/matrixop_test.cpp:58-109: X = trsm(A, B) must satisfy gemm(op(A), X) == B at 1e-10,
    5 x 6, all side / uplo / trans combinations."""
    m, n = 5, 6
    rng = np.random.default_rng(11)
    for side, lower, trans in itertools.product([141, 142], [True, False], "NT"):
        na = m
        mx, nx = (m, n) if side == 141 else (n, m)
        A = rng.uniform(-1, 1, (na, na))
        A = np.asfortranarray(np.tril(A) if lower else np.triu(A))
        B = rnd(rng, mx, nx)
        X = B.copy(order="F")
        orc.dtrsm(side, 122 if lower else 121, OPS[trans], 131, mx, nx, 1.0, A, X)
        Bt = np.zeros((mx, nx), order="F")
        if side == 141:
            orc.dgemm(OPS[trans], 111, mx, nx, na, 1.0, A, X, 0.0, Bt)
        else:
            orc.dgemm(111, OPS[trans], mx, nx, na, 1.0, X, A, 0.0, Bt)
        scale = max(1.0, np.abs(X).max())
        assert np.abs(Bt - B).max() <= 1e-10 * scale


def test_dtrsm_diagonal_and_alpha_zero(orc):
    rng = np.random.default_rng(5)
    d = 1.0 + rng.uniform(0, 1, 7)
    A = np.asfortranarray(np.diag(d))
    B0 = rnd(rng, 7, 4)
    B = B0.copy(order="F")
    orc.dtrsm(141, 122, 111, 131, 7, 4, 1.0, A, B)
    assert bits_equal(B, np.asfortranarray(B0 / d[:, None]))
    B = np.full((7, 4), np.nan, order="F")
    orc.dtrsm(141, 122, 111, 131, 7, 4, 0.0, A, B)
    assert (B == 0).all()


@pytest.mark.parametrize("m,n", [(10, 12), (64, 64), (65, 3), (1, 70), (33, 129)])
@pytest.mark.parametrize("pad", [1, 8, 32])
def test_dgeam_copy_pad_transpose_bit_exact(orc, m, n, pad):
    rng = np.random.default_rng(m * n + pad)
    A = rnd(rng, m, n, m + 3)
    A[0, 0] = -0.0
    ld = ((m + pad - 1) // pad) * pad
    out = np.full((ld, n), np.nan, order="F")
    orc.dgeam(111, 111, m, n, 1.0, A, 0.0, out, out)      # MatrixMove, no transpose
    assert bits_equal(out[:m], A[:m]) and np.isnan(out[m:]).all()
    ldt = ((n + pad - 1) // pad) * pad
    outT = np.full((ldt, m), np.nan, order="F")
    orc.dgeam(112, 111, n, m, 1.0, A, 0.0, outT, outT)    # MatrixMove, transpose
    assert bits_equal(outT[:n], np.asfortranarray(A[:m].T)) and np.isnan(outT[n:]).all()
    back = np.full((m, n), np.nan, order="F")
    orc.dgeam(112, 111, m, n, 1.0, outT, 0.0, back, back)  # transposing twice is the identity
    assert bits_equal(back, A[:m])


@pytest.mark.parametrize("beta", [0.0, 0.5, 1.0, -2.0])
@pytest.mark.parametrize("trans", [111, 112])
def test_dgeam_accumulate_closed_form(orc, beta, trans):
    m, n = 23, 17
    rng = np.random.default_rng(int(beta * 10) + trans)
    S = rnd(rng, n, m) if trans == 112 else rnd(rng, m, n)
    C0 = rnd(rng, m, n, m + 1)
    C = C0.copy(order="F")
    orc.dgeam(trans, 111, m, n, 1.0, S, beta, C, C)
    Sl = S.T if trans == 112 else S
    want = Sl + beta * C0[:m] if beta != 0 else Sl   # beta*c exact for powers of two
    assert bits_equal(C[:m], np.asfortranarray(want))
    assert np.isnan(C[m:]).all()


def test_dgeam_scale_and_zero_fill(orc):
    rng = np.random.default_rng(2)
    A = rnd(rng, 9, 5)
    out = np.full((9, 5), np.nan, order="F")
    orc.dgeam(111, 111, 9, 5, -2.0, A, 0.0, out, out)
    assert bits_equal(out, np.asfortranarray(-2.0 * A))
    nanmat = np.full((9, 5), np.nan, order="F")
    orc.dgeam(111, 111, 9, 5, 0.0, nanmat, 0.0, nanmat, nanmat)   # MatrixSyrkAlloc's zero fill
    assert (nanmat == 0).all()


def test_dfill_properties(orc):
    a = orc.fill(50, 40, 53, seed=1, kind=0)
    assert np.isnan(a[50:]).all()
    assert (a[:50] >= -1).all() and (a[:50] < 1).all()
    assert abs(a[:50].mean()) < 0.1 and 0.25 < a[:50].var() < 0.42      # uniform[-1,1): var 1/3
    b = orc.fill(50, 40, 50, seed=1, kind=0)
    assert bits_equal(a[:50], b)                                         # independent of ld
    assert not bits_equal(orc.fill(50, 40, seed=2), b)                   # depends on the seed
    s = orc.fill(30, 30, seed=4, kind=1)
    assert bits_equal(s, np.asfortranarray(s.T))
    t = orc.fill(30, 30, seed=5, kind=2)
    assert np.isnan(t[np.triu_indices(30, 1)]).all()
    d = np.diag(t)
    assert (d >= 1).all() and (d < 2).all()
    low = t[np.tril_indices(30, -1)]
    assert (np.abs(low) <= 1 / 30).all()
    f = orc.fill(30, 30, seed=5, kind=4)
    assert bits_equal(np.tril(f), np.tril(np.nan_to_num(t))) and bits_equal(f, np.asfortranarray(f.T))
    u = orc.fill(20, 20, seed=6, kind=3)
    assert (u > 0).all() and (u <= 1).all()


def test_dfill_known_values(orc):
    """Generator pinned by hand: splitmix64 finaliser of seed*phi + (j<<32 | i)."""
    def mix(z):
        M = (1 << 64) - 1
        z = (z + 0x9E3779B97F4A7C15) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        return z ^ (z >> 31)
    a = orc.fill(4, 3, seed=9)
    for i in range(4):
        for j in range(3):
            z = mix((9 * 0x9E3779B97F4A7C15 + ((j << 32) | i)) & ((1 << 64) - 1))
            assert a[i, j] == 2.0 * ((z >> 11) / 2.0 ** 53) - 1.0


def test_cblas_backend_agrees_with_loops(orc):
    rng = np.random.default_rng(8)
    A, B = rnd(rng, 40, 30), rnd(rng, 30, 20)
    C1 = np.zeros((40, 20), order="F")
    orc.dgemm(111, 111, 40, 20, 30, 1.0, A, B, 0.0, C1)
    threads, name = orc.cblas_on()
    try:
        if threads == 0:
            pytest.skip("no host CBLAS on this machine")
        C2 = np.zeros((40, 20), order="F")
        orc.dgemm(111, 111, 40, 20, 30, 1.0, A, B, 0.0, C2)
        assert fro(C1 - C2) <= 16 * 30 * EPS * fro(A) * fro(B)
    finally:
        orc.cblas_off()
