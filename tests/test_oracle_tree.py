"""Pins layer 2 of the CPU oracle: the variant trees and the workspace accounting.

Checks: (a) the workspace bytes of each variant against element counts worked out by hand from
the reference's rule (src/matrix_ops/matrixop.h:172-185); (b) every variant computes what the
default variant computes — the identity the reference's own tests assert
(tests/executor_test.cpp:23-86 GEMM, :139-222 TRSM, :234-287 SYRK) — and the default variant is
layer 1, pinned separately; (c) nested trees of the kind tests/matrixop_test.cpp:230-302 builds."""
import itertools

import numpy as np
import pytest

from util import EPS, bits_equal, fro

GEMM_VARIANTS = ["".join(v) for v in itertools.product("NT", repeat=3)]
PAD_VARIANTS = ["".join(v) + "".join(p) for v in itertools.product("NT", repeat=3)
                for p in itertools.product("NP", repeat=3)]
BOOL_VARIANTS = ["FF", "FT", "TF", "TT"]
OPS = {"N": 111, "T": 112}


def rnd(rng, m, n, ld=None):
    ld = max(m, 1) if ld is None else ld
    a = np.full((ld, n), np.nan, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n))
    return a


def up(x, p):
    return (x + p - 1) // p * p


def test_gemm_workspace_by_hand(orc):
    m, n, k = 70, 45, 62
    # opA = opB = N, ld = rows.  Elements: A^T copy k*m, B^T copy n*k, C^T scratch n*m.
    want = {"NNN": 0, "TNN": k * m, "NTN": n * k, "TTN": k * m + n * k,
            "NNT": n * m, "TNT": k * m + n * m, "NTT": n * k + n * m,
            "TTT": k * m + n * k + n * m}
    for v, elems in want.items():
        assert orc.gemm_workspace(v, 111, 111, m, n, k, m, k, m) == 8 * elems, v


def test_gemm_pad_workspace_by_hand(orc):
    m, n, k = 70, 45, 62
    assert orc.gemm_workspace("NNNNNN", 111, 111, m, n, k, m, k, m) == 0
    # padA: copy of A (m x k) with ld = roundup(m, 32)
    assert orc.gemm_workspace("NNNPNN", 111, 111, m, n, k, m, k, m) == 8 * up(m, 32) * k
    # padB: copy of B (k x n) with ld = roundup(k, 32)
    assert orc.gemm_workspace("NNNNPN", 111, 111, m, n, k, m, k, m) == 8 * up(k, 32) * n
    # padC: product into an m x n scratch with ld = roundup(m, 32)
    assert orc.gemm_workspace("NNNNNP", 111, 111, m, n, k, m, k, m) == 8 * up(m, 32) * n
    # transA + padA: A^T is k x m, ld = roundup(k, 32); transC + padC: n x m, ld = roundup(n, 32)
    assert orc.gemm_workspace("TNTPNP", 111, 111, m, n, k, m, k, m) == \
        8 * (up(k, 32) * m + up(n, 32) * m)
    assert orc.gemm_workspace("TTTPPP", 111, 111, m, n, k, m, k, m) == \
        8 * (up(k, 32) * m + up(n, 32) * k + up(n, 32) * m)


def test_syrk_trsm_workspace_by_hand(orc):
    n, k = 213, 74
    # trans = N: A is n x k.  transA: k x n copy.  transC: n x n scratch.
    assert orc.syrk_workspace("FF", 122, 111, n, k, n, n) == 0
    assert orc.syrk_workspace("TF", 122, 111, n, k, n, n) == 8 * k * n
    assert orc.syrk_workspace("FT", 122, 111, n, k, n, n) == 8 * n * n
    assert orc.syrk_workspace("TT", 122, 111, n, k, n, n) == 8 * (k * n + n * n)
    m, nn = 435, 527
    # left: A is m x m.  swap_side: B^T (nn x m) scratch.  transA: m x m copy.
    assert orc.trsm_workspace("FF", 141, 122, 111, 131, m, nn, m, m) == 0
    assert orc.trsm_workspace("FT", 141, 122, 111, 131, m, nn, m, m) == 8 * m * m
    assert orc.trsm_workspace("TF", 141, 122, 111, 131, m, nn, m, m) == 8 * nn * m
    assert orc.trsm_workspace("TT", 141, 122, 111, 131, m, nn, m, m) == 8 * (m * m + nn * m)
    # right: A is nn x nn
    assert orc.trsm_workspace("FT", 142, 122, 111, 131, m, nn, nn, m) == 8 * nn * nn


def test_bad_variant_strings_and_short_workspace(orc):
    rng = np.random.default_rng(0)
    A, B, C = rnd(rng, 8, 6), rnd(rng, 6, 5), rnd(rng, 8, 5)
    assert orc.gemm_workspace("NNX", 111, 111, 8, 5, 6, 8, 6, 8) == -1
    assert orc.gemm_workspace("NN", 111, 111, 8, 5, 6, 8, 6, 8) == -1
    assert orc.syrk_workspace("NT", 122, 111, 8, 5, 8, 8) == -1
    assert orc.gemm_variant("TNN", 111, 111, 8, 5, 6, 1.0, A, B, 0.0, C, ws_bytes=8) == -2


@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
@pytest.mark.parametrize("variant", GEMM_VARIANTS + PAD_VARIANTS[::5])
def test_gemm_variants_equal_default(orc, ta, tb, variant):
    m, n, k = 70, 45, 62          # tests/executor_test.cpp:15-17
    rng = np.random.default_rng(1)
    A = rnd(rng, k if ta == "T" else m, m if ta == "T" else k)
    B = rnd(rng, n if tb == "T" else k, k if tb == "T" else n)
    C0 = rnd(rng, m, n, m + 3)
    ref = C0.copy(order="F")
    orc.dgemm(OPS[ta], OPS[tb], m, n, k, 1.0, A, B, 0.5, ref)
    C = C0.copy(order="F")
    assert orc.gemm_variant(variant, OPS[ta], OPS[tb], m, n, k, 1.0, A, B, 0.5, C) == 0
    assert fro(C[:m] - ref[:m]) <= 16 * k * EPS * (fro(A) * fro(B) + 0.5 * fro(C0[:m]))
    assert not np.allclose(C[:m], C0[:m])
    assert np.isnan(C[m:]).all()                # padding rows of the caller's C untouched
    if variant in ("NNN", "NNNNNN"):
        assert bits_equal(C, ref)               # the default variant is the plain call


@pytest.mark.parametrize("uplo,trans", list(itertools.product([121, 122], "NT")))
@pytest.mark.parametrize("variant", BOOL_VARIANTS)
def test_syrk_variants_equal_default(orc, uplo, trans, variant):
    n, k = 213, 74                # tests/executor_test.cpp:231-232
    rng = np.random.default_rng(2)
    A = rnd(rng, k if trans == "T" else n, n if trans == "T" else k)
    C0 = rnd(rng, n, n)
    ref = C0.copy(order="F")
    orc.dsyrk(uplo, OPS[trans], n, k, -1.0, A, 1.0, ref)
    C = C0.copy(order="F")
    assert orc.syrk_variant(variant, uplo, OPS[trans], n, k, -1.0, A, 1.0, C) == 0
    tri = np.tril if uplo == 122 else np.triu
    assert fro(tri(C) - tri(ref)) <= 16 * k * EPS * (fro(A) ** 2 + fro(C0))
    if variant[1] == "F":
        # written straight into C: the other triangle is bit-unchanged
        other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
        assert bits_equal(other(C), other(C0))


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [121, 122], "NT", [131, 132])))
@pytest.mark.parametrize("variant", BOOL_VARIANTS)
def test_trsm_variants_equal_default(orc, side, uplo, trans, diag, variant):
    m, n = 43, 52
    rng = np.random.default_rng(3)
    na = m if side == 141 else n
    A = rng.uniform(-1, 1, (na, na)) / na
    A[np.diag_indices(na)] = 1.0 + rng.uniform(0, 1, na)
    A = np.asfortranarray(A)      # both triangles finite: the transposing variants copy all of A
    B0 = rnd(rng, m, n, m + 1)
    ref = B0.copy(order="F")
    orc.dtrsm(side, uplo, OPS[trans], diag, m, n, 1.0, A, ref)
    B = B0.copy(order="F")
    assert orc.trsm_variant(variant, side, uplo, OPS[trans], diag, m, n, 1.0, A, B) == 0
    assert np.allclose(B[:m], ref[:m], rtol=1e-12, atol=1e-13)
    assert np.isnan(B[m:]).all()


def test_workspace_is_exactly_enough(orc):
    """One byte less than the reported need must be refused (executor.h:49-51)."""
    rng = np.random.default_rng(4)
    m, n, k = 12, 9, 7
    A, B, C = rnd(rng, m, k), rnd(rng, k, n), rnd(rng, m, n)
    for v in GEMM_VARIANTS[1:]:
        need = orc.gemm_workspace(v, 111, 111, m, n, k, m, k, m)
        assert need > 0
        assert orc.gemm_variant(v, 111, 111, m, n, k, 1.0, A, B, 0.0, C, ws_bytes=need - 8) == -2
        assert orc.gemm_variant(v, 111, 111, m, n, k, 1.0, A, B, 0.0, C, ws_bytes=need) == 0
