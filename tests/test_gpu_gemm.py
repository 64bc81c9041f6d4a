"""GPU parity of rtat_dgemm / rtat_dgemm_ex (through the C ABI) against the CPU oracle.
Bar: ||C - C_ref||_F <= 16 k eps (|alpha| ||A||_F ||B||_F + |beta| ||C0||_F)."""
import itertools

import numpy as np
import pytest

from util import EPS, bits_equal, fro, gemm_bound, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112
OPS = {"N": N, "T": T}


def rnd(rng, m, n, ld=None):
    ld = max(m, 1) if ld is None else ld
    a = np.full((ld, n), np.nan, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n))
    return a


def run_case(handle, orc, ta, tb, m, n, k, alpha, beta, extra=(0, 0, 0), variant=None, seed=0):
    rng = np.random.default_rng(seed + m + 7 * n + 13 * k)
    ar, ac = (k, m) if ta == "T" else (m, k)
    br, bc = (n, k) if tb == "T" else (k, n)
    A = rnd(rng, ar, ac, max(ar, 1) + extra[0])
    B = rnd(rng, br, bc, max(br, 1) + extra[1])
    C0 = rnd(rng, m, n, max(m, 1) + extra[2])
    want = C0.copy(order="F")
    orc.dgemm(OPS[ta], OPS[tb], m, n, k, alpha, A, B, beta, want)
    dC = to_dev(C0)
    handle.dgemm(OPS[ta], OPS[tb], m, n, k, alpha, to_dev(A), A.shape[0], to_dev(B), B.shape[0],
                 beta, dC, C0.shape[0], variant=variant)
    got = to_host(dC, C0.shape[0], n)
    if beta == 0.0:
        C0l = np.zeros((m, n))
    else:
        C0l = C0[:m]
    bound = gemm_bound(k, alpha, A[:ar], B[:br], beta, C0l)
    err = fro(got[:m] - want[:m])
    assert err <= bound, (ta, tb, m, n, k, variant, err, bound)
    # rows m..ld-1 of C are never written
    assert bits_equal(got[m:], C0[m:])
    return got


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
def test_reference_test_shapes(handle, orc, ta, tb, variant):
    # tests/executor_test.cpp:15-17 (70,45,62), matrixop_test.cpp:34-36 (26,27,34),
    # planning_test.cpp:89-91 (23,16,35)
    for (m, n, k) in [(70, 45, 62), (26, 27, 34), (23, 16, 35)]:
        run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.0, variant=variant)


@pytest.mark.parametrize("variant", [1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
def test_tile_multiples_and_ragged_edges(handle, orc, ta, tb, variant):
    orc.cblas_on()
    try:
        for (m, n, k, extra) in [(256, 256, 64, (0, 0, 0)), (512, 384, 130, (0, 0, 0)),
                                 (300, 200, 77, (3, 3, 3)), (129, 257, 33, (1, 2, 3)),
                                 (1, 1, 1, (0, 0, 0)), (17, 515, 16, (2, 0, 1))]:
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.5, extra=extra, variant=variant)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
def test_ragged_tiles_with_long_k(handle, orc, ta, tb, variant):
    """Tiles that hang over the edge of C take the same vector loads as interior ones, with
    clamped rows, for all but the last panels of a long k.  Odd and even m, n; leading
    dimensions made even (16-byte vector path, NaN padding rows right behind the data) and
    left tight and odd (scalar path)."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(301, 203, 200), (130, 67, 161), (1, 3, 96), (255, 129, 80)]:
            ar = k if ta == "T" else m
            br = n if tb == "T" else k
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.5, extra=(ar % 2, br % 2, 0),
                     variant=variant)
            run_case(handle, orc, ta, tb, m, n, k, -1.0, 0.0, extra=(1 - ar % 2, 1 - br % 2, 1),
                     variant=variant, seed=5)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T")])
def test_tail_tiles_split_along_k(handle, orc, ta, tb, variant):
    """Few tiles and a long k: the tiles left over after the last full round of workgroups are
    computed in K slices and summed by a second kernel.  Ragged m, n and a k that is not a
    whole number of panels, beta != 0, plus a shape with more tiles than workgroup slots."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(300, 200, 1000), (129, 65, 2049), (64, 64, 4096), (2100, 2200, 300)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.5, -0.5, variant=variant)
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.0, extra=(1, 1, 1), variant=variant,
                     seed=9)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T")])
def test_tail_tiles_cut_into_pieces(handle, orc, ta, tb, variant):
    """More tiles than one round of workgroups, a leftover between one per CU and a full round,
    and a k too short for K slices: the leftover tiles are computed as 64 x 64 pieces by a
    second launch.  Ragged edges, so that pieces hang over the edge of C or fall outside it."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(3621, 3700, 40), (5300, 2477, 33)]:
            run_case(handle, orc, ta, tb, m, n, k, -1.0, 1.0, variant=variant)
            run_case(handle, orc, ta, tb, m, n, k, 0.5, 0.0, extra=(1, 3, 1), variant=variant,
                     seed=4)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
def test_small_problems_on_32x32_tiles(handle, orc, ta, tb):
    """The automatic choice computes a problem of up to two 32 x 32 tiles per CU and a k of at
    most 512 (768 from one tile per CU on) in one launch of 32 x 32 tiles.  Shapes inside that
    range and on its edges: ragged m and n, K tails, odd leading dimensions, beta != 0; one wave
    of such a tile owns a single 16 x 16 block."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(512, 512, 512), (200, 300, 400), (97, 61, 500), (33, 31, 17),
                          (32, 32, 16), (640, 640, 520), (512, 512, 768), (2048, 32, 250),
                          (31, 2050, 129), (700, 690, 512)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.0, variant=0)
            run_case(handle, orc, ta, tb, m, n, k, -0.75, 0.5, extra=(1, 3, 1), variant=0, seed=5)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", list(itertools.product("NT", "NT")))
def test_thin_edge_tiles_skip_their_empty_blocks(handle, orc, ta, tb, variant):
    """Launches of two rounds of workgroups or more in which the last tile row and column hold
    only a few rows / columns of C (8 and 3 of 128; 24 and 40 of 64 for the smallest shape):
    those tiles leave out the MFMA blocks without an element of C.  k covers the K-tail loop
    and the last panel; beta != 0 and the bits behind C's rows show that nothing else is
    touched."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(4104, 4099, 70), (8344, 2088, 33)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.5, extra=(1, 3, 2), variant=variant)
        run_case(handle, orc, ta, tb, 4104, 4099, 16, -1.0, 0.0, variant=variant, seed=3)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T")])
def test_one_extra_tile_on_a_few_cus_cut_along_k(handle, orc, ta, tb, variant):
    """More tiles than CUs, and the count modulo the CUs is at most half the CUs (8 or 16 tiles
    of 128 x 64, 128 x 128 or 64 x 64 on a 256-CU device; 113 and 73 tiles of 64 x 64 for the
    last two shapes): only those last tiles are cut into K slices, every tile before them is
    computed whole."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(1500, 1400, 600), (2100, 2048, 300), (1511, 1400, 257), (1600, 1600, 300),
                          (1856, 1850, 400)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.25, -0.5, variant=variant)
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.0, extra=(2, 1, 3), variant=variant,
                     seed=6)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 2, 3, 4])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T")])
def test_slices_fill_the_workgroup_slots(handle, orc, ta, tb, variant):
    """A problem of less than one round of tiles whose slices would leave workgroup slots
    empty: some of the tiles get one slice more (on 256 CUs, 105 tiles of 128 x 128 as
    13 x 4 + 92 x 5 slices).  The other shape has 152 leftover tiles behind a full round, which
    all get three slices."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(1024, 10624, 520), (333, 4444, 2100)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.0, -1.0, variant=variant)
            run_case(handle, orc, ta, tb, m, n, k, -0.5, 0.0, extra=(1, 2, 1), variant=variant,
                     seed=8)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("variant", [0, 4])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T")])
def test_uneven_load_of_the_smallest_shape_cut_along_k(handle, orc, ta, tb, variant):
    """Less than a round of 64 x 64 tiles, but more tiles than CUs and more than half of the CUs
    one tile ahead of the rest (on 256 CUs: 400 and 462 tiles), 48 K panels or more: every tile
    is cut into two slices, some into three.  With 329 tiles (the last shape) only the 73 odd
    ones are cut."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(1280, 1280, 1152), (1300, 1400, 800), (400, 3000, 777)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.5, variant=variant)
            run_case(handle, orc, ta, tb, m, n, k, -1.5, 0.0, extra=(3, 0, 1), variant=variant,
                     seed=9)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_automatic_shape_may_cut_a_sparse_round_along_k(handle, orc, ta, tb):
    """At most one 64 x 64 tile per CU and a mid-length k: the automatic shape choice prices
    the K slices and takes them where they pay (on 256 CUs: 800 x 800 x 1600, 700 x 900 x 1000,
    832^3); a fixed shape keeps to the rule and computes whole tiles.  Both against CBLAS."""
    orc.cblas_on()
    try:
        for (m, n, k) in [(800, 800, 1600), (700, 900, 1000), (832, 832, 832), (1000, 1020, 1000)]:
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.5, variant=0)
            run_case(handle, orc, ta, tb, m, n, k, 0.5, 0.0, extra=(1, 2, 3), variant=0, seed=10)
            run_case(handle, orc, ta, tb, m, n, k, 1.0, 0.5, variant=4)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (1.0, 1.0), (-0.75, 0.5), (2.0, -1.0)])
def test_alpha_beta(handle, orc, alpha, beta):
    run_case(handle, orc, "T", "N", 200, 150, 96, alpha, beta)


def test_beta_zero_ignores_nan_in_c(handle, orc):
    rng = np.random.default_rng(1)
    m, n, k = 140, 130, 50
    A, B = rnd(rng, m, k), rnd(rng, k, n)
    dC = to_dev(np.full((m, n), np.nan, order="F"))
    handle.dgemm(N, N, m, n, k, 1.0, to_dev(A), m, to_dev(B), k, 0.0, dC, m)
    got = to_host(dC, m, n)
    assert np.isfinite(got).all()
    assert fro(got - A @ B) <= 16 * k * EPS * fro(A) * fro(B)


def test_identity_operands_are_exact(handle):
    rng = np.random.default_rng(2)
    n = 192
    B = rnd(rng, n, n)
    I = np.asfortranarray(np.eye(n))
    for (ta, tb, A_, B_) in [(N, N, I, B), (N, N, B, I), (T, N, I, B), (N, T, B, I)]:
        dC = to_dev(np.full((n, n), np.nan, order="F"))
        handle.dgemm(ta, tb, n, n, n, 1.0, to_dev(A_), n, to_dev(B_), n, 0.0, dC, n)
        assert bits_equal(to_host(dC, n, n), B)


def test_quick_returns_and_scaling_only(handle, orc):
    import torch
    rng = np.random.default_rng(3)
    m, n = 50, 40
    C0 = rnd(rng, m, n)
    dC = to_dev(C0)
    x = torch.zeros(8, dtype=torch.float64, device="cuda")
    handle.dgemm(N, N, m, n, 0, 1.0, x, m, x, 1, 0.5, dC, m)              # k == 0: C = beta C
    assert bits_equal(to_host(dC, m, n), np.asfortranarray(0.5 * C0))
    handle.dgemm(N, N, m, n, 5, 0.0, None, m, None, 5, 0.0, dC, m)         # alpha == beta == 0
    assert (to_host(dC, m, n) == 0).all()
    assert handle.dgemm(N, N, 0, n, 5, 1.0, x, 1, x, 5, 0.0, dC, 1, check=False) == 0
    assert handle.dgemm(N, N, m, n, 5, 1.0, x, m - 1, x, 5, 0.0, dC, m, check=False) == 3
    assert handle.dgemm(N, 7, m, n, 5, 1.0, x, m, x, 5, 0.0, dC, m, check=False) == 10
    assert handle.dgemm(N, N, m, n, 5, 1.0, x, m, x, 5, 0.0, dC, m, variant=9, check=False) == 3


def test_config_c1_512_through_every_kernel_variant(handle, orc):
    """DGEMM 512^3, NN, alpha 1, beta 0, ld = M, iid uniform[-1,1] from the seeded generator,
    checked against host CBLAS."""
    import torch
    n = 512
    threads, _ = orc.cblas_on()
    try:
        A, B = orc.fill(n, n, seed=1), orc.fill(n, n, seed=2)
        want = np.zeros((n, n), order="F")
        orc.dgemm(N, N, n, n, n, 1.0, A, B, 0.0, want)
        dA = torch.empty(n * n, dtype=torch.float64, device="cuda")
        dB = torch.empty_like(dA)
        handle.dfill(dA, n, n, n, 1)
        handle.dfill(dB, n, n, n, 2)
        for variant in range(5):
            dC = to_dev(np.full((n, n), np.nan, order="F"))
            handle.dgemm(N, N, n, n, n, 1.0, dA, n, dB, n, 0.0, dC, n, variant=variant)
            assert fro(to_host(dC, n, n) - want) <= 16 * n * EPS * fro(A) * fro(B)
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("n", [1024, 2048])
def test_config_c2_tn_sweep_small_sizes(handle, orc, n):
    """opA = T, opB = N, alpha 1, beta 0.5, ld = rows: oracle via host CBLAS."""
    import torch
    orc.cblas_on()
    try:
        A, B, C0 = orc.fill(n, n, seed=1), orc.fill(n, n, seed=2), orc.fill(n, n, seed=3)
        want = C0.copy(order="F")
        orc.dgemm(T, N, n, n, n, 1.0, A, B, 0.5, want)
        dC = to_dev(C0)
        handle.dgemm(T, N, n, n, n, 1.0, to_dev(A), n, to_dev(B), n, 0.5, dC, n)
        assert fro(to_host(dC, n, n) - want) <= gemm_bound(n, 1.0, A, B, 0.5, C0)
    finally:
        orc.cblas_off()


def test_full_size_linearity_8192(handle):
    """n = 8192, opA = T: no CPU oracle at this size; check C(A, B1 + B2) = C(A, B1) + C(A, B2)
    within the bar, and one column against a float64 matrix-vector product in torch."""
    import torch
    n = 8192
    A = torch.empty(n * n, dtype=torch.float64, device="cuda")
    B1, B2, C1, C2, C3 = (torch.empty_like(A) for _ in range(5))
    handle.dfill(A, n, n, n, 1)
    handle.dfill(B1, n, n, n, 2)
    handle.dfill(B2, n, n, n, 4)
    handle.dgemm(T, N, n, n, n, 1.0, A, n, B1, n, 0.0, C1, n)
    handle.dgemm(T, N, n, n, n, 1.0, A, n, B2, n, 0.0, C2, n)
    B1.add_(B2)
    handle.dgemm(T, N, n, n, n, 1.0, A, n, B1, n, 0.0, C3, n)
    na, nb = float(A.norm()), float(B1.norm())
    err = float((C3 - C1 - C2).norm())
    assert err <= 3 * 16 * n * EPS * na * nb
    # column 5 of C3 = A^T b  (A is stored k x m column-major: view (m, k) row-major = A^T)
    col = A.view(n, n) @ B1.view(n, n)[5]
    assert float((C3.view(n, n)[5] - col).norm()) <= 16 * n * EPS * na * float(B1.view(n, n)[5].norm())


def test_tile_footprint_beyond_4gib_uses_64_bit_addressing(handle, orc):
    """A k-major operand whose leading dimension is so long that one tile's rows span more than
    4 GiB cannot use 32-bit lane offsets; the launcher must notice and the kernel fall back to
    64-bit element addressing.  A^T is k x m with k = 8.6 M (4.4 GB), B k x 8."""
    import torch
    m, n, k = 64, 8, 8_600_000
    assert 63 * k * 8 >= 2 ** 32
    dA = torch.empty(k * m, dtype=torch.float64, device="cuda")
    dB = torch.empty(k * n, dtype=torch.float64, device="cuda")
    handle.dfill(dA, k, m, k, 21)
    handle.dfill(dB, k, n, k, 22)
    dC = to_dev(np.full((m, n), np.nan, order="F"))
    handle.dgemm(T, N, m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m, variant=4)
    got = to_host(dC, m, n)
    A = to_host(dA, k, m)
    B = to_host(dB, k, n)
    del dA, dB
    orc.cblas_on()
    try:
        want = np.zeros((m, n), order="F")
        orc.dgemm(T, N, m, n, k, 1.0, A, B, 0.0, want)
    finally:
        orc.cblas_off()
    assert fro(got - want) <= 16 * k * EPS * fro(A) * fro(B)


def test_lent_workspace_means_no_split_and_same_answer(handle, orc):
    """A handle that was lent a workspace allocates nothing of its own, so tail tiles are
    computed unsplit; the result meets the same bar."""
    import torch
    ws = torch.empty(1 << 16, dtype=torch.float64, device="cuda")
    handle.set_workspace(ws, ws.numel() * 8)
    orc.cblas_on()
    try:
        for variant in (0, 2, 4):
            run_case(handle, orc, "T", "N", 300, 200, 3000, 1.5, -0.5, variant=variant)
    finally:
        orc.cblas_off()
        handle.set_workspace(None, 0)
