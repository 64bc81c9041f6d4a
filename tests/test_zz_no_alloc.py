"""rtat_dtrsm_static, the entry point that allocates nothing, against rtat_dtrsm: the same
solve through both doors of the C ABI, twice in a row on one GPU (the second call smaller, so
that whatever the first left in the shared static scratch is still there), on a fresh handle
that owns no TRSM scratch of its own.  Bit for bit against rtat_dtrsm with a lent workspace (the
same code path), and both by the backward residual bar 16*M*eps."""
import numpy as np
import pytest

from util import bits_equal, fro, to_dev, to_host

pytestmark = pytest.mark.gpu
EPS = np.finfo(np.float64).eps
LEFT, RIGHT, UPPER, LOWER, N, T, NON_UNIT, UNIT = 141, 142, 121, 122, 111, 112, 131, 132


def _triangle(rng, na, lower):
    a = rng.uniform(-1, 1, (na, na)) / na
    a = np.tril(a, -1) if lower else np.triu(a, 1)
    return np.asfortranarray(a + np.diag(1.0 + rng.uniform(0, 1, na)))


def _solve_both(side, uplo, trans, diag, m, n, alpha, seed):
    import torch
    from rtatblas_amd import native
    rng = np.random.default_rng(seed)
    na = m if side == LEFT else n
    A = _triangle(rng, na, uplo == LOWER)
    lda, ldb = na + 3, m + 5
    Ap = np.full((lda, na), np.nan, order="F")
    Ap[:na] = A
    # the opposite triangle must never be read
    Ap[:na][np.triu_indices(na, 1) if uplo == LOWER else np.tril_indices(na, -1)] = np.nan
    B0 = np.full((ldb, n), np.nan, order="F")
    B0[:m] = rng.uniform(-1, 1, (m, n))
    dA = to_dev(Ap)

    fresh = native.Handle()          # owns no TRSM scratch: the static call must not need any
    fresh.set_stream(torch.cuda.current_stream())
    lent = native.Handle()
    lent.set_stream(torch.cuda.current_stream())
    ws_bytes = lent.lib.rtat_dtrsm_workspace_bytes(side, m, n)
    ws = torch.empty(ws_bytes // 8 + 2, dtype=torch.float64, device="cuda")
    lent.set_workspace(ws, ws.numel() * 8)
    try:
        dX = to_dev(B0)
        fresh.dtrsm_static(side, uplo, trans, diag, m, n, alpha, dA, lda, dX, ldb)
        dY = to_dev(B0)
        lent.dtrsm(side, uplo, trans, diag, m, n, alpha, dA, lda, dY, ldb)
        torch.cuda.synchronize()
        X, Y = to_host(dX, ldb, n), to_host(dY, ldb, n)
        panel_rows, cus = fresh.last_launch()["trsm_panel_rows"], fresh.peaks()[2]
    finally:
        torch.cuda.synchronize()
        fresh.close()
        lent.close()
    assert bits_equal(X[:m], Y[:m])
    assert np.isnan(X[m:]).all()
    # backward residual of the static call's answer
    M = A.copy()
    if diag == UNIT:
        np.fill_diagonal(M, 1.0)
    opM = M.T if trans == T else M
    R = opM @ X[:m] if side == LEFT else X[:m] @ opM
    assert fro(R - alpha * B0[:m]) <= 16 * na * EPS * fro(M) * fro(X[:m])
    return panel_rows, cus


def test_static_matches_dtrsm_twice_in_a_row_second_smaller():
    _solve_both(LEFT, LOWER, N, NON_UNIT, 1500, 700, 1.0, seed=1)
    _solve_both(LEFT, LOWER, N, NON_UNIT, 333, 90, 1.0, seed=2)


@pytest.mark.parametrize("side,uplo,trans,diag,m,n", [
    (LEFT, UPPER, T, UNIT, 2048, 1030),
    (RIGHT, LOWER, N, NON_UNIT, 900, 1100),
    (RIGHT, UPPER, T, NON_UNIT, 4100, 4096),   # the largest order the static scratch serves
    # ... in the layout that sizes it: between 2049 and 4096 right-hand sides on 256 CUs the
    # solve takes 1024-row panels, whose packed blocks need 32 + 4 * 28 blocks at order 4096
    (LEFT, LOWER, N, NON_UNIT, 4096, 3000),
    (LEFT, LOWER, T, NON_UNIT, 129, 5),
])
def test_static_other_cases(side, uplo, trans, diag, m, n):
    panel_rows, cus = _solve_both(side, uplo, trans, diag, m, n, -0.75, seed=m + n)
    if (m, n) == (4096, 3000) and cus == 256:
        assert panel_rows == 1024


def test_static_rejects_orders_beyond_its_scratch_and_accepts_empty():
    import torch
    from rtatblas_amd import native
    h = native.Handle()
    h.set_stream(torch.cuda.current_stream())
    try:
        big = 4097
        dA = torch.zeros(8, dtype=torch.float64, device="cuda")
        before = dA.clone()
        st = h.dtrsm_static(LEFT, LOWER, N, NON_UNIT, big, 1, 1.0, dA, big, dA, big, check=False)
        assert native.STATUS_NAMES[st] == "NOT_SUPPORTED"
        st = h.dtrsm_static(RIGHT, LOWER, N, NON_UNIT, 1, big, 1.0, dA, big, dA, 1, check=False)
        assert native.STATUS_NAMES[st] == "NOT_SUPPORTED"
        assert h.dtrsm_static(LEFT, LOWER, N, NON_UNIT, 0, 4, 1.0, dA, 1, dA, 1, check=False) == 0
        torch.cuda.synchronize()
        assert torch.equal(dA, before)
    finally:
        h.close()


def test_static_call_inside_a_capture_on_a_fresh_handle():
    """What the entry point is for: a handle that has never run a TRSM records one into a graph
    (rtat_dtrsm would report ALLOC_FAILED there) and every replay gives the eager answer."""
    import torch
    from rtatblas_amd import native
    rng = np.random.default_rng(5)
    m, n = 700, 300
    L = _triangle(rng, m, True)
    B0 = np.asfortranarray(rng.uniform(-1, 1, (m, n)))
    dL, dB = to_dev(L), to_dev(B0)
    dX = torch.zeros(m * n, dtype=torch.float64, device="cuda")
    # Another handle runs the call once eagerly, so that the kernels' code is on the device
    # before the capture begins (loading it is the runtime's business, not this library's).
    warm = native.Handle()
    warm.set_stream(torch.cuda.current_stream())
    dX.copy_(dB)
    warm.dtrsm_static(LEFT, LOWER, N, NON_UNIT, m, n, 1.0, dL, m, dX, m)
    torch.cuda.synchronize()
    warm.close()
    h = native.Handle()
    cap = torch.cuda.Stream()
    try:
        h.set_stream(cap)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cap):
            dX.copy_(dB)
            h.dtrsm_static(LEFT, LOWER, N, NON_UNIT, m, n, 1.0, dL, m, dX, m)
        want = None
        for rep in range(3):
            dX.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = to_host(dX, m, n).copy()
            if want is None:
                want = got
                assert fro(L @ got - B0) <= 16 * m * EPS * fro(L) * fro(got)
            assert bits_equal(got, want), rep
    finally:
        torch.cuda.synchronize()
        h.close()
