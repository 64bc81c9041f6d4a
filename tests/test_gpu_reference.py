"""Parity against THE REFERENCE ITSELF: the reference's executors, compiled from its own
sources on hipBLAS (oracle/_ref/librtat_ref.so), run on the same seeded inputs as this
library's variant trees.  Bars: copy / pad / transpose bit-exact; GEMM / SYRK within
16 k eps normwise of each other (the one-sided bar, although both sides round: the measured
differences are a few thousandths of it); TRSM by each side's backward residual and mutual
agreement.  Skipped when the reference library was not
built (it is built where the reference tree is available)."""
import itertools

import numpy as np
import pytest

from util import EPS, bits_equal, fro, gemm_bound, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112


@pytest.fixture(scope="module")
def ref(handle):
    # `handle` first: torch must bring up its HIP runtime before another library that links
    # libamdhip64 is loaded, or the process ends up with two runtimes and no visible device.
    from util import reference_or_skip
    ref_py = reference_or_skip()
    ref_py.load()
    return ref_py


@pytest.fixture(scope="module")
def ws():
    import torch
    return torch.full((4 << 20,), float("nan"), dtype=torch.float64, device="cuda")


def stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def test_workspace_accounting_equals_the_references(ref):  # noqa: needs no kernel, only the library
    from rtatblas_amd import planner
    m, n, k = 1007, 409, 615
    for method in ("gemm", "gemm_pad"):
        p = planner.Planner(method)
        for v in p.variants():
            for ta, tb in itertools.product([N, T], [N, T]):
                lda, ldb = (k if ta == T else m) + 3, (n if tb == T else k) + 3
                assert p.gemm_workspace(v, ta, tb, m, n, k, lda, ldb, m + 3) == \
                    ref.gemm_workspace(v, ta, tb, m, n, k, lda, ldb, m + 3)


@pytest.mark.parametrize("m,n,pad", [(10, 12, 32), (257, 100, 8), (1000, 77, 1), (64, 64, 32)])
def test_geam_move_bit_exact_with_hipblas(handle, ref, orc, m, n, pad):
    A = orc.fill(m, n, m + 3, seed=11)
    dA = to_dev(A)
    for trans in (False, True):
        om, on = (n, m) if trans else (m, n)
        ld = (om + pad - 1) // pad * pad
        mine = to_dev(np.full((ld, on), np.nan, order="F"))
        theirs = to_dev(np.full((ld, on), np.nan, order="F"))
        handle.dgeam(T if trans else N, N, om, on, 1.0, dA, m + 3, 0.0, mine, ld, mine, ld)
        ref.geam(T if trans else N, N, om, on, 1.0, dA, m + 3, 0.0, theirs, ld, theirs, ld, stream())
        assert bits_equal(to_host(mine, ld, on), to_host(theirs, ld, on))


@pytest.mark.parametrize("beta", [0.5, 1.0])
def test_geam_accumulate_bit_exact_with_hipblas(handle, ref, orc, beta):
    m, n = 301, 259
    S = orc.fill(n, m, n + 1, seed=12)
    C0 = orc.fill(m, n, m + 2, seed=13)
    mine, theirs = to_dev(C0), to_dev(C0)
    handle.dgeam(T, N, m, n, 1.0, to_dev(S), n + 1, beta, mine, m + 2, mine, m + 2)
    ref.geam(T, N, m, n, 1.0, to_dev(S), n + 1, beta, theirs, m + 2, theirs, m + 2, stream())
    assert bits_equal(to_host(mine, m + 2, n), to_host(theirs, m + 2, n))


@pytest.mark.parametrize("ta,tb", list(itertools.product([N, T], [N, T])))
def test_gemm_variants_against_the_reference(handle, ref, orc, ws, ta, tb):
    from rtatblas_amd import planner
    m, n, k = 270, 245, 262
    A = orc.fill(k if ta == T else m, m if ta == T else k, seed=1)
    B = orc.fill(n if tb == T else k, k if tb == T else n, seed=2)
    C0 = orc.fill(m, n, m + 3, seed=3)
    dA, dB = to_dev(A), to_dev(B)
    for method in ("gemm", "gemm_pad"):
        p = planner.Planner(method)
        for v in (p.variants() if method == "gemm" else p.variants()[1::7]):
            mine, theirs = to_dev(C0), to_dev(C0)
            p.gemm(handle, v, ta, tb, m, n, k, 1.0, dA, A.shape[0], dB, B.shape[0], 0.5, mine,
                   m + 3, ws, ws.numel() * 8)
            ref.gemm(v, ta, tb, m, n, k, 1.0, dA, A.shape[0], dB, B.shape[0], 0.5, theirs, m + 3,
                     ws, ws.numel() * 8, stream())
            a, b = to_host(mine, m + 3, n), to_host(theirs, m + 3, n)
            assert fro(a[:m] - b[:m]) <= gemm_bound(k, 1.0, A, B, 0.5, C0[:m]), v
            assert bits_equal(a[m:], b[m:])


@pytest.mark.parametrize("uplo,trans", list(itertools.product([121, 122], [N, T])))
def test_syrk_variants_against_the_reference(handle, ref, orc, ws, uplo, trans):
    from rtatblas_amd import planner
    n, k = 213, 74
    A = orc.fill(k if trans == T else n, n if trans == T else k, seed=4)
    C0 = orc.fill(n, n, seed=5, kind=1)
    p = planner.Planner("syrk")
    for v in p.variants():
        mine, theirs = to_dev(C0), to_dev(C0)
        p.syrk(handle, v, uplo, trans, n, k, -1.0, to_dev(A), A.shape[0], 1.0, mine, n, ws,
               ws.numel() * 8)
        ref.syrk(v, uplo, trans, n, k, -1.0, to_dev(A), A.shape[0], 1.0, theirs, n, ws,
                 ws.numel() * 8, stream())
        a, b = to_host(mine, n, n), to_host(theirs, n, n)
        tri = np.tril if uplo == 122 else np.triu
        assert fro(tri(a) - tri(b)) <= 16 * k * EPS * (fro(A) ** 2 + fro(C0)), v
        other = (lambda x: np.triu(x, 1)) if uplo == 122 else (lambda x: np.tril(x, -1))
        assert bits_equal(other(a), other(b)), v    # incl. the beta-scaling quirk of "?T"


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [121, 122], [N, T], [131, 132])))
def test_trsm_variants_against_the_reference(handle, ref, orc, ws, side, uplo, trans, diag):
    from rtatblas_amd import planner
    m, n = 243, 252
    na = m if side == 141 else n
    A = orc.fill(na, na, seed=6, kind=4)
    B0 = orc.fill(m, n, seed=7)
    p = planner.Planner("trsm")
    for v in p.variants():
        mine, theirs = to_dev(B0), to_dev(B0)
        p.trsm(handle, v, side, uplo, trans, diag, m, n, 1.0, to_dev(A), na, mine, m, ws,
               ws.numel() * 8)
        ref.trsm(v, side, uplo, trans, diag, m, n, 1.0, to_dev(A), na, theirs, m, ws,
                 ws.numel() * 8, stream())
        a, b = to_host(mine, m, n), to_host(theirs, m, n)
        assert np.allclose(a, b, rtol=1e-9, atol=1e-12), v


def test_full_size_configs_against_the_reference(handle, ref, ws):
    """The benchmark configurations at their real sizes, this library and the reference (its
    executors on hipBLAS) side by side on the same device operands; norms are taken on the
    device.  DGEMM opA=T n=8192 beta=0.5; DGEMM 10007x4099x6151 with ld = rows+3; DSYRK lower
    8192/2048 alpha=beta=1; DTRSM left/lower/N/non-unit 8192."""
    import torch
    from rtatblas_amd import native, planner

    def dev(count):
        return torch.empty(count, dtype=torch.float64, device="cuda")

    def view(t, ld, rows, cols):
        return t.view(cols, ld)[:, :rows]          # column-major (ld, cols) seen as cols x rows

    def fro_dev(x):
        return float(torch.linalg.norm(x.reshape(-1)))

    gp = planner.Planner("gemm")
    for (ta, m, n, k, pad, beta) in [(T, 8192, 8192, 8192, 0, 0.5), (N, 10007, 4099, 6151, 3, 0.0)]:
        ar, ac = (k, m) if ta == T else (m, k)
        lda, ldb, ldc = ar + pad, k + pad, m + pad
        A, B, C0 = dev(lda * ac), dev(ldb * n), dev(ldc * n)
        handle.dfill(A, ar, ac, lda, 1)
        handle.dfill(B, k, n, ldb, 2)
        handle.dfill(C0, m, n, ldc, 3)
        mine, theirs = C0.clone(), C0.clone()
        gp.gemm(handle, "NNN", ta, N, m, n, k, 1.0, A, lda, B, ldb, beta, mine, ldc, ws, ws.numel() * 8)
        ref.gemm("NNN", ta, N, m, n, k, 1.0, A, lda, B, ldb, beta, theirs, ldc, ws, ws.numel() * 8,
                 stream())
        torch.cuda.synchronize()
        diff = fro_dev(view(mine, ldc, m, n) - view(theirs, ldc, m, n))
        bound = 16 * k * EPS * (fro_dev(view(A, lda, ar, ac)) * fro_dev(view(B, ldb, k, n))
                                    + abs(beta) * fro_dev(view(C0, ldc, m, n)))
        print("DGEMM %dx%dx%d: difference / (16 k eps bar) = %.2e" % (m, n, k, diff / bound))
        assert diff <= bound, (ta, m, n, k, diff, bound)
        if pad:     # padding rows (NaN from the fill) are untouched by both
            assert torch.equal(view(mine, ldc, ldc, n)[:, m:].view(torch.int64),
                               view(C0, ldc, ldc, n)[:, m:].view(torch.int64))
        del A, B, C0, mine, theirs

    n, k = 8192, 2048
    A, C0 = dev(n * k), dev(n * n)
    handle.dfill(A, n, k, n, 1)
    handle.dfill(C0, n, n, n, 3, native.FILL_SYMMETRIC)
    mine, theirs = C0.clone(), C0.clone()
    sp = planner.Planner("syrk")
    sp.syrk(handle, "FF", 122, N, n, k, 1.0, A, n, 1.0, mine, n, ws, ws.numel() * 8)
    ref.syrk("FF", 122, N, n, k, 1.0, A, n, 1.0, theirs, n, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()
    lower = torch.triu(torch.ones(n, n, dtype=torch.bool, device="cuda"))   # cols x rows view
    d = (view(mine, n, n, n) - view(theirs, n, n, n)) * lower
    bound = 16 * k * EPS * (fro_dev(A) ** 2 + fro_dev(C0))
    assert fro_dev(d) <= bound
    # the strict upper triangle is untouched by both
    assert torch.equal((view(mine, n, n, n).view(torch.int64))[~lower],
                       (view(C0, n, n, n).view(torch.int64))[~lower])
    del A, C0, mine, theirs, d, lower

    m = 8192
    L, B0 = dev(m * m), dev(m * m)
    handle.dfill(L, m, m, m, 1, native.FILL_TRI_LOWER)       # strict upper triangle = NaN
    handle.dfill(B0, m, m, m, 2)
    mine, theirs = B0.clone(), B0.clone()
    tp = planner.Planner("trsm")
    tp.trsm(handle, "FF", 141, 122, N, 131, m, m, 1.0, L, m, mine, m, ws, ws.numel() * 8)
    ref.trsm("FF", 141, 122, N, 131, m, m, 1.0, L, m, theirs, m, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()
    assert bool(torch.isfinite(mine).all())
    # forward agreement, scaled by the conditioning of the (well-conditioned) triangle
    rel = fro_dev(mine - theirs) / fro_dev(theirs)
    assert rel <= 1e-10, rel
    # backward residual of this library's solution through its own DGEMM: L X - B
    Lz = torch.nan_to_num(L, nan=0.0)
    R = B0.clone()
    handle.dgemm(N, N, m, m, m, 1.0, Lz, m, mine, m, -1.0, R, m)
    torch.cuda.synchronize()
    assert fro_dev(R) <= 16 * m * EPS * fro_dev(Lz) * fro_dev(mine)


@pytest.mark.parametrize("ta,m,n,k,pad,beta", [(T, 1024, 1024, 1024, 0, 0.5), (T, 2048, 2048, 2048, 0, 0.5),
                                               (T, 4096, 4096, 4096, 0, 0.5), (T, 16384, 16384, 16384, 0, 0.5),
                                               (N, 65536, 256, 256, 3, 0.0), (N, 512, 512, 512, 0, 0.0)])
def test_remaining_dgemm_configs_against_the_reference(handle, ref, ws, ta, m, n, k, pad, beta):
    """The other sizes of the opA = T sweep (n = 1024 ... 16384, beta = 0.5), the tall-skinny
    65536 x 256 x 256 with ld = rows + 3 and the 512^3 plumbing case: this library and the
    reference on the same device operands, norms on the device, padding rows untouched."""
    import torch
    from rtatblas_amd import planner

    def view(t, ld, rows, cols):
        return t.view(cols, ld)[:, :rows]

    def fro_dev(x):
        return float(torch.linalg.norm(x.reshape(-1)))

    ar, ac = (k, m) if ta == T else (m, k)
    lda, ldb, ldc = ar + pad, k + pad, m + pad
    A = torch.empty(lda * ac, dtype=torch.float64, device="cuda")
    B = torch.empty(ldb * n, dtype=torch.float64, device="cuda")
    C0 = torch.empty(ldc * n, dtype=torch.float64, device="cuda")
    handle.dfill(A, ar, ac, lda, 1)
    handle.dfill(B, k, n, ldb, 2)
    handle.dfill(C0, m, n, ldc, 3)
    mine, theirs = C0.clone(), C0.clone()
    gp = planner.Planner("gemm")
    gp.gemm(handle, "NNN", ta, N, m, n, k, 1.0, A, lda, B, ldb, beta, mine, ldc, ws, ws.numel() * 8)
    ref.gemm("NNN", ta, N, m, n, k, 1.0, A, lda, B, ldb, beta, theirs, ldc, ws, ws.numel() * 8,
             stream())
    torch.cuda.synchronize()
    diff = fro_dev(view(mine, ldc, m, n) - view(theirs, ldc, m, n))
    bound = 16 * k * EPS * (fro_dev(view(A, lda, ar, ac)) * fro_dev(view(B, ldb, k, n))
                                + abs(beta) * fro_dev(view(C0, ldc, m, n)))
    print("DGEMM %dx%dx%d: difference / (16 k eps bar) = %.2e" % (m, n, k, diff / bound))
    assert diff <= bound, (ta, m, n, k, diff, bound)
    if pad:
        assert torch.equal(view(mine, ldc, ldc, n)[:, m:].view(torch.int64),
                           view(C0, ldc, ldc, n)[:, m:].view(torch.int64))


@pytest.mark.parametrize("trans,m,n,lda,ldc,beta", [
    (True, 8192, 8192, 8192, 8192, 0.0), (True, 16384, 16384, 16384, 16384, 0.0),
    (False, 8192, 8192, 8192, 8224, 0.0), (True, 8192, 8192, 8192, 8192, 0.5),
    (False, 10007, 6151, 10010, 10016, 0.0), (False, 6151, 4099, 6154, 6176, 0.0),
    (False, 65536, 256, 65539, 65536, 0.0), (True, 6151, 10007, 10010, 6151, 0.0),
    (True, 4099, 6151, 6154, 4099, 0.5), (False, 8192, 8192, 8192, 8192, 0.5)])
def test_full_size_geam_bit_exact_with_hipblas(handle, ref, trans, m, n, lda, ldc, beta):
    """The bandwidth-bound nodes at the benchmark's sizes (transposes of 8192^2 and 16384^2,
    the pad copies and the transpose of the awkward DGEMM's operands, accumulates with beta =
    0.5): this library's kernels and hipBLAS geam on the same device operands, bit for bit,
    padding rows included."""
    import torch
    ar, ac = (n, m) if trans else (m, n)
    S = torch.empty(lda * ac, dtype=torch.float64, device="cuda")
    handle.dfill(S, ar, ac, lda, 21)
    C0 = torch.empty(ldc * n, dtype=torch.float64, device="cuda")
    handle.dfill(C0, m, n, ldc, 22)                      # padding rows are NaN
    mine, theirs = C0.clone(), C0.clone()
    op = T if trans else N
    handle.dgeam(op, N, m, n, 1.0, S, lda, beta, mine, ldc, mine, ldc)
    ref.geam(op, N, m, n, 1.0, S, lda, beta, theirs, ldc, theirs, ldc, stream())
    torch.cuda.synchronize()
    assert torch.equal(mine.view(torch.int64), theirs.view(torch.int64))
    assert not torch.equal(mine.view(torch.int64), C0.view(torch.int64))


@pytest.mark.parametrize("side,uplo,trans,diag", [(141, 121, T, 131), (142, 122, N, 131),
                                                  (142, 121, T, 132), (141, 122, T, 132)])
def test_full_size_trsm_other_cases_against_the_reference(handle, ref, ws, side, uplo, trans, diag):
    """M = N = 8192 for combinations other than the benchmark's (upper, transposed, right side,
    unit diagonal): agreement with the reference on hipBLAS and the backward residual through
    this library's DGEMM.  The triangle that is not referenced holds NaN."""
    import torch
    from rtatblas_amd import native, planner

    def fro_dev(x):
        return float(torch.linalg.norm(x.reshape(-1)))

    m = 8192
    L = torch.empty(m * m, dtype=torch.float64, device="cuda")
    B0 = torch.empty(m * m, dtype=torch.float64, device="cuda")
    handle.dfill(L, m, m, m, 1, native.FILL_TRI_LOWER)       # strict upper triangle = NaN
    if uplo == 121:                                          # the same triangle, stored upper
        L = L.view(m, m).t().contiguous().view(-1)
    handle.dfill(B0, m, m, m, 2)
    mine, theirs = B0.clone(), B0.clone()
    tp = planner.Planner("trsm")
    tp.trsm(handle, "FF", side, uplo, trans, diag, m, m, 1.0, L, m, mine, m, ws, ws.numel() * 8)
    ref.trsm("FF", side, uplo, trans, diag, m, m, 1.0, L, m, theirs, m, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()
    assert bool(torch.isfinite(mine).all())
    rel = fro_dev(mine - theirs) / fro_dev(theirs)
    assert rel <= 1e-10, rel
    Lz = torch.nan_to_num(L, nan=0.0)
    if diag == 132:                                          # unit: the stored diagonal is ignored
        Lv = Lz.view(m, m)
        Lv.diagonal().fill_(1.0)
    R = B0.clone()
    if side == 141:
        handle.dgemm(trans, N, m, m, m, 1.0, Lz, m, mine, m, -1.0, R, m)     # op(A) X - B
    else:
        handle.dgemm(N, trans, m, m, m, 1.0, mine, m, Lz, m, -1.0, R, m)     # X op(A) - B
    torch.cuda.synchronize()
    assert fro_dev(R) <= 16 * m * EPS * fro_dev(Lz) * fro_dev(mine)


@pytest.mark.parametrize("uplo,trans", [(121, N), (122, T), (121, T)])
def test_full_size_syrk_other_cases_against_the_reference(handle, ref, ws, uplo, trans):
    """N = 8192, K = 2048 for the combinations other than the benchmark's lower / no-trans."""
    import torch
    from rtatblas_amd import native, planner

    def fro_dev(x):
        return float(torch.linalg.norm(x.reshape(-1)))

    n, k = 8192, 2048
    ar, ac = (k, n) if trans == T else (n, k)
    A = torch.empty(ar * ac, dtype=torch.float64, device="cuda")
    C0 = torch.empty(n * n, dtype=torch.float64, device="cuda")
    handle.dfill(A, ar, ac, ar, 1)
    handle.dfill(C0, n, n, n, 3, native.FILL_SYMMETRIC)
    mine, theirs = C0.clone(), C0.clone()
    sp = planner.Planner("syrk")
    sp.syrk(handle, "FF", uplo, trans, n, k, 1.0, A, ar, 1.0, mine, n, ws, ws.numel() * 8)
    ref.syrk("FF", uplo, trans, n, k, 1.0, A, ar, 1.0, theirs, n, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()
    tri = torch.triu(torch.ones(n, n, dtype=torch.bool, device="cuda"))     # [col][row]: row <= col is upper
    wanted = tri if uplo == 122 else tri.t()        # view is cols x rows: lower triangle = col <= row
    d = (mine.view(n, n) - theirs.view(n, n)) * wanted
    assert fro_dev(d) <= 16 * k * EPS * (fro_dev(A) ** 2 + fro_dev(C0))
    assert torch.equal(mine.view(n, n).view(torch.int64)[~wanted], C0.view(n, n).view(torch.int64)[~wanted])
    assert not torch.equal(mine, C0)


@pytest.mark.parametrize("n", [1024, 4096])
@pytest.mark.parametrize("spread,least_cond", [(0.4, 3e1), (0.6, 2e2), (0.8, 2e3), (1.0, 2e4),
                                               (1.2, 5e5), (1.5, 4e7)])
def test_trsm_backward_residual_as_diagonal_blocks_get_ill_conditioned(handle, ref, ws, n, spread,
                                                                       least_cond):
    """DTRSM inverts the 128 x 128 diagonal blocks of A explicitly, so its backward error could
    grow with their condition numbers.  Here the blocks' strict lower triangles are uniform in
    [-spread, spread] on a diagonal in [1, 2) (condition numbers from 4e1 at spread 0.4 to 5e10 at
    spread 1.5) while the rest of A stays small, and the solve is compared with the reference's
    (hipBLAS, which inverts diagonal blocks as well) on the same input: the backward residual
    |AX - B| / (|A| |X|) must stay within 4 x the reference's and within 16 M eps."""
    import torch
    nrhs = 256
    g = torch.Generator(device="cuda").manual_seed(n)
    U = torch.rand(n, n, dtype=torch.float64, device="cuda", generator=g) * 2 - 1
    idx = torch.arange(n, device="cuda") // 128
    in_block = idx[:, None] == idx[None, :]
    A = torch.where(in_block, U * spread, U / n).tril(-1) + torch.diag(
        1 + torch.rand(n, dtype=torch.float64, device="cuda", generator=g))
    conds = [float(torch.linalg.cond(A[i:i + 128, i:i + 128])) for i in range(0, n, 128)]
    assert min(conds) >= least_cond, conds
    Acm = A.t().contiguous()                              # column-major storage of A
    B = torch.rand(nrhs, n, dtype=torch.float64, device="cuda", generator=g) * 2 - 1   # [col][row]
    mine, theirs = B.clone(), B.clone()
    handle.dtrsm(141, 122, N, 131, n, nrhs, 1.0, Acm, n, mine, n)
    ref.trsm("FF", 141, 122, N, 131, n, nrhs, 1.0, Acm, n, theirs, n, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()

    def residual(X):
        Xm = X.t()
        return float(torch.linalg.norm(A @ Xm - B.t()) /
                     (torch.linalg.norm(A) * torch.linalg.norm(Xm)))

    ours, refs = residual(mine), residual(theirs)
    print("n=%d block cond %.1e..%.1e: residual ours %.2e, reference %.2e, bar %.2e"
          % (n, min(conds), max(conds), ours, refs, 16 * n * EPS))
    assert ours <= 4 * refs
    assert ours <= 16 * n * EPS


def test_fused_variants_against_the_references_unfused_trees(handle, ref, orc, ws):
    """The fused forms ("NNX", "FX", "XF": the transposition of the result done by the kernel, one
    launch, no scratch) against the trees the reference builds for "NNT", "FT" and "TF" on
    hipBLAS: same inputs, the bars of the routines."""
    from rtatblas_amd import planner
    m, n, k = 270, 245, 262
    A, B, C0 = orc.fill(k, m, seed=1), orc.fill(k, n, seed=2), orc.fill(m, n, m + 3, seed=3)
    mine, theirs = to_dev(C0), to_dev(C0)
    planner.Planner("gemm_fused").gemm(handle, "NNX", T, N, m, n, k, 1.0, to_dev(A), k, to_dev(B), k,
                                       0.5, mine, m + 3, None, 0)
    ref.gemm("NNT", T, N, m, n, k, 1.0, to_dev(A), k, to_dev(B), k, 0.5, theirs, m + 3, ws,
             ws.numel() * 8, stream())
    a, b = to_host(mine, m + 3, n), to_host(theirs, m + 3, n)
    assert fro(a[:m] - b[:m]) <= gemm_bound(k, 1.0, A, B, 0.5, C0[:m])
    assert bits_equal(a[m:], b[m:])

    ns, ks = 213, 74
    As, Cs = orc.fill(ns, ks, seed=4), orc.fill(ns, ns, seed=5, kind=1)
    mine, theirs = to_dev(Cs), to_dev(Cs)
    planner.Planner("syrk_fused").syrk(handle, "FX", 122, N, ns, ks, -1.0, to_dev(As), ns, 1.0, mine,
                                       ns, None, 0)
    ref.syrk("FT", 122, N, ns, ks, -1.0, to_dev(As), ns, 1.0, theirs, ns, ws, ws.numel() * 8, stream())
    a, b = to_host(mine, ns, ns), to_host(theirs, ns, ns)
    assert fro(np.tril(a) - np.tril(b)) <= 16 * ks * EPS * (fro(As) ** 2 + fro(Cs))
    assert bits_equal(np.triu(a, 1), np.triu(Cs, 1))        # beta = 1: the tree leaves it as well

    mt, nt = 243, 252
    At, Bt = orc.fill(mt, mt, seed=6, kind=4), orc.fill(mt, nt, seed=7)
    mine, theirs = to_dev(Bt), to_dev(Bt)
    planner.Planner("trsm_fused").trsm(handle, "XF", 141, 122, N, 131, mt, nt, 1.0, to_dev(At), mt,
                                       mine, mt, None, 0)
    ref.trsm("TF", 141, 122, N, 131, mt, nt, 1.0, to_dev(At), mt, theirs, mt, ws, ws.numel() * 8,
             stream())
    assert np.allclose(to_host(mine, mt, nt), to_host(theirs, mt, nt), rtol=1e-9, atol=1e-12)
