"""The drop-in, compiled and run: the reference's own sources (gpu-api, timing, methods and the
header-only matrix-op tree) built twice by oracle/Makefile - once as they ship, on hipBLAS
(`make -C oracle ref`), once with the BLAS alias block of their gpu-api.h rebound to
include/rtat_native.h and linked against librtat_native.so instead (`make -C oracle ref_native`).
Both builds are driven through the same extern "C" doors (oracle/ref_shim.cpp) on the same device
buffers.  Bars: workspace sizes equal; copy / pad / transpose / accumulate bit-exact; GEMM /
SYRK within 16 k eps normwise; TRSM agreeing, each answer within the backward-residual bar.
Skipped when the libraries were not built (they are built where the reference tree is mounted)."""
import itertools

import numpy as np
import pytest

from util import EPS, bits_equal, fro, gemm_bound, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112


@pytest.fixture(scope="module")
def both(handle):
    # `handle` first: torch must bring up its HIP runtime before another library that links
    # libamdhip64 is loaded.
    from util import reference_or_skip
    ref_py = reference_or_skip(native=True)
    on_hipblas, on_native = ref_py.load(), ref_py.load(native=True)
    assert not on_hipblas.on_native and on_native.on_native
    return on_hipblas, on_native


@pytest.fixture(scope="module")
def ws():
    import torch
    return torch.full((4 << 20,), float("nan"), dtype=torch.float64, device="cuda")


def stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def test_the_native_build_links_no_hipblas(both):
    import os
    import subprocess
    from oracle import ref_py
    out = subprocess.run(["readelf", "-d", ref_py.NATIVE_LIB_PATH], stdout=subprocess.PIPE, text=True)
    if out.returncode == 0:
        needed = [l for l in out.stdout.splitlines() if "NEEDED" in l]
        assert any("librtat_native" in l for l in needed)
        assert not any("hipblas" in l or "rocblas" in l for l in needed)
    assert os.path.getsize(ref_py.NATIVE_LIB_PATH) > 0


def test_workspace_sizes_equal(both):
    on_hipblas, on_native = both
    m, n, k = 1007, 409, 615
    variants = ["".join(v) for v in itertools.product("NT", repeat=3)]
    variants += ["".join(v) + "".join(p) for v in itertools.product("NT", repeat=3)
                 for p in itertools.product("NP", repeat=3)]
    assert len(variants) == 72
    for v in variants:
        for ta, tb in itertools.product([N, T], [N, T]):
            lda, ldb = (k if ta == T else m) + 3, (n if tb == T else k) + 3
            a = on_hipblas.gemm_workspace(v, ta, tb, m, n, k, lda, ldb, m + 3)
            assert a >= 0 and a == on_native.gemm_workspace(v, ta, tb, m, n, k, lda, ldb, m + 3), v


@pytest.mark.parametrize("m,n,pad", [(10, 12, 32), (257, 100, 8), (1000, 77, 1), (64, 64, 32),
                                     (3000, 2500, 32)])
def test_geam_bit_exact(both, orc, m, n, pad):
    on_hipblas, on_native = both
    A = orc.fill(m, n, m + 3, seed=11)
    dA = to_dev(A)
    for trans in (False, True):
        om, on = (n, m) if trans else (m, n)
        ld = (om + pad - 1) // pad * pad
        for beta in (0.0, 0.5, 1.0):
            C0 = orc.fill(om, on, ld, seed=12)
            a, b = to_dev(C0), to_dev(C0)
            op = T if trans else N
            on_hipblas.geam(op, N, om, on, 1.0, dA, m + 3, beta, a, ld, a, ld, stream())
            on_native.geam(op, N, om, on, 1.0, dA, m + 3, beta, b, ld, b, ld, stream())
            assert bits_equal(to_host(a, ld, on), to_host(b, ld, on)), (trans, beta)


@pytest.mark.parametrize("ta,tb", list(itertools.product([N, T], [N, T])))
def test_gemm_every_variant(both, orc, ws, ta, tb):
    on_hipblas, on_native = both
    m, n, k = 270, 245, 262
    A = orc.fill(k if ta == T else m, m if ta == T else k, seed=1)
    B = orc.fill(n if tb == T else k, k if tb == T else n, seed=2)
    C0 = orc.fill(m, n, m + 3, seed=3)
    dA, dB = to_dev(A), to_dev(B)
    variants = ["".join(v) for v in itertools.product("NT", repeat=3)]
    variants += ["".join(v) + "".join(p) for v in itertools.product("NT", repeat=3)
                 for p in itertools.product("NP", repeat=3)][1::5]
    worst = 0.0
    for v in variants:
        a, b = to_dev(C0), to_dev(C0)
        on_hipblas.gemm(v, ta, tb, m, n, k, 1.0, dA, A.shape[0], dB, B.shape[0], 0.5, a, m + 3, ws,
                        ws.numel() * 8, stream())
        on_native.gemm(v, ta, tb, m, n, k, 1.0, dA, A.shape[0], dB, B.shape[0], 0.5, b, m + 3, ws,
                       ws.numel() * 8, stream())
        x, y = to_host(a, m + 3, n), to_host(b, m + 3, n)
        bar = gemm_bound(k, 1.0, A, B, 0.5, C0[:m])
        worst = max(worst, fro(x[:m] - y[:m]) / bar)
        assert fro(x[:m] - y[:m]) <= bar, v
        assert bits_equal(x[m:], y[m:]), v
    print("GEMM variants: worst difference / (16 k eps bar) = %.2e" % worst)


@pytest.mark.parametrize("uplo,trans", list(itertools.product([121, 122], [N, T])))
def test_syrk_every_variant(both, orc, ws, uplo, trans):
    on_hipblas, on_native = both
    n, k = 213, 74
    A = orc.fill(k if trans == T else n, n if trans == T else k, seed=4)
    C0 = orc.fill(n, n, seed=5, kind=1)
    dA = to_dev(A)
    for v in ("FF", "FT", "TF", "TT"):
        a, b = to_dev(C0), to_dev(C0)
        on_hipblas.syrk(v, uplo, trans, n, k, -1.0, dA, A.shape[0], 1.0, a, n, ws, ws.numel() * 8,
                        stream())
        on_native.syrk(v, uplo, trans, n, k, -1.0, dA, A.shape[0], 1.0, b, n, ws, ws.numel() * 8,
                       stream())
        x, y = to_host(a, n, n), to_host(b, n, n)
        tri = np.tril if uplo == 122 else np.triu
        assert fro(tri(x) - tri(y)) <= 16 * k * EPS * (fro(A) ** 2 + fro(C0)), v
        other = (lambda z: np.triu(z, 1)) if uplo == 122 else (lambda z: np.tril(z, -1))
        assert bits_equal(other(x), other(y)), v     # incl. the beta-scaling quirk of "?T"


@pytest.mark.parametrize("side,uplo,trans,diag",
                         list(itertools.product([141, 142], [121, 122], [N, T], [131, 132])))
def test_trsm_every_case_and_variant(both, orc, ws, side, uplo, trans, diag):
    on_hipblas, on_native = both
    m, n = 243, 252
    na = m if side == 141 else n
    A = orc.fill(na, na, seed=6, kind=4)
    B0 = orc.fill(m, n, seed=7)
    dA = to_dev(A)
    M = (np.tril(A) if uplo == 122 else np.triu(A)).copy()
    if diag == 132:
        np.fill_diagonal(M, 1.0)
    opM = M.T if trans == T else M
    for v in ("FF", "FT", "TF", "TT"):
        a, b = to_dev(B0), to_dev(B0)
        on_hipblas.trsm(v, side, uplo, trans, diag, m, n, 1.0, dA, na, a, m, ws, ws.numel() * 8,
                        stream())
        on_native.trsm(v, side, uplo, trans, diag, m, n, 1.0, dA, na, b, m, ws, ws.numel() * 8,
                       stream())
        x, y = to_host(a, m, n), to_host(b, m, n)
        assert np.allclose(x, y, rtol=1e-9, atol=1e-12), v
        for sol in (x, y):
            r = opM @ sol - B0 if side == 141 else sol @ opM - B0
            assert fro(r) <= 16 * na * EPS * fro(M) * fro(sol), v


def test_full_size_configs(both, handle, ws):
    """The benchmark configurations through the reference's executors on either boundary: DGEMM
    opA = T n = 8192 beta = 0.5 and 10007 x 4099 x 6151 with ld = rows + 3, DSYRK lower
    8192 / 2048, DTRSM left / lower 8192.  Norms are taken on the device."""
    import torch
    from rtatblas_amd import native
    on_hipblas, on_native = both

    def dev(count):
        return torch.empty(count, dtype=torch.float64, device="cuda")

    def view(t, ld, rows, cols):
        return t.view(cols, ld)[:, :rows]

    def fro_dev(x):
        return float(torch.linalg.norm(x.reshape(-1)))

    for (ta, m, n, k, pad, beta) in [(T, 8192, 8192, 8192, 0, 0.5), (N, 10007, 4099, 6151, 3, 0.0)]:
        ar, ac = (k, m) if ta == T else (m, k)
        lda, ldb, ldc = ar + pad, k + pad, m + pad
        A, B, C0 = dev(lda * ac), dev(ldb * n), dev(ldc * n)
        handle.dfill(A, ar, ac, lda, 1)
        handle.dfill(B, k, n, ldb, 2)
        handle.dfill(C0, m, n, ldc, 3)
        a, b = C0.clone(), C0.clone()
        on_hipblas.gemm("NNN", ta, N, m, n, k, 1.0, A, lda, B, ldb, beta, a, ldc, ws, ws.numel() * 8,
                        stream())
        on_native.gemm("NNN", ta, N, m, n, k, 1.0, A, lda, B, ldb, beta, b, ldc, ws, ws.numel() * 8,
                       stream())
        torch.cuda.synchronize()
        diff = fro_dev(view(a, ldc, m, n) - view(b, ldc, m, n))
        bar = 16 * k * EPS * (fro_dev(view(A, lda, ar, ac)) * fro_dev(view(B, ldb, k, n))
                              + abs(beta) * fro_dev(view(C0, ldc, m, n)))
        print("DGEMM %dx%dx%d: difference / (16 k eps bar) = %.2e" % (m, n, k, diff / bar))
        assert diff <= bar
        assert torch.equal(a.view(n, ldc)[:, m:].view(torch.int64),
                           b.view(n, ldc)[:, m:].view(torch.int64))
        del A, B, C0, a, b

    n, k = 8192, 2048
    A, C0 = dev(n * k), dev(n * n)
    handle.dfill(A, n, k, n, 1)
    handle.dfill(C0, n, n, n, 3, native.FILL_SYMMETRIC)
    a, b = C0.clone(), C0.clone()
    on_hipblas.syrk("FF", 122, N, n, k, 1.0, A, n, 1.0, a, n, ws, ws.numel() * 8, stream())
    on_native.syrk("FF", 122, N, n, k, 1.0, A, n, 1.0, b, n, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()
    lower = torch.triu(torch.ones(n, n, dtype=torch.bool, device="cuda"))   # cols x rows view
    d = (a.view(n, n) - b.view(n, n)) * lower
    assert fro_dev(d) <= 16 * k * EPS * (fro_dev(A) ** 2 + fro_dev(C0))
    assert torch.equal(a.view(n, n).view(torch.int64)[~lower], b.view(n, n).view(torch.int64)[~lower])
    del A, C0, a, b, d, lower

    m = 8192
    L, B0 = dev(m * m), dev(m * m)
    handle.dfill(L, m, m, m, 1, native.FILL_TRI_LOWER)       # strict upper triangle = NaN
    handle.dfill(B0, m, m, m, 2)
    a, b = B0.clone(), B0.clone()
    on_hipblas.trsm("FF", 141, 122, N, 131, m, m, 1.0, L, m, a, m, ws, ws.numel() * 8, stream())
    on_native.trsm("FF", 141, 122, N, 131, m, m, 1.0, L, m, b, m, ws, ws.numel() * 8, stream())
    torch.cuda.synchronize()
    assert bool(torch.isfinite(b).all())
    rel = fro_dev(a - b) / fro_dev(a)
    assert rel <= 1e-10, rel
