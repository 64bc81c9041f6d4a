"""Seeded random sweep of shapes, leading dimensions, scalars, operand flags and kernel variants
through the C ABI against the CPU oracle (host CBLAS backend): the combinations of ragged edges,
odd leading dimensions, K tails, tail splitting, tail subdivision, thin edge tiles and triangle
masks that the hand-picked cases may miss.  Bars as in the other GPU tests."""
import numpy as np
import pytest

from util import EPS, bits_equal, fro, gemm_bound, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112
UP, LO = 121, 122


def padded(rng, m, n, ld):
    a = np.full((ld, n), np.nan, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n))
    return a


def dims(rng):
    kind = rng.integers(0, 6)
    if kind == 5:      # two rounds of tiles or more, a thin last tile row and column
        return (128 * int(rng.integers(32, 38)) + int(rng.integers(1, 40)),
                128 * int(rng.integers(32, 36)) + int(rng.integers(1, 40)), int(rng.integers(8, 80)))
    if kind == 4:      # more than a round of tiles and a short k (leftover tiles cut into pieces)
        return int(rng.integers(2800, 4300)), int(rng.integers(2800, 4300)), int(rng.integers(4, 48))
    if kind == 0:      # small and ragged
        return int(rng.integers(1, 200)), int(rng.integers(1, 200)), int(rng.integers(1, 300))
    if kind == 1:      # a few tiles, long k (tail splitting)
        return int(rng.integers(60, 700)), int(rng.integers(60, 700)), int(rng.integers(900, 3000))
    if kind == 2:      # more tiles than workgroup slots for the small shapes
        return int(rng.integers(1500, 2600)), int(rng.integers(1500, 2600)), int(rng.integers(130, 400))
    return int(rng.integers(1, 70)), int(rng.integers(300, 1500)), int(rng.integers(16, 600))


@pytest.mark.parametrize("seed", range(6))
def test_random_dgemm(handle, orc, seed):
    rng = np.random.default_rng(1000 + seed)
    orc.cblas_on()
    try:
        for _ in range(10):
            m, n, k = dims(rng)
            ta, tb = rng.choice([N, T]), rng.choice([N, T])
            ar, ac = (k, m) if ta == T else (m, k)
            br, bc = (n, k) if tb == T else (k, n)
            A = padded(rng, ar, ac, ar + int(rng.integers(0, 4)))
            B = padded(rng, br, bc, br + int(rng.integers(0, 4)))
            C0 = padded(rng, m, n, m + int(rng.integers(0, 4)))
            alpha = float(rng.choice([1.0, -1.0, 0.5, 1.75]))
            beta = float(rng.choice([0.0, 1.0, -0.5]))
            variant = int(rng.integers(0, 5))
            want = C0.copy(order="F")
            orc.dgemm(ta, tb, m, n, k, alpha, A, B, beta, want)
            dC = to_dev(C0)
            handle.dgemm(ta, tb, m, n, k, alpha, to_dev(A), A.shape[0], to_dev(B), B.shape[0], beta,
                         dC, C0.shape[0], variant=variant)
            got = to_host(dC, C0.shape[0], n)
            bound = gemm_bound(k, alpha, A[:ar], B[:br], beta, C0[:m] if beta else np.zeros((m, n)))
            case = (seed, ta, tb, m, n, k, alpha, beta, variant, A.shape[0], B.shape[0], C0.shape[0])
            assert fro(got[:m] - want[:m]) <= bound, case
            assert bits_equal(got[m:], C0[m:]), case
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("seed", range(4))
def test_random_dsyrk(handle, orc, seed):
    rng = np.random.default_rng(2000 + seed)
    orc.cblas_on()
    try:
        for _ in range(8):
            n, _, k = dims(rng)
            uplo, trans = rng.choice([UP, LO]), rng.choice([N, T])
            ar, ac = (k, n) if trans == T else (n, k)
            A = padded(rng, ar, ac, ar + int(rng.integers(0, 4)))
            C0 = padded(rng, n, n, n + int(rng.integers(0, 4)))
            alpha = float(rng.choice([1.0, -1.0, 0.5]))
            beta = float(rng.choice([0.0, 1.0, -0.5]))
            variant = int(rng.integers(0, 5))
            want = np.nan_to_num(C0).copy(order="F") if beta == 0.0 else C0.copy(order="F")
            orc.dsyrk(uplo, trans, n, k, alpha, A, beta, want)
            dC = to_dev(C0)
            handle.dsyrk(uplo, trans, n, k, alpha, to_dev(A), A.shape[0], beta, dC, C0.shape[0],
                         variant=variant)
            got = to_host(dC, C0.shape[0], n)
            tri = np.tril if uplo == LO else np.triu
            bound = 16 * k * EPS * (abs(alpha) * fro(A[:ar]) ** 2 + abs(beta) * fro(C0[:n]))
            case = (seed, uplo, trans, n, k, alpha, beta, variant)
            assert fro(tri(got[:n]) - tri(want[:n])) <= bound, case
            other = (lambda x: np.triu(x, 1)) if uplo == LO else (lambda x: np.tril(x, -1))
            assert bits_equal(other(got[:n]), other(C0[:n])), case
            assert bits_equal(got[n:], C0[n:]), case
    finally:
        orc.cblas_off()


@pytest.mark.parametrize("seed", range(4))
def test_random_dtrsm(handle, seed):
    rng = np.random.default_rng(3000 + seed)
    for _ in range(8):
        m, n, _ = dims(rng)
        m, n = min(m, 1400), min(n, 1400)
        side, uplo = int(rng.choice([141, 142])), int(rng.choice([UP, LO]))
        trans, diag = int(rng.choice([N, T])), int(rng.choice([131, 132]))
        na = m if side == 141 else n
        Tm = rng.uniform(-1, 1, (na, na)) / na
        Tm = np.tril(Tm) if uplo == LO else np.triu(Tm)
        Tm[np.diag_indices(na)] = 1.0 if diag == 132 else 1.0 + rng.uniform(0, 1, na)
        lda = na + int(rng.integers(0, 4))
        stored = np.full((lda, na), np.nan, order="F")
        stored[:na] = Tm
        mask = np.triu(np.ones((na, na), bool), 1) if uplo == LO else np.tril(np.ones((na, na), bool), -1)
        stored[:na][mask] = np.nan
        if diag == 132:
            stored[:na][np.diag_indices(na)] = np.nan
        B0 = padded(rng, m, n, m + int(rng.integers(0, 4)))
        alpha = float(rng.choice([1.0, -0.5, 2.0]))
        dB = to_dev(B0)
        handle.dtrsm(side, uplo, trans, diag, m, n, alpha, to_dev(stored), lda, dB, B0.shape[0])
        got = to_host(dB, B0.shape[0], n)
        X = got[:m]
        case = (seed, side, uplo, trans, diag, m, n, alpha, lda, B0.shape[0])
        assert np.isfinite(X).all(), case
        opT = Tm.T if trans == T else Tm
        resid = (opT @ X - alpha * B0[:m]) if side == 141 else (X @ opT - alpha * B0[:m])
        assert fro(resid) <= 16 * na * EPS * fro(opT) * fro(X), case
        assert bits_equal(got[m:], B0[m:]), case


@pytest.mark.parametrize("seed", range(3))
def test_random_trsm_many_right_hand_sides(handle, seed):
    """Random solves in both precisions whose right-hand sides reach past 16 per CU (the
    32-wide panel workgroups) as well as the counts around it, with every panel option and tile
    shape, odd leading dimensions, the other triangle and a unit diagonal poisoned with NaN;
    checked on the device by the backward residual, the padding rows of B by their NaNs."""
    import torch
    from rtatblas_amd import native
    gen = np.random.default_rng(7000 + seed)
    for it in range(24):
        dt = [torch.float64, torch.float32][int(gen.integers(0, 2))]
        side, uplo = int(gen.choice([141, 142])), int(gen.choice([UP, LO]))
        trans, diag = int(gen.choice([N, T])), int(gen.choice([131, 132]))
        na = int(gen.choice([1, 17, 128, 129, 300, 513, 700, 1024, 1025, 1500, 2049]))
        nrhs = int(gen.choice([1, 16, 33, 1000, 2049, 4095, 4097, 4200, 5000, 8193]))
        m, n = (na, nrhs) if side == 141 else (nrhs, na)
        lda, ldb = na + int(gen.choice([0, 1, 3])), m + int(gen.choice([0, 1, 5]))
        variant = native.kernel_options(int(gen.integers(0, 5)), 0, int(gen.integers(0, 3)))
        alpha = float(gen.choice([1.0, -0.5, 2.0]))
        g = torch.Generator(device="cuda")
        g.manual_seed(100 * seed + it)
        # a[j, i] = element (i, j): column-major storage with leading dimension lda
        a = (torch.rand(na, lda, generator=g, device="cuda", dtype=torch.float64) * 2 - 1) / na
        idx = torch.arange(na, device="cuda")
        a[idx, idx] = 1.0 + torch.rand(na, generator=g, device="cuda", dtype=torch.float64)
        full = a[:, :na].t().contiguous()
        tri = torch.tril(full) if uplo == LO else torch.triu(full)
        if diag == 132:
            tri[idx, idx] = 1.0
        op = tri.t() if trans == T else tri
        ones = torch.ones(na, na, dtype=torch.bool, device="cuda")
        stored = full.clone()
        stored[torch.triu(ones, 1) if uplo == LO else torch.tril(ones, -1)] = float("nan")
        if diag == 132:
            stored[idx, idx] = float("nan")
        dev_a = torch.full((na, lda), float("nan"), device="cuda", dtype=torch.float64)
        dev_a[:, :na] = stored.t()
        b0 = torch.rand(n, ldb, generator=g, device="cuda", dtype=torch.float64) * 2 - 1
        b0[:, m:] = float("nan")
        dev_a, dev_b = dev_a.to(dt).clone(), b0.to(dt).clone()
        call = handle.dtrsm if dt == torch.float64 else handle.strsm
        call(side, uplo, trans, diag, m, n, alpha, dev_a, lda, dev_b, ldb, variant=variant)
        torch.cuda.synchronize()
        x, b = dev_b[:, :m].t().double(), b0[:, :m].t().to(dt).double()
        case = (seed, it, str(dt), side, uplo, trans, diag, m, n, lda, ldb, variant, alpha)
        assert bool(torch.isfinite(x).all()), case
        resid = (op.to(dt).double() @ x - alpha * b) if side == 141 else (x @ op.to(dt).double() - alpha * b)
        eps = EPS if dt == torch.float64 else float(np.finfo(np.float32).eps)
        assert float(resid.norm()) <= 16 * na * eps * float(op.norm()) * float(x.norm()), case
        assert ldb == m or bool(torch.isnan(dev_b[:, m:]).all()), case


@pytest.mark.parametrize("seed", range(3))
def test_random_geam_bit_exact(handle, seed):
    """copy / pad / transpose / scale / accumulate / zero fill in double and single precision:
    random shapes (small, mid-size, past the streaming thresholds, very tall and very flat),
    leading dimensions, base offsets into the buffers (columns that split cache lines), all
    four op combinations, in place or not.  Scalars with exact products, so the result has one
    rounding and must match torch's bit for bit, the elements around C included."""
    import torch
    rng = np.random.default_rng(3000 + seed)

    def view(buf, off, ld, rows, cols):        # [col][row] view of a column-major rows x cols
        return buf[off:off + ld * cols].view(cols, ld)[:, :rows]

    for _ in range(150):
        kind = rng.integers(0, 10)
        if kind < 5:
            m, n = int(rng.integers(1, 700)), int(rng.integers(1, 700))
        elif kind < 8:
            m, n = int(rng.integers(700, 5000)), int(rng.integers(700, 5000))
        elif kind == 8:
            m, n = int(rng.integers(5000, 9000)), int(rng.integers(5000, 9000))
        else:
            m, n = (int(rng.integers(30000, 70000)), int(rng.integers(100, 700)))[::int(rng.choice([1, -1]))]
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        alpha = float(rng.choice([0.0, 1.0, 1.0, -1.0, 0.5, 2.0]))
        beta = float(rng.choice([0.0, 0.0, 1.0, 0.5, -2.0]))
        pads = [int(rng.choice([0, 0, 1, 2, 3, 8, 16, 32, 37])) for _ in range(3)]
        offs = [int(rng.choice([0, 0, 0, 1, 2, 5, 16])) for _ in range(3)]
        ar, ac = (n, m) if ta else (m, n)
        br, bc = (n, m) if tb else (m, n)
        lda, ldb, ldc = ar + pads[0], br + pads[1], m + pads[2]
        inplace = (not tb) and beta != 0.0 and rng.integers(0, 2) == 1
        if inplace:
            ldb, offs[1] = ldc, offs[2]
        dt = torch.float64 if rng.integers(0, 4) else torch.float32
        A = torch.empty(offs[0] + lda * ac + 4, dtype=dt, device="cuda").uniform_(-1, 1)
        C0 = torch.empty(offs[2] + ldc * n + 20, dtype=dt, device="cuda").uniform_(-1, 1)
        B = C0 if inplace else torch.empty(offs[1] + ldb * bc + 4, dtype=dt, device="cuda").uniform_(-1, 1)
        Cb = C0.clone()
        Bb = Cb if inplace else B
        Av, Bv = view(A, offs[0], lda, ar, ac), view(B, offs[1], ldb, br, bc).clone()
        opA, opB = (Av.t() if ta else Av), (Bv.t() if tb else Bv)
        want = C0.clone()
        Wv = view(want, offs[2], ldc, m, n)
        if alpha != 0 and beta != 0:
            Wv[:] = alpha * opA + beta * opB
        elif alpha != 0:
            Wv[:] = alpha * opA
        elif beta != 0:
            Wv[:] = beta * opB
        else:
            Wv[:] = 0
        call = handle.dgeam if dt == torch.float64 else handle.sgeam
        call(T if ta else N, T if tb else N, m, n, alpha, A[offs[0]:], lda, beta, Bb[offs[1]:], ldb,
             Cb[offs[2]:], ldc)
        bits = torch.int64 if dt == torch.float64 else torch.int32
        case = (seed, m, n, ta, tb, alpha, beta, lda, ldb, ldc, offs, inplace, str(dt))
        assert torch.equal(Cb.view(bits), want.view(bits)), case
