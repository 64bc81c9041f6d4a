"""GPU parity of rtat_dgeam / rtat_dfill (through the C ABI) against the CPU oracle.
Bar: bit-exact for copy / pad / transpose (alpha = 1, beta = 0), for scaling, and for
accumulates whose alpha is 1 (every accumulate the matrix-op tree builds)."""
import itertools

import numpy as np
import pytest

from util import bits_equal, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112


def rnd(rng, m, n, ld=None):
    ld = max(m, 1) if ld is None else ld
    a = np.full((ld, n), np.nan, order="F")
    a[:m] = rng.uniform(-1, 1, (m, n))
    return a


SHAPES = [(10, 12), (64, 64), (65, 3), (1, 70), (33, 129), (257, 100), (512, 8), (1000, 77),
          (70, 45)]


@pytest.mark.parametrize("m,n", SHAPES)
@pytest.mark.parametrize("pad,extra", [(1, 0), (8, 3), (32, 1), (32, 2)])
def test_move_copy_and_transpose_bit_exact(handle, orc, m, n, pad, extra):
    rng = np.random.default_rng(m * 131 + n + pad)
    A = rnd(rng, m, n, m + extra)
    A[0, 0] = -0.0
    dA = to_dev(A)
    for trans in (False, True):
        om, on = (n, m) if trans else (m, n)
        ld = (om + pad - 1) // pad * pad
        want = np.full((ld, on), np.nan, order="F")
        orc.dgeam(T if trans else N, N, om, on, 1.0, A, 0.0, want, want)
        out = to_dev(np.full((ld, on), np.nan, order="F"))
        handle.dgeam(T if trans else N, N, om, on, 1.0, dA, A.shape[0], 0.0, out, ld, out, ld)
        got = to_host(out, ld, on)
        assert bits_equal(got, want), (m, n, pad, trans)   # NaN padding rows included


@pytest.mark.parametrize("m,n,extra", [(4096, 9, 0), (4099, 37, 1), (6001, 20, 2), (2500, 33, 1),
                                       (12288, 5, 0), (12290, 3, 0)])
def test_tall_columns_copy_scale_fill_bit_exact(handle, orc, m, n, extra):
    """Columns of 2048 .. 12288 elements: the non-transposed kernel walks one long stretch of a
    column per pass (16-byte and, with an odd leading dimension, 8-byte accesses), ragged at
    the end; longer columns take the other shape.  Copy, scale, zero fill and, for
    contrast, the accumulate."""
    rng = np.random.default_rng(m + n)
    A = rnd(rng, m, n, m + extra)
    B0 = rnd(rng, m, n, m + 32)
    for alpha, beta in [(1.0, 0.0), (-2.5, 0.0), (0.0, 0.0), (1.0, 0.5)]:
        want = B0.copy(order="F")
        orc.dgeam(N, N, m, n, alpha, A, beta, want, want)
        dB = to_dev(B0)
        handle.dgeam(N, N, m, n, alpha, to_dev(A), A.shape[0], beta, dB, B0.shape[0], dB,
                     B0.shape[0])
        assert bits_equal(to_host(dB, B0.shape[0], n), want), (m, n, alpha, beta)
    # single precision: twice the elements per 16-byte vector, tall from 8192 rows
    Af = np.full((8300 + extra, 4), np.nan, dtype=np.float32, order="F")
    Af[:8300] = rng.uniform(-1, 1, (8300, 4)).astype(np.float32)
    outf = to_dev(np.full((8304, 4), np.nan, dtype=np.float32, order="F"))
    handle.sgeam(N, N, 8300, 4, 1.0, to_dev(Af), Af.shape[0], 0.0, outf, 8304, outf, 8304)
    gotf = to_host(outf, 8304, 4)
    assert np.array_equal(gotf[:8300].view(np.uint32), Af[:8300].view(np.uint32))
    assert np.isnan(gotf[8300:]).all()


@pytest.mark.parametrize("m,n", [(23, 17), (128, 64), (301, 259)])
@pytest.mark.parametrize("beta", [0.0, 0.5, 1.0, -2.0])
@pytest.mark.parametrize("trans", [False, True])
def test_accumulate_in_place_bit_exact(handle, orc, m, n, beta, trans):
    rng = np.random.default_rng(int(beta * 4) + m)
    S = rnd(rng, n, m, n + 1) if trans else rnd(rng, m, n, m + 2)
    C0 = rnd(rng, m, n, m + 3)
    want = C0.copy(order="F")
    orc.dgeam(T if trans else N, N, m, n, 1.0, S, beta, want, want)
    dS, dC = to_dev(S), to_dev(C0)
    handle.dgeam(T if trans else N, N, m, n, 1.0, dS, S.shape[0], beta, dC, C0.shape[0], dC,
                 C0.shape[0])
    assert bits_equal(to_host(dC, C0.shape[0], n), want)


@pytest.mark.parametrize("ta,tb", list(itertools.product([N, T], [N, T])))
def test_all_four_op_combinations(handle, orc, ta, tb):
    m, n = 45, 70
    rng = np.random.default_rng(ta * 7 + tb)
    A = rnd(rng, n, m) if ta == T else rnd(rng, m, n)
    B = rnd(rng, n, m) if tb == T else rnd(rng, m, n)
    want = np.full((m + 1, n), np.nan, order="F")
    orc.dgeam(ta, tb, m, n, 1.0, A, 0.5, B, want)
    out = to_dev(np.full((m + 1, n), np.nan, order="F"))
    handle.dgeam(ta, tb, m, n, 1.0, to_dev(A), A.shape[0], 0.5, to_dev(B), B.shape[0], out, m + 1)
    assert bits_equal(to_host(out, m + 1, n), want)


def test_scale_zero_fill_and_single_operand_forms(handle, orc):
    m, n = 72, 31
    rng = np.random.default_rng(5)
    A = rnd(rng, m, n)
    dA = to_dev(A)
    out = to_dev(np.full((m, n), np.nan, order="F"))
    handle.dgeam(N, N, m, n, -2.0, dA, m, 0.0, out, m, out, m)          # test-only alpha (-2)
    assert bits_equal(to_host(out, m, n), np.asfortranarray(-2.0 * A))
    nan = to_dev(np.full((m, n), np.nan, order="F"))
    handle.dgeam(N, N, m, n, 0.0, nan, m, 0.0, nan, m, nan, m)          # zero fill of NaN scratch
    assert (to_host(nan, m, n) == 0).all()
    out2 = to_dev(np.full((n, m), np.nan, order="F"))
    handle.dgeam(N, T, n, m, 0.0, None, n, 1.0, dA, m, out2, n)         # beta-only, transposed
    assert bits_equal(to_host(out2, n, m), np.asfortranarray(A.T))


def test_argument_errors_and_quick_returns(handle):
    import torch
    x = torch.zeros(64, dtype=torch.float64, device="cuda")
    assert handle.dgeam(N, N, 0, 5, 1.0, x, 1, 0.0, x, 1, x, 1, check=False) == 0
    assert handle.dgeam(N, N, 8, 8, 1.0, x, 4, 0.0, x, 8, x, 8, check=False) == 3   # lda < m
    assert handle.dgeam(N, N, 8, 8, 1.0, x, 8, 0.0, x, 8, x, 4, check=False) == 3   # ldc < m
    assert handle.dgeam(5, N, 8, 8, 1.0, x, 8, 0.0, x, 8, x, 8, check=False) == 10  # bad enum
    assert handle.dgeam(T, N, 8, 8, 1.0, x, 8, 0.0, x, 8, x, 8, check=False) == 3   # in-place T


@pytest.mark.parametrize("kind", [0, 1, 2, 3, 4])
def test_fill_matches_host_generator(handle, orc, kind):
    import torch
    m = n = 130
    ld = m + 5
    d = torch.zeros(ld * n, dtype=torch.float64, device="cuda")
    handle.dfill(d, m, n, ld, 42, kind)
    assert bits_equal(to_host(d, ld, n), orc.fill(m, n, ld, seed=42, kind=kind))


def test_large_transpose_round_trip(handle):
    """Full-size property check (8192 x 8192, ld = rows): transposing twice is the identity."""
    import torch
    n = 8192
    a = torch.empty(n * n, dtype=torch.float64, device="cuda")
    handle.dfill(a, n, n, n, 7, 0)
    t = torch.empty_like(a)
    b = torch.empty_like(a)
    handle.dgeam(T, N, n, n, 1.0, a, n, 0.0, t, n, t, n)
    handle.dgeam(T, N, n, n, 1.0, t, n, 0.0, b, n, b, n)
    assert torch.equal(a.view(torch.int64), b.view(torch.int64))
    assert torch.equal(t.view(n, n).view(torch.int64), a.view(n, n).t().contiguous().view(torch.int64))


def test_full_size_streaming_paths_bit_exact(handle):
    """8192^2 doubles: past 512 MiB of traffic the kernels switch to non-temporal accesses.
    Transpose, pad copy, transpose-accumulate and fill against torch on the device."""
    import torch
    n, ldp = 8192, 8192 + 32
    S = torch.empty(n * n, dtype=torch.float64, device="cuda")
    handle.dfill(S, n, n, n, 5)
    Sm = S.view(n, n)                                   # [col][row] of the column-major matrix

    D = torch.full((n * n,), float("nan"), dtype=torch.float64, device="cuda")
    handle.dgeam(T, N, n, n, 1.0, S, n, 0.0, D, n, D, n)                  # D = S^T
    assert torch.equal(D.view(n, n).view(torch.int64), Sm.t().contiguous().view(torch.int64))

    P = torch.full((n * ldp,), float("nan"), dtype=torch.float64, device="cuda")
    handle.dgeam(N, N, n, n, 1.0, S, n, 0.0, P, ldp, P, ldp)              # pad copy
    Pm = P.view(n, ldp)
    assert torch.equal(Pm[:, :n].contiguous().view(torch.int64), Sm.view(torch.int64))
    assert bool(torch.isnan(Pm[:, n:]).all())                             # padding rows untouched

    C0 = torch.empty(n * n, dtype=torch.float64, device="cuda")
    handle.dfill(C0, n, n, n, 6)
    C = C0.clone()
    handle.dgeam(T, N, n, n, 1.0, S, n, 0.5, C, n, C, n)                  # C = S^T + 0.5 C
    want = Sm.t() + 0.5 * C0.view(n, n)                                   # 0.5 * c is exact
    assert torch.equal(C.view(n, n).view(torch.int64), want.contiguous().view(torch.int64))

    handle.dgeam(N, N, n, n, 0.0, S, n, 0.0, P, ldp, P, ldp)              # zero fill of the logical part
    assert bool((Pm[:, :n] == 0).all()) and bool(torch.isnan(Pm[:, n:]).all())


@pytest.mark.parametrize("m,n,extra_a,extra_c,offset", [(2500, 300, 0, 1, 0), (4099, 513, 3, 0, 0),
                                                        (1100, 1000, 1, 3, 0), (1024, 256, 0, 0, 5),
                                                        (2048, 96, 2, 16, 8), (30, 5000, 0, 0, 0),
                                                        (100, 3000, 3, 3, 0), (300, 2501, 1, 1, 0),
                                                        (256, 4000, 3, 3, 0), (640, 999, 0, 3, 2)])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_transpose_into_columns_that_split_cache_lines(handle, m, n, extra_a, extra_c, offset, beta):
    """C's columns start inside 128-byte lines (odd ldc, or a base offset into the buffer): the
    tile rows are dealt to the XCDs in contiguous eighths, or, for a C of few tile rows (the
    last five shapes: 1 to 5 of them), the column tiles round-robin.  Bit-exact, rows ldc - m of
    every column and the elements around C untouched."""
    import torch
    lda, ldc = n + extra_a, m + extra_c
    g = torch.Generator(device="cuda").manual_seed(m + n)
    S = torch.rand(lda * m, dtype=torch.float64, device="cuda", generator=g)
    buf0 = torch.rand(offset + ldc * n + 16, dtype=torch.float64, device="cuda", generator=g)
    buf = buf0.clone()
    C = buf[offset:]
    handle.dgeam(T, N, m, n, 1.0, S, lda, beta, C, ldc, C, ldc)
    want = buf0.clone()
    Wm = want[offset:offset + ldc * n].view(n, ldc)
    At = S.view(m, lda)[:, :n].t()
    Wm[:, :m] = At + beta * Wm[:, :m] if beta else At
    assert torch.equal(buf.view(torch.int64), want.view(torch.int64))


@pytest.mark.parametrize("m,n,lda,ldc,offset", [(6151, 10007, 10010, 6153, 0), (8192, 8192, 8192, 8195, 0),
                                                (8200, 8190, 8190, 8200, 3), (65539, 600, 603, 65539, 0),
                                                (4700, 4600, 4600, 4701, 0), (4608, 4608, 4608, 4608, 0)])
def test_full_size_transpose_into_columns_that_split_cache_lines_bit_exact(handle, m, n, lda, ldc, offset):
    """The streaming (non-temporal) kernels with the tile rows dealt to the XCDs in contiguous
    eighths: odd ldc, a base offset, ragged edges, a very tall C; the last two shapes stream as
    transposes (past 288 MiB of traffic) but not as accumulates (512 MiB), the last one into
    aligned columns.  Transpose and transpose-accumulate against torch on the device, padding
    rows and surroundings included."""
    import torch
    S = torch.empty(lda * m, dtype=torch.float64, device="cuda")
    handle.dfill(S, n, m, lda, 11)
    S.nan_to_num_(nan=-3.0)                             # rows n .. lda of A are never read anyway
    At = S.view(m, lda)[:, :n].t()
    buf0 = torch.empty(offset + ldc * n + 16, dtype=torch.float64, device="cuda")
    buf0.uniform_(-1, 1)
    for beta in (0.0, 0.5):
        buf = buf0.clone()
        C = buf[offset:]
        handle.dgeam(T, N, m, n, 1.0, S, lda, beta, C, ldc, C, ldc)
        want = buf0.clone()
        Wm = want[offset:offset + ldc * n].view(n, ldc)
        Wm[:, :m] = At + beta * Wm[:, :m] if beta else At
        assert torch.equal(buf.view(torch.int64), want.view(torch.int64)), beta
        del buf, want


@pytest.mark.parametrize("m,n,lda,ldc,offset,single", [
    (10, 2500000, 2500000, 11, 0, False),      # fewer rows than a line holds, more tile columns than grid.y
    (3000000, 8, 8, 3000001, 1, False),        # one tile column, 23438 shifted tile rows
    (12000, 9000, 9003, 12001, 5, True),       # floats: 32 elements per line
    (5000, 5000, 5000, 5001, 0, False),        # every column shifted by one more element
    (129, 160000, 160000, 144, 7, False),      # ldc a multiple of the line, base off a line
])
def test_streaming_transpose_with_row_tiles_shifted_onto_lines_bit_exact(handle, m, n, lda, ldc,
                                                                         offset, single):
    """Large traffic into a C whose columns start inside 128-byte lines: the row tiles are
    shifted, column by column, onto C's lines.  Transpose and in-place transpose-accumulate
    against torch on the device; padding rows and the elements around C must keep their bits."""
    import torch
    dt = torch.float32 if single else torch.float64
    it = torch.int32 if single else torch.int64
    geam = handle.sgeam if single else handle.dgeam
    g = torch.Generator(device="cuda").manual_seed(m + n)
    S = torch.rand(lda * m, dtype=dt, device="cuda", generator=g)
    At = S.view(m, lda)[:, :n].t()
    buf0 = torch.rand(offset + ldc * n + 40, dtype=dt, device="cuda", generator=g)
    for beta in (0.0, 0.5):
        buf = buf0.clone()
        C = buf[offset:]
        geam(T, N, m, n, 1.0, S, lda, beta, C, ldc, C, ldc)
        want = buf0.clone()
        Wm = want[offset:offset + ldc * n].view(n, ldc)
        Wm[:, :m] = At + beta * Wm[:, :m] if beta else At
        assert torch.equal(buf.view(it), want.view(it)), beta
        del buf, want


@pytest.mark.parametrize("m,n,ld", [(1000, 37, 1024), (512, 700, 512), (2999, 64, 3072), (1, 5, 512),
                                    (8192, 300, 8192)])
@pytest.mark.parametrize("single", [False, True])
def test_zero_fill_of_page_aligned_columns(handle, m, n, ld, single):
    """Columns that start on 4 KiB boundaries are zeroed by the one-store-per-lane kernel:
    the logical m x n becomes zero, rows m .. ld of every column and the elements behind the
    last column keep their NaN."""
    import torch
    dt = torch.float32 if single else torch.float64
    esz = 4 if single else 8
    ld = ld * (2 if single else 1)                      # keeps ld * element size a multiple of 4096
    raw = torch.full((ld * n + 4096,), float("nan"), dtype=dt, device="cuda")
    skip = (-raw.data_ptr() % 4096) // esz              # first element on a 4 KiB boundary
    C = raw[skip:]
    assert C.data_ptr() % 4096 == 0
    (handle.sgeam if single else handle.dgeam)(N, N, m, n, 0.0, C, ld, 0.0, C, ld, C, ld)
    body = C[:ld * n].view(n, ld)
    assert bool((body[:, :m] == 0).all())
    assert bool(torch.isnan(body[:, m:]).all())
    assert bool(torch.isnan(raw[:skip]).all()) and bool(torch.isnan(C[ld * n:]).all())


@pytest.mark.parametrize("first,second", [
    ((N, 1000, 77, 3, 32), (T, 257, 100, 1, 8)),          # pad copy + transpose, odd source ld
    ((T, 513, 300, 0, 1), (T, 64, 64, 2, 32)),            # two transposes
    ((N, 4099, 37, 1, 1), (N, 4096, 64, 0, 32)),          # element-wise and 16-byte copies
    ((N, 0, 5, 0, 1), (T, 70, 45, 0, 1)),                 # an empty job
    ((N, 10007, 700, 3, 32), (N, 6151, 500, 3, 32)),      # slices of the awkward DGEMM's operands
])
@pytest.mark.parametrize("single", [False, True])
def test_two_moves_in_one_launch_bit_exact(handle, first, second, single):
    """rtat_dmove_pair / rtat_smove_pair against the same two moves through rtat_dgeam /
    rtat_sgeam: copies, pad copies and transposes, bit for bit, padding rows untouched."""
    import torch
    dt = torch.float32 if single else torch.float64
    it = torch.int32 if single else torch.int64
    geam = handle.sgeam if single else handle.dgeam
    g = torch.Generator(device="cuda").manual_seed(11)
    jobs, want = [], []
    for (op, m, n, extra, pad) in (first, second):
        ar, ac = (n, m) if op == T else (m, n)
        lda = max(ar + extra, 1)
        ldc = max((m + pad - 1) // pad * pad, 1)
        S = torch.rand(lda * ac + 1, dtype=dt, device="cuda", generator=g)
        D0 = torch.rand(ldc * n + 1, dtype=dt, device="cuda", generator=g)
        one, two = D0.clone(), D0.clone()
        if m and n:
            geam(op, N, m, n, 1.0, S, lda, 0.0, one, ldc, one, ldc)
        jobs.append((op, m, n, S, lda, two, ldc))
        want.append(one)
    handle.move_pair(jobs[0], jobs[1], single=single)
    for job, ref in zip(jobs, want):
        assert torch.equal(job[5].view(it), ref.view(it))


def test_two_moves_argument_errors(handle):
    import torch
    x = torch.zeros(64, dtype=torch.float64, device="cuda")
    y = torch.zeros(64, dtype=torch.float64, device="cuda")
    ok = (N, 8, 8, x, 8, y, 8)
    assert handle.move_pair(ok, (N, 8, 8, x, 4, y, 8), check=False) == 3      # lda < m
    assert handle.move_pair((T, 8, 4, x, 3, y, 8), ok, check=False) == 3      # lda < n for a transpose
    assert handle.move_pair(ok, (5, 8, 8, x, 8, y, 8), check=False) == 10     # bad enum
    assert handle.move_pair((N, 8, 8, x, 8, x, 8), ok, check=False) == 3      # in place
    assert handle.move_pair((N, 0, 0, None, 1, None, 1), (N, 0, 3, None, 1, None, 1), check=False) == 0


@pytest.mark.parametrize("both", [False, True])
def test_transpose_from_a_leading_dimension_past_32_bit_tile_offsets(handle, both):
    """A leading dimension of 67.2 million doubles: eight columns of the source span more than
    4 GiB, so the transposing kernels switch to 64-bit lane offsets.  C = A^T (+ 0.5 B^T when
    both operands are transposed), bit-exact."""
    import torch
    m, n, lda = 3, 1000, 67_200_000
    S = torch.empty(lda * (m - 1) + n, dtype=torch.float64, device="cuda")
    Sv = S.as_strided((m, n), (lda, 1))                  # [column of A][row of A]
    g = torch.Generator(device="cuda").manual_seed(3)
    Sv.copy_(torch.rand(m, n, dtype=torch.float64, device="cuda", generator=g))
    D = torch.full((n * (m + 2),), float("nan"), dtype=torch.float64, device="cuda")
    if both:
        handle.dgeam(T, T, m, n, 1.0, S, lda, 0.5, S, lda, D, m + 2)
        want = Sv + 0.5 * Sv
    else:
        handle.dgeam(T, N, m, n, 1.0, S, lda, 0.0, D, m + 2, D, m + 2)
        want = Sv
    got = D.view(n, m + 2)
    assert torch.equal(got[:, :m].contiguous().view(torch.int64), want.t().contiguous().view(torch.int64))
    assert bool(torch.isnan(got[:, m:]).all())


def test_streaming_probes(handle):
    """rtat_hbm_probe: the copy copies, the write writes its pattern, the read leaves its sink
    alone; sizes must be whole 32 KiB grains and pointers 16-byte aligned."""
    import torch
    from rtatblas_amd import native
    nbytes = 3 << 20
    src = torch.rand(nbytes // 8, dtype=torch.float64, device="cuda")
    dst = torch.zeros(nbytes // 8, dtype=torch.float64, device="cuda")
    handle.hbm_probe(native.PROBE_COPY, src, dst, nbytes)
    assert torch.equal(src, dst)
    sink = torch.full((256,), 7.0, dtype=torch.float64, device="cuda")
    handle.hbm_probe(native.PROBE_READ, src, sink, nbytes)
    assert bool((sink == 7.0).all())
    handle.hbm_probe(native.PROBE_WRITE, None, dst, nbytes)
    assert bool((dst.view(-1, 2) == torch.tensor([1.0, 2.0], dtype=torch.float64, device="cuda")).all())
    assert handle.hbm_probe(native.PROBE_COPY, src, dst, nbytes - 8, check=False) == 3
    assert handle.hbm_probe(native.PROBE_COPY, src[1:], dst, 1 << 20, check=False) == 3
    assert handle.hbm_probe(9, src, dst, nbytes, check=False) == 10
    assert handle.hbm_probe(native.PROBE_COPY, src, dst, 0) == 0
