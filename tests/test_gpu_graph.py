"""The entry points only enqueue kernels on the handle's stream (no allocation once a workspace
is lent, no synchronisation, no memset nodes), so a sequence of calls can be captured in a HIP
graph and replayed.  Every replay is checked bit for bit against the same calls run eagerly on
the same inputs, with eager work and synchronisations between the replays."""
import numpy as np
import pytest

from util import bits_equal, to_dev, to_host

pytestmark = pytest.mark.gpu
N, T = 111, 112


def test_captured_sequence_replays_bit_exactly(handle):
    import torch
    rng = np.random.default_rng(3)
    m, n, k = 300, 260, 700
    A = np.asfortranarray(rng.uniform(-1, 1, (k, m)))
    B = np.asfortranarray(rng.uniform(-1, 1, (k, n)))
    L = np.asfortranarray(np.tril(rng.uniform(-1, 1, (m, m)) / m) + 2 * np.eye(m))
    dA, dB, dL = to_dev(A), to_dev(B), to_dev(L)
    dC = torch.zeros(m * n, dtype=torch.float64, device="cuda")
    dS = torch.zeros(m * m, dtype=torch.float64, device="cuda")
    dT = torch.zeros(n * m, dtype=torch.float64, device="cuda")
    ws = torch.empty(1 << 20, dtype=torch.float64, device="cuda")

    def sequence():
        handle.dgemm(T, N, m, n, k, 1.0, dA, k, dB, k, 0.0, dC, m)            # C = A^T B
        handle.dsyrk(122, T, m, k, 1.0, dA, k, 0.0, dS, m)                    # S = A^T A (lower)
        handle.dtrsm(141, 122, N, 131, m, n, 1.0, dL, m, dC, m)               # C = L^-1 C
        handle.dgeam(T, N, n, m, 1.0, dC, m, 0.0, dT, n, dT, n)               # T = C^T

    handle.set_workspace(ws, ws.numel() * 8)
    cap = torch.cuda.Stream()
    try:
        handle.set_stream(cap)
        with torch.cuda.stream(cap):
            sequence()                                # first launches outside the capture
        cap.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cap):
            sequence()
        for rep in range(3):
            # new inputs, eager result first
            dA.copy_(torch.from_numpy(np.ascontiguousarray(
                rng.uniform(-1, 1, k * m))).cuda())
            torch.cuda.synchronize()
            with torch.cuda.stream(cap):
                sequence()
            cap.synchronize()
            want_t, want_s = to_host(dT, n, m).copy(), to_host(dS, m, m).copy()
            dT.zero_()
            dS.zero_()
            dC.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert bits_equal(to_host(dT, n, m), want_t), rep
            assert bits_equal(np.tril(to_host(dS, m, m)), np.tril(want_s)), rep
    finally:
        handle.set_stream(torch.cuda.current_stream())
        handle.set_workspace(None, 0)


def test_first_calls_inside_a_capture_allocate_nothing():
    """A fresh handle owns no scratch yet.  Inside a capture it must not allocate any: TRSM
    reports the missing scratch and leaves the capture usable; a GEMM whose tail would be
    split runs unsplit, and the captured graph replays to the right answer."""
    import torch
    from rtatblas_amd import native
    from util import fro, gemm_bound
    rng = np.random.default_rng(9)
    # 3 x 3 tiles of 128 x 128 with a long K: the auto heuristic would cut tails along K
    m, n, k = 384, 384, 4608
    A = np.asfortranarray(rng.uniform(-1, 1, (m, k)))
    B = np.asfortranarray(rng.uniform(-1, 1, (k, n)))
    L = np.asfortranarray(np.tril(rng.uniform(-1, 1, (m, m)) / m) + 2 * np.eye(m))
    dA, dB, dL = to_dev(A), to_dev(B), to_dev(L)
    dC = torch.zeros(m * n, dtype=torch.float64, device="cuda")
    h = native.Handle()
    cap = torch.cuda.Stream()
    try:
        h.set_stream(cap)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cap):
            st = h.dtrsm(141, 122, N, 131, m, n, 1.0, dL, m, dC, m, check=False)
            h.dgemm(N, N, m, n, k, 1.0, dA, m, dB, k, 0.0, dC, m)
        assert native.STATUS_NAMES[st] == "ALLOC_FAILED"
        for _ in range(2):
            dC.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = to_host(dC, m, n)
            assert fro(got - A @ B) <= gemm_bound(k, 1.0, A, B, 0.0, got)
        # outside the capture the same handle allocates as usual
        with torch.cuda.stream(cap):
            h.dtrsm(141, 122, N, 131, m, n, 1.0, dL, m, dC, m)
        cap.synchronize()
        X = to_host(dC, m, n)
        assert fro(L @ X - got) <= 16 * m * np.finfo(np.float64).eps * fro(L) * fro(X)
    finally:
        torch.cuda.synchronize()
        h.close()


def test_graph_captured_before_the_scratch_grew_still_replays():
    """A TRSM recorded into a graph names the handle's scratch block of that moment.  A later,
    larger TRSM on the same handle makes the handle allocate a bigger block; the old one must
    stay alive, or every replay of the graph would read and write freed memory."""
    import torch
    from rtatblas_amd import native
    rng = np.random.default_rng(17)
    m, n, big = 640, 200, 3000
    L = np.asfortranarray(np.tril(rng.uniform(-1, 1, (m, m)) / m) + 2 * np.eye(m))
    Lb = np.asfortranarray(np.tril(rng.uniform(-1, 1, (big, big)) / big) + 2 * np.eye(big))
    B0 = np.asfortranarray(rng.uniform(-1, 1, (m, n)))
    dL, dLb, dB = to_dev(L), to_dev(Lb), to_dev(B0)
    dX = torch.zeros(m * n, dtype=torch.float64, device="cuda")
    dXb = torch.ones(big * 64, dtype=torch.float64, device="cuda")
    h = native.Handle()
    cap = torch.cuda.Stream()
    try:
        h.set_stream(cap)
        with torch.cuda.stream(cap):
            dX.copy_(dB)
            h.dtrsm(141, 122, N, 131, m, n, 1.0, dL, m, dX, m)      # allocates the first block
        cap.synchronize()
        want = to_host(dX, m, n).copy()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cap):
            dX.copy_(dB)
            h.dtrsm(141, 122, N, 131, m, n, 1.0, dL, m, dX, m)
        with torch.cuda.stream(cap):
            h.dtrsm(141, 122, N, 131, big, 64, 1.0, dLb, big, dXb, big)  # outgrows the block
        cap.synchronize()
        # fresh allocations of the old block's size would land on it, had it been freed
        spoil = [torch.full((1 << 20,), float("nan"), dtype=torch.float64, device="cuda")
                 for _ in range(8)]
        for rep in range(3):
            dX.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert bits_equal(to_host(dX, m, n), want), rep
        del spoil
    finally:
        torch.cuda.synchronize()
        h.close()


def test_first_compute_call_of_a_fresh_handle_allocates_nothing():
    """The GEMM tail scratch comes with the handle (rtat_create), so no compute call has to
    allocate it inside a caller's event pair: device memory in use does not move across the
    first DGEMM of a new handle, on a shape whose tail tiles are cut along K, and the call did
    cut them."""
    import torch
    from rtatblas_amd import native
    m = n = k = 3072
    dA = torch.rand(m * k, dtype=torch.float64, device="cuda")
    dB = torch.rand(k * n, dtype=torch.float64, device="cuda")
    dC = torch.zeros(m * n, dtype=torch.float64, device="cuda")
    st = torch.cuda.current_stream()
    torch.cuda.synchronize()
    before_create = torch.cuda.mem_get_info()[0]
    h = native.Handle()
    h.set_stream(st)
    torch.cuda.synchronize()
    with_handle = torch.cuda.mem_get_info()[0]
    assert before_create - with_handle >= 64 << 20        # the scratch is there already
    for _ in range(3):
        h.dgemm(N, N, m, n, k, 1.0, dA, m, dB, k, 0.0, dC, m)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == with_handle
    info = h.last_launch()
    assert info["split_tiles"] > 0 and info["split_slices"] >= 2, info
    h.close()


def test_destroy_during_capture_is_refused_and_leaves_the_capture_valid():
    """rtat_destroy frees device memory, which a stream that records into a graph must not see:
    it returns NOT_SUPPORTED, frees nothing, and the capture and the handle stay usable."""
    import torch
    from rtatblas_amd import native
    n = 256
    dA = torch.rand(n * n, dtype=torch.float64, device="cuda")
    dC = torch.zeros(n * n, dtype=torch.float64, device="cuda")
    cap = torch.cuda.Stream()
    h = native.Handle()
    h.set_stream(cap)
    with torch.cuda.stream(cap):
        h.dgemm(N, N, n, n, n, 1.0, dA, n, dA, n, 0.0, dC, n)      # kernels loaded before capture
    cap.synchronize()
    want = dC.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=cap):
        h.dgemm(N, N, n, n, n, 1.0, dA, n, dA, n, 0.0, dC, n)
        assert native.STATUS_NAMES[h.lib.rtat_destroy(h.h)] == "NOT_SUPPORTED"
    dC.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(dC, want)
    h.close()                                                     # outside a capture: fine
