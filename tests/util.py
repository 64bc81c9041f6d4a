"""Helpers shared by the tests: host <-> device movement of column-major matrices and the
error measures the parity bars are written in."""
import numpy as np

EPS = np.finfo(np.float64).eps


def to_dev(a):
    """(ld, n) Fortran numpy array -> flat torch tensor on cuda:0 with the same memory order."""
    import torch
    flat = np.ascontiguousarray(a.reshape(-1, order="F"))
    return torch.from_numpy(flat).cuda()


def to_host(t, ld, n):
    """Flat device tensor -> (ld, n) Fortran numpy array."""
    return t.cpu().numpy().reshape((ld, n), order="F")


def fro(a):
    return float(np.linalg.norm(a))


def gemm_bound(k, alpha, A, B, beta, C0):
    """Normwise bar for C = alpha*A*B + beta*C0: 16*k*eps*(|alpha| |A|_F |B|_F + |beta| |C0|_F)."""
    c0 = 0.0 if beta == 0.0 else abs(beta) * fro(C0)
    return 16.0 * max(k, 1) * EPS * (abs(alpha) * fro(A) * fro(B) + c0)


def bits_equal(a, b):
    """True when two float arrays are identical bit for bit (NaN payloads and -0 included)."""
    return np.array_equal(a.view(np.uint64), b.view(np.uint64))


def reference_or_skip(native=False):
    """The reference's own sources compiled into oracle/_ref/ are the strongest parity evidence
    these tests have, and they exist only where the reference tree was mounted at build time.
    Without them the tests that drive them skip - unless the builds are known to be expected
    (RTAT_REQUIRE_REF=1, or the marker the build step leaves beside them): then a missing
    library is a failure, not a quiet loss of coverage."""
    import os
    import pytest
    from oracle import ref_py
    if ref_py.available() and (not native or ref_py.available(native=True)):
        return ref_py
    what = "oracle/_ref/librtat_ref.so%s not built" % (" / librtat_ref_native.so" if native else "")
    marker = os.path.join(os.path.dirname(ref_py.LIB_PATH), "REQUIRED")
    if os.environ.get("RTAT_REQUIRE_REF") == "1" or os.path.exists(marker):
        pytest.fail(what + " although the reference builds are required here")
    pytest.skip(what)
