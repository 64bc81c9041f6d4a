"""ctypes binding of oracle/librtat_oracle.so for numpy arrays.

TEST INFRASTRUCTURE: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg only.  Matrices are numpy float64 arrays in Fortran order whose first dimension is the
leading dimension (shape (ld, n)); the logical matrix is the top m rows.
"""
import ctypes as C
import glob
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "librtat_oracle.so")

OP_N, OP_T = 111, 112
UPPER, LOWER = 121, 122
NON_UNIT, UNIT = 131, 132
LEFT, RIGHT = 141, 142

_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "librtat_oracle.so"], check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        lib = C.CDLL(LIB_PATH)
        d, i, vp, pd = C.c_double, C.c_int, C.c_void_p, C.c_void_p
        lib.orc_dgemm.argtypes = [i, i, i, i, i, d, pd, i, pd, i, d, pd, i]
        lib.orc_dsyrk.argtypes = [i, i, i, i, d, pd, i, d, pd, i]
        lib.orc_dtrsm.argtypes = [i, i, i, i, i, i, d, pd, i, pd, i]
        lib.orc_dgeam.argtypes = [i, i, i, i, d, pd, i, d, pd, i, pd, i]
        lib.orc_dfill.argtypes = [pd, i, i, i, C.c_uint64, i]
        lib.orc_cblas_on.argtypes = [C.c_char_p]
        lib.orc_cblas_on.restype = i
        lib.orc_cblas_name.restype = C.c_char_p
        lib.orc_gemm_workspace.argtypes = [C.c_char_p, i, i, i, i, i, i, i, i]
        lib.orc_gemm_workspace.restype = C.c_long
        lib.orc_gemm_variant.argtypes = [C.c_char_p, i, i, i, i, i, d, pd, i, pd, i, d, pd, i, vp,
                                         C.c_size_t]
        lib.orc_syrk_workspace.argtypes = [C.c_char_p, i, i, i, i, i, i]
        lib.orc_syrk_workspace.restype = C.c_long
        lib.orc_syrk_variant.argtypes = [C.c_char_p, i, i, i, i, d, pd, i, d, pd, i, vp,
                                         C.c_size_t]
        lib.orc_trsm_workspace.argtypes = [C.c_char_p, i, i, i, i, i, i, i, i]
        lib.orc_trsm_workspace.restype = C.c_long
        lib.orc_trsm_variant.argtypes = [C.c_char_p, i, i, i, i, i, i, d, pd, i, pd, i, vp,
                                         C.c_size_t]
        _lib = lib
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data


def _ld(a):
    assert a.flags.f_contiguous and a.dtype == np.float64
    return max(1, a.shape[0])


def empty(m, n, ld=None):
    """Uninitialised (ld, n) Fortran array; logical part is [:m]."""
    ld = max(m, 1) if ld is None else ld
    return np.empty((ld, n), dtype=np.float64, order="F")


def fill(m, n, ld=None, seed=1, kind=0):
    a = empty(m, n, ld)
    load().orc_dfill(_p(a), m, n, a.shape[0], seed, kind)
    return a


def dgemm(ta, tb, m, n, k, alpha, A, B, beta, Cm):
    load().orc_dgemm(ta, tb, m, n, k, alpha, _p(A), _ld(A), _p(B), _ld(B), beta, _p(Cm), _ld(Cm))


def dsyrk(uplo, trans, n, k, alpha, A, beta, Cm):
    load().orc_dsyrk(uplo, trans, n, k, alpha, _p(A), _ld(A), beta, _p(Cm), _ld(Cm))


def dtrsm(side, uplo, trans, diag, m, n, alpha, A, B):
    load().orc_dtrsm(side, uplo, trans, diag, m, n, alpha, _p(A), _ld(A), _p(B), _ld(B))


def dgeam(ta, tb, m, n, alpha, A, beta, B, Cm):
    load().orc_dgeam(ta, tb, m, n, alpha, _p(A), 1 if A is None else _ld(A), beta, _p(B),
                     1 if B is None else _ld(B), _p(Cm), _ld(Cm))


def gemm_workspace(variant, ta, tb, m, n, k, lda, ldb, ldc):
    return load().orc_gemm_workspace(variant.encode(), ta, tb, m, n, k, lda, ldb, ldc)


def gemm_variant(variant, ta, tb, m, n, k, alpha, A, B, beta, Cm, ws_bytes=None):
    need = gemm_workspace(variant, ta, tb, m, n, k, _ld(A), _ld(B), _ld(Cm))
    if need < 0:
        return -1
    nbytes = need if ws_bytes is None else ws_bytes
    ws = np.full(max(nbytes // 8, 1), np.nan)
    return load().orc_gemm_variant(variant.encode(), ta, tb, m, n, k, alpha, _p(A), _ld(A),
                                   _p(B), _ld(B), beta, _p(Cm), _ld(Cm), _p(ws), nbytes)


def syrk_workspace(variant, uplo, trans, n, k, lda, ldc):
    return load().orc_syrk_workspace(variant.encode(), uplo, trans, n, k, lda, ldc)


def syrk_variant(variant, uplo, trans, n, k, alpha, A, beta, Cm, ws_bytes=None):
    need = syrk_workspace(variant, uplo, trans, n, k, _ld(A), _ld(Cm))
    if need < 0:
        return -1
    nbytes = need if ws_bytes is None else ws_bytes
    ws = np.full(max(nbytes // 8, 1), np.nan)
    return load().orc_syrk_variant(variant.encode(), uplo, trans, n, k, alpha, _p(A), _ld(A),
                                   beta, _p(Cm), _ld(Cm), _p(ws), nbytes)


def trsm_workspace(variant, side, uplo, trans, diag, m, n, lda, ldb):
    return load().orc_trsm_workspace(variant.encode(), side, uplo, trans, diag, m, n, lda, ldb)


def trsm_variant(variant, side, uplo, trans, diag, m, n, alpha, A, B, ws_bytes=None):
    need = trsm_workspace(variant, side, uplo, trans, diag, m, n, _ld(A), _ld(B))
    if need < 0:
        return -1
    nbytes = need if ws_bytes is None else ws_bytes
    ws = np.full(max(nbytes // 8, 1), np.nan)
    return load().orc_trsm_variant(variant.encode(), side, uplo, trans, diag, m, n, alpha, _p(A),
                                   _ld(A), _p(B), _ld(B), _p(ws), nbytes)


def find_cblas():
    """Path of a host CBLAS: system OpenBLAS, else the LP64 OpenBLAS SciPy bundles."""
    for pat in ("/usr/lib/x86_64-linux-gnu/libopenblas.so*", "/usr/lib64/libopenblas.so*"):
        hits = sorted(glob.glob(pat))
        if hits:
            return hits[0]
    try:
        import scipy
        libs = os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)), "scipy.libs")
        hits = sorted(glob.glob(os.path.join(libs, "libscipy_openblas-*.so")))
        if hits:
            return hits[0]
    except ImportError:
        pass
    return None


def cblas_on():
    """Switch gemm/syrk/trsm to host CBLAS.  Returns (threads, library name); (0, 'loops')
    when none is available."""
    path = find_cblas()
    threads = load().orc_cblas_on(path.encode() if path else None)
    return threads, load().orc_cblas_name().decode()


def cblas_off():
    load().orc_cblas_off()
