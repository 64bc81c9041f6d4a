"""ctypes binding of oracle/_ref/librtat_ref.so: the reference's own executors on hipBLAS.
TEST INFRASTRUCTURE (tests/ and bench.py's reference-timing leg).  available() is False when
the library was not built (it is built where the reference tree is mounted)."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_ref", "librtat_ref.so")
_lib = None


def available():
    return os.path.exists(LIB_PATH)


def load():
    global _lib
    if _lib is None:
        lib = C.CDLL(LIB_PATH)
        i, d, vp, cp, sz = C.c_int, C.c_double, C.c_void_p, C.c_char_p, C.c_size_t
        pf = C.POINTER(C.c_float)
        lib.ref_gemm_workspace.restype = C.c_longlong
        lib.ref_gemm_workspace.argtypes = [cp, i, i, i, i, i, i, i, i]
        lib.ref_gemm.argtypes = [cp, i, i, i, i, i, d, vp, i, vp, i, d, vp, i, vp, sz, vp, pf]
        lib.ref_syrk.argtypes = [cp, i, i, i, i, d, vp, i, d, vp, i, vp, sz, vp, pf]
        lib.ref_trsm.argtypes = [cp, i, i, i, i, i, i, d, vp, i, vp, i, vp, sz, vp, pf]
        lib.ref_geam.argtypes = [i, i, i, i, d, vp, i, d, vp, i, vp, i, vp]
        _lib = lib
    return _lib


def _p(x):
    return None if x is None else (x if isinstance(x, int) else x.data_ptr())


def gemm(variant, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, ws, ws_bytes, stream):
    """Runs the reference's variant; returns the ms its own Device_Timer measured."""
    ms = C.c_float(-1)
    rc = load().ref_gemm(variant.encode(), ta, tb, m, n, k, alpha, _p(A), lda, _p(B), ldb, beta,
                         _p(Cm), ldc, _p(ws), ws_bytes, stream, C.byref(ms))
    if rc != 0:
        raise RuntimeError("ref_gemm(%s) failed: %d" % (variant, rc))
    return ms.value


def syrk(variant, uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, ws, ws_bytes, stream):
    ms = C.c_float(-1)
    rc = load().ref_syrk(variant.encode(), uplo, trans, n, k, alpha, _p(A), lda, beta, _p(Cm), ldc,
                         _p(ws), ws_bytes, stream, C.byref(ms))
    if rc != 0:
        raise RuntimeError("ref_syrk(%s) failed: %d" % (variant, rc))
    return ms.value


def trsm(variant, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, ws, ws_bytes, stream):
    ms = C.c_float(-1)
    rc = load().ref_trsm(variant.encode(), side, uplo, trans, diag, m, n, alpha, _p(A), lda, _p(B),
                         ldb, _p(ws), ws_bytes, stream, C.byref(ms))
    if rc != 0:
        raise RuntimeError("ref_trsm(%s) failed: %d" % (variant, rc))
    return ms.value


def geam(ta, tb, m, n, alpha, A, lda, beta, B, ldb, Cm, ldc, stream):
    rc = load().ref_geam(ta, tb, m, n, alpha, _p(A), lda, beta, _p(B), ldb, _p(Cm), ldc, stream)
    if rc != 0:
        raise RuntimeError("ref_geam failed: %d" % rc)


def gemm_workspace(variant, ta, tb, m, n, k, lda, ldb, ldc):
    return load().ref_gemm_workspace(variant.encode(), ta, tb, m, n, k, lda, ldb, ldc)
