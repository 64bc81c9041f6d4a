"""ctypes binding of the reference's own executors, compiled from the reference's sources by
oracle/Makefile in two builds: oracle/_ref/librtat_ref.so (on hipBLAS, `make ref`) and
oracle/_ref/librtat_ref_native.so (the same sources with their BLAS aliases rebound to
librtat_native.so, `make ref_native`).  TEST INFRASTRUCTURE (tests/ and bench.py's
reference-timing leg).  The module-level functions drive the hipBLAS build; RefLib(path) binds
either.  available() is False when a library was not built (they are built where the reference
tree is mounted)."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_ref", "librtat_ref.so")
NATIVE_LIB_PATH = os.path.join(HERE, "_ref", "librtat_ref_native.so")


def _p(x):
    return None if x is None else (x if isinstance(x, int) else x.data_ptr())


class RefLib:
    """One build of the reference behind the extern "C" doors of oracle/ref_shim.cpp."""

    def __init__(self, path):
        lib = C.CDLL(path)
        i, d, vp, cp, sz = C.c_int, C.c_double, C.c_void_p, C.c_char_p, C.c_size_t
        pf = C.POINTER(C.c_float)
        lib.ref_on_native.restype = i
        lib.ref_gemm_workspace.restype = C.c_longlong
        lib.ref_gemm_workspace.argtypes = [cp, i, i, i, i, i, i, i, i]
        lib.ref_gemm.argtypes = [cp, i, i, i, i, i, d, vp, i, vp, i, d, vp, i, vp, sz, vp, pf]
        lib.ref_syrk.argtypes = [cp, i, i, i, i, d, vp, i, d, vp, i, vp, sz, vp, pf]
        lib.ref_trsm.argtypes = [cp, i, i, i, i, i, i, d, vp, i, vp, i, vp, sz, vp, pf]
        lib.ref_geam.argtypes = [i, i, i, i, d, vp, i, d, vp, i, vp, i, vp]
        self.lib = lib
        self.on_native = bool(lib.ref_on_native())

    def gemm(self, variant, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, ws, ws_bytes,
             stream):
        """Runs the reference's variant; returns the ms its own Device_Timer measured."""
        ms = C.c_float(-1)
        rc = self.lib.ref_gemm(variant.encode(), ta, tb, m, n, k, alpha, _p(A), lda, _p(B), ldb,
                               beta, _p(Cm), ldc, _p(ws), ws_bytes, stream, C.byref(ms))
        if rc != 0:
            raise RuntimeError("ref_gemm(%s) failed: %d" % (variant, rc))
        return ms.value

    def syrk(self, variant, uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, ws, ws_bytes, stream):
        ms = C.c_float(-1)
        rc = self.lib.ref_syrk(variant.encode(), uplo, trans, n, k, alpha, _p(A), lda, beta,
                               _p(Cm), ldc, _p(ws), ws_bytes, stream, C.byref(ms))
        if rc != 0:
            raise RuntimeError("ref_syrk(%s) failed: %d" % (variant, rc))
        return ms.value

    def trsm(self, variant, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, ws, ws_bytes,
             stream):
        ms = C.c_float(-1)
        rc = self.lib.ref_trsm(variant.encode(), side, uplo, trans, diag, m, n, alpha, _p(A), lda,
                               _p(B), ldb, _p(ws), ws_bytes, stream, C.byref(ms))
        if rc != 0:
            raise RuntimeError("ref_trsm(%s) failed: %d" % (variant, rc))
        return ms.value

    def geam(self, ta, tb, m, n, alpha, A, lda, beta, B, ldb, Cm, ldc, stream):
        rc = self.lib.ref_geam(ta, tb, m, n, alpha, _p(A), lda, beta, _p(B), ldb, _p(Cm), ldc,
                               stream)
        if rc != 0:
            raise RuntimeError("ref_geam failed: %d" % rc)

    def gemm_workspace(self, variant, ta, tb, m, n, k, lda, ldb, ldc):
        return self.lib.ref_gemm_workspace(variant.encode(), ta, tb, m, n, k, lda, ldb, ldc)


_libs = {}


def available(native=False):
    return os.path.exists(NATIVE_LIB_PATH if native else LIB_PATH)


def load(native=False):
    """The reference on hipBLAS (default) or on librtat_native.so."""
    if native not in _libs:
        _libs[native] = RefLib(NATIVE_LIB_PATH if native else LIB_PATH)
        assert _libs[native].on_native == native
    return _libs[native]


def gemm(*a):
    return load().gemm(*a)


def syrk(*a):
    return load().syrk(*a)


def trsm(*a):
    return load().trsm(*a)


def geam(*a):
    return load().geam(*a)


def gemm_workspace(*a):
    return load().gemm_workspace(*a)
