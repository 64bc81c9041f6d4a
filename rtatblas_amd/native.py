"""ctypes binding of librtat_native.so (the C ABI in include/rtat_native.h).

Plumbing for tests, the smoke check and the bench: device memory and streams come from
torch, every matrix argument is a raw device pointer.  There is no fallback: if the library
has not been built, loading raises.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "librtat_native.so")

OP_N, OP_T = 111, 112
FILL_UPPER, FILL_LOWER = 121, 122
DIAG_NON_UNIT, DIAG_UNIT = 131, 132
SIDE_LEFT, SIDE_RIGHT = 141, 142

GEMM_AUTO, GEMM_T256x128, GEMM_T128x128, GEMM_T128x64, GEMM_T64x64 = 0, 1, 2, 3, 4
GEMM_VARIANT_COUNT = 5
TAIL_AUTO, TAIL_WHOLE, TAIL_SPLIT = 0, 1, 2
PANEL_AUTO, PANEL_512, PANEL_1024 = 0, 1, 2


def kernel_options(tile=GEMM_AUTO, tail=TAIL_AUTO, panel=PANEL_AUTO):
    """RTAT_KERNEL_OPTIONS: the word the *_ex entry points take as `variant`."""
    return tile | (tail << 8) | (panel << 12)


PROBE_READ, PROBE_WRITE, PROBE_COPY = 0, 1, 2
FILL_IID, FILL_SYMMETRIC, FILL_TRI_LOWER, FILL_UNIT_INTERVAL, FILL_TRI_FULL = 0, 1, 2, 3, 4

STATUS_NAMES = {0: "SUCCESS", 1: "NOT_INITIALIZED", 2: "ALLOC_FAILED", 3: "INVALID_VALUE",
                5: "EXECUTION_FAILED", 7: "NOT_SUPPORTED", 9: "HANDLE_IS_NULLPTR",
                10: "INVALID_ENUM"}

_pd = C.POINTER(C.c_double)
_pf = C.POINTER(C.c_float)
_vp = C.c_void_p
_i = C.c_int

# name -> (restype, argtypes); every symbol include/rtat_native.h declares.
SIGNATURES = {
    "rtat_create": (_i, [C.POINTER(_vp)]),
    "rtat_destroy": (_i, [_vp]),
    "rtat_set_stream": (_i, [_vp, _vp]),
    "rtat_get_stream": (_i, [_vp, C.POINTER(_vp)]),
    "rtat_set_workspace": (_i, [_vp, _vp, C.c_size_t]),
    "rtat_dtrsm_workspace_bytes": (C.c_size_t, [_i, _i, _i]),
    "rtat_dgemm": (_i, [_vp, _i, _i, _i, _i, _i, _pd, _vp, _i, _vp, _i, _pd, _vp, _i]),
    "rtat_dsyrk": (_i, [_vp, _i, _i, _i, _i, _pd, _vp, _i, _pd, _vp, _i]),
    "rtat_dtrsm": (_i, [_vp, _i, _i, _i, _i, _i, _i, _pd, _vp, _i, _vp, _i]),
    "rtat_dtrsm_static": (_i, [_vp, _i, _i, _i, _i, _i, _i, _pd, _vp, _i, _vp, _i]),
    "rtat_dgeam": (_i, [_vp, _i, _i, _i, _i, _pd, _vp, _i, _pd, _vp, _i, _vp, _i]),
    "rtat_sgemm": (_i, [_vp, _i, _i, _i, _i, _i, _pf, _vp, _i, _vp, _i, _pf, _vp, _i]),
    "rtat_ssyrk": (_i, [_vp, _i, _i, _i, _i, _pf, _vp, _i, _pf, _vp, _i]),
    "rtat_strsm": (_i, [_vp, _i, _i, _i, _i, _i, _i, _pf, _vp, _i, _vp, _i]),
    "rtat_sgeam": (_i, [_vp, _i, _i, _i, _i, _pf, _vp, _i, _pf, _vp, _i, _vp, _i]),
    "rtat_gemm_variant_name": (C.c_char_p, [_i]),
    "rtat_tail_mode_name": (C.c_char_p, [_i]),
    "rtat_trsm_panel_name": (C.c_char_p, [_i]),
    "rtat_last_launch": (_i, [_vp, _vp]),
    "rtat_dgemm_ex": (_i, [_vp, _i, _i, _i, _i, _i, _pd, _vp, _i, _vp, _i, _pd, _vp, _i, _i]),
    "rtat_dsyrk_ex": (_i, [_vp, _i, _i, _i, _i, _pd, _vp, _i, _pd, _vp, _i, _i]),
    "rtat_dtrsm_ex": (_i, [_vp, _i, _i, _i, _i, _i, _i, _pd, _vp, _i, _vp, _i, _i]),
    "rtat_sgemm_ex": (_i, [_vp, _i, _i, _i, _i, _i, _pf, _vp, _i, _vp, _i, _pf, _vp, _i, _i]),
    "rtat_ssyrk_ex": (_i, [_vp, _i, _i, _i, _i, _pf, _vp, _i, _pf, _vp, _i, _i]),
    "rtat_strsm_ex": (_i, [_vp, _i, _i, _i, _i, _i, _i, _pf, _vp, _i, _vp, _i, _i]),
    "rtat_dfill": (_i, [_vp, _vp, _i, _i, _i, C.c_uint64, _i]),
    "rtat_sfill": (_i, [_vp, _vp, _i, _i, _i, C.c_uint64, _i]),
    "rtat_device_peaks": (_i, [_vp, _pd, _pd, C.POINTER(_i)]),
    "rtat_dmove_pair": (_i, [_vp, _vp, _vp]),
    "rtat_smove_pair": (_i, [_vp, _vp, _vp]),
    "rtat_hbm_probe": (_i, [_vp, _i, _vp, _vp, C.c_size_t]),
    "rtat_version": (C.c_char_p, []),
}

class LaunchInfo(C.Structure):
    """rtat_launch_info_t."""
    _fields_ = [("tile", C.c_char * 16), ("tiles", _i), ("split_tiles", _i), ("split_slices", _i),
                ("subdivided", _i), ("trsm_panel_rows", _i), ("trsm_panel_width", _i)]


class Move(C.Structure):
    """rtat_move_t: one job of rtat_dmove_pair / rtat_smove_pair."""
    _fields_ = [("trans", _i), ("m", _i), ("n", _i), ("A", _vp), ("lda", _i), ("C", _vp),
                ("ldc", _i)]


_lib = None


def load():
    """The loaded library with argument types set.  Raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: run `python -m rtatblas_amd.build` (hipcc, gfx950) first; "
                "there is no CPU fallback" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


class RtatError(RuntimeError):
    def __init__(self, what, status):
        super().__init__("%s returned %d (%s)" % (what, status, STATUS_NAMES.get(status, "?")))
        self.status = status


def _check(what, status):
    if status != 0:
        raise RtatError(what, status)


def _ptr(x):
    """Device pointer of a torch tensor (or an int / None passed through)."""
    if x is None:
        return None
    if isinstance(x, int):
        return x
    return x.data_ptr()


class Handle:
    """rtat_handle_t bound to a stream (default: torch's current stream on cuda:0)."""

    def __init__(self, stream=None):
        self.lib = load()
        h = _vp()
        _check("rtat_create", self.lib.rtat_create(C.byref(h)))
        self.h = h
        if stream is not None:
            self.set_stream(stream)

    def set_stream(self, stream):
        raw = stream if isinstance(stream, int) or stream is None else stream.cuda_stream
        _check("rtat_set_stream", self.lib.rtat_set_stream(self.h, raw))

    def close(self):
        if self.h is not None:
            self.lib.rtat_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # Each method returns the status unless check=True (default), in which case it raises.
    def dgemm(self, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, variant=None,
              check=True):
        a, b = C.c_double(alpha), C.c_double(beta)
        if variant is None:
            st = self.lib.rtat_dgemm(self.h, ta, tb, m, n, k, C.byref(a), _ptr(A), lda, _ptr(B),
                                     ldb, C.byref(b), _ptr(Cm), ldc)
        else:
            st = self.lib.rtat_dgemm_ex(self.h, ta, tb, m, n, k, C.byref(a), _ptr(A), lda,
                                        _ptr(B), ldb, C.byref(b), _ptr(Cm), ldc, variant)
        if check:
            _check("rtat_dgemm", st)
        return st

    def dsyrk(self, uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, variant=None, check=True):
        a, b = C.c_double(alpha), C.c_double(beta)
        if variant is None:
            st = self.lib.rtat_dsyrk(self.h, uplo, trans, n, k, C.byref(a), _ptr(A), lda,
                                     C.byref(b), _ptr(Cm), ldc)
        else:
            st = self.lib.rtat_dsyrk_ex(self.h, uplo, trans, n, k, C.byref(a), _ptr(A), lda,
                                        C.byref(b), _ptr(Cm), ldc, variant)
        if check:
            _check("rtat_dsyrk", st)
        return st

    def dtrsm(self, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, variant=None,
              check=True):
        a = C.c_double(alpha)
        if variant is None:
            st = self.lib.rtat_dtrsm(self.h, side, uplo, trans, diag, m, n, C.byref(a), _ptr(A),
                                     lda, _ptr(B), ldb)
        else:
            st = self.lib.rtat_dtrsm_ex(self.h, side, uplo, trans, diag, m, n, C.byref(a),
                                        _ptr(A), lda, _ptr(B), ldb, variant)
        if check:
            _check("rtat_dtrsm", st)
        return st

    def dtrsm_static(self, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, check=True):
        a = C.c_double(alpha)
        st = self.lib.rtat_dtrsm_static(self.h, side, uplo, trans, diag, m, n, C.byref(a),
                                        _ptr(A), lda, _ptr(B), ldb)
        if check:
            _check("rtat_dtrsm_static", st)
        return st

    def dgeam(self, ta, tb, m, n, alpha, A, lda, beta, B, ldb, Cm, ldc, check=True):
        a, b = C.c_double(alpha), C.c_double(beta)
        st = self.lib.rtat_dgeam(self.h, ta, tb, m, n, C.byref(a), _ptr(A), lda, C.byref(b),
                                 _ptr(B), ldb, _ptr(Cm), ldc)
        if check:
            _check("rtat_dgeam", st)
        return st

    def sgemm(self, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, variant=None,
              check=True):
        a, b = C.c_float(alpha), C.c_float(beta)
        st = self.lib.rtat_sgemm_ex(self.h, ta, tb, m, n, k, C.byref(a), _ptr(A), lda, _ptr(B),
                                    ldb, C.byref(b), _ptr(Cm), ldc,
                                    GEMM_AUTO if variant is None else variant)
        if check:
            _check("rtat_sgemm", st)
        return st

    def ssyrk(self, uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, variant=None, check=True):
        a, b = C.c_float(alpha), C.c_float(beta)
        st = self.lib.rtat_ssyrk_ex(self.h, uplo, trans, n, k, C.byref(a), _ptr(A), lda,
                                    C.byref(b), _ptr(Cm), ldc,
                                    GEMM_AUTO if variant is None else variant)
        if check:
            _check("rtat_ssyrk", st)
        return st

    def strsm(self, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, variant=None,
              check=True):
        a = C.c_float(alpha)
        st = self.lib.rtat_strsm_ex(self.h, side, uplo, trans, diag, m, n, C.byref(a), _ptr(A),
                                    lda, _ptr(B), ldb, GEMM_AUTO if variant is None else variant)
        if check:
            _check("rtat_strsm", st)
        return st

    def sgeam(self, ta, tb, m, n, alpha, A, lda, beta, B, ldb, Cm, ldc, check=True):
        a, b = C.c_float(alpha), C.c_float(beta)
        st = self.lib.rtat_sgeam(self.h, ta, tb, m, n, C.byref(a), _ptr(A), lda, C.byref(b),
                                 _ptr(B), ldb, _ptr(Cm), ldc)
        if check:
            _check("rtat_sgeam", st)
        return st

    def dfill(self, A, m, n, ld, seed, kind=FILL_IID, check=True):
        st = self.lib.rtat_dfill(self.h, _ptr(A), m, n, ld, seed, kind)
        if check:
            _check("rtat_dfill", st)
        return st

    def sfill(self, A, m, n, ld, seed, kind=FILL_IID, check=True):
        st = self.lib.rtat_sfill(self.h, _ptr(A), m, n, ld, seed, kind)
        if check:
            _check("rtat_sfill", st)
        return st

    def move_pair(self, first, second, single=False, check=True):
        """first, second: (trans, m, n, A, lda, C, ldc) tuples."""
        jobs = [Move(t, m, n, _ptr(A), lda, _ptr(Cm), ldc) for (t, m, n, A, lda, Cm, ldc) in
                (first, second)]
        fn = self.lib.rtat_smove_pair if single else self.lib.rtat_dmove_pair
        st = fn(self.h, C.byref(jobs[0]), C.byref(jobs[1]))
        if check:
            _check("rtat_move_pair", st)
        return st

    def hbm_probe(self, kind, src, dst, nbytes, check=True):
        st = self.lib.rtat_hbm_probe(self.h, kind, _ptr(src), _ptr(dst), nbytes)
        if check:
            _check("rtat_hbm_probe", st)
        return st

    def set_workspace(self, ptr, nbytes):
        _check("rtat_set_workspace", self.lib.rtat_set_workspace(self.h, _ptr(ptr), nbytes))

    def last_launch(self):
        """What the last GEMM-core launch on this handle did, as a dict."""
        info = LaunchInfo()
        _check("rtat_last_launch", self.lib.rtat_last_launch(self.h, C.byref(info)))
        return {"tile": info.tile.decode(), "tiles": info.tiles, "split_tiles": info.split_tiles,
                "split_slices": info.split_slices, "subdivided": info.subdivided,
                "trsm_panel_rows": info.trsm_panel_rows,
                "trsm_panel_width": info.trsm_panel_width}

    def peaks(self):
        f, b, cu = C.c_double(), C.c_double(), C.c_int()
        _check("rtat_device_peaks",
               self.lib.rtat_device_peaks(self.h, C.byref(f), C.byref(b), C.byref(cu)))
        return f.value, b.value, cu.value


def variant_name(v):
    s = load().rtat_gemm_variant_name(v)
    return s.decode() if s is not None else None


def tail_mode_name(v):
    s = load().rtat_tail_mode_name(v)
    return s.decode() if s is not None else None


def trsm_panel_name(v):
    s = load().rtat_trsm_panel_name(v)
    return s.decode() if s is not None else None


def version():
    return load().rtat_version().decode()
