"""ctypes binding of librtat.so's planner C ABI (include/rtat_planner.h): the variant trees
and the autotuning planner of the C++ host layer, driven from Python for tests and the bench."""
import ctypes as C
import json
import os

from . import native

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "librtat.so")

_vp, _i, _d, _cp, _sz, _ll = C.c_void_p, C.c_int, C.c_double, C.c_char_p, C.c_size_t, C.c_longlong

SIGNATURES = {
    "rtat_planner_create": (_vp, [_cp]),
    "rtat_planner_destroy": (None, [_vp]),
    "rtat_planner_configure": (_i, [_vp, _i, _i]),
    "rtat_planner_set_refinement": (_i, [_vp, _i, _d]),
    "rtat_planner_use_reference_defaults": (_i, [_vp]),
    "rtat_planner_set_tie_margin": (_i, [_vp, _d]),
    "rtat_planner_set_filter": (_i, [_vp, _cp]),
    "rtat_planner_learn_filter": (_i, [_vp, _cp, _d]),
    "rtat_planner_gemm_admitted": (_cp, [_vp, _i, _i, _i, _i, _i]),
    "rtat_planner_syrk_admitted": (_cp, [_vp, _i, _i, _i, _i]),
    "rtat_planner_trsm_admitted": (_cp, [_vp, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_variant_count": (_i, [_vp]),
    "rtat_planner_variant_name": (_i, [_vp, _i, _cp, _sz]),
    "rtat_planner_gemm_workspace": (_ll, [_vp, _cp, _i, _i, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_syrk_workspace": (_ll, [_vp, _cp, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_trsm_workspace": (_ll, [_vp, _cp, _i, _i, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_gemm_workspace_max": (_ll, [_vp, _i, _i, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_syrk_workspace_max": (_ll, [_vp, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_trsm_workspace_max": (_ll, [_vp, _i, _i, _i, _i, _i, _i, _i, _i]),
    "rtat_planner_gemm": (_i, [_vp, _vp, _cp, _i, _i, _i, _i, _i, _d, _vp, _i, _vp, _i, _d, _vp,
                               _i, _vp, _sz, _cp, _sz]),
    "rtat_planner_syrk": (_i, [_vp, _vp, _cp, _i, _i, _i, _i, _d, _vp, _i, _d, _vp, _i, _vp, _sz,
                               _cp, _sz]),
    "rtat_planner_trsm": (_i, [_vp, _vp, _cp, _i, _i, _i, _i, _i, _i, _d, _vp, _i, _vp, _i, _vp,
                               _sz, _cp, _sz]),
    "rtat_planner_stats_json": (_cp, [_vp]),
    "rtat_planner_plans_json": (_cp, [_vp]),
    "rtat_planner_load_plans": (_i, [_vp, _cp]),
    "rtat_planner_last_error": (_cp, []),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        native.load()  # librtat.so depends on librtat_native.so
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run `python -m rtatblas_amd.build` first" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def _ptr(x):
    if x is None or isinstance(x, int):
        return x
    return x.data_ptr()


class Planner:
    """One Planning_System<...<double>>: "gemm", "gemm_pad", "gemm_tile", "gemm_pad_tile",
    "syrk", "syrk_tile", "trsm", "trsm_tile" and the "*_fused" families."""

    def __init__(self, method, tests_until_converge=None, statistic=None):
        self.lib = load()
        self.method = method
        self.p = self.lib.rtat_planner_create(method.encode())
        if not self.p:
            raise ValueError(self.lib.rtat_planner_last_error().decode())
        if tests_until_converge is not None or statistic is not None:
            self.lib.rtat_planner_configure(self.p, tests_until_converge or 3,
                                            1 if statistic is None else statistic)

    def set_refinement(self, extra_tests, margin=0.05):
        self.lib.rtat_planner_set_refinement(self.p, extra_tests, margin)

    def set_tie_margin(self, margin):
        self.lib.rtat_planner_set_tie_margin(self.p, margin)

    def set_filter(self, patterns):
        """Comma-separated glob patterns over variant names; None admits everything."""
        rc = self.lib.rtat_planner_set_filter(self.p, None if patterns is None else patterns.encode())
        if rc != 0:
            self._fail("rtat_planner_set_filter", rc)

    def learn_filter(self, stats, slack=0.1):
        """Admit, per problem class, only the variants that came within `slack` of the fastest
        in `stats` (a report of this method, as stats() returns it)."""
        rc = self.lib.rtat_planner_learn_filter(self.p, json.dumps(stats).encode(), slack)
        if rc < 0:
            self._fail("rtat_planner_learn_filter", rc)
        return rc

    def _names(self, text, what):
        if text is None:
            self._fail(what, -1)
        return text.decode().split()

    def gemm_admitted(self, ta, tb, m, n, k):
        return self._names(self.lib.rtat_planner_gemm_admitted(self.p, ta, tb, m, n, k),
                           "rtat_planner_gemm_admitted")

    def syrk_admitted(self, uplo, trans, n, k):
        return self._names(self.lib.rtat_planner_syrk_admitted(self.p, uplo, trans, n, k),
                           "rtat_planner_syrk_admitted")

    def trsm_admitted(self, side, uplo, trans, diag, m, n):
        return self._names(self.lib.rtat_planner_trsm_admitted(self.p, side, uplo, trans, diag, m, n),
                           "rtat_planner_trsm_admitted")

    def use_reference_defaults(self):
        self.lib.rtat_planner_use_reference_defaults(self.p)

    def close(self):
        if self.p:
            self.lib.rtat_planner_destroy(self.p)
            self.p = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _fail(self, what, rc):
        raise RuntimeError("%s failed (%d): %s" % (what, rc,
                                                   self.lib.rtat_planner_last_error().decode()))

    def variants(self):
        out = []
        buf = C.create_string_buffer(48)
        for i in range(self.lib.rtat_planner_variant_count(self.p)):
            self.lib.rtat_planner_variant_name(self.p, i, buf, 48)
            out.append(buf.value.decode())
        return out

    def gemm_workspace(self, variant, ta, tb, m, n, k, lda, ldb, ldc):
        if variant is None:
            return self.lib.rtat_planner_gemm_workspace_max(self.p, ta, tb, m, n, k, lda, ldb, ldc)
        return self.lib.rtat_planner_gemm_workspace(self.p, variant.encode(), ta, tb, m, n, k, lda,
                                                    ldb, ldc)

    def syrk_workspace(self, variant, uplo, trans, n, k, lda, ldc):
        if variant is None:
            return self.lib.rtat_planner_syrk_workspace_max(self.p, uplo, trans, n, k, lda, ldc)
        return self.lib.rtat_planner_syrk_workspace(self.p, variant.encode(), uplo, trans, n, k,
                                                    lda, ldc)

    def trsm_workspace(self, variant, side, uplo, trans, diag, m, n, lda, ldb):
        if variant is None:
            return self.lib.rtat_planner_trsm_workspace_max(self.p, side, uplo, trans, diag, m, n,
                                                            lda, ldb)
        return self.lib.rtat_planner_trsm_workspace(self.p, variant.encode(), side, uplo, trans,
                                                    diag, m, n, lda, ldb)

    def gemm(self, handle, variant, ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, Cm, ldc, ws,
             ws_bytes):
        """variant None = the planner's own plan.  Returns the variant that ran."""
        chosen = C.create_string_buffer(48)
        rc = self.lib.rtat_planner_gemm(self.p, handle.h, None if variant is None else variant.encode(),
                                        ta, tb, m, n, k, alpha, _ptr(A), lda, _ptr(B), ldb, beta,
                                        _ptr(Cm), ldc, _ptr(ws), ws_bytes, chosen, 48)
        if rc != 0:
            self._fail("rtat_planner_gemm", rc)
        return chosen.value.decode()

    def syrk(self, handle, variant, uplo, trans, n, k, alpha, A, lda, beta, Cm, ldc, ws, ws_bytes):
        chosen = C.create_string_buffer(48)
        rc = self.lib.rtat_planner_syrk(self.p, handle.h, None if variant is None else variant.encode(),
                                        uplo, trans, n, k, alpha, _ptr(A), lda, beta, _ptr(Cm), ldc,
                                        _ptr(ws), ws_bytes, chosen, 48)
        if rc != 0:
            self._fail("rtat_planner_syrk", rc)
        return chosen.value.decode()

    def trsm(self, handle, variant, side, uplo, trans, diag, m, n, alpha, A, lda, B, ldb, ws,
             ws_bytes):
        chosen = C.create_string_buffer(48)
        rc = self.lib.rtat_planner_trsm(self.p, handle.h, None if variant is None else variant.encode(),
                                        side, uplo, trans, diag, m, n, alpha, _ptr(A), lda, _ptr(B),
                                        ldb, _ptr(ws), ws_bytes, chosen, 48)
        if rc != 0:
            self._fail("rtat_planner_trsm", rc)
        return chosen.value.decode()

    def stats(self):
        s = self.lib.rtat_planner_stats_json(self.p)
        if s is None:
            self._fail("rtat_planner_stats_json", -1)
        return json.loads(s.decode())

    def plans(self):
        s = self.lib.rtat_planner_plans_json(self.p)
        if s is None:
            self._fail("rtat_planner_plans_json", -1)
        return json.loads(s.decode())

    def load_plans(self, doc):
        rc = self.lib.rtat_planner_load_plans(self.p, json.dumps(doc).encode())
        if rc < 0:
            self._fail("rtat_planner_load_plans", rc)
        return rc
