"""The C-ABI library loads and exports every function include/rtat_native.h (the boundary) and
include/rtat_measure.h (measurement aids) declare.  No compute call is made, so this runs
without a GPU."""
import ctypes
import os
import re

from rtatblas_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(headers=("rtat_native.h", "rtat_measure.h")):
    names = set()
    for header in headers:
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(rtat_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_header_declares_the_boundary():
    names = declared_functions(("rtat_native.h",))
    assert "rtat_hbm_probe" not in names          # a measurement aid, not part of the boundary
    for must in ("rtat_create", "rtat_destroy", "rtat_set_stream", "rtat_get_stream", "rtat_dgemm",
                 "rtat_dsyrk", "rtat_dtrsm", "rtat_dgeam", "rtat_dgemm_ex", "rtat_dfill"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(native.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_every_declared_symbol():
    assert sorted(native.SIGNATURES) == declared_functions()


def test_no_compute_metadata_calls():
    assert native.version().startswith("rtat-native")
    assert [native.variant_name(v) for v in range(native.GEMM_VARIANT_COUNT)] == [
        "auto", "256x128", "128x128", "128x64", "64x64"]
    assert native.variant_name(99) is None
    lib = native.load()
    # one 128 x 128 inverse per diagonal block + the 28 packed off-diagonal blocks of every
    # 1024-row panel, the larger of the two panel layouts (+ alignment)
    assert lib.rtat_dtrsm_workspace_bytes(native.SIDE_LEFT, 8192, 100) == (64 + 8 * 28) * 128 * 128 * 8 + 16
    assert lib.rtat_dtrsm_workspace_bytes(native.SIDE_RIGHT, 8192, 100) == (1 + 28) * 128 * 128 * 8 + 16
    # a null handle is reported, not dereferenced
    assert lib.rtat_destroy(None) == 9
