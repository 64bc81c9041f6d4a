#!/usr/bin/env python3
"""Build step of `make -C oracle ref_native`: writes a gpu-api.h for the reference in which the
BLAS alias block (src/gpu-api/gpu-api.h:87-113 - handle and enum types, blasCreate ... blasDgemm
... BLAS_OP_T, all aliases of hipBLAS names) is rebound to include/rtat_native.h, exactly the
edit a maintainer of the reference would make to put librtat_native.so under it.  Everything
else of the header is passed through untouched.

    python make_native_gpu_api.py <reference gpu-api.h> <output gpu-api.h>

The output holds the reference's text: it goes to the ignored build directory oracle/_ref/ and
is never committed.  TEST INFRASTRUCTURE.
"""
import sys

BINDING = """\
  // ---- BLAS boundary rebound to librtat_native (include/rtat_native.h) ----
  using blasHandle_t = rtat_handle_t;
  using blasOperation_t = rtat_operation_t;
  using blasStatus_t = rtat_status_t;
  constexpr auto BLAS_STATUS_SUCCESS = RTAT_STATUS_SUCCESS;
  constexpr auto blasCreate = rtat_create;
  constexpr auto blasDestroy = rtat_destroy;
  constexpr auto blasDgeam = rtat_dgeam;
  constexpr auto blasDgemm = rtat_dgemm;
  constexpr auto blasDtrsm = rtat_dtrsm;
  constexpr auto blasDsyrk = rtat_dsyrk;
  constexpr auto blasSgeam = rtat_sgeam;
  constexpr auto blasSgemm = rtat_sgemm;
  constexpr auto blasStrsm = rtat_strsm;
  constexpr auto blasSsyrk = rtat_ssyrk;
  inline blasStatus_t blasGetStream(blasHandle_t h, Stream_t* s) {
    rtat_stream_t raw = nullptr;
    const blasStatus_t st = rtat_get_stream(h, &raw);
    *s = static_cast<Stream_t>(raw);
    return st;
  }
  inline blasStatus_t blasSetStream(blasHandle_t h, Stream_t s) { return rtat_set_stream(h, s); }
  using blasSideMode_t = rtat_side_t;
  using blasDiagType_t = rtat_diag_t;
  using blasFillMode_t = rtat_fill_t;
  constexpr auto BLAS_SIDE_LEFT = RTAT_SIDE_LEFT;
  constexpr auto BLAS_SIDE_RIGHT = RTAT_SIDE_RIGHT;
  constexpr auto BLAS_DIAG_NON_UNIT = RTAT_DIAG_NON_UNIT;
  constexpr auto BLAS_DIAG_UNIT = RTAT_DIAG_UNIT;
  constexpr auto BLAS_FILL_MODE_LOWER = RTAT_FILL_LOWER;
  constexpr auto BLAS_FILL_MODE_UPPER = RTAT_FILL_UPPER;
  constexpr auto BLAS_OP_N = RTAT_OP_N;
  constexpr auto BLAS_OP_T = RTAT_OP_T;
"""


def main(src, dst):
    lines = open(src).read().split("\n")
    first = next(i for i, l in enumerate(lines) if "using blasHandle_t" in l)
    last = next(i for i, l in enumerate(lines) if "BLAS_OP_T" in l and "constexpr" in l)
    block = lines[first:last + 1]
    # the block must be what this script was written against: nothing but BLAS aliases
    if not all(("_RTAT_GPU_BLAS(" in l or "_RTAT_GPU_ENUM(BLAS_" in l or not l.strip()) for l in block):
        sys.exit("make_native_gpu_api: the BLAS alias block of %s is not the one expected" % src)
    out = []
    for i, l in enumerate(lines):
        if "#include <hipblas/hipblas.h>" in l:
            out.append("#include <rtat_native.h>")
        elif i == first:
            out.extend(BINDING.rstrip("\n").split("\n"))
        elif first < i <= last:
            continue
        else:
            out.append(l)
    open(dst, "w").write("\n".join(out))


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2])
