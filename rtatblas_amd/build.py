"""Build recipe for the native libraries of this package (hipcc, gfx950 only).

    python -m rtatblas_amd.build            # everything
    python -m rtatblas_amd.build native     # librtat_native.so (HIP kernels + C ABI)
    python -m rtatblas_amd.build host       # librtat.so (C++ host layer + planner C API)
    python -m rtatblas_amd.build apps       # run_tests driver

Objects go to rtatblas_amd/_obj, libraries to rtatblas_amd/lib.  Nothing is compiled at
import time: tests, the smoke check and the bench load what this step left in the tree.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
OBJ = os.path.join(PKG, "_obj")
LIB = os.path.join(PKG, "lib")
BIN = os.path.join(PKG, "bin")

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

# -packed-fp32-ops off: hipcc otherwise forms v_pk_*_f32 from ordinary float code.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-Wno-unused-parameter",
          "-I" + os.path.join(ROOT, "include")]

NATIVE_SOURCES = ["api.hip", "geam.hip", "gemm.hip", "trsm.hip"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    noise = ("packed-fp32-ops", "is not a recognized feature")
    out = "\n".join(l for l in proc.stdout.splitlines() if not any(s in l for s in noise))
    if out.strip():
        print(out)


def _compile_many(jobs, workers):
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for fut in [pool.submit(_run, cmd) for cmd in jobs]:
            fut.result()


def build_native(workers=4):
    """HIP kernels + C ABI -> lib/librtat_native.so."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB, exist_ok=True)
    jobs, objs = [], []
    for src in NATIVE_SOURCES:
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        objs.append(obj)
        jobs.append([HIPCC, "-c", os.path.join(CSRC, src), "-o", obj] + COMMON + DEVICE_FLAGS)
    _compile_many(jobs, workers)
    out = os.path.join(LIB, "librtat_native.so")
    _run([HIPCC, "-shared", "-o", out] + objs + ["--offload-arch=gfx950"])
    return out


def host_sources():
    return sorted(os.path.join(dp, f) for dp, _, fs in os.walk(os.path.join(HOST, "src"))
                  for f in fs if f.endswith(".cpp"))


def host_includes():
    dirs = [os.path.join(HOST, d) for d in
            ("gpu-api", "timing", "matrix_ops", "methods", "planning", "json", "app", "")]
    return ["-I" + d for d in dirs]


def build_host(workers=4):
    """C++ host layer (matrix-op tree, methods, planner, C API) -> lib/librtat.so."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB, exist_ok=True)
    jobs, objs = [], []
    for src in host_sources():
        obj = os.path.join(OBJ, "host_" + os.path.basename(src).replace(".cpp", ".o"))
        objs.append(obj)
        jobs.append([HIPCC, "-x", "c++", "-c", src, "-o", obj, "-D__HIP_PLATFORM_AMD__"] + COMMON
                    + host_includes() + ["-I/opt/rocm/include"])
    _compile_many(jobs, workers)
    out = os.path.join(LIB, "librtat.so")
    _run([HIPCC, "-shared", "-o", out] + objs +
         ["-L" + LIB, "-lrtat_native", "-Wl,-rpath,$ORIGIN", "-L/opt/rocm/lib", "-lamdhip64"])
    return out


def build_apps(workers=4):
    """run_tests, the JSON-driven driver -> bin/run_tests."""
    os.makedirs(BIN, exist_ok=True)
    link = ["-L" + LIB, "-lrtat", "-lrtat_native", "-Wl,-rpath,$ORIGIN/../lib",
            "-L/opt/rocm/lib", "-lamdhip64"]
    inc = COMMON + host_includes() + ["-I/opt/rocm/include", "-D__HIP_PLATFORM_AMD__"]
    _run([HIPCC, "-x", "c++", os.path.join(HOST, "app", "run_tests.cpp"), "-o",
          os.path.join(BIN, "run_tests")] + inc + link)


def build_all(workers=4):
    build_native(workers)
    build_host(workers)
    build_apps(workers)


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    {"all": build_all, "native": build_native, "host": build_host, "apps": build_apps}[what]()
    print("built:", what)
