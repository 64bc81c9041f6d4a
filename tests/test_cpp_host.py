"""Runs the C++ tests of the host layer (tests/cpp/rtat_cpp_tests.cpp, modelled on the
reference's GoogleTest suites): the device-free subset here, the rest on the GPU."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin", "rtat_cpp_tests")


def run(mode):
    assert os.path.exists(BIN), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    proc = subprocess.run([BIN, mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=900)
    failed = re.findall(r"\[FAILED\] (\S+)", proc.stdout)
    m = re.search(r"SUMMARY ran=(\d+) failed=(\d+)", proc.stdout)
    assert m, proc.stdout[-3000:]
    assert proc.returncode == 0 and not failed, "failed: %s\n%s" % (failed, proc.stdout[-6000:])
    return int(m.group(1))


def test_cpp_host_layer_without_a_device():
    assert run("--cpu") >= 20


@pytest.mark.gpu
def test_cpp_host_layer_on_the_gpu():
    assert run("--gpu") >= 20


def test_planner_abi_exports_every_declared_symbol():
    import ctypes
    from rtatblas_amd import planner
    text = open(os.path.join(ROOT, "include", "rtat_planner.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(rtat_planner_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(planner.SIGNATURES)
    lib = ctypes.CDLL(planner.LIB_PATH)
    assert not [n for n in declared if not hasattr(lib, n)]
    p = planner.Planner("gemm_pad")
    assert len(p.variants()) == 64 and p.variants()[0] == "NNNNNN"
    assert planner.Planner("syrk").variants() == ["FF", "FT", "TF", "TT"]
    assert planner.Planner("gemm_tile").variants()[:2] == ["NNN/auto", "NNN/256x128"]
    assert len(planner.Planner("gemm_pad_tile").variants()) == 960
    assert planner.Planner("syrk_tile").variants()[:4] == [
        "FF/auto/auto", "FF/auto/whole", "FF/auto/split", "FF/256x128/auto"]
    assert planner.Planner("trsm_tile").variants()[-1] == "TT/64x64/split/1024"
    # "X" (the fused form) is the tree of the untransposed switch: named, not enumerated
    assert planner.Planner("gemm_fused").variants()[:3] == ["NNN", "NNT", "NTN"]
    assert planner.Planner("syrk_fused").variants() == ["FF", "FT", "TF", "TT"]
    assert planner.Planner("trsm_fused").variants() == ["FF", "FT", "TF", "TT"]
    p = planner.Planner("gemm_pad_tile")
    p.set_filter("NNN???/*/*")
    assert len(p.gemm_admitted(111, 111, 100, 100, 100)) == 120
    p.set_filter("TTTPPP/64x64/split")
    assert p.gemm_admitted(111, 111, 100, 100, 100) == ["NNNNNN/auto/auto", "TTTPPP/64x64/split"]
    p.set_filter(None)
    assert len(p.gemm_admitted(111, 111, 100, 100, 100)) == 960
    m, n, k = 100, 80, 60       # the fused forms need no scratch of their own
    assert planner.Planner("gemm_fused").gemm_workspace("NNX", 111, 111, m, n, k, m, k, m) == 0
    assert planner.Planner("gemm_fused").gemm_workspace("NNT", 111, 111, m, n, k, m, k, m) == 8 * n * m
    assert planner.Planner("syrk_fused").syrk_workspace("FX", 122, 111, n, k, n, n) == 0
    assert planner.Planner("trsm_fused").trsm_workspace("XF", 141, 122, 111, 131, m, n, m, m) == 0
    with pytest.raises(ValueError):
        planner.Planner("nope")


def test_planner_workspace_matches_oracle(orc):
    """The C++ tree's workspace accounting against the C oracle's, for every variant, no GPU."""
    from rtatblas_amd import planner
    m, n, k = 1007, 409, 615
    for ta, tb in [(111, 111), (112, 111), (111, 112), (112, 112)]:
        lda = (k if ta == 112 else m) + 3
        ldb = (n if tb == 112 else k) + 3
        for method in ("gemm", "gemm_pad"):
            p = planner.Planner(method)
            for v in p.variants():
                assert p.gemm_workspace(v, ta, tb, m, n, k, lda, ldb, m + 3) == \
                    orc.gemm_workspace(v, ta, tb, m, n, k, lda, ldb, m + 3), (method, v)
    p = planner.Planner("syrk")
    for v in p.variants():
        for trans in (111, 112):
            lda = (k if trans == 112 else n)
            assert p.syrk_workspace(v, 122, trans, n, k, lda, n) == \
                orc.syrk_workspace(v, 122, trans, n, k, lda, n)
    p = planner.Planner("trsm")
    for v in p.variants():
        for side in (141, 142):
            na = m if side == 141 else n
            assert p.trsm_workspace(v, side, 122, 111, 131, m, n, na, m) == \
                orc.trsm_workspace(v, side, 122, 111, 131, m, n, na, m)


def test_planner_workspace_max_is_the_largest_variants(orc):
    """calculate_workspace without a variant (reference planning_system.h:116-118): the largest
    need over the method's variants, hand-computed here for the all-transposing ones - GEMM
    TTT k*m + n*k + n*m elements, SYRK TT k*n + n*n, TRSM TT (swap + transposed A) na*na + n*m."""
    from rtatblas_amd import planner
    m, n, k = 1007, 409, 615
    p = planner.Planner("gemm")
    assert p.gemm_workspace(None, 111, 111, m, n, k, m, k, m) == \
        max(p.gemm_workspace(v, 111, 111, m, n, k, m, k, m) for v in p.variants()) == \
        8 * (k * m + n * k + n * m)
    p = planner.Planner("syrk")
    assert p.syrk_workspace(None, 122, 111, n, k, n, n) == \
        max(p.syrk_workspace(v, 122, 111, n, k, n, n) for v in p.variants()) == 8 * (k * n + n * n)
    p = planner.Planner("trsm")
    assert p.trsm_workspace(None, 141, 122, 111, 131, m, n, m, m) == \
        max(p.trsm_workspace(v, 141, 122, 111, 131, m, n, m, m) for v in p.variants()) == \
        8 * (m * m + n * m)
    assert planner.Planner("gemm").syrk_workspace(None, 122, 111, n, k, n, n) < 0   # wrong method
