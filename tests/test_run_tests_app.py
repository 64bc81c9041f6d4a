"""The JSON-driven driver (rtatblas_amd/bin/run_tests, the counterpart of the reference's
src/app/run_tests.cpp) on the shipped input files for the benchmark configurations
(rtatblas_amd/host/app/configs) and on reduced copies of them."""
import glob
import json
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "rtatblas_amd", "bin", "run_tests")
CONFIGS = sorted(glob.glob(os.path.join(ROOT, "rtatblas_amd", "host", "app", "configs", "*.json")))


def test_shipped_inputs_are_well_formed():
    assert len(CONFIGS) == 5
    for path in CONFIGS:
        doc = json.load(open(path))
        kw = doc["keywords"]
        assert kw["run_type"] in ("exhaustive", "autotune")
        assert kw["method"] in ("gemm", "gemm_pad", "gemm_tile", "syrk", "trsm")
        assert kw["data_type"] in ("double", "float") and kw["repetitions"] >= 1
        assert doc["problems"]


def run(doc, tmp_path):
    path = tmp_path / "in.json"
    path.write_text(json.dumps(doc))
    proc = subprocess.run([BIN, str(path)], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return json.loads(proc.stdout)


@pytest.mark.gpu
def test_c1_through_the_plan(tmp_path):
    doc = json.load(open([p for p in CONFIGS if "c1_" in p][0]))
    out = run(doc, tmp_path)
    assert out["keywords"] == doc["keywords"]
    (report,) = out["problems"]
    assert report["key"] == {k: doc["problems"][0][k] for k in ("transA", "transB", "m", "n", "k")}
    options = report["options"]
    assert len(options) == 64                                   # every pad variant was tried
    counts = sorted(len(o["times"]) for o in options)
    assert counts[0] == 3 and sum(counts) == 200                # 3 samples each, the rest on the plan
    assert all(t > 0 for o in options for t in o["times"])


@pytest.mark.gpu
@pytest.mark.parametrize("name,shrink", [
    ("c2_", {"m": 768, "n": 768, "k": 768}), ("c3_", {"m": 1007, "n": 409, "k": 615}),
    ("c4_", {"n": 1024, "k": 256}), ("c5_", {"m": 1024, "n": 1024})])
def test_reduced_configs_exhaustive(tmp_path, name, shrink):
    doc = json.load(open([p for p in CONFIGS if name in p][0]))
    doc["problems"] = [dict(doc["problems"][0], **shrink)]
    doc["keywords"]["repetitions"] = 2
    out = run(doc, tmp_path)
    (report,) = out["problems"]
    variants = {"gemm": 8, "gemm_pad": 64, "syrk": 4, "trsm": 4}[doc["keywords"]["method"]]
    assert len(report["options"]) == variants
    assert all(len(o["times"]) == 2 and min(o["times"]) > 0 for o in report["options"])


@pytest.mark.gpu
@pytest.mark.parametrize("name,method,variants,shrink", [
    ("c2_", "gemm_fused", 8, {"m": 768, "n": 768, "k": 768}),
    ("c4_", "syrk_fused", 4, {"n": 1024, "k": 256}),
    ("c5_", "trsm_fused", 4, {"m": 1024, "n": 1024})])
def test_fused_families_through_the_driver(tmp_path, name, method, variants, shrink):
    """The same inputs with the method switched to the family that spells the fused forms: the
    fused form is the plain call, so the driver enumerates the reference's variants."""
    doc = json.load(open([p for p in CONFIGS if name in p][0]))
    doc["problems"] = [dict(doc["problems"][0], **shrink)]
    doc["keywords"]["method"] = method
    doc["keywords"]["repetitions"] = 2
    out = run(doc, tmp_path)
    (report,) = out["problems"]
    assert len(report["options"]) == variants
    assert all(len(o["times"]) == 2 and min(o["times"]) > 0 for o in report["options"])


@pytest.mark.gpu
@pytest.mark.parametrize("name,method,pattern,variants,shrink", [
    ("c3_", "gemm_pad_tile", "NNN???/*/*", 120, {"m": 1007, "n": 409, "k": 615}),
    ("c4_", "syrk_tile", None, 60, {"n": 1024, "k": 512}),
    ("c5_", "trsm_tile", "FF/*/*/*", 45, {"m": 1536, "n": 512})])
def test_kernel_option_families_through_the_driver(tmp_path, name, method, pattern, variants,
                                                   shrink):
    """The benchmark inputs through the families that add tile shape, tail mode and panel
    height to the reference's switches, exhaustively under the input file's filter."""
    doc = json.load(open([p for p in CONFIGS if name in p][0]))
    doc["problems"] = [dict(doc["problems"][0], **shrink)]
    doc["keywords"]["method"] = method
    doc["keywords"]["repetitions"] = 2
    if pattern:
        doc["keywords"]["filter"] = pattern
    out = run(doc, tmp_path)
    (report,) = out["problems"]
    assert len(report["options"]) == variants
    assert all(set(o["option"]) >= {"tile", "tail"} for o in report["options"])
    assert all(len(o["times"]) == 2 and min(o["times"]) > 0 for o in report["options"])
