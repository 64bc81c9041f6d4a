"""The plan-file vocabulary against the fixtures in tests/golden/plan_vocabulary.json (the key
and variant documents the reference's tests/json_test.cpp round-trips): every document must
decode and encode back unchanged through the planner C ABI, and plans load from a statistics
report in the reference's format.  No GPU involved."""
import json
import os

import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "plan_vocabulary.json")


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def canon(entries):
    return sorted(json.dumps(e, sort_keys=True) for e in entries)


@pytest.mark.parametrize("method", ["gemm", "gemm_pad", "syrk", "trsm", "gemm_tile",
                                    "gemm_pad_tile", "syrk_tile", "trsm_tile"])
def test_plan_documents_round_trip(golden, method):
    from rtatblas_amd import planner
    p = planner.Planner(method)
    assert p.plans() == []
    assert p.load_plans(golden[method]) == len(golden[method])
    assert canon(p.plans()) == canon(golden[method])
    # loading the planner's own output again changes nothing
    q = planner.Planner(method)
    q.load_plans(p.plans())
    assert canon(q.plans()) == canon(golden[method])


def test_plan_from_a_statistics_report(golden):
    from rtatblas_amd import planner
    p = planner.Planner("gemm")
    assert p.load_plans(golden["gemm_statistics"]) == 1
    plans = p.plans()
    assert plans[0]["key"] == golden["gemm_statistics"][0]["key"]
    assert plans[0]["plan"] == golden["gemm_statistics_expected_plan"]


def test_malformed_documents_are_refused(golden):
    from rtatblas_amd import planner
    p = planner.Planner("syrk")
    bad = [{"key": {"uplo": "Sideways", "trans": "N", "n": 1, "k": 1},
            "plan": {"transA": "T", "transC": "F"}}]
    with pytest.raises(Exception):
        p.load_plans(bad)
    with pytest.raises(Exception):
        p.load_plans(golden["trsm"])      # TRSM keys are not SYRK keys
    q = planner.Planner("trsm_tile")
    for field, value in (("tile", "96x96"), ("tail", "sometimes"), ("panel", "768")):
        entry = json.loads(json.dumps(golden["trsm_tile"][0]))
        entry["plan"][field] = value
        with pytest.raises(Exception):
            q.load_plans([entry])
    with pytest.raises(Exception):
        q.load_plans(golden["trsm"])      # plans of the plain family lack the kernel options
    assert q.plans() == []
    assert p.plans() == []
