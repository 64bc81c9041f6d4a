"""Writes tests/golden/plan_vocabulary.json: the JSON documents for problem keys and variant
descriptors that the reference's own tests round-trip (tests/json_test.cpp: SYRK key n=6741
k=2463, :11-37; SYRK options, :39-60; TRSM key m=10025 n=4001, :62-104; TRSM options, :106-128;
GEMM key m=500 n=200 k=900, :130-160; GEMM pad options, :162-215), arranged as plan files
([{"key": ..., "plan": ...}]) per method.  The values are typed in from those tests; nothing
of the reference is imported or run.  The sections gemm_tile, gemm_pad_tile, syrk_tile and
trsm_tile have no counterpart in the reference: they pin this library's own plan-file
vocabulary for the kernel options ("tile", "tail", "panel") on the reference's keys.

    python tests/golden/make_plan_fixtures.py
"""
import itertools
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def gemm_keys():
    return [{"transA": a, "transB": b, "m": 500, "n": 200, "k": 900}
            for a, b in itertools.product("NT", "NT")]


def main():
    doc = {}
    # every GEMM variant against the reference's GEMM key, cycling through its four op pairs
    plain = [{"transA": a, "transB": b, "transC": c} for a, b, c in itertools.product("NT", repeat=3)]
    doc["gemm"] = [{"key": dict(gemm_keys()[i % 4], k=900 + i), "plan": p}
                   for i, p in enumerate(plain)]
    pad = [{"transA": a, "transB": b, "transC": c, "padA": pa, "padB": pb, "padC": pc}
           for a, b, c, pa, pb, pc in itertools.product("NT", "NT", "NT", "NP", "NP", "NP")]
    doc["gemm_pad"] = [{"key": dict(gemm_keys()[i % 4], k=900 + i), "plan": p}
                       for i, p in enumerate(pad)]
    syrk_opts = [{"transA": a, "transC": c} for a, c in itertools.product("TF", "TF")]
    doc["syrk"] = [{"key": {"uplo": u, "trans": t, "n": 6741, "k": 2463}, "plan": syrk_opts[i]}
                   for i, (u, t) in enumerate(itertools.product(["Lower", "Upper"], "NT"))]
    trsm_opts = [{"swap_side": s, "transA": a} for a, s in itertools.product("TF", "TF")]
    doc["trsm"] = [{"key": {"side": s, "uplo": u, "trans": t, "diag": d, "m": 10025, "n": 4001},
                    "plan": trsm_opts[i % 4]}
                   for i, (s, u, t, d) in enumerate(itertools.product(
                       ["Left", "Right"], ["Lower", "Upper"], "NT", ["Unit", "Non-Unit"]))]
    tiles = ["auto", "256x128", "128x128", "128x64", "64x64"]
    tails = ["auto", "whole", "split"]
    panels = ["auto", "512", "1024"]
    doc["gemm_tile"] = [{"key": dict(gemm_keys()[i % 4], k=900 + i), "plan": dict(plain[i % 8], tile=t)}
                        for i, t in enumerate(tiles * 2)]
    doc["gemm_pad_tile"] = [{"key": dict(gemm_keys()[i % 4], k=900 + i),
                             "plan": dict(pad[(7 * i) % 64], tile=t, tail=tl)}
                            for i, (t, tl) in enumerate(itertools.product(tiles, tails))]
    doc["syrk_tile"] = [{"key": {"uplo": ["Lower", "Upper"][i % 2], "trans": "NT"[i // 2 % 2],
                                 "n": 6741 + i, "k": 2463},
                         "plan": dict(syrk_opts[i % 4], tile=t, tail=tl)}
                        for i, (t, tl) in enumerate(itertools.product(tiles, tails))]
    doc["trsm_tile"] = [{"key": {"side": ["Left", "Right"][i % 2], "uplo": ["Lower", "Upper"][i // 2 % 2],
                                 "trans": "NT"[i // 4 % 2], "diag": ["Unit", "Non-Unit"][i // 8 % 2],
                                 "m": 10025 + i, "n": 4001},
                         "plan": dict(trsm_opts[i % 4], tile=t, tail=tl, panel=pn)}
                        for i, (t, tl, pn) in enumerate(itertools.product(tiles, tails, panels))]
    # a statistics report in the reference's format (planner_statistics.h:50-67): the plan
    # loaded from it is the variant with the smallest median
    doc["gemm_statistics"] = [{
        "key": {"transA": "T", "transB": "N", "m": 500, "n": 200, "k": 900},
        "options": [
            {"option": {"transA": "N", "transB": "N", "transC": "N"}, "times": [9.0, 2.0, 2.5]},
            {"option": {"transA": "T", "transB": "N", "transC": "N"}, "times": [1.5, 1.75, 8.0]},
            {"option": {"transA": "N", "transB": "N", "transC": "T"}, "times": [3.0, 3.0, 3.0]},
        ]}]
    doc["gemm_statistics_expected_plan"] = {"transA": "T", "transB": "N", "transC": "N"}
    with open(os.path.join(HERE, "plan_vocabulary.json"), "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
        f.write("\n")


if __name__ == "__main__":
    main()
