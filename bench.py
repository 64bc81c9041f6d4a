#!/usr/bin/env python3
"""Benchmark of the rtat execution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

Workload (the configuration the headline metric is quoted on): DGEMM C = alpha*A^T*B + beta*C,
M = N = K = 8192, fp64, opA = T, opB = N, alpha = 1, beta = 0.5, iid uniform[-1,1) operands from
the seeded generator, column-major, ld = rows.  One step = one pass of that call through the
C ABI (rtat_dgemm) with operands already resident in HBM.  Prints ONE JSON line on stdout;
everything else goes to stderr.

Besides the headline value the line carries
  roofline      fp64 MFMA roofline of the DGEMM kernel: algorithmic flop (2 n^3) per launch over
                the launch duration measured with events on the handle's stream;
  cpu_baseline  the same DGEMM on the host cores through the CPU oracle's CBLAS backend
                (OpenBLAS), timed in this run, core count stated; entries `dsyrk` and `dtrsm`
                carry the same for the DSYRK and DTRSM configurations;
  ops           the other rows of the hot path at their config sizes: DSYRK (N=8192, K=2048),
                DTRSM (M=N=8192), the awkward-shape DGEMMs, transpose / pad-copy / accumulate
                as TFLOP/s or GB/s with their roofline fractions; bandwidth rows also carry
                their fraction of what a plain streaming copy kernel reaches in this run
                (`hbm_streaming`: rtat_hbm_probe read / write / copy over 512 MiB);
  autotune      every benchmark configuration through the planner (Planning_System over the
                variant trees): the headline DGEMM (`gemm` and `gemm_tile` families), 512^3
                (`gemm_pad`), both awkward shapes (`gemm_pad_tile`: pad-copy variants against
                the masked-edge kernel under every tile shape and tail mode), DSYRK
                (`syrk_tile`) and DTRSM (`trsm_tile`: tile shape, tail mode, panel height); every
                admitted variant timed, then the committed plan head to head against the best
                fixed variants;
  reference     when oracle/_ref/librtat_ref.so is present: the reference's own executors on
                hipBLAS on the same operands, for comparison.

`--kernels-only` runs three launches each of the DGEMM, a pad copy and a transpose (then of the
DSYRK and the DTRSM) and `--hbm-probe-only` twenty launches each of the plain streaming read /
write / copy kernels; both print nothing but a short JSON: the targets of the rocprofv3 runs
behind profiles/.
"""
import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP64_MFMA = 78.6e12   # MI355X datasheet, dense fp64 matrix
PEAK_FP32_MFMA = 157.3e12  # MI355X datasheet, dense fp32 matrix
PEAK_HBM = 8.0e12          # MI355X datasheet, HBM3E
# HBM bytes per launch come from rocprofv3 counter runs whose summaries are tracked under
# profiles/; the lines "traffic_bytes_per_launch <key> = <bytes>" of this file are read at run time.
TRAFFIC_FILE = os.path.join("profiles", "hbm_traffic_per_launch.md")
N_OP, T_OP = 111, 112
LOWER, LEFT, NON_UNIT = 122, 141, 131


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def event_times(torch, stream, fn, reps, warmup):
    """Per-call durations in ms, measured by event pairs recorded on `stream`.  Calls shorter
    than 5 ms are timed in back-to-back batches of about 10 ms (one event pair per batch), so
    that the device does not fall idle between two samples and the per-call figure is the
    steady-state one, as the headline's K back-to-back steps are (a 1.9 ms call timed one at a
    time, with the host synchronising in between, reads 3 % slower); longer calls get one
    event pair each."""
    def timed(count):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(count):
            fn()
        e1.record(stream)
        e1.synchronize()
        return e0.elapsed_time(e1) / count

    for _ in range(warmup):
        fn()
    stream.synchronize()
    probe = timed(1)
    batch = 1 if probe >= 5.0 else max(1, min(200, int(10.0 / max(probe, 1e-3))))
    if batch > 1:
        timed(batch)                      # bring the clocks up before the first kept sample
    return [timed(batch) for _ in range(reps)]


def measured_traffic():
    """{key: bytes per launch} from the tracked profile summary; empty if the file is absent."""
    out = {}
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 4 and parts[0] == "traffic_bytes_per_launch" and parts[2] == "=":
                    out[parts[1]] = float(parts[3])
                if len(parts) == 3 and parts[0] == "measured_on_commit" and parts[1] == "=":
                    out["measured_on_commit"] = parts[2]
    except OSError:
        pass
    return out


def median(xs):
    s = sorted(xs)
    return s[len(s) // 2]


def cpu_baseline(n, reps):
    """Host CBLAS DGEMM, DSYRK and DTRSM (same ops, same generator) through the oracle; returns
    the JSON object: the DGEMM figure at top level, `dsyrk` and `dtrsm` beside it."""
    import numpy as np
    from oracle import oracle_py as orc
    threads, name = orc.cblas_on()
    kind_note = "OpenBLAS cblas_%s via the CPU oracle" if threads else "oracle loops (no CBLAS found), %s"
    cores = max(threads, 1)
    lib = os.path.basename(name)
    if not threads:
        n = min(n, 512)

    def best_of(fn):
        fn()  # warm-up
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return min(ts)

    A, B, C = orc.fill(n, n, seed=1), orc.fill(n, n, seed=2), orc.fill(n, n, seed=3)
    best = best_of(lambda: orc.dgemm(T_OP, N_OP, n, n, n, 1.0, A, B, 0.5, C))
    out = {"value": 2.0 * n ** 3 / best / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
           "sample": "%s, DGEMM opA=T opB=N n=%d alpha=1 beta=0.5, 1 warm-up + %d timed runs, "
                     "best %.3f s (%s)" % (kind_note % "dgemm", n, reps, best, lib)}
    del B
    # DSYRK lower / N, N = n, K = n / 4, alpha = beta = 1 (the config: 8192 / 2048).
    ks = max(n // 4, 1)
    As = orc.fill(n, ks, seed=1)
    Cs = orc.fill(n, n, seed=3, kind=1)
    best = best_of(lambda: orc.dsyrk(LOWER, N_OP, n, ks, 1.0, As, 1.0, Cs))
    out["dsyrk"] = {"value": n * (n + 1.0) * ks / best / 1e12, "unit": "TFLOP/s", "cores": cores,
                    "kind": "port",
                    "sample": "%s, DSYRK lower N n=%d k=%d alpha=1 beta=1, 1 warm-up + %d timed "
                              "runs, best %.3f s (%s)" % (kind_note % "dsyrk", n, ks, reps, best, lib)}
    del As, Cs
    # DTRSM left / lower / N / non-unit, M = N = n, well-conditioned triangle, alpha = 1.  The
    # solve is in place: B is restored from a copy before each run, outside the clock.
    L = orc.fill(n, n, seed=1, kind=4)
    B0 = orc.fill(n, n, seed=2)
    X = B0.copy(order="F")
    ts = []
    for it in range(reps + 1):
        np.copyto(X, B0)
        t0 = time.perf_counter()
        orc.dtrsm(LEFT, LOWER, N_OP, NON_UNIT, n, n, 1.0, L, X)
        if it:
            ts.append(time.perf_counter() - t0)
    best = min(ts)
    out["dtrsm"] = {"value": float(n) ** 3 / best / 1e12, "unit": "TFLOP/s", "cores": cores,
                    "kind": "port",
                    "sample": "%s, DTRSM left lower N non-unit m=n=%d alpha=1, 1 warm-up + %d timed "
                              "runs, best %.3f s (%s)" % (kind_note % "dtrsm", n, reps, best, lib)}
    orc.cblas_off()
    return out


def plan_check(stream, method, run, spell, admitted, pattern=None):
    """One routine through the planner.  Three passes: (1) every admitted variant a few times
    as a fixed variant; (2) a fresh planner explores (3 samples each, a run-off among the close
    ones) until it commits a plan; (3) the plan, the default variant and the fastest fixed
    variants of pass 1 head to head, interleaved round by round so that clock drift hits them
    alike.  The committed plan must be no slower than the best of them: <= 1.005 x its median
    plus 1 us (the resolution of an event pair around a single call).  run(planner, variant)
    performs one call (variant None = the planner's own plan) and returns the variant that ran;
    spell(option) turns a variant document into that name; admitted(planner) lists the names
    the planner may try."""
    from rtatblas_amd import planner

    def make():
        p = planner.Planner(method)
        if pattern:
            p.set_filter(pattern)
        return p

    def medians(p, skip):
        return {spell(o["option"]): median(o["times"][skip:]) for o in p.stats()[0]["options"]
                if len(o["times"]) > skip}

    warm = make()                         # a throw-away pass: the first variant timed must not
    names = admitted(warm)                # be the one that meets an idle GPU
    for _ in range(3):
        run(warm, names[0])
    stream.synchronize()
    fixed = make()
    for v in names:
        for _ in range(3):
            run(fixed, v)
    stream.synchronize()
    med = medians(fixed, 1)
    tuned = make()
    chosen = None
    calls = 0
    while not tuned.plans() and calls < len(names) * 12:   # explore (3 samples each + the run-off)
        for _ in range(len(names)):
            chosen = run(tuned, None)
        calls += len(names)
    chosen = run(tuned, None)
    stream.synchronize()
    # head to head: the plan against the default and the five fastest fixed variants of pass 1
    rivals = sorted(med, key=med.get)[:5]
    for v in (names[0], chosen):
        if v not in rivals:
            rivals.append(v)
    duel = make()
    # Rounds: the medians of one and the same launch under two names still differ by chance -
    # five spellings of DSYRK 8192/2048 that all make the same two launches, 38 samples each:
    # 1.8825 ... 1.8871 ms, 0.25 % end to end; with 15 samples 0.6 % was seen - and the bar below
    # is 0.5 %.  Short calls scatter more and cost less: more rounds.
    rounds = 40 if med[names[0]] >= 1.0 else 60
    shuffle = random.Random(20240229).shuffle
    for r in range(rounds):
        # every round in another order (seeded shuffles): what a variant leaves in the caches,
        # and the clock it leaves the GPU at, is felt by the next.  Identical launches under two
        # names measured 0.7 % apart in a fixed order, and still 0.5 % apart over 40 rounds of
        # one rotated and reversed order, in which a variant only ever follows its two
        # neighbours in the list (a variant that first transposes an operand, say).
        order = list(rivals)
        shuffle(order)
        for v in order:
            run(duel, v)
    stream.synchronize()
    head = medians(duel, 1)
    best = min(head, key=head.get)
    # the same comparison round by round (both ran within a few calls of each other, so drift
    # cancels): the median over the rounds of plan time / best fixed variant's time
    per_round = {spell(o["option"]): o["times"] for o in duel.stats()[0]["options"]}
    paired = median([a / b for a, b in zip(per_round[chosen][1:], per_round[best][1:])])
    out = {"method": method, "filter": pattern, "variants": len(names), "plan": chosen,
           "plan_ms": head[chosen], "best_fixed": best, "best_fixed_ms": head[best],
           "default": names[0], "default_ms": head[names[0]],
           "plan_over_best_fixed": head[chosen] / head[best],
           "plan_over_best_fixed_round_by_round": paired,
           "calls_until_committed": calls, "head_to_head_rounds": rounds, "head_to_head_ms": head,
           "plan_not_slower_than_best_fixed": head[chosen] <= head[best] * 1.005 + 0.001}
    if len(med) <= 16:
        out["fixed_variant_ms"] = med
    else:  # the fastest and the slowest of a large family
        order = sorted(med, key=med.get)
        out["fixed_variant_ms"] = {k: med[k] for k in order[:6] + order[-2:]}
    return out


def spell_gemm(o):
    return o["transA"] + o["transB"] + o["transC"]


def spell_gemm_pad(o):
    return spell_gemm(o) + o["padA"] + o["padB"] + o["padC"]


def spell_gemm_tile(o):
    return spell_gemm(o) + "/" + o["tile"]


def spell_gemm_pad_tile(o):
    return spell_gemm_pad(o) + "/" + o["tile"] + "/" + o["tail"]


def autotune_check(torch, stream, h, n, A, B, Cm):
    """Every benchmark configuration through its planner."""
    from rtatblas_amd import native, planner

    def gemm_case(method, spell, ta, tb, m, nn, k, lda, ldb, ldc, alpha, beta, Ad, Bd, Cd,
                  pattern=None):
        need = planner.Planner(method).gemm_workspace(None, ta, tb, m, nn, k, lda, ldb, ldc)
        ws = torch.empty(need // 8 + 1, dtype=torch.float64, device="cuda")
        res = plan_check(
            stream, method,
            lambda p, v: p.gemm(h, v, ta, tb, m, nn, k, alpha, Ad, lda, Bd, ldb, beta, Cd, ldc, ws,
                                need),
            spell, lambda p: p.gemm_admitted(ta, tb, m, nn, k), pattern)
        res["workspace_bytes"] = need
        return res

    # C2 at the headline size: the reference's eight transpose trees (an explicit transpose + NN
    # kernel against the direct TN kernel), then the same jointly with the tile shape.
    out = gemm_case("gemm", spell_gemm, T_OP, N_OP, n, n, n, n, n, n, 1.0, 0.5, A, B, Cm)
    out["dgemm_tn_n%d_gemm_tile" % n] = gemm_case("gemm_tile", spell_gemm_tile, T_OP, N_OP, n, n,
                                                  n, n, n, n, 1.0, 0.5, A, B, Cm)
    # C1: 512^3 NN, alpha 1, beta 0, ld = 512, transpose and pad variants enumerated.
    c1 = 512
    out["dgemm_nn_512_gemm_pad"] = gemm_case("gemm_pad", spell_gemm_pad, N_OP, N_OP, c1, c1, c1, c1,
                                             c1, c1, 1.0, 0.0, A, B, Cm)
    # C3: the awkward shapes, NN, ld = rows + 3: pad-copy variants against the masked-edge
    # kernel, jointly with tile shape and tail mode (the explicit transposes filtered out:
    # 8 x 5 x 3 = 120 of the family's 960 variants).
    for (mm, nn, kk) in [(10007, 4099, 6151), (65536, 256, 256)]:
        Aa = torch.empty((mm + 3) * kk, dtype=torch.float64, device="cuda")
        Ba = torch.empty((kk + 3) * nn, dtype=torch.float64, device="cuda")
        Ca = torch.empty((mm + 3) * nn, dtype=torch.float64, device="cuda")
        h.dfill(Aa, mm, kk, mm + 3, 1)
        h.dfill(Ba, kk, nn, kk + 3, 2)
        h.dfill(Ca, mm, nn, mm + 3, 3)
        out["dgemm_nn_%dx%dx%d_ld+3_gemm_pad_tile" % (mm, nn, kk)] = gemm_case(
            "gemm_pad_tile", spell_gemm_pad_tile, N_OP, N_OP, mm, nn, kk, mm + 3, kk + 3, mm + 3,
            1.0, 0.0, Aa, Ba, Ca, pattern="NNN???/*/*")
        del Aa, Ba, Ca

    # C4: the reference's [tA][tC] switches jointly with tile shape and tail mode (60 variants).
    ns, ks = 8192, 2048
    As = torch.empty(ns * ks, dtype=torch.float64, device="cuda")
    Cs = torch.empty(ns * ns, dtype=torch.float64, device="cuda")
    h.dfill(As, ns, ks, ns, 1)
    h.dfill(Cs, ns, ns, ns, 3, native.FILL_SYMMETRIC)
    need = planner.Planner("syrk_tile").syrk_workspace(None, LOWER, N_OP, ns, ks, ns, ns)
    ws = torch.empty(need // 8 + 1, dtype=torch.float64, device="cuda")
    out["dsyrk_lower_n8192_k2048_syrk_tile"] = plan_check(
        stream, "syrk_tile",
        lambda p, v: p.syrk(h, v, LOWER, N_OP, ns, ks, 1.0, As, ns, 1.0, Cs, ns, ws, need),
        lambda o: o["transA"] + o["transC"] + "/" + o["tile"] + "/" + o["tail"],
        lambda p: p.syrk_admitted(LOWER, N_OP, ns, ks))
    del ws, As

    # C5: [swap][tA] jointly with tile shape, tail mode and panel height; the side swap (a
    # transposing copy of B there and back) filtered out: 2 x 5 x 3 x 3 = 90 of 180 variants.
    m = 8192
    L = torch.empty(m * m, dtype=torch.float64, device="cuda")
    h.dfill(L, m, m, m, 1, native.FILL_TRI_FULL)
    h.dfill(Cs, m, m, m, 2)
    need = planner.Planner("trsm_tile").trsm_workspace(None, LEFT, LOWER, N_OP, NON_UNIT, m, m, m, m)
    ws = torch.empty(need // 8 + 1, dtype=torch.float64, device="cuda")
    out["dtrsm_left_lower_n8192_trsm_tile"] = plan_check(
        stream, "trsm_tile",
        lambda p, v: p.trsm(h, v, LEFT, LOWER, N_OP, NON_UNIT, m, m, 1.0, L, m, Cs, m, ws, need),
        lambda o: o["swap_side"] + o["transA"] + "/" + o["tile"] + "/" + o["tail"] + "/" + o["panel"],
        lambda p: p.trsm_admitted(LEFT, LOWER, N_OP, NON_UNIT, m, m), pattern="F?/*/*/*")
    del ws, L, Cs
    out["all_plans_not_slower_than_best_fixed"] = all(
        v["plan_not_slower_than_best_fixed"] for v in [out] + [x for x in out.values()
                                                               if isinstance(x, dict) and "plan" in x])
    return out


def reference_timings(torch, stream, h, n, A, B, Cm):
    """The reference's own executors on hipBLAS (oracle/_ref), same operands; None if absent."""
    try:
        from oracle import ref_py
        if not ref_py.available():
            return None
        ref_py.load()
    except Exception as e:
        log("reference library unavailable:", repr(e))
        return None
    raw = stream.cuda_stream
    out = {"what": "csnowdon2/rtatblas executors compiled from the reference sources, on hipBLAS"}
    ts = event_times(torch, stream, lambda: ref_py.gemm("NNN", T_OP, N_OP, n, n, n, 1.0, A, n, B, n,
                                                        0.5, Cm, n, None, 0, raw), 10, 2)
    out["dgemm_tn_n%d" % n] = {"ms": median(ts), "TFLOP/s": 2.0 * n ** 3 / (median(ts) * 1e-3) / 1e12}
    ns, ks = 8192, 2048
    As = torch.empty(ns * ks, dtype=torch.float64, device="cuda")
    Cs = torch.empty(ns * ns, dtype=torch.float64, device="cuda")
    h.dfill(As, ns, ks, ns, 1)
    h.dfill(Cs, ns, ns, ns, 3, 1)
    ts = event_times(torch, stream, lambda: ref_py.syrk("FF", LOWER, N_OP, ns, ks, 1.0, As, ns, 1.0,
                                                        Cs, ns, None, 0, raw), 10, 2)
    out["dsyrk_lower_n8192_k2048"] = {"ms": median(ts),
                                     "TFLOP/s": ns * (ns + 1.0) * ks / (median(ts) * 1e-3) / 1e12}
    del As
    m = 8192
    L = torch.empty(m * m, dtype=torch.float64, device="cuda")
    B0 = torch.empty_like(L)
    h.dfill(L, m, m, m, 1, 4)
    h.dfill(B0, m, m, m, 2)

    def solve():
        Cs.copy_(B0)
        ref_py.trsm("FF", LEFT, LOWER, N_OP, NON_UNIT, m, m, 1.0, L, m, Cs, m, None, 0, raw)

    t_ms = median(event_times(torch, stream, solve, 5, 1)) - median(
        event_times(torch, stream, lambda: Cs.copy_(B0), 5, 1))
    out["dtrsm_left_lower_n8192"] = {"ms": t_ms, "TFLOP/s": float(m) ** 3 / (t_ms * 1e-3) / 1e12}
    ts = event_times(torch, stream, lambda: ref_py.geam(T_OP, N_OP, m, m, 1.0, L, m, 0.0, Cs, m, Cs,
                                                        m, raw), 20, 3)
    out["transpose_8192"] = {"ms": median(ts), "GB/s": 2.0 * m * m * 8 / (median(ts) * 1e-3) / 1e9}
    return out


def hipblas_sweep(h, stream):
    """The four entry points against hipBLAS (what the reference computes with) on the same
    device buffers, event-timed in batches; one JSON line with a row per shape.  Not part of
    the default run: `python bench.py --hipblas-sweep`."""
    import ctypes as C
    import torch
    from rtatblas_amd import native
    hb = C.CDLL("libhipblas.so")
    hh = C.c_void_p()
    if hb.hipblasCreate(C.byref(hh)) != 0:
        raise RuntimeError("hipblasCreate failed")
    hb.hipblasSetStream(hh, C.c_void_p(stream.cuda_stream))

    def ptr(t):
        return C.c_void_p(t.data_ptr())

    def per_call(fn):
        return sorted(event_times(torch, stream, fn, 5, 2))[2]       # median, ms per call

    def dev(elems, seed, m, n, ld, kind=native.FILL_IID):
        t = torch.empty(elems, dtype=torch.float64, device="cuda")
        h.dfill(t, m, n, ld, seed, kind)
        return t

    rows = []
    one, zero, half = C.c_double(1.0), C.c_double(0.0), C.c_double(0.5)

    def add(op, shape, ours, theirs, unit_work, unit):
        rows.append({"op": op, "shape": shape, "ours_us": round(ours * 1e3, 2),
                     "hipblas_us": round(theirs * 1e3, 2),
                     "hipblas_over_ours": round(theirs / ours, 3),
                     "ours_" + unit: round(unit_work / (ours * 1e-3) / 1e12, 3)})

    with torch.cuda.stream(stream):
        for (ta, tb, m, n, k, pad) in (
                [(N_OP, N_OP, s, s, s, 0) for s in (256, 512, 1024, 2048, 4096)] +
                [(T_OP, N_OP, s, s, s, 0) for s in (256, 512, 1024, 2048, 4096, 8192)] +
                [(N_OP, T_OP, s, s, s, 0) for s in (512, 768, 2048)] +
                [(N_OP, N_OP, 200, 300, 400, 0), (N_OP, N_OP, 1000, 1000, 1000, 0),
                 (N_OP, N_OP, 8192, 8192, 128, 0), (N_OP, N_OP, 8192, 8192, 512, 0),
                 (N_OP, N_OP, 8192, 512, 8192, 0), (N_OP, N_OP, 512, 512, 8192, 0),
                 (N_OP, N_OP, 64, 8192, 8192, 0), (N_OP, N_OP, 10007, 4099, 6151, 3),
                 (N_OP, N_OP, 65536, 256, 256, 3), (T_OP, N_OP, 5000, 5000, 5000, 0)]):
            ar, ac = (k, m) if ta == T_OP else (m, k)
            br, bc = (n, k) if tb == T_OP else (k, n)
            lda, ldb, ldc = ar + pad, br + pad, m + pad
            A, B = dev(lda * ac, 1, ar, ac, lda), dev(ldb * bc, 2, br, bc, ldb)
            Cm = dev(ldc * n, 3, m, n, ldc)
            flop = 2.0 * m * n * k
            ours = per_call(lambda: h.dgemm(ta, tb, m, n, k, 1.0, A, lda, B, ldb, 0.0, Cm, ldc))
            theirs = per_call(lambda: hb.hipblasDgemm(hh, ta, tb, m, n, k, C.byref(one), ptr(A),
                                                      lda, ptr(B), ldb, C.byref(zero), ptr(Cm),
                                                      ldc))
            add("dgemm_%s%s" % ("nt"[ta == T_OP], "nt"[tb == T_OP]),
                "%dx%dx%d%s" % (m, n, k, "_ld+3" if pad else ""), ours, theirs, flop, "TFLOP/s")
            del A, B, Cm
        for (n, k) in [(512, 256), (1024, 512), (2048, 2048), (4096, 512), (8192, 2048)]:
            A, Cm = dev(n * k, 1, n, k, n), dev(n * n, 2, n, n, n)
            flop = float(n) * (n + 1) * k
            ours = per_call(lambda: h.dsyrk(LOWER, N_OP, n, k, 1.0, A, n, 1.0, Cm, n))
            theirs = per_call(lambda: hb.hipblasDsyrk(hh, LOWER, N_OP, n, k, C.byref(one), ptr(A),
                                                      n, C.byref(one), ptr(Cm), n))
            add("dsyrk_lower_n", "%d/%d" % (n, k), ours, theirs, flop, "TFLOP/s")
            del A, Cm
        for (m, n) in [(512, 512), (2048, 2048), (4096, 4096), (8192, 256), (8192, 8192)]:
            A = dev(m * m, 1, m, m, m, native.FILL_TRI_FULL)
            B0 = dev(m * n, 2, m, n, m)
            B = B0.clone()
            flop = float(m) * m * n
            restore = per_call(lambda: B.copy_(B0))

            def ours_fn():
                B.copy_(B0)
                h.dtrsm(LEFT, LOWER, N_OP, NON_UNIT, m, n, 1.0, A, m, B, m)

            def theirs_fn():
                B.copy_(B0)
                hb.hipblasDtrsm(hh, LEFT, LOWER, N_OP, NON_UNIT, m, n, C.byref(one), ptr(A), m,
                                ptr(B), m)

            ours = per_call(ours_fn) - restore
            theirs = per_call(theirs_fn) - restore
            add("dtrsm_left_lower_n", "%dx%d" % (m, n), ours, theirs, flop, "TFLOP/s")
            del A, B, B0
        for (ta, m, n, pad, beta) in [(T_OP, 8192, 8192, 0, 0.0), (T_OP, 8192, 8192, 3, 0.0),
                                     (T_OP, 8192, 8192, 0, 0.5), (N_OP, 8192, 8192, 0, 0.0),
                                     (T_OP, 256, 65536, 3, 0.0), (T_OP, 100, 100000, 0, 0.0),
                                     (T_OP, 6151, 10007, 3, 0.0), (N_OP, 10007, 6151, 3, 0.0),
                                     (T_OP, 2048, 2048, 0, 0.0)]:
            ar, ac = (n, m) if ta == T_OP else (m, n)
            lda, ldc = ar + pad, m + pad
            A, Cm = dev(lda * ac, 1, ar, ac, lda), dev(ldc * n, 2, m, n, ldc)
            byts = (3.0 if beta else 2.0) * m * n * 8
            be = half if beta else zero
            ours = per_call(lambda: h.dgeam(ta, N_OP, m, n, 1.0, A, lda, beta, Cm, ldc, Cm, ldc))
            theirs = per_call(lambda: hb.hipblasDgeam(hh, ta, N_OP, m, n, C.byref(one), ptr(A),
                                                      lda, C.byref(be), ptr(Cm), ldc, ptr(Cm),
                                                      ldc))
            add("dgeam_%s%s" % ("nt"[ta == T_OP], "_acc" if beta else ""),
                "%dx%d%s" % (m, n, "_ld+3" if pad else ""), ours, theirs, byts, "TB/s")
            del A, Cm
        stream.synchronize()
    hb.hipblasDestroy(hh)
    behind = [r for r in rows if r["hipblas_over_ours"] < 0.97]
    print(json.dumps({"hipblas_sweep": rows, "rows": len(rows),
                      "rows_behind_hipblas_by_more_than_3_percent": len(behind),
                      "behind": [r["op"] + " " + r["shape"] for r in behind]}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--n", type=int, default=8192, help="DGEMM size (default: the config's 8192)")
    ap.add_argument("--quick", action="store_true", help="skip the per-op table and CPU baseline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--hbm-probe-only", action="store_true",
                    help="20 launches each of the plain read / write / copy streaming kernels over "
                         "512 MiB and nothing else (profiling target)")
    ap.add_argument("--kernels-only", action="store_true",
                    help="a few launches of the main kernels and nothing else (profiling target)")
    ap.add_argument("--hipblas-sweep", action="store_true",
                    help="time the four entry points against hipBLAS over some forty shapes and "
                         "nothing else")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, "
            "no sharding in this path)" % args.gpus)
        sys.exit(2)

    import torch
    from rtatblas_amd import native
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    torch.cuda.set_device(0)
    stream = torch.cuda.Stream()
    h = native.Handle()
    h.set_stream(stream)
    flops_peak_rt, hbm_peak_rt, cus = h.peaks()

    if args.hipblas_sweep:
        hipblas_sweep(h, stream)
        return

    if args.hbm_probe_only:
        pb = 512 << 20
        with torch.cuda.stream(stream):
            P0 = torch.ones(pb // 8, dtype=torch.float64, device="cuda")
            P1 = torch.empty(pb // 8, dtype=torch.float64, device="cuda")
            for kind in (native.PROBE_READ, native.PROBE_WRITE, native.PROBE_COPY):
                for _ in range(20):
                    h.hbm_probe(kind, P0, P1, pb)
            stream.synchronize()
        print(json.dumps({"hbm_probe_only": True, "bytes": pb}), flush=True)
        return

    n = args.n
    with torch.cuda.stream(stream):
        A = torch.empty(n * n, dtype=torch.float64, device="cuda")
        B = torch.empty_like(A)
        Cm = torch.empty_like(A)
        h.dfill(A, n, n, n, 1)
        h.dfill(B, n, n, n, 2)
        h.dfill(Cm, n, n, n, 3)

        def step():
            h.dgemm(T_OP, N_OP, n, n, n, 1.0, A, n, B, n, 0.5, Cm, n)

        if args.kernels_only:
            D = torch.empty(n * (n + 32), dtype=torch.float64, device="cuda")
            # the awkward DGEMM's A (10007 x 6151, ld 10010) transposed into ld = 6151: columns
            # that split cache lines on both sides
            S2 = torch.empty(10010 * 6151, dtype=torch.float64, device="cuda")
            D2 = torch.empty(6151 * 10007, dtype=torch.float64, device="cuda")
            h.dfill(S2, 10007, 6151, 10010, 5)
            for _ in range(3):
                step()
                h.dgeam(N_OP, N_OP, n, n, 1.0, A, n, 0.0, D, n + 32, D, n + 32)
                h.dgeam(T_OP, N_OP, n, n, 1.0, A, n, 0.0, D, n, D, n)
                h.dgeam(T_OP, N_OP, 6151, 10007, 1.0, S2, 10010, 0.0, D2, 6151, D2, 6151)
            # DSYRK (lower, N, n x 2048, alpha = beta = 1) over Cm, and DTRSM (left, lower, N,
            # non-unit) with a well-conditioned triangle in D and B as the right-hand sides.
            h.dfill(D, n, n, n, 1, native.FILL_TRI_LOWER)
            for _ in range(3):
                h.dsyrk(LOWER, N_OP, n, 2048, 1.0, A, n, 1.0, Cm, n)
                h.dtrsm(LEFT, LOWER, N_OP, NON_UNIT, n, n, 1.0, D, n, B, n)
            stream.synchronize()
            print(json.dumps({"kernels_only": True, "n": n}), flush=True)
            return

        # ---- headline: W warm-up steps, then exactly K timed steps between two syncs.
        for _ in range(args.warmup):
            step()
        stream.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        stream.synchronize()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        flop = 2.0 * n ** 3
        value = flop * args.steps / wall / 1e12
        ms_per_step = wall / args.steps * 1e3

        # ---- roofline of the dominant kernel: per-launch duration by events on this stream.
        per_launch = event_times(torch, stream, step, max(5, min(args.steps, 20)), 1)
        avg_ms = sum(per_launch) / len(per_launch)
        achieved = flop / (avg_ms * 1e-3) / 1e12
        traffic = measured_traffic()
        launch = h.last_launch()          # what rtat_dgemm's automatic choice ran this on
        roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_FP64_MFMA / 1e12,
                    "unit": "TFLOP/s", "frac": achieved / (PEAK_FP64_MFMA / 1e12),
                    "traffic": traffic.get("dgemm_tn_n%d" % n),
                    "traffic_source": "%s (rocprofv3 FETCH_SIZE + WRITE_SIZE of an earlier run of "
                                      "this kernel, not of this run; measured on commit %s)"
                                      % (TRAFFIC_FILE, traffic.get("measured_on_commit", "?"))
                                      if "dgemm_tn_n%d" % n in traffic else None,
                    "algorithmic_bytes": (3 + 1) * n * n * 8.0,
                    "kernel": "gemm_kernel<double, %sx16, TN>" % launch["tile"],
                    "launch": launch,
                    "avg_launch_ms": avg_ms, "min_launch_ms": min(per_launch),
                    "peak_runtime_derived": flops_peak_rt / 1e12}

        ops = {}
        hbm = None
        if not args.quick:
            # What a plain streaming kernel gets over 512 MiB in this run: the yardstick of
            # the bandwidth rows below (a copy moves 2 x 512 MiB).
            pb = 512 << 20
            P0 = torch.empty(pb // 8, dtype=torch.float64, device="cuda")
            P1 = torch.empty(pb // 8, dtype=torch.float64, device="cuda")
            P0.fill_(1.0)
            hbm = {"bytes": pb, "what": "rtat_hbm_probe: plain 16-byte non-temporal streaming "
                                        "kernels, median of 20 event-timed launches"}
            for name, kind, moved in (("read", native.PROBE_READ, pb), ("write", native.PROBE_WRITE, pb),
                                      ("copy", native.PROBE_COPY, 2 * pb)):
                ts = event_times(torch, stream, lambda: h.hbm_probe(kind, P0, P1, pb), 20, 3)
                hbm[name + "_GB/s"] = moved / (median(ts) * 1e-3) / 1e9
            hbm["copy_frac_of_peak"] = hbm["copy_GB/s"] / (PEAK_HBM / 1e9)
            del P0, P1

            def bw_row(ms, moved):
                gbs = moved / (ms * 1e-3) / 1e9
                return {"ms": ms, "GB/s": gbs, "frac_of_peak": gbs / (PEAK_HBM / 1e9),
                        "frac_of_streaming_copy": gbs / hbm["copy_GB/s"]}

            # DSYRK lower / N, N = 8192, K = 2048, alpha = beta = 1, C symmetric.
            ns, ks = 8192, 2048
            As = torch.empty(ns * ks, dtype=torch.float64, device="cuda")
            Cs = torch.empty(ns * ns, dtype=torch.float64, device="cuda")
            h.dfill(As, ns, ks, ns, 1)
            h.dfill(Cs, ns, ns, ns, 3, native.FILL_SYMMETRIC)
            ts = event_times(torch, stream,
                             lambda: h.dsyrk(LOWER, N_OP, ns, ks, 1.0, As, ns, 1.0, Cs, ns), 10, 2)
            tf = ns * (ns + 1.0) * ks / (median(ts) * 1e-3) / 1e12
            ops["dsyrk_lower_n8192_k2048"] = {"ms": median(ts), "TFLOP/s": tf,
                                             "frac_of_peak": tf / (PEAK_FP64_MFMA / 1e12),
                                             "traffic": traffic.get("dsyrk_lower_n8192_k2048"),
                                             "algorithmic_bytes": (ns * ks + ns * (ns + 1.0)) * 8.0}
            del As, Cs
            # DTRSM left / lower / N / non-unit, M = N = 8192, alpha = 1 (in place: B is restored
            # from a copy before each solve; the copy is timed alone and subtracted).
            m = 8192
            L = torch.empty(m * m, dtype=torch.float64, device="cuda")
            B0 = torch.empty_like(L)
            X = torch.empty_like(L)
            h.dfill(L, m, m, m, 1, native.FILL_TRI_LOWER)
            h.dfill(B0, m, m, m, 2)

            def solve():
                X.copy_(B0)
                h.dtrsm(LEFT, LOWER, N_OP, NON_UNIT, m, m, 1.0, L, m, X, m)

            ts = event_times(torch, stream, solve, 7, 2)
            tc = event_times(torch, stream, lambda: X.copy_(B0), 7, 2)
            t_ms = median(ts) - median(tc)
            tf = float(m) ** 3 / (t_ms * 1e-3) / 1e12
            ops["dtrsm_left_lower_n8192"] = {"ms": t_ms, "TFLOP/s": tf,
                                            "frac_of_peak": tf / (PEAK_FP64_MFMA / 1e12),
                                            "timing": "median(copy of B + solve) - median(copy of B)",
                                            "traffic": traffic.get("dtrsm_left_lower_n8192"),
                                            "algorithmic_bytes": (m * (m + 1.0) / 2 + 2.0 * m * m) * 8.0}
            # The same solve at other orders and with few right-hand sides (left / lower / N /
            # non-unit, order x right-hand sides), timed the same way on views of the operands.
            for (mt, nt) in [(4096, 4096), (2048, 2048), (8192, 1024), (8192, 256)]:
                def solve_t():
                    X[:mt * nt].copy_(B0[:mt * nt])
                    h.dtrsm(LEFT, LOWER, N_OP, NON_UNIT, mt, nt, 1.0, L, m, X, mt)

                ts = event_times(torch, stream, solve_t, 9, 2)
                tc = event_times(torch, stream, lambda: X[:mt * nt].copy_(B0[:mt * nt]), 9, 2)
                t_ms = median(ts) - median(tc)
                tf = float(mt) * mt * nt / (t_ms * 1e-3) / 1e12
                ops["dtrsm_left_lower_%dx%d" % (mt, nt)] = {
                    "ms": t_ms, "TFLOP/s": tf, "frac_of_peak": tf / (PEAK_FP64_MFMA / 1e12)}
            del L, B0, X
            # Awkward shapes: NN, ld = rows + 3, alpha 1, beta 0 (masked-edge kernel, no pad copy).
            for (mm, nn, kk) in [(10007, 4099, 6151), (65536, 256, 256)]:
                Aa = torch.empty((mm + 3) * kk, dtype=torch.float64, device="cuda")
                Ba = torch.empty((kk + 3) * nn, dtype=torch.float64, device="cuda")
                Ca = torch.empty((mm + 3) * nn, dtype=torch.float64, device="cuda")
                h.dfill(Aa, mm, kk, mm + 3, 1)
                h.dfill(Ba, kk, nn, kk + 3, 2)
                h.dfill(Ca, mm, nn, mm + 3, 3)
                ts = event_times(torch, stream,
                                 lambda: h.dgemm(N_OP, N_OP, mm, nn, kk, 1.0, Aa, mm + 3, Ba, kk + 3,
                                                 0.0, Ca, mm + 3), 10, 2)
                tf = 2.0 * mm * nn * kk / (median(ts) * 1e-3) / 1e12
                ops["dgemm_nn_%dx%dx%d_ld+3" % (mm, nn, kk)] = {
                    "ms": median(ts), "TFLOP/s": tf, "frac_of_peak": tf / (PEAK_FP64_MFMA / 1e12)}
                del Aa, Ba, Ca
            # Bandwidth-bound nodes at 8192^2 (2 n^2 8 bytes; accumulate with beta != 0: 3 n^2 8).
            nb = 8192
            S = torch.empty(nb * nb, dtype=torch.float64, device="cuda")
            D = torch.empty(nb * (nb + 32), dtype=torch.float64, device="cuda")
            h.dfill(S, nb, nb, nb, 5)
            h.dfill(D, nb, nb, nb, 6)
            cases = {
                "transpose_8192": (lambda: h.dgeam(T_OP, N_OP, nb, nb, 1.0, S, nb, 0.0, D, nb, D, nb), 2),
                "pad_copy_8192_ld8224": (lambda: h.dgeam(N_OP, N_OP, nb, nb, 1.0, S, nb, 0.0, D, nb + 32, D, nb + 32), 2),
                "transpose_accumulate_8192_beta0.5": (lambda: h.dgeam(T_OP, N_OP, nb, nb, 1.0, S, nb, 0.5, D, nb, D, nb), 3),
            }
            for name, (fn, passes) in cases.items():
                ts = event_times(torch, stream, fn, 20, 3)
                ops[name] = bw_row(median(ts), passes * nb * nb * 8.0)
            del S, D
            # The same nodes at 16384^2 and on the operands of the awkward DGEMM (ld = rows + 3):
            # the pad copy into ld rounded up to 32, and the transpose into ld = rows.
            for name, tr, gm, gn, lda, ldc in (
                    ("transpose_16384", True, 16384, 16384, 16384, 16384),
                    ("pad_copy_10007x6151_ld10010_to_10016", False, 10007, 6151, 10010, 10016),
                    ("pad_copy_6151x4099_ld6154_to_6176", False, 6151, 4099, 6154, 6176),
                    ("pad_copy_65536x256_ld65539_to_65536", False, 65536, 256, 65539, 65536),
                    ("transpose_6151x10007_ld10010_to_6151", True, 6151, 10007, 10010, 6151)):
                ar, ac = (gn, gm) if tr else (gm, gn)       # stored shape of the source
                S = torch.empty(lda * ac, dtype=torch.float64, device="cuda")
                D = torch.empty(ldc * gn, dtype=torch.float64, device="cuda")
                h.dfill(S, ar, ac, lda, 5)
                ts = event_times(torch, stream,
                                 lambda: h.dgeam(T_OP if tr else N_OP, N_OP, gm, gn, 1.0, S, lda, 0.0, D,
                                                 ldc, D, ldc), 20, 3)
                ops[name] = bw_row(median(ts), 2.0 * gm * gn * 8.0)
                del S, D
            # Size sweep of the headline call (opA = T, opB = N, alpha 1, beta 0.5, ld = n).
            for nn in (1024, 2048, 4096, 16384):
                Aa = torch.empty(nn * nn, dtype=torch.float64, device="cuda")
                Ba = torch.empty_like(Aa)
                Ca = torch.empty_like(Aa)
                h.dfill(Aa, nn, nn, nn, 1)
                h.dfill(Ba, nn, nn, nn, 2)
                h.dfill(Ca, nn, nn, nn, 3)
                ts = event_times(torch, stream,
                                 lambda: h.dgemm(T_OP, N_OP, nn, nn, nn, 1.0, Aa, nn, Ba, nn, 0.5,
                                                 Ca, nn), 5 if nn > 8192 else 10, 2)
                tf = 2.0 * nn ** 3 / (median(ts) * 1e-3) / 1e12
                ops["dgemm_tn_n%d" % nn] = {"ms": median(ts), "TFLOP/s": tf,
                                            "frac_of_peak": tf / (PEAK_FP64_MFMA / 1e12)}
                del Aa, Ba, Ca
            # Single precision (fp32 matrix peak 157.3 TFLOP/s), same kernel templates.
            nf = 8192
            Af = torch.empty(nf * nf, dtype=torch.float32, device="cuda")
            Bf = torch.empty_like(Af)
            Cf = torch.empty_like(Af)
            h.sfill(Af, nf, nf, nf, 1)
            h.sfill(Bf, nf, nf, nf, 2)
            h.sfill(Cf, nf, nf, nf, 3)
            ts = event_times(torch, stream,
                             lambda: h.sgemm(T_OP, N_OP, nf, nf, nf, 1.0, Af, nf, Bf, nf, 0.5, Cf,
                                             nf), 10, 2)
            tf = 2.0 * nf ** 3 / (median(ts) * 1e-3) / 1e12
            ops["sgemm_tn_n8192"] = {"ms": median(ts), "TFLOP/s": tf,
                                     "frac_of_fp32_peak": tf / (PEAK_FP32_MFMA / 1e12)}
            del Af, Bf, Cf

        autotune = None
        reference = None
        if not args.quick:
            autotune = autotune_check(torch, stream, h, n, A, B, Cm)
            reference = reference_timings(torch, stream, h, n, A, B, Cm)

    cpu = None
    if not args.quick and not args.no_cpu:
        try:
            cpu = cpu_baseline(n, 3)
        except Exception as e:  # the baseline is reported, never required for the GPU figure
            log("cpu baseline failed:", repr(e))

    line = {
        "metric": "fp64 TFLOP/s (GEMM/SYRK/TRSM, n=8192) + % of MI355X fp64 MFMA peak",
        "value_is": "the DGEMM row; DSYRK and DTRSM are ops.dsyrk_lower_n8192_k2048 and "
                    "ops.dtrsm_left_lower_n8192",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": "DGEMM C=alpha*A^T*B+beta*C, M=N=K=%d, fp64, opA=T opB=N, alpha=1 "
                               "beta=0.5, column-major ld=rows, iid uniform[-1,1) seeds 1/2/3; one "
                               "step = one rtat_dgemm call" % n,
                   "pct_of_fp64_mfma_peak": 100.0 * value / (PEAK_FP64_MFMA / 1e12),
                   "compute_units": cus},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "hbm_streaming": hbm,
        "ops": ops,
        "autotune": autotune,
        "reference": reference,
        "library": native.version(),
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
