"""CPU baseline leg of bench.py: times the CPU restatement of the reference path on this host.

TEST / MEASUREMENT INFRASTRUCTURE ONLY.  The number it produces is a reported baseline, not a
target: the reference itself (MKL + TBB) cannot be built in this image, so the timed code is this
repository's own restatement ("kind": "port").
"""
import os
import time

import numpy as np

import oracle


def run(nf, B, R, lr, budget_s):
    """Runs whole training steps of the given model on the host until about budget_s seconds of
    CPU work are spent (at least one step), and returns the cpu_baseline object of the bench line.
    If one full step does not fit the budget, the batch per replica is cut down (the work per step
    is linear in it) and the sample says so."""
    L = len(nf) - 1
    flop_full = 3 * 2.0 * R * B * sum(nf[l] * nf[l + 1] for l in range(L))
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    # the double-accumulating oracle sustains roughly 2.5 GFLOP/s per core
    est_step_s = flop_full / (2.5e9 * cores)
    Bs = B
    while Bs > 16 and est_step_s * Bs / B > budget_s:
        Bs //= 2
    X, Ws, bs, dY = oracle.make_problem(nf, Bs, R, seed=1)
    flop = flop_full * Bs / B
    steps, t0 = 0, time.perf_counter()
    while True:
        oracle.mlp_step(nf, Bs, R, X, dY, Ws, bs, lr)
        steps += 1
        spent = time.perf_counter() - t0
        if spent + spent / steps > budget_s or steps >= 50:
            break
    ms = spent / steps * 1e3
    return {
        "value": round(flop / (ms * 1e-3) / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "ms_per_step": round(ms, 2),
        "sample": f"{steps} full step(s) of the same model with batch {Bs} per replica x {R} replicas"
                  f"{'' if Bs == B else f' (cut down from {B}; work per step is linear in the batch)'}, "
                  "float64-accumulating OpenMP oracle (oracle/mlp_oracle.c)",
    }
