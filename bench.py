#!/usr/bin/env python3
"""Benchmark of the MLP training step (forward, backward, gradient reduce + SGD) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config C2]

A "step" is one pass of the whole hot path over one batch of seeded synthetic input: L forward
GEMMs, L weight-gradient GEMMs (R replicas each), L bias gradients, L input-gradient GEMMs and
the R-way gradient reduce with the SGD update.  Inputs and weights are resident in HBM before
the timed region starts.  Default schedule: the weight-gradient GEMMs and the per-layer reduce+SGD
launches trail the chain of input-gradient GEMMs on a second stream.  The timed loop is the
reference's: K consecutive steps, each on the weights the step before left, with the reference's
learning rate of 1e-10 (mlp_omp.cc:435-737 with alpha at :609,699,718,729), at which the
sum-reduced updates stay finite however many steps are run (--lr 0.01 --restore-each-step times
the same step at the learning rate of the parity tests, with a device copy of the weights added
to every step).

After the headline configuration (--config, default C2) the default run times the other benchmark
configurations the same way on fresh handles and reports them under other_configs
(--other-configs none skips them).  --gemm and --update time single entry points instead.

Prints one JSON line:
  value          whole-step throughput, TFLOP/s on the reference's FLOP model
                 3 * 2 * (R*B) * sum_l N_l*N_{l+1}   (mlp_omp.cc:492,584,675)
  ms_per_step    wall clock of the timed loop / K
  roofline       the GEMM kernels (the dominant kernels): FLOP per launch / average launch
                 duration, against the fp32 MFMA peak.  Durations come from HIP events attached
                 to each kernel dispatch on the stream it is launched on (start and stop event of
                 hipExtLaunchKernelGGL), in a second pass over the same K steps in which every
                 kernel runs alone (one stream, one update launch): overlapping kernels cannot be
                 timed individually
  roofline_reduce  the reduce+SGD kernel: (R+2)*4*P bytes / its launch duration, against HBM peak
  cpu_baseline   the CPU restatement of the reference's mlp_omp timed on this host's cores
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

CONFIGS = {
    # name: (layer widths N_0 .. N_L, batch per replica, replicas, dtype)
    "C1": ([512] * 4, 256, 2, "f32"),
    "C2": ([1024] * 9, 1024, 4, "f32"),
    "C3": ([4096] * 5, 2048, 2, "f32"),
    "C4": ([2048] * 21, 256, 8, "f32"),
    "C5": ([8192] * 9, 4096, 4, "bf16"),
    # the reference's own default model (mlp_bench_common.h:26), four sockets of 1024 rows
    "ref": ([1024] * 7 + [1], 1024, 4, "f32"),
    "ref16": ([1024] * 7 + [1], 1024, 4, "bf16"),   # the same model on the bf16 path (matrix-vector kernels for 1024 -> 1)
}
PEAK_TFLOPS = {"f32": 157.3, "bf16": 2516.6}  # MI355X dense MFMA peaks
PEAK_HBM_GBPS = 8000.0
METRIC = "MLP fwd+bwd+reduce step ms & TFLOP/s on 1 MI355X; grad-reduce GB/s"

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic_pmc.json")
KERNEL_SOURCES = os.path.join(ROOT, "tbb_test_amd", "csrc")


def kernel_source_hash():
    """sha256 over the kernel sources: the measured traffic figures belong to one state of them."""
    import hashlib

    h = hashlib.sha256()
    for name in sorted(os.listdir(KERNEL_SOURCES)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            h.update(open(os.path.join(KERNEL_SOURCES, name), "rb").read())
    return h.hexdigest()


def measured_traffic(config):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, each
    scaled by what the same counter reads for the plain device copy of the weight snapshot), as
    recorded in profiles/traffic_pmc.json together with the hash of the kernel sources they were
    measured on.  Returns ({"gemm": bytes, "reduce": bytes}, note); figures are None when nothing
    was recorded for the configuration or when the kernels have changed since."""
    try:
        data = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return {}, "no traffic file"
    if data.get("source_hash") != kernel_source_hash():
        return {}, "kernel sources changed since the counters were read (profiles/traffic_pmc.json is stale)"
    return data.get("configs", {}).get(config, {}), data.get("how", "")


def cpu_baseline(nf, B, R, lr, budget_s):
    """Times the CPU restatement of the reference path on this host (rank 0, N = 1 only)."""
    import oracle
    from oracle import cpu_baseline as port

    return port.run(nf, B, R, lr, budget_s)


def raw_gemm(args, np, capi):
    """One GEMM entry point alone, as the profiles quote it: C = A[M,K] * B[N,K]^T (+ ReLU), operands with
    random signs, exponents and mantissas (what the power-limited bf16 rate depends on), K launches between
    two stream synchronisations."""
    import ctypes
    import time

    M, N, K = (int(x) for x in args.gemm.split(","))
    lib = capi.lib()
    if args.hvariant:
        capi.check(lib.mi_set_hgemm_variant(args.hvariant))
    if args.variants:
        for kind, v in enumerate(int(x) for x in args.variants.split(",")):
            capi.check(lib.mi_set_gemm_variant(kind, v))
    rng = np.random.default_rng(args.seed)
    bf16 = args.gemm_dtype == "bf16"

    def operand(rows):
        if bf16:  # sign | exponent 2^-3 .. 2^2 | 7 mantissa bits
            v = (rng.integers(0, 2, (rows, K), dtype=np.uint16) << 15) | ((0x7c + rng.integers(0, 6, (rows, K), dtype=np.uint16)) << 7) \
                | rng.integers(0, 128, (rows, K), dtype=np.uint16)
            return capi.DeviceBuffer.from_numpy(v.astype(np.uint16))
        return capi.DeviceBuffer.from_numpy(rng.standard_normal((rows, K), dtype=np.float32))

    A, Bm = operand(M), operand(N)
    C = capi.DeviceBuffer(M * N * (2 if bf16 else 4))
    fn = lib.mi_hgemm_nt if bf16 else lib.mi_sgemm_nt

    def launch():
        capi.check(fn(M, N, K, A.ptr, K, Bm.ptr, K, C.ptr, N, None, 1, None))

    for _ in range(max(args.warmup, 20)):   # also brings the clocks up
        launch()
    capi.check(lib.mi_stream_sync(None))
    t0 = time.perf_counter()
    for _ in range(args.steps):
        launch()
    capi.check(lib.mi_stream_sync(None))
    us = (time.perf_counter() - t0) / args.steps * 1e6
    peak = 2516.6 if bf16 else 157.3
    tflops = 2.0 * M * N * K / us / 1e6
    print(json.dumps({"gemm": f"{args.gemm_dtype} nt {M}x{N}x{K}", "hvariant": args.hvariant, "variants": args.variants,
                      "launches": args.steps, "us_per_launch": round(us, 1), "tflops": round(tflops, 1),
                      "frac_of_peak": round(tflops / peak, 4)}))


def raw_update(args, np, capi):
    """The reduce+SGD entry points alone on one weight matrix [rows x cols] with R gradient copies,
    K launches between two stream synchronisations (mlp_omp.cc:240-252 is the pass they stand for):
      fp32        mi_reduce_sgd_raw         reads R gradients + W, writes W                  (R + 2) * 4 bytes per weight
      fp32+bf16   mi_reduce_sgd_bf16_raw    the same plus the bf16 copy of W                 + 2
      fp32+bf16+T mi_reduce_sgd_bf16t_raw   the same plus the transposed bf16 copy, tiled    + 2 + 2
    Comparing the three shows what each extra write stream costs.  lr = 0: the weights stay what
    they are however many launches run."""
    import ctypes

    rows, cols, R, *extra = (int(x) for x in args.update.split(","))
    n = rows * cols
    layers = extra[1] if len(extra) > 1 else 1   # matrices laid out one behind the other, as a model's layers are
    stride = layers * n + (extra[0] if extra else 0)     # floats between consecutive replicas' gradients
    lib = capi.lib()
    rng = np.random.default_rng(args.seed)
    w = rng.standard_normal(n, dtype=np.float32)
    g = rng.standard_normal(n, dtype=np.float32)
    W, G = capi.DeviceBuffer(layers * n * 4), capi.DeviceBuffer(R * stride * 4)
    for l in range(layers):
        capi.check(lib.mi_memcpy_h2d(W.ptr + l * n * 4, w.ctypes.data_as(ctypes.c_void_p), n * 4))
        for r in range(R):
            capi.check(lib.mi_memcpy_h2d(G.ptr + (r * stride + l * n) * 4, g.ctypes.data_as(ctypes.c_void_p), n * 4))
    W16, W16T = capi.DeviceBuffer(layers * n * 2), capi.DeviceBuffer(layers * n * 2)
    lr = ctypes.c_float(0.0)
    turn = [0]

    def at(buf, elem_bytes):     # the matrix of the current launch inside its arena
        return buf.ptr + (turn[0] % layers) * n * elem_bytes

    kinds = {
        "fp32": (lambda: lib.mi_reduce_sgd_raw(at(W, 4), at(G, 4), n, stride, R, lr, None), (R + 2) * 4.0),
        "fp32+bf16": (lambda: lib.mi_reduce_sgd_bf16_raw(at(W, 4), at(W16, 2), at(G, 4), n, stride, R, lr, None), (R + 2) * 4.0 + 2),
        "fp32+bf16+bf16T": (lambda: lib.mi_reduce_sgd_bf16t_raw(at(W, 4), at(W16, 2), at(W16T, 2), at(G, 4), rows, cols, stride, R, lr, None),
                            (R + 2) * 4.0 + 4),
    }
    out = {"update": f"{rows} x {cols}, R = {R}, {layers} matrices taken in turn, replica stride {stride} floats", "launches": args.steps, "peak_gbps": PEAK_HBM_GBPS, "kernels": {}}
    for name, (fn, bytes_per_weight) in kinds.items():
        for _ in range(max(args.warmup, 5)):
            capi.check(fn())
            turn[0] += 1
        capi.check(lib.mi_stream_sync(None))
        t0 = time.perf_counter()
        for _ in range(args.steps):
            capi.check(fn())
            turn[0] += 1
        capi.check(lib.mi_stream_sync(None))
        us = (time.perf_counter() - t0) / args.steps * 1e6
        gbps = bytes_per_weight * n / us / 1e3
        out["kernels"][name] = {"us_per_launch": round(us, 1), "bytes_per_launch": bytes_per_weight * n,
                                "gbps": round(gbps, 1), "frac_of_peak": round(gbps / PEAK_HBM_GBPS, 4)}
    print(json.dumps(out))


def other_config_names(args):
    """--other-configs: 'auto' = every other benchmark configuration when the headline config runs
    untuned with default schedule flags, 'none' = skip, or a comma-separated list."""
    if args.other_configs == "none":
        return []
    if args.other_configs == "auto":
        tuned = (args.config != "C2" or args.hvariant or args.variants or args.serial_backward or args.flat_update
                 or args.no_graph or args.restore_each_step)
        return [] if tuned else [c for c in ("C1", "C3", "C4", "C5", "ref") if c != args.config]
    names = [c for c in args.other_configs.split(",") if c]
    for c in names:
        if c not in CONFIGS:
            raise SystemExit(f"bench.py: unknown configuration {c!r} in --other-configs")
    return names


def measure_config(config, args, steps, warmup, info, np, capi, hostlib, min_loop_s=0.0, probe=True):
    """Times one benchmark configuration on a fresh handle and returns the fields of the JSON line.
    min_loop_s > 0: the timed loop runs at least that long (more steps than `steps` for the models
    whose step takes microseconds)."""
    nf, B, R, dtype = CONFIGS[config]
    layers = len(nf) - 1

    X, Ws, dY = hostlib.init_problem(nf, B, R, args.seed)
    flags = (0 if args.flat_update else capi.FLAG_PER_LAYER_UPDATE) | (capi.FLAG_SERIAL_BACKWARD if args.serial_backward else 0)
    if args.no_graph:
        flags |= capi.FLAG_NO_GRAPH
    h = capi.MlpHandle(nf, B, R, dtype=capi.MI_BF16 if dtype == "bf16" else capi.MI_F32, flags=flags)
    if args.hvariant:
        capi.check(capi.lib().mi_set_hgemm_variant(args.hvariant))
    if args.variants:
        for kind, v in enumerate(int(x) for x in args.variants.split(",")):
            capi.check(capi.lib().mi_set_gemm_variant(kind, v))
    for l in range(layers):
        h.set_weights(l, Ws[l], None)
    h.set_input(X)
    h.set_dy(dY)
    h.snapshot_weights()
    params, _ = h.param_count()

    def one_step():
        if args.restore_each_step:
            h.restore_weights()
        h.step(args.lr)

    # Untimed spin-up so that the GPU has left its idle clock state before anything is measured
    # (the first tens of milliseconds after idle run at reduced clocks), then the W warm-up steps.
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.3:
        for _ in range(10):
            one_step()
        h.sync()
    for _ in range(warmup):
        one_step()
    h.sync()
    if min_loop_s > 0:   # a first short loop sizes the timed one
        t0 = time.perf_counter()
        for _ in range(steps):
            one_step()
        h.sync()
        per_step = (time.perf_counter() - t0) / steps
        steps = int(min(max(steps, min_loop_s / max(per_step, 1e-9)), 2000))
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    h.sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / steps * 1e3

    # per-kernel durations: K more steps, from the initial weights again, with a HIP event pair
    # around every launch
    h.restore_weights()
    h.enable_timing(True)
    h.reset_timings()
    for _ in range(steps):
        one_step()
    ms, cnt = h.timings()
    h.enable_timing(False)
    finite = all(bool(np.isfinite(h.weight(l)).all()) for l in range(layers))
    sched = h.schedule()     # what the timed loop actually ran (the library also looks at the shapes)
    h.close()

    # What the matrix cores sustain right now with no memory traffic at all (register-resident
    # MFMA loop, run on the warm device): context for the roofline fraction, which stays priced
    # against the published peak.  The bf16 rate is power-limited and depends on the operand
    # values (dense random operands draw more than constant ones); the fp32 rate does not.
    def mfma_rate(operands):
        import ctypes

        r = ctypes.c_double()
        capi.check(capi.lib().mi_probe_mfma_rate(1 if dtype == "bf16" else 0, operands, ctypes.byref(r), None))
        return round(r.value, 1)
    mfma_only = None
    if probe:
        mfma_only = {"unit": "TFLOP/s", "random_operands": mfma_rate(2), "ones": mfma_rate(1), "zeros": mfma_rate(0),
                     "how": "loop of independent MFMAs on register operands, no memory traffic, measured right "
                            "after the steps above (mi_probe_mfma_rate)"}
        if dtype == "bf16":  # the large GEMMs use 16x16x32 MFMAs (the figures above); the 32x32x16 shape for comparison
            mfma_only["random_operands_32x32x16"] = mfma_rate(3)

    rows = R * B
    # FLOP of the forward / weight-gradient / input-gradient GEMM of layer l: 2 * rows * N_l * N_{l+1}.
    # The roofline object prices the dominant kernel: the GEMM launches of the widest layers (all of
    # them in the square benchmark configurations; the 1024 -> 1 layer of `ref` runs on the
    # matrix-vector kernels and is left out of the MFMA figure).
    layer_flop = [2.0 * rows * nf[l] * nf[l + 1] for l in range(layers)]
    gemm_flop_step = 3 * sum(layer_flop)
    flop_per_gemm = max(layer_flop)
    wide = [l for l in range(layers) if layer_flop[l] == flop_per_gemm]
    gemm_ms = float(ms[0:3][:, wide].sum())
    gemm_launches = int(cnt[0:3][:, wide].sum())
    gemm_avg_ms = gemm_ms / gemm_launches
    gemm_tflops = flop_per_gemm / (gemm_avg_ms * 1e-3) / 1e12
    per_phase = {capi.BREAKDOWN_NAMES[i]: float(ms[i].sum() / steps) for i in range(4)}

    upd_launches = int(cnt[3].sum())
    upd_ms = float(ms[3].sum()) / upd_launches
    # the event-timed pass always runs the update as one launch over all layers
    upd_bytes = (R + 2) * 4.0 * params
    if dtype == "bf16":
        upd_bytes += 4.0 * params   # the bf16 copy and the transposed bf16 copy of the weights
    upd_gbps = upd_bytes / (upd_ms * 1e-3) / 1e9

    peak = PEAK_TFLOPS[dtype]
    traffic, traffic_note = measured_traffic(config)
    schedule = ("weight and input gradient of a layer in one launch, one stream" if sched["paired_backward"]
                else "weight-gradient GEMMs on a second stream" if sched["dual_streams"] else "backward pass on one stream")
    schedule += ", per-layer update on the second stream" if sched["per_layer_update"] else ", one update launch"
    schedule += ", graph replay" if sched["graph"] else ", eager launches"
    out = {
        "metric": METRIC,
        "value": round(gemm_flop_step / (ms_per_step * 1e-3) / 1e12, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {"workload": f"{config}: {layers} FC layers, widths "
                               + (f"{nf[0]} throughout" if len(set(nf)) == 1 else " ".join(str(v) for v in nf))
                               + f", ReLU between layers, batch {B} per replica x {R} replicas, "
                               + ("every step from the initial weights" if args.restore_each_step else "consecutive steps")
                               + f", lr {args.lr}, seed {args.seed}"
                               + ("" if args.restore_each_step else
                                  " (the reference's loop and its alpha, mlp_omp.cc:609; the loop at the lr = 0.01 of the "
                                  "benchmark configurations, which needs every step to start from the initial weights to "
                                  "stay finite, is --lr 0.01 --restore-each-step)"),
                   "schedule": schedule, "device": info["name"], "num_cus": info["num_cus"]},
        "gemm_flop_per_step": gemm_flop_step,
        "phase_ms_per_step": {k: round(v, 4) for k, v in per_phase.items()},
        "gemm_tflops": round(gemm_tflops, 2),
        "reduce_gbps": round(upd_gbps, 1),
        "weights_finite": finite,
        "roofline": {"kernel": "gemm_f32_dma (nt, nn, tn)" if dtype == "f32" else
                               "gemm_bf16_x32w4 (spans of the weight gradient include the column-sum fold or row-sum "
                               "kernel of the bias gradient and, for operands no GEMM epilogue wrote transposed, the "
                               "transpose launches)",
                     "bound": "mfma", "achieved": round(gemm_tflops, 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(gemm_tflops / peak, 4),
                     "traffic": traffic.get("gemm"), "traffic_note": traffic_note,
                     "flop_per_launch": flop_per_gemm, "avg_launch_us": round(gemm_avg_ms * 1e3, 2),
                     "launches": gemm_launches, "mfma_only_rate": mfma_only},
        "roofline_reduce": {"kernel": "reduce_sgd_vec4" if dtype == "f32" else "reduce_sgd_tile (one launch per layer)",
                            "bound": "hbm", "achieved": round(upd_gbps, 1),
                            "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": round(upd_gbps / PEAK_HBM_GBPS, 4),
                            "traffic": traffic.get("reduce"),
                            "bytes_per_launch": upd_bytes, "avg_launch_us": round(upd_ms * 1e3, 2)},
    }
    if sched["paired_backward"]:
        # the timed loop ran gemm_f32_splitk_pair (weight and input gradient of a layer in one launch);
        # the event-timed pass keeps separate launches so that every phase has a figure of its own
        out["roofline"]["note"] = ("phase_ms_per_step, gemm_tflops and this object time the separate weight-gradient and "
                                   "input-gradient launches (gemm_f32_splitk); ms_per_step and value come from the loop "
                                   "that runs them paired in one launch per layer")
    return out


def alive_at_exit():
    """One line on stderr about what this process still holds when it is about to exit: threads
    other than the main one and child processes (the OpenMP pool of the CPU baseline ends with the
    process; its task-graph arenas are joined in their destructor)."""
    import threading

    threads = [t.name for t in threading.enumerate() if t is not threading.main_thread()]
    children = []
    try:
        me = os.getpid()
        for pid in os.listdir("/proc"):
            if pid.isdigit():
                try:
                    fields = open(f"/proc/{pid}/stat").read().rsplit(")", 1)[1].split()
                    if int(fields[1]) == me:
                        children.append(int(pid))
                except (OSError, IndexError, ValueError):
                    pass
        native = len(os.listdir(f"/proc/{me}/task"))
    except OSError:
        native = -1
    print(f"bench.py exit: python threads besides main {threads}, native threads {native}, child processes {children}",
          file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="C2", choices=sorted(CONFIGS))
    ap.add_argument("--lr", type=float, default=1e-10, help="learning rate (default: the reference benchmark's alpha)")
    ap.add_argument("--restore-each-step", action="store_true",
                    help="start every step from the initial weights (a device copy inside the timed region): "
                         "keeps a loop at a visible learning rate such as 0.01 finite")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--flat-update", action="store_true",
                    help="one update launch at the end of the step instead of per-layer updates on the second stream")
    ap.add_argument("--hvariant", type=int, default=0, help="tuning: forced bf16 GEMM tile variant")
    ap.add_argument("--variants", default="", help="tuning: forced GEMM tile variants 'nt,nn,tn'")
    ap.add_argument("--serial-backward", action="store_true", help="whole backward pass on one stream")
    ap.add_argument("--no-graph", action="store_true", help="tuning: every step launched eagerly instead of replaying its graph")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--gemm", default="", metavar="M,N,K",
                    help="instead of the training step: time the forward-type GEMM entry point alone (mi_hgemm_nt / "
                         "mi_sgemm_nt, dtype of --gemm-dtype, dense random operands) and print one JSON line")
    ap.add_argument("--gemm-dtype", default="bf16", choices=["bf16", "f32"])
    ap.add_argument("--update", default="", metavar="ROWS,COLS,R[,PAD[,LAYERS]]",
                    help="instead of the training step: time the raw reduce+SGD entry points alone on one weight matrix "
                         "(mi_reduce_sgd_raw, mi_reduce_sgd_bf16_raw, mi_reduce_sgd_bf16t_raw) and print one JSON line; "
                         "PAD = floats between the end of one replica's gradients and the start of the next (default 0), LAYERS = "
                         "matrices laid out one behind the other and taken in turn, launch by launch (default 1)")
    ap.add_argument("--other-configs", default="auto",
                    help="'auto' (default): after the headline configuration C2 also time C1, C3, C4, C5 and ref with "
                         "fresh handles and report them under other_configs; 'none'; or a comma-separated list")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; there is no multi-GPU path (no collectives). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np

    from tbb_test_amd import capi, hostlib

    if args.gemm:
        raw_gemm(args, np, capi)
        return
    if args.update:
        raw_update(args, np, capi)
        return

    info = capi.device_info()
    out = measure_config(args.config, args, args.steps, args.warmup, info, np, capi, hostlib)
    others = other_config_names(args)
    if others:
        # The other benchmark configurations, each with a fresh handle in this process, after the
        # headline measurement: short figures only (the headline's fields stay as they are).
        out["other_configs"] = {}
        for name in others:
            try:
                full = measure_config(name, args, args.steps, args.warmup, info, np, capi, hostlib, min_loop_s=0.2,
                                      probe=False)
                out["other_configs"][name] = {
                    "ms_per_step": full["ms_per_step"], "value": full["value"], "steps": full["steps"],
                    "gemm_frac": full["roofline"]["frac"], "reduce_frac": full["roofline_reduce"]["frac"],
                    "gemm_avg_launch_us": full["roofline"]["avg_launch_us"],
                    "reduce_avg_launch_us": full["roofline_reduce"]["avg_launch_us"],
                    "dtype": full["dtype"], "schedule": full["config"]["schedule"], "weights_finite": full["weights_finite"]}
                if "note" in full["roofline"]:
                    out["other_configs"][name]["note"] = full["roofline"]["note"]
            except Exception as exc:   # the headline line is printed whatever happens to the extras
                out["other_configs"][name] = {"error": f"{type(exc).__name__}: {exc}"}
    if args.cpu_seconds > 0:
        nf, B, R, _ = CONFIGS[args.config]
        out["cpu_baseline"] = cpu_baseline(nf, B, R, args.lr, args.cpu_seconds)
    print(json.dumps(out), flush=True)
    alive_at_exit()


if __name__ == "__main__":
    main()
