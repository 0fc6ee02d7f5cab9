"""GPU parity of exactly what bench.py times: a handle built with MI_FLAG_PER_LAYER_UPDATE (graph
on) whose step replays its captured graph with the weight-gradient GEMMs and the per-layer
reduce + SGD launches trailing the input-gradient chain on the second stream -- the GPU
counterpart of the reference loop with OVERLAP_ALL_REDUCE (mlp_omp.cc:435-737 with
:601-615,692-723).  Two loops: consecutive steps (bench.py's and the reference's loop, each step on
the weights the step before left), and snapshot, then [restore, step] repeated (every replay
starts from the same weights, so one oracle step checks a replayed step at a learning rate that
moves the weights visibly).

Config 2 (the benchmark's headline) runs at full size against the float64-accumulating oracle and,
bit for bit, against the serial eager schedule.  Config 5 (bf16, 52.8 TFLOP per step) is checked
through mi_mlp_step on sampled rows for every layer, with the oracle fed the device's own
operands (one row per 256-row tile of every output, all replicas of every weight gradient), and the
update of every layer is re-derived bit-exactly from the device's gradients.
Bounds: 1e-4 (fp32) / 2e-2 (bf16), norm-wise and element-wise."""
import numpy as np
import pytest

import oracle
from conftest import BF16_TOL, FP32_TOL, close, elem_err, rel_err
from tbb_test_amd import capi, hostlib

pytestmark = pytest.mark.gpu
LR = 0.01
BENCH_FLAGS = capi.FLAG_PER_LAYER_UPDATE   # what bench.py passes by default


def build(nf, B, R, seed, dtype=capi.MI_F32, flags=0):
    X, Ws, dY = hostlib.init_problem(nf, B, R, seed)   # the initialisation bench.py uses
    h = capi.MlpHandle(nf, B, R, dtype=dtype, flags=flags)
    for l in range(len(nf) - 1):
        h.set_weights(l, Ws[l], None)
    h.set_input(X)
    h.set_dy(dY)
    return h, X, Ws, dY


def bench_loop(h, steps, snapshot=True):
    """Every step starts from the snapshot (a benchmark loop whose values cannot drift)."""
    if snapshot:
        h.snapshot_weights()
    for _ in range(steps):
        h.restore_weights()
        h.step(LR)
    h.sync()


def bf16_round(a):
    """fp32 -> bf16 (round to nearest even) -> fp32, numpy restatement of the device rounding."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return (u.astype(np.uint32) << 16).view(np.float32)


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32 if a.dtype == np.float32 else np.uint64)


def test_config_2_benchmarked_schedule_full_size():
    nf, B, R = [1024] * 9, 1024, 4
    L = len(nf) - 1
    h, X, Ws, dY = build(nf, B, R, seed=1, flags=BENCH_FLAGS)
    bench_loop(h, 4)            # step 1 eager, steps 2-4 replay the graph
    sched = h.schedule()
    assert sched == {"dual_streams": True, "per_layer_update": True, "graph": True, "fused_transposes": 0,
                     "paired_backward": False}

    bs = [np.zeros(n, np.float32) for n in nf[1:]]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR)
    acts = [h.activation(l) for l in range(L + 1)]
    flips = 0
    for l in range(L + 1):
        assert close(acts[l], ref.acts[l], FP32_TOL), f"activation {l}: {rel_err(acts[l], ref.acts[l])}, {elem_err(acts[l], ref.acts[l])}"
        flips += int(np.count_nonzero((acts[l] > 0) != (ref.acts[l] > 0)))
    assert flips < 100, f"{flips} mask disagreements: more than rounding explains"
    # backward on the device's own activations (identical ReLU masks)
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, given_acts=acts)
    assert close(h.dx(), ref.dX, FP32_TOL), "dX"
    for l in range(L):
        for r in range(R):
            assert close(h.wgrad_of(l, r), ref.dW[r][l], FP32_TOL), f"dW layer {l} replica {r}"
            assert close(h.bgrad_of(l, r), ref.db[r][l], FP32_TOL), f"db layer {l} replica {r}"
        assert close(h.weight(l), ref.W_new[l], FP32_TOL), f"updated W {l}"
        assert close(h.bias(l), ref.b_new[l], FP32_TOL), f"updated b {l}"

    # and bit for bit what the serial eager schedule computes (one stream, one update launch)
    hs, *_ = build(nf, B, R, seed=1, flags=capi.FLAG_NO_GRAPH | capi.FLAG_SERIAL_BACKWARD)
    bench_loop(hs, 1)
    assert hs.schedule() == {"dual_streams": False, "per_layer_update": False, "graph": False, "fused_transposes": 0,
                             "paired_backward": False}
    assert np.array_equal(bits(h.dx()), bits(hs.dx()))
    for l in range(L):
        assert np.array_equal(bits(h.weight(l)), bits(hs.weight(l))), f"W {l}"
        assert np.array_equal(bits(h.bias(l)), bits(hs.bias(l))), f"b {l}"
        for r in (0, R - 1):
            assert np.array_equal(bits(h.wgrad_of(l, r)), bits(hs.wgrad_of(l, r))), f"dW {l} {r}"
    h.close()
    hs.close()


@pytest.mark.parametrize("lr", [1e-10, 1e-5])
def test_config_2_consecutive_steps_as_the_benchmark_runs_them(lr):
    """bench.py's timed loop at full size: consecutive steps, no restore in between, at the
    reference's alpha (1e-10, mlp_omp.cc:609: an update of about one ulp of a weight) and at a rate
    that moves the weights by some tenths of a per cent per step.  Step 1 runs eagerly, steps 2 and 3
    replay the graph.  Bit for bit what the serial eager schedule computes.  At the larger rate the
    third step is also checked against the oracle started from the device's weights after two steps:
    a free-running oracle chain cannot be held to 1e-4 here, because a ReLU mask entry that
    rounding decides differently (14 of 37 million in the first step) changes a whole row of every
    earlier layer's gradient by per cents, and the next steps amplify it (9 000 entries two steps
    later)."""
    nf, B, R = [1024] * 9, 1024, 4
    L = len(nf) - 1
    h, X, Ws, dY = build(nf, B, R, seed=1, flags=BENCH_FLAGS)
    hs, *_ = build(nf, B, R, seed=1, flags=capi.FLAG_NO_GRAPH | capi.FLAG_SERIAL_BACKWARD)
    for step in range(3):
        if step == 2:
            h.sync()
            W2 = [h.weight(l) for l in range(L)]
            b2 = [h.bias(l) for l in range(L)]
        h.step(lr)
        hs.step(lr)
    h.sync(); hs.sync()
    assert h.schedule()["graph"] and h.schedule()["dual_streams"] and h.schedule()["per_layer_update"]
    assert not hs.schedule()["graph"] and not hs.schedule()["dual_streams"]
    assert np.array_equal(bits(h.dx()), bits(hs.dx()))
    for l in range(L):
        assert np.array_equal(bits(h.weight(l)), bits(hs.weight(l))), f"W {l}"
        assert np.array_equal(bits(h.bias(l)), bits(hs.bias(l))), f"b {l}"
        for r in (0, R - 1):
            assert np.array_equal(bits(h.wgrad_of(l, r)), bits(hs.wgrad_of(l, r))), f"dW {l} {r}"
    hs.close()
    if lr >= 1e-6:
        assert max(rel_err(W2[l] - Ws[l], 0 * Ws[l]) for l in range(L)) > 1e-4    # two updates have moved the weights
        ref = oracle.mlp_step(nf, B, R, X, dY, W2, b2, lr)
        acts = [h.activation(l) for l in range(L + 1)]
        for l in range(L + 1):
            assert close(acts[l], ref.acts[l], FP32_TOL), f"activation {l} of the third step"
        ref = oracle.mlp_step(nf, B, R, X, dY, W2, b2, lr, given_acts=acts)   # backward on identical ReLU masks
        assert close(h.dx(), ref.dX, FP32_TOL), "dX of the third step"
        for l in range(L):
            for r in (0, R - 1):
                assert close(h.wgrad_of(l, r), ref.dW[r][l], FP32_TOL), f"dW layer {l} replica {r}"
            assert close(h.weight(l), ref.W_new[l], FP32_TOL), f"W {l} after the third step"
            assert close(h.bias(l), ref.b_new[l], FP32_TOL), f"b {l} after the third step"
    h.close()


def test_learning_rate_change_needs_no_new_graph_and_is_applied():
    """The update kernels read -lr from device memory: a replayed graph follows a changing rate."""
    nf, B, R = [256, 256, 256], 128, 2
    hg, X, Ws, dY = build(nf, B, R, seed=3, flags=BENCH_FLAGS)
    he, *_ = build(nf, B, R, seed=3, flags=capi.FLAG_NO_GRAPH | capi.FLAG_SERIAL_BACKWARD)
    for lr in (1e-3, 1e-3, 5e-4, 2e-3, 2e-3):
        hg.step(lr)
        he.step(lr)
    hg.sync(); he.sync()
    assert hg.schedule()["graph"]
    for l in range(2):
        assert np.array_equal(bits(hg.weight(l)), bits(he.weight(l)))
    bs = [np.zeros(n, np.float32) for n in nf[1:]]
    for lr in (1e-3, 1e-3, 5e-4, 2e-3, 2e-3):
        ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, lr)
        Ws, bs = ref.W_new, ref.b_new
    for l in range(2):
        assert close(hg.weight(l), Ws[l], FP32_TOL)
    hg.close(); he.close()


@pytest.mark.parametrize("variant", [16, 31])
def test_variant_change_after_capture_is_honoured(variant):
    """A handle that captured its graph re-captures after mi_set_gemm_variant; results keep their
    tolerance and the forced kernel is the one that runs (its bits differ from the automatic one's
    only through the summation order, so the check is parity, not equality).  Variant 16: 64 x 64
    tiles instead of the split-K kernel.  Variant 31: 128 x 128 x 32 with direct-to-LDS loads, 96 KB
    of dynamic LDS -- a kernel whose one-time attribute call must not land inside the new capture:
    the step after the change runs eagerly, the one after that captures."""
    nf, B, R = [512, 512, 512], 256, 2
    h, X, Ws, dY = build(nf, B, R, seed=9, flags=BENCH_FLAGS)
    bench_loop(h, 3)
    assert h.schedule()["graph"]
    lib = capi.lib()
    try:
        for kind in range(3):
            capi.check(lib.mi_set_gemm_variant(kind, variant))
        h.restore_weights()
        h.step(LR)
        h.sync()
        assert not h.schedule()["graph"]      # the old graph is gone, this step ran eagerly
        bench_loop(h, 3, snapshot=False)
        assert h.schedule()["graph"]
    finally:
        for kind in range(3):
            lib.mi_set_gemm_variant(kind, 0)
    bs = [np.zeros(n, np.float32) for n in nf[1:]]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR)
    for l in range(2):
        assert close(h.weight(l), ref.W_new[l], FP32_TOL)
    h.close()


def test_capture_after_a_first_step_under_per_kernel_timing():
    """A handle whose first steps ran with per-kernel timing on (separate launches on one stream)
    has not yet launched the kernels of its real schedule; the first untimed step still runs
    eagerly, the capture comes after it, and replayed steps match the oracle."""
    nf, B, R = [1024, 1024, 1024], 1024, 4     # large enough for the 84 KB direct-to-LDS kernels on two streams
    h, X, Ws, dY = build(nf, B, R, seed=4, flags=BENCH_FLAGS)
    h.snapshot_weights()
    h.enable_timing(True)
    for _ in range(2):
        h.restore_weights()
        h.step(LR)
    ms, cnt = h.timings()
    h.enable_timing(False)
    assert cnt[:3].sum() == 2 * 3 * 2 and ms[:3].sum() > 0
    h.restore_weights()
    h.step(LR)
    h.sync()
    assert not h.schedule()["graph"]
    bench_loop(h, 2, snapshot=False)
    sched = h.schedule()
    assert sched["graph"] and sched["dual_streams"] and sched["per_layer_update"]
    bs = [np.zeros(n, np.float32) for n in nf[1:]]
    acts = [h.activation(l) for l in range(3)]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, given_acts=acts)
    for l in range(2):
        assert close(h.weight(l), ref.W_new[l], FP32_TOL), f"W {l}"
    assert close(h.dx(), ref.dX, FP32_TOL)
    h.close()


def test_config_5_step_every_layer_on_sampled_rows():
    nf, B, R = [8192] * 9, 4096, 4
    L, MB = len(nf) - 1, B * R
    flags = BENCH_FLAGS | capi.FLAG_KEEP_GRADIENTS   # every dZ_l stays readable after the step
    h, X, Ws, dY = build(nf, B, R, seed=5, dtype=capi.MI_BF16, flags=flags)
    bench_loop(h, 3)
    sched = h.schedule()
    assert sched["per_layer_update"] and sched["graph"] and not sched["dual_streams"]
    assert sched["fused_transposes"] == 2 * (L - 1)   # every transposed copy came out of a GEMM epilogue

    rng = np.random.default_rng(0)
    # one batch row in every 256-row tile of the activations, and one output feature (= row of dW)
    # in every 256-row tile of the weight gradients: whole rows, so every tile of every GEMM is touched
    rows = np.arange(0, MB, 256) + rng.integers(0, 256, MB // 256)
    ms = np.arange(0, nf[-1], 256) + rng.integers(0, 256, nf[-1] // 256)

    prev = h.activation(0)
    for l in range(L):                       # forward: layer by layer on the device's own input
        cur = h.activation(l + 1)
        want = oracle.fc_forward(prev[rows], Ws[l], None, relu=(l < L - 1))
        assert close(cur[rows], want, BF16_TOL), f"forward layer {l}"
        prev = cur
    del prev, cur

    for l in reversed(range(L)):             # backward: every layer
        dz = h.dz(l)
        a = h.activation(l)
        out = h.dx() if l == 0 else h.dz(l - 1)
        want = oracle.fc_dgrad(dz[rows], Ws[l], a[rows] if l > 0 else None)
        assert close(out[rows], want, BF16_TOL), f"input gradient layer {l}"
        if l > 0:
            assert np.all(out[rows][a[rows] <= 0] == 0)
        grads = []
        for r in range(R):
            sl = slice(r * B, (r + 1) * B)
            dW = h.wgrad_of(l, r)[ms]
            grads.append(dW)
            want = dz[sl][:, ms].astype(np.float64).T @ a[sl].astype(np.float64)
            assert close(dW, want, BF16_TOL), f"dW layer {l} replica {r}"
            assert close(h.bgrad_of(l, r), dz[sl].astype(np.float64).sum(0), BF16_TOL), f"db layer {l} replica {r}"
        del dz, a, out
        # the update, re-derived bit-exactly from the device's own gradients (fp32 master weights),
        # and both bf16 copies the next step's GEMMs read
        W_new = h.weight(l)
        want = oracle.reduce_sgd(Ws[l][ms].ravel(), np.stack([g.ravel() for g in grads]), LR).reshape(len(ms), -1)
        assert np.array_equal(bits(W_new[ms]), bits(want)), f"updated W {l}"
        db = np.stack([h.bgrad_of(l, r) for r in range(R)])
        assert np.array_equal(bits(h.bias(l)), bits(oracle.reduce_sgd(np.zeros(nf[l + 1], np.float32), db, LR))), f"updated b {l}"
        shadow = h.weight_shadow(l)
        assert np.array_equal(bits(shadow), bits(bf16_round(W_new))), f"bf16 copy of W {l}"
        assert np.array_equal(bits(h.weight_shadow(l, transposed=True)), bits(np.ascontiguousarray(shadow.T))), f"bf16 copy of W^T {l}"
        del W_new, shadow

    # the rotating three-buffer schedule (what bench.py runs) gives the same bits
    h2, *_ = build(nf, B, R, seed=5, dtype=capi.MI_BF16, flags=BENCH_FLAGS)
    bench_loop(h2, 3)
    assert np.array_equal(bits(h.dx()), bits(h2.dx()))
    for l in range(L):
        assert np.array_equal(bits(h.weight(l)), bits(h2.weight(l))), f"W {l}"
    h.close()
    h2.close()
