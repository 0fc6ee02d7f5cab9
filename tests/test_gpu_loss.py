"""GPU parity of the loss front-end (SquaredL2Distance + AveragedLoss, mlp_caffe2.py:221-239) and of
the step timeline export (format of the reference's trace.log, mlp_tbb.cc:85-104,1379-1392).

The loss kernel is compared with the CPU oracle on the device's own forward output (the gradient
is elementwise, so this isolates it from GEMM rounding); the step in loss mode is compared with the
oracle step fed that gradient.  Bounds: dY 1e-6 (one fp32 multiply), loss 1e-6 (double
accumulation on both sides), updated weights 1e-4; bf16 model: dY 2^-8 (one bf16 rounding)."""
import json

import numpy as np
import pytest

import oracle
from conftest import BF16_TOL, FP32_TOL, rel_err
from tbb_test_amd import capi

pytestmark = pytest.mark.gpu

LR = 1e-3


def build(nf, B, R, seed, flags=0, dtype=None):
    X, Ws, bs, _ = oracle.make_problem(nf, B, R, seed)
    rng = np.random.default_rng(seed + 17)
    bs = [(0.1 * rng.standard_normal(b.shape)).astype(np.float32) for b in bs]
    labels = rng.standard_normal((R * B, nf[-1])).astype(np.float32)
    h = capi.MlpHandle(nf, B, R, flags=flags) if dtype is None else capi.MlpHandle(nf, B, R, dtype=dtype, flags=flags)
    for l in range(len(nf) - 1):
        h.set_weights(l, Ws[l], bs[l])
    h.set_input(X)
    h.set_labels(labels)
    return h, (X, Ws, bs, labels)


CONFIGS = {
    "rect": ([256, 384, 128, 640], 128, 3),
    "ragged": ([100, 70, 33, 1], 37, 2),      # reference-default style last layer of width 1
    "single_replica": ([128, 128], 64, 1),
}


@pytest.mark.parametrize("name", list(CONFIGS))
def test_loss_kernel_matches_oracle_on_device_predictions(name):
    nf, B, R = CONFIGS[name]
    L = len(nf) - 1
    h, (X, Ws, bs, labels) = build(nf, B, R, seed=31, flags=capi.FLAG_NO_GRAPH)
    for l in range(L):
        h.forward(l)
    h.loss_backward()
    h.sync()
    pred = h.activation(L)
    dY_ref, loss_ref = oracle.l2_loss(pred, labels, R)
    assert rel_err(h.dz(L - 1), dY_ref) <= 1e-6
    per, total = h.loss()
    np.testing.assert_allclose(per, loss_ref, rtol=1e-6)
    assert abs(total - loss_ref.sum()) <= 1e-6 * abs(loss_ref.sum())
    # and the forward output itself is the oracle's
    ref_fwd = oracle.mlp_step(nf, B, R, X, dY_ref, Ws, bs, LR)
    assert rel_err(pred, ref_fwd.acts[L]) <= FP32_TOL
    h.close()


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("flags", [capi.FLAG_NO_GRAPH, 0, capi.FLAG_PER_LAYER_UPDATE])
def test_step_in_loss_mode_matches_oracle(name, flags):
    nf, B, R = CONFIGS[name]
    L = len(nf) - 1
    h, (X, Ws, bs, labels) = build(nf, B, R, seed=77, flags=flags)
    h.step(LR)
    h.sync()
    acts = [h.activation(l) for l in range(L + 1)]
    dY_ref, loss_ref = oracle.l2_loss(acts[L], labels, R)
    ref = oracle.mlp_step(nf, B, R, X, dY_ref, Ws, bs, LR, given_acts=acts)
    assert rel_err(h.dz(L - 1), dY_ref) <= 1e-6
    assert rel_err(h.dx(), ref.dX) <= FP32_TOL
    for l in range(L):
        assert rel_err(h.weight(l), ref.W_new[l]) <= FP32_TOL, f"updated W {l}"
        assert rel_err(h.bias(l), ref.b_new[l]) <= FP32_TOL, f"updated b {l}"
    np.testing.assert_allclose(h.loss()[0], loss_ref, rtol=1e-6)
    h.close()


def test_loss_decreases_over_steps_and_graph_replay_matches_eager():
    """Sign and scale of the whole chain: a few small SGD steps on fixed data reduce the loss; the
    graph-replayed steps (from the second on) give the bits of eager steps."""
    nf, B, R = [64, 96, 32], 48, 2
    losses = {}
    weights = {}
    for flags in (capi.FLAG_NO_GRAPH, 0):
        h, _ = build(nf, B, R, seed=5, flags=flags)
        seq = []
        for _ in range(5):
            h.step(1e-3)
            seq.append(h.loss()[1])
        losses[flags] = seq
        weights[flags] = [h.weight(l) for l in range(len(nf) - 1)]
        h.close()
    seq = losses[0]
    assert all(b < a for a, b in zip(seq, seq[1:])), seq
    assert losses[0] == losses[capi.FLAG_NO_GRAPH]
    for a, b in zip(weights[0], weights[capi.FLAG_NO_GRAPH]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_set_dy_leaves_loss_mode():
    nf, B, R = CONFIGS["rect"]
    h, (X, Ws, bs, labels) = build(nf, B, R, seed=3)
    h.step(LR)
    h.step(LR)  # graph captured in loss mode
    _, _, _, dY = oracle.make_problem(nf, B, R, 3)
    for l in range(len(nf) - 1):
        h.set_weights(l, Ws[l], bs[l])
    h.set_dy(dY)
    h.step(LR)
    h.sync()
    assert rel_err(h.dz(len(nf) - 2), dY) == 0.0
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR)
    for l in range(len(nf) - 1):
        assert rel_err(h.weight(l), ref.W_new[l]) <= FP32_TOL
    h.close()


def test_loss_mode_bf16_model():
    nf, B, R = [256, 256, 128], 128, 2
    L = len(nf) - 1
    h, (X, Ws, bs, labels) = build(nf, B, R, seed=13, flags=capi.FLAG_NO_GRAPH, dtype=capi.MI_BF16)
    h.step(LR)
    h.sync()
    pred = h.activation(L)   # bf16 values widened to fp32
    dY_ref, loss_ref = oracle.l2_loss(pred, labels, R)
    assert rel_err(h.dz(L - 1), dY_ref) <= 2.0 ** -8
    np.testing.assert_allclose(h.loss()[0], loss_ref, rtol=1e-6)
    acts = [h.activation(l) for l in range(L + 1)]
    ref = oracle.mlp_step(nf, B, R, X, dY_ref, Ws, bs, LR, given_acts=acts)
    for l in range(L):
        assert rel_err(h.weight(l) - Ws[l], ref.W_new[l] - Ws[l]) <= BF16_TOL, f"weight update {l}"
    h.close()


def test_bf16_explicit_loss_backward_after_set_dy_refreshes_the_transposed_gradient():
    """Per-operation use: labels, then an uploaded dY (which leaves loss mode and caches dY^T for the
    weight gradient of the last layer), then an explicit loss_backward that rewrites dY on the
    device.  The weight and bias gradient of the last layer must come from the rewritten dY."""
    nf, B, R = [256, 256, 128], 128, 2
    L = len(nf) - 1
    h, (X, Ws, bs, labels) = build(nf, B, R, seed=21, flags=capi.FLAG_NO_GRAPH, dtype=capi.MI_BF16)
    _, _, _, dY = oracle.make_problem(nf, B, R, 21)
    h.set_dy(dY)
    for l in range(L):
        h.forward(l)
    h.loss_backward()
    h.wgrad(L - 1)
    h.sync()
    dz = h.dz(L - 1)          # what the loss kernel wrote (bf16 values)
    dY_ref, _ = oracle.l2_loss(h.activation(L), labels, R)
    assert rel_err(dz, dY_ref) <= 2.0 ** -8
    assert rel_err(dz, dY) > 0.5   # nothing like the uploaded gradient
    a = h.activation(L - 1)
    for r in range(R):
        sl = slice(r * B, (r + 1) * B)
        want = dz[sl].astype(np.float64).T @ a[sl].astype(np.float64)
        assert rel_err(h.wgrad_of(L - 1, r), want) <= BF16_TOL, f"dW replica {r}"
        assert rel_err(h.bgrad_of(L - 1, r), dz[sl].astype(np.float64).sum(0)) <= BF16_TOL, f"db replica {r}"
    h.close()


def test_loss_without_labels_is_an_error():
    h = capi.MlpHandle([32, 32], 16, 1)
    with pytest.raises(capi.MiError):
        h.loss_backward()
    with pytest.raises(capi.MiError):
        h.loss()
    h.close()


@pytest.mark.parametrize("nf", [[128, 256, 128, 64], [128, 200, 128, 64]], ids=["small", "ragged"])
@pytest.mark.parametrize("flags", [0, capi.FLAG_PER_LAYER_UPDATE, capi.FLAG_SERIAL_BACKWARD])
def test_trace_step_writes_reference_style_timeline(tmp_path, flags, nf):
    B, R = 64, 2
    L = len(nf) - 1
    h, _ = build(nf, B, R, seed=9, flags=flags)
    h2, _ = build(nf, B, R, seed=9, flags=flags | capi.FLAG_NO_GRAPH)
    path = tmp_path / "trace.log"
    h.trace_step(LR, str(path))
    h2.step(LR)
    for l in range(L):  # tracing changes nothing in the arithmetic
        assert np.array_equal(h.weight(l).view(np.uint32), h2.weight(l).view(np.uint32))
    events = json.loads(path.read_text())
    begins = [e for e in events if e["ph"] == "B"]
    assert len(events) == 2 * len(begins)
    names = sorted(e["name"] for e in begins)
    paired = h.schedule()["paired_backward"]
    assert paired == (nf == [128, 256, 128, 64])   # the small model runs the fewest-launches schedule
    if paired:
        expect = [f"FC_{l}_0" for l in range(L)] + [f"FCWgtGradient+FCBwdGradient_{l}_0" for l in range(L)] + ["L2Loss_0"]
    else:
        expect = [f"FC_{l}_0" for l in range(L)] + [f"FCWgtGradient_{l}_0" for l in range(L)] + \
                 [f"FCBwdGradient_{l}_0" for l in range(L)] + ["L2Loss_0"]
    if flags & capi.FLAG_PER_LAYER_UPDATE and not paired:
        expect += [f"ReduceScatterAllGather_{l}_0" for l in range(L)]
    else:
        expect += ["ReduceScatterAllGather_all_0"]
    assert names == sorted(expect)
    # per stream: begin/end alternate and time does not run backwards
    for tid in (0, 1):
        mine = [e for e in events if e["tid"] == tid]
        assert all(e["pid"] == 0 for e in mine)
        assert [e["ph"] for e in mine] == ["B", "E"] * (len(mine) // 2)
        ts = [e["ts"] for e in mine]
        assert all(b >= a for a, b in zip(ts, ts[1:])), ts
    if paired or (flags & capi.FLAG_SERIAL_BACKWARD and not flags & capi.FLAG_PER_LAYER_UPDATE):
        assert all(e["tid"] == 0 for e in events)
    elif not flags & capi.FLAG_SERIAL_BACKWARD:
        assert any(e["tid"] == 1 for e in events)
    # forward precedes backward: FC_{L-1} ends before the backward of layer L-1 begins
    order = {e["name"]: e["ts"] for e in begins}
    first_bwd = f"FCWgtGradient+FCBwdGradient_{L - 1}_0" if paired else f"FCBwdGradient_{L - 1}_0"
    assert order[f"FC_{L - 1}_0"] <= order[first_bwd]
    h.close()
    h2.close()
