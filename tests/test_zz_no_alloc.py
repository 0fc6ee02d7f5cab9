"""mi_l2_loss_static -- the loss front-end for callers that cannot allocate -- against the existing
entry points it is a variant of (mi_loss_backward + mi_mlp_get_loss on a handle), through the C ABI.

Both run the same kernel with the same summation order, so the bar is bit equality: of dY
(fp32, or bf16 widened to fp32) and of the per-replica losses (doubles).  Calls come in pairs, the
second on a smaller input, because every call on a GPU shares one device-resident scratch array
that keeps the previous call's contents."""
import ctypes

import numpy as np
import pytest

import oracle
from tbb_test_amd import capi

pytestmark = pytest.mark.gpu


def handle_loss(nf, B, R, seed, dtype):
    """pred, labels, dY and per-replica losses from the handle API (the existing entry points)."""
    X, Ws, bs, _ = oracle.make_problem(nf, B, R, seed)
    rng = np.random.default_rng(seed + 1)
    labels = rng.standard_normal((R * B, nf[-1])).astype(np.float32)
    h = capi.MlpHandle(nf, B, R, dtype=dtype, flags=capi.FLAG_NO_GRAPH)
    L = len(nf) - 1
    for l in range(L):
        h.set_weights(l, Ws[l], bs[l])
    h.set_input(X)
    h.set_labels(labels)
    for l in range(L):
        h.forward(l)
    h.loss_backward()
    h.sync()
    out = h.activation(L), labels, h.dz(L - 1), h.loss()[0]
    h.close()
    return out


def to_bf16_bits(a):
    """fp32 values that are exactly representable in bf16 -> their 16-bit patterns."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    assert not np.any(u & 0xFFFF)
    return (u >> 16).astype(np.uint16)


def static_loss(dtype, R, B, N, pred, labels):
    lib = capi.lib()
    if dtype == capi.MI_BF16:
        d_pred = capi.DeviceBuffer.from_numpy(to_bf16_bits(pred))
        d_dy = capi.DeviceBuffer(R * B * N * 2)
    else:
        d_pred = capi.DeviceBuffer.from_numpy(pred)
        d_dy = capi.DeviceBuffer(R * B * N * 4)
    d_label = capi.DeviceBuffer.from_numpy(labels)
    d_loss = capi.DeviceBuffer(R * 8)
    d_dy.zero()
    d_loss.zero()
    capi.check(lib.mi_l2_loss_static(dtype, R, B, N, d_pred.ptr, d_label.ptr, d_dy.ptr, d_loss.ptr, None))
    capi.check(lib.mi_stream_sync(None))
    if dtype == capi.MI_BF16:
        dy = (d_dy.to_numpy((R * B, N), np.uint16).astype(np.uint32) << 16).view(np.float32)
    else:
        dy = d_dy.to_numpy((R * B, N), np.float32)
    loss = d_loss.to_numpy((R,), np.float64)
    for b in (d_pred, d_dy, d_label, d_loss):
        b.free()
    return dy, loss


@pytest.mark.parametrize("dtype", [capi.MI_F32, capi.MI_BF16], ids=["f32", "bf16"])
def test_static_scratch_loss_equals_handle_loss_on_two_calls_in_a_row(dtype):
    cases = [([128, 256, 320], 96, 5, 41),   # first call: 5 replicas of 96 x 320
             ([64, 33], 17, 2, 42)]          # second call, smaller: 2 replicas of 17 x 33 (ragged)
    expected = [handle_loss(nf, B, R, seed, dtype) for nf, B, R, seed in cases]
    for (nf, B, R, _), (pred, labels, dy_ref, loss_ref) in zip(cases, expected):
        dy, loss = static_loss(dtype, R, B, nf[-1], pred, labels)
        assert np.array_equal(dy.view(np.uint32), dy_ref.view(np.uint32)), (nf, B, R)
        assert np.array_equal(loss.view(np.uint64), np.asarray(loss_ref, dtype=np.float64).view(np.uint64)), (nf, B, R)
        # and the value itself is the oracle's loss on these predictions
        _, loss_oracle = oracle.l2_loss(pred, labels, R)
        np.testing.assert_allclose(loss, loss_oracle, rtol=1e-6)


def test_static_scratch_loss_rejects_what_does_not_fit():
    lib = capi.lib()
    buf = capi.DeviceBuffer(4096)
    assert lib.mi_l2_loss_static(capi.MI_F32, 1025, 1, 1, buf.ptr, buf.ptr, buf.ptr, buf.ptr, None) == -1
    assert b"1024" in lib.mi_last_error()
    assert lib.mi_l2_loss_static(capi.MI_F32, 0, 1, 1, buf.ptr, buf.ptr, buf.ptr, buf.ptr, None) == -1
    assert lib.mi_l2_loss_static(7, 1, 1, 1, buf.ptr, buf.ptr, buf.ptr, buf.ptr, None) == -1
    assert lib.mi_l2_loss_static(capi.MI_F32, 1, 1, 1, None, buf.ptr, buf.ptr, buf.ptr, None) == -1
    buf.free()
