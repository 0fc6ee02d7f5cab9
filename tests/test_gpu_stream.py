"""The `stream` argument of the raw entry points with a stream of the caller's.

The reference's call sites run concurrently from many host threads, each thread's operations in its
own program order (mlp_omp.cc:474-488 for the GEMMs, mlp_omp.cc:56-63 for the update).  The C ABI
expresses that order with a HIP stream.  Here the caller creates one with hipStreamCreateWithFlags
(through ctypes, on the HIP runtime that libmi_mlp.so has already loaded), enqueues

    Y = relu(X W^T + b)            mi_sgemm_nt
    dW_r = Y_r^T X_r, db_r         mi_sgemm_tn    (the forward output doubles as the upstream gradient,
                                                   as in the reference: mlp_omp.cc:565)
    W <- W - lr sum_r dW_r         mi_reduce_sgd_raw

twice in a row on it with no host synchronisation in between -- every operation reads what the one
before wrote, and the second pass reads the W the first pass updated -- then waits with
mi_stream_sync(stream) and compares with the CPU oracle run in the same order.  Bounds: 1e-4 on Y
and dW, the update bit-exact from the device's own gradients."""
import ctypes

import numpy as np
import pytest

import oracle
from conftest import FP32_TOL, close
from tbb_test_amd import capi

pytestmark = pytest.mark.gpu

HIP_STREAM_NON_BLOCKING = 1


def hip_runtime():
    capi.lib()                                  # libmi_mlp.so is linked against the runtime: it is loaded now
    rt = ctypes.CDLL("libamdhip64.so")
    rt.hipStreamCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
    rt.hipStreamDestroy.argtypes = [ctypes.c_void_p]
    rt.hipStreamQuery.argtypes = [ctypes.c_void_p]
    return rt


def _dev(a):
    return capi.DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.float32))


@pytest.mark.parametrize("B,R,K,N", [(512, 2, 512, 512),      # 128 x 64 tiles
                                     (1024, 4, 1024, 1024),   # the direct-to-LDS kernels of config 2
                                     (96, 3, 200, 72)])       # guarded tiles, dynamic replica count
def test_chain_of_raw_operations_on_a_caller_stream(B, R, K, N):
    M = B * R
    LR = 1e-3
    rng = np.random.default_rng(B + K + N)
    X = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    W0 = (rng.uniform(-1, 1, (N, K)) * np.sqrt(6.0 / (N + K))).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, N).astype(np.float32)
    rt = hip_runtime()
    lib = capi.lib()
    stream = ctypes.c_void_p()
    assert rt.hipStreamCreateWithFlags(ctypes.byref(stream), HIP_STREAM_NON_BLOCKING) == 0
    assert stream.value is not None
    dX, dW, db = _dev(X), _dev(W0), _dev(b)
    stride = N * K + 64     # replicas not back to back
    # every buffer is filled by a host-synchronous upload: nothing of the set-up is still in flight
    # on another stream when the caller's stream starts
    dY, dG, dS = _dev(np.zeros(M * N)), _dev(np.zeros(R * stride)), _dev(np.zeros(R * N))
    # the first pass's results are kept by device copies on the same stream (the update kernel with
    # one replica and lr = -1 adds its source to a zeroed destination: dst = fma(1, src, 0) = src)
    keep = [(_dev(np.zeros(M * N)), dY, M * N), (_dev(np.zeros(R * stride)), dG, R * stride), (_dev(np.zeros(N * K)), dW, N * K)]
    try:
        for turn in range(2):
            capi.check(lib.mi_sgemm_nt(M, N, K, dX.ptr, K, dW.ptr, K, dY.ptr, N, db.ptr, 1, stream))
            capi.check(lib.mi_sgemm_tn(R, N, K, B, dY.ptr, N, dX.ptr, K, dG.ptr, K, stride, dS.ptr, N, stream))
            capi.check(lib.mi_reduce_sgd_raw(dW.ptr, dG.ptr, N * K, stride, R, ctypes.c_float(LR), stream))
            if turn == 0:
                for dst, src, n in keep:
                    capi.check(lib.mi_reduce_sgd_raw(dst.ptr, src.ptr, n, n, 1, ctypes.c_float(-1.0), stream))
        capi.check(lib.mi_stream_sync(stream))
        assert rt.hipStreamQuery(stream) == 0    # nothing left on the caller's stream
        y1 = keep[0][0].to_numpy((M, N))
        g1 = keep[1][0].to_numpy((R, stride))[:, :N * K]
        w1 = keep[2][0].to_numpy((N, K))
        y2 = dY.to_numpy((M, N))
        g2 = dG.to_numpy((R, stride))[:, :N * K]
        s2 = dS.to_numpy((R, N))
        w2 = dW.to_numpy((N, K))
    finally:
        rt.hipStreamDestroy(stream)

    # first pass from W0, second pass from the device's own W after the first (so that each pass is held to 1e-4 by itself)
    for Wstart, y, g, w in ((W0, y1, g1, w1), (w1, y2, g2, w2)):
        Y = oracle.fc_forward(X, Wstart, b, relu=True)
        assert close(y, Y, FP32_TOL), "forward output"
        for r in range(R):
            sl = slice(r * B, (r + 1) * B)
            dWr, dbr = oracle.fc_wgrad(y[sl], X[sl])       # on the device's own Y: same ReLU pattern
            assert close(g[r].reshape(N, K), dWr, FP32_TOL), f"weight gradient of replica {r}"
            if y is y2:
                assert close(s2[r], dbr, FP32_TOL), f"bias gradient of replica {r}"
        want = oracle.reduce_sgd(Wstart.ravel(), g, LR).reshape(N, K)
        assert np.array_equal(w.view(np.uint32), want.view(np.uint32)), "update: bit-exact from the device's gradients"
    assert not np.array_equal(w1, W0) and not np.array_equal(w2, w1)
    assert not np.array_equal(y1, y2)   # the second forward pass saw the updated weights
