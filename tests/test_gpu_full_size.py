"""GPU parity at the full sizes of the benchmark configurations 3, 4 and 5.

Configs 3 and 4 (fp32) are small enough for the float64-accumulating oracle (a few seconds on the
host): forward compared directly, backward on the device's own activations (identical ReLU masks),
bound 1e-4.  Config 5 (bf16, 52.8 TFLOP per step) is out of the oracle's reach, so every operation
is checked on sampled rows against the oracle fed with the device's own operands, bound 2e-2, and
the update is re-derived bit-exactly on sampled rows from the device's own gradients."""
import numpy as np
import pytest

import oracle
from conftest import BF16_TOL, FP32_TOL, rel_err
from tbb_test_amd import capi, hostlib

pytestmark = pytest.mark.gpu
LR = 0.01


def build(nf, B, R, seed, dtype=capi.MI_F32, flags=0):
    X, Ws, dY = hostlib.init_problem(nf, B, R, seed)
    h = capi.MlpHandle(nf, B, R, dtype=dtype, flags=flags)
    for l in range(len(nf) - 1):
        h.set_weights(l, Ws[l], None)
    h.set_input(X)
    h.set_dy(dY)
    return h, X, Ws, dY


@pytest.mark.parametrize("name,nf,B,R", [("C3", [4096] * 5, 2048, 2), ("C4", [2048] * 21, 256, 8),
                                         # the reference's own default model (mlp_bench_common.h:26): last layer 1024 -> 1
                                         ("ref", [1024] * 7 + [1], 1024, 4)])
def test_fp32_config_full_size(name, nf, B, R):
    L = len(nf) - 1
    h, X, Ws, dY = build(nf, B, R, seed=7, flags=capi.FLAG_PER_LAYER_UPDATE)
    h.snapshot_weights()
    for _ in range(2):              # the second step replays the captured graph
        h.restore_weights()
        h.step(LR)
    bs = [np.zeros(n, np.float32) for n in nf[1:]]
    h.sync()
    acts = [h.activation(l) for l in range(L + 1)]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR)
    flips = 0
    for l in range(L + 1):
        assert rel_err(acts[l], ref.acts[l]) <= FP32_TOL, f"{name} activation {l}"
        flips += int(np.count_nonzero((acts[l] > 0) != (ref.acts[l] > 0)))
    assert flips < 1000, flips
    del ref
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, given_acts=acts)
    assert rel_err(h.dx(), ref.dX) <= FP32_TOL
    for l in range(L):
        for r in range(R):
            assert rel_err(h.wgrad_of(l, r), ref.dW[r][l]) <= FP32_TOL, (l, r)
            assert rel_err(h.bgrad_of(l, r), ref.db[r][l]) <= FP32_TOL, (l, r)
        assert rel_err(h.weight(l), ref.W_new[l]) <= FP32_TOL, l
        assert rel_err(h.bias(l), ref.b_new[l]) <= FP32_TOL, l
    h.close()


def test_bf16_config_5_full_size_sampled():
    nf, B, R = [8192] * 9, 4096, 4
    L = len(nf) - 1
    MB = B * R
    h, X, Ws, dY = build(nf, B, R, seed=5, dtype=capi.MI_BF16, flags=capi.FLAG_NO_GRAPH)
    rng = np.random.default_rng(0)
    rows = np.sort(rng.choice(MB, 16, replace=False))

    # forward, every layer: sampled rows of the device's input -> oracle -> device's output rows
    for l in range(L):
        h.forward(l)
    prev = h.activation(0)
    for l in range(L):
        cur = h.activation(l + 1)
        want = oracle.fc_forward(prev[rows], Ws[l], None, relu=(l < L - 1))
        assert rel_err(cur[rows], want) <= BF16_TOL, f"forward layer {l}"
        if l < L - 1:
            assert 0.3 < np.count_nonzero(cur[rows]) / cur[rows].size < 0.7  # ReLU keeps about half
        prev = cur
    del prev, cur

    # backward, the last two layers: weight gradient (sampled output rows m), bias gradient,
    # input gradient (sampled batch rows) -- each against the oracle on the device's operands
    ms = np.sort(rng.choice(nf[-1], 8, replace=False))
    for l in (L - 1, L - 2):
        dz = h.dz(l)                      # dY for the last layer, else the output of dgrad(l+1)
        a = h.activation(l)
        h.wgrad(l)
        for r in (0, R - 1):
            sl = slice(r * B, (r + 1) * B)
            dW = h.wgrad_of(l, r)
            want = dz[sl][:, ms].astype(np.float64).T @ a[sl].astype(np.float64)
            assert rel_err(dW[ms], want) <= BF16_TOL, f"dW layer {l} replica {r}"
            assert rel_err(h.bgrad_of(l, r), dz[sl].astype(np.float64).sum(0)) <= BF16_TOL, f"db layer {l}"
        h.dgrad(l)
        out = h.dz(l - 1)
        want = oracle.fc_dgrad(dz[rows], Ws[l], a[rows])
        assert rel_err(out[rows], want) <= BF16_TOL, f"dgrad layer {l}"
        assert np.all(out[rows][a[rows] <= 0] == 0)
        del dz, a, out

    # update of the last layer from the device's own gradients: bit-exact on sampled rows
    l = L - 1
    grads = [h.wgrad_of(l, r)[ms] for r in range(R)]
    h.reduce_sgd_layer(l, LR)
    W_new = h.weight(l)[ms]
    want = oracle.reduce_sgd(Ws[l][ms].ravel(), np.stack([g.ravel() for g in grads]), LR).reshape(len(ms), -1)
    assert np.array_equal(W_new.view(np.uint32), want.view(np.uint32))
    h.close()


@pytest.mark.parametrize("M,N,K,R", [(4096, 1024, 1024, 4), (4096, 4096, 4096, 2)])
def test_gemm_size_independent_properties_at_full_size(M, N, K, R):
    """Properties that need no oracle, at the GEMM shapes of configs 2 and 3, for the three raw
    entry points: scaling an operand by a power of two scales the result bit for bit (no tile is
    dropped, duplicated or mixed up), a second run gives the same bits, and the result of a
    one-hot operand is the selected row / column of the other operand, exactly."""
    rng = np.random.default_rng(M + N + K)
    lib = capi.lib()
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)      # forward: X [M x K]
    W = rng.uniform(-1, 1, (N, K)).astype(np.float32)      # W [N x K]
    dZ = rng.standard_normal((M, N)).astype(np.float32)    # gradient [M x N]
    dA, dW_, ddZ = (capi.DeviceBuffer.from_numpy(x) for x in (A, W, dZ))
    dA2, ddZ2 = capi.DeviceBuffer.from_numpy(2 * A), capi.DeviceBuffer.from_numpy(2 * dZ)
    out_y, out_dx, out_dw = capi.DeviceBuffer(M * N * 4), capi.DeviceBuffer(M * K * 4), capi.DeviceBuffer(R * N * K * 4)

    def fwd(x):
        capi.check(lib.mi_sgemm_nt(M, N, K, x.ptr, K, dW_.ptr, K, out_y.ptr, N, None, 0, None))
        return out_y.to_numpy((M, N))

    def dgrad(g):
        capi.check(lib.mi_sgemm_nn(M, K, N, g.ptr, N, dW_.ptr, K, out_dx.ptr, K, None, 0, None))
        return out_dx.to_numpy((M, K))

    def wgrad(g):
        capi.check(lib.mi_sgemm_tn(R, N, K, M // R, g.ptr, N, dA.ptr, K, out_dw.ptr, K, N * K, None, 0, None))
        return out_dw.to_numpy((R, N, K))

    for fn, one, two in ((fwd, dA, dA2), (dgrad, ddZ, ddZ2), (wgrad, ddZ, ddZ2)):
        base = fn(one)
        again = fn(one)
        doubled = fn(two)
        assert np.array_equal(base.view(np.uint32), again.view(np.uint32)), fn.__name__
        assert np.array_equal((2 * base).view(np.uint32), doubled.view(np.uint32)), fn.__name__
        assert np.isfinite(base).all() and np.abs(base).max() > 0

    # one-hot rows of X pick columns of W^T: Y[i, :] = W[:, k_i]
    picks = rng.integers(0, K, M)
    onehot = np.zeros((M, K), np.float32)
    onehot[np.arange(M), picks] = 1.0
    d1 = capi.DeviceBuffer.from_numpy(onehot)
    assert np.array_equal(fwd(d1), W[:, picks].T)
    for b in (dA, dW_, ddZ, dA2, ddZ2, out_y, out_dx, out_dw, d1):
        b.free()
