"""GPU parity at the full sizes of the benchmark configurations 3, 4 and 5.

Configs 3 and 4 (fp32) are small enough for the float64-accumulating oracle (a few seconds on the
host): forward compared directly, backward on the device's own activations (identical ReLU masks),
bound 1e-4 norm-wise and element-wise.  Config 5 (bf16, 52.8 TFLOP per step) is out of the oracle's reach, so every operation
is checked on sampled rows against the oracle fed with the device's own operands, bound 2e-2, and
the update is re-derived bit-exactly on sampled rows from the device's own gradients."""
import numpy as np
import pytest

import oracle
from conftest import BF16_TOL, FP32_TOL, close, elem_err, rel_err
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
        assert close(acts[l], ref.acts[l], FP32_TOL), f"{name} activation {l}: {rel_err(acts[l], ref.acts[l])}, {elem_err(acts[l], ref.acts[l])}"
        flips += int(np.count_nonzero((acts[l] > 0) != (ref.acts[l] > 0)))
    assert flips < 1000, flips
    del ref
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, given_acts=acts)
    assert close(h.dx(), ref.dX, FP32_TOL), "dX"
    for l in range(L):
        for r in range(R):
            assert close(h.wgrad_of(l, r), ref.dW[r][l], FP32_TOL), (l, r)
            assert close(h.bgrad_of(l, r), ref.db[r][l], FP32_TOL), (l, r)
        assert close(h.weight(l), ref.W_new[l], FP32_TOL), l
        assert close(h.bias(l), ref.b_new[l], FP32_TOL), l
    h.close()


def test_bf16_reference_default_model_full_size():
    """The reference's default model (1024 x 6 -> 1, mlp_bench_common.h:26) as a bf16 model at full
    size: six 1024-wide layers on the MFMA kernels and the 1024 -> 1 layer on the bf16 matrix-vector
    kernels, through mi_mlp_step on the benchmarked schedule, against the fp32 oracle (2e-2, norm-wise
    and element-wise); backward on the device's own activations (identical ReLU masks)."""
    nf, B, R = [1024] * 7 + [1], 1024, 4
    L = len(nf) - 1
    h, X, Ws, dY = build(nf, B, R, seed=7, dtype=capi.MI_BF16, flags=capi.FLAG_PER_LAYER_UPDATE | capi.FLAG_KEEP_GRADIENTS)
    h.snapshot_weights()
    for _ in range(2):              # the second step replays the captured graph
        h.restore_weights()
        h.step(LR)
    h.sync()
    bs = [np.zeros(n, np.float32) for n in nf[1:]]
    acts = [h.activation(l) for l in range(L + 1)]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR)
    for l in range(L + 1):   # the free-running chain: norm-wise (rounding to bf16 accumulates from layer to layer)
        assert rel_err(acts[l], ref.acts[l]) <= BF16_TOL, f"activation {l}"
    W16 = [_widen(_to_bf16_bits(W)) for W in Ws]   # the bf16 copies the GEMMs multiply with
    for l in range(L):       # each layer on the device's own operands: both bounds
        want = oracle.fc_forward(acts[l], W16[l], None, relu=(l < L - 1))
        assert close(acts[l + 1], want, BF16_TOL), f"forward layer {l}: {rel_err(acts[l + 1], want)}, {elem_err(acts[l + 1], want)}"
    # backward, the free-running chain (every dZ_l is rounded to bf16 on the way down): norm-wise
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, given_acts=acts)
    assert rel_err(h.dx(), ref.dX) <= BF16_TOL, "dX"
    for l in range(L):
        for r in range(R):
            assert rel_err(h.wgrad_of(l, r), ref.dW[r][l]) <= BF16_TOL, (l, r)
        assert rel_err(h.weight(l), ref.W_new[l]) <= BF16_TOL, l
    # ... and every operation on the device's own operands (bf16 activations, gradients and weight
    # copies; what is left is the order of the fp32 sums and the rounding of the result): both bounds
    for l in reversed(range(L)):
        dz, a = h.dz(l), acts[l]
        out = h.dx() if l == 0 else h.dz(l - 1)
        want = oracle.fc_dgrad(dz, W16[l], a if l > 0 else None)
        assert close(out, want, BF16_TOL), f"input gradient layer {l}: {rel_err(out, want)}, {elem_err(out, want)}"
        grads, dbs = [], []
        for r in range(R):
            sl = slice(r * B, (r + 1) * B)
            dW, db = oracle.fc_wgrad(dz[sl], a[sl])
            grads.append(h.wgrad_of(l, r))
            dbs.append(h.bgrad_of(l, r))
            assert close(grads[-1], dW, BF16_TOL), f"dW layer {l} replica {r}"
            assert close(dbs[-1], db, BF16_TOL) or nf[l + 1] == 1, f"db layer {l} replica {r}"
            assert rel_err(dbs[-1], db) <= BF16_TOL, f"db layer {l} replica {r}"
        want = oracle.reduce_sgd(Ws[l].ravel(), np.stack([g.ravel() for g in grads]), LR).reshape(Ws[l].shape)
        assert np.array_equal(h.weight(l).view(np.uint32), want.view(np.uint32)), f"updated W {l}: bit-exact from the device's gradients"
        want = oracle.reduce_sgd(np.zeros(nf[l + 1], np.float32), np.stack(dbs), LR)
        assert np.array_equal(h.bias(l).view(np.uint32), want.view(np.uint32)), f"updated b {l}"
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


def _random_bf16_bits(rng, rows, cols):
    """Dense random bf16 patterns: random sign, exponent 2^-3 .. 2^2, seven random mantissa bits."""
    v = rng.integers(0, 1 << 16, (rows, cols), dtype=np.uint16)
    sign, mant, e = v & 0x8000, v & 0x7F, (v >> 7) % 6
    return (sign | ((0x7C + e) << 7) | mant).astype(np.uint16)


def _to_bf16_bits(a):
    """fp32 -> bf16 bit pattern, round to nearest even (numpy restatement of the device rounding)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _widen(bits16):
    return (np.asarray(bits16, np.uint16).astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("which", ["nt", "nn", "tn"])
def test_bf16_gemm_size_independent_properties_at_full_size(which):
    """The bf16 entry points at the GEMM shapes of config 5 -- 16384 x 8192 x 8192 for the forward and
    the input-gradient GEMM, 4 x (8192 x 8192 x 4096) for the weight gradient: 1024 tiles of 256 x 256
    per launch, far beyond what the oracle can multiply.  Properties that need no oracle: a second run
    gives the same bits; doubling an operand (exponent + 1, exact in bf16) doubles every result bit
    for bit (products and fp32 sums scale exactly, and so does the final rounding to bf16), which a
    dropped, duplicated or misplaced tile would break; a one-hot operand picks rows of the other
    operand exactly; the masked kernel writes zero exactly where the mask is not positive."""
    lib = capi.lib()
    rng = np.random.default_rng({"nt": 11, "nn": 12, "tn": 13}[which])
    if which == "tn":
        R, M, N, K = 4, 8192, 8192, 4096       # dW_r = At_r [M x K] * Bt_r [N x K]^T, fp32 out
        At, Bt = _random_bf16_bits(rng, R * M, K), _random_bf16_bits(rng, R * N, K)
        dA, dB = capi.DeviceBuffer.from_numpy(At), capi.DeviceBuffer.from_numpy(Bt)
        dA2 = capi.DeviceBuffer.from_numpy((At + 0x80).astype(np.uint16))
        out = capi.DeviceBuffer(R * M * N * 4)

        def run(a):
            capi.check(lib.mi_hgemm_tn(R, M, N, K, a.ptr, K, M * K, dB.ptr, K, N * K, out.ptr, N, M * N, None))
            capi.check(lib.mi_stream_sync(None))
            return out.to_numpy((R, M, N))
        base = run(dA)
        assert np.array_equal(base.view(np.uint32), run(dA).view(np.uint32)), "second run"
        assert np.isfinite(base).all() and np.count_nonzero(base) > 0.99 * base.size
        doubled = run(dA2)
        assert np.array_equal((2 * base).view(np.uint32), doubled.view(np.uint32)), "doubled operand"
        del doubled
        # a sampled row of every 256-row tile against float64 on the host (exact products, fp32 sums: 1e-5)
        rows = np.arange(0, M, 256) + rng.integers(0, 256, M // 256)
        for r in range(R):
            want = _widen(At[r * M + rows]).astype(np.float64) @ _widen(Bt[r * N:(r + 1) * N]).astype(np.float64).T
            assert close(base[r][rows], want, 1e-5), f"replica {r}"
        del base
        picks = rng.integers(0, K, R * M)
        onehot = np.zeros((R * M, K), np.uint16)
        onehot[np.arange(R * M), picks] = 0x3F80     # 1.0
        d1 = capi.DeviceBuffer.from_numpy(onehot)
        got = run(d1)
        for r in range(R):
            want = _widen(Bt[r * N:(r + 1) * N][:, picks[r * M:(r + 1) * M]]).T
            assert np.array_equal(got[r], want), f"one-hot rows, replica {r}"
        for b in (dA, dB, dA2, out, d1):
            b.free()
        return

    M, N, K = 16384, 8192, 8192
    A, Bm = _random_bf16_bits(rng, M, K), _random_bf16_bits(rng, N, K)
    dA, dB = capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(Bm)
    dA2 = capi.DeviceBuffer.from_numpy((A + 0x80).astype(np.uint16))
    out = capi.DeviceBuffer(M * N * 2)
    mask = dmask = None
    if which == "nn":
        mask = np.where(rng.integers(0, 2, (M, N), dtype=np.uint8) == 1, np.uint16(0x3F80), np.uint16(0xBF80))   # +1 / -1
        mask[::7, ::5] = 0                                                                                   # and some zeros
        dmask = capi.DeviceBuffer.from_numpy(mask)

    def run(a):
        if which == "nt":
            capi.check(lib.mi_hgemm_nt(M, N, K, a.ptr, K, dB.ptr, K, out.ptr, N, None, 0, None))
        else:
            capi.check(lib.mi_hgemm_nn(M, N, K, a.ptr, K, dB.ptr, K, out.ptr, N, dmask.ptr, N, None))
        capi.check(lib.mi_stream_sync(None))
        return out.to_numpy((M, N), np.uint16)
    base = run(dA)
    assert np.array_equal(base, run(dA)), "second run"
    fb = _widen(base)
    assert np.isfinite(fb).all()
    if which == "nn":
        keep = _widen(mask) > 0
        assert np.all(base[~keep] == 0), "masked entries are +0"
        assert np.count_nonzero(fb[keep]) > 0.99 * np.count_nonzero(keep)
    else:
        assert np.count_nonzero(fb) > 0.99 * fb.size
    assert np.array_equal(_widen(run(dA2)), 2 * fb), "doubled operand"
    # one sampled row of every 256-row tile against float64 on the host; bound: one rounding to bf16 (2^-8)
    rows = np.arange(0, M, 256) + rng.integers(0, 256, M // 256)
    want = _widen(A[rows]).astype(np.float64) @ _widen(Bm).astype(np.float64).T
    if which == "nn":
        want = np.where(keep[rows], want, 0.0)
    assert close(fb[rows], want, 2.0 ** -8), "sampled rows"
    del fb, base
    picks = rng.integers(0, K, M)
    onehot = np.zeros((M, K), np.uint16)
    onehot[np.arange(M), picks] = 0x3F80
    d1 = capi.DeviceBuffer.from_numpy(onehot)
    got = run(d1)
    want = np.ascontiguousarray(Bm[:, picks].T)
    if which == "nn":
        want = np.where(keep, want, np.uint16(0))
    assert np.array_equal(got, want), "one-hot rows"
    for b in (dA, dB, dA2, out, d1) + ((dmask,) if dmask else ()):
        b.free()
