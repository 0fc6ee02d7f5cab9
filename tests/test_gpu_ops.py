"""GPU parity of the raw C-ABI operations (mi_sgemm_nt / nn / tn, mi_reduce_sgd_raw) against the
CPU oracle on identical seeded inputs.  fp32 bound: rel-err <= 1e-4; the reduce is bit-exact."""
import ctypes

import numpy as np
import pytest

import oracle
from conftest import FP32_TOL, rel_err
from tbb_test_amd import capi

pytestmark = pytest.mark.gpu


def _dev(a):
    return capi.DeviceBuffer.from_numpy(np.ascontiguousarray(a, dtype=np.float32))


def _rand(rng, *shape):
    return rng.uniform(-1.0, 1.0, size=shape).astype(np.float32)


def run_nt(X, W, b, relu, variant=0, ld_pad=0):
    M, K = X.shape
    N = W.shape[0]
    lib = capi.lib()
    Xp = np.zeros((M, K + ld_pad), np.float32); Xp[:, :K] = X
    Wp = np.zeros((N, K + ld_pad), np.float32); Wp[:, :K] = W
    dX, dW = _dev(Xp), _dev(Wp)
    dC = capi.DeviceBuffer(max(M * (N + ld_pad), 1) * 4)
    dC.zero()
    db = _dev(b) if b is not None else None
    capi.check(lib.mi_set_gemm_variant(0, variant))
    try:
        capi.check(lib.mi_sgemm_nt(M, N, K, dX.ptr, K + ld_pad, dW.ptr, K + ld_pad, dC.ptr, N + ld_pad,
                                   db.ptr if db else None, int(relu), None))
        capi.check(lib.mi_stream_sync(None))
    finally:
        lib.mi_set_gemm_variant(0, 0)
    return dC.to_numpy((M, N + ld_pad))[:, :N]


def run_nn(dZ, W, mask, variant=0):
    M, K = dZ.shape
    N = W.shape[1]
    lib = capi.lib()
    dA, dB = _dev(dZ), _dev(W)
    dC = capi.DeviceBuffer(max(M * N, 1) * 4)
    dm = _dev(mask) if mask is not None else None
    capi.check(lib.mi_set_gemm_variant(1, variant))
    try:
        capi.check(lib.mi_sgemm_nn(M, N, K, dA.ptr, K, dB.ptr, N, dC.ptr, N, dm.ptr if dm else None, N, None))
        capi.check(lib.mi_stream_sync(None))
    finally:
        lib.mi_set_gemm_variant(1, 0)
    return dC.to_numpy((M, N))


def run_tn(dZ, A, R, variant=0, with_colsum=True):
    RK, M = dZ.shape
    N = A.shape[1]
    K = RK // R
    lib = capi.lib()
    dA, dB = _dev(dZ), _dev(A)
    stride = M * N + 64  # replicas deliberately not back to back
    dC = capi.DeviceBuffer(R * stride * 4)
    dS = capi.DeviceBuffer(R * (M + 3) * 4)
    capi.check(lib.mi_set_gemm_variant(2, variant))
    try:
        capi.check(lib.mi_sgemm_tn(R, M, N, K, dA.ptr, M, dB.ptr, N, dC.ptr, N, stride,
                                   dS.ptr if with_colsum else None, M + 3, None))
        capi.check(lib.mi_stream_sync(None))
    finally:
        lib.mi_set_gemm_variant(2, 0)
    C = dC.to_numpy((R, stride))[:, :M * N].reshape(R, M, N)
    S = dS.to_numpy((R, M + 3))[:, :M]
    return C, S


# shapes: (M, N, K).  Multiples of the MFMA tiles, tile edges, and ragged sizes that take the
# any-shape kernel.
GEMM_SHAPES = [
    (128, 128, 32), (256, 128, 64), (128, 256, 96), (512, 512, 512), (384, 640, 160),
    (64, 64, 32), (192, 64, 64),
    # split-K kernel with direct-to-LDS loads (forward GEMM, K a multiple of 256): four wavefronts and
    # one sub-block of 64 k each at K = 256; from K = 512 on eight wavefronts with two, three, five and
    # eight sub-blocks of 32 k each
    (64, 96, 256), (512, 512, 512), (64, 64, 768), (96, 64, 1280), (32, 32, 2048),
    # tile grids whose XCD-aware orders divide by something that is not a power of two:
    # 8 x 3 tiles (contiguous range per XCD), 32 x 24 tiles (super-tiles, 3 per row)
    (1024, 384, 64), (4096, 3072, 32),
    # K loops of the direct-load kernels: a single step, and the longest conditional tail of a ring of four
    (128, 128, 16), (128, 128, 320),
    # the short-K weight gradient with chained replicas at its own size (2048 x 2048 outputs, K = 256 per replica)
    (2048, 2048, 256),
    # 144 tiles of 128 x 128: fewer than the CUs, still more than the 128 up to which half tiles are chosen
    (1536, 1536, 32),
    (1, 1, 1), (5, 3, 7), (100, 130, 50), (129, 127, 33), (257, 64, 1000), (64, 1, 64), (1, 300, 17),
    # ragged but 16-byte aligned storage: the guarded MFMA kernels
    (132, 260, 100), (1000, 520, 200), (36, 4, 64), (300, 128, 36), (128, 300, 4),
    # skinny layers (one of N / M / K of the forward / weight-gradient / input-gradient GEMM at most
    # 16): the matrix-vector kernels, at the shapes of the reference's default last layer 1024 -> 1
    (4096, 1, 1024), (1, 1024, 1024), (4096, 1024, 1), (333, 16, 130), (16, 333, 130), (130, 333, 16), (50, 7, 1030),
]
VARIANTS = [0, 8, 9, 10, 11, 12, 15, 16, 17, 21, 22, 30, 31, 33, 34, 35, 36, 37, 50, 51]   # 35: weight gradient, one workgroup walks all replicas


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("shape", GEMM_SHAPES)
def test_sgemm_nt_matches_oracle(shape, variant):
    M, N, K = shape
    rng = np.random.default_rng(1000 + M + 7 * N + 13 * K)
    X, W, b = _rand(rng, M, K), _rand(rng, N, K), _rand(rng, N)
    for relu, bias in ((True, b), (False, None)):
        got = run_nt(X, W, bias, relu, variant)
        want = oracle.fc_forward(X, W, bias, relu)
        assert rel_err(got, want) <= FP32_TOL, (shape, variant, relu)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("shape", GEMM_SHAPES)
def test_sgemm_nn_matches_oracle(shape, variant):
    M, N, K = shape
    rng = np.random.default_rng(2000 + M + 7 * N + 13 * K)
    dZ, W, act = _rand(rng, M, K), _rand(rng, K, N), _rand(rng, M, N)
    act[act < 0.3] = 0.0  # a ReLU output: exact zeros and positives
    for mask in (act, None):
        got = run_nn(dZ, W, mask, variant)
        want = oracle.fc_dgrad(dZ, W, mask)
        assert rel_err(got, want) <= FP32_TOL, (shape, variant, mask is not None)
        if mask is not None:
            assert np.all(got[act <= 0] == 0.0)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("R", [1, 2, 3])
@pytest.mark.parametrize("shape", GEMM_SHAPES)
def test_sgemm_tn_matches_oracle(shape, R, variant):
    M, N, K = shape
    rng = np.random.default_rng(3000 + M + 7 * N + 13 * K + R)
    dZ, A = _rand(rng, R * K, M), _rand(rng, R * K, N)
    C, S = run_tn(dZ, A, R, variant)
    for r in range(R):
        dW, db = oracle.fc_wgrad(dZ[r * K:(r + 1) * K], A[r * K:(r + 1) * K])
        assert rel_err(C[r], dW) <= FP32_TOL, (shape, R, variant, r)
        assert rel_err(S[r], db) <= FP32_TOL, (shape, R, variant, r)


def test_sgemm_leading_dimension_padding():
    """Operands stored with the host Matrix layout (ld = ncols + 16) are read in place."""
    rng = np.random.default_rng(5)
    X, W, b = _rand(rng, 256, 128), _rand(rng, 128, 128), _rand(rng, 128)
    got = run_nt(X, W, b, True, 0, ld_pad=16)
    assert rel_err(got, oracle.fc_forward(X, W, b, True)) <= FP32_TOL


def test_sgemm_special_cases():
    """Closed forms: identity weight reproduces the input; all-negative pre-activations are
    clamped to zero by the ReLU; a one-hot row of dZ picks one row of W."""
    n = 128
    rng = np.random.default_rng(9)
    X = _rand(rng, 256, n)
    eye = np.eye(n, dtype=np.float32)
    assert np.array_equal(run_nt(X, eye, None, False), X)
    assert np.array_equal(run_nt(np.abs(X), -eye, None, True), np.zeros_like(X))
    dZ = np.zeros((128, n), np.float32)
    dZ[np.arange(128), (np.arange(128) * 5) % n] = 1.0
    W = _rand(rng, n, 256)
    assert np.array_equal(run_nn(dZ, W, None), W[(np.arange(128) * 5) % n])


# ---- reduce + SGD ------------------------------------------------------------------------------

def run_reduce(W, G, lr, stride=None):
    R, n = G.shape
    stride = n if stride is None else stride
    Gp = np.zeros((R, stride), np.float32)
    Gp[:, :n] = G
    dW, dG = _dev(W), _dev(Gp)
    lib = capi.lib()
    capi.check(lib.mi_reduce_sgd_raw(dW.ptr, dG.ptr, n, stride, R, ctypes.c_float(lr), None))
    capi.check(lib.mi_stream_sync(None))
    return dW.to_numpy((n,))


@pytest.mark.parametrize("R", [1, 2, 3, 4, 8])
def test_reduce_sgd_reference_known_answer(R):
    """The reference's own start-up check (mlp_omp.cc:325-373): G_r[i][j] = r + i + j,
    W[i][j] = i*j, lr = 1  =>  W' = i*j - ((i + j)*R + R*(R-1)/2), exactly (all values are integers
    below 2^24).  Run on the reference's layer-0 shape, padded rows included (1024 x 1040)."""
    rows, cols, ld = 1024, 1024, 1040
    i = np.arange(rows, dtype=np.float32)[:, None]
    j = np.arange(cols, dtype=np.float32)[None, :]
    W = np.zeros((rows, ld), np.float32)
    W[:, :cols] = i * j
    G = np.zeros((R, rows, ld), np.float32)
    for r in range(R):
        G[r, :, :cols] = r + i + j
    got = run_reduce(W.ravel(), G.reshape(R, -1), 1.0).reshape(rows, ld)
    expected = i * j - ((i + j) * R + R * (R - 1) / 2)
    assert np.array_equal(got[:, :cols], expected.astype(np.float32))
    assert np.all(got[:, cols:] == 0.0)


@pytest.mark.parametrize("n,stride", [(1, 1), (3, 5), (4, 4), (1023, 1023), (4096, 4100), (100003, 100004),
                                      (1 << 20, 1 << 20)])
@pytest.mark.parametrize("R", [1, 2, 4, 5, 8])
def test_reduce_sgd_bit_exact_vs_oracle(n, stride, R):
    rng = np.random.default_rng(n + R)
    W = _rand(rng, n)
    G = rng.standard_normal((R, n)).astype(np.float32)
    got = run_reduce(W, G, 0.01, stride)
    want = oracle.reduce_sgd(W, G, 0.01)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_reduce_sgd_r1_is_plain_sgd():
    rng = np.random.default_rng(3)
    W, G = _rand(rng, 5000), _rand(rng, 1, 5000)
    got = run_reduce(W, G, 0.5)
    assert rel_err(got, W.astype(np.float64) - 0.5 * G[0].astype(np.float64)) <= 1e-6


def test_argument_errors_are_reported_not_fatal():
    lib = capi.lib()
    assert lib.mi_sgemm_nt(-1, 4, 4, None, 4, None, 4, None, 4, None, 0, None) == -1
    assert b"negative" in lib.mi_last_error()
    assert lib.mi_reduce_sgd_raw(None, None, 16, 16, 0, ctypes.c_float(0.1), None) == -1
    buf = capi.DeviceBuffer(64)
    assert lib.mi_sgemm_nt(4, 4, 4, buf.ptr, 2, buf.ptr, 4, buf.ptr, 4, None, 0, None) == -1  # lda < K
    # empty problems are fine
    assert lib.mi_sgemm_nt(0, 4, 4, None, 4, None, 4, None, 4, None, 0, None) == 0
    assert lib.mi_reduce_sgd_raw(None, None, 0, 0, 2, ctypes.c_float(0.1), None) == 0


def test_k_zero_leaves_the_epilogue_of_an_all_zero_product():
    """An empty contraction is a sum of nothing: C = relu(bias), 0 and 0 (cblas_sgemm with k = 0 and
    beta = 0 writes zeros as well)."""
    rng = np.random.default_rng(11)
    M, N = 70, 130
    b = _rand(rng, N)
    got = run_nt(np.zeros((M, 0), np.float32), np.zeros((N, 0), np.float32), b, True)
    assert np.array_equal(got, np.broadcast_to(np.maximum(b, 0.0), (M, N)))
    got = run_nn(np.zeros((M, 0), np.float32), np.zeros((0, N), np.float32), None)
    assert np.array_equal(got, np.zeros((M, N), np.float32))
    C, S = run_tn(np.zeros((0, M), np.float32), np.zeros((0, N), np.float32), 2)
    assert np.array_equal(C, np.zeros((2, M, N), np.float32)) and np.array_equal(S, np.zeros((2, M), np.float32))


def test_mfma_rate_probe_reports_a_plausible_rate():
    """The register-resident MFMA loop cannot beat the published peak by more than clock tolerance
    and must come close to it: a rate far below would mean the probe measures something else."""
    lib = capi.lib()
    for dtype, peak in ((capi.MI_F32, 157.3), (capi.MI_BF16, 2516.6)):
        for operands in (1, 2):
            r = ctypes.c_double()
            capi.check(lib.mi_probe_mfma_rate(dtype, operands, ctypes.byref(r), None))
            assert 0.4 * peak < r.value < 1.1 * peak, (dtype, operands, r.value)
    assert lib.mi_probe_mfma_rate(7, 1, ctypes.byref(r), None) == -1 and b"dtype" in lib.mi_last_error()
    assert lib.mi_probe_mfma_rate(capi.MI_F32, 5, ctypes.byref(r), None) == -1
