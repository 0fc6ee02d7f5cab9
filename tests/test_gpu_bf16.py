"""GPU parity of the bf16 path (bf16 operands, fp32 MFMA accumulation, fp32 master weights and
gradients) against the fp32 CPU oracle.  Bound: rel-err <= 2e-2 (max|a-e| / max|e|).  Raw GEMMs
are fed bf16-representable inputs, so their only error is the accumulation order and the final
rounding of the output to bf16 (2^-9 relative); their bound is tighter and stated per test."""
import ctypes

import numpy as np
import pytest

import oracle
from conftest import BF16_TOL, rel_err
from tbb_test_amd import capi

pytestmark = pytest.mark.gpu


def to_bf16_bits(a):
    """fp32 -> bf16 bit pattern, round to nearest even (numpy restatement of the device rounding)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def from_bf16_bits(h):
    return (np.asarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def bf16_round(a):
    return from_bf16_bits(to_bf16_bits(a))


def dev16(a):
    return capi.DeviceBuffer.from_numpy(to_bf16_bits(a))


def test_bf16_helpers_round_to_nearest_even():
    x = np.array([1.0, 1.0 + 2 ** -8, 1.0 + 2 ** -7 + 2 ** -8, -3.140625, 1e-30], np.float32)
    got = bf16_round(x)
    assert got[0] == 1.0 and got[1] == 1.0 and got[2] == np.float32(1.0 + 2 ** -6) and got[3] == np.float32(-3.140625)
    # the device conversion kernel agrees bit for bit
    rng = np.random.default_rng(0)
    v = rng.standard_normal(100003).astype(np.float32)
    src = capi.DeviceBuffer.from_numpy(v)
    dst = capi.DeviceBuffer(v.size * 2)
    lib = capi.lib()
    capi.check(lib.mi_convert_f32_to_bf16(dst.ptr, src.ptr, v.size, None))
    back = capi.DeviceBuffer(v.size * 4)
    capi.check(lib.mi_convert_bf16_to_f32(back.ptr, dst.ptr, v.size, None))
    capi.check(lib.mi_stream_sync(None))
    assert np.array_equal(dst.to_numpy((v.size,), np.uint16), to_bf16_bits(v))
    assert np.array_equal(back.to_numpy((v.size,)), bf16_round(v))


HSHAPES = [(64, 64, 32), (128, 128, 64), (256, 256, 96), (512, 256, 128), (256, 512, 32), (7, 5, 9), (100, 130, 50),
           (129, 64, 40), (256, 256, 512),
           # K loops of the direct-load kernels: one step, and every length of the conditional tail after
           # the branch-free turns of the ring (two buffers at BK = 64, four at BK = 32)
           (256, 256, 64), (256, 256, 192), (256, 256, 320), (256, 256, 448),
           # twelve 256 x 256 tiles, three K steps
           (1024, 768, 192),
           # 288 tiles of 128 x 128 (72 of 256 x 256): what the automatic choice gives to the eight-wavefront
           # 128 x 128 x 64 instance; 144 tiles of 256 x 256: the smallest problem it gives to the 256 x 256 kernel
           (2048, 2304, 128), (3072, 3072, 64)]
HVARIANTS = [0, 3, 4, 5, 13, 17, 18, 19, 21, 22, 25, 27, 28, 29, 30, 32]
# 21, 22: guarded any-shape MFMA instances; 25: 19 without wave priorities; 27, 28: 16x16x32 MFMAs;
# 29 / 30: 27 with all / pairs of the batch entries of a weight gradient chained in one workgroup;
# 32: the 256 x 256 x 64 tile with four wavefronts of 128 x 128 and a hand-ordered K step


@pytest.mark.parametrize("variant", HVARIANTS)
@pytest.mark.parametrize("shape", HSHAPES)
def test_hgemm_forward_and_input_gradient(shape, variant):
    M, N, K = shape
    rng = np.random.default_rng(M + 3 * N + 5 * K)
    A = bf16_round(rng.uniform(-1, 1, (M, K)))
    B = bf16_round(rng.uniform(-1, 1, (N, K)))
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    act = bf16_round(np.maximum(rng.uniform(-1, 1, (M, N)), 0))
    lib = capi.lib()
    dA, dB, dbias, dact = dev16(A), dev16(B), capi.DeviceBuffer.from_numpy(bias), dev16(act)
    dC = capi.DeviceBuffer(M * N * 2)
    capi.check(lib.mi_set_hgemm_variant(variant))
    try:
        capi.check(lib.mi_hgemm_nt(M, N, K, dA.ptr, K, dB.ptr, K, dC.ptr, N, dbias.ptr, 1, None))
        capi.check(lib.mi_stream_sync(None))
        got = from_bf16_bits(dC.to_numpy((M, N), np.uint16))
        assert rel_err(got, oracle.fc_forward(A, B, bias, True)) <= 4e-3, (shape, variant)
        # input gradient: C = A * Bt^T with the mask; the oracle takes the untransposed weight
        capi.check(lib.mi_hgemm_nn(M, N, K, dA.ptr, K, dB.ptr, K, dC.ptr, N, dact.ptr, N, None))
        capi.check(lib.mi_stream_sync(None))
        got = from_bf16_bits(dC.to_numpy((M, N), np.uint16))
        want = oracle.fc_dgrad(A, np.ascontiguousarray(B.T), act)
        assert rel_err(got, want) <= 4e-3, (shape, variant)
        assert np.all(got[act <= 0] == 0.0)
    finally:
        lib.mi_set_hgemm_variant(0)


# one dimension of at most 16: the matrix-vector kernels (forward: N, weight gradient: M, input gradient: K)
SKINNY_SHAPES = [(4096, 1, 1024), (1, 1024, 1024), (4096, 1024, 1), (300, 16, 200), (16, 300, 200), (300, 200, 16),
                 (50, 3, 77), (5, 130, 33), (61, 67, 2), (2, 3, 1000), (1, 1, 1)]


@pytest.mark.parametrize("shape", SKINNY_SHAPES)
def test_hgemm_skinny_shapes_all_entry_points(shape):
    """Layers of at most 16 outputs, as the reference's default model ends in (1024 -> 1,
    mlp_bench_common.h:26): forward (bias, ReLU on and off), input gradient with mask, and the
    batched fp32-result product of the weight gradient, each against the oracle.  Inputs are exact
    in bf16, so only the order of the fp32 sums and the final rounding differ."""
    M, N, K = shape
    rng = np.random.default_rng(7 * M + 3 * N + K)
    A = bf16_round(rng.uniform(-1, 1, (M, K)))
    B = bf16_round(rng.uniform(-1, 1, (N, K)))
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    act = bf16_round(np.maximum(rng.uniform(-1, 1, (M, N)), 0))
    lib = capi.lib()
    dA, dB, dbias, dact = dev16(A), dev16(B), capi.DeviceBuffer.from_numpy(bias), dev16(act)
    dC = capi.DeviceBuffer(M * N * 2)
    for relu in (1, 0):
        capi.check(lib.mi_hgemm_nt(M, N, K, dA.ptr, K, dB.ptr, K, dC.ptr, N, dbias.ptr, relu, None))
        capi.check(lib.mi_stream_sync(None))
        got = from_bf16_bits(dC.to_numpy((M, N), np.uint16))
        assert rel_err(got, oracle.fc_forward(A, B, bias, bool(relu))) <= 4e-3, (shape, relu)
    capi.check(lib.mi_hgemm_nn(M, N, K, dA.ptr, K, dB.ptr, K, dC.ptr, N, dact.ptr, N, None))
    capi.check(lib.mi_stream_sync(None))
    got = from_bf16_bits(dC.to_numpy((M, N), np.uint16))
    assert rel_err(got, oracle.fc_dgrad(A, np.ascontiguousarray(B.T), act)) <= 4e-3, shape
    assert np.all(got[act <= 0] == 0.0)
    # weight-gradient form: R batch entries, fp32 results, entries and results not back to back
    # (result stride: once odd, once a multiple of 16 bytes, which allows vector stores)
    R = 3
    sa, sb = M * K + 8, N * K + 16
    At = np.zeros((R, sa), np.float32)
    Bt = np.zeros((R, sb), np.float32)
    for r in range(R):
        At[r, :M * K] = bf16_round(rng.standard_normal(M * K))
        Bt[r, :N * K] = bf16_round(rng.uniform(-1, 1, N * K))
    dAt, dBt = dev16(At), dev16(Bt)
    for sc in (M * N + 5, (M * N + 3) // 4 * 4 + 8):
        dW = capi.DeviceBuffer(R * sc * 4)
        dW.zero()
        capi.check(lib.mi_hgemm_tn(R, M, N, K, dAt.ptr, K, sa, dBt.ptr, K, sb, dW.ptr, N, sc, None))
        capi.check(lib.mi_stream_sync(None))
        out = dW.to_numpy((R, sc))
        for r in range(R):
            want = At[r, :M * K].reshape(M, K).astype(np.float64) @ Bt[r, :N * K].reshape(N, K).astype(np.float64).T
            assert rel_err(out[r, :M * N].reshape(M, N), want) <= 1e-5, (shape, r, sc)
            assert np.all(out[r, M * N:] == 0)


@pytest.mark.parametrize("shape", [(130, 70, 100), (64, 64, 64), (33, 200, 17)])
def test_hgemm_on_operands_that_allow_no_vector_access(shape):
    """Operands that start one element past a 16-byte boundary, with leading dimensions that are
    not multiples of 8: the guarded MFMA instances read them element by element."""
    M, N, K = shape
    rng = np.random.default_rng(M * N + K)
    lda, ldb, ldc = K + 3, K + 5, N + 1
    A = bf16_round(rng.uniform(-1, 1, (M, lda)))
    B = bf16_round(rng.uniform(-1, 1, (N, ldb)))
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    lib = capi.lib()
    pad = np.zeros(1, np.uint16)
    dA = capi.DeviceBuffer.from_numpy(np.concatenate([pad, to_bf16_bits(A).ravel()]))
    dB = capi.DeviceBuffer.from_numpy(np.concatenate([pad, to_bf16_bits(B).ravel()]))
    dbias = capi.DeviceBuffer.from_numpy(bias)
    dC = capi.DeviceBuffer((1 + M * ldc) * 2)
    dC.zero()
    capi.check(lib.mi_hgemm_nt(M, N, K, dA.ptr + 2, lda, dB.ptr + 2, ldb, dC.ptr + 2, ldc, dbias.ptr, 0, None))
    capi.check(lib.mi_stream_sync(None))
    out = from_bf16_bits(dC.to_numpy((1 + M * ldc,), np.uint16))[1:].reshape(M, ldc)
    assert rel_err(out[:, :N], oracle.fc_forward(A[:, :K], B[:, :K], bias, False)) <= 4e-3
    assert np.all(out[:, N:] == 0)   # nothing written between the rows of C


@pytest.mark.parametrize("variant", [0, 27])
@pytest.mark.parametrize("ldc_extra,c_shift", [(4, 0), (0, 1), (8, 0)])
def test_hgemm_16x16x32_kernel_gives_way_when_c_or_the_mask_allow_no_16_byte_access(variant, ldc_extra, c_shift):
    """The 16x16x32 kernel writes C and reads the ReLU mask in 16-byte pieces.  With a leading
    dimension of C that is no multiple of 8, or C (or the mask) starting off a 16-byte boundary, the
    32x32x16 kernel of the same tile runs instead: results as good, nothing written between rows.
    (ldc_extra = 8 keeps the alignment: the 16x16x32 kernel itself with a padded C.)"""
    M, N, K = 512, 256, 128
    rng = np.random.default_rng(ldc_extra * 7 + c_shift)
    A = bf16_round(rng.uniform(-1, 1, (M, K)))
    B = bf16_round(rng.uniform(-1, 1, (N, K)))
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    act = bf16_round(np.maximum(rng.uniform(-1, 1, (M, N)), 0))
    ldc = N + ldc_extra
    lib = capi.lib()
    dA, dB, dbias = dev16(A), dev16(B), capi.DeviceBuffer.from_numpy(bias)
    mask_padded = np.zeros((M, ldc), np.uint16)
    mask_padded[:, :N] = to_bf16_bits(act)
    dmask = capi.DeviceBuffer.from_numpy(np.concatenate([np.zeros(c_shift, np.uint16), mask_padded.ravel()]))
    dC = capi.DeviceBuffer((c_shift + M * ldc) * 2)
    capi.check(lib.mi_set_hgemm_variant(variant))
    try:
        for kind in ("forward", "input gradient"):
            dC.zero()
            if kind == "forward":
                capi.check(lib.mi_hgemm_nt(M, N, K, dA.ptr, K, dB.ptr, K, dC.ptr + 2 * c_shift, ldc, dbias.ptr, 1, None))
                want = oracle.fc_forward(A, B, bias, True)
            else:
                capi.check(lib.mi_hgemm_nn(M, N, K, dA.ptr, K, dB.ptr, K, dC.ptr + 2 * c_shift, ldc,
                                           dmask.ptr + 2 * c_shift, ldc, None))
                want = oracle.fc_dgrad(A, np.ascontiguousarray(B.T), act)
            capi.check(lib.mi_stream_sync(None))
            out = from_bf16_bits(dC.to_numpy((c_shift + M * ldc,), np.uint16))[c_shift:].reshape(M, ldc)
            assert rel_err(out[:, :N], want) <= 4e-3, kind
            assert np.all(out[:, N:] == 0), kind
    finally:
        lib.mi_set_hgemm_variant(0)


@pytest.mark.parametrize("variant", HVARIANTS)
@pytest.mark.parametrize("R", [1, 3])
@pytest.mark.parametrize("shape", HSHAPES)
def test_hgemm_weight_gradient_via_transposed_copies(shape, R, variant):
    """dW_r = dZ_r^T A_r computed from the K-contiguous copies dZ_r^T, A_r^T that
    mi_transpose_bf16 makes; fp32 output; bias gradient from mi_rowsum_bf16."""
    M, N, K = shape
    rng = np.random.default_rng(M + N + K + R)
    dZ = bf16_round(rng.standard_normal((R * K, M)))
    A = bf16_round(rng.uniform(-1, 1, (R * K, N)))
    lib = capi.lib()
    d_dz, d_a = dev16(dZ), dev16(A)
    d_dzT, d_aT = capi.DeviceBuffer(R * M * K * 2), capi.DeviceBuffer(R * N * K * 2)
    dC = capi.DeviceBuffer(R * M * N * 4)
    dS = capi.DeviceBuffer(R * M * 4)
    capi.check(lib.mi_transpose_bf16(R, K, M, d_dz.ptr, M, K * M, d_dzT.ptr, K, M * K, None))
    capi.check(lib.mi_transpose_bf16(R, K, N, d_a.ptr, N, K * N, d_aT.ptr, K, N * K, None))
    capi.check(lib.mi_set_hgemm_variant(variant))
    try:
        capi.check(lib.mi_hgemm_tn(R, M, N, K, d_dzT.ptr, K, M * K, d_aT.ptr, K, N * K, dC.ptr, N, M * N, None))
    finally:
        lib.mi_set_hgemm_variant(0)
    capi.check(lib.mi_rowsum_bf16(R, M, K, d_dzT.ptr, K, M * K, dS.ptr, M, None))
    capi.check(lib.mi_stream_sync(None))
    assert np.array_equal(d_dzT.to_numpy((R, M, K), np.uint16),
                          to_bf16_bits(dZ).reshape(R, K, M).transpose(0, 2, 1))  # the transpose is exact
    C = dC.to_numpy((R, M, N))
    S = dS.to_numpy((R, M))
    for r in range(R):
        dW, db = oracle.fc_wgrad(dZ[r * K:(r + 1) * K], A[r * K:(r + 1) * K])
        assert rel_err(C[r], dW) <= 1e-4, (shape, R, variant)   # fp32 output of exact bf16 products
        assert rel_err(S[r], db) <= 1e-4


@pytest.mark.parametrize("variant", [29, 30])
@pytest.mark.parametrize("R,K", [(2, 256), (4, 256), (3, 384), (4, 512), (2, 640), (6, 256), (2, 320), (2, 128)])
def test_hgemm_weight_gradient_with_chained_replicas(R, K, variant):
    """The 16x16x32 kernel walking several replicas of a weight gradient in one workgroup (variant 29:
    all of them, 30: pairs): K loops of 4, 6, 8 and 10 steps per replica (the chain needs an even
    number of at least four; K = 320 and 128 fall back to one workgroup per replica), six output
    tiles, replicas and operands not back to back.  Against the oracle per replica, and bit for bit
    against the same kernel without chaining (the summation order within a replica is the same)."""
    M, N = 512, 768
    rng = np.random.default_rng(R * 1000 + K + variant)
    sa, sb, sc = M * K + 256, N * K + 512, M * N + 64      # element strides between replicas
    At = np.zeros((R, sa), np.float32)
    Bt = np.zeros((R, sb), np.float32)
    for r in range(R):
        At[r, :M * K] = bf16_round(rng.standard_normal(M * K))
        Bt[r, :N * K] = bf16_round(rng.uniform(-1, 1, N * K))
    lib = capi.lib()
    dA, dB = dev16(At), dev16(Bt)
    out = {}
    for v in (variant, 27):
        dC = capi.DeviceBuffer(R * sc * 4)
        dC.zero()
        capi.check(lib.mi_set_hgemm_variant(v))
        try:
            capi.check(lib.mi_hgemm_tn(R, M, N, K, dA.ptr, K, sa, dB.ptr, K, sb, dC.ptr, N, sc, None))
            capi.check(lib.mi_stream_sync(None))
        finally:
            lib.mi_set_hgemm_variant(0)
        out[v] = dC.to_numpy((R, sc))
        dC.free()
    for r in range(R):
        a, b = At[r, :M * K].reshape(M, K), Bt[r, :N * K].reshape(N, K)
        want = a.astype(np.float64) @ b.astype(np.float64).T
        assert rel_err(out[variant][r, :M * N].reshape(M, N), want) <= 1e-5, f"replica {r}"
        assert np.all(out[variant][r, M * N:] == 0), "nothing written between the replicas"
    assert np.array_equal(out[variant].view(np.uint32), out[27].view(np.uint32))


def test_reduce_sgd_writes_bf16_copy():
    rng = np.random.default_rng(4)
    n, R = 100003, 4
    W = rng.uniform(-1, 1, n).astype(np.float32)
    G = rng.standard_normal((R, n)).astype(np.float32)
    dW, dG = capi.DeviceBuffer.from_numpy(W), capi.DeviceBuffer.from_numpy(G)
    d16 = capi.DeviceBuffer(n * 2 + 16)
    capi.check(capi.lib().mi_reduce_sgd_bf16_raw(dW.ptr, d16.ptr, dG.ptr, n, n, R, ctypes.c_float(0.01), None))
    capi.check(capi.lib().mi_stream_sync(None))
    want = oracle.reduce_sgd(W, G, 0.01)
    got = dW.to_numpy((n,))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(d16.to_numpy((n,), np.uint16), to_bf16_bits(want))


@pytest.mark.parametrize("rows,cols", [(128, 192), (64, 64), (512, 320), (128, 512), (192, 256), (100, 70), (64, 72)])
@pytest.mark.parametrize("R", [1, 3, 4])
def test_reduce_sgd_writes_both_bf16_copies_in_one_pass(rows, cols, R):
    """The update of one weight matrix with the bf16 copy and the transposed bf16 copy (tiled kernel
    for multiples of 64, flat kernel + transpose otherwise): fp32 result bit-exact against the
    oracle, both copies equal to its rounding; replica stride larger than the matrix."""
    rng = np.random.default_rng(rows + cols + R)
    n, stride = rows * cols, rows * cols + 256
    W = rng.uniform(-1, 1, n).astype(np.float32)
    G = rng.standard_normal((R, stride)).astype(np.float32)
    dW, dG = capi.DeviceBuffer.from_numpy(W), capi.DeviceBuffer.from_numpy(G)
    d16, d16t = capi.DeviceBuffer(n * 2), capi.DeviceBuffer(n * 2)
    capi.check(capi.lib().mi_reduce_sgd_bf16t_raw(dW.ptr, d16.ptr, d16t.ptr, dG.ptr, rows, cols, stride, R,
                                                  ctypes.c_float(0.01), None))
    capi.check(capi.lib().mi_stream_sync(None))
    want = oracle.reduce_sgd(W, G[:, :n], 0.01)
    assert np.array_equal(dW.to_numpy((n,)).view(np.uint32), want.view(np.uint32))
    want16 = to_bf16_bits(want).reshape(rows, cols)
    assert np.array_equal(d16.to_numpy((rows, cols), np.uint16), want16)
    assert np.array_equal(d16t.to_numpy((cols, rows), np.uint16), want16.T)


@pytest.mark.parametrize("rows,cols", [(2368, 2304), (2304, 2368)])
def test_reduce_sgd_both_bf16_copies_in_the_streaming_regime(rows, cols):
    """A matrix beyond what the caches hold ((R + 1) * rows * cols * 4 bytes > 192 MB) takes the
    streaming instance of the tiled update: non-temporal accesses and the tiles walked in bands of 16
    tile rows -- 64 x 128 tiles when the width is a multiple of 128 (2304: 37 tile rows, i.e. two
    whole bands and one of 5 rows), 64 x 64 tiles otherwise (2368 columns).  R = 8, the replicas'
    gradients not back to back.  Same bars as the cached regime: fp32 bit-exact, both copies equal to
    its rounding; then the flat kernel with the bf16 copy in the same regime."""
    R, tail = 8, 2368 + 64
    rng = np.random.default_rng(99)
    n = rows * cols
    stride = n + tail
    assert (R + 1) * n * 4 > 192e6
    W = rng.uniform(-1, 1, stride).astype(np.float32)
    G = rng.standard_normal((R, stride)).astype(np.float32)
    dW, dG = capi.DeviceBuffer.from_numpy(W), capi.DeviceBuffer.from_numpy(G)
    d16, d16t = capi.DeviceBuffer(stride * 2), capi.DeviceBuffer(n * 2)
    capi.check(capi.lib().mi_reduce_sgd_bf16t_raw(dW.ptr, d16.ptr, d16t.ptr, dG.ptr, rows, cols, stride, R,
                                                  ctypes.c_float(0.01), None))
    capi.check(capi.lib().mi_stream_sync(None))
    want = oracle.reduce_sgd(W[:n], G[:, :n], 0.01)
    assert np.array_equal(dW.to_numpy((stride,))[:n].view(np.uint32), want.view(np.uint32))
    want16 = to_bf16_bits(want).reshape(rows, cols)
    assert np.array_equal(d16.to_numpy((stride,), np.uint16)[:n].reshape(rows, cols), want16)
    assert np.array_equal(d16t.to_numpy((cols, rows), np.uint16), want16.T)
    # the flat kernel with the bf16 copy in the same regime (non-temporal bf16 store)
    dW2 = capi.DeviceBuffer.from_numpy(W)
    d16b = capi.DeviceBuffer(stride * 2)
    capi.check(capi.lib().mi_reduce_sgd_bf16_raw(dW2.ptr, d16b.ptr, dG.ptr, stride, stride, R, ctypes.c_float(0.01), None))
    capi.check(capi.lib().mi_stream_sync(None))
    want_all = oracle.reduce_sgd(W, G, 0.01)
    assert np.array_equal(dW2.to_numpy((stride,)).view(np.uint32), want_all.view(np.uint32))
    assert np.array_equal(d16b.to_numpy((stride,), np.uint16), to_bf16_bits(want_all))
    for b in (dW, dG, d16, d16t, dW2, d16b):
        b.free()


LR = 0.01
STEP_CONFIGS = {
    "square": ([256, 256, 256, 256], 128, 2),
    "rect": ([256, 512, 128, 384], 128, 3),
    "ragged": ([100, 72, 40, 24], 37, 2),
    "skinny_last": ([128, 96, 1], 64, 2),        # the reference's default model ends like this
    "skinny_hidden": ([128, 8, 128], 64, 2),     # every GEMM of both layers has one small dimension
}


def _check_bf16_step(nf, B, R, flags, seed=31, expect_fused=None):
    L = len(nf) - 1
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=seed)
    rng = np.random.default_rng(1)
    bs = [(0.1 * rng.standard_normal(b.shape)).astype(np.float32) for b in bs]
    h = capi.MlpHandle(nf, B, R, dtype=capi.MI_BF16, flags=flags)
    for l in range(L):
        h.set_weights(l, Ws[l], bs[l])
    h.set_input(X)
    h.set_dy(dY)
    for _ in range(1 if flags & capi.FLAG_NO_GRAPH else 2):   # with graphs: the second call is the replay
        h.snapshot_weights() if _ == 0 else h.restore_weights()
        h.step(LR)
    h.sync()
    if expect_fused is not None:  # the transposed operand copies came out of the GEMM epilogues, not a fallback
        assert h.schedule()["fused_transposes"] == expect_fused
    relu_last = bool(flags & capi.FLAG_RELU_LAST)
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, relu_last=relu_last)
    acts = [h.activation(l) for l in range(L + 1)]
    for l in range(L + 1):
        assert rel_err(acts[l], ref.acts[l]) <= BF16_TOL, f"activation {l}"
    # The ReLU mask [A > 0] is discontinuous: about one activation in a hundred lies closer to
    # zero than the bf16 forward error, and each such flip changes a gradient entry by its full
    # size.  The backward pass is therefore compared with the fp32 oracle evaluated on the
    # device's own (bf16) activations, i.e. with identical masks.
    flipped = sum(int(np.count_nonzero((acts[l] > 0) != (ref.acts[l] > 0))) for l in range(1, L))
    total = sum(acts[l].size for l in range(1, L))
    assert flipped <= 0.03 * total, f"{flipped} of {total} masks differ"
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, LR, given_acts=acts, relu_last=relu_last)
    assert rel_err(h.dx(), ref.dX) <= BF16_TOL
    for l in range(L):
        for r in range(R):
            assert rel_err(h.wgrad_of(l, r), ref.dW[r][l]) <= BF16_TOL, (l, r)
            assert rel_err(h.bgrad_of(l, r), ref.db[r][l]) <= BF16_TOL, (l, r)
        assert rel_err(h.weight(l), ref.W_new[l]) <= BF16_TOL
        if nf[l + 1] > 16:
            assert rel_err(h.bias(l), ref.b_new[l]) <= BF16_TOL
        else:
            # a handful of entries (one, for a layer of one output): the norm-wise bound has no large
            # neighbour to lean on and b - lr * sum(db) may cancel, so the bound is put on the update
            assert rel_err(h.bias(l) - bs[l], ref.b_new[l] - bs[l]) <= BF16_TOL
    h.close()


@pytest.mark.parametrize("name", list(STEP_CONFIGS))
@pytest.mark.parametrize("flags", [capi.FLAG_NO_GRAPH, 0, capi.FLAG_PER_LAYER_UPDATE,
                                   capi.FLAG_NO_GRAPH | capi.FLAG_RELU_LAST, capi.FLAG_RELU_LAST | capi.FLAG_PER_LAYER_UPDATE])
def test_bf16_step_matches_fp32_oracle(name, flags):
    nf, B, R = STEP_CONFIGS[name]
    _check_bf16_step(nf, B, R, flags)


@pytest.mark.parametrize("variant", [13, 17, 18, 19, 25, 27, 28, 32])
@pytest.mark.parametrize("flags", [capi.FLAG_NO_GRAPH, 0])
def test_bf16_step_on_the_large_tile_kernels(variant, flags):
    """The direct-load kernels (256 x 256 and 128 x 128 tiles), which small models never pick by
    themselves: whole steps against the full oracle with their fused transposed outputs (staged
    through the LDS) and the ReLU mask tile brought into the LDS.  The per-replica batch is a
    multiple of the tile height, which the fused transposed output needs; the test asserts that
    all 2 (L-1) transposed copies were written by the GEMM epilogues."""
    lib = capi.lib()
    capi.check(lib.mi_set_hgemm_variant(variant))
    try:
        nf = [256, 512, 256, 512, 256]
        _check_bf16_step(nf, 256, 2, flags, seed=77, expect_fused=2 * (len(nf) - 2))
    finally:
        lib.mi_set_hgemm_variant(0)


def test_bf16_step_falls_back_to_transpose_launches_when_the_batch_does_not_fit_the_tile():
    lib = capi.lib()
    capi.check(lib.mi_set_hgemm_variant(19))
    try:
        _check_bf16_step([256, 512, 256], 128, 2, capi.FLAG_NO_GRAPH, seed=78, expect_fused=0)
    finally:
        lib.mi_set_hgemm_variant(0)


@pytest.mark.parametrize("flags", [capi.FLAG_NO_GRAPH, 0])
def test_fused_transposes_are_counted_per_layer_when_only_some_layers_allow_them(flags):
    """Widths 64 100 64 64 64 64: the GEMMs around the 100-wide activation run on the guarded tiles,
    which write no transposed copy.  A_3^T, A_4^T (forward of layers 2, 3) and dZ_1^T, dZ_2^T, dZ_3^T
    (input gradient of layers 2, 3, 4) come out of GEMM epilogues, A_1^T, A_2^T and dZ_0^T from
    transpose launches: 5 fused copies, counted per layer although dZ rotates through 3 buffers
    (dZ_0 and dZ_3 share one)."""
    _check_bf16_step([64, 100, 64, 64, 64, 64], 64, 2, flags, seed=41, expect_fused=5)


def test_bf16_master_weights_stay_fp32():
    """The update is applied to the fp32 master copy: a step whose update is far below bf16
    resolution still changes the weights."""
    nf, B, R = [128, 128], 64, 1
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=2)
    h = capi.MlpHandle(nf, B, R, dtype=capi.MI_BF16, flags=capi.FLAG_NO_GRAPH)
    h.set_weights(0, Ws[0], bs[0])
    h.set_input(X)
    h.set_dy(dY)
    h.step(1e-7)
    h.sync()
    W1 = h.weight(0)
    assert not np.array_equal(W1, Ws[0])
    assert np.abs(W1 - Ws[0]).max() < 1e-4
    h.close()
