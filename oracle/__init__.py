"""CPU oracle of the MLP training step -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this package.
It wraps oracle/liboracle.so (built from mlp_oracle.c by `make -C oracle`) for numpy arrays, and
re-exports the pure-Python partition restatement.  Nothing under tbb_test_amd/ uses it.
"""
import ctypes
import os
import subprocess

import numpy as np

from . import partition  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None

_f32 = np.float32
_vp = ctypes.c_void_p
_ci = ctypes.c_int


def _load():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            subprocess.check_call(["make", "-C", _HERE, "liboracle.so"], stdout=subprocess.DEVNULL)
        lib = ctypes.CDLL(path)
        lib.oracle_fc_forward.argtypes = [_ci, _ci, _ci, _vp, _ci, _vp, _ci, _vp, _ci, _vp, _ci]
        lib.oracle_fc_wgrad.argtypes = [_ci, _ci, _ci, _vp, _ci, _vp, _ci, _vp, _ci, _vp]
        lib.oracle_fc_dgrad.argtypes = [_ci, _ci, _ci, _vp, _ci, _vp, _ci, _vp, _ci, _vp, _ci]
        lib.oracle_reduce_sgd.argtypes = [_vp, _vp, ctypes.c_size_t, ctypes.c_size_t, _ci, ctypes.c_float]
        lib.oracle_mlp_step.argtypes = [_ci, ctypes.POINTER(_ci), _ci, _ci, _ci, _ci, ctypes.c_float, _vp, _vp, _vp, _vp,
                                        _vp, _vp]
        lib.oracle_mlp_step.restype = _ci
        lib.oracle_l2_loss.argtypes = [_ci, _ci, _ci, _vp, _ci, _vp, _ci, _vp, _ci, _vp]
        for fn in (lib.oracle_fc_forward, lib.oracle_fc_wgrad, lib.oracle_fc_dgrad, lib.oracle_reduce_sgd, lib.oracle_l2_loss):
            fn.restype = None
        _lib = lib
    return _lib


def _c(a):
    a = np.ascontiguousarray(a, dtype=_f32)
    return a


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def fc_forward(X, W, b=None, relu=False):
    """Y = X @ W.T + b, optional ReLU (float64 accumulation, one rounding)."""
    X, W = _c(X), _c(W)
    b = None if b is None else _c(b)
    M, K = X.shape
    N = W.shape[0]
    assert W.shape[1] == K
    Y = np.empty((M, N), dtype=_f32)
    _load().oracle_fc_forward(M, N, K, _p(X), K, _p(W), K, _p(b), int(relu), _p(Y), N)
    return Y


def fc_wgrad(dZ, A):
    """(dW, db) for ONE replica: dW = dZ.T @ A, db = dZ.sum(0)."""
    dZ, A = _c(dZ), _c(A)
    K, M = dZ.shape
    N = A.shape[1]
    assert A.shape[0] == K
    dW = np.empty((M, N), dtype=_f32)
    db = np.empty((M,), dtype=_f32)
    _load().oracle_fc_wgrad(M, N, K, _p(dZ), M, _p(A), N, _p(dW), N, _p(db))
    return dW, db


def fc_dgrad(dZ, W, mask_src=None):
    """dA = dZ @ W, multiplied by [mask_src > 0] when given."""
    dZ, W = _c(dZ), _c(W)
    M, K = dZ.shape
    N = W.shape[1]
    assert W.shape[0] == K
    mask_src = None if mask_src is None else _c(mask_src)
    dA = np.empty((M, N), dtype=_f32)
    _load().oracle_fc_dgrad(M, N, K, _p(dZ), K, _p(W), N, _p(mask_src), N, _p(dA), N)
    return dA


def reduce_sgd(W, G, lr):
    """W <- fma(-lr, sum_r G[r], W) with fp32 adds in replica order.  G has shape [R, n]; returns
    the updated copy of W."""
    W = _c(W).copy()
    G = _c(G)
    R, n = G.shape
    assert W.size == n
    _load().oracle_reduce_sgd(_p(W), _p(G), n, n, R, lr)
    return W


class StepResult:
    pass


def l2_loss(pred, label, R):
    """SquaredL2Distance + AveragedLoss per replica and its gradient w.r.t. pred.
    pred, label: [R*B, N].  Returns (dY [R*B, N] float32, loss_per_replica [R] float64)."""
    pred, label = _c(pred), _c(label)
    MB, N = pred.shape
    assert label.shape == pred.shape and MB % R == 0
    dY = np.empty_like(pred)
    loss = np.zeros(R, dtype=np.float64)
    lib = _load()
    lib.oracle_l2_loss(R, MB // R, N, _p(pred), N, _p(label), N, _p(dY), N, loss.ctypes.data_as(ctypes.c_void_p))
    return dY, loss


def mlp_step(nf, B, R, X, dY, Ws, bs, lr, relu_last=False, given_acts=None):
    """Runs one full step.  Ws[l]: [nf[l+1], nf[l]], bs[l]: [nf[l+1]].
    Returns an object with acts (list of L+1 arrays), dW[r][l], db[r][l], dX, W_new[l], b_new[l].
    given_acts (list of L+1 arrays): skip the forward pass and run the backward pass on these."""
    L = len(nf) - 1
    MB = R * B
    flat = np.concatenate([np.concatenate([_c(Ws[l]).ravel(), _c(bs[l]).ravel()]) for l in range(L)])
    P = flat.size
    if given_acts is None:
        acts = np.empty(sum(MB * n for n in nf), dtype=_f32)
    else:
        acts = np.concatenate([_c(a).ravel() for a in given_acts])
        assert acts.size == sum(MB * n for n in nf)
    dWall = np.empty(R * P, dtype=_f32)
    dX = np.empty((MB, nf[0]), dtype=_f32)
    X, dY = _c(X), _c(dY)
    arr = (_ci * len(nf))(*nf)
    rc = _load().oracle_mlp_step(L, arr, B, R, int(relu_last), int(given_acts is not None), lr, _p(X), _p(dY), _p(flat), _p(acts), _p(dWall),
                                 _p(dX))
    if rc != 0:
        raise MemoryError("oracle_mlp_step failed")
    res = StepResult()
    res.acts, off = [], 0
    for n in nf:
        res.acts.append(acts[off:off + MB * n].reshape(MB, n))
        off += MB * n
    res.dW = [[None] * L for _ in range(R)]
    res.db = [[None] * L for _ in range(R)]
    res.W_new, res.b_new = [], []
    off = 0
    for l in range(L):
        nw, nb = nf[l + 1] * nf[l], nf[l + 1]
        for r in range(R):
            res.dW[r][l] = dWall[r * P + off:r * P + off + nw].reshape(nf[l + 1], nf[l])
            res.db[r][l] = dWall[r * P + off + nw:r * P + off + nw + nb]
        res.W_new.append(flat[off:off + nw].reshape(nf[l + 1], nf[l]))
        res.b_new.append(flat[off + nw:off + nw + nb])
        off += nw + nb
    res.dX = dX
    return res


# ---- seeded inputs: numpy restatement of the counter-based generator of the host library ------

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)


def _mix64(z):
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def rand_raw(seed, stream, first, count):
    """raw(seed, stream, i) for i in [first, first+count)."""
    with np.errstate(over="ignore"):
        key = _mix64(np.uint64(seed) + _GOLDEN * np.uint64(stream + 1))
        i = np.arange(first + 1, first + count + 1, dtype=np.uint64)
        return _mix64(key + _GOLDEN * i)


def rand_uniform(seed, stream, first, count, low, high):
    u = (rand_raw(seed, stream, first, count) >> np.uint64(40)).astype(np.float64) * 2.0 ** -24
    low, high = _f32(low), _f32(high)
    return (low + (high - low) * u.astype(_f32)).astype(_f32)


def rand_normal(seed, stream, first, count, mean=0.0, std=1.0):
    """Box-Muller, two counters per value, starting at counter `first`."""
    raw = rand_raw(seed, stream, first, 2 * count)
    u1 = ((raw[0::2] >> np.uint64(40)).astype(np.float64) + 1.0) * 2.0 ** -24
    u2 = (raw[1::2] >> np.uint64(40)).astype(np.float64) * 2.0 ** -24
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (_f32(mean) + _f32(std) * z.astype(_f32)).astype(_f32)


def make_problem(nf, B, R, seed):
    """Seeded inputs of one benchmark configuration: X ~ U[-1,1] (stream 0), W_l Xavier-uniform
    (stream 1+l), b = 0, dY ~ N(0,1) (stream 1000)."""
    L = len(nf) - 1
    MB = B * R
    X = rand_uniform(seed, 0, 0, MB * nf[0], -1.0, 1.0).reshape(MB, nf[0])
    Ws, bs = [], []
    for l in range(L):
        a = float(np.sqrt(6.0 / (nf[l] + nf[l + 1])))
        Ws.append(rand_uniform(seed, 1 + l, 0, nf[l + 1] * nf[l], -a, a).reshape(nf[l + 1], nf[l]))
        bs.append(np.zeros(nf[l + 1], dtype=_f32))
    dY = rand_normal(seed, 1000, 0, MB * nf[L]).reshape(MB, nf[L])
    return X, Ws, bs, dY
