"""ctypes binding of include/mi_mlp_host.h (libmi_mlp_host.so): the benchmark's host-side helpers
(work partition, ring topology, seeded fills).  No GPU involved."""
import ctypes
import os
from ctypes import POINTER, c_double, c_float, c_int, c_size_t, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ip = POINTER(c_int)

SIGNATURES = {
    "mi_host_set_nsockets": ([c_int], None),
    "mi_host_get_work_per_socket": ([c_int], c_int),
    "mi_host_get_partition": ([c_int, c_int, c_int, c_int, _ip], None),
    "mi_host_get_intra_socket_2dpartition": ([c_int, c_int, c_double, c_int, c_int, c_int, _ip], None),
    "mi_host_get_2dpartition": ([c_int, c_int, c_double, c_int, c_int, c_int, c_int, _ip], None),
    "mi_host_get_2dpartition_omp": ([c_int, c_int, c_double, c_int, c_int, _ip], c_int),
    "mi_host_get_my_ring_info": ([c_int, c_int, _ip], None),
    "mi_host_rand_seed": ([c_uint64], None),
    "mi_host_rand_stream": ([c_uint64], None),
    "mi_host_rand_raw": ([c_uint64, c_uint64, c_uint64], c_uint64),
    "mi_host_rand_uniform": ([c_void_p, c_size_t, c_float, c_float], None),
    "mi_host_rand_normal": ([c_void_p, c_size_t, c_float, c_float], None),
    "mi_host_rand_ints": ([c_void_p, c_int, c_int, c_int, c_int], c_int),
    "mi_host_init_problem": ([c_int, _ip, c_int, c_int, c_uint64, c_void_p, c_void_p, c_void_p], None),
}

_lib = None


def lib_path():
    return os.path.join(_HERE, "lib", "libmi_mlp_host.so")


def lib():
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise OSError(f"{path} is missing: build it with `make -C tbb_test_amd`")
        handle = ctypes.CDLL(path)
        for name, (argtypes, restype) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = handle
    return _lib


def partition_1d(work, nsockets, sid, T, t):
    out = (c_int * 2)()
    lib().mi_host_set_nsockets(nsockets)
    lib().mi_host_get_partition(work, sid, T, t, out)
    return tuple(out)


def partition_2d_intra(m, n, ar, m_align, T, t):
    out = (c_int * 4)()
    lib().mi_host_get_intra_socket_2dpartition(m, n, ar, int(m_align), T, t, out)
    return tuple(out)


def partition_2d(m, n, ar, m_align, nsockets, sid, T, t):
    out = (c_int * 4)()
    lib().mi_host_set_nsockets(nsockets)
    lib().mi_host_get_2dpartition(m, n, ar, int(m_align), sid, T, t, out)
    return tuple(out)


def ring_info(sid, task, nsockets):
    out = (c_int * 3)()
    lib().mi_host_set_nsockets(nsockets)
    lib().mi_host_get_my_ring_info(sid, task, out)
    return tuple(out)


def init_problem(nf, B, R, seed):
    """Seeded benchmark inputs (X, [W_l], dY) as dense numpy arrays."""
    L = len(nf) - 1
    MB = B * R
    X = np.empty((MB, nf[0]), np.float32)
    dY = np.empty((MB, nf[L]), np.float32)
    W = np.empty(sum(nf[l] * nf[l + 1] for l in range(L)), np.float32)
    arr = (c_int * len(nf))(*nf)
    lib().mi_host_init_problem(L, arr, B, R, seed, X.ctypes.data_as(c_void_p), W.ctypes.data_as(c_void_p),
                               dY.ctypes.data_as(c_void_p))
    Ws, off = [], 0
    for l in range(L):
        n = nf[l] * nf[l + 1]
        Ws.append(W[off:off + n].reshape(nf[l + 1], nf[l]))
        off += n
    return X, Ws, dY
