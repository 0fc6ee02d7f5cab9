"""CPU baseline leg of bench.py: times the restatements of the reference's two CPU schedulers on
this host's cores -- the OpenMP SPMD loop of mlp_omp (oracle/mlp_omp_port.c) and the task graph of
mlp_tbb (oracle/mlp_dag_port.cc).

TEST / MEASUREMENT INFRASTRUCTURE ONLY.  The number is a reported baseline, not a target.  The
reference itself (MKL + TBB) cannot be built in this image, so the timed code is this repository's
restatement ("kind": "port"): same thread layout, same 2-D work partition, same ring
reduce-scatter / all-gather with fused SGD, one sequential SGEMM call per thread.  SGEMM is
OpenBLAS as shipped inside scipy (single-threaded per call, like the reference uses MKL), or the
built-in kernel of the port when that library cannot be found.
"""
import ctypes
import glob
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None
_vp, _ci = ctypes.c_void_p, ctypes.c_int


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "libmlp_omp_port.so")
        if not os.path.exists(path):
            subprocess.check_call(["make", "-C", _HERE, "libmlp_omp_port.so"], stdout=subprocess.DEVNULL)
        l = ctypes.CDLL(path)
        l.port_mlp_run.argtypes = [_ci, ctypes.POINTER(_ci), _ci, _ci, _ci, ctypes.c_float, _ci, _vp, _vp, _vp, _ci,
                                   _ci, _ci, _vp, _vp, _vp, ctypes.POINTER(ctypes.c_double)]
        l.port_mlp_run.restype = _ci
        l.port_mlp_dag_run.argtypes = l.port_mlp_run.argtypes
        l.port_mlp_dag_run.restype = _ci
        l.port_mlp_run_overlap.argtypes = [_ci, ctypes.POINTER(_ci), _ci, _ci, _ci, _ci, ctypes.c_float, _ci, _vp, _vp, _vp,
                                           _ci, _ci, _ci, _vp, _vp, _vp, ctypes.POINTER(ctypes.c_double)]
        l.port_mlp_run_overlap.restype = _ci
        l.port_comm_threads.argtypes = [_ci]
        l.port_comm_threads.restype = _ci
        l.port_mlp_dag_comm_tasks.argtypes = [_ci]
        l.port_mlp_dag_comm_tasks.restype = _ci
        l.port_check_all_reduce.argtypes = [_ci, _ci, _ci, _ci]
        l.port_check_all_reduce.restype = _ci
        l.port_partition_2d.argtypes = [_ci, _ci, ctypes.c_double, _ci, _ci, _ci, _ci, _ci, ctypes.POINTER(_ci)]
        l.port_partition_2d_intra.argtypes = [_ci, _ci, ctypes.c_double, _ci, _ci, _ci, ctypes.POINTER(_ci)]
        l.port_ring_info.argtypes = [_ci, _ci, _ci, ctypes.POINTER(_ci)]
        _lib = l
    return _lib


_blas = None


def find_sgemm():
    """(address of a cblas_sgemm-compatible function or None, description)."""
    global _blas
    if _blas is not None:
        return _blas
    _blas = (None, "built-in blocked SGEMM of the port")
    try:
        import scipy
        pattern = os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)), "scipy.libs", "libscipy_openblas*.so")
        for path in sorted(glob.glob(pattern)):
            blas = ctypes.CDLL(path)
            if hasattr(blas, "scipy_cblas_sgemm"):
                if hasattr(blas, "scipy_openblas_set_num_threads"):
                    blas.scipy_openblas_set_num_threads(1)
                addr = ctypes.cast(blas.scipy_cblas_sgemm, _vp).value
                _blas = (addr, f"OpenBLAS cblas_sgemm ({os.path.basename(path)}), 1 thread per call")
                _blas_keepalive.append(blas)
                break
    except Exception:
        pass
    return _blas


_blas_keepalive = []


def host_cores():
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    return max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))


def run_port(nf, B, R, T, lr, X, dY, W_flat, warmup, iters, restore=True, relu_last=False, use_blas=True,
             scheduler="omp", comm_threads=0):
    """One call of a port.  scheduler: "omp" (SPMD loop of mlp_omp) or "dag" (task graph of mlp_tbb).
    comm_threads ("omp" only): threads per socket that run the all-reduce beside the backward GEMMs
    (the reference's OVERLAP_ALL_REDUCE schedule); 0 = every thread does both, one after the other;
    -1 = the reference's table by threads per socket (mlp_bench_common.h:40-48).
    Returns (W_out flat, dX, times_ms[5])."""
    L = len(nf) - 1
    MB = B * R
    X = np.ascontiguousarray(X, np.float32)
    dY = np.ascontiguousarray(dY, np.float32)
    W_flat = np.ascontiguousarray(W_flat, np.float32)
    W_out = np.empty_like(W_flat)
    dX = np.empty((MB, nf[0]), np.float32)
    times = (ctypes.c_double * 5)()
    arr = (_ci * len(nf))(*nf)
    sgemm = find_sgemm()[0] if use_blas else None
    tail = (lr, int(relu_last), X.ctypes.data_as(_vp), dY.ctypes.data_as(_vp), W_flat.ctypes.data_as(_vp), warmup, iters,
            int(restore), sgemm, W_out.ctypes.data_as(_vp), dX.ctypes.data_as(_vp), times)
    if scheduler == "omp" and comm_threads != 0:
        rc = lib().port_mlp_run_overlap(L, arr, B, R, T, comm_threads, *tail)
    else:
        fn = {"omp": lib().port_mlp_run, "dag": lib().port_mlp_dag_run}[scheduler]
        rc = fn(L, arr, B, R, T, *tail)
    if rc != 0:
        raise RuntimeError(f"{scheduler} port failed with {rc}")
    return W_out, dX, list(times)


def run(nf, B, R, lr, budget_s):
    """The cpu_baseline object of the bench line: whole training steps of the given model, same
    seeded inputs as the GPU run, for about budget_s seconds."""
    import oracle

    L = len(nf) - 1
    cores = host_cores()
    T = max(1, cores // R)
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=1)
    W_flat = np.concatenate([np.concatenate([Ws[l].ravel(), bs[l].ravel()]) for l in range(L)])
    flop = 3 * 2.0 * R * B * sum(nf[l] * nf[l + 1] for l in range(L))
    Tc = lib().port_comm_threads(T)   # the reference's table: communication threads from 5 threads per socket on
    _, _, t = run_port(nf, B, R, T, lr, X, dY, W_flat, 1, 1, comm_threads=Tc)          # warm caches, estimate the step time
    # two thirds of the budget for the OpenMP restatement (the reported value), one third for the task graph
    est = max(t[4] * 1e-3, 1e-6)
    iters = int(max(1, min(200, (budget_s * 2 / 3 - 2 * est) / est)))
    _, _, t = run_port(nf, B, R, T, lr, X, dY, W_flat, 1, iters, comm_threads=Tc)
    ms = t[4]
    out = {
        "value": round(flop / (ms * 1e-3) / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": R * T,
        "kind": "port",
        "ms_per_step": round(ms, 3),
        "phase_ms_per_step": {"fwd": round(t[0], 3), "wgt_grad": round(t[1], 3), "bwd": round(t[2], 3),
                              "wgt_update": round(t[3], 3)},
        "sgemm": find_sgemm()[1],
        "sample": f"{iters} full step(s) of the same workload (same model, batch and seeded inputs), "
                  f"{R} replicas x {T} threads = {R * T} OpenMP threads on {cores} host cores, "
                  + (f"{Tc} of the {T} running the all-reduce beside the backward GEMMs (OVERLAP_ALL_REDUCE), " if Tc else
                     "all-reduce after the GEMMs of a layer (the reference's table sets no communication thread aside "
                     "below 5 threads per socket), ")
                  + "restatement of mlp_omp (oracle/mlp_omp_port.c)",
    }
    # The same figures in the units and wording of the reference's report_timing()
    # (mlp_bench_common.cc:92-149): GF/s per core for the GEMM phases (mlp_omp.cc:492,584,675 count
    # 2 m n k per phase), GB/s per socket for the update with the reference's byte model
    # 2 (sockets - 1) * 4 * sum rows * cols (reduce-scatter + all-gather, mlp_omp.cc:163,288).  The
    # port keeps per-phase totals only, so the per-layer lines and the imbalance column are not given.
    nthreads = R * T
    phase_flop = 2.0 * R * B * sum(nf[l] * nf[l + 1] for l in range(L))
    ring_bytes = 2.0 * (R - 1) * 4.0 * sum(nf[l] * nf[l + 1] for l in range(L))

    def rate(amount, t_ms, per):
        return amount / (t_ms * 1e-3) / per / 1e9 if t_ms > 0 else 0.0
    out["report_timing"] = (
        f"total fwd {t[0]:g} ms/iter ({rate(phase_flop, t[0], nthreads):g} GF/s/core), "
        f"wgt_grad {t[1]:g} ms/iter ({rate(phase_flop, t[1], nthreads):g} GF/s/core), "
        f"bwd {t[2]:g} ms/iter ({rate(phase_flop, t[2], nthreads):g} GF/s/core), "
        f"wgt_update {t[3]:g} ms/iter ({rate(ring_bytes, t[3], R):g} GB/s/socket); "
        f"wall clock time {ms:g} ms/iter")
    dag_iters = int(max(1, min(100, (budget_s / 3 - est) / est)))
    _, _, td = run_port(nf, B, R, T, lr, X, dY, W_flat, 1, dag_iters, scheduler="dag")
    out["task_graph"] = {
        "value": round(flop / (td[4] * 1e-3) / 1e12, 5),
        "unit": "TFLOP/s",
        "ms_per_step": round(td[4], 3),
        "sample": f"{dag_iters} full step(s), {R} arenas x {T} threads, restatement of mlp_tbb's dependency graph "
                  "(oracle/mlp_dag_port.cc)",
    }
    return out
