"""Pins the CPU baseline (oracle/mlp_omp_port.c, the OpenMP restatement of the reference's mlp_omp
that bench.py times) against the float64-accumulating oracle, its ring all-reduce against the
reference's closed-form start-up check (mlp_omp.cc:325-373), and its C restatement of the work
partition against the fixture produced by the compiled reference.  No GPU."""
import ctypes
import gzip
import json
import os

import numpy as np
import pytest

import oracle
from oracle import cpu_baseline as cb
from oracle import partition as P

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("ns,T", [(1, 1), (1, 3), (2, 2), (2, 5), (3, 2), (4, 2), (4, 4), (5, 3), (8, 1), (8, 2)])
def test_ring_all_reduce_known_answer(ns, T):
    assert cb.lib().port_check_all_reduce(64, 80, ns, T) == 0
    assert cb.lib().port_check_all_reduce(33, 16, ns, T) == 0  # rows not a multiple of the socket count


def test_port_partition_matches_reference_fixture():
    with gzip.open(os.path.join(HERE, "golden", "partition_golden.json.gz"), "rt") as f:
        golden = json.load(f)
    out = (ctypes.c_int * 4)()
    lib = cb.lib()
    for c in golden["partition_2d"][::7]:
        it = iter(c["blocks"])
        for sid in c["sids"]:
            for t in range(c["T"]):
                lib.port_partition_2d(c["m"], c["n"], c["ar"], c["m_align"], c["ns"], sid, c["T"], t, out)
                assert list(out) == next(it)
    out3 = (ctypes.c_int * 3)()
    for ns in (2, 4, 8):
        for sid in range(ns):
            for task in (0, 1):
                lib.port_ring_info(ns, sid, task, out3)
                assert tuple(out3) == P.ring_info(sid, task, ns)


@pytest.mark.parametrize("nf,B,R,T,relu_last", [([96, 64, 80, 32], 24, 2, 2, False), ([64, 64, 64], 16, 4, 2, True),
                                               ([100, 70, 33, 1], 10, 3, 1, False), ([48, 48], 8, 1, 4, False)])
@pytest.mark.parametrize("use_blas", [True, False])
def test_port_step_matches_oracle(nf, B, R, T, relu_last, use_blas):
    L = len(nf) - 1
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=8)
    rng = np.random.default_rng(2)
    bs = [(0.1 * rng.standard_normal(b.shape)).astype(np.float32) for b in bs]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, 0.01, relu_last=relu_last)
    flat = np.concatenate([np.concatenate([Ws[l].ravel(), bs[l].ravel()]) for l in range(L)])
    want = np.concatenate([np.concatenate([ref.W_new[l].ravel(), ref.b_new[l].ravel()]) for l in range(L)])
    got, dX, times = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 0, 1, relu_last=relu_last, use_blas=use_blas)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    assert np.abs(dX - ref.dX).max() <= 1e-5 * max(np.abs(ref.dX).max(), 1e-30)
    assert times[4] > 0
    # restoring the weights before every step makes repeated steps idempotent
    again, _, _ = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 1, 2, restore=True, relu_last=relu_last,
                              use_blas=use_blas)
    assert np.abs(again - want).max() <= 1e-5 * np.abs(want).max()


@pytest.mark.parametrize("nf,B,R,T,Tc", [([96, 64, 80, 32], 24, 2, 5, -1),    # the reference's table: 1 of 5 threads
                                        ([64, 64, 64], 16, 2, 3, 1), ([64, 64, 64], 16, 2, 4, 2),
                                        ([100, 70, 33, 1], 10, 3, 2, 1), ([48, 48], 8, 1, 3, 1),
                                        ([64, 48, 64, 32], 20, 4, 2, 1)])
def test_port_overlapped_schedule_matches_oracle(nf, B, R, T, Tc):
    """The reference's OVERLAP_ALL_REDUCE schedule (mlp_omp.cc:519-524,601-615,692-723): the last Tc
    threads of a socket run the all-gather of layer l+1 beside the weight gradient of layer l and the
    reduce-scatter of layer l beside its input gradient.  Same results as the oracle, also over
    restored and over consecutive steps."""
    L = len(nf) - 1
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=8)
    rng = np.random.default_rng(2)
    bs = [(0.1 * rng.standard_normal(b.shape)).astype(np.float32) for b in bs]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, 0.01)
    flat = np.concatenate([np.concatenate([Ws[l].ravel(), bs[l].ravel()]) for l in range(L)])
    want = np.concatenate([np.concatenate([ref.W_new[l].ravel(), ref.b_new[l].ravel()]) for l in range(L)])
    got, dX, times = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 0, 1, use_blas=False, comm_threads=Tc)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    assert np.abs(dX - ref.dX).max() <= 1e-5 * max(np.abs(ref.dX).max(), 1e-30)
    assert times[3] > 0 and times[4] > 0
    again, _, _ = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 1, 2, restore=True, use_blas=False, comm_threads=Tc)
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))
    # two un-restored steps: the all-gather of a step must have landed before the next forward pass
    step2 = oracle.mlp_step(nf, B, R, X, dY, ref.W_new, ref.b_new, 0.01)
    want2 = np.concatenate([np.concatenate([step2.W_new[l].ravel(), step2.b_new[l].ravel()]) for l in range(L)])
    got2, _, _ = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 0, 2, restore=False, use_blas=False, comm_threads=Tc)
    assert np.abs(got2 - want2).max() <= 2e-5 * np.abs(want2).max()


def test_overlap_table_and_argument_check():
    lib = cb.lib()
    assert [lib.port_comm_threads(T) for T in (1, 4, 5, 9, 10, 19, 20, 28)] == [0, 0, 1, 1, 2, 2, 4, 4]
    nf, B, R = [32, 32], 8, 2
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=1)
    flat = np.concatenate([Ws[0].ravel(), bs[0].ravel()])
    with pytest.raises(RuntimeError):   # no thread left for the GEMMs
        cb.run_port(nf, B, R, 2, 0.01, X, dY, flat, 0, 1, use_blas=False, comm_threads=2)


# ---- the task-graph restatement (mlp_tbb) -----------------------------------------------------------

@pytest.mark.parametrize("nf,B,R,T,relu_last", [([96, 64, 80, 32], 24, 2, 2, False), ([64, 64, 64], 16, 4, 2, True),
                                               ([100, 70, 33, 1], 10, 3, 1, False), ([48, 48], 8, 1, 4, False),
                                               ([64, 48, 64], 20, 2, 5, False), ([64, 64], 12, 3, 3, True)])
def test_task_graph_step_matches_oracle_and_the_spmd_port(nf, B, R, T, relu_last):
    """Final weights and dX of the dependency-graph scheduler: against the float64 oracle, and bit for
    bit against the OpenMP restatement wherever both cut the same blocks (T < 5: no threads are set
    aside for the all-reduce, so GEMM blocks and ring spans coincide)."""
    L = len(nf) - 1
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=8)
    rng = np.random.default_rng(2)
    bs = [(0.1 * rng.standard_normal(b.shape)).astype(np.float32) for b in bs]
    ref = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, 0.01, relu_last=relu_last)
    flat = np.concatenate([np.concatenate([Ws[l].ravel(), bs[l].ravel()]) for l in range(L)])
    want = np.concatenate([np.concatenate([ref.W_new[l].ravel(), ref.b_new[l].ravel()]) for l in range(L)])
    got, dX, times = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 0, 1, relu_last=relu_last, use_blas=False,
                                 scheduler="dag")
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    assert np.abs(dX - ref.dX).max() <= 1e-5 * max(np.abs(ref.dX).max(), 1e-30)
    assert times[4] > 0
    if T < 5 and (T == 1 or R < 3):
        # identical block shapes and the same left-to-right ring arithmetic.  (With T >= 2 and 3..7
        # sockets the SPMD port gives odd threads the reversed ring while the graph has a single
        # all-reduce task per socket, so the sums are associated differently.)
        omp, dX_omp, _ = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 0, 1, relu_last=relu_last, use_blas=False)
        assert np.array_equal(got.view(np.uint32), omp.view(np.uint32))
        assert np.array_equal(dX.view(np.uint32), dX_omp.view(np.uint32))
    # several passes over the same graph object, weights restored inside the step: idempotent
    again, _, _ = cb.run_port(nf, B, R, T, 0.01, X, dY, flat, 2, 3, restore=True, relu_last=relu_last, use_blas=False,
                              scheduler="dag")
    assert np.array_equal(again.view(np.uint32), got.view(np.uint32))


def test_task_graph_without_restore_accumulates_steps():
    """Two un-restored steps equal two oracle steps in sequence (the graph is re-run, not rebuilt)."""
    nf, B, R, T = [32, 48, 16], 8, 2, 2
    L = len(nf) - 1
    X, Ws, bs, dY = oracle.make_problem(nf, B, R, seed=3)
    flat = np.concatenate([np.concatenate([Ws[l].ravel(), bs[l].ravel()]) for l in range(L)])
    step1 = oracle.mlp_step(nf, B, R, X, dY, Ws, bs, 1e-3)
    step2 = oracle.mlp_step(nf, B, R, X, dY, step1.W_new, step1.b_new, 1e-3)
    want = np.concatenate([np.concatenate([step2.W_new[l].ravel(), step2.b_new[l].ravel()]) for l in range(L)])
    got, _, _ = cb.run_port(nf, B, R, T, 1e-3, X, dY, flat, 0, 2, restore=False, use_blas=False, scheduler="dag")
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()


def test_comm_task_table():
    """Threads set aside for the all-reduce (mlp_bench_common.h:40-48), at least one task."""
    lib = cb.lib()
    assert [lib.port_mlp_dag_comm_tasks(T) for T in (1, 4, 5, 9, 10, 19, 20, 28)] == [1, 1, 1, 1, 2, 2, 4, 4]
