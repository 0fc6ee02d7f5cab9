"""Writes partition_golden.json.gz from the compiled reference (oracle/_ref/libref_partition.so).

Run in the build container only (needs the reference checkout to have been compiled with
`make -C oracle ref`):  python tests/golden/gen_partition_golden.py
The JSON holds inputs and the reference's outputs, nothing else.
"""
import ctypes
import gzip
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))

ref = ctypes.CDLL(os.path.join(ROOT, "oracle", "_ref", "libref_partition.so"))
I = ctypes.c_int
ref.ref_get_partition.argtypes = [I, I, I, I, ctypes.POINTER(I)]
ref.ref_get_intra_socket_2dpartition.argtypes = [I, I, ctypes.c_double, I, I, I, ctypes.POINTER(I)]
ref.ref_get_2dpartition.argtypes = [I, I, ctypes.c_double, I, I, I, I, ctypes.POINTER(I)]

# (m, n) pairs: the GEMM shapes of the benchmark configs (fwd/dX: m = R*B, dW: m = n_out), the
# reference's own default model (1024-wide, last layer n = 1), and small / ragged edge cases.
SHAPES = [
    (512, 512), (4096, 1024), (1024, 1024), (4096, 4096), (2048, 2048), (16384, 8192),
    (8192, 8192), (1024, 1), (1, 1024), (8192, 1), (1, 1), (15, 15), (16, 16), (17, 17),
    (1000, 1000), (1000, 17), (17, 1000), (100, 8), (9, 9), (33, 129),
]
ASPECTS = [4.0, 0.5]
NSOCKETS = [1, 2, 4, 8]
THREADS = [1, 4, 5, 8, 10, 16, 20, 28]
WORKS_1D = [1, 7, 16, 100, 1000, 1024, 4096, 8192, 1040 * 1024]


def main():
    out2 = (I * 2)()
    out4 = (I * 4)()
    cases_1d, cases_intra, cases_2d = [], [], []
    for ns in NSOCKETS:
        ref.ref_set_nsockets(ns)
        for T in THREADS:
            for work in WORKS_1D:
                rows = []
                for sid in range(ns):
                    for t in range(T):
                        ref.ref_get_partition(work, sid, T, t, out2)
                        rows.append(list(out2))
                cases_1d.append({"work": work, "ns": ns, "T": T, "ranges": rows})
            for (m, n) in SHAPES:
                for ar in ASPECTS:
                    for m_align in (0, 1):
                        # global version: first and last socket, every thread
                        rows = []
                        for sid in sorted({0, ns - 1}):
                            for t in range(T):
                                ref.ref_get_2dpartition(m, n, ar, m_align, sid, T, t, out4)
                                rows.append(list(out4))
                        cases_2d.append({"m": m, "n": n, "ar": ar, "m_align": m_align, "ns": ns,
                                         "T": T, "sids": sorted({0, ns - 1}), "blocks": rows})
                        if ns == 1:  # the intra-socket version does not depend on nsockets
                            rows = []
                            for t in range(T):
                                ref.ref_get_intra_socket_2dpartition(m, n, ar, m_align, T, t, out4)
                                rows.append(list(out4))
                            cases_intra.append({"m": m, "n": n, "ar": ar, "m_align": m_align,
                                                "T": T, "blocks": rows})
    doc = {
        "source": "compiled reference Partition.cc (get_partition, get_intra_socket_2dpartition, "
                  "get_2dpartition with explicit socket/thread ids)",
        "partition_1d": cases_1d,
        "partition_2d_intra": cases_intra,
        "partition_2d": cases_2d,
    }
    path = os.path.join(HERE, "partition_golden.json.gz")
    with open(path, "wb") as raw, gzip.GzipFile(fileobj=raw, mode="wb", mtime=0) as f:
        f.write(json.dumps(doc, separators=(",", ":")).encode())
    print(path, os.path.getsize(path), "bytes;", len(cases_1d), len(cases_intra), len(cases_2d), "cases")


if __name__ == "__main__":
    main()
