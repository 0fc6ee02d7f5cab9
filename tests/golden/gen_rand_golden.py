"""Writes rand_golden.json: the first values of the benchmark's seeded generator, produced by the
host library (tbb_test_amd/host/Rand.cc).  The generator is this repository's own design (the
reference draws from an MKL stream that exists only inside MKL), so the fixture does not pin
parity with the reference; it pins the generator against drift: the oracle's numpy restatement,
the host library and every later revision must keep reproducing these values, or seeded test
inputs silently change.

    python tests/golden/gen_rand_golden.py
"""
import ctypes
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from tbb_test_amd import hostlib  # noqa: E402


def main():
    lib = hostlib.lib()
    doc = {"raw": [], "uniform": [], "normal": [], "problem": {}}
    for seed, stream in [(0, 0), (1, 0), (1, 1), (1234, 7), (2 ** 63 + 5, 1000)]:
        doc["raw"].append({"seed": seed, "stream": stream,
                           "values": [int(lib.mi_host_rand_raw(seed, stream, i)) for i in range(8)]})
    for seed, stream, low, high in [(1, 0, -1.0, 1.0), (42, 3, 0.0, 1.0), (7, 2, -0.1, 0.1)]:
        buf = np.empty(16, np.float32)
        lib.mi_host_rand_seed(seed)
        lib.mi_host_rand_stream(stream)
        lib.mi_host_rand_uniform(buf.ctypes.data_as(ctypes.c_void_p), buf.size, low, high)
        doc["uniform"].append({"seed": seed, "stream": stream, "low": low, "high": high,
                               "hex": [v.hex() for v in buf.astype(float)]})
    for seed, stream in [(1, 1000), (99, 5)]:
        buf = np.empty(16, np.float32)
        lib.mi_host_rand_seed(seed)
        lib.mi_host_rand_stream(stream)
        lib.mi_host_rand_normal(buf.ctypes.data_as(ctypes.c_void_p), buf.size, 0.0, 1.0)
        doc["normal"].append({"seed": seed, "stream": stream, "hex": [v.hex() for v in buf.astype(float)]})
    nf, B, R, seed = [8, 6, 4], 3, 2, 2024
    X, Ws, dY = hostlib.init_problem(nf, B, R, seed)
    doc["problem"] = {"nf": nf, "B": B, "R": R, "seed": seed,
                      "X_row0": [float(v).hex() for v in X[0]],
                      "W0_row0": [float(v).hex() for v in Ws[0][0]],
                      "W1_row0": [float(v).hex() for v in Ws[1][0]],
                      "dY_row0": [float(v).hex() for v in dY[0]]}
    path = os.path.join(HERE, "rand_golden.json")
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
