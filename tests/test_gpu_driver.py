"""The mlp_hip executable end to end on the GPU: start-up self-test of the reduce (the reference's
check_all_reduce_correctness, mlp_omp.cc:325-373), the timed loop, report and checksum, and the
optional loss front-end and timeline."""
import json
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tbb_test_amd", "bin", "mlp_hip")


def run(*args):
    out = subprocess.run([EXE, *args], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    return out.stdout


def test_driver_runs_config_and_prints_report_and_checksum():
    text = run("2", "--config", "C1", "--warmup", "1", "--iters", "3")
    assert "config C1: 3 layers" in text
    assert re.search(r"step [0-9.e+-]+ ms, [0-9.e+-]+ TFLOP/s", text)
    assert "nan" not in text.lower()


def test_report_timing_figures_are_consistent():
    """The per-layer lines of report_timing (format of mlp_bench_common.cc:92-149): the rate printed
    for a phase is the phase's FLOP (2 * rows * N_l * N_{l+1}, mlp_omp.cc:492,584,675) over the
    printed time, the total line adds the layers up, and the update moves (R + 2) * 4 bytes per
    parameter."""
    text = run("4", "--config", "C2", "--warmup", "2", "--iters", "5")
    rows, width, L, R = 4 * 1024, 1024, 8, 4
    flop = 2.0 * rows * width * width
    pat = re.compile(r"\[layer (\d+)\] fwd ([0-9.e+-]+) ms/iter \(([0-9.e+-]+) TF/s\), wgt_grad ([0-9.e+-]+) ms/iter "
                     r"\(([0-9.e+-]+) TF/s\), bwd ([0-9.e+-]+) ms/iter \(([0-9.e+-]+) TF/s\), wgt_update ([0-9.e+-]+) ms/iter "
                     r"\(([0-9.e+-]+) GB/s\)")
    lines = pat.findall(text)
    assert len(lines) == L, text
    sums = [0.0, 0.0, 0.0]
    for l, *vals in lines:
        vals = [float(v) for v in vals]
        for k in range(3):
            ms, tf = vals[2 * k], vals[2 * k + 1]
            assert ms > 0 and abs(tf - flop / (ms * 1e-3) / 1e12) <= 1e-3 * tf, (l, k, ms, tf)
            assert 20 < tf < 157.3          # an fp32 GEMM rate below the MFMA peak
            sums[k] += ms
    upd_ms, upd_gbs = float(lines[0][7]), float(lines[0][8])   # the timed pass runs one update launch, booked on layer 0
    params = L * (width * width + width)
    assert abs(upd_gbs - (R + 2) * 4.0 * params / (upd_ms * 1e-3) / 1e9) <= 1e-3 * upd_gbs
    assert all(float(line[7]) == 0 for line in lines[1:])
    m = re.search(r"total fwd ([0-9.e+-]+) ms/iter \(([0-9.e+-]+) TF/s\), wgt_grad ([0-9.e+-]+) ms/iter", text)
    assert m and abs(float(m.group(1)) - sums[0]) <= 1e-3 * sums[0]
    assert abs(float(m.group(2)) - L * flop / (sums[0] * 1e-3) / 1e12) <= 1e-3 * float(m.group(2))
    wall = float(re.search(r"wall clock time ([0-9.e+-]+) ms/iter", text).group(1))
    assert 0.8 * sum(sums) < wall < 2.0 * sum(sums)


def test_driver_is_deterministic_across_schedules():
    """Same seed, same checksum lines whether the step is replayed from a graph, launched kernel by
    kernel, or updates per layer on the second stream."""
    def checksum(*extra):
        text = run("2", "--config", "C1", "--warmup", "0", "--iters", "2", *extra)
        lines = [l for l in text.splitlines() if "l1" in l.lower() or "trace" in l.lower() or "checksum" in l.lower()]
        assert lines, text
        return lines
    base = checksum()
    assert checksum("--no-graph") == base
    assert checksum("--overlap") == base


def test_driver_loss_and_trace(tmp_path):
    path = tmp_path / "trace.log"
    text = run("2", "--config", "C1", "--warmup", "1", "--iters", "2", "--loss", "l2", "--trace", str(path))
    m = re.search(r"loss ([0-9.e+-]+) \(per replica: ([0-9.e+-]+) ([0-9.e+-]+)\)", text)
    assert m, text
    total, a, b = (float(x) for x in m.groups())
    assert total > 0 and abs(total - (a + b)) <= 1e-9 * total
    events = json.loads(path.read_text())
    names = {e["name"] for e in events if e["ph"] == "B"}
    # config 1 is a small model: the two backward GEMMs of a layer share one launch
    assert {"FC_0_0", "FCWgtGradient+FCBwdGradient_2_0", "FCWgtGradient+FCBwdGradient_1_0", "L2Loss_0"} <= names


def test_driver_rejects_unknown_loss():
    out = subprocess.run([EXE, "2", "--config", "C1", "--loss", "hinge"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 1 and "unknown loss" in out.stderr
