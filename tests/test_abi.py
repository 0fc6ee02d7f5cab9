"""The C-ABI libraries load and export every symbol their headers declare; failure paths that need
no GPU behave as documented; the product has no CPU fallback and does not touch the oracle.  No GPU
compute is launched here."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

import tbb_test_amd
from tbb_test_amd import capi, hostlib

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)))


def test_libmi_mlp_exports_every_declared_symbol():
    names = declared_functions("mi_mlp.h")
    assert len(names) >= 40
    lib = ctypes.CDLL(capi.lib_path())
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in mi_mlp.h but not exported: {missing}"
    # and the Python binding covers all of them (mi_last_error is bound separately)
    unbound = [n for n in names if n not in capi.SIGNATURES and n != "mi_last_error"]
    assert not unbound, f"not bound in capi.py: {unbound}"


def test_libmi_mlp_host_exports_every_declared_symbol():
    names = declared_functions("mi_mlp_host.h")
    lib = ctypes.CDLL(hostlib.lib_path())
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert sorted(hostlib.SIGNATURES) == names


def _gpu_present():
    return os.path.exists("/dev/kfd")


@pytest.mark.skipif(_gpu_present(), reason="checks the no-device error path")
def test_no_device_is_an_error_not_a_fallback():
    with pytest.raises(capi.MiError) as e:
        capi.device_info()
    assert e.value.code == -3
    with pytest.raises(capi.MiError) as e:
        capi.MlpHandle([8, 8], 4, 1)
    assert e.value.code == -3 and "no HIP device" in str(e.value)


def test_argument_validation_needs_no_device():
    lib = capi.lib()
    h = ctypes.c_void_p()
    nf = (ctypes.c_int * 2)(8, 0)
    assert lib.mi_mlp_create(ctypes.byref(h), 1, nf, 4, 1, 0, 0) == -1 and b"nfeatures[1]" in lib.mi_last_error()
    assert lib.mi_mlp_create(ctypes.byref(h), 0, nf, 4, 1, 0, 0) == -1
    assert lib.mi_mlp_create(ctypes.byref(h), 1, nf, 4, 1, 7, 0) == -1 and b"dtype" in lib.mi_last_error()
    assert lib.mi_mlp_step(None, ctypes.c_float(0.1)) == -1 and b"null handle" in lib.mi_last_error()
    assert lib.mi_mlp_destroy(None) == 0
    assert lib.mi_set_gemm_variant(5, 1) == -1
    assert lib.mi_sgemm_nn(4, 4, 4, None, 4, None, 4, None, 4, None, 4, None) == -1


def test_missing_library_raises(monkeypatch, tmp_path):
    """There is no fallback implementation: without the built library the binding raises."""
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "lib_path", lambda: str(tmp_path / "libmi_mlp.so"))
    with pytest.raises(OSError, match="no fallback"):
        capi.lib()


def test_product_does_not_use_the_oracle():
    """Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may touch oracle/."""
    offenders = []
    for dirpath, _, files in os.walk(os.path.join(ROOT, "tbb_test_amd")):
        if any(part in dirpath for part in ("/build", "/lib", "/bin", "__pycache__")):
            continue
        for f in files:
            if f.endswith((".py", ".cc", ".h", ".hip", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                if re.search(r"import oracle|from oracle|oracle/|liboracle|[\"'/]_work/", text):
                    offenders.append(os.path.join(dirpath, f))
    assert not offenders, offenders
    bench = open(os.path.join(ROOT, "bench.py")).read()
    uses = [m.start() for m in re.finditer(r"import oracle|from oracle", bench)]
    body = bench[bench.index("def cpu_baseline"):bench.index("def main")]
    assert uses and all(bench.index("def cpu_baseline") < u < bench.index("def main") for u in uses), body


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0 and "ONE GPU" in out.stderr
