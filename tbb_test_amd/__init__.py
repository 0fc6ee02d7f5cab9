"""MI355X (gfx950) implementation of the tbb_test MLP training step.

The product is two native libraries built by ``make -C tbb_test_amd`` (or
``__graft_entry__.build()``):

* ``lib/libmi_mlp.so``      hand-written HIP kernels behind the C ABI of ``include/mi_mlp.h``
* ``lib/libmi_mlp_host.so`` host-side API of the benchmark (Partition, Rand, ring info)

plus the C++ driver ``bin/mlp_hip``.  This package is a thin ctypes binding over the two
libraries; it contains no arithmetic of its own and no CPU fallback: if a library is missing,
importing the binding raises.
"""
from .capi import (  # noqa: F401
    MiError,
    MlpHandle,
    device_info,
    lib,
    lib_path,
    BREAKDOWN_NAMES,
)
