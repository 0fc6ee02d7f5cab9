"""ctypes binding of include/mi_mlp.h (libmi_mlp.so).

Only argument marshalling happens here.  Every failure of the native library is raised as
MiError with the library's own message; there is no fallback path.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_longlong, c_size_t, c_uint, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

MI_F32, MI_BF16 = 0, 1
FLAG_RELU_LAST, FLAG_NO_GRAPH, FLAG_PER_LAYER_UPDATE, FLAG_SERIAL_BACKWARD, FLAG_KEEP_GRADIENTS = 1, 2, 4, 8, 16
BREAKDOWN_NAMES = ("fwd", "wgt_grad", "bwd", "wgt_update", "wgt_update_reduce_scatter", "wgt_update_allgather")
NUM_BREAKDOWNS = len(BREAKDOWN_NAMES)


class MiError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"mi_mlp error {code}: {message}")
        self.code = code


def lib_path():
    return os.path.join(_HERE, "lib", "libmi_mlp.so")


_f32p = POINTER(c_float)

# name -> (argtypes); every function returns int status unless listed in _NON_STATUS
SIGNATURES = {
    "mi_device_info": [c_char_p, c_int, POINTER(c_int), POINTER(c_int), POINTER(c_size_t)],
    "mi_malloc": [POINTER(c_void_p), c_size_t],
    "mi_free": [c_void_p],
    "mi_memcpy_h2d": [c_void_p, c_void_p, c_size_t],
    "mi_memcpy_d2h": [c_void_p, c_void_p, c_size_t],
    "mi_memset": [c_void_p, c_int, c_size_t],
    "mi_stream_sync": [c_void_p],
    "mi_set_gemm_variant": [c_int, c_int],
    "mi_sgemm_nt": [c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    "mi_sgemm_nn": [c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    "mi_sgemm_tn": [c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_longlong,
                    c_void_p, c_longlong, c_void_p],
    "mi_reduce_sgd_raw": [c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_float, c_void_p],
    "mi_reduce_sgd_bf16_raw": [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_float, c_void_p],
    "mi_reduce_sgd_bf16t_raw": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_size_t, c_int, c_float, c_void_p],
    "mi_hgemm_nt": [c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    "mi_hgemm_nn": [c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p],
    "mi_hgemm_tn": [c_int, c_int, c_int, c_int, c_void_p, c_int, c_longlong, c_void_p, c_int, c_longlong, c_void_p,
                    c_int, c_longlong, c_void_p],
    "mi_transpose_bf16": [c_int, c_int, c_int, c_void_p, c_int, c_longlong, c_void_p, c_int, c_longlong, c_void_p],
    "mi_probe_mfma_rate": [c_int, c_int, POINTER(c_double), c_void_p],
    "mi_rowsum_bf16": [c_int, c_int, c_int, c_void_p, c_int, c_longlong, c_void_p, c_longlong, c_void_p],
    "mi_set_hgemm_variant": [c_int],
    "mi_convert_f32_to_bf16": [c_void_p, c_void_p, c_size_t, c_void_p],
    "mi_convert_bf16_to_f32": [c_void_p, c_void_p, c_size_t, c_void_p],
    "mi_mlp_create": [POINTER(c_void_p), c_int, POINTER(c_int), c_int, c_int, c_int, c_uint],
    "mi_mlp_destroy": [c_void_p],
    "mi_mlp_set_weights": [c_void_p, c_int, c_void_p, c_int, c_void_p],
    "mi_mlp_set_input": [c_void_p, c_void_p, c_int],
    "mi_mlp_set_dy": [c_void_p, c_void_p, c_int],
    "mi_fc_forward": [c_void_p, c_int],
    "mi_fc_wgrad": [c_void_p, c_int],
    "mi_fc_bgrad": [c_void_p, c_int],
    "mi_fc_dgrad": [c_void_p, c_int],
    "mi_reduce_sgd": [c_void_p, c_float],
    "mi_reduce_sgd_layer": [c_void_p, c_int, c_float],
    "mi_mlp_step": [c_void_p, c_float],
    "mi_mlp_sync": [c_void_p],
    "mi_mlp_get_activation": [c_void_p, c_int, c_void_p, c_int],
    "mi_mlp_get_weight": [c_void_p, c_int, c_void_p, c_int],
    "mi_mlp_get_bias": [c_void_p, c_int, c_void_p],
    "mi_mlp_get_wgrad": [c_void_p, c_int, c_int, c_void_p, c_int],
    "mi_mlp_get_bgrad": [c_void_p, c_int, c_int, c_void_p],
    "mi_mlp_get_dx": [c_void_p, c_void_p, c_int],
    "mi_mlp_get_dz": [c_void_p, c_int, c_void_p, c_int],
    "mi_mlp_snapshot_weights": [c_void_p],
    "mi_mlp_restore_weights": [c_void_p],
    "mi_mlp_param_count": [c_void_p, POINTER(c_size_t), POINTER(c_size_t)],
    "mi_mlp_get_weight_shadow": [c_void_p, c_int, c_int, c_void_p, c_int],
    "mi_mlp_get_schedule": [c_void_p, POINTER(c_int)],
    "mi_mlp_enable_timing": [c_void_p, c_int],
    "mi_mlp_reset_timings": [c_void_p],
    "mi_mlp_get_timings": [c_void_p, POINTER(c_double), POINTER(c_longlong)],
    "mi_mlp_set_labels": [c_void_p, c_void_p, c_int],
    "mi_loss_backward": [c_void_p],
    "mi_mlp_get_loss": [c_void_p, POINTER(c_double), POINTER(c_double)],
    "mi_mlp_trace_step": [c_void_p, c_float, c_char_p],
    "mi_l2_loss_static": [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
}

_lib = None


def lib():
    """Loads libmi_mlp.so (once).  Raises OSError if it has not been built."""
    global _lib
    if _lib is None:
        path = lib_path()
        if not os.path.exists(path):
            raise OSError(f"{path} is missing: build it with `make -C tbb_test_amd` "
                          "(there is no fallback implementation)")
        handle = ctypes.CDLL(path)
        handle.mi_last_error.restype = c_char_p
        handle.mi_last_error.argtypes = []
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = c_int
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise MiError(code, lib().mi_last_error().decode(errors="replace"))


def _host_f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(c_void_p)


def device_info():
    name = ctypes.create_string_buffer(256)
    cus, mhz, mem = c_int(), c_int(), c_size_t()
    check(lib().mi_device_info(name, 256, ctypes.byref(cus), ctypes.byref(mhz), ctypes.byref(mem)))
    return {"name": name.value.decode(), "num_cus": cus.value, "clock_mhz": mhz.value, "hbm_bytes": mem.value}


class DeviceBuffer:
    """A device allocation made through mi_malloc, with numpy upload/download."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = c_void_p()
        check(lib().mi_malloc(ctypes.byref(p), max(self.nbytes, 1)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        if a.nbytes:
            check(lib().mi_memcpy_h2d(buf.ptr, a.ctypes.data_as(c_void_p), a.nbytes))
        return buf

    def to_numpy(self, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        if out.nbytes:
            check(lib().mi_memcpy_d2h(out.ctypes.data_as(c_void_p), self.ptr, out.nbytes))
        return out

    def zero(self):
        check(lib().mi_memset(self.ptr, 0, self.nbytes))

    def free(self):
        if self.ptr:
            lib().mi_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class MlpHandle:
    """The model resident in HBM (mi_mlp_* handle API)."""

    def __init__(self, nfeatures, batch_per_replica, replicas, dtype=MI_F32, flags=0):
        self.nf = [int(v) for v in nfeatures]
        self.L = len(self.nf) - 1
        self.B, self.R = int(batch_per_replica), int(replicas)
        self.MB = self.B * self.R
        self._h = c_void_p()
        arr = (c_int * len(self.nf))(*self.nf)
        check(lib().mi_mlp_create(ctypes.byref(self._h), self.L, arr, self.B, self.R, dtype, flags))

    def close(self):
        if self._h:
            lib().mi_mlp_destroy(self._h)
            self._h = c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # uploads
    def set_weights(self, l, W, b=None):
        W, wp = _host_f32(W)
        assert W.shape == (self.nf[l + 1], self.nf[l])
        bp = None
        if b is not None:
            b, bp = _host_f32(b)
            assert b.shape == (self.nf[l + 1],)
        check(lib().mi_mlp_set_weights(self._h, l, wp, W.shape[1], bp))

    def set_input(self, X):
        X, xp = _host_f32(X)
        assert X.shape == (self.MB, self.nf[0])
        check(lib().mi_mlp_set_input(self._h, xp, X.shape[1]))

    def set_dy(self, dY):
        dY, p = _host_f32(dY)
        assert dY.shape == (self.MB, self.nf[self.L])
        check(lib().mi_mlp_set_dy(self._h, p, dY.shape[1]))

    def set_labels(self, Y):
        """Switches to loss mode: every step derives dY = (pred - Y) / B from its forward output."""
        Y, p = _host_f32(Y)
        assert Y.shape == (self.MB, self.nf[self.L])
        check(lib().mi_mlp_set_labels(self._h, p, Y.shape[1]))

    def loss(self):
        """(loss_per_replica [R], total) of the last step in loss mode."""
        per = (c_double * self.R)()
        tot = c_double()
        check(lib().mi_mlp_get_loss(self._h, per, ctypes.byref(tot)))
        return np.array(per[:]), tot.value

    def loss_backward(self): check(lib().mi_loss_backward(self._h))

    def trace_step(self, lr, path):
        """One step with an event pair around every launch; writes a Chrome-trace style timeline."""
        check(lib().mi_mlp_trace_step(self._h, float(lr), os.fsencode(path)))

    # operations
    def forward(self, l): check(lib().mi_fc_forward(self._h, l))
    def wgrad(self, l): check(lib().mi_fc_wgrad(self._h, l))
    def bgrad(self, l): check(lib().mi_fc_bgrad(self._h, l))
    def dgrad(self, l): check(lib().mi_fc_dgrad(self._h, l))
    def reduce_sgd(self, lr): check(lib().mi_reduce_sgd(self._h, lr))
    def reduce_sgd_layer(self, l, lr): check(lib().mi_reduce_sgd_layer(self._h, l, lr))
    def step(self, lr): check(lib().mi_mlp_step(self._h, lr))
    def sync(self): check(lib().mi_mlp_sync(self._h))

    # downloads
    def _get(self, fn, shape, *idx):
        out = np.empty(shape, dtype=np.float32)
        args = list(idx) + [out.ctypes.data_as(c_void_p)]
        if len(shape) == 2:
            args.append(shape[1])
        check(fn(self._h, *args))
        return out

    def activation(self, l): return self._get(lib().mi_mlp_get_activation, (self.MB, self.nf[l]), l)
    def weight(self, l): return self._get(lib().mi_mlp_get_weight, (self.nf[l + 1], self.nf[l]), l)
    def bias(self, l): return self._get(lib().mi_mlp_get_bias, (self.nf[l + 1],), l)
    def wgrad_of(self, l, r): return self._get(lib().mi_mlp_get_wgrad, (self.nf[l + 1], self.nf[l]), l, r)
    def bgrad_of(self, l, r): return self._get(lib().mi_mlp_get_bgrad, (self.nf[l + 1],), l, r)
    def dx(self): return self._get(lib().mi_mlp_get_dx, (self.MB, self.nf[0]))
    def dz(self, l): return self._get(lib().mi_mlp_get_dz, (self.MB, self.nf[l + 1]), l)

    def weight_shadow(self, l, transposed=False):
        """bf16 models: the bf16 copy of W_l (or of W_l^T) the GEMMs read, widened to fp32."""
        shape = (self.nf[l], self.nf[l + 1]) if transposed else (self.nf[l + 1], self.nf[l])
        return self._get(lib().mi_mlp_get_weight_shadow, shape, l, int(transposed))

    def schedule(self):
        """What the last step did: dict(dual_streams, per_layer_update, graph, fused_transposes, paired_backward)."""
        info = (c_int * 5)()
        check(lib().mi_mlp_get_schedule(self._h, info))
        return {"dual_streams": bool(info[0]), "per_layer_update": bool(info[1]), "graph": bool(info[2]),
                "fused_transposes": int(info[3]), "paired_backward": bool(info[4])}

    def snapshot_weights(self): check(lib().mi_mlp_snapshot_weights(self._h))
    def restore_weights(self): check(lib().mi_mlp_restore_weights(self._h))

    def param_count(self):
        p, s = c_size_t(), c_size_t()
        check(lib().mi_mlp_param_count(self._h, ctypes.byref(p), ctypes.byref(s)))
        return p.value, s.value

    # timing
    def enable_timing(self, on=True): check(lib().mi_mlp_enable_timing(self._h, int(on)))
    def reset_timings(self): check(lib().mi_mlp_reset_timings(self._h))

    def timings(self):
        """(ms, launches): arrays of shape [NUM_BREAKDOWNS, L]."""
        n = NUM_BREAKDOWNS * self.L
        ms = (c_double * n)()
        cnt = (c_longlong * n)()
        check(lib().mi_mlp_get_timings(self._h, ms, cnt))
        return (np.array(ms[:]).reshape(NUM_BREAKDOWNS, self.L), np.array(cnt[:]).reshape(NUM_BREAKDOWNS, self.L))
