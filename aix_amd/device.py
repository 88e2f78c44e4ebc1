"""ctypes binding of include/aixhip.h (libaixhip.so): the lazy, fusing device, one function per
method of the AIX device interface."""
import ctypes as C
import os

from . import kernels as K
from ._build import library_path

Tensor = K.Tensor
_T = C.POINTER(Tensor)
_P = C.c_void_p


class FuseConfig(C.Structure):
    _fields_ = [("elementwise_fusion", C.c_int32), ("multi_output_kernels", C.c_int32), ("absorb_fills", C.c_int32),
                ("diagnostics", C.c_int32), ("flush_threshold", C.c_uint64), ("max_buffer_slots", C.c_uint64),
                ("supports_strided_fusion", C.c_int32), ("eager_idle_fills", C.c_int32)]


class FlushDiagnostics(C.Structure):
    _fields_ = [("ops_recorded", C.c_uint64), ("fusible_subgraphs", C.c_uint64), ("fused_ops", C.c_uint64),
                ("fallback_ops", C.c_uint64), ("dispatches_saved", C.c_uint64), ("fills_absorbed", C.c_uint64),
                ("kernel_cache_hits", C.c_uint64), ("kernel_cache_misses", C.c_uint64),
                ("subgraph_summary", C.c_char * 256), ("fallback_summary", C.c_char * 128)]


_BIN = [_P, _T, _T, _T]
_UN = [_P, _T, _T]
_SIGNATURES = {
    "aixhip_device_create": [C.c_int, C.POINTER(_P)],
    "aixhip_device_destroy": [_P],
    "aixhip_allocate": [_P, C.c_size_t, C.POINTER(_P)],
    "aixhip_allocate_typed": [_P, C.c_size_t, C.c_int, C.POINTER(_P)],
    "aixhip_deallocate": [_P, _P],
    "aixhip_add": _BIN, "aixhip_sub": _BIN, "aixhip_mul": _BIN, "aixhip_div": _BIN, "aixhip_pow": _BIN, "aixhip_matmul": _BIN,
    "aixhip_unary": _UN, "aixhip_sum": _UN, "aixhip_sqrt": _UN, "aixhip_sin": _UN, "aixhip_cos": _UN, "aixhip_tanh": _UN,
    "aixhip_log": _UN, "aixhip_exp": _UN, "aixhip_max": _UN, "aixhip_argmax": _UN, "aixhip_argmax_indices": _UN,
    "aixhip_contiguous": _UN, "aixhip_reduce_to": _UN, "aixhip_max_to": _UN,
    "aixhip_fill": [_P, _P, C.c_int, _T],
    "aixhip_fill_min": [_P, _T],
    "aixhip_transpose": [_P, _T, _T, C.c_size_t, C.c_size_t],
    "aixhip_copy": [_P, _P, C.c_int, _P, C.c_int, C.c_size_t],
    "aixhip_copy_immediate": [_P, _P, C.c_int, _P, C.c_int, C.c_size_t],
    "aixhip_argmax_to": [_P, _T, _T, C.c_size_t],
    "aixhip_argmax_indices_to": [_P, _T, _T, C.c_size_t],
    "aixhip_slice_set": [_P, _T, _T, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t],
    "aixhip_tril": [_P, _T, _T, C.c_int64],
    "aixhip_triu": [_P, _T, _T, C.c_int64],
    "aixhip_index_select": [_P, _T, _T, _T, C.c_size_t],
    "aixhip_index_add": [_P, _T, _T, _T, C.c_size_t],
    "aixhip_empty_cache": [_P],
    "aixhip_synchronize": [_P],
    "aixhip_flush": [_P],
    "aixhip_copy_to_host": [_P, _P, _P, C.c_size_t],
    "aixhip_copy_from_host": [_P, _P, _P, C.c_size_t],
    "aixhip_get_fuse_config": [_P, C.POINTER(FuseConfig)],
    "aixhip_set_fuse_config": [_P, C.POINTER(FuseConfig)],
    "aixhip_last_flush_diagnostics": [_P, C.POINTER(FlushDiagnostics)],
    "aixhip_fuse_kernel_cache_stats": [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "aixhip_batched_launch_stats": [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "aixhip_set_cache_limit": [_P, C.c_uint64],
    "aixhip_capture_begin": [_P],
    "aixhip_capture_end": [_P, C.POINTER(_P)],
    "aixhip_capture_abort": [_P],
    "aixhip_graph_replay": [_P, _P],
    "aixhip_graph_destroy": [_P, _P],
    "aixhip_memory_stats": [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
}
_OTHER = {
    "aixhip_last_error": ([], C.c_char_p),
    "aixhip_type": ([_P], C.c_int32),
    "aixhip_name": ([_P], C.c_char_p),
    "aixhip_data_type_size": ([C.c_int], C.c_size_t),
    "aixhip_kernel_context": ([_P], _P),
}
EXPORTED = sorted(list(_SIGNATURES) + list(_OTHER))

_lib = None


def load():
    """Load libaixhip.so (and, through it, libaixhip_kernels.so).  Never builds, never falls back."""
    global _lib
    if _lib is None:
        K.load()
        path = library_path("libaixhip.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is not built; run aix_amd.build() (or `make -C aix_amd/csrc`)")
        lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
        for name, sig in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = sig
            fn.restype = C.c_int32
        for name, (sig, res) in _OTHER.items():
            fn = getattr(lib, name)
            fn.argtypes = sig
            fn.restype = res
        _lib = lib
    return _lib


class AixHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"[status {status}] {message}")
        self.status = status


def check(status):
    if status != 0:
        raise AixHipError(status, load().aixhip_last_error().decode(errors="replace"))


class Device:
    """Owns an aixhip_device."""

    def __init__(self, index=0):
        self.lib = load()
        h = _P()
        check(self.lib.aixhip_device_create(index, C.byref(h)))
        self.handle = h

    def close(self):
        if self.handle:
            self.lib.aixhip_device_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def call(self, name, *args):
        check(getattr(self.lib, "aixhip_" + name)(self.handle, *args))

    def status(self, name, *args):
        return getattr(self.lib, "aixhip_" + name)(self.handle, *args)

    def allocate(self, nbytes):
        p = _P()
        check(self.lib.aixhip_allocate(self.handle, nbytes, C.byref(p)))
        return p.value

    def deallocate(self, ptr):
        check(self.lib.aixhip_deallocate(self.handle, ptr))

    def synchronize(self):
        check(self.lib.aixhip_synchronize(self.handle))

    def flush(self):
        check(self.lib.aixhip_flush(self.handle))

    def to_host(self, array, ptr):
        check(self.lib.aixhip_copy_to_host(self.handle, array.ctypes.data, ptr, array.nbytes))

    def from_host(self, ptr, array):
        check(self.lib.aixhip_copy_from_host(self.handle, ptr, array.ctypes.data, array.nbytes))

    def fuse_config(self):
        c = FuseConfig()
        check(self.lib.aixhip_get_fuse_config(self.handle, C.byref(c)))
        return c

    def set_fuse_config(self, cfg):
        check(self.lib.aixhip_set_fuse_config(self.handle, C.byref(cfg)))

    def diagnostics(self):
        d = FlushDiagnostics()
        check(self.lib.aixhip_last_flush_diagnostics(self.handle, C.byref(d)))
        return d

    def kernel_cache_stats(self):
        h, m = C.c_uint64(), C.c_uint64()
        check(self.lib.aixhip_fuse_kernel_cache_stats(self.handle, C.byref(h), C.byref(m)))
        return h.value, m.value

    def batched_launch_stats(self):
        n, k = C.c_uint64(), C.c_uint64()
        check(self.lib.aixhip_batched_launch_stats(self.handle, C.byref(n), C.byref(k)))
        return n.value, k.value

    def kernel_context(self):
        return _P(self.lib.aixhip_kernel_context(self.handle))
