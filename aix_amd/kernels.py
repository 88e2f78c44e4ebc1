"""ctypes binding of include/aixhip_kernels.h (libaixhip_kernels.so): the eager kernel layer."""
import ctypes as C
import os

from ._build import library_path

MAX_RANK = 16
F64, F32, F16, BF16, I64, I32, I16, I8, U8 = range(9)
ADD, SUB, MUL, DIV, POW = range(5)
NEG, SQRT, SIN, COS, TANH, LOG, EXP = range(7)
SUM, MAX, ARGMAX, ARGMAX_ONEHOT = range(4)
MEM_DEVICE, MEM_MANAGED, MEM_PINNED = range(3)


class Tensor(C.Structure):
    """aixhip_tensor: POD image of aix::DeviceTensorParams."""
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
                ("offset", C.c_uint64), ("size", C.c_uint64),
                ("shape", C.c_uint64 * MAX_RANK), ("strides", C.c_uint64 * MAX_RANK)]


class FillItem(C.Structure):
    """aixk_fill_item"""
    _fields_ = [("dst", C.c_void_p), ("bits", C.c_uint64), ("elements", C.c_uint32), ("element_size", C.c_uint32)]


class SliceItem(C.Structure):
    """aixk_slice_item"""
    _fields_ = [("src", Tensor), ("dst", Tensor), ("dim", C.c_uint64), ("start", C.c_uint64), ("end", C.c_uint64), ("step", C.c_uint64)]


class ArgmaxItem(C.Structure):
    """aixk_argmax_item"""
    _fields_ = [("src", Tensor), ("dst", Tensor), ("dim", C.c_uint64)]


class ColsumItem(C.Structure):
    """aixk_colsum_item"""
    _fields_ = [("src", Tensor), ("dst", Tensor), ("init_bits", C.c_uint64)]


class PartialsItem(C.Structure):
    """aixk_partials_item"""
    _fields_ = [("partials", C.c_void_p), ("count", C.c_uint64), ("dst", Tensor), ("init_bits", C.c_uint64)]


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int32),
                ("clock_khz", C.c_int32), ("large_bar", C.c_int32), ("wavefront", C.c_int32),
                ("total_mem", C.c_uint64), ("lds_per_block", C.c_uint64)]


class AixHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"[status {status}] {message}")
        self.status = status


_T = C.POINTER(Tensor)
_P = C.c_void_p
_SIGNATURES = {
    "aixk_create": [C.c_int, C.POINTER(_P)],
    "aixk_destroy": [_P],
    "aixk_info": [_P, C.POINTER(DeviceInfo)],
    "aixk_alloc": [_P, C.c_size_t, C.c_int, C.POINTER(_P)],
    "aixk_free": [_P, _P, C.c_int],
    "aixk_copy_in": [_P, _P, _P, C.c_size_t],
    "aixk_copy_out": [_P, _P, _P, C.c_size_t],
    "aixk_copy_dev": [_P, _P, _P, C.c_size_t],
    "aixk_zero": [_P, _P, C.c_size_t],
    "aixk_sync": [_P],
    "aixk_binary": [_P, C.c_int, _T, _T, _T],
    "aixk_unary": [_P, C.c_int, _T, _T],
    "aixk_fill": [_P, _P, C.c_int, _T],
    "aixk_fill_min": [_P, _T],
    "aixk_fill_many": [_P, _P, C.c_uint32],
    "aixk_cast": [_P, _P, C.c_int, _P, C.c_int, C.c_uint64],
    "aixk_contiguous": [_P, _T, _T],
    "aixk_transpose": [_P, _T, _T, C.c_uint64, C.c_uint64],
    "aixk_slice_set": [_P, _T, _T, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64],
    "aixk_slice_set_many": [_P, _P, C.c_uint32],
    "aixk_slice_set_init": [_P, _T, _T, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64],
    "aixk_tri": [_P, C.c_int, _T, _T, C.c_int64],
    "aixk_index_select": [_P, _T, _T, _T, C.c_uint64],
    "aixk_index_add": [_P, _T, _T, _T, C.c_uint64],
    "aixk_reduce_all": [_P, C.c_int, _T, _T],
    "aixk_reduce_all_noalloc": [_P, C.c_int, _T, _T],
    "aixk_reduce_to": [_P, C.c_int, _T, _T],
    "aixk_reduce_to_init": [_P, C.c_int, _T, _T, C.c_uint64],
    "aixk_sum_partials": [_P, _P, C.c_uint64, _T, C.c_uint64],
    "aixk_sum_partials_many": [_P, _P, C.c_uint32],
    "aixk_argmax_to": [_P, C.c_int, _T, _T, C.c_uint64],
    "aixk_argmax_onehot_many": [_P, _P, C.c_uint32],
    "aixk_sum_columns_many": [_P, _P, C.c_uint32],
    "aixk_matmul": [_P, _T, _T, _T],
    "aixk_matmul_route": [_P, C.POINTER(C.c_int32), C.POINTER(C.c_int32)],
    "aixk_capture_begin": [_P],
    "aixk_capture_end": [_P, C.POINTER(_P)],
    "aixk_capture_abort": [_P],
    "aixk_graph_launch": [_P, _P],
    "aixk_graph_nodes": [_P, C.POINTER(C.c_uint64)],
    "aixk_graph_destroy": [_P, _P],
    "aixk_mfma_only_rate": [_P, C.c_int32, C.c_int32, _P, C.c_uint32, C.c_double, C.POINTER(C.c_float), C.POINTER(C.c_float)],
    "aixk_matmul_batched": [_P, _T, _T, _T],
    "aixk_matmul_grouped": [_P, _T, _T, _T, C.c_uint32],
    "aixk_rtc_get": [_P, C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(_P), C.POINTER(C.c_int32)],
    "aixk_rtc_launch": [_P, _P, C.c_uint32, C.c_uint32, _P, C.c_size_t],
    "aixk_rtc_launch_many": [_P, _P, C.c_uint32, _P, C.c_size_t, C.c_size_t, C.c_uint32],
    "aixk_rtc_stats": [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "aixk_rtc_disk_stats": [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "aixk_event_create": [_P, C.POINTER(_P)],
    "aixk_event_record": [_P, _P],
    "aixk_event_query": [_P, _P, C.POINTER(C.c_int32)],
    "aixk_event_elapsed_ms": [_P, _P, _P, C.POINTER(C.c_float)],
    "aixk_event_destroy": [_P, _P],
}
_OTHER = {
    "aixk_last_error": ([], C.c_char_p),
    "aixk_dtype_size": ([C.c_int], C.c_size_t),
    "aixk_rtc_prelude": ([], C.c_char_p),
}
EXPORTED = sorted(list(_SIGNATURES) + list(_OTHER))

_lib = None


def load():
    """Load libaixhip_kernels.so (never builds, never falls back)."""
    global _lib
    if _lib is None:
        path = library_path("libaixhip_kernels.so")
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


def check(status):
    if status != 0:
        raise AixHipError(status, load().aixk_last_error().decode(errors="replace"))


class Context:
    """Owns an aixk_ctx; thin convenience wrapper for tests and the benchmark."""

    def __init__(self, device_index=0):
        self.lib = load()
        h = _P()
        check(self.lib.aixk_create(device_index, C.byref(h)))
        self.handle = h

    def close(self):
        if self.handle:
            self.lib.aixk_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def info(self):
        out = DeviceInfo()
        check(self.lib.aixk_info(self.handle, C.byref(out)))
        return out

    def alloc(self, nbytes, kind=MEM_DEVICE):
        p = _P()
        check(self.lib.aixk_alloc(self.handle, nbytes, kind, C.byref(p)))
        return p.value

    def free(self, ptr, kind=MEM_DEVICE):
        check(self.lib.aixk_free(self.handle, ptr, kind))

    def upload(self, ptr, array):
        check(self.lib.aixk_copy_in(self.handle, ptr, array.ctypes.data, array.nbytes))

    def download(self, array, ptr):
        check(self.lib.aixk_copy_out(self.handle, array.ctypes.data, ptr, array.nbytes))

    def sync(self):
        check(self.lib.aixk_sync(self.handle))

    def call(self, name, *args):
        check(getattr(self.lib, name)(self.handle, *args))

    # timing helpers -----------------------------------------------------------------
    def event(self):
        e = _P()
        check(self.lib.aixk_event_create(self.handle, C.byref(e)))
        return e

    def record(self, ev):
        check(self.lib.aixk_event_record(self.handle, ev))

    def elapsed_ms(self, start, stop):
        ms = C.c_float()
        check(self.lib.aixk_event_elapsed_ms(self.handle, start, stop, C.byref(ms)))
        return ms.value
