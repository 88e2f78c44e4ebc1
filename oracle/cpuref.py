"""ctypes binding of the CPU oracle (oracle/libcpuref.so) and, where it was built, of the
reference's own CPU device (oracle/_ref/libaixref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF_BUILT_NOTE = os.path.join(HERE, "ref_built.note")
MAX_RANK = 16


def ref_expected():
    """True where this tree was built with the reference present: oracle/_ref must then be there too."""
    return os.path.exists(REF_BUILT_NOTE)

F64, F32, F16, BF16, I64, I32, I16, I8, U8 = range(9)
DTYPE_NAMES = ["f64", "f32", "f16", "bf16", "i64", "i32", "i16", "i8", "u8"]
# numpy storage type per element type (bf16 lives in uint16 words)
NP_STORAGE = [np.float64, np.float32, np.float16, np.uint16, np.int64, np.int32, np.int16, np.int8, np.uint8]
ITEMSIZE = [8, 4, 2, 2, 8, 4, 2, 1, 1]

ADD, SUB, MUL, DIV, POW = range(5)
NEG, SQRT, SIN, COS, TANH, LOG, EXP = range(7)


class TensorDesc(C.Structure):
    """POD operand descriptor; same layout as cpuref_tensor and aixhip_tensor."""
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
                ("offset", C.c_uint64), ("size", C.c_uint64),
                ("shape", C.c_uint64 * MAX_RANK), ("strides", C.c_uint64 * MAX_RANK)]


def row_major(shape):
    strides, run = [], 1
    for ext in reversed(shape):
        strides.append(run)
        run *= ext
    return list(reversed(strides))


def numel(shape):
    n = 1
    for e in shape:
        n *= e
    return n


def make_desc(ptr, dtype, shape, strides=None, offset=0, size=None):
    d = TensorDesc()
    d.data = ptr
    d.dtype = dtype
    d.rank = len(shape)
    d.offset = offset
    d.size = numel(shape) if size is None else size
    st = row_major(shape) if strides is None else strides
    for i, (e, s) in enumerate(zip(shape, st)):
        d.shape[i] = e
        d.strides[i] = s
    return d


def desc_of(arr, dtype, shape=None, strides=None, offset=0, size=None):
    """Descriptor over a numpy storage array (kept alive by the caller)."""
    shape = list(arr.shape) if shape is None else list(shape)
    return make_desc(arr.ctypes.data, dtype, shape, strides, offset, size)


# ---- bf16 helpers on the numpy side (bit-level model used to pin the oracle) ----
def f32_to_bf16_bits(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = ((u & 0x7F800000) == 0x7F800000) & ((u & 0x007FFFFF) != 0)
    hi = u >> 16
    rest = u & 0xFFFF
    up = (rest > 0x8000) | ((rest == 0x8000) & ((hi & 1) == 1))
    out = np.where(nan, hi | 0x40, hi + up.astype(np.uint64))
    return out.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_storage(values_f64, dtype):
    """Round a float64 numpy array into the storage array of an element type."""
    v = np.asarray(values_f64)
    if dtype == BF16:
        return f32_to_bf16_bits(v.astype(np.float32))
    return v.astype(NP_STORAGE[dtype])


def to_float64(storage, dtype):
    if dtype == BF16:
        return bf16_bits_to_f32(storage).astype(np.float64)
    return np.asarray(storage).astype(np.float64)


def build(ref=True, force=False):
    """(Re)build the oracle; the reference-backed libraries only where the reference exists.
    force=True recompiles even what is up to date."""
    extra = ["-B"] if force else []
    subprocess.check_call(["make", "-s", "-C", HERE, "all"] + extra)
    if ref and os.path.isdir(os.environ.get("AIX_REFERENCE_DIR", "/root/reference")):
        subprocess.check_call(["make", "-s", "-C", HERE, "ref"] + extra)
        # a note beside (not inside) _ref/ that the reference-backed libraries belong to this tree: a test that finds
        # the note but not the libraries fails instead of skipping
        with open(REF_BUILT_NOTE, "w") as f:
            f.write("oracle/_ref was built from the reference tree by oracle/Makefile (target ref)\n")


_T = C.POINTER(TensorDesc)
_SIGS = {
    "binary": [C.c_int, _T, _T, _T],
    "unary": [C.c_int, _T, _T],
    "fill": [C.c_void_p, C.c_int, _T],
    "fill_min": [_T],
    "copy": [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_uint64],
    "contiguous": [_T, _T],
    "transpose": [_T, _T, C.c_uint64, C.c_uint64],
    "sum": [_T, _T], "max": [_T, _T], "argmax": [_T, _T], "argmax_indices": [_T, _T],
    "reduce_to": [_T, _T], "max_to": [_T, _T],
    "argmax_to": [_T, _T, C.c_uint64], "argmax_indices_to": [_T, _T, C.c_uint64],
    "matmul": [_T, _T, _T],
    "tril": [_T, _T, C.c_int64], "triu": [_T, _T, C.c_int64],
}
_CPUREF_ONLY = {
    "slice_set": [_T, _T, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int],
    "index_select": [_T, _T, _T, C.c_uint64, C.c_int],
    "index_add": [_T, _T, _T, C.c_uint64, C.c_int],
    "sum_wide": [_T, C.POINTER(C.c_double), C.POINTER(C.c_double)],
    "reduce_to_wide": [_T, _T, C.c_void_p, C.c_void_p],
    "matmul_wide": [_T, _T, C.c_void_p, C.c_void_p, C.c_int],
    "matmul_rows": [_T, _T, _T, C.c_int],
    "matmul_stack": [_T, _T, _T, C.c_int],
    "matmul_stack_wide": [_T, _T, _T, C.c_int],
}
_REF_ONLY = {
    "slice_set": [_T, _T, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64],
    "index_select": [_T, _T, _T, C.c_uint64],
    "index_add": [_T, _T, _T, C.c_uint64],
}


class _Lib:
    def __init__(self, path, prefix, extra):
        self._lib = C.CDLL(path)
        for name, sig in list(_SIGS.items()) + list(extra.items()):
            fn = getattr(self._lib, prefix + name)
            fn.argtypes = sig
            fn.restype = C.c_int
            setattr(self, name, fn)


_cpuref = None
_aixref = None


def lib():
    """The restatement library; built on first use if absent."""
    global _cpuref
    if _cpuref is None:
        path = os.path.join(HERE, "libcpuref.so")
        if not os.path.exists(path):
            build(ref=False)
        _cpuref = _Lib(path, "cpuref_", _CPUREF_ONLY)
        _cpuref._lib.cpuref_ulp_hist_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p, C.c_int]
        _cpuref._lib.cpuref_ulp_hist_f32.restype = C.c_uint64
    return _cpuref


def ref_lib():
    """The compiled reference CPU device, or None where oracle/_ref was not built."""
    global _aixref
    if _aixref is None:
        path = os.path.join(HERE, "_ref", "libaixref.so")
        if not os.path.exists(path):
            return None
        _aixref = _Lib(path, "aixref_", _REF_ONLY)
    return _aixref


def ulp_hist_f32(x, y, nbins=16):
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    y = np.ascontiguousarray(y, dtype=np.float32).ravel()
    assert x.size == y.size
    hist = np.zeros(nbins, dtype=np.uint64)
    worst = lib()._lib.cpuref_ulp_hist_f32(x.ctypes.data, y.ctypes.data, x.size, hist.ctypes.data, nbins)
    return int(worst), hist
