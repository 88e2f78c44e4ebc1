"""The C-ABI libraries load and export every symbol their headers declare (no GPU needed; no
compute is called).  Also checks that the POD descriptor has one layout on all three sides."""
import ctypes as C
import os
import re

import pytest

from aix_amd import kernels as K
from oracle import cpuref as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"\w+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    names = declared("aixhip_kernels.h", "aixk_")
    assert len(names) >= 30
    lib = K.load()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert sorted(K.EXPORTED) == names, "the Python binding must cover the header exactly"


def test_device_library_exports_every_declared_symbol():
    from aix_amd import device as D
    names = declared("aixhip.h", "aixhip_")
    assert len(names) >= 50
    lib = D.load()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert sorted(D.EXPORTED) == names, "the Python binding must cover the header exactly"
    # one entry point per virtual of aix::Device (39 of them: type, name, 3 memory, 32 operators, emptyCache, synchronize)
    virtuals = ["type", "name", "allocate", "allocate_typed", "deallocate", "add", "sub", "mul", "div", "unary", "fill",
                "fill_min", "sum", "sqrt", "sin", "cos", "tanh", "log", "exp", "pow", "max", "argmax", "argmax_indices",
                "matmul", "transpose", "copy", "copy_immediate", "contiguous", "reduce_to", "max_to", "argmax_to",
                "argmax_indices_to", "slice_set", "tril", "triu", "index_select", "index_add", "empty_cache", "synchronize"]
    assert len(virtuals) == 39 and all("aixhip_" + v in names for v in virtuals)


def test_descriptor_layout_is_shared():
    assert C.sizeof(K.Tensor) == C.sizeof(O.TensorDesc) == 8 + 4 + 4 + 8 + 8 + 16 * 8 * 2
    for (n1, _), (n2, _) in zip(K.Tensor._fields_, O.TensorDesc._fields_):
        assert n1 == n2 and getattr(K.Tensor, n1).offset == getattr(O.TensorDesc, n2).offset
    lib = K.load()
    for dt in range(9):
        assert lib.aixk_dtype_size(dt) == O.ITEMSIZE[dt] == O.lib()._lib.cpuref_dtype_size(dt)


def test_no_gpu_means_a_loud_error_not_a_fallback():
    """Without a visible GPU the context refuses to exist; nothing computes on the CPU."""
    lib = K.load()
    h = C.c_void_p()
    rc = lib.aixk_create(0, C.byref(h))
    if rc == 0:                      # running on a GPU box: just clean up
        lib.aixk_destroy(h)
        pytest.skip("a GPU is visible here")
    assert rc == 3 and lib.aixk_last_error()


def test_prelude_is_the_device_header():
    text = K.load().aixk_rtc_prelude().decode()
    assert "namespace aixd" in text and "bf16_down" in text
    assert text == open(os.path.join(ROOT, "aix_amd", "csrc", "hip", "aix_device.h")).read()
