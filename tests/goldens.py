"""Runs the literal cases of tests/golden/reference_literals.json against a backend.

A backend exposes run(op_name, args...) over HostTensors; two exist: the CPU oracle and the GPU
kernels (through the C ABI).  The same expectations are applied to both."""
import ctypes as C
import json
import os

import numpy as np

import aixtest as T
from oracle import cpuref as O

HERE = os.path.dirname(os.path.abspath(__file__))
DT = {n: i for i, n in enumerate(O.DTYPE_NAMES)}
UNARY = {"neg": O.NEG, "sqrt": O.SQRT, "sin": O.SIN, "cos": O.COS, "tanh": O.TANH, "log": O.LOG, "exp": O.EXP}
BINARY = {"add": O.ADD, "sub": O.SUB, "mul": O.MUL, "div": O.DIV, "pow": O.POW}


def load_cases():
    with open(os.path.join(HERE, "golden", "reference_literals.json")) as f:
        return json.load(f)["cases"]


def tensor_from(spec, dtype):
    vals = np.array(spec["values"], dtype=np.float64)
    return T.HostTensor(O.to_storage(vals, dtype), dtype, spec["shape"], spec.get("strides"), spec.get("offset", 0))


def lowest_of(dtype):
    t = T.empty(dtype, [1])
    assert O.lib().fill_min(C.byref(t.desc())) == 0
    return t.storage[0]


class OracleBackend:
    """Runs ops with the CPU oracle; results are left in the HostTensors' storage."""
    name = "oracle"

    def __init__(self):
        self.lib = O.lib()

    def unary(self, op, a, out):
        return self.lib.unary(op, C.byref(a.desc()), C.byref(out.desc()))

    def binary(self, op, a, b, out):
        return self.lib.binary(op, C.byref(a.desc()), C.byref(b.desc()), C.byref(out.desc()))

    def copy(self, src, sdt, dst, ddt, n):
        return self.lib.copy(src.storage.ctypes.data, sdt, dst.storage.ctypes.data, ddt, n)

    def fill(self, scalar, sdt, out):
        return self.lib.fill(scalar.ctypes.data, sdt, C.byref(out.desc()))

    def simple(self, name, *tensors, extra=()):
        extra = tuple(extra)
        if name == "slice_set":
            extra = extra + (1,)           # destination offset honoured (reference GPU semantics)
        if name in ("index_select", "index_add"):
            extra = extra + (1,)           # index tensor addressed through its view
        return getattr(self.lib, name)(*[C.byref(t.desc()) for t in tensors], *extra)


def run_case(case, backend):
    op = case["op"]
    dtypes = range(9) if case.get("dtype") == "*" else [DT[case["dtype"]]] if "dtype" in case else [None]
    for dtype in dtypes:
        what = f"{case['name']} [{backend.name}] {'' if dtype is None else O.DTYPE_NAMES[dtype]}"
        if op in ("argmax", "argmax_indices"):
            a = tensor_from(case["a"], dtype)
            out = T.empty(O.I32, [] if op == "argmax" else case["a"]["shape"], fill=-9)
            assert backend.simple(op, a, out) == 0
            T.assert_same_bits(out.storage[:len(case["expect_i32"])], np.array(case["expect_i32"], np.int32), what)
        elif op in ("argmax_to", "argmax_indices_to"):
            a = tensor_from(case["a"], dtype)
            out = T.empty(O.I32, case.get("dst_shape", case["a"]["shape"]), fill=-9 if op == "argmax_to" else 0)
            assert backend.simple(op, a, out, extra=(case["dim"],)) == 0
            T.assert_same_bits(out.storage, np.array(case["expect_i32"], np.int32), what)
        elif op == "copy":
            sdt, ddt = DT[case["src_dtype"]], DT[case["dst_dtype"]]
            src = T.HostTensor(O.to_storage(np.array(case["values"], np.float64), sdt), sdt, [len(case["values"])])
            dst = T.empty(ddt, [len(case["values"])])
            assert backend.copy(src, sdt, dst, ddt, src.size) == 0
            if "expect_bits16" in case:
                T.assert_same_bits(dst.storage.view(np.uint16), np.array(case["expect_bits16"], np.uint16), what)
            else:
                T.assert_same_bits(dst.storage, np.array(case["expect"]).astype(O.NP_STORAGE[ddt]), what)
        elif op == "fill":
            sdt, ddt = DT[case["src_dtype"]], DT[case["dst_dtype"]]
            scalar = O.to_storage(np.array([case["scalar"]], np.float64), sdt)
            dst = T.empty(ddt, [case["count"]], fill=7)
            assert backend.fill(scalar, sdt, dst) == 0
            T.assert_same_bits(dst.storage, np.array(case["expect"]).astype(O.NP_STORAGE[ddt]), what)
        elif op in ("unary", "binary"):
            a = tensor_from(case["a"], dtype)
            out = T.empty(dtype, case["a"]["shape"])
            if op == "unary":
                assert backend.unary(UNARY[case["fn"]], a, out) == 0
            else:
                assert backend.binary(BINARY[case["fn"]], a, tensor_from(case["b"], dtype), out) == 0
            expect = np.array(case["expect"], np.float64)
            if "rel" in case:         # CheckVectorApproxValues: relative 1e-4 (Targets/AIXTests/Utils.hpp:17-20)
                np.testing.assert_allclose(out.values().reshape(-1), expect, rtol=case["rel"], err_msg=what)
            else:
                T.assert_same_bits(out.storage, expect.astype(O.NP_STORAGE[dtype]), what)
        elif op == "matmul":
            a, b = tensor_from(case["a"], dtype), tensor_from(case["b"], dtype)
            out = T.empty(dtype, [case["a"]["shape"][0], case["b"]["shape"][1]])
            assert backend.simple("matmul", a, b, out) == 0
            T.assert_same_bits(out.storage, np.array(case["expect"]).astype(O.NP_STORAGE[dtype]), what)
        elif op in ("reduce_to", "max_to"):
            a = tensor_from(case["a"], dtype)
            init = case["dst_init"]
            dst = T.empty(dtype, case["dst_shape"], fill=lowest_of(dtype) if init == "lowest" else None)
            if init != "lowest":
                dst.storage[:] = O.to_storage(np.array(init, np.float64), dtype)
            assert backend.simple(op, a, dst) == 0
            T.assert_same_bits(dst.storage, np.array(case["expect"]).astype(O.NP_STORAGE[dtype]), what)
        elif op == "slice_set":
            a = tensor_from(case["a"], dtype)
            dst = tensor_from(case["dst"], dtype)
            assert backend.simple(op, a, dst, extra=(case["dim"], case["start"], case["end"], case["step"])) == 0
            T.assert_same_bits(dst.storage, np.array(case["expect_storage"]).astype(O.NP_STORAGE[dtype]), what)
        elif op in ("index_select", "index_add"):
            a = tensor_from(case["a"], dtype)
            spec = case["indices"]
            idx = T.HostTensor(np.array(spec["values"], np.int32), O.I32, spec["shape"], spec.get("strides"))
            dst = T.empty(dtype, case["dst_shape"])
            if "dst_init" in case:
                dst.storage[:] = O.to_storage(np.array(case["dst_init"], np.float64), dtype)
            assert backend.simple(op, a, dst, idx, extra=(case["dim"],)) == 0
            T.assert_same_bits(dst.storage, np.array(case["expect"]).astype(O.NP_STORAGE[dtype]), what)
        else:
            raise AssertionError(f"golden case {case['name']}: unknown op {op}")
