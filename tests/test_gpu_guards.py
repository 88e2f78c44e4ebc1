"""Guards of the kernel layer: indices at and beyond the ends of the indexed dimension, and in-place single
operators (result aliasing the first operand, Targets/AIXLib/aixCore.hpp:1447, 1451) on the precompiled elementwise
kernels for each launch shape (flat, rows, gather)."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import gpuharness as G
from oracle import cpuref as O

CPU = O.lib()
NAMES = O.DTYPE_NAMES
ids = lambda d: NAMES[d]  # noqa: E731


def okc(rc):
    assert rc == 0, rc


@pytest.fixture(scope="module")
def gpu():
    g = G.Gpu()
    yield g
    g.close()
    g.ctx.close()


def test_oracle_refuses_indices_outside_the_dimension():
    """CPU side of the guard: the oracle returns 'invalid argument' and touches nothing."""
    src = T.HostTensor(np.arange(12, dtype=np.float32), O.F32, [4, 3])
    for bad in (-1, 4, 2 ** 31 - 1, -2 ** 31):
        idx = T.HostTensor(np.array([0, bad, 3], np.int32), O.I32, [3])
        out = T.empty(O.F32, [3, 3], fill=7)
        assert CPU.index_select(C.byref(src.desc()), C.byref(out.desc()), C.byref(idx.desc()), 0, 1) == 1
        assert np.all(out.storage == 7)
        acc = T.empty(O.F32, [4, 3], fill=7)
        upd = T.HostTensor(np.ones(9, np.float32), O.F32, [3, 3])
        assert CPU.index_add(C.byref(upd.desc()), C.byref(acc.desc()), C.byref(idx.desc()), 0, 1) == 1
        assert np.all(acc.storage == 7)
    idx = T.HostTensor(np.array([0, 3], np.int32), O.I32, [2])           # both ends of the range are fine
    out = T.empty(O.F32, [2, 3])
    okc(CPU.index_select(C.byref(src.desc()), C.byref(out.desc()), C.byref(idx.desc()), 0, 1))
    assert np.array_equal(out.storage, np.array([0, 1, 2, 9, 10, 11], np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [O.F32, O.BF16, O.F16, O.I32, O.U8, O.F64], ids=ids)
def test_index_ops_at_the_ends_of_the_dimension(gpu, dtype):
    """Indices 0 and extent-1 (valid) against the oracle; indices outside [0, extent) touch no memory: indexSelect
    writes zeros for them, indexAdd leaves the destination alone."""
    rng = np.random.default_rng(31 + dtype)
    for shape, dim in (([5, 8], 0), ([3, 7, 4], 1), ([6], 0), ([4, 6, 2], 2)):
        extent = shape[dim]
        src = T.contiguous_tensor(rng, dtype, shape)
        _, dsrc = gpu.put(src)
        ends = np.array([0, extent - 1, extent - 1, 0], np.int32)
        idx = T.HostTensor(ends, O.I32, [4])
        _, didx = gpu.put(idx)
        sel = list(shape)
        sel[dim] = 4
        want = T.empty(dtype, sel)
        okc(CPU.index_select(C.byref(src.desc()), C.byref(want.desc()), C.byref(idx.desc()), dim, 1))
        po, do = gpu.put(T.empty(dtype, sel, fill=3))
        G.run_gpu(gpu, "aixk_index_select", G.ref(dsrc), G.ref(do), G.ref(didx), dim)
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"indexSelect ends {NAMES[dtype]} {shape} dim={dim}")

        upd = T.HostTensor(O.to_storage(rng.integers(0, 4, O.numel(sel)).astype(np.float64), dtype), dtype, sel)
        acc = T.HostTensor(O.to_storage(rng.integers(0, 5, O.numel(shape)).astype(np.float64), dtype), dtype, shape)
        want = acc.clone()
        okc(CPU.index_add(C.byref(upd.desc()), C.byref(want.desc()), C.byref(idx.desc()), dim, 1))
        _, dupd = gpu.put(upd)
        pa, dacc = gpu.put(acc)
        G.run_gpu(gpu, "aixk_index_add", G.ref(dupd), G.ref(dacc), G.ref(didx), dim)
        T.assert_same_bits(gpu.fetch(pa, want.storage), want.storage, f"indexAdd ends {NAMES[dtype]} {shape} dim={dim}")

        # the same calls with two indices outside the range: valid rows as before, the others guarded
        mixed = np.array([0, -1, extent - 1, extent], np.int32)
        valid = np.array([True, False, True, False])
        midx = T.HostTensor(mixed, O.I32, [4])
        _, dmidx = gpu.put(midx)
        po, do = gpu.put(T.empty(dtype, sel, fill=3))
        G.run_gpu(gpu, "aixk_index_select", G.ref(dsrc), G.ref(do), G.ref(dmidx), dim)
        got = np.ascontiguousarray(np.moveaxis(gpu.fetch(po, np.zeros(O.numel(sel), O.NP_STORAGE[dtype])).reshape(sel), dim, 0)).reshape(4, -1)
        full = np.ascontiguousarray(np.moveaxis(src.gather(), dim, 0)).reshape(extent, -1)
        assert np.array_equal(got[0].view(np.uint8), full[0].view(np.uint8)) and np.array_equal(got[2].view(np.uint8), full[extent - 1].view(np.uint8))
        assert not got[1].view(np.uint8).any() and not got[3].view(np.uint8).any()
        clean = T.HostTensor(np.where(valid, mixed, 0).astype(np.int32), O.I32, [4])
        upd_valid = np.moveaxis(upd.gather().copy(), dim, 0)
        upd_valid[~valid] = O.to_storage(np.zeros(1), dtype)[0]          # what a skipped row adds: nothing
        upd2 = T.HostTensor(np.ascontiguousarray(np.moveaxis(upd_valid, 0, dim)), dtype, sel)
        want = acc.clone()
        okc(CPU.index_add(C.byref(upd2.desc()), C.byref(want.desc()), C.byref(clean.desc()), dim, 1))
        pa, dacc = gpu.put(acc)
        G.run_gpu(gpu, "aixk_index_add", G.ref(dupd), G.ref(dacc), G.ref(dmidx), dim)
        T.assert_same_bits(gpu.fetch(pa, want.storage), want.storage, f"indexAdd guarded {NAMES[dtype]} {shape} dim={dim}")
        gpu.release()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_single_in_place_operators(gpu, dtype):
    """out aliases a on each launch shape of the precompiled kernels: flat (dense operands), rows (b a broadcast
    row or column) and gather (b a transposed view)."""
    rng = np.random.default_rng(8100 + dtype)
    for shape in ([1000], [37, 64], [16, 48], [5, 7, 9]):
        layouts = ["contig"]
        if len(shape) >= 2:
            layouts += ["row", "column", "transposed"]
        for layout in layouts:
            a = T.contiguous_tensor(rng, dtype, shape, int_span=30)
            if layout == "contig":
                b = T.contiguous_tensor(rng, dtype, shape, int_span=30)
            elif layout == "row":
                b = T.HostTensor(T.random_values(rng, shape[-1], dtype, int_span=30), dtype, shape, [0] * (len(shape) - 1) + [1])
            elif layout == "column":
                lead = O.numel(shape[:-1])
                b = T.HostTensor(T.random_values(rng, lead, dtype, int_span=30), dtype, shape, O.row_major(shape[:-1] + [1])[:-1] + [0])
            else:
                b = T.view_tensor(rng, dtype, shape, "transposed", int_span=30)
            for op in (O.ADD, O.MUL, O.SUB):
                want = a.clone()
                okc(CPU.binary(op, C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc())))
                pa, da = gpu.put(a)
                _, db = gpu.put(b)
                G.run_gpu(gpu, "aixk_binary", op, G.ref(da), G.ref(db), G.ref(da))
                T.assert_same_bits(gpu.fetch(pa, want.storage), want.storage, f"in-place op {op} {NAMES[dtype]} {shape} {layout}")
            want = a.clone()
            okc(CPU.unary(O.NEG, C.byref(a.desc()), C.byref(want.desc())))
            pa, da = gpu.put(a)
            G.run_gpu(gpu, "aixk_unary", O.NEG, G.ref(da), G.ref(da))
            T.assert_same_bits(gpu.fetch(pa, want.storage), want.storage, f"in-place negate {NAMES[dtype]} {shape}")
            gpu.release()
