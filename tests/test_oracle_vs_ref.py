"""Differential pin of the oracle: every operator of oracle/cpuref.cpp must produce the same
bits as the reference's own DeviceCPU (compiled from the reference tree into
oracle/_ref/libaixref.so) on seeded inputs, for all nine element types and for contiguous,
transposed, sliced, broadcast and offset views.  Skipped where oracle/_ref was not built."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
from oracle import cpuref as O

REF = O.ref_lib()
pytestmark = pytest.mark.skipif(REF is None, reason="oracle/_ref not built (reference tree absent)")
CPU = O.lib()


def both(fn_name, make_args, outs):
    """Run one op on both libraries; `outs` are HostTensors whose storage is the result."""
    results = []
    for lib in (CPU, REF):
        local = [o.clone() for o in outs]
        rc = getattr(lib, fn_name)(*make_args(local))
        results.append((rc, [o.storage.copy() for o in local]))
    (rc_a, a), (rc_b, b) = results
    assert rc_a == rc_b, (fn_name, rc_a, rc_b)
    return a, b


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
@pytest.mark.parametrize("op", [O.ADD, O.SUB, O.MUL, O.DIV, O.POW], ids=["add", "sub", "mul", "div", "pow"])
def test_binary(op, dtype):
    rng = np.random.default_rng(1000 + op * 16 + dtype)
    for trial in range(12):
        shape = T.random_shape(rng)
        ka, kb = rng.choice(T.VIEW_KINDS, 2)
        kw = {}
        if dtype in T.INT_DTYPES:
            kw = dict(int_span=6 if op == O.POW else 100)
        a = T.view_tensor(rng, dtype, shape, ka, **kw)
        b = T.view_tensor(rng, dtype, shape, kb, **kw)
        if dtype in T.INT_DTYPES and op == O.DIV:
            b.storage[b.storage == 0] = 3
        out = T.empty(dtype, shape)
        x, y = both("binary", lambda o: (op, C.byref(a.desc()), C.byref(b.desc()), C.byref(o[0].desc())), [out])
        T.assert_same_bits_nan_ok(x[0], y[0], dtype, f"binary op={op} {O.DTYPE_NAMES[dtype]} {shape} {ka}/{kb}")


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
@pytest.mark.parametrize("op", range(7), ids=["neg", "sqrt", "sin", "cos", "tanh", "log", "exp"])
def test_unary(op, dtype):
    rng = np.random.default_rng(2000 + op * 16 + dtype)
    for trial in range(10):
        shape = T.random_shape(rng)
        kind = rng.choice(T.VIEW_KINDS)
        a = T.view_tensor(rng, dtype, shape, kind, lo=-4.0, hi=12.0)
        out = T.empty(dtype, shape)
        x, y = both("unary", lambda o: (op, C.byref(a.desc()), C.byref(o[0].desc())), [out])
        T.assert_same_bits_nan_ok(x[0], y[0], dtype, f"unary op={op} {O.DTYPE_NAMES[dtype]} {shape} {kind}")


SPECIALS = [0.0, -0.0, 1.0, -1.0, 0.5, 255.0, 256.0, 300.0, -129.0, 32767.6, -32768.9, 65504.0, 65520.0,
            1e9, -1e9, 3e9, 2147483647.0, 2147483648.0, -2147483649.0, 9.3e18, -9.3e18, 1e30, -1e30,
            float("inf"), float("-inf"), float("nan"), 1e-8, 6e-8, 5.96e-8, 2.98e-8, 6.1e-5, 3.14]


@pytest.mark.parametrize("src", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
@pytest.mark.parametrize("dst", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_copy_and_fill(src, dst):
    rng = np.random.default_rng(3000 + src * 16 + dst)
    if src in T.FLOAT_DTYPES:
        with np.errstate(over="ignore", invalid="ignore"):
            vals = np.concatenate([np.array(SPECIALS), rng.uniform(-400, 400, 64), rng.uniform(-1, 1, 32) * 1e6])
            st = O.to_storage(vals, src)
    else:
        info = np.iinfo(O.NP_STORAGE[src])
        st = np.concatenate([np.array([info.min, info.max, 0, 1, -1 if info.min < 0 else 2], dtype=O.NP_STORAGE[src]),
                             rng.integers(info.min, info.max, 64, endpoint=True).astype(O.NP_STORAGE[src])])
    n = st.size
    out = T.empty(dst, [n])
    x, y = both("copy", lambda o: (st.ctypes.data, src, o[0].storage.ctypes.data, dst, n), [out])
    T.assert_same_bits_nan_ok(x[0], y[0], dst, f"copy {O.DTYPE_NAMES[src]}->{O.DTYPE_NAMES[dst]}")
    for k in range(0, n, 7):
        scalar = st[k:k + 1].copy()
        out = T.empty(dst, [5])
        x, y = both("fill", lambda o: (scalar.ctypes.data, src, C.byref(o[0].desc())), [out])
        T.assert_same_bits_nan_ok(x[0], y[0], dst, f"fill {O.DTYPE_NAMES[src]}->{O.DTYPE_NAMES[dst]} {scalar}")


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_fill_min_full_reductions_and_argmax(dtype):
    rng = np.random.default_rng(4000 + dtype)
    out = T.empty(dtype, [9])
    x, y = both("fill_min", lambda o: (C.byref(o[0].desc()),), [out])
    T.assert_same_bits(x[0], y[0], "fillMin")
    for trial in range(12):
        shape = T.random_shape(rng)
        kind = rng.choice(T.VIEW_KINDS)
        a = T.view_tensor(rng, dtype, shape, kind, int_span=3)    # small span -> many ties
        for name, odt, oshape in (("sum", dtype, []), ("max", dtype, []), ("argmax", O.I32, []),
                                  ("argmax_indices", O.I32, shape)):
            out = T.empty(odt, oshape)
            x, y = both(name, lambda o: (C.byref(a.desc()), C.byref(o[0].desc())), [out])
            T.assert_same_bits_nan_ok(x[0], y[0], odt, f"{name} {O.DTYPE_NAMES[dtype]} {shape} {kind}")
    # wrong result dtype -> invalid_argument on both
    a = T.contiguous_tensor(rng, dtype, [4])
    bad = T.empty(O.F32, [])
    for name in ("argmax", "argmax_indices"):
        assert getattr(CPU, name)(C.byref(a.desc()), C.byref(bad.desc())) == 1
        assert getattr(REF, name)(C.byref(a.desc()), C.byref(bad.desc())) == 1


def reduced_shapes(rng, shape):
    """Destination shapes a caller may pass to reduceTo/maxTo for a source shape."""
    rank = len(shape)
    outs = []
    for _ in range(3):
        mask = [bool(rng.integers(0, 2)) for _ in shape]
        outs.append([1 if m else e for e, m in zip(shape, mask)])        # keep-dim form
    outs.append([1] * rank)
    k = int(rng.integers(0, rank))
    outs.append(shape[k:])                                                # leading dims dropped
    outs.append([1 if i % 2 else e for i, e in enumerate(shape[k:])])
    return outs


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_reduce_to_and_max_to(dtype):
    rng = np.random.default_rng(5000 + dtype)
    for trial in range(10):
        shape = T.random_shape(rng, max_rank=5, max_extent=6)
        kind = rng.choice(T.VIEW_KINDS)
        src = T.view_tensor(rng, dtype, shape, kind, int_span=20)
        for dshape in reduced_shapes(rng, shape):
            init = T.contiguous_tensor(rng, dtype, dshape, int_span=5)    # accumulate-into contract
            for name in ("reduce_to", "max_to"):
                x, y = both(name, lambda o: (C.byref(src.desc()), C.byref(o[0].desc())), [init])
                T.assert_same_bits_nan_ok(x[0], y[0], dtype, f"{name} {O.DTYPE_NAMES[dtype]} {shape}->{dshape} {kind}")


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_argmax_to_family(dtype):
    rng = np.random.default_rng(6000 + dtype)
    for trial in range(14):
        shape = T.random_shape(rng, max_rank=4, max_extent=6)
        kind = rng.choice(["contig", "contig", "transposed", "sliced", "offset"])
        src = T.view_tensor(rng, dtype, shape, kind, int_span=2)
        dim = int(rng.integers(0, len(shape)))
        keep = [1 if d == dim else e for d, e in enumerate(shape)]
        for dshape in (keep, [e for d, e in enumerate(shape) if d != dim] or [1]):
            out = T.empty(O.I32, dshape, fill=-7)
            x, y = both("argmax_to", lambda o: (C.byref(src.desc()), C.byref(o[0].desc()), dim), [out])
            T.assert_same_bits(x[0], y[0], f"argmaxTo {O.DTYPE_NAMES[dtype]} {shape} dim={dim} {kind} -> {dshape}")
        onehot = T.empty(O.I32, shape)
        x, y = both("argmax_indices_to", lambda o: (C.byref(src.desc()), C.byref(o[0].desc()), dim), [onehot])
        T.assert_same_bits(x[0], y[0], f"argmaxIndicesTo {O.DTYPE_NAMES[dtype]} {shape} dim={dim} {kind}")


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_matmul(dtype):
    rng = np.random.default_rng(7000 + dtype)
    for trial in range(10):
        m, k, n = (int(v) for v in rng.integers(1, 24, 3))
        ka, kb = rng.choice(["contig", "transposed", "sliced", "offset"], 2)
        a = T.view_tensor(rng, dtype, [m, k], ka, int_span=9)
        b = T.view_tensor(rng, dtype, [k, n], kb, int_span=9)
        out = T.empty(dtype, [m, n])
        x, y = both("matmul", lambda o: (C.byref(a.desc()), C.byref(b.desc()), C.byref(o[0].desc())), [out])
        T.assert_same_bits(x[0], y[0], f"matmul {O.DTYPE_NAMES[dtype]} {m}x{k}x{n} {ka}/{kb}")
        # the threaded row-split variant is the same arithmetic
        out2 = T.empty(dtype, [m, n])
        assert CPU.matmul_rows(C.byref(a.desc()), C.byref(b.desc()), C.byref(out2.desc()), 3) == 0
        T.assert_same_bits(out2.storage, y[0], "matmul_rows")


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_layout_ops(dtype):
    rng = np.random.default_rng(8000 + dtype)
    for trial in range(10):
        shape = T.random_shape(rng, max_rank=4, max_extent=7)
        rank = len(shape)
        kind = rng.choice(T.VIEW_KINDS)
        src = T.view_tensor(rng, dtype, shape, kind)
        # contiguous
        out = T.empty(dtype, shape)
        x, y = both("contiguous", lambda o: (C.byref(src.desc()), C.byref(o[0].desc())), [out])
        T.assert_same_bits(x[0], y[0], f"contiguous {shape} {kind}")
        # transpose (device op; contiguous source)
        csrc = T.contiguous_tensor(rng, dtype, shape)
        d0, d1 = (int(v) for v in rng.integers(0, rank, 2))
        tshape = list(shape)
        tshape[d0], tshape[d1] = tshape[d1], tshape[d0]
        out = T.empty(dtype, tshape)
        x, y = both("transpose", lambda o: (C.byref(csrc.desc()), C.byref(o[0].desc()), d0, d1), [out])
        T.assert_same_bits(x[0], y[0], f"transpose {shape} {d0},{d1}")
        # tril / triu with strided dst
        if rank >= 2:
            for name in ("tril", "triu"):
                diag = int(rng.integers(-3, 4))
                dst = T.view_tensor(rng, dtype, shape, rng.choice(["contig", "transposed", "sliced", "offset"]))
                x, y = both(name, lambda o: (C.byref(src.desc()), C.byref(o[0].desc()), diag), [dst])
                T.assert_same_bits(x[0], y[0], f"{name} {shape} diag={diag}")
        # sliceSet into a larger dst (offset 0: the CPU device ignores dst.offset)
        dim = int(rng.integers(0, rank))
        step = int(rng.integers(1, 3))
        start = int(rng.integers(0, 3))
        big = list(shape)
        big[dim] = start + (shape[dim] - 1) * step + 1 + int(rng.integers(0, 2))
        end = min(big[dim], start + shape[dim] * step)
        assert (end - start + step - 1) // step == shape[dim]
        dst = T.view_tensor(rng, dtype, big, rng.choice(["contig", "transposed"]))
        for lib, extra in ((CPU, (0,)), (REF, ())):
            pass
        a_dst, b_dst = dst.clone(), dst.clone()
        assert CPU.slice_set(C.byref(src.desc()), C.byref(a_dst.desc()), dim, start, end, step, 0) == 0
        assert REF.slice_set(C.byref(src.desc()), C.byref(b_dst.desc()), dim, start, end, step) == 0
        T.assert_same_bits(a_dst.storage, b_dst.storage, f"sliceSet {shape}->{big} dim={dim}")
        # indexSelect / indexAdd
        ni = int(rng.integers(1, 6))
        idx = HostIdx = T.HostTensor(rng.integers(0, shape[dim], ni).astype(np.int32), O.I32, [ni])
        sel_shape = list(shape)
        sel_shape[dim] = ni
        a_out, b_out = T.empty(dtype, sel_shape), T.empty(dtype, sel_shape)
        assert CPU.index_select(C.byref(src.desc()), C.byref(a_out.desc()), C.byref(idx.desc()), dim, 0) == 0
        assert REF.index_select(C.byref(src.desc()), C.byref(b_out.desc()), C.byref(idx.desc()), dim) == 0
        T.assert_same_bits(a_out.storage, b_out.storage, f"indexSelect {shape} dim={dim}")
        upd = T.view_tensor(rng, dtype, sel_shape, kind)
        acc = T.contiguous_tensor(rng, dtype, shape)
        a_acc, b_acc = acc.clone(), acc.clone()
        assert CPU.index_add(C.byref(upd.desc()), C.byref(a_acc.desc()), C.byref(idx.desc()), dim, 0) == 0
        assert REF.index_add(C.byref(upd.desc()), C.byref(b_acc.desc()), C.byref(idx.desc()), dim) == 0
        T.assert_same_bits(a_acc.storage, b_acc.storage, f"indexAdd {shape} dim={dim}")


def test_half_conversions_exhaustive():
    """All 65536 f16 and bf16 patterns up to f32 and back, and f32 -> 16 bit on a dense sample
    around every rounding boundary, against the reference's conversion code."""
    pats = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    for dt in (O.F16, O.BF16):
        st = pats.view(O.NP_STORAGE[dt]) if dt == O.F16 else pats
        up_a, up_b = np.zeros(65536, np.float32), np.zeros(65536, np.float32)
        assert CPU.copy(st.ctypes.data, dt, up_a.ctypes.data, O.F32, 65536) == 0
        assert REF.copy(st.ctypes.data, dt, up_b.ctypes.data, O.F32, 65536) == 0
        T.assert_same_bits(up_a.view(np.uint32), up_b.view(np.uint32), f"{O.DTYPE_NAMES[dt]}->f32")
        # each representable value, one f32 step either side of it, and each midpoint
        base = up_b.view(np.uint32).astype(np.int64)
        nxt = np.roll(base, -1)
        cand = np.concatenate([base, base + 1, base - 1, (base + nxt) // 2, (base + nxt) // 2 + 1,
                               (base + nxt) // 2 - 1]) & 0xFFFFFFFF
        f = cand.astype(np.uint32).view(np.float32).copy()
        dn_a, dn_b = np.zeros(f.size, np.uint16), np.zeros(f.size, np.uint16)
        assert CPU.copy(f.ctypes.data, O.F32, dn_a.ctypes.data, dt, f.size) == 0
        assert REF.copy(f.ctypes.data, O.F32, dn_b.ctypes.data, dt, f.size) == 0
        T.assert_same_bits(dn_a, dn_b, f"f32->{O.DTYPE_NAMES[dt]}")
