"""Parity of the gfx950 kernels (through the C ABI of libaixhip_kernels.so) against the CPU oracle
on identical seeded inputs, following the reference's device-parity pattern
(Targets/AIXTests/DeviceTests.cpp:199-233: same raw device call on the CPU device and on the
device under test, then compare).

Tolerances (stated per test):
  * integers, indices, data movement, casts, fill: bit-exact;
  * f64/f32/f16/bf16 add, sub, mul, div, negate, sqrt: bit-exact;
  * f32 sin/cos/tanh/log/exp/pow: <= 2 ulp; f64: <= 4 ulp; f16/bf16: <= 1 ulp of the 16-bit type;
  * float reductions and f32 matmul: |err| <= 1e-5 x sum|terms| against an exactly accumulated
    oracle; f16/bf16 additionally allow the final rounding of the result (2^-10 / 2^-8 relative);
  * f16/bf16 matmul: <= 2e-2 x sum|a||b|.
"""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import gpuharness as G
from aix_amd import kernels as K
from oracle import cpuref as O

pytestmark = pytest.mark.gpu
CPU = O.lib()
NAMES = O.DTYPE_NAMES
ids = lambda d: NAMES[d]  # noqa: E731

SIZES = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257,
         511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049]      # as DeviceTests.cpp:30-31


@pytest.fixture(scope="module")
def gpu():
    g = G.Gpu()
    yield g
    g.close()
    g.ctx.close()


def okc(rc):
    assert rc == 0, rc


# ---- elementwise ----------------------------------------------------------------------------------
def binary_rule(op, dtype):
    if dtype in T.INT_DTYPES or op != O.POW:
        return G.EXACT
    return {O.F32: 2, O.F64: 4, O.F16: 1, O.BF16: 1}[dtype]


def unary_rule(op, dtype):
    if op == O.SQRT and dtype == O.F64:
        # The CPU evaluates sqrt in 80-bit long double and rounds a second time to double
        # (aixDeviceCPU.cpp:162-163); about 1 result in 10^4 is then one unit away from the
        # correctly rounded double the GPU returns.
        return 1
    if dtype in T.INT_DTYPES or op in (O.NEG, O.SQRT):
        return G.EXACT
    return {O.F32: 2, O.F64: 4, O.F16: 1, O.BF16: 1}[dtype]


def check_binary(gpu, op, a, b, what):
    dtype = a.dtype
    want = T.empty(dtype, a.shape)
    okc(CPU.binary(op, C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc())))
    _, da = gpu.put(a)
    _, db = gpu.put(b)
    po, do = gpu.put(T.empty(dtype, a.shape))
    G.run_gpu(gpu, "aixk_binary", op, G.ref(da), G.ref(db), G.ref(do))
    got = gpu.fetch(po, want.storage)
    G.compare(got, want.storage, dtype, binary_rule(op, dtype), what)


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
@pytest.mark.parametrize("op", [O.ADD, O.SUB, O.MUL, O.DIV, O.POW], ids=["add", "sub", "mul", "div", "pow"])
def test_binary_views(gpu, op, dtype):
    rng = np.random.default_rng(11000 + op * 16 + dtype)
    kw = dict(int_span=5 if op == O.POW else 100) if dtype in T.INT_DTYPES else dict(lo=0.05, hi=3.0) if op == O.POW else {}
    for trial in range(14):
        shape = T.random_shape(rng, max_rank=5)
        ka, kb = rng.choice(T.VIEW_KINDS, 2)
        a = T.view_tensor(rng, dtype, shape, ka, **kw)
        b = T.view_tensor(rng, dtype, shape, kb, **kw)
        check_binary(gpu, op, a, b, f"binary op={op} {NAMES[dtype]} {shape} {ka}/{kb}")
    gpu.release()


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16], ids=ids)
def test_pow_squares_and_cubes(gpu, dtype):
    """Exponents 2 and 3 are evaluated as products (GELU's x^3 and its derivative): the same bar as every other
    pow against the CPU's long-double powl, over signs, zeros, tiny and huge bases, infinities and NaN, with the
    exponent as a broadcast scalar and as a full tensor that mixes 2, 3 and other exponents."""
    rng = np.random.default_rng(11900 + dtype)
    n = 4096
    base = np.concatenate([rng.uniform(-30, 30, n - 24), [0.0, -0.0, 1.0, -1.0, 1e-13, -1e-13, 1e-20, 3e12, -3e12, 1e19, -1e19, 2.5e38,
                                                           np.inf, -np.inf, np.nan, 65504.0, -65504.0, 6e-8, 255.0, -255.0, 0.5, -0.5, 1e-5, -1e-5]])
    a = T.HostTensor(O.to_storage(base, dtype), dtype, [n])
    for e in (2.0, 3.0):
        b = T.HostTensor(O.to_storage(np.array([e]), dtype), dtype, [n], [0])
        check_binary(gpu, O.POW, a, b, f"pow {NAMES[dtype]} exponent {e} (scalar)")
    mixed = T.HostTensor(O.to_storage(rng.choice([2.0, 3.0, 2.5, -1.0, 0.0, 1.0], n), dtype), dtype, [n])
    positive = T.HostTensor(O.to_storage(np.abs(base) + 0.05, dtype), dtype, [n])
    check_binary(gpu, O.POW, positive, mixed, f"pow {NAMES[dtype]} mixed exponents")
    gpu.release()


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_binary_sizes_and_broadcast_rows(gpu, dtype):
    """Flat sizes 1..2049 (vector body + tail) and the row / column / scalar broadcast forms the
    front-end produces (bias add, Tensor op scalar)."""
    rng = np.random.default_rng(12000 + dtype)
    for n in SIZES:
        a = T.contiguous_tensor(rng, dtype, [n])
        b = T.contiguous_tensor(rng, dtype, [n])
        check_binary(gpu, O.ADD, a, b, f"add {NAMES[dtype]} n={n}")
        check_binary(gpu, O.MUL, a, b, f"mul {NAMES[dtype]} n={n}")
    gpu.release()
    for rows, cols in [(3, 8), (5, 64), (17, 1024), (64, 96), (7, 33), (130, 2048)]:
        a = T.contiguous_tensor(rng, dtype, [rows, cols])
        row = T.HostTensor(T.random_values(rng, cols, dtype), dtype, [rows, cols], [0, 1])
        col = T.HostTensor(T.random_values(rng, rows, dtype), dtype, [rows, cols], [1, 0])
        sc = T.HostTensor(T.random_values(rng, 1, dtype), dtype, [rows, cols], [0, 0])
        for other, name in ((row, "row"), (col, "col"), (sc, "scalar")):
            check_binary(gpu, O.ADD, a, other, f"add {NAMES[dtype]} [{rows},{cols}] + {name}")
            check_binary(gpu, O.SUB, other, a, f"sub {NAMES[dtype]} {name} - [{rows},{cols}]")
        gpu.release()


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
@pytest.mark.parametrize("op", range(7), ids=["neg", "sqrt", "sin", "cos", "tanh", "log", "exp"])
def test_unary(gpu, op, dtype):
    rng = np.random.default_rng(13000 + op * 16 + dtype)
    cases = []
    for trial in range(8):
        shape = T.random_shape(rng)
        cases.append((shape, rng.choice(T.VIEW_KINDS)))
    cases += [([n], "contig") for n in (1, 5, 64, 257, 2049, 40000)]
    for shape, kind in cases:
        lo, hi = (-4.0, 8.0)
        if op in (O.SQRT, O.LOG):
            lo, hi = (0.0, 30.0)
        a = T.view_tensor(rng, dtype, shape, kind, lo=lo, hi=hi, int_span=12)
        want = T.empty(dtype, shape)
        okc(CPU.unary(op, C.byref(a.desc()), C.byref(want.desc())))
        _, da = gpu.put(a)
        po, do = gpu.put(T.empty(dtype, shape))
        G.run_gpu(gpu, "aixk_unary", op, G.ref(da), G.ref(do))
        got = gpu.fetch(po, want.storage)
        G.compare(got, want.storage, dtype, unary_rule(op, dtype), f"unary op={op} {NAMES[dtype]} {shape} {kind}")
    gpu.release()


def test_unary_f32_special_values(gpu):
    """Signed zeros, infinities, NaN, denormals and large arguments through every f32 function."""
    vals = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-38, 3e-39, 88.7, 89.0, -87.0,
                     -104.0, 1e10, -1e10, 0.5, 2.0, 3.1415927, 1e-4, 9.0, 16.0, 1e38, 3.4e38, 100.0, 710.0], dtype=np.float32)
    a = T.HostTensor(vals, O.F32, [vals.size])
    for op in range(7):
        want = T.empty(O.F32, a.shape)
        okc(CPU.unary(op, C.byref(a.desc()), C.byref(want.desc())))
        _, da = gpu.put(a)
        po, do = gpu.put(T.empty(O.F32, a.shape))
        G.run_gpu(gpu, "aixk_unary", op, G.ref(da), G.ref(do))
        got = gpu.fetch(po, want.storage)
        G.compare(got, want.storage, O.F32, unary_rule(op, O.F32), f"special values op={op}")
    gpu.release()


def test_f32_transcendental_ulp_histogram(gpu):
    """1M-point ulp histograms of each f32 function against the oracle; the bound is 2 ulp."""
    rng = np.random.default_rng(14000)
    n = 1 << 20
    for op, lo, hi in ((O.SIN, -20, 20), (O.COS, -20, 20), (O.TANH, -10, 10), (O.EXP, -80, 80), (O.LOG, 1e-30, 1e30)):
        if op == O.LOG:
            x = np.exp(rng.uniform(np.log(lo), np.log(hi), n)).astype(np.float32)
        else:
            x = rng.uniform(lo, hi, n).astype(np.float32)
        a = T.HostTensor(x, O.F32, [n])
        want = T.empty(O.F32, [n])
        okc(CPU.unary(op, C.byref(a.desc()), C.byref(want.desc())))
        _, da = gpu.put(a)
        po, do = gpu.put(T.empty(O.F32, [n]))
        G.run_gpu(gpu, "aixk_unary", op, G.ref(da), G.ref(do))
        got = gpu.fetch(po, want.storage)
        worst, hist = O.ulp_hist_f32(got, want.storage)
        print(f"ulp histogram op={op}: worst={worst} hist={hist[:6].tolist()}")
        assert worst <= 2, (op, worst, hist)
        gpu.release()


# ---- fill / fillMin / cast ------------------------------------------------------------------------
SPECIALS = [0.0, -0.0, 1.0, -1.0, 0.5, 255.0, 256.0, 300.0, -129.0, 32767.6, -32768.9, 65504.0, 65520.0,
            1e9, -1e9, 3e9, 2147483647.0, 2147483648.0, -2147483649.0, 9.3e18, -9.3e18, 1e30, -1e30,
            float("inf"), float("-inf"), float("nan"), 1e-8, 6e-8, 5.96e-8, 2.98e-8, 6.1e-5, 3.14]


@pytest.mark.parametrize("src", T.ALL_DTYPES, ids=ids)
def test_cast_and_fill(gpu, src):
    rng = np.random.default_rng(15000 + src)
    if src in T.FLOAT_DTYPES:
        with np.errstate(over="ignore", invalid="ignore"):
            vals = np.concatenate([np.array(SPECIALS), rng.uniform(-400, 400, 2100), rng.uniform(-1, 1, 64) * 1e6])
            st = O.to_storage(vals, src)
    else:
        info = np.iinfo(O.NP_STORAGE[src])
        st = np.concatenate([np.array([info.min, info.max, 0, 1, 2], dtype=O.NP_STORAGE[src]),
                             rng.integers(info.min, info.max, 2100, endpoint=True).astype(O.NP_STORAGE[src])])
    n = st.size
    ps = gpu.raw(st.nbytes)
    gpu.ctx.upload(ps, st)
    for dst in T.ALL_DTYPES:
        for count in (n, 1, 13):                                   # vector body + tails
            want = np.zeros(count, dtype=O.NP_STORAGE[dst])
            okc(CPU.copy(st.ctypes.data, src, want.ctypes.data, dst, count))
            pd = gpu.raw(want.nbytes)
            G.run_gpu(gpu, "aixk_cast", ps, src, pd, dst, count)
            got = gpu.fetch(pd, want)
            T.assert_same_bits_nan_ok(got, want, dst, f"cast {NAMES[src]}->{NAMES[dst]} n={count}")
        # unaligned source and destination (offset by one element)
        if n > 40:
            want = np.zeros(33, dtype=O.NP_STORAGE[dst])
            okc(CPU.copy(st[1:].ctypes.data, src, want.ctypes.data, dst, 33))
            pd = gpu.raw(want.nbytes + 16)
            G.run_gpu(gpu, "aixk_cast", ps + st.itemsize, src, pd + want.itemsize, dst, 33)
            got = np.empty_like(want)
            gpu.ctx.download(got, pd + want.itemsize)
            T.assert_same_bits_nan_ok(got, want, dst, f"unaligned cast {NAMES[src]}->{NAMES[dst]}")
        for k in list(range(0, 40)) + [n - 1]:
            scalar = st[k:k + 1].copy()
            for count in (1, 19, 300):
                want = T.empty(dst, [count])
                okc(CPU.fill(scalar.ctypes.data, src, C.byref(want.desc())))
                po, do = gpu.put(T.empty(dst, [count]))
                G.run_gpu(gpu, "aixk_fill", scalar.ctypes.data, src, G.ref(do))
                got = gpu.fetch(po, want.storage)
                T.assert_same_bits_nan_ok(got, want.storage, dst, f"fill {NAMES[src]}->{NAMES[dst]} {scalar} n={count}")
        gpu.release()
        ps = gpu.raw(st.nbytes)
        gpu.ctx.upload(ps, st)
    want = T.empty(src, [77])
    okc(CPU.fill_min(C.byref(want.desc())))
    po, do = gpu.put(T.empty(src, [77]))
    G.run_gpu(gpu, "aixk_fill_min", G.ref(do))
    T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"fillMin {NAMES[src]}")
    gpu.release()


def test_f32_to_bf16_every_class_of_input(gpu):
    """The device rounds f32 to bf16 with the hardware conversion; the reference does it on the integer image
    (aixFloat16.hpp:783-805: round to nearest even; NaN = upper half with bit 6 set).  All 65 536 upper halves
    x 48 lower halves (the rounding boundary and its neighbours, zero, all ones, random) -- every exponent,
    every NaN payload class, infinities, subnormals -- must give the same 16 bits, NaN payloads included."""
    rng = np.random.default_rng(15500)
    low = np.concatenate([np.array([0, 1, 2, 0x7FFE, 0x7FFF, 0x8000, 0x8001, 0x8002, 0xFFFE, 0xFFFF, 0x4000, 0xC000], np.uint32),
                          rng.integers(0, 0x10000, 36).astype(np.uint32)])
    bits = ((np.arange(0x10000, dtype=np.uint32)[:, None] << 16) | low[None, :]).reshape(-1)
    src = bits.view(np.float32)
    want = np.zeros(src.size, np.uint16)
    okc(CPU.copy(src.ctypes.data, O.F32, want.ctypes.data, O.BF16, src.size))
    ps, pd = gpu.raw(src.nbytes), gpu.raw(want.nbytes)
    gpu.ctx.upload(ps, src)
    G.run_gpu(gpu, "aixk_cast", ps, O.F32, pd, O.BF16, src.size)
    T.assert_same_bits(gpu.fetch(pd, want), want, "f32 -> bf16")
    gpu.release()


# ---- data movement --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_contiguous_and_transpose(gpu, dtype):
    rng = np.random.default_rng(16000 + dtype)
    cases = [(T.random_shape(rng, max_rank=5, max_extent=7), rng.choice(T.VIEW_KINDS)) for _ in range(12)]
    # 2-D and batched transposes through the LDS-tiled kernel, incl. ragged edges
    cases += [([n, m], "transposed") for n, m in [(1, 1), (1, 70), (63, 65), (64, 64), (129, 257), (300, 5), (5, 300), (513, 1025)]]
    cases += [([3, 70, 130], "transposed"), ([96, 256], "sliced"), ([33, 48], "offset")]
    cases += [([128, 192], "transposed"), ([3, 64, 128], "transposed"), ([256, 64], "transposed")]   # whole tiles: 16-byte path
    cases += [([256, 384], "transposed"), ([384, 256], "transposed"), ([2, 256, 128], "transposed")]  # whole 128 x 64 / 128 x 128 tiles, grouped order
    for shape, kind in cases:
        src = T.view_tensor(rng, dtype, shape, kind)
        want = T.empty(dtype, shape)
        okc(CPU.contiguous(C.byref(src.desc()), C.byref(want.desc())))
        _, ds = gpu.put(src)
        po, do = gpu.put(T.empty(dtype, shape))
        G.run_gpu(gpu, "aixk_contiguous", G.ref(ds), G.ref(do))
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"contiguous {NAMES[dtype]} {shape} {kind} strides={src.strides}")
        gpu.release()
    for trial in range(10):
        shape = T.random_shape(rng, max_rank=4, max_extent=40, max_numel=60000)
        rank = len(shape)
        a = T.contiguous_tensor(rng, dtype, shape)
        d0, d1 = (int(v) for v in rng.integers(0, rank, 2))
        tshape = list(shape)
        tshape[d0], tshape[d1] = tshape[d1], tshape[d0]
        want = T.empty(dtype, tshape)
        okc(CPU.transpose(C.byref(a.desc()), C.byref(want.desc()), d0, d1))
        _, da = gpu.put(a)
        po, do = gpu.put(T.empty(dtype, tshape))
        G.run_gpu(gpu, "aixk_transpose", G.ref(da), G.ref(do), d0, d1)
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"transpose {NAMES[dtype]} {shape} {d0},{d1}")
        gpu.release()


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.I8, O.F64], ids=ids)
def test_contiguous_of_permuted_rows(gpu, dtype):
    """Copies whose unit of movement is a whole row while the dims in front of it are permuted -- attention's
    [batch, heads, seq, d] <-> [batch, seq, heads, d] -- with hops of 4 KB and more between consecutive rows on the
    source side: walked in source order.  Also a permutation of three leading dims, a sliced source with an offset,
    and the mirror case (short hops in the source), which stays on the destination-order kernel."""
    rng = np.random.default_rng(16500 + dtype)
    esz = np.dtype(O.NP_STORAGE[dtype]).itemsize
    d = 64 // esz * 2                                                   # rows of 128 bytes
    for (B, H, S) in ((2, 3, 40), (1, 5, 33)):
        stored = T.random_values(rng, B * H * S * d + 3 * d, dtype, int_span=100)
        views = {
            "heads<->seq": T.HostTensor(stored, dtype, [B, S, H, d], [H * S * d, d, S * d, 1]),
            "seq<->heads, short hops": T.HostTensor(stored, dtype, [B, H, S, d], [H * S * d, d, H * d, 1]),
            "offset": T.HostTensor(stored, dtype, [B, S, H, d], [H * S * d, d, S * d, 1], offset=2 * d),
        }
        big = T.random_values(rng, 3 * 4 * 5 * 2 * 4096 // esz, dtype, int_span=100)
        row = 4096 // esz
        views["three dims"] = T.HostTensor(big, dtype, [5, 4, 3, 2, d], [2 * row, 5 * 2 * row, 4 * 5 * 2 * row, row, 1])
        for name, src in views.items():
            want = T.empty(dtype, src.shape)
            okc(CPU.contiguous(C.byref(src.desc()), C.byref(want.desc())))
            _, ds = gpu.put(src)
            po, do = gpu.put(T.empty(dtype, src.shape))
            G.run_gpu(gpu, "aixk_contiguous", G.ref(ds), G.ref(do))
            T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"contiguous {NAMES[dtype]} {name} {src.shape} strides={src.strides}")
        gpu.release()


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_slice_set_tri_index_ops(gpu, dtype):
    rng = np.random.default_rng(17000 + dtype)
    for trial in range(12):
        shape = T.random_shape(rng, max_rank=4, max_extent=9)
        rank = len(shape)
        kind = rng.choice(T.VIEW_KINDS)
        src = T.view_tensor(rng, dtype, shape, kind)
        _, dsrc = gpu.put(src)
        # sliceSet into a strided, offset window (dst offset honoured as on the reference GPU device)
        dim = int(rng.integers(0, rank))
        step = int(rng.integers(1, 3))
        start = int(rng.integers(0, 3))
        big = list(shape)
        big[dim] = start + (shape[dim] - 1) * step + 1 + int(rng.integers(0, 2))
        end = min(big[dim], start + shape[dim] * step)
        dst = T.view_tensor(rng, dtype, big, rng.choice(["contig", "transposed", "offset", "sliced"]))
        want = dst.clone()
        okc(CPU.slice_set(C.byref(src.desc()), C.byref(want.desc()), dim, start, end, step, 1))
        pd, dd = gpu.put(dst)
        G.run_gpu(gpu, "aixk_slice_set", G.ref(dsrc), G.ref(dd), dim, start, end, step)
        T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, f"sliceSet {NAMES[dtype]} {shape}->{big} dim={dim}")
        # the same with the destination's initialisation folded in: fill(v) + sliceSet in one pass over a dense dst
        scalar = T.random_values(rng, 1, dtype, int_span=50)
        want = T.empty(dtype, big)
        okc(CPU.fill(scalar.ctypes.data, dtype, C.byref(want.desc())))
        okc(CPU.slice_set(C.byref(src.desc()), C.byref(want.desc()), dim, start, end, step, 1))
        pd, dd = gpu.put(T.empty(dtype, big, fill=3))                   # every element must be overwritten
        bits = int(np.frombuffer(scalar.tobytes().ljust(8, b"\0"), dtype=np.uint64)[0])
        G.run_gpu(gpu, "aixk_slice_set_init", G.ref(dsrc), G.ref(dd), dim, start, end, step, bits)
        T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, f"fill + sliceSet {NAMES[dtype]} {shape}->{big} dim={dim}")
        # tril / triu
        if rank >= 2:
            for upper in (0, 1):
                diag = int(rng.integers(-3, 4))
                dst = T.view_tensor(rng, dtype, shape, rng.choice(["contig", "transposed", "sliced", "offset"]))
                want = dst.clone()
                okc((CPU.triu if upper else CPU.tril)(C.byref(src.desc()), C.byref(want.desc()), diag))
                pd, dd = gpu.put(dst)
                G.run_gpu(gpu, "aixk_tri", upper, G.ref(dsrc), G.ref(dd), diag)
                T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, f"tri upper={upper} {NAMES[dtype]} {shape} diag={diag}")
        # indexSelect / indexAdd with strided int32 indices
        ni = int(rng.integers(1, 7))
        raw_idx = rng.integers(0, shape[dim], 2 * ni + 1).astype(np.int32)
        idx = T.HostTensor(raw_idx, O.I32, [ni], [2], 1)
        _, didx = gpu.put(idx)
        sel = list(shape)
        sel[dim] = ni
        want = T.empty(dtype, sel)
        okc(CPU.index_select(C.byref(src.desc()), C.byref(want.desc()), C.byref(idx.desc()), dim, 1))
        po, do = gpu.put(T.empty(dtype, sel))
        G.run_gpu(gpu, "aixk_index_select", G.ref(dsrc), G.ref(do), G.ref(didx), dim)
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"indexSelect {NAMES[dtype]} {shape} dim={dim}")
        # updates are small whole numbers so that sums are exact in every float type and the
        # order in which duplicates are accumulated cannot matter
        upd_vals = rng.integers(0 if dtype == O.U8 else -3, 4, O.numel(sel)).astype(np.float64)
        upd = T.HostTensor(O.to_storage(upd_vals, dtype), dtype, sel)
        acc = T.HostTensor(O.to_storage(rng.integers(0, 5, O.numel(shape)).astype(np.float64), dtype), dtype, shape)
        want = acc.clone()
        okc(CPU.index_add(C.byref(upd.desc()), C.byref(want.desc()), C.byref(idx.desc()), dim, 1))
        _, dupd = gpu.put(upd)
        pa, dacc = gpu.put(acc)
        G.run_gpu(gpu, "aixk_index_add", G.ref(dupd), G.ref(dacc), G.ref(didx), dim)
        T.assert_same_bits(gpu.fetch(pa, want.storage), want.storage, f"indexAdd {NAMES[dtype]} {shape} dim={dim}")
        gpu.release()


# ---- reductions -----------------------------------------------------------------------------------
def float_sum_tolerance(dtype):
    # accumulation error bound (relative to sum |x|) + one rounding of the result in its own type
    return {O.F64: (1e-12, 0.0), O.F32: (1e-5, 0.0), O.F16: (1e-5, 2.0 ** -10), O.BF16: (1e-5, 2.0 ** -8)}[dtype]


def check_sum_like(got_storage, dtype, exact, scale, what):
    tol, final = float_sum_tolerance(dtype)
    got = O.to_float64(got_storage, dtype)
    exact = np.asarray(exact, dtype=np.float64)
    scale = np.asarray(scale, dtype=np.float64)
    G.assert_close_to_wide(got, exact, scale + (final / max(tol, 1e-300)) * np.abs(exact) + 1e-30, tol, what)


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_reduce_all(gpu, dtype):
    rng = np.random.default_rng(18000 + dtype)
    cases = [([n], "contig") for n in SIZES + [70001, 1 << 20]]
    cases += [(T.random_shape(rng, max_rank=4, max_extent=12, max_numel=20000), rng.choice(T.VIEW_KINDS)) for _ in range(10)]
    for shape, kind in cases:
        a = T.view_tensor(rng, dtype, shape, kind, int_span=3)
        _, da = gpu.put(a)
        what = f"{NAMES[dtype]} {shape} {kind}"
        # sum
        po, do = gpu.put(T.empty(dtype, []))
        G.run_gpu(gpu, "aixk_reduce_all", K.SUM, G.ref(da), G.ref(do))
        got = gpu.fetch(po, np.zeros(1, O.NP_STORAGE[dtype]))
        if dtype in T.INT_DTYPES:
            want = T.empty(dtype, [])
            okc(CPU.sum(C.byref(a.desc()), C.byref(want.desc())))
            T.assert_same_bits(got, want.storage, "sum " + what)
        else:
            s, sa = C.c_double(), C.c_double()
            okc(CPU.sum_wide(C.byref(a.desc()), C.byref(s), C.byref(sa)))
            check_sum_like(got, dtype, [s.value], [sa.value], "sum " + what)
        # max, argmax, one-hot: exact
        for kind_code, name, odt, oshape in ((K.MAX, "max", dtype, []), (K.ARGMAX, "argmax", O.I32, []),
                                             (K.ARGMAX_ONEHOT, "argmax_indices", O.I32, shape)):
            want = T.empty(odt, oshape)
            okc(getattr(CPU, name)(C.byref(a.desc()), C.byref(want.desc())))
            po, do = gpu.put(T.empty(odt, oshape, fill=-5 if odt == O.I32 else None))
            G.run_gpu(gpu, "aixk_reduce_all", kind_code, G.ref(da), G.ref(do))
            T.assert_same_bits_nan_ok(gpu.fetch(po, want.storage), want.storage, odt, f"{name} " + what)
        gpu.release()
    # int32-only results (aixDeviceCPU.cpp:1027-1030)
    a = T.contiguous_tensor(rng, dtype, [4])
    _, da = gpu.put(a)
    _, bad = gpu.put(T.empty(O.F32, []))
    assert gpu.ctx.lib.aixk_reduce_all(gpu.ctx.handle, K.ARGMAX, G.ref(da), G.ref(bad)) == 1
    assert b"int32" in gpu.ctx.lib.aixk_last_error()
    gpu.release()


@pytest.mark.parametrize("dtype", [O.F64, O.F32, O.F16, O.BF16], ids=ids)
def test_max_argmax_nan_rules(gpu, dtype):
    """NaN never wins unless it leads its slot (strict '>' scan / std::max on the CPU)."""
    base = np.array([1.0, 5.0, np.nan, 7.0, np.nan, 7.0, 2.0, -np.inf], dtype=np.float64)
    for lead_nan in (False, True):
        for n in (8, 300, 5000):
            vals = np.resize(base, n).copy()
            if lead_nan:
                vals[0] = np.nan
            a = T.HostTensor(O.to_storage(vals, dtype), dtype, [n])
            _, da = gpu.put(a)
            for kind_code, name, odt, oshape in ((K.MAX, "max", dtype, []), (K.ARGMAX, "argmax", O.I32, []),
                                                 (K.ARGMAX_ONEHOT, "argmax_indices", O.I32, [n])):
                want = T.empty(odt, oshape)
                okc(getattr(CPU, name)(C.byref(a.desc()), C.byref(want.desc())))
                po, do = gpu.put(T.empty(odt, oshape))
                G.run_gpu(gpu, "aixk_reduce_all", kind_code, G.ref(da), G.ref(do))
                T.assert_same_bits_nan_ok(gpu.fetch(po, want.storage), want.storage, odt, f"{name} nan lead={lead_nan} n={n}")
            # per-row: rows of 4 with NaN in leading / middle positions
            rows = T.HostTensor(O.to_storage(np.resize(np.array([np.nan, 1, 2, 2, 3, np.nan, 3, 1, -1, -1, np.nan, np.nan]), 96), dtype), dtype, [24, 4])
            _, dr = gpu.put(rows)
            want = T.empty(O.I32, [24, 1])
            okc(CPU.argmax_to(C.byref(rows.desc()), C.byref(want.desc()), 1))
            po, do = gpu.put(T.empty(O.I32, [24, 1]))
            G.run_gpu(gpu, "aixk_argmax_to", 0, G.ref(dr), G.ref(do), 1)
            T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, "argmaxTo with NaN")
            init = T.HostTensor(O.to_storage(np.resize(np.array([-np.inf, np.nan, 2.5]), 24), dtype), dtype, [24, 1])
            want = init.clone()
            okc(CPU.max_to(C.byref(rows.desc()), C.byref(want.desc())))
            pi, di = gpu.put(init)
            G.run_gpu(gpu, "aixk_reduce_to", K.MAX, G.ref(dr), G.ref(di))
            T.assert_same_bits_nan_ok(gpu.fetch(pi, want.storage), want.storage, dtype, "maxTo with NaN")
            gpu.release()


def reduced_shapes(rng, shape):
    rank = len(shape)
    outs = []
    for _ in range(3):
        mask = [bool(rng.integers(0, 2)) for _ in shape]
        outs.append([1 if m else e for e, m in zip(shape, mask)])
    outs.append([1] * rank)
    k = int(rng.integers(0, rank))
    outs.append(shape[k:])
    outs.append([1 if i % 2 else e for i, e in enumerate(shape[k:])])
    return outs


ROUTE_CASES = [  # (source shape, view kind, destination shape) chosen to hit every kernel route
    ([300, 4096], "contig", [300, 1]),        # inner, workgroup per row, vector loads
    ([300, 4100], "contig", [300, 1]),        # inner, long ragged rows
    ([2000, 96], "contig", [2000, 1]),        # inner, wave per row
    ([64, 100], "sliced", [64, 1]),           # inner, scalar loads
    ([500, 10], "contig", [500, 1]),          # short rows: generic, lane per slot
    ([3000, 512], "contig", [1, 512]),        # outer, rows split over workgroups + finish pass
    ([40, 8192], "contig", [1, 8192]),        # outer, single chunk
    ([777, 130], "contig", [130]),            # outer, ragged columns, dst rank dropped
    ([6, 500, 64], "contig", [6, 1, 64]),     # outer with a leading kept dim
    ([50, 70], "transposed", [50, 1]),        # generic
    ([9, 40, 33], "contig", [1, 40, 1]),      # two reduced dims: generic, workgroup per slot
    ([128, 128], "contig", [1, 1]),           # everything folds into one slot
    ([5, 7], "broadcast", [1, 7]),
    ([130, 2304], "contig", [1, 2304]),       # outer, wide rows: workgroups side by side, rows split into chunks
    ([3, 70, 2048], "contig", [3, 1, 2048]),  # the same with a leading kept dim
    ([2, 64, 2048], "contig", [1, 64, 2048]), # a handful of rows (the pair axis of a composed ReLU): wide route, one chunk
    ([1100, 2048], "contig", [1, 2048]),      # outer, many dense rows a workgroup holds whole: one sequential stream per workgroup
    ([2, 1030, 5120], "contig", [2, 1, 5120]),# the same with a leading kept dim and five column tiles per lane
    ([3, 6000, 64], "contig", [3, 6000, 1]),  # very many short rows (softmax rows of a stack of score matrices): several rows per wave
    ([17001, 48], "contig", [17001, 1]),      # the same, rows that leave lanes idle, a ragged last group of rows
    ([7, 4100], "contig", [1, 4100]),         # the same, ragged columns
    ([4, 3, 1024], "contig", [4, 1, 1024]),   # the same with a leading kept dim
]


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_reduce_to_with_folded_initialisation(gpu, dtype):
    """aixk_reduce_to_init(init) == fill(init) followed by aixk_reduce_to, bit for bit (same kernels,
    the destination's old contents replaced by a constant), on every route; and with garbage in dst
    beforehand to show dst is never read.  MAX with the lowest value is what max(dim) issues."""
    rng = np.random.default_rng(19500 + dtype)
    lowest = {O.F64: np.array([-np.finfo(np.float64).max]), O.F32: np.array([-np.finfo(np.float32).max], np.float32),
              O.F16: np.array([0xFBFF], np.uint16), O.BF16: np.array([0xFF7F], np.uint16),
              O.I64: np.array([np.iinfo(np.int64).min]), O.I32: np.array([np.iinfo(np.int32).min], np.int32),
              O.I16: np.array([np.iinfo(np.int16).min], np.int16), O.I8: np.array([-128], np.int8), O.U8: np.array([0], np.uint8)}[dtype]
    for shape, kind, dshape in ROUTE_CASES:
        src = T.view_tensor(rng, dtype, shape, kind, int_span=20)
        _, ds = gpu.put(src)
        for code, bits_arr in ((K.SUM, np.zeros(1, O.NP_STORAGE[dtype])), (K.SUM, O.to_storage(np.array([3.0]), dtype)), (K.MAX, lowest)):
            bits = int.from_bytes(bits_arr.tobytes()[:O.ITEMSIZE[dtype]], "little")
            filled = T.HostTensor(np.resize(bits_arr.view(O.NP_STORAGE[dtype]), max(1, int(np.prod(dshape)))).copy(), dtype, dshape)
            pa, da = gpu.put(filled)
            G.run_gpu(gpu, "aixk_reduce_to", code, G.ref(ds), G.ref(da))
            want = gpu.fetch(pa, filled.storage)
            garbage = T.contiguous_tensor(rng, dtype, dshape, int_span=50)
            pb, db = gpu.put(garbage)
            G.run_gpu(gpu, "aixk_reduce_to_init", code, G.ref(ds), G.ref(db), C.c_uint64(bits))
            T.assert_same_bits_nan_ok(gpu.fetch(pb, filled.storage), want, dtype, f"reduce_to_init {NAMES[dtype]} {shape}->{dshape} {kind} code {code}")
        gpu.release()


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_reduce_to_and_max_to(gpu, dtype):
    rng = np.random.default_rng(19000 + dtype)
    cases = list(ROUTE_CASES)
    for _ in range(8):
        shape = T.random_shape(rng, max_rank=5, max_extent=6)
        kind = rng.choice(T.VIEW_KINDS)
        cases += [(shape, kind, d) for d in reduced_shapes(rng, shape)]
    for shape, kind, dshape in cases:
        src = T.view_tensor(rng, dtype, shape, kind, int_span=20)
        _, ds = gpu.put(src)
        init = T.contiguous_tensor(rng, dtype, dshape, int_span=5)      # the ops accumulate INTO dst
        what = f"{NAMES[dtype]} {shape}->{dshape} {kind}"
        # maxTo: exact
        want = init.clone()
        okc(CPU.max_to(C.byref(src.desc()), C.byref(want.desc())))
        pi, di = gpu.put(init)
        G.run_gpu(gpu, "aixk_reduce_to", K.MAX, G.ref(ds), G.ref(di))
        T.assert_same_bits_nan_ok(gpu.fetch(pi, want.storage), want.storage, dtype, "maxTo " + what)
        # reduceTo
        pi, di = gpu.put(init)
        G.run_gpu(gpu, "aixk_reduce_to", K.SUM, G.ref(ds), G.ref(di))
        got = gpu.fetch(pi, init.storage)
        if dtype in T.INT_DTYPES:
            want = init.clone()
            okc(CPU.reduce_to(C.byref(src.desc()), C.byref(want.desc())))
            T.assert_same_bits(got, want.storage, "reduceTo " + what)
        else:
            exact = init.values().reshape(-1).copy()
            scale = np.abs(exact)
            okc(CPU.reduce_to_wide(C.byref(src.desc()), C.byref(init.desc()), exact.ctypes.data, scale.ctypes.data))
            check_sum_like(got, dtype, exact, scale, "reduceTo " + what)
        gpu.release()


ARG_CASES = [  # (shape, kind, dim)
    ([512, 700], "contig", 0), ([3000, 256], "contig", 0), ([40, 8192], "contig", 0),
    ([300, 4096], "contig", 1), ([2000, 96], "contig", 1), ([500, 10], "contig", 1),
    ([6, 500, 64], "contig", 1), ([9, 40, 33], "contig", 2), ([9, 40, 33], "contig", 0),
    ([3, 2], "transposed", 1), ([64, 100], "transposed", 0),
    ([2, 40, 2048], "contig", 0), ([5, 4100], "contig", 0), ([3, 2, 1024], "contig", 1),    # a handful of rows, wide and narrow columns
    ([20000, 64], "contig", 1), ([1100, 3072], "contig", 0), ([2, 300, 64], "contig", 0), ([4, 2, 1028], "contig", 1), ([7, 36], "contig", 0),                                                               # very many short rows: several rows per wave
]


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_argmax_to_family(gpu, dtype):
    rng = np.random.default_rng(20000 + dtype)
    cases = list(ARG_CASES)
    for _ in range(12):
        shape = T.random_shape(rng, max_rank=4, max_extent=6)
        cases.append((shape, rng.choice(["contig", "contig", "transposed", "sliced", "offset"]), int(rng.integers(0, len(shape)))))
    for shape, kind, dim in cases:
        src = T.view_tensor(rng, dtype, shape, kind, int_span=2, lo=-1, hi=1)
        if dtype in T.FLOAT_DTYPES:                                  # force ties: quantise to 5 levels
            src.storage[:] = O.to_storage(np.round(O.to_float64(src.storage, dtype) * 2) / 2, dtype)
        _, ds = gpu.put(src)
        keep = [1 if d == dim else e for d, e in enumerate(shape)]
        for dshape in (keep, [e for d, e in enumerate(shape) if d != dim] or [1]):
            want = T.empty(O.I32, dshape, fill=-7)
            okc(CPU.argmax_to(C.byref(src.desc()), C.byref(want.desc()), dim))
            po, do = gpu.put(T.empty(O.I32, dshape, fill=-7))
            G.run_gpu(gpu, "aixk_argmax_to", 0, G.ref(ds), G.ref(do), dim)
            T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"argmaxTo {NAMES[dtype]} {shape} dim={dim} {kind} -> {dshape}")
        want = T.empty(O.I32, shape)
        okc(CPU.argmax_indices_to(C.byref(src.desc()), C.byref(want.desc()), dim))
        po, do = gpu.put(T.empty(O.I32, shape))
        G.run_gpu(gpu, "aixk_argmax_to", 1, G.ref(ds), G.ref(do), dim)
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"argmaxIndicesTo {NAMES[dtype]} {shape} dim={dim} {kind}")
        # the same with the zero-fill of the destination folded in: whatever dst held is overwritten
        po, do = gpu.put(T.empty(O.I32, shape, fill=7))
        G.run_gpu(gpu, "aixk_argmax_to", 2, G.ref(ds), G.ref(do), dim)
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"fill(0) + argmaxIndicesTo {NAMES[dtype]} {shape} dim={dim} {kind}")
        gpu.release()
    src = T.contiguous_tensor(rng, dtype, [4, 4])
    _, ds = gpu.put(src)
    _, bad = gpu.put(T.empty(O.F32, [4]))
    assert gpu.ctx.lib.aixk_argmax_to(gpu.ctx.handle, 0, G.ref(ds), G.ref(bad), 1) == 1
    gpu.release()


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16], ids=ids)
def test_argmax_down_wide_columns_split_into_row_chunks(gpu, dtype):
    """argmax along dim 0 of wide rows whose rows are split into chunks over workgroups, float types: the (value, row)
    records of a column's chunks are folded by a second stage.  What the fold must get right: the first of equal values
    across chunks, +0 and -0 as equals, columns of nothing but NaNs and minus infinities (row 0), a leading NaN (row 0),
    a NaN elsewhere (never wins), a value found in the last chunk only, a kept leading dim, the one-hot form -- and calls
    in a row on different data (the records live in scratch memory that the next call reuses)."""
    rng = np.random.default_rng(20500 + dtype)
    ninf, nan = -np.inf, np.nan
    for shape, dim in (([1100, 3072], 0), ([3, 700, 2048], 1), ([2000, 2048], 0), ([640, 4096], 0)):
        R, Cw = shape[dim], shape[-1]
        for rep in range(2):
            vals = np.round(rng.uniform(-1, 1, size=shape) * 2) / 2            # five levels: ties everywhere
            v2 = vals.reshape(-1, R, Cw)
            v2[:, :, 0] = nan                                                  # nothing but NaNs
            v2[:, :, 1] = ninf                                                 # nothing but minus infinities
            v2[:, :, 2] = ninf; v2[:, 0, 2] = nan                              # a leading NaN above minus infinities
            v2[:, :, 3] = 0.25; v2[:, 0, 3] = nan                              # a leading NaN wins
            v2[:, :, 4] = 0.25; v2[:, R // 2, 4] = nan                         # a NaN elsewhere never wins: row 0
            v2[:, :, 5] = -1.0; v2[:, R - 1, 5] = -0.0; v2[:, R - 3, 5] = 0.0  # +0 before -0: the first of the two
            v2[:, :, 6] = -1.0; v2[:, R - 3, 6] = -0.0; v2[:, R - 1, 6] = 0.0  # -0 before +0: the first of the two
            v2[:, :, 7] = ninf; v2[:, R - 1, 7] = -60000.0                    # found in the last chunk only
            v2[:, :, 8] = 0.5                                                  # all equal: row 0
            v2[:, :, 9] = ninf; v2[:, 5, 9] = np.inf; v2[:, 900 % R, 9] = np.inf
            src = T.HostTensor(O.to_storage(vals.reshape(-1), dtype), dtype, shape)
            _, ds = gpu.put(src)
            keep = [1 if d == dim else e for d, e in enumerate(shape)]
            want = T.empty(O.I32, keep, fill=-7)
            okc(CPU.argmax_to(C.byref(src.desc()), C.byref(want.desc()), dim))
            po, do = gpu.put(T.empty(O.I32, keep, fill=-7))
            G.run_gpu(gpu, "aixk_argmax_to", 0, G.ref(ds), G.ref(do), dim)
            got = gpu.fetch(po, want.storage)
            T.assert_same_bits(got, want.storage, f"argmaxTo {NAMES[dtype]} {shape} dim={dim} call {rep}")
            lead = got.reshape(-1, Cw)[:, :10]
            assert (lead[:, [0, 1, 2, 3, 4, 8]] == 0).all() and (lead[:, 5] == R - 3).all() and (lead[:, 6] == R - 3).all() and (lead[:, 7] == R - 1).all()
            assert (lead[:, 9] == min(5, 900 % R)).all()
            want = T.empty(O.I32, shape)
            okc(CPU.argmax_indices_to(C.byref(src.desc()), C.byref(want.desc()), dim))
            po, do = gpu.put(T.empty(O.I32, shape))
            G.run_gpu(gpu, "aixk_argmax_to", 1, G.ref(ds), G.ref(do), dim)
            T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"argmaxIndicesTo {NAMES[dtype]} {shape} dim={dim} call {rep}")
            gpu.release()


# ---- matmul ---------------------------------------------------------------------------------------
MM_SIZES = [(1, 1, 1), (2, 3, 4), (1, 64, 1), (1, 257, 33), (33, 1, 17), (64, 64, 64), (65, 63, 67), (128, 256, 64),
            (257, 129, 513), (100, 300, 50), (512, 512, 512), (31, 1024, 9)]   # incl. DeviceTests.cpp:2806-2875 style edges


def check_matmul(gpu, a, b, what):
    dtype = a.dtype
    m, k, n = a.shape[0], a.shape[1], b.shape[1]
    _, da = gpu.put(a)
    _, db = gpu.put(b)
    po, do = gpu.put(T.empty(dtype, [m, n]))
    G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(do))
    got = gpu.fetch(po, np.zeros(m * n, O.NP_STORAGE[dtype]))
    if dtype in T.INT_DTYPES:
        want = T.empty(dtype, [m, n])
        okc(CPU.matmul_rows(C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc()), 8))
        return T.assert_same_bits(got, want.storage, what)
    exact = np.zeros(m * n)
    scale = np.zeros(m * n)
    okc(CPU.matmul_wide(C.byref(a.desc()), C.byref(b.desc()), exact.ctypes.data, scale.ctypes.data, 8))
    tol = {O.F64: 1e-12, O.F32: 1e-5, O.F16: 2e-2, O.BF16: 2e-2}[dtype]
    G.assert_close_to_wide(O.to_float64(got, dtype), exact, scale + 1e-30, tol, what)
    # and much tighter in practice for the 16-bit types: f32 accumulation + one final rounding
    if dtype in (O.F16, O.BF16):
        final = 2.0 ** -10 if dtype == O.F16 else 2.0 ** -8
        G.assert_close_to_wide(O.to_float64(got, dtype), exact, 1e-5 * scale + final * np.abs(exact) + 1e-30, 1.0, what + " (tight)")


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_matmul(gpu, dtype):
    rng = np.random.default_rng(21000 + dtype)
    for (m, k, n) in MM_SIZES:
        kinds = [("contig", "contig")]
        if (m, k, n) in ((65, 63, 67), (128, 256, 64), (100, 300, 50), (257, 129, 513)):
            kinds += [("transposed", "contig"), ("contig", "transposed"), ("transposed", "transposed"), ("offset", "sliced")]
        for ka, kb in kinds:
            scale = 1.0 / np.sqrt(k)
            a = T.view_tensor(rng, dtype, [m, k], ka, lo=-scale, hi=scale, int_span=9)
            b = T.view_tensor(rng, dtype, [k, n], kb, lo=-1, hi=1, int_span=9)
            check_matmul(gpu, a, b, f"matmul {NAMES[dtype]} {m}x{k}x{n} {ka}/{kb}")
        gpu.release()


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16], ids=ids)
def test_matmul_mfma_tiles(gpu, dtype):
    """Shapes that run on the matrix cores: ragged M and N against both workgroup tile sizes, every
    operand layout (row-major, transposed view, sliced, offset), K tails inside a K step."""
    rng = np.random.default_rng(23000 + dtype)
    cases = [((256, 256, 256), "contig", "contig"), ((300, 520, 264), "contig", "contig"), ((1000, 72, 130), "contig", "transposed"),
             ((129, 1048, 131), "transposed", "contig"), ((640, 136, 384), "transposed", "transposed"),
             ((200, 200, 200), "sliced", "offset"), ((96, 4096, 80), "contig", "contig"),
             ((2085, 512, 4101), "contig", "contig"), ((2048, 264, 4096), "contig", "transposed"),     # 256x256 tiles
             # whole 256x256 tiles and K steps of 64: the LDS-direct kernel (1, 2, 3 and 5 K steps; swizzled and plain tile numbering)
             ((2048, 64, 4096), "contig", "transposed"), ((2048, 128, 4096), "contig", "contig"),
             ((4096, 192, 2048), "transposed", "contig"), ((2304, 320, 3840), "contig", "transposed"),
             ((2048, 256, 4096), "transposed", "transposed"), ((4096, 128, 2048), "contig", "sliced")]
    for (m, k, n), ka, kb in cases:
        scale = 1.0 / np.sqrt(k)
        a = T.view_tensor(rng, dtype, [m, k], ka, lo=-scale, hi=scale)
        b = T.view_tensor(rng, dtype, [k, n], kb, lo=-1, hi=1)
        check_matmul(gpu, a, b, f"mfma matmul {NAMES[dtype]} {m}x{k}x{n} {ka}/{kb}")
        gpu.release()


@pytest.mark.parametrize("dtype", [O.F16, O.BF16], ids=ids)
def test_matmul_mid_tiles(gpu, dtype):
    """16-bit products of whole 128 x {128, 192, 256} x 64 tiles, at least half a tile per compute unit: the LDS-direct
    kernel on its smaller tiles.  The widths pick the tile (960 = 5 x 192 and no multiple of 128; 640 = 5 x 128 and no
    multiple of 192 or 256; 2048 under 31 tile rows: 248 tiles of 128 x 256 fill the chip in one round, 496 of 128 x 128
    would take two), every operand layout is consumed where it lies, with 1, 2, 3 and 5 K steps, sliced operands (row
    pitch above the extent), and the shapes of a d = 768 transformer's projections."""
    rng = np.random.default_rng(23700 + dtype)
    layouts = [("contig", "contig"), ("contig", "transposed"), ("transposed", "contig"), ("transposed", "transposed")]
    cases = []
    for n in (960, 640):
        for k, (ka, kb) in zip((64, 128, 192, 320), layouts):
            cases.append(((4096, k, n), ka, kb))
        for k, (ka, kb) in zip((320, 64, 128, 192), layouts):
            cases.append(((4096, k, n), ka, kb))
    for k, (ka, kb) in zip((128, 192, 64, 320), layouts):
        cases.append(((3968, k, 2048), ka, kb))
    cases += [((4096, 128, 960), "sliced", "sliced"), ((4096, 192, 640), "sliced", "transposed"),
              ((8192, 768, 768), "contig", "contig"), ((8192, 768, 768), "contig", "transposed"), ((8192, 768, 768), "transposed", "contig"),
              ((8192, 3072, 768), "contig", "contig"), ((8192, 768, 2304), "contig", "transposed")]
    for (m, k, n), ka, kb in cases:
        scale = 1.0 / np.sqrt(k)
        a = T.view_tensor(rng, dtype, [m, k], ka, lo=-scale, hi=scale)
        b = T.view_tensor(rng, dtype, [k, n], kb, lo=-1, hi=1)
        check_matmul(gpu, a, b, f"mid-tile matmul {NAMES[dtype]} {m}x{k}x{n} {ka}/{kb}")
        gpu.release()


@pytest.mark.parametrize("dtype", [O.F16, O.BF16], ids=ids)
def test_matmul_random_whole_tile_shapes(gpu, dtype):
    """Random 16-bit products whose extents are multiples of the tile sizes (M of 128, N of 64, K of 64) in random operand
    layouts: whichever kernel and tile the cost model picks -- 256 x 256, 128 x {128, 192, 256}, the register-staged
    tiles below half a tile per compute unit, K splits under a long K -- the result must stay within the 16-bit matmul
    bar of the exactly accumulated product.  Tile counts that are and are not multiples of 8 (the XCD-aware numbering is
    a bijection only for the former), odd numbers of tile rows, one to twelve K steps."""
    rng = np.random.default_rng(23900 + dtype)
    for trial in range(14):
        m = 128 * int(rng.integers(1, 41))
        n = 64 * int(rng.integers(1, 41))
        k = 64 * int(rng.integers(1, 13)) if trial % 5 else 64 * int(rng.integers(64, 80))
        if trial == 0:
            m, n, k = 128 * 37, 192 * 7, 64 * 3                 # 259 tiles of 128 x 192: plain numbering, a ragged last group of tile rows
        ka, kb = (str(rng.choice(["contig", "transposed"])) for _ in range(2))
        scale = 1.0 / np.sqrt(k)
        a = T.view_tensor(rng, dtype, [m, k], ka, lo=-scale, hi=scale)
        b = T.view_tensor(rng, dtype, [k, n], kb, lo=-1, hi=1)
        check_matmul(gpu, a, b, f"random whole-tile matmul {NAMES[dtype]} {m}x{k}x{n} {ka}/{kb}")
        gpu.release()


@pytest.mark.parametrize("dtype", [O.F16, O.BF16], ids=ids)
def test_matmul_small_tiles(gpu, dtype):
    """16-bit outputs too small for 64 x 64 tiles to fill the chip (attention heads and the like): the
    32 x 32-tile kernel that splits K over its four waves, every operand layout consumed in place --
    one to nine K steps, ragged tiles, K tails, extents that are no multiple of 8 (those are gathered)."""
    rng = np.random.default_rng(23500 + dtype)
    layouts = [("contig", "contig"), ("contig", "transposed"), ("transposed", "contig"), ("transposed", "transposed")]
    for (m, k, n) in [(512, 64, 512), (512, 512, 64), (64, 512, 512), (96, 40, 72), (72, 200, 88), (64, 8, 64), (104, 576, 40), (99, 64, 101)]:
        for ka, kb in layouts + [("sliced", "offset")]:
            scale = 1.0 / np.sqrt(k)
            a = T.view_tensor(rng, dtype, [m, k], ka, lo=-scale, hi=scale)
            b = T.view_tensor(rng, dtype, [k, n], kb, lo=-1, hi=1)
            check_matmul(gpu, a, b, f"small matmul {NAMES[dtype]} {m}x{k}x{n} {ka}/{kb}")
        gpu.release()


def _route(gpu):
    """(took the split-plane f32 route, was redone in IEEE arithmetic) for the last aixk_matmul."""
    route, redone = C.c_int32(-1), C.c_int32(-1)
    G.run_gpu(gpu, "aixk_matmul_route", C.byref(route), C.byref(redone))
    return route.value, redone.value


@pytest.mark.parametrize("mkn", [(4096, 256, 2048), (4096, 264, 4096)], ids=["planes_in_registers", "planes_in_memory"])
def test_matmul_f32_large_tiles_small_magnitudes(gpu, mkn):
    """Large f32 products run on the bf16 matrix pipe with every operand split into three bf16 planes -- tile by tile in
    registers (gemm_x3_k), or, from one whole 256 x 256 tile per compute unit on, once into memory (split_planes_k, here
    with a K that is padded to the next multiple of 64) for the LDS-direct 16-bit kernel to multiply six plane pairs deep.  The planes carry
    f32's 24 bits only down to 2^-110 (bf16's grid ends at 2^-133), so operands below that -- here in matrices WITHOUT
    any infinity or NaN, which would send the product to the IEEE kernel for their own reasons -- must be noticed and the
    product redone in IEEE f32 arithmetic, as the CPU device computes it (aixDeviceCPU.cpp:362-389: plain f32, no range
    limits).  Small values the planes do carry, and products and sums that land in f32's subnormals, stay on the split-plane
    kernel (the matrix unit keeps subnormals).  Bar: 1e-5 of the sum of |a||b| against exactly accumulated products
    (cpuref_matmul_wide), plus K quanta of 2^-149 where results are subnormal (each f32 product rounds by up to half a
    quantum there on the CPU too)."""
    rng = np.random.default_rng(25600)
    m, k, n = mkn                                               # 512 tiles of 128 x 128 / 256 tiles of 256 x 256: the split-plane routes
    in_memory = n == 4096
    U = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    P = rng.uniform(0.1, 1.0, (k, n)).astype(np.float32)
    V = (rng.uniform(0.25, 1.0, (m, k)) * rng.choice([-1.0, 1.0], (m, k))).astype(np.float32)     # magnitudes within two binades
    one_tiny_row = (U / np.sqrt(k)).astype(np.float32)
    one_tiny_row[2000, :] = (U[2000] * np.float32(1e-37)).astype(np.float32)
    one_tiny_entry = (U / np.sqrt(k)).astype(np.float32)
    one_tiny_entry[123, 45] = np.float32(3e-39)
    with np.errstate(under="ignore"):
        cases = [                                               # (name, A, B, redone in IEEE arithmetic?)
            ("ordinary", (U / np.sqrt(k)).astype(np.float32), P, 0),
            ("A at 1e-20 (planes exact)", (V * np.float32(1e-20)).astype(np.float32), P, 0),
            ("A at 1e-29 (planes exact)", (V * np.float32(1e-29)).astype(np.float32), P, 0),
            ("A at 1e-33", (U * np.float32(1e-33)).astype(np.float32), P, 1),
            ("A at 1e-36", (U * np.float32(1e-36)).astype(np.float32), P, 1),
            ("A at 3e-38", (U * np.float32(3e-38)).astype(np.float32), P, 1),
            ("A at 1e-41 (subnormal)", (U * np.float32(1e-41)).astype(np.float32), P, 1),
            ("one row at 1e-37 in an ordinary A", one_tiny_row, P, 1),
            ("one subnormal entry in an ordinary A", one_tiny_entry, P, 1),
            ("A at 1e-36 times B at 1e30", (U * np.float32(1e-36)).astype(np.float32), (P * np.float32(1e30)).astype(np.float32), 1),
            ("ordinary A times B at 1e-36", (U / np.sqrt(k)).astype(np.float32), (P * np.float32(1e-36)).astype(np.float32), 1),
            ("subnormal products: A at 1e-20, B at 1e-22", (V * np.float32(1e-20)).astype(np.float32), (P * np.float32(1e-22)).astype(np.float32), 0),
            ("products below the subnormals: A at 1e-25, B at 1e-25", (V * np.float32(1e-25)).astype(np.float32), (P * np.float32(1e-25)).astype(np.float32), 0),
        ]
    floor = k * 2.0 ** -149
    for name, A, B, want_redone in cases:
        if in_memory and name.startswith(("A at 1e-20", "A at 1e-33", "A at 3e", "A at 1e-41", "A at 1e-36 times", "products below")):
            continue                                            # (the scales are the first shape's business; here: who notices, in every layout)
        for layout in ("NN", "TN", "NT", "TT"):
            if layout == "TN" and name.startswith(("A at 1e-2", "A at 3e", "products below")):
                continue                                        # (one layout is enough for the variations of one scale)
            if layout in ("NT", "TT") and not (in_memory and name in ("ordinary", "one subnormal entry in an ordinary A", "ordinary A times B at 1e-36")):
                continue                                        # (a transposed B matters to the pass that writes the planes to memory)
            a = T.HostTensor(A if layout[0] == "N" else np.ascontiguousarray(A.T), O.F32, [m, k], None if layout[0] == "N" else [1, m])
            b = T.HostTensor(B if layout[1] == "N" else np.ascontiguousarray(B.T), O.F32, [k, n], None if layout[1] == "N" else [1, k])
            _, da = gpu.put(a)
            _, db = gpu.put(b)
            po, do = gpu.put(T.empty(O.F32, [m, n]))
            G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(do))
            route, redone = _route(gpu)
            got = gpu.fetch(po, np.zeros(m * n, np.float32))
            gpu.release()
            assert (route, redone) == (1, want_redone), (name, layout, route, redone)
            exact, scale = np.zeros(m * n), np.zeros(m * n)
            okc(CPU.matmul_wide(C.byref(a.desc()), C.byref(b.desc()), exact.ctypes.data, scale.ctypes.data, 8))
            err = np.abs(got.astype(np.float64) - exact)
            bad = np.flatnonzero(~(err <= 1e-5 * scale + floor))
            assert bad.size == 0, (name, layout, bad.size, int(bad[0]), float(got[bad[0]]), float(exact[bad[0]]), float(scale[bad[0]]))
            if not want_redone and scale.min() > 2.0 ** -100:    # far inside the bar in practice: three planes carry all 24 bits
                assert np.all(err <= 4e-7 * scale), (name, layout, float((err / scale).max()))


@pytest.mark.parametrize("mkn", [(4096, 256, 2048), (4096, 264, 4096)], ids=["planes_in_registers", "planes_in_memory"])
def test_matmul_f32_large_tiles_special_values(gpu, mkn):
    """Large f32 products run on the bf16 matrix pipe with every operand split into three bf16 planes (in registers tile by
    tile, or once into memory: the two shapes).
    Rows with an infinity, a NaN, both infinities, or a value next to FLT_MAX must come out as IEEE arithmetic has
    them (inf, NaN, NaN, finite); their neighbours in the same 16-byte chunk and everything else stay within the
    f32 matmul bar.  (Non-finite operands send the whole product to the IEEE kernel; small magnitudes are the test above.)"""
    rng = np.random.default_rng(25500)
    m, k, n = mkn
    A = (rng.uniform(-1, 1, (m, k)) / np.sqrt(k)).astype(np.float32)
    B = rng.uniform(0.1, 1.0, (k, n)).astype(np.float32)
    A[7, 5] = np.inf
    A[130, 9] = np.nan
    A[131, 250] = -np.inf
    A[300, 3], A[300, 77] = np.inf, -np.inf
    A[1000, :] = 0.0
    A[1000, 17] = np.float32(3.3e38)                  # times at most 1: finite in f32, would be inf if rounded up to bf16 first
    for layout in ("NN", "TN"):
        a = T.HostTensor(A if layout == "NN" else np.ascontiguousarray(A.T), O.F32, [m, k], None if layout == "NN" else [1, m])
        b = T.HostTensor(B, O.F32, [k, n])
        _, da = gpu.put(a)
        _, db = gpu.put(b)
        po, do = gpu.put(T.empty(O.F32, [m, n]))
        G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(do))
        assert _route(gpu) == (1, 1), layout
        got = gpu.fetch(po, np.zeros(m * n, np.float32)).reshape(m, n)
        assert np.all(got[7] == np.inf), layout
        assert np.all(np.isnan(got[130])) and np.all(np.isnan(got[300])), layout
        assert np.all(got[131] == -np.inf), layout
        with np.errstate(invalid="ignore", over="ignore"):
            exact = A.astype(np.float64) @ B.astype(np.float64)
            scale = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
        ordinary = np.ones(m, bool)
        ordinary[[7, 130, 131, 300]] = False
        assert np.all(np.isfinite(got[ordinary])), layout
        err = np.abs(got[ordinary] - exact[ordinary])
        assert np.all(err <= 1e-5 * scale[ordinary] + 1e-44), (layout, float((err / (scale[ordinary] + 1e-300)).max()))
        # and far inside the bar in practice: three planes carry all 24 bits
        assert np.all(err[:6] <= 4e-7 * scale[ordinary][:6]), layout
        gpu.release()


def test_matmul_identity_and_ones(gpu):
    """Mathematical pins: A.I == A exactly; ones[m,k].ones[k,n] == k exactly (f32, f16, bf16)."""
    rng = np.random.default_rng(22000)
    for dtype in (O.F32, O.F16, O.BF16):
        a = T.contiguous_tensor(rng, dtype, [96, 160])
        eye = T.HostTensor(O.to_storage(np.eye(160).reshape(-1), dtype), dtype, [160, 160])
        _, da = gpu.put(a)
        _, de = gpu.put(eye)
        po, do = gpu.put(T.empty(dtype, [96, 160]))
        G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(de), G.ref(do))
        T.assert_same_bits(gpu.fetch(po, a.storage), a.storage, f"A.I {NAMES[dtype]}")
        ones_a = T.HostTensor(O.to_storage(np.ones(70 * 200), dtype), dtype, [70, 200])
        ones_b = T.HostTensor(O.to_storage(np.ones(200 * 90), dtype), dtype, [200, 90])
        _, d1 = gpu.put(ones_a)
        _, d2 = gpu.put(ones_b)
        po, do = gpu.put(T.empty(dtype, [70, 90]))
        G.run_gpu(gpu, "aixk_matmul", G.ref(d1), G.ref(d2), G.ref(do))
        got = O.to_float64(gpu.fetch(po, np.zeros(70 * 90, O.NP_STORAGE[dtype])), dtype)
        assert np.all(got == 200.0), f"ones.ones {NAMES[dtype]}"
        gpu.release()


@pytest.mark.parametrize("dtype", [O.BF16, O.F16, O.I16, O.F32], ids=ids)
def test_index_add_with_many_duplicates(gpu, dtype):
    """Embedding-gradient shapes: hundreds of updates landing on a few dozen rows (16-bit types update two
    neighbouring elements per compare-and-swap).  Whole-number updates keep every partial sum exact, so the
    order in which duplicates arrive cannot matter and the result equals the CPU's bit for bit."""
    rng = np.random.default_rng(27000 + dtype)
    for shape, dim, ni in (([50, 64], 0, 700), ([4, 9, 6], 1, 40), ([3, 5, 8], 2, 64), ([7, 10], 0, 33)):
        sel = list(shape)
        sel[dim] = ni
        idx = T.HostTensor(rng.integers(0, shape[dim], ni).astype(np.int32), O.I32, [ni])
        upd = T.HostTensor(O.to_storage(rng.integers(-2, 3, O.numel(sel)).astype(np.float64), dtype), dtype, sel)
        acc = T.HostTensor(O.to_storage(rng.integers(-4, 5, O.numel(shape)).astype(np.float64), dtype), dtype, shape)
        want = acc.clone()
        okc(CPU.index_add(C.byref(upd.desc()), C.byref(want.desc()), C.byref(idx.desc()), dim, 1))
        _, didx = gpu.put(idx)
        _, dupd = gpu.put(upd)
        pa, dacc = gpu.put(acc)
        G.run_gpu(gpu, "aixk_index_add", G.ref(dupd), G.ref(dacc), G.ref(didx), dim)
        T.assert_same_bits(gpu.fetch(pa, want.storage), want.storage, f"indexAdd {NAMES[dtype]} {shape} dim={dim} x{ni}")
        gpu.release()


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=ids)
def test_tri_on_dense_stacks(gpu, dtype):
    """tril / triu of dense tensors whose rows are whole 16-byte vectors (a stack of attention score matrices):
    the vector kernel, every diagonal from all-zero to all-kept, vectors that straddle the edge."""
    rng = np.random.default_rng(26000 + dtype)
    for shape in ([2, 3, 24, 32], [40, 48], [5, 16, 64]):
        src = T.contiguous_tensor(rng, dtype, shape, int_span=50)
        _, dsrc = gpu.put(src)
        for upper in (0, 1):
            for diag in (-shape[-2] - 1, -7, -1, 0, 1, 5, 13, shape[-1] + 1):
                want = T.empty(dtype, shape, fill=3)
                okc((CPU.triu if upper else CPU.tril)(C.byref(src.desc()), C.byref(want.desc()), diag))
                pd, dd = gpu.put(T.empty(dtype, shape, fill=3))
                G.run_gpu(gpu, "aixk_tri", upper, G.ref(dsrc), G.ref(dd), diag)
                T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, f"tri upper={upper} {NAMES[dtype]} {shape} diag={diag}")
        gpu.release()


# ---- stacks of products (beyond the reference: its matmul is 2-D only) -----------------------------
def _matrix_of(ht, index):
    """The 2-D view of matrix `index` (a tuple over the leading dims) of a stacked HostTensor."""
    nb = len(ht.shape) - 2
    off = ht.offset + sum(i * s for i, s in zip(index, ht.strides[:nb]))
    return T.HostTensor(ht.storage, ht.dtype, ht.shape[nb:], ht.strides[nb:], off)


def check_matmul_stack(gpu, a, b, what, against_each=True):
    """aixk_matmul_batched against (1) the oracle's stack -- integers bit for bit, floats within the matmul bar of
    the exactly accumulated products -- and (2) aixk_matmul issued matrix by matrix on the same views: bit for bit
    where the stack is issued product by product (f32, integers); the one-launch 16-bit route may add the f32
    partial sums in another order than the 2-D route picks for a single small product, so there the two agree to
    f32 accumulation error plus the final rounding."""
    dtype = a.dtype
    lead, m, k, n = a.shape[:-2], a.shape[-2], a.shape[-1], b.shape[-1]
    count = int(np.prod(lead))
    pa, da = gpu.put(a)
    pb, db = gpu.put(b)
    po, do = gpu.put(T.empty(dtype, lead + [m, n]))
    G.run_gpu(gpu, "aixk_matmul_batched", G.ref(da), G.ref(db), G.ref(do))
    got = gpu.fetch(po, np.zeros(count * m * n, O.NP_STORAGE[dtype]))
    if dtype in T.INT_DTYPES:
        want = T.empty(dtype, lead + [m, n])
        okc(CPU.matmul_stack(C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc()), 8))
        T.assert_same_bits(got, want.storage, what)
    tol = {O.F64: 1e-12, O.F32: 1e-5, O.F16: 2e-2, O.BF16: 2e-2}.get(dtype)
    p1, d1 = gpu.put(T.empty(dtype, [m, n]))
    for flat, index in enumerate(np.ndindex(*lead)):
        a2, b2 = _matrix_of(a, index), _matrix_of(b, index)
        mine = got[flat * m * n:(flat + 1) * m * n]
        if dtype not in T.INT_DTYPES:
            exact = np.zeros(m * n)
            scale = np.zeros(m * n)
            okc(CPU.matmul_wide(C.byref(a2.desc()), C.byref(b2.desc()), exact.ctypes.data, scale.ctypes.data, 8))
            G.assert_close_to_wide(O.to_float64(mine, dtype), exact, scale + 1e-30, tol, f"{what} matrix {index}")
        if against_each:
            G.run_gpu(gpu, "aixk_matmul", G.ref(G.kdesc(a2, pa)), G.ref(G.kdesc(b2, pb)), G.ref(d1))
            single = gpu.fetch(p1, mine)
            if dtype in (O.F16, O.BF16):
                final = 2.0 ** -10 if dtype == O.F16 else 2.0 ** -8
                # two roundings of two f32 sums that differ in the order of their terms: each within half an ulp of its own sum
                G.assert_close_to_wide(O.to_float64(mine, dtype), O.to_float64(single, dtype), 2e-5 * scale + 2 * final * np.abs(exact) + 1e-30, 1.0,
                                       f"{what} matrix {index} against the 2-D entry point")
            else:
                T.assert_same_bits(mine, single, f"{what} matrix {index} against the 2-D entry point")


@pytest.mark.parametrize("dtype", [O.BF16, O.F16, O.F32, O.I32], ids=ids)
def test_matmul_stacks(gpu, dtype):
    """Attention-shaped stacks through every view the front-end builds: q, k, v stored [batch, seq, heads, d]
    and seen as [batch, heads, seq, d] (permuted leading dims), k transposed on its last two dims, a
    transposed first operand (the gradient products), a second operand shared by the whole stack (stride 0),
    sliced stacks with an offset, ragged extents.  The 16-bit cases run as one launch, f32 and integers as
    one launch per matrix."""
    rng = np.random.default_rng(24000 + dtype)
    B, H, S, D = 2, 3, 96, 64
    def draw(count, lo, hi):
        return O.to_storage(rng.integers(-9, 9, count) if dtype in T.INT_DTYPES else rng.uniform(lo, hi, count), dtype)
    q = draw(B * S * H * D, -0.2, 0.2)
    kk = draw(B * S * H * D, -1, 1)
    heads = [S * H * D, D, H * D, 1]                       # [batch, heads, seq, d] over [batch, seq, heads, d] storage
    heads_t = [S * H * D, D, 1, H * D]                     # ... with the last two dims transposed: [batch, heads, d, seq]
    q4 = T.HostTensor(q, dtype, [B, H, S, D], heads)
    kT = T.HostTensor(kk, dtype, [B, H, D, S], heads_t)
    check_matmul_stack(gpu, q4, kT, f"scores {NAMES[dtype]}")                                  # [S, D] . [D, S]
    p = T.HostTensor(draw(B * H * S * S, -0.1, 0.1), dtype, [B, H, S, S])
    v4 = T.HostTensor(kk, dtype, [B, H, S, D], heads)
    check_matmul_stack(gpu, p, v4, f"p.v {NAMES[dtype]}")                                      # [S, S] . [S, D]
    pT = T.HostTensor(p.storage, dtype, [B, H, S, S], [H * S * S, S * S, 1, S])
    check_matmul_stack(gpu, pT, v4, f"pT.v {NAMES[dtype]}")                                    # transposed first operand
    check_matmul_stack(gpu, p, T.HostTensor(kk, dtype, [B, H, S, D], [0, 0, H * D, 1]), f"shared second operand {NAMES[dtype]}")
    gpu.release()
    # a slice of a stack (offset, fewer matrices than stored), ragged extents, rank 3
    wide = T.HostTensor(draw(5 * 72 * 104, -0.2, 0.2), dtype, [3, 72, 88], [72 * 104, 104, 1], offset=72 * 104 + 8)
    other = T.HostTensor(draw(4 * 88 * 80, -1, 1), dtype, [3, 88, 80], None, offset=88 * 80)
    check_matmul_stack(gpu, wide, other, f"sliced stack {NAMES[dtype]}")
    # whole 128 x {128, 192} tiles, eight K steps and half a tile per compute unit over the stack: the LDS-direct kernel's
    # smaller tiles with blockIdx.y numbering the matrices -- plain, with permuted leading dims, a transposed first operand
    if dtype in (O.F16, O.BF16):
        big_a = T.HostTensor(draw(2 * 4 * 512 * 512, -0.05, 0.05), dtype, [2, 4, 512, 512], [512 * 512, 2 * 512 * 512, 512, 1])
        big_b = T.HostTensor(draw(2 * 4 * 512 * 768, -1, 1), dtype, [2, 4, 512, 768])
        check_matmul_stack(gpu, big_a, big_b, f"stack of whole 128 x 192 tiles {NAMES[dtype]}")
        big_at = T.HostTensor(big_a.storage, dtype, [8, 512, 512], [512 * 512, 1, 512])
        big_c = T.HostTensor(draw(8 * 512 * 640, -1, 1), dtype, [8, 512, 640])
        check_matmul_stack(gpu, big_at, big_c, f"stack of whole 128 x 128 tiles, transposed first operand {NAMES[dtype]}")
        gpu.release()
        # K = 64 with both operands K-contiguous and two whole 128 x 128 tiles per compute unit over the stack: the kernel
        # without LDS (attention's scores at their real shape: heads as a permuted view, k transposed) -- 32 matrices
        # numbered XCD by XCD, 44 in plain order, unequal tile counts per side
        for (b2, h2, s2, t2) in ((4, 8, 512, 512), (11, 4, 512, 512), (8, 8, 256, 640)):
            qs = draw(b2 * s2 * h2 * 64, -0.5, 0.5)
            ks = draw(b2 * t2 * h2 * 64, -1, 1)
            qv = T.HostTensor(qs, dtype, [b2, h2, s2, 64], [s2 * h2 * 64, 64, h2 * 64, 1])
            kv = T.HostTensor(ks, dtype, [b2, h2, 64, t2], [t2 * h2 * 64, 64, 1, h2 * 64])
            check_matmul_stack(gpu, qv, kv, f"{b2 * h2} score products [{s2}, 64] x [64, {t2}] {NAMES[dtype]}")
            gpu.release()
    # matrices too small or too odd for the matrix-core route
    check_matmul_stack(gpu, T.HostTensor(draw(7 * 5 * 3, -1, 1), dtype, [7, 5, 3]), T.HostTensor(draw(7 * 3 * 4, -1, 1), dtype, [7, 3, 4]),
                       f"tiny stack {NAMES[dtype]}")
    gpu.release()


@pytest.mark.parametrize("dtype", [O.BF16, O.F16], ids=ids)
@pytest.mark.parametrize("case", [(96, 512, 512), (100, 256, 2048), (192, 512, 512), (96, 1024, 1024)], ids=str)
def test_matmul_k64_stacks_at_every_sweep_length(gpu, dtype, case):
    """Stacks of K = 64 products with K-contiguous operands, large enough that a wave of the kernel without LDS sweeps two,
    four and eight blocks of 64 columns (on 256 compute units: the cases in this order 2, 4, 4, 8), the matrices numbered
    XCD by XCD (counts that are multiples of 8) and in plain order (100).  Small integers: every sum is exact in f32, so
    the result is the one rounding of the exact product and the check is bit equality with numpy."""
    count, m, n = case
    rng = np.random.default_rng(25500 + count + m + dtype)
    av = rng.integers(-3, 4, (count, m, 64)).astype(np.float32)
    bv = rng.integers(-3, 4, (count, n, 64)).astype(np.float32)                # stored [n, k]: the transposed second operand
    a = T.HostTensor(O.to_storage(av.reshape(-1), dtype), dtype, [count, m, 64])
    b = T.HostTensor(O.to_storage(bv.reshape(-1), dtype), dtype, [count, 64, n], [n * 64, 1, 64])
    pa, da = gpu.put(a)
    pb, db = gpu.put(b)
    po, do = gpu.put(T.empty(dtype, [count, m, n], fill=1))
    G.run_gpu(gpu, "aixk_matmul_batched", G.ref(da), G.ref(db), G.ref(do))
    got = gpu.fetch(po, np.zeros(count * m * n, O.NP_STORAGE[dtype]))
    want = np.matmul(av, bv.transpose(0, 2, 1))                                # |sums| <= 576: exact in f32, rounded once to the 16-bit type below
    T.assert_same_bits(got, O.to_storage(want.reshape(-1).astype(np.float64), dtype), f"{count} products [{m}, 64] x [64, {n}] {NAMES[dtype]}")
    gpu.release()


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.I32], ids=ids)
def test_matmul_stacks_random_views(gpu, dtype):
    """Stacks with one to three leading dims in a random storage order (so the leading dims of a and b collapse
    differently, or not at all), an operand shared along a random leading dim (stride 0), extents that are and are not
    multiples of the 16-byte chunk, matrices stored transposed: against the oracle's stack and the 2-D entry point."""
    rng = np.random.default_rng(24800 + dtype)
    for trial in range(10):
        nlead = int(rng.integers(1, 4))
        lead = [int(v) for v in rng.integers(1, 4, nlead)]
        m, k, n = (int(v) for v in rng.choice([8, 24, 40, 64, 72, 96, 100], 3))
        if trial % 3 == 0:
            m, n = 64, 64                                            # large enough for the one-launch route (16-bit types)
            k = int(rng.choice([16, 64, 136]))

        def operand(rows, cols):
            """Random storage order of the leading dims, matrix stored plain or transposed, maybe shared along one dim."""
            order = list(rng.permutation(nlead))
            shared = int(rng.integers(0, nlead)) if rng.random() < 0.3 else -1
            transposed = rng.random() < 0.5
            strides = [0] * nlead
            run = rows * cols
            for d in reversed(order):
                if d == shared:
                    continue
                strides[d] = run
                run *= lead[d]
            offset = int(rng.integers(0, 3)) * 8
            values = rng.integers(-9, 9, run + offset) if dtype in T.INT_DTYPES else rng.uniform(-1, 1, run + offset) / np.sqrt(k)
            mat = [1, rows] if transposed else [cols, 1]
            return T.HostTensor(O.to_storage(values, dtype), dtype, lead + [rows, cols], strides + mat, offset)

        a, b = operand(m, k), operand(k, n)
        check_matmul_stack(gpu, a, b, f"random stack {NAMES[dtype]} lead={lead} {m}x{k}x{n} a.strides={a.strides} b.strides={b.strides}")
        gpu.release()


def test_matmul_stack_edges(gpu):
    """Rank 2 is the 2-D entry point; empty stacks and K = 0; more matrices than one launch numbers (stride-0
    stacks of one product: every result matrix equals the single product); mismatched operands are refused."""
    rng = np.random.default_rng(24500)
    dtype = O.BF16
    a = T.HostTensor(O.to_storage(rng.uniform(-0.3, 0.3, 64 * 16), dtype), dtype, [64, 16])
    b = T.HostTensor(O.to_storage(rng.uniform(-1, 1, 16 * 64), dtype), dtype, [16, 64])
    pa, da = gpu.put(a)
    pb, db = gpu.put(b)
    p1, d1 = gpu.put(T.empty(dtype, [64, 64]))
    G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(d1))
    one = gpu.fetch(p1, np.zeros(64 * 64, np.uint16))
    p2, d2 = gpu.put(T.empty(dtype, [64, 64], fill=7))
    G.run_gpu(gpu, "aixk_matmul_batched", G.ref(da), G.ref(db), G.ref(d2))
    T.assert_same_bits(gpu.fetch(p2, one), one, "rank 2 through the stacked entry point")
    for count in (3, 65535, 65536 + 5):
        sa = T.HostTensor(a.storage, dtype, [count, 64, 16], [0, 16, 1])
        sb = T.HostTensor(b.storage, dtype, [count, 16, 64], [0, 64, 1])
        po, do = gpu.put(T.empty(dtype, [count, 64, 64], fill=7))
        G.run_gpu(gpu, "aixk_matmul_batched", G.ref(G.kdesc(sa, pa)), G.ref(G.kdesc(sb, pb)), G.ref(do))
        got = gpu.fetch(po, np.zeros(count * 4096, np.uint16)).reshape(count, 4096)
        assert np.all(got == one[None, :]), f"{count} copies of one product"
        gpu.release()
        pa, da = gpu.put(a)
        pb, db = gpu.put(b)
    # empty stack: nothing written; K = 0: zeros
    po, do = gpu.put(T.empty(dtype, [2, 4, 4], fill=7))
    empty_a, empty_b, empty_o = G.kdesc(T.HostTensor(a.storage, dtype, [0, 4, 8]), pa), G.kdesc(T.HostTensor(b.storage, dtype, [0, 8, 4]), pb), G.kdesc(T.empty(dtype, [0, 4, 4]), po)
    G.run_gpu(gpu, "aixk_matmul_batched", G.ref(empty_a), G.ref(empty_b), G.ref(empty_o))
    assert np.all(gpu.fetch(po, np.zeros(32, np.uint16)) == 7)
    k0_a, k0_b = G.kdesc(T.HostTensor(a.storage, dtype, [2, 4, 0]), pa), G.kdesc(T.HostTensor(b.storage, dtype, [2, 0, 4]), pb)
    G.run_gpu(gpu, "aixk_matmul_batched", G.ref(k0_a), G.ref(k0_b), G.ref(do))
    assert np.all(gpu.fetch(po, np.zeros(32, np.uint16)) == 0)
    # refusals
    lib = gpu.ctx.lib
    three = G.kdesc(T.HostTensor(a.storage, dtype, [2, 8, 16]), pa)
    other_lead = G.kdesc(T.HostTensor(b.storage, dtype, [3, 16, 8]), pb)
    out3 = G.kdesc(T.empty(dtype, [2, 8, 8]), po)
    assert lib.aixk_matmul_batched(gpu.ctx.handle, G.ref(three), G.ref(other_lead), G.ref(out3)) != 0          # leading dims differ
    assert lib.aixk_matmul_batched(gpu.ctx.handle, G.ref(three), G.ref(db), G.ref(out3)) != 0                  # ranks differ
    bad_inner = G.kdesc(T.HostTensor(b.storage, dtype, [2, 8, 8]), pb)
    assert lib.aixk_matmul_batched(gpu.ctx.handle, G.ref(three), G.ref(bad_inner), G.ref(out3)) != 0           # inner dims differ
    gpu.release()


# ---- the reference's own literal vectors through the GPU kernels ----------------------------------
import goldens  # noqa: E402

_CASES = goldens.load_cases()


@pytest.mark.parametrize("case", _CASES, ids=[c["name"] for c in _CASES])
def test_reference_literals_on_gpu(gpu, case):
    goldens.run_case(case, G.KernelBackend(gpu))
