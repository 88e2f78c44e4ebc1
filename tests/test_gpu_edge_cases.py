"""Edge cases of the operand descriptor through the kernel C ABI: empty tensors, rank-0 tensors, the
maximum rank of 16, one dimension too many.

The reference's loops simply do not execute for an empty operand (every CPU kernel is a counted loop,
aixDeviceCPU.cpp:28-94) and its GPU device caps the rank at 16 (aixDeviceMetal.cpp:671-672); the
kernels here must return success without touching memory for the former and a clean error for the
latter.  Rank 16 itself must work, through the same index arithmetic as any other view."""
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


@pytest.fixture(scope="module")
def gpu():
    g = G.Gpu()
    yield g
    g.close()
    g.ctx.close()


def okc(rc):
    assert rc == 0, rc


def _sentinel(gpu, nbytes=4096):
    """A device buffer full of 0xA5 to hand to a kernel that must not write."""
    host = np.full(nbytes, 0xA5, np.uint8)
    p = gpu.raw(nbytes)
    gpu.ctx.upload(p, host)
    return p, host


def _desc(ptr, dtype, shape, strides=None, offset=0):
    d = K.Tensor()
    d.data = ptr
    d.dtype = dtype
    d.rank = len(shape)
    d.offset = offset
    d.size = int(np.prod(shape)) if len(shape) else 1
    st = O.row_major(list(shape)) if strides is None else strides
    for i, (e, s) in enumerate(zip(shape, st)):
        d.shape[i] = e
        d.strides[i] = s
    return d


@pytest.mark.parametrize("dtype", [O.F32, O.BF16, O.I64, O.U8], ids=lambda d: NAMES[d])
def test_empty_operands_do_nothing(gpu, dtype):
    p, host = _sentinel(gpu)
    q, _ = _sentinel(gpu)
    out, _ = _sentinel(gpu)
    for shape in ([0], [0, 7], [5, 0, 3]):
        a, b, r = _desc(p, dtype, shape), _desc(q, dtype, shape), _desc(out, dtype, shape)
        for op in (O.ADD, O.MUL, O.DIV, O.POW):
            G.run_gpu(gpu, "aixk_binary", op, G.ref(a), G.ref(b), G.ref(r))
        for op in (O.NEG, O.SQRT, O.EXP):
            G.run_gpu(gpu, "aixk_unary", op, G.ref(a), G.ref(r))
        one = np.ones(1, np.float32)
        G.run_gpu(gpu, "aixk_fill", one.ctypes.data, O.F32, G.ref(r))
        G.run_gpu(gpu, "aixk_fill_min", G.ref(r))
        G.run_gpu(gpu, "aixk_contiguous", G.ref(a), G.ref(r))
        G.run_gpu(gpu, "aixk_cast", p, dtype, out, O.F32, 0)
        # reducing nothing into something leaves the destination as it is (reduceTo adds, maxTo keeps the larger)
        keep = _desc(out, dtype, [1] * len(shape))
        G.run_gpu(gpu, "aixk_reduce_to", 0, G.ref(a), G.ref(keep))
        G.run_gpu(gpu, "aixk_reduce_to", 1, G.ref(a), G.ref(keep))
    # matmul with an empty M, N or K extent
    for (m, k, n) in ((0, 8, 8), (8, 8, 0)):
        G.run_gpu(gpu, "aixk_matmul", G.ref(_desc(p, dtype, [m, k])), G.ref(_desc(q, dtype, [k, n])), G.ref(_desc(out, dtype, [m, n])))
    got = gpu.fetch(out, host)
    assert np.array_equal(got, host), "an operator on empty operands wrote to its result"
    gpu.release()


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.I32], ids=lambda d: NAMES[d])
def test_rank_zero_tensors(gpu, dtype):
    rng = np.random.default_rng(41000 + dtype)
    a = T.HostTensor(T.random_values(rng, 1, dtype, int_span=50), dtype, [])
    b = T.HostTensor(T.random_values(rng, 1, dtype, int_span=50), dtype, [])
    want = T.empty(dtype, [])
    okc(CPU.binary(O.ADD, C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc())))
    _, da = gpu.put(a)
    _, db = gpu.put(b)
    po, do = gpu.put(T.empty(dtype, []))
    G.run_gpu(gpu, "aixk_binary", O.ADD, G.ref(da), G.ref(db), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, "rank-0 add")
    # a rank-0 value read through a stride-0 view of rank 3 (Tensor op scalar)
    big = T.contiguous_tensor(rng, dtype, [3, 4, 5], int_span=50)
    view = T.HostTensor(a.storage, dtype, [3, 4, 5], [0, 0, 0])
    want = T.empty(dtype, [3, 4, 5])
    okc(CPU.binary(O.MUL, C.byref(big.desc()), C.byref(view.desc()), C.byref(want.desc())))
    _, dbig = gpu.put(big)
    _, dview = gpu.put(view)
    po, do = gpu.put(T.empty(dtype, [3, 4, 5]))
    G.run_gpu(gpu, "aixk_binary", O.MUL, G.ref(dbig), G.ref(dview), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, "tensor * rank-0 scalar view")
    # sum of a rank-0 tensor is itself
    po, do = gpu.put(T.empty(dtype, []))
    G.run_gpu(gpu, "aixk_reduce_all", 0, G.ref(da), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, a.storage), a.storage, "sum of a rank-0 tensor")
    gpu.release()


@pytest.mark.parametrize("dtype", [O.F32, O.BF16, O.I16], ids=lambda d: NAMES[d])
def test_rank_16_views(gpu, dtype):
    """[2] * 16 = 65 536 elements walked through permuted strides (no two neighbouring dimensions can
    be merged), a broadcast dimension pattern, and reduced over every other dimension."""
    rng = np.random.default_rng(42000 + dtype)
    shape = [2] * 16
    dense = O.row_major(shape)
    perm = [15, 0, 14, 1, 13, 2, 12, 3, 11, 4, 10, 5, 9, 6, 8, 7]
    permuted = [dense[p] for p in perm]                                   # a 16-D transpose of the same storage
    a = T.HostTensor(T.random_values(rng, 1 << 16, dtype, int_span=50), dtype, shape, permuted)
    bc = [0 if d % 2 else s for d, s in enumerate(O.row_major([2 if d % 2 == 0 else 1 for d in range(16)]))]
    b = T.HostTensor(T.random_values(rng, 1 << 8, dtype, int_span=50), dtype, shape, bc)      # broadcast along the odd dimensions
    want = T.empty(dtype, shape)
    okc(CPU.binary(O.ADD, C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc())))
    _, da = gpu.put(a)
    _, db = gpu.put(b)
    po, do = gpu.put(T.empty(dtype, shape))
    G.run_gpu(gpu, "aixk_binary", O.ADD, G.ref(da), G.ref(db), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"rank-16 add {NAMES[dtype]}")
    # gather the permuted view
    want = T.empty(dtype, shape)
    okc(CPU.contiguous(C.byref(a.desc()), C.byref(want.desc())))
    po, do = gpu.put(T.empty(dtype, shape))
    G.run_gpu(gpu, "aixk_contiguous", G.ref(da), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"rank-16 contiguous {NAMES[dtype]}")
    # reduce over the odd dimensions into [2, 1, 2, 1, ...]
    dshape = [2 if d % 2 == 0 else 1 for d in range(16)]
    if dtype in T.INT_DTYPES:
        want = T.empty(dtype, dshape, fill=0)
        okc(CPU.reduce_to(C.byref(a.desc()), C.byref(want.desc())))
        po, do = gpu.put(T.empty(dtype, dshape, fill=0))
        G.run_gpu(gpu, "aixk_reduce_to", 0, G.ref(da), G.ref(do))
        T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"rank-16 reduceTo {NAMES[dtype]}")
    want = T.empty(dtype, dshape)
    okc(CPU.fill_min(C.byref(want.desc())))
    okc(CPU.max_to(C.byref(a.desc()), C.byref(want.desc())))
    init = want.clone()
    okc(CPU.fill_min(C.byref(init.desc())))
    po, do = gpu.put(init)
    G.run_gpu(gpu, "aixk_reduce_to", 1, G.ref(da), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, want.storage), want.storage, f"rank-16 maxTo {NAMES[dtype]}")
    gpu.release()


def test_seventeen_dimensions_are_refused(gpu):
    p, host = _sentinel(gpu)
    q, _ = _sentinel(gpu)
    bad = K.Tensor()
    bad.data = p
    bad.dtype = O.F32
    bad.rank = 17
    bad.size = 1
    good = _desc(q, O.F32, [1])
    lib = gpu.ctx.lib
    assert lib.aixk_binary(gpu.ctx.handle, O.ADD, G.ref(bad), G.ref(good), G.ref(good)) == 1
    assert lib.aixk_unary(gpu.ctx.handle, O.NEG, G.ref(bad), G.ref(good)) == 1
    assert lib.aixk_contiguous(gpu.ctx.handle, G.ref(bad), G.ref(good)) == 1
    assert lib.aixk_reduce_all(gpu.ctx.handle, 0, G.ref(bad), G.ref(good)) == 1
    assert b"" != lib.aixk_last_error()
    gpu.ctx.sync()
    assert np.array_equal(gpu.fetch(q, host), host)
    gpu.release()


def test_rank_16_views_through_the_device(gpu):
    """The lazy device takes views of more than 8 dimensions as well (they bypass the generated kernels,
    which index at most 8 collapsed dimensions): result equal to the CPU evaluation, work before and
    after them still ordered."""
    import devharness as H
    dev = H.Dev()
    try:
        rng = np.random.default_rng(43000)
        shape = [2] * 16
        dense = O.row_major(shape)
        perm = [15, 0, 14, 1, 13, 2, 12, 3, 11, 4, 10, 5, 9, 6, 8, 7]
        a = T.HostTensor(T.random_values(rng, 1 << 16, O.F32), O.F32, shape, [dense[p] for p in perm])
        b = T.contiguous_tensor(rng, O.F32, shape)
        t1, t2, want = T.empty(O.F32, shape), T.empty(O.F32, shape), T.empty(O.F32, shape)
        okc(CPU.binary(O.MUL, C.byref(b.desc()), C.byref(b.desc()), C.byref(t1.desc())))       # recorded, fusable
        okc(CPU.binary(O.ADD, C.byref(a.desc()), C.byref(t1.desc()), C.byref(t2.desc())))      # rank-16 strided operand
        okc(CPU.unary(O.NEG, C.byref(t2.desc()), C.byref(want.desc())))
        pa, da = dev.put(a)
        pb, db = dev.put(b)
        p1, p2, p3 = dev.raw(t1.storage.nbytes), dev.raw(t1.storage.nbytes), dev.raw(t1.storage.nbytes)
        d1, d2, d3 = H.kdesc(t1, p1), H.kdesc(t2, p2), H.kdesc(want, p3)
        dev.dev.call("mul", H.ref(db), H.ref(db), H.ref(d1))
        dev.dev.call("add", H.ref(da), H.ref(d1), H.ref(d2))
        dev.dev.call("unary", H.ref(d2), H.ref(d3))
        T.assert_same_bits(dev.fetch(p3, want.storage), want.storage, "rank-16 operand between recorded operators")
        dev.release()
    finally:
        dev.close()


def test_more_than_four_giga_elements(gpu):
    """2^32 + 4099 uint8 elements: every flat index beyond 32 bits.  add, cast, fill, max and the
    strided gather (a [2, n/2] transpose would not fit the ragged count, so a sliced view: every second
    element of the first half) against numpy."""
    n = (1 << 32) + 4099
    rng = np.random.default_rng(44000)
    a = rng.integers(0, 256, n, dtype=np.uint8)
    b = rng.integers(0, 256, n, dtype=np.uint8)
    pa, pb, po = gpu.raw(n), gpu.raw(n), gpu.raw(n)
    gpu.ctx.upload(pa, a)
    gpu.ctx.upload(pb, b)
    da, db, do = _desc(pa, O.U8, [n]), _desc(pb, O.U8, [n]), _desc(po, O.U8, [n])
    G.run_gpu(gpu, "aixk_binary", O.ADD, G.ref(da), G.ref(db), G.ref(do))
    got = np.empty(n, np.uint8)
    gpu.ctx.download(got, po)
    want = a + b                                             # uint8 wraps, as the device does
    assert np.array_equal(got[-8192:], want[-8192:]) and np.array_equal(got[:8192], want[:8192])
    assert np.array_equal(got, want), "uint8 add beyond 2^32 elements"
    # max over everything, and with the only 255 placed past the 32-bit boundary
    a2 = np.minimum(a, 254)
    a2[(1 << 32) + 77] = 255
    gpu.ctx.upload(pa, a2)
    pm = gpu.raw(256)
    G.run_gpu(gpu, "aixk_reduce_all", 1, G.ref(da), G.ref(_desc(pm, O.U8, [1])))
    m = np.zeros(1, np.uint8)
    gpu.ctx.download(m, pm)
    assert m[0] == 255
    # cast to int8 over the whole range (integer to integer is the plain C++ conversion: it wraps)
    G.run_gpu(gpu, "aixk_cast", pa, O.U8, po, O.I8, n)
    gpu.ctx.download(got, po)
    assert np.array_equal(got, a2), "u8 -> i8 cast beyond 2^32 elements"
    # fill, then check both ends and the total
    seven = np.array([7], np.uint8)
    G.run_gpu(gpu, "aixk_fill", seven.ctypes.data, O.U8, G.ref(do))
    gpu.ctx.download(got, po)
    assert got.min() == 7 and got.max() == 7
    # strided gather with offsets and strides beyond 32 bits: every second element of the upper half
    half = n // 2
    cnt = (n - half) // 2
    src = _desc(pa, O.U8, [cnt], [2], offset=half)
    G.run_gpu(gpu, "aixk_contiguous", G.ref(src), G.ref(_desc(po, O.U8, [cnt])))
    gpu.ctx.download(got, po)
    assert np.array_equal(got[:cnt], a2[half:half + 2 * cnt:2]), "strided gather beyond 2^32"
    gpu.release()


def test_generated_kernel_beyond_four_giga_elements():
    """The same count through the lazy device: y = (a + b) * a as one generated kernel on uint8."""
    import devharness as H
    dev = H.Dev()
    try:
        n = (1 << 32) + 4099
        rng = np.random.default_rng(44001)
        a = T.HostTensor(rng.integers(0, 256, n, dtype=np.uint8), O.U8, [n])
        b = T.HostTensor(rng.integers(0, 256, n, dtype=np.uint8), O.U8, [n])
        pa, da = dev.put(a)
        pb, db = dev.put(b)
        pt, py = dev.raw(n, keep=False), dev.raw(n)
        dt, dy = H.kdesc(a, pt), H.kdesc(a, py)
        dev.dev.call("add", H.ref(da), H.ref(db), H.ref(dt))
        dev.dev.call("mul", H.ref(dt), H.ref(da), H.ref(dy))
        dev.dev.deallocate(pt)
        got = dev.fetch(py, a.storage)
        want = (a.storage + b.storage) * a.storage          # uint8 arithmetic wraps on both sides
        assert np.array_equal(got, want)
        dev.release()
    finally:
        dev.close()
