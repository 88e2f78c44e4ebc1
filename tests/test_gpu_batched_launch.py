"""The kernel-layer entry points that carry several pieces of work in one launch, through the C ABI: aixk_fill_many
(small fills, each item a pattern already in its destination's element type), aixk_rtc_launch_many (several argument
blocks of one runtime-compiled kernel, each with its share of the grid), aixk_slice_set_many (several sliceSet calls) and
aixk_argmax_onehot_many (several argmaxIndicesTo calls with their zero fill) and aixk_sum_columns_many (several reduceTo
calls down the columns of a matrix, with the fill of their destination) and aixk_sum_partials_many (the second halves of
several sums over everything).
Results against numpy (fills and an exact elementwise body) and the CPU oracle's sliceSet, sizes down to one element and
ragged tails, and the argument checks they promise."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import gpuharness as G
from aix_amd import kernels as K
from oracle import cpuref as O

CPU = O.lib()

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    g = G.Gpu()
    yield g
    g.close()
    g.ctx.close()


def _items(entries):
    arr = (K.FillItem * len(entries))()
    for k, (dst, bits, n, esz) in enumerate(entries):
        arr[k].dst, arr[k].bits, arr[k].elements, arr[k].element_size = dst, bits, n, esz
    return arr


def test_fill_many_writes_every_item_and_nothing_else(gpu):
    rng = np.random.default_rng(51000)
    cases = []      # (pointer to the guarded buffer, elements, element size, pattern)
    for esz, dtype in ((1, np.uint8), (2, np.uint16), (4, np.uint32), (8, np.uint64)):
        for n in (1, 2, 255, 256, 257, 4099, 65536):
            pattern = int(rng.integers(1, 2 ** (8 * esz - 1), dtype=np.uint64))
            p = gpu.raw((n + 32) * esz)                              # 16 guard elements on either side
            gpu.ctx.upload(p, np.full(n + 32, 0x5A, dtype=np.uint8).repeat(esz)[: (n + 32) * esz].copy())
            cases.append((p, n, esz, dtype, pattern))
    entries = [(p + 16 * esz, pattern, n, esz) for p, n, esz, _, pattern in cases]
    G.run_gpu(gpu, "aixk_fill_many", _items(entries), len(entries))
    for p, n, esz, dtype, pattern in cases:
        got = gpu.fetch(p, np.zeros(n + 32, dtype))
        guard = np.frombuffer(bytes([0x5A]) * esz, dtype=dtype)[0]
        assert np.all(got[16:16 + n] == dtype(pattern & (2 ** (8 * esz) - 1))), (n, esz)
        assert np.all(got[:16] == guard) and np.all(got[16 + n:] == guard), ("guards", n, esz)
    # 40 items in one call (at most 32 travel with a launch: two launches inside), every one on an address of its own
    many = [(cases[k % len(cases)][0] + (16 + k // len(cases)) * cases[k % len(cases)][2], k + 1, 1, cases[k % len(cases)][2]) for k in range(40)]
    G.run_gpu(gpu, "aixk_fill_many", _items(many), len(many))
    for dst, bits, _, esz in many:
        got = gpu.fetch(dst, np.zeros(1, {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[esz]))
        assert int(got[0]) == bits
    gpu.release()


def test_fill_many_checks_its_items(gpu):
    p = gpu.raw(1 << 20)
    lib, h = gpu.ctx.lib, gpu.ctx.handle
    assert lib.aixk_fill_many(h, _items([(p, 1, 4, 3)]), 1) == 1            # element size 3
    assert lib.aixk_fill_many(h, _items([(p, 1, 65537, 4)]), 1) == 1        # too many elements for one item
    assert lib.aixk_fill_many(h, _items([(p + 2, 1, 4, 4)]), 1) == 1        # misaligned for its element size
    assert lib.aixk_fill_many(h, _items([(None, 1, 4, 4)]), 1) == 1         # null destination
    assert lib.aixk_fill_many(h, None, 0) == 0                              # nothing to do is fine
    gpu.ctx.sync()
    gpu.release()


SOURCE = r"""
#include "aix_device.h"
using namespace aixd;
struct Args { const float* x; float* y; float scale; float shift; u64 n; };
extern "C" __global__ __launch_bounds__(256) void axpb_many(const Args* table, const u32* starts, u32 count)
{
    u32 lo = 0, hi = count;
    while (hi - lo > 1) { const u32 mid = (lo + hi) / 2; if (starts[mid] <= blockIdx.x) lo = mid; else hi = mid; }
    const Args a = table[lo];
    const u32 bid = blockIdx.x - starts[lo], gdim = starts[lo + 1] - starts[lo];
    const float* x = global_ptr<const float>((u64)a.x);
    float* y = global_ptr<float>((u64)a.y);
    for (u64 i = (u64)bid * 256 + threadIdx.x; i < a.n; i += (u64)gdim * 256) y[i] = x[i] * a.scale + a.shift;
}
"""


class Args(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("scale", C.c_float), ("shift", C.c_float), ("n", C.c_uint64)]


def _table(blocks, grids):
    """Argument blocks back to back, then count + 1 uint32: the first workgroup of every share and the grid size."""
    raw = b"".join(bytes(b) for b in blocks)
    starts = np.concatenate([[0], np.cumsum(grids)]).astype(np.uint32)
    return raw + starts.tobytes(), len(raw)


def test_launch_many_runs_every_argument_block(gpu):
    rng = np.random.default_rng(52000)
    mod = C.c_void_p()
    cached = C.c_int32()
    G.run_gpu(gpu, "aixk_rtc_get", b"test|axpb_many", SOURCE.encode(), b"axpb_many", C.byref(mod), C.byref(cached))
    sizes = [1, 255, 256, 257, 1000, 65537, 3, 300000]
    xs = [rng.integers(-8, 9, n).astype(np.float32) for n in sizes]               # small integers: a*x + b is exact
    blocks, grids, outs = [], [], []
    for k, (n, x) in enumerate(zip(sizes, xs)):
        px, py = gpu.raw(n * 4), gpu.raw(n * 4)
        gpu.ctx.upload(px, x)
        blocks.append(Args(px, py, float(k + 1), float(-k), n))
        grids.append(max(1, min((n + 255) // 256, 7 + k)))                       # some shares loop, some do not
        outs.append(py)
    table, starts_offset = _table(blocks, grids)
    buf = C.create_string_buffer(table, len(table))
    G.run_gpu(gpu, "aixk_rtc_launch_many", mod, 256, buf, len(table), starts_offset, len(blocks))
    buf.raw = b"\0" * len(table)                                                 # the host's copy may be reused as soon as the call returns
    for k, (x, py) in enumerate(zip(xs, outs)):
        got = gpu.fetch(py, x)
        assert np.array_equal(got, x * np.float32(k + 1) + np.float32(-k)), sizes[k]
    # the checks: shares out of order, a first share that does not start at 0, a table too large, starts outside the table
    lib, h = gpu.ctx.lib, gpu.ctx.handle
    bad, off = _table(blocks[:2], [4, 4])
    starts = np.frombuffer(bad[off:], np.uint32).copy()
    for wrong in ([0, 4, 4], [1, 4, 8], [0, 8, 4]):
        t = bad[:off] + np.array(wrong, np.uint32).tobytes()
        assert lib.aixk_rtc_launch_many(h, mod, 256, C.create_string_buffer(t, len(t)), len(t), off, 2) == 1, wrong
    assert lib.aixk_rtc_launch_many(h, mod, 256, C.create_string_buffer(bad, len(bad)), len(bad), off + 8, 2) == 1       # starts run past the end
    big = b"\0" * ((256 << 10) + 8)
    assert lib.aixk_rtc_launch_many(h, mod, 256, C.create_string_buffer(big, len(big)), len(big), 0, 1) == 1
    assert lib.aixk_rtc_launch_many(h, mod, 256, None, 0, 0, 0) == 1
    gpu.ctx.sync()
    gpu.release()


def _slice_items(entries):
    arr = (K.SliceItem * len(entries))()
    for k, (src, dst, dim, start, end, step) in enumerate(entries):
        arr[k].src, arr[k].dst, arr[k].dim, arr[k].start, arr[k].end, arr[k].step = src, dst, dim, start, end, step
    return arr


@pytest.mark.parametrize("dtype", [O.F32, O.BF16, O.I8, O.F64], ids=["f32", "bf16", "i8", "f64"])
def test_slice_set_many_is_slice_set_item_by_item(gpu, dtype):
    """Random sources (contiguous, transposed, sliced, offset views) into windows of separate destinations, and a
    destination that receives all its column blocks from different sources (a cat): bit-identical to the oracle's
    sliceSet applied item by item."""
    rng = np.random.default_rng(53000 + dtype)
    entries, checks = [], []
    for trial in range(40):
        shape = T.random_shape(rng, max_rank=4, max_extent=9)
        src = T.view_tensor(rng, dtype, shape, rng.choice(T.VIEW_KINDS))
        _, dsrc = gpu.put(src)
        dim = int(rng.integers(0, len(shape)))
        step, start = int(rng.integers(1, 3)), int(rng.integers(0, 3))
        big = list(shape)
        big[dim] = start + (shape[dim] - 1) * step + 1 + int(rng.integers(0, 2))
        end = min(big[dim], start + shape[dim] * step)
        dst = T.view_tensor(rng, dtype, big, rng.choice(["contig", "transposed", "offset", "sliced"]))
        want = dst.clone()
        assert CPU.slice_set(C.byref(src.desc()), C.byref(want.desc()), dim, start, end, step, 1) == 0
        pd, dd = gpu.put(dst)
        entries.append((dsrc, dd, dim, start, end, step))
        checks.append((pd, want, f"item {trial} {shape}->{big} dim={dim}"))
    # one destination, twelve column blocks, every one from a source of its own (the last a strided view)
    rows, width, parts = 37, 8, 12
    whole = T.empty(dtype, [rows, width * parts], fill=3)
    want = whole.clone()
    pw, dw = gpu.put(whole)
    for k in range(parts):
        src = T.view_tensor(rng, dtype, [rows, width], "transposed" if k == parts - 1 else "contig")
        _, dsrc = gpu.put(src)
        assert CPU.slice_set(C.byref(src.desc()), C.byref(want.desc()), 1, k * width, (k + 1) * width, 1, 1) == 0
        entries.append((dsrc, dw, 1, k * width, (k + 1) * width, 1))
    checks.append((pw, want, "twelve column blocks of one destination"))
    G.run_gpu(gpu, "aixk_slice_set_many", _slice_items(entries), len(entries))
    for pd, want, what in checks:
        T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, "sliceSet of several items: " + what)
    gpu.release()


def test_slice_set_many_checks_its_items(gpu):
    rng = np.random.default_rng(54000)
    src = T.contiguous_tensor(rng, O.F32, [4, 8])
    dst = T.empty(O.F32, [4, 32], fill=1)
    other = T.contiguous_tensor(rng, O.BF16, [4, 8])
    obig = T.empty(O.BF16, [4, 32], fill=1)
    _, ds = gpu.put(src)
    pd, dd = gpu.put(dst)
    _, d16 = gpu.put(other)
    _, d16big = gpu.put(obig)
    lib, h = gpu.ctx.lib, gpu.ctx.handle
    good = (ds, dd, 1, 0, 8, 1)
    assert lib.aixk_slice_set_many(h, None, 0) == 0                                           # nothing to do is fine
    assert lib.aixk_slice_set_many(h, _slice_items([good, (ds, dd, 1, 28, 36, 1)]), 2) == 1    # window beyond the destination
    assert lib.aixk_slice_set_many(h, _slice_items([good, (ds, dd, 1, 8, 12, 1)]), 2) == 1     # source larger than the window
    assert lib.aixk_slice_set_many(h, _slice_items([good, (ds, dd, 2, 8, 16, 1)]), 2) == 1     # no such dim
    assert lib.aixk_slice_set_many(h, _slice_items([good, (ds, dd, 1, 8, 16, 0)]), 2) == 1     # step 0
    assert lib.aixk_slice_set_many(h, _slice_items([good, (ds, d16big, 1, 8, 16, 1)]), 2) == 1   # element types differ within an item
    assert lib.aixk_slice_set_many(h, _slice_items([good, (d16, d16big, 1, 8, 16, 1)]), 2) == 1  # element sizes differ between items
    assert lib.aixk_slice_set_many(h, _slice_items([good] * 513), 513) == 1                    # more items than one call takes
    gpu.ctx.sync()
    got = gpu.fetch(pd, dst.storage)
    assert np.all(got == 1), "a refused call must launch nothing"
    gpu.release()


def _argmax_items(entries):
    arr = (K.ArgmaxItem * len(entries))()
    for k, (src, dst, dim) in enumerate(entries):
        arr[k].src, arr[k].dst, arr[k].dim = src, dst, dim
    return arr


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.F16], ids=["bf16", "f32", "f16"])
def test_argmax_onehot_many_is_fill_and_argmax_indices_item_by_item(gpu, dtype):
    """Dense tensors reduced along their last dim leave in one launch; a set with an item of another kind (another dim,
    a strided source) runs item by item.  Either way every destination equals zeros + the oracle's argmaxIndicesTo:
    ties (values on a coarse grid) go to the first maximum, a row of NaNs picks its first element."""
    rng = np.random.default_rng(55000 + dtype)

    def case(shape, dim, kind="contig"):
        src = T.view_tensor(rng, dtype, shape, kind, lo=-2, hi=2)
        vals = O.to_float64(src.storage, dtype)
        src.storage[:] = O.to_storage(np.round(vals * 4) / 4, dtype)
        if shape[-1] >= 64:
            src.storage[: shape[-1]] = O.to_storage(np.full(shape[-1], np.nan), dtype)       # the first row: NaNs only
        want = T.empty(O.I32, shape)
        assert CPU.argmax_indices_to(C.byref(src.desc()), C.byref(want.desc()), dim) == 0
        _, dsrc = gpu.put(src)
        pd, dd = gpu.put(T.empty(O.I32, shape, fill=9))                                      # every element must be written
        return (dsrc, dd, dim), (pd, want, f"{shape} dim={dim} {kind}")

    together = [case([64, 512], 1), case([3, 40, 64], 2), case([1, 32], 1), case([517, 96], 1), case([2, 2, 2, 128], 3)]
    G.run_gpu(gpu, "aixk_argmax_onehot_many", _argmax_items([c[0] for c in together]), len(together))
    for _, (pd, want, what) in together:
        T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, "argmaxIndicesTo of several items, one launch: " + what)
    mixed = [case([64, 512], 1), case([40, 64], 0), case([8, 48], 1, "transposed"), case([5, 30], 1)]
    G.run_gpu(gpu, "aixk_argmax_onehot_many", _argmax_items([c[0] for c in mixed]), len(mixed))
    for _, (pd, want, what) in mixed:
        T.assert_same_bits(gpu.fetch(pd, want.storage), want.storage, "argmaxIndicesTo of several items, item by item: " + what)
    lib, h = gpu.ctx.lib, gpu.ctx.handle
    assert lib.aixk_argmax_onehot_many(h, None, 0) == 0
    bad_src, bad_dst, _ = together[0][0]
    wrong = K.Tensor.from_buffer_copy(bad_dst)
    wrong.dtype = O.F32
    assert lib.aixk_argmax_onehot_many(h, _argmax_items([together[1][0], (bad_src, wrong, 1)]), 2) == 1      # result must be int32
    gpu.ctx.sync()
    gpu.release()


def _colsum_items(entries):
    arr = (K.ColsumItem * len(entries))()
    for k, (src, dst, bits) in enumerate(entries):
        arr[k].src, arr[k].dst, arr[k].init_bits = src, dst, bits
    return arr


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.F16], ids=["bf16", "f32", "f16"])
def test_sum_columns_many_is_fill_and_reduce_to_item_by_item(gpu, dtype):
    """Dense matrices summed down their columns leave in two launches for all of them; a set with an item of another kind
    (a strided source, a column count that is no multiple of 4, a row sum) runs item by item.  Either way every destination
    equals fill(init) + the oracle's reduceTo: against the sums in wide arithmetic, 1e-5 of the sum of the terms'
    magnitudes plus one rounding in the result's type (2^-10 for f16, 2^-8 for bf16), as for aixk_reduce_to."""
    rng = np.random.default_rng(56000 + dtype)
    tol, final = {O.F32: (1e-5, 0.0), O.F16: (1e-5, 2.0 ** -10), O.BF16: (1e-5, 2.0 ** -8)}[dtype]

    def case(shape, dshape, init_value, kind="contig"):
        src = T.view_tensor(rng, dtype, shape, kind, lo=-2, hi=2)
        bits_arr = O.to_storage(np.array([init_value]), dtype)
        bits = int.from_bytes(bits_arr.tobytes()[:O.ITEMSIZE[dtype]], "little")
        n = max(1, int(np.prod(dshape)))
        filled = T.HostTensor(np.resize(bits_arr.view(O.NP_STORAGE[dtype]), n).copy(), dtype, dshape)
        exact = filled.values().reshape(-1).copy()
        scale = np.abs(exact)
        assert CPU.reduce_to_wide(C.byref(src.desc()), C.byref(filled.desc()), exact.ctypes.data, scale.ctypes.data) == 0
        _, dsrc = gpu.put(src)
        garbage = T.HostTensor(np.resize(O.to_storage(np.array([777.0]), dtype), n).copy(), dtype, dshape)      # never read
        pd, dd = gpu.put(garbage)
        return (dsrc, dd, bits), (pd, garbage, exact, scale, f"{shape}->{dshape} init {init_value} {kind}")

    def check(cases, how):
        for _, (pd, like, exact, scale, what) in cases:
            got = O.to_float64(gpu.fetch(pd, like.storage), dtype)
            G.assert_close_to_wide(got, exact, scale + (final / tol) * np.abs(exact) + 1e-30, tol, f"column sums of several items, {how}: {what}")

    together = [case([8192, 768], [768], 0.0), case([2, 4], [1, 4], 3.0), case([700, 260], [260], -1.5), case([3, 50, 1024], [1024], 0.0),
                case([16, 31, 8], [1, 1, 8], 0.25), case([4099, 12], [12], 0.0)]
    G.run_gpu(gpu, "aixk_sum_columns_many", _colsum_items([c[0] for c in together]), len(together))
    check(together, "together")
    mixed = [case([64, 512], [512], 0.0), case([40, 64], [40, 1], 1.0), case([48, 8], [8], 0.0, "transposed"), case([50, 30], [30], 2.0), case([1, 16], [16], 0.0)]
    G.run_gpu(gpu, "aixk_sum_columns_many", _colsum_items([c[0] for c in mixed]), len(mixed))
    check(mixed, "item by item")
    lib, h = gpu.ctx.lib, gpu.ctx.handle
    assert lib.aixk_sum_columns_many(h, None, 0) == 0
    bad_src, bad_dst, _ = together[0][0]
    wrong = K.Tensor.from_buffer_copy(bad_dst)
    wrong.dtype = O.I32
    assert lib.aixk_sum_columns_many(h, _colsum_items([together[1][0], (bad_src, wrong, 0)]), 2) == 1      # element types must agree
    gpu.ctx.sync()
    gpu.release()


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.F16, O.F64], ids=["bf16", "f32", "f16", "f64"])
def test_sum_partials_many_lands_every_sum(gpu, dtype):
    """Item k is aixk_sum_partials of its fields: dst = init + the sum of `count` partial sums (f32; f64 for f64), rounded
    once.  One launch for destinations of one element type, item by item for a mixed set.  Against numpy's float64 sum:
    1e-5 of the sum of magnitudes (1e-12 for f64) plus one rounding of the result."""
    rng = np.random.default_rng(57000 + dtype)
    bounds = {O.F64: (1e-12, 0.0), O.F32: (1e-5, 0.0), O.F16: (1e-5, 2.0 ** -10), O.BF16: (1e-5, 2.0 ** -8)}

    def case(count, init_value, dt=dtype):
        parts = rng.uniform(-1, 1, count).astype(np.float64 if dt == O.F64 else np.float32)
        pp = gpu.raw(parts.nbytes)
        gpu.ctx.upload(pp, parts)
        init_arr = O.to_storage(np.array([init_value]), dt)
        bits = int.from_bytes(init_arr.tobytes()[:O.ITEMSIZE[dt]], "little")
        garbage = T.HostTensor(O.to_storage(np.array([777.0]), dt).copy(), dt, [])
        pd, dd = gpu.put(garbage)
        init_exact = float(O.to_float64(init_arr, dt)[0])
        exact = init_exact + float(np.sum(parts.astype(np.float64)))
        scale = abs(init_exact) + float(np.sum(np.abs(parts.astype(np.float64))))
        return (pp, count, dd, bits), (pd, garbage, dt, exact, scale, f"{count} partials, init {init_value}")

    def items_of(cases):
        arr = (K.PartialsItem * len(cases))()
        for k, ((pp, count, dd, bits), _) in enumerate(cases):
            arr[k].partials, arr[k].count, arr[k].dst, arr[k].init_bits = pp, count, dd, bits
        return arr

    def check(cases, how):
        for _, (pd, like, dt, exact, scale, what) in cases:
            got = float(O.to_float64(gpu.fetch(pd, like.storage), dt)[0])
            t, f = bounds[dt]
            assert abs(got - exact) <= t * scale + f * abs(exact) + 1e-30, f"sums of partials, {how}: {what}: got {got!r}, exact {exact!r}"

    together = [case(1, 0.0), case(7, 3.0), case(256, -1.5), case(2049, 0.0), case(100000, 0.25)]
    G.run_gpu(gpu, "aixk_sum_partials_many", items_of(together), len(together))
    check(together, "one launch")
    if dtype != O.F64:
        mixed = [case(300, 1.0), case(5, 0.0, O.F32 if dtype != O.F32 else O.BF16), case(4097, 2.0)]
        G.run_gpu(gpu, "aixk_sum_partials_many", items_of(mixed), len(mixed))
        check(mixed, "item by item")
    lib, h = gpu.ctx.lib, gpu.ctx.handle
    assert lib.aixk_sum_partials_many(h, None, 0) == 0
    bad = items_of(together[:2])
    bad[1].count = 0
    assert lib.aixk_sum_partials_many(h, bad, 2) == 1                    # an item without partials is refused (by the single call)
    gpu.ctx.sync()
    gpu.release()
