"""Runs of small matmul calls issued as one launch.

The interface has no batch dimension (Targets/AIXLib/aixCore.hpp:943-976): a batch of products, or attention over
(sequence, head) pairs, reaches the device as a run of 2-D matmul calls.  The kernel layer can issue `count` separate
products of one shape in one launch (aixk_matmul_grouped: the operand addresses come from a table in device memory), and
the device holds small 16-bit matmul calls back until something else happens and then issues them together.  Checked
here: the grouped launch against the same products issued one by one -- within f32 accumulation error plus the final
rounding, like the stacked launch -- and against the exactly accumulated oracle; the device-level grouping with
dependent products, products of another shape in between, elementwise work before, between and after, results that are
freed before the flush, and a group long enough to wrap the table ring."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import devharness as H
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


@pytest.fixture(scope="module")
def dev():
    d = H.Dev()
    yield d
    d.close()


def exact_product(a, b):
    m, n = a.shape[0], b.shape[1]
    exact, scale = np.zeros(m * n), np.zeros(m * n)
    assert CPU.matmul_wide(C.byref(a.desc()), C.byref(b.desc()), exact.ctypes.data, scale.ctypes.data, 8) == 0
    return exact, scale


def operand(rng, dtype, rows, cols, layout):
    """A [rows, cols] operand: dense, a transposed view of a dense [cols, rows], or a slice of a wider matrix."""
    if layout == "N":
        return T.HostTensor(T.random_values(rng, rows * cols, dtype, lo=-0.5, hi=0.5), dtype, [rows, cols])
    if layout == "T":
        return T.HostTensor(T.random_values(rng, rows * cols, dtype, lo=-0.5, hi=0.5), dtype, [rows, cols], [1, rows])
    wide = cols + 16
    return T.HostTensor(T.random_values(rng, rows * wide, dtype, lo=-0.5, hi=0.5), dtype, [rows, cols], [wide, 1], 8)


def array_of(descs):
    arr = (K.Tensor * len(descs))()
    for i, d in enumerate(descs):
        C.memmove(C.byref(arr[i]), C.byref(d), C.sizeof(K.Tensor))
    return arr


@pytest.mark.parametrize("dtype", [O.BF16, O.F16], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("case", [(64, 64, 64, "N", "N", 5), (512, 64, 512, "N", "T", 7), (512, 512, 64, "N", "N", 3), (512, 512, 64, "T", "N", 4),
                                  (128, 256, 192, "S", "S", 6), (512, 512, 512, "N", "N", 9), (96, 40, 72, "N", "N", 3),
                                  # whole 128 x {128, 192} tiles and K >= 512: the LDS-direct kernel's smaller tiles, addresses from the table
                                  (768, 1024, 768, "T", "N", 6), (384, 512, 640, "N", "T", 10), (256, 576, 512, "S", "N", 16),
                                  # K = 64, both operands K-contiguous, two 128 x 128 tiles per compute unit: the kernel without LDS reads the table
                                  (512, 64, 512, "N", "T", 32), (256, 64, 384, "S", "T", 86),
                                  # 216 whole 256 x 256 tiles over the group: one round of the chip on that kernel's largest tile, in every layout
                                  (768, 576, 768, "T", "N", 24), (768, 512, 768, "N", "T", 24), (768, 512, 768, "T", "T", 24), (768, 512, 768, "N", "N", 24)], ids=str)
def test_grouped_launch_matches_single_launches(gpu, dtype, case):
    m, k, n, la, lb, count = case
    rng = np.random.default_rng(9100 + m + k + n + dtype)
    a = [operand(rng, dtype, m, k, la) for _ in range(count)]
    b = [operand(rng, dtype, k, n, lb) for _ in range(count)]
    da = [gpu.put(t)[1] for t in a]
    db = [gpu.put(t)[1] for t in b]
    outs = [gpu.put(T.empty(dtype, [m, n], fill=1)) for _ in range(count)]
    singles = [gpu.put(T.empty(dtype, [m, n], fill=2)) for _ in range(count)]
    G.run_gpu(gpu, "aixk_matmul_grouped", array_of(da), array_of(db), array_of([d for _, d in outs]), count)
    for i in range(count):
        G.run_gpu(gpu, "aixk_matmul", G.ref(da[i]), G.ref(db[i]), G.ref(singles[i][1]))
    final = 2.0 ** -10 if dtype == O.F16 else 2.0 ** -8
    like = np.zeros(m * n, O.NP_STORAGE[dtype])
    for i in range(count):
        exact, scale = exact_product(a[i], b[i])
        got = O.to_float64(gpu.fetch(outs[i][0], like), dtype)
        one = O.to_float64(gpu.fetch(singles[i][0], like), dtype)
        G.assert_close_to_wide(got, exact, 1e-5 * scale + final * np.abs(exact) + 1e-30, 1.0, f"grouped product {i} of {case}")
        G.assert_close_to_wide(got, one, 2e-5 * scale + 2 * final * np.abs(exact) + 1e-30, 1.0, f"grouped against single, product {i} of {case}")
    gpu.release()


def test_grouped_entry_point_falls_back_product_by_product(gpu):
    """f32 products, products of different shapes and a count of one are not grouped: every product then gets exactly
    what aixk_matmul gives it, and a bad descriptor in the run is refused like a bad single call."""
    rng = np.random.default_rng(9200)
    shapes = [(40, 24, 56), (40, 24, 56), (33, 17, 9)]
    a = [T.contiguous_tensor(rng, O.F32, [m, k]) for m, k, _ in shapes]
    b = [T.contiguous_tensor(rng, O.F32, [k, n]) for _, k, n in shapes]
    da, db = [gpu.put(t)[1] for t in a], [gpu.put(t)[1] for t in b]
    outs = [gpu.put(T.empty(O.F32, [m, n])) for m, _, n in shapes]
    singles = [gpu.put(T.empty(O.F32, [m, n])) for m, _, n in shapes]
    G.run_gpu(gpu, "aixk_matmul_grouped", array_of(da), array_of(db), array_of([d for _, d in outs]), 3)
    for i in range(3):
        G.run_gpu(gpu, "aixk_matmul", G.ref(da[i]), G.ref(db[i]), G.ref(singles[i][1]))
        like = np.zeros(shapes[i][0] * shapes[i][2], np.float32)
        T.assert_same_bits(gpu.fetch(outs[i][0], like), gpu.fetch(singles[i][0], like), f"fallback product {i}")
    G.run_gpu(gpu, "aixk_matmul_grouped", array_of(da[:1]), array_of(db[:1]), array_of([outs[0][1]]), 1)
    G.run_gpu(gpu, "aixk_matmul_grouped", None, None, None, 0)
    bad = array_of([da[0], da[2]])                                       # inner dimensions of the second product differ
    rc = gpu.ctx.lib.aixk_matmul_grouped(gpu.ctx.handle, bad, array_of([db[0], db[0]]), array_of([outs[0][1], outs[1][1]]), 2)
    assert rc == 1
    gpu.release()


def device_matmul(dev, da, db, shape, dtype):
    out = T.empty(dtype, shape)
    po = dev.raw(out.storage.nbytes)
    dev.dev.call("matmul", H.ref(da), H.ref(db), H.ref(H.kdesc(out, po)))
    return po, out


@pytest.mark.parametrize("dtype", [O.BF16, O.F16], ids=lambda d: NAMES[d])
def test_device_groups_runs_of_small_products(dev, dtype):
    """A run of 40 attention-sized products through the device interface with everything that must break or keep a
    group in between; every result against the exactly accumulated oracle."""
    rng = np.random.default_rng(9300 + dtype)
    S, Dh = 128, 64
    final = 2.0 ** -10 if dtype == O.F16 else 2.0 ** -8
    checks = []

    def product(a, da, b, db):
        po, out = device_matmul(dev, da, db, [a.shape[0], b.shape[1]], dtype)
        checks.append((po, out, a, b))
        return po, out

    qs = [T.contiguous_tensor(rng, dtype, [S, Dh], lo=-0.5, hi=0.5) for _ in range(40)]
    ks = [T.HostTensor(T.random_values(rng, S * Dh, dtype, lo=-0.5, hi=0.5), dtype, [Dh, S], [1, Dh]) for _ in range(40)]
    dq = [dev.put(t)[1] for t in qs]
    dk = [dev.put(t)[1] for t in ks]
    for i in range(20):                                                  # one group of 20
        product(qs[i], dq[i], ks[i], dk[i])
    other_a, other_b = T.contiguous_tensor(rng, dtype, [64, 128], lo=-0.5, hi=0.5), T.contiguous_tensor(rng, dtype, [128, 64], lo=-0.5, hi=0.5)
    product(other_a, dev.put(other_a)[1], other_b, dev.put(other_b)[1])  # another shape: the group so far is issued, a new one starts
    for i in range(20, 30):
        product(qs[i], dq[i], ks[i], dk[i])
    # a product that reads a pending result: scores . v with v [S, Dh]; it must see the finished scores
    v = T.contiguous_tensor(rng, dtype, [S, Dh], lo=-0.5, hi=0.5)
    _, dv = dev.put(v)
    p_scores, scores = product(qs[30], dq[30], ks[30], dk[30])
    po_mix, mix = device_matmul(dev, H.kdesc(scores, p_scores), dv, [S, Dh], dtype)
    # an elementwise operator recorded on a pending result, then more products
    doubled = T.empty(dtype, [S, S])
    p_doubled = dev.raw(doubled.storage.nbytes)
    dev.dev.call("add", H.ref(H.kdesc(scores, p_scores)), H.ref(H.kdesc(scores, p_scores)), H.ref(H.kdesc(doubled, p_doubled)))
    for i in range(31, 40):
        product(qs[i], dq[i], ks[i], dk[i])
    # a result freed before anything flushed: the product still runs, into a block nobody reads, and nothing else is disturbed
    p_dropped, _ = device_matmul(dev, dq[0], dk[0], [S, S], dtype)
    dev.free(p_dropped)

    like = np.zeros(S * S, O.NP_STORAGE[dtype])
    for po, out, a, b in checks:
        exact, scale = exact_product(a, b)
        got = O.to_float64(dev.fetch(po, out.storage), dtype)
        G.assert_close_to_wide(got, exact, 1e-5 * scale + final * np.abs(exact) + 1e-30, 1.0, f"grouped device product {a.shape} x {b.shape}")
    got_scores = dev.fetch(p_scores, like)
    sc = T.HostTensor(got_scores, dtype, [S, S])
    exact, scale = exact_product(sc, v)
    G.assert_close_to_wide(O.to_float64(dev.fetch(po_mix, mix.storage), dtype), exact, 1e-5 * scale + final * np.abs(exact) + 1e-30, 1.0, "product of a pending result")
    want = T.empty(dtype, [S, S])
    assert CPU.binary(O.ADD, C.byref(sc.desc()), C.byref(sc.desc()), C.byref(want.desc())) == 0
    T.assert_same_bits(dev.fetch(p_doubled, like), want.storage, "elementwise operator on a pending result")
    dev.release()


def test_long_runs_wrap_the_table_ring(dev):
    """30 000 products in runs of 500 with a synchronize only at the end: the tables of the grouped launches (12 KB each)
    wrap around the 1 MB ring several times while earlier launches may still be queued."""
    rng = np.random.default_rng(9400)
    dtype, S = O.BF16, 64
    a = [T.contiguous_tensor(rng, dtype, [S, S], lo=-0.5, hi=0.5) for _ in range(8)]
    da = [dev.put(t)[1] for t in a]
    results = []
    for lap in range(60):
        for i in range(500):
            if lap % 10 == 0 and i < 8:
                results.append((device_matmul(dev, da[i], da[(i + lap) % 8], [S, S], dtype), i, (i + lap) % 8))
            else:
                po, _ = device_matmul(dev, da[i % 8], da[(i * 3) % 8], [S, S], dtype)
                dev.free(po)
        dev.dev.call("flush")
    for (po, out), i, j in results:
        exact, scale = exact_product(a[i], a[j])
        got = O.to_float64(dev.fetch(po, out.storage), dtype)
        G.assert_close_to_wide(got, exact, 1e-5 * scale + 2.0 ** -8 * np.abs(exact) + 1e-30, 1.0, f"product {i} x {j} after wrapping")
    dev.release()
