"""The benchmark's own sizes through size-independent properties.

The element-by-element oracle comparisons of test_gpu_kernels.py run at sizes the CPU oracle finishes in
seconds.  Here the kernels run at the sizes the benchmark quotes -- [8192, 8192] f32 for the reductions,
the broadcast add and the transpose copy, 1024^3, 4096^3 and 8192^3 in f32 / bf16 / f16 and the batch of 64 512^3
products for the matmuls -- and are checked with what the mathematics fixes at any size (1024^3 and the batch are
small enough for the exactly accumulated oracle on every element):

  * exact operators (max, argmax, x + v, transpose) against numpy on the same data, bit for bit;
    transpose twice is the identity;
  * sums against float64 sums within 1e-5 * sum|x| (the accumulation order is the implementation's);
  * matmul: C . 1 = A . (B . 1) (a checksum of every element of C, evaluated in float64 from the inputs in
    O(n^2)), 96 randomly chosen entries against float64 dot products, A . I = A exactly -- for every
    operand layout the kernels consume in place.

Everything goes through the C ABI of libaixhip_kernels.so."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import gpuharness as G
from oracle import cpuref as O

pytestmark = pytest.mark.gpu
NAMES = O.DTYPE_NAMES
CPU = O.lib()


@pytest.fixture(scope="module")
def gpu():
    g = G.Gpu()
    yield g
    g.close()
    g.ctx.close()


@pytest.fixture(scope="module")
def big():
    """x [8192, 8192] f32 with many exact ties (quantised to 1/64) and v [8192]."""
    rng = np.random.default_rng(5150)
    x = (np.round(rng.uniform(-1, 1, (8192, 8192)) * 64) / 64).astype(np.float32)
    v = rng.uniform(-1, 1, 8192).astype(np.float32)
    return x, v


def _tensor(arr, dtype, shape, strides=None):
    return T.HostTensor(arr.reshape(-1), dtype, shape, strides)


def test_reductions_at_benchmark_size(gpu, big):
    x, _ = big
    R, Cn = x.shape
    src = _tensor(x, O.F32, [R, Cn])
    _, ds = gpu.put(src)
    abs_rows = np.abs(x, dtype=np.float64).sum(axis=1)

    # sum(1): fill(0) + reduceTo into [R, 1]
    out = T.empty(O.F32, [R, 1], fill=0)
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_reduce_to", 0, G.ref(ds), G.ref(do))
    got = gpu.fetch(po, out.storage).astype(np.float64)
    want = x.sum(axis=1, dtype=np.float64)
    assert np.all(np.abs(got - want) <= 1e-5 * abs_rows + 1e-30), float(np.abs(got - want).max())

    # max(1): lowest + maxTo; exact
    out = T.empty(O.F32, [R, 1], fill=float(np.finfo(np.float32).min))
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_reduce_to", 1, G.ref(ds), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, out.storage), x.max(axis=1), "max(1) at [8192, 8192]")

    # argmax(0): the first maximum of every column (the data is full of ties)
    out = T.empty(O.I32, [1, Cn], fill=-1)
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_argmax_to", 0, G.ref(ds), G.ref(do), 0)
    T.assert_same_bits(gpu.fetch(po, out.storage), x.argmax(axis=0).astype(np.int32), "argmax(0) at [8192, 8192]")

    # sum(): everything into one element
    out = T.empty(O.F32, [1], fill=0)
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_reduce_all", 0, G.ref(ds), G.ref(do))
    got = float(gpu.fetch(po, out.storage)[0])
    want = float(x.sum(dtype=np.float64))
    assert abs(got - want) <= 1e-5 * float(abs_rows.sum()), (got, want)
    gpu.release()


def test_broadcast_add_and_transpose_at_benchmark_size(gpu, big):
    x, v = big
    R, Cn = x.shape
    px, dx = gpu.put(_tensor(x, O.F32, [R, Cn]))
    _, dv = gpu.put(_tensor(v, O.F32, [R, Cn], [0, 1]))              # the row vector read through a stride-0 view
    out = T.empty(O.F32, [R, Cn])
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_binary", O.ADD, G.ref(dx), G.ref(dv), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, out.storage), (x + v[None, :]).reshape(-1), "x + v at [8192, 8192]")

    # x.transpose(0, 1).contiguous(): a gather through the transposed view; twice gives x back
    d_t = G.kdesc(_tensor(x, O.F32, [Cn, R], [1, Cn]), px)             # the transposed view of the device copy of x
    G.run_gpu(gpu, "aixk_contiguous", G.ref(d_t), G.ref(do))
    once = gpu.fetch(po, out.storage)
    T.assert_same_bits(once, np.ascontiguousarray(x.T).reshape(-1), "transpose copy at [8192, 8192]")
    pb, db = gpu.put(T.empty(O.F32, [R, Cn]))
    d_tt = G.kdesc(_tensor(x, O.F32, [R, Cn], [1, R]), po)             # the transposed view of the transposed copy
    G.run_gpu(gpu, "aixk_contiguous", G.ref(d_tt), G.ref(db))
    T.assert_same_bits(gpu.fetch(pb, out.storage), x.reshape(-1), "transpose twice")
    gpu.release()


def _matmul_properties(gpu, dtype, n, layout, rng, tol_rel):
    """A [m, k] . B [k, n] (n: one extent for m = k = n, or (m, k, n)) with A and / or B held transposed in memory
    (layout 'NN', 'NT', 'TN', 'TT': T = the operand is stored as its transpose and read through a transposed view)."""
    m, k, n = (n, n, n) if isinstance(n, int) else n
    scale = 1.0 / np.sqrt(k)
    a_store = O.to_storage(rng.uniform(-scale, scale, m * k), dtype)
    b_store = O.to_storage(rng.uniform(-1, 1, k * n), dtype)
    a_t, b_t = layout[0] == "T", layout[1] == "T"
    # logical A[i, k]: stored row-major, or stored as [k, i] and viewed with strides (1, m)
    A = O.to_float64(a_store, dtype).reshape((k, m) if a_t else (m, k))
    B = O.to_float64(b_store, dtype).reshape((n, k) if b_t else (k, n))
    if a_t:
        A = A.T
    if b_t:
        B = B.T
    ha = T.HostTensor(a_store, dtype, [m, k], [1, m] if a_t else None)
    hb = T.HostTensor(b_store, dtype, [k, n], [1, k] if b_t else None)
    _, da = gpu.put(ha)
    _, db = gpu.put(hb)
    out = T.empty(dtype, [m, n])
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(do))
    Cg = O.to_float64(gpu.fetch(po, out.storage), dtype).reshape(m, n)

    # checksum of every element: C . 1 = A . (B . 1); bound = rounding of the output type on sum_j |C_ij| plus
    # the accumulation bound on |A| . (|B| . 1)
    eps_out = {O.F32: 2.0 ** -24, O.F16: 2.0 ** -11, O.BF16: 2.0 ** -8}[dtype]
    want_rows = A @ B.sum(axis=1)
    mag_rows = np.abs(A) @ np.abs(B).sum(axis=1)
    got_rows = Cg.sum(axis=1)
    bound = eps_out * np.abs(Cg).sum(axis=1) + tol_rel * mag_rows
    bad = np.abs(got_rows - want_rows) > bound
    assert not bad.any(), f"{NAMES[dtype]} {n}^3 {layout}: row checksum off by {float(np.abs(got_rows - want_rows).max())} (bound {float(bound.min())})"
    # the same over columns catches a transposed or permuted result that keeps the row sums
    want_cols = A.sum(axis=0) @ B
    got_cols = Cg.sum(axis=0)
    mag_cols = np.abs(A).sum(axis=0) @ np.abs(B)
    bound = eps_out * np.abs(Cg).sum(axis=0) + tol_rel * mag_cols
    assert np.all(np.abs(got_cols - want_cols) <= bound), f"{NAMES[dtype]} {n}^3 {layout}: column checksum"
    # single entries against float64 dot products
    idx = np.stack([rng.integers(0, m, size=96), rng.integers(0, n, size=96)], axis=1)
    for i, j in idx:
        want = float(A[i, :] @ B[:, j])
        mag = float(np.abs(A[i, :]) @ np.abs(B[:, j]))
        assert abs(Cg[i, j] - want) <= eps_out * abs(want) + tol_rel * mag + 1e-30, (layout, int(i), int(j), Cg[i, j], want)
    gpu.release()


def _rect_properties(gpu, dtype, m, k, n, layout, rng, tol_rel):
    """The same checks for A [m, k] . B [k, n]: row and column checksums of every element of C against float64
    from the inputs in O(mk + kn), and 64 single entries against float64 dot products."""
    a_t, b_t = layout[0] == "T", layout[1] == "T"
    a_store = O.to_storage(rng.uniform(-1, 1, m * k) / np.sqrt(k), dtype)
    b_store = O.to_storage(rng.uniform(-1, 1, k * n), dtype)
    A = O.to_float64(a_store, dtype).reshape((k, m) if a_t else (m, k))
    B = O.to_float64(b_store, dtype).reshape((n, k) if b_t else (k, n))
    A = A.T if a_t else A
    B = B.T if b_t else B
    ha = T.HostTensor(a_store, dtype, [m, k], [1, m] if a_t else None)
    hb = T.HostTensor(b_store, dtype, [k, n], [1, k] if b_t else None)
    _, da = gpu.put(ha)
    _, db = gpu.put(hb)
    out = T.empty(dtype, [m, n])
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(do))
    Cg = O.to_float64(gpu.fetch(po, out.storage), dtype).reshape(m, n)
    eps_out = {O.F32: 2.0 ** -24, O.F16: 2.0 ** -11, O.BF16: 2.0 ** -8}[dtype]
    what = f"{NAMES[dtype]} [{m},{k}]x[{k},{n}] {layout}"
    got, want, mag = Cg.sum(axis=1), A @ B.sum(axis=1), np.abs(A) @ np.abs(B).sum(axis=1)
    assert np.all(np.abs(got - want) <= eps_out * np.abs(Cg).sum(axis=1) + tol_rel * mag), what + ": row checksum"
    got, want, mag = Cg.sum(axis=0), A.sum(axis=0) @ B, np.abs(A).sum(axis=0) @ np.abs(B)
    assert np.all(np.abs(got - want) <= eps_out * np.abs(Cg).sum(axis=0) + tol_rel * mag), what + ": column checksum"
    for i, j in zip(rng.integers(0, m, 64), rng.integers(0, n, 64)):
        want = float(A[i, :] @ B[:, j])
        assert abs(Cg[i, j] - want) <= eps_out * abs(want) + tol_rel * float(np.abs(A[i, :]) @ np.abs(B[:, j])) + 1e-30, (what, int(i), int(j))
    gpu.release()


@pytest.mark.parametrize("tile", [(2048, 3072), (2048, 2048), (1024, 2048)], ids=["128x128", "128x64", "64x64"])
@pytest.mark.parametrize("layout", ["NN", "NT", "TN", "TT"])
def test_matmul_prefetch_ring_every_remainder(gpu, tile, layout):
    """Interior tiles of the mid-size kernel fetch their operands several K steps ahead through a ring of register stages
    and finish the steps left over after the last whole turn of the ring one step ahead; tiles on a ragged edge take
    bounds-checked loads throughout.  Every number of left-over steps for rings of 2 and 3 stages, with whole tiles only
    and with a ragged last tile row and column next to interior tiles, for each tile size and operand form."""
    m, n = tile
    bk = 64 if tile == (1024, 2048) else 32
    rng = np.random.default_rng(6600 + m + n)
    for steps in (7, 8, 9, 10, 11, 12, 13):
        _rect_properties(gpu, O.BF16, m, steps * bk, n, layout, rng, 1e-5)
    _rect_properties(gpu, O.F16, m - 40, 11 * bk, n - 24, layout, rng, 1e-5)
    _rect_properties(gpu, O.BF16, m - 8, 10 * bk + 8, n, layout, rng, 1e-5)         # K not a whole number of steps: checked loads everywhere


@pytest.mark.parametrize("case", [
    (8192, 768, 768, "NT"), (8192, 768, 768, "NN"), (8192, 3072, 768, "NN"),      # activations x weights: 128 x 128 / 128 x 64 tiles
    (768, 8192, 768, "TN"), (768, 8192, 768, "TT"),                                 # a weight gradient (x^T . dy, both given row-major) and the same with dy transposed: 128 x 128 tiles, K split 6 ways
    (768, 8192, 3072, "TT"), (3072, 8192, 768, "TN"), (768, 8192, 2304, "TT"),      # K split 3 and 2 ways
    (768, 8192, 8192, "TT"),                                                        # the output projection's gradient: K split 2 ways
    (64, 8192, 768, "TN"), (512, 4096, 96, "NN"),                                   # a long K under a result less than a 128 x 128 tile wide: 64 x 64 tiles, K split
], ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}{c[3]}")
def test_matmul_transformer_shapes_bf16(gpu, case):
    """The mid-size products of a d = 768 transformer step at 8192 tokens, at their real shapes: every tile
    size of the mid-size kernel, with and without K splits, operands consumed where they lie."""
    m, k, n, layout = case
    _rect_properties(gpu, O.BF16, m, k, n, layout, np.random.default_rng(6400 + m + n), 1e-5)


@pytest.mark.parametrize("case", [(4096, 784, 2048, "NN"), (2048, 4096, 2048, "TT"), (784, 4096, 2048, "TT"), (2048, 4096, 10, "TN"), (4096, 2048, 2048, "NT")],
                         ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}{c[3]}")
def test_matmul_mlp_shapes_f32(gpu, case):
    """The products of the 784-2048-2048-10 MLP at batch 4096, at their real shapes: the split-plane kernel with
    and without K splits, and the f32 MFMA kernel with K splits for the ten-column weight gradient."""
    m, k, n, layout = case
    _rect_properties(gpu, O.F32, m, k, n, layout, np.random.default_rng(6500 + m + n), 1e-5)


@pytest.mark.parametrize("layout", ["NN", "NT", "TN", "TT"])
@pytest.mark.parametrize("dtype", [O.BF16, O.F16], ids=lambda d: NAMES[d])
def test_matmul_4096_cubed_16bit(gpu, dtype, layout):
    _matmul_properties(gpu, dtype, 4096, layout, np.random.default_rng(6000 + dtype), 1e-5)


# the products of a d = 768 transformer step at 8192 tokens: results of 256-384 tiles (128 x 192 and 192 x 128 tiles where
# the widths are multiples of 192), weight gradients with K = 8192 split over workgroups, the output projection's gradients
TRANSFORMER_PRODUCTS = [((8192, 768, 768), "NN"), ((8192, 768, 768), "NT"), ((8192, 768, 768), "TN"), ((8192, 768, 768), "TT"),
                        ((8192, 3072, 768), "NN"), ((8192, 3072, 768), "NT"), ((8192, 768, 3072), "NN"), ((8192, 768, 3072), "NT"),
                        ((8192, 8192, 768), "NT"), ((768, 8192, 8192), "TN"), ((768, 8192, 768), "TN"), ((768, 8192, 3072), "TN"),
                        ((3072, 8192, 768), "TN"), ((2048, 2048, 2048), "NN"), ((1536, 768, 8192), "NN"), ((768, 8192, 8192), "NN")]


@pytest.mark.parametrize("shape,layout", TRANSFORMER_PRODUCTS, ids=[f"{s[0]}x{s[1]}x{s[2]}-{l}" for s, l in TRANSFORMER_PRODUCTS])
@pytest.mark.parametrize("dtype", [O.BF16, O.F16], ids=lambda d: NAMES[d])
def test_matmul_transformer_shapes(gpu, dtype, shape, layout):
    _matmul_properties(gpu, dtype, shape, layout, np.random.default_rng(6300 + dtype), 1e-5)


@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
def test_matmul_4096_cubed_f32(gpu, layout):
    _matmul_properties(gpu, O.F32, 4096, layout, np.random.default_rng(6100), 1e-5)


def test_matmul_8192_cubed_bf16(gpu):
    _matmul_properties(gpu, O.BF16, 8192, "NN", np.random.default_rng(6200), 1e-5)


@pytest.mark.parametrize("dtype", [O.F32, O.F16], ids=lambda d: NAMES[d])
def test_matmul_8192_cubed_f32_f16(gpu, dtype):
    _matmul_properties(gpu, dtype, 8192, "NN", np.random.default_rng(6210 + dtype), 1e-5)


@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
@pytest.mark.parametrize("dtype", [O.F32, O.BF16, O.F16], ids=lambda d: NAMES[d])
def test_matmul_1024_cubed(gpu, dtype, layout):
    """The smallest size of the sweep, every element: at 1024^3 the exactly accumulated oracle is affordable, so this
    is a full comparison (|err| <= 1e-5 x sum|a||b| plus the rounding of the result type), not a checksum."""
    n = 1024
    rng = np.random.default_rng(6220 + dtype)
    a_t, b_t = layout[0] == "T", layout[1] == "T"
    a = T.HostTensor(O.to_storage(rng.uniform(-1, 1, n * n) / np.sqrt(n), dtype), dtype, [n, n], [1, n] if a_t else None)
    b = T.HostTensor(O.to_storage(rng.uniform(-1, 1, n * n) / np.sqrt(n), dtype), dtype, [n, n], [1, n] if b_t else None)
    _, da = gpu.put(a)
    _, db = gpu.put(b)
    out = T.empty(dtype, [n, n])
    po, do = gpu.put(out)
    G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(db), G.ref(do))
    got = O.to_float64(gpu.fetch(po, out.storage), dtype)
    exact, mag = np.zeros(n * n), np.zeros(n * n)
    assert CPU.matmul_wide(C.byref(a.desc()), C.byref(b.desc()), exact.ctypes.data, mag.ctypes.data, 16) == 0
    eps_out = {O.F32: 2.0 ** -24, O.F16: 2.0 ** -11, O.BF16: 2.0 ** -8}[dtype]
    bad = np.abs(got - exact) > eps_out * np.abs(exact) + 1e-5 * mag + 1e-30
    assert not bad.any(), f"{NAMES[dtype]} 1024^3 {layout}: {int(bad.sum())} elements beyond the bound"
    gpu.release()


def _stack_data(rng, dtype, count, n):
    a = T.HostTensor(O.to_storage(rng.uniform(-1, 1, count * n * n) / np.sqrt(n), dtype), dtype, [count, n, n])
    b = T.HostTensor(O.to_storage(rng.uniform(-1, 1, count * n * n) / np.sqrt(n), dtype), dtype, [count, n, n])
    exact, mag = np.zeros(count * n * n), np.zeros(count * n * n)
    for i in range(count):
        a2 = T.HostTensor(a.storage, dtype, [n, n], None, i * n * n)
        b2 = T.HostTensor(b.storage, dtype, [n, n], None, i * n * n)
        e, m = np.zeros(n * n), np.zeros(n * n)
        assert CPU.matmul_wide(C.byref(a2.desc()), C.byref(b2.desc()), e.ctypes.data, m.ctypes.data, 16) == 0
        exact[i * n * n:(i + 1) * n * n], mag[i * n * n:(i + 1) * n * n] = e, m
    return a, b, exact, mag


def test_matmul_batch_of_64_bf16_both_forms(gpu):
    """[64, 512, 512] x [64, 512, 512] bf16, every element against the exactly accumulated oracle: once as the
    interface has it (64 matmul calls on select(0, i) views, offset != 0, aixCore.hpp:943-976) and once as one call on
    the stacks; the two forms must also agree with each other within the rounding of the result type."""
    count, n, dtype = 64, 512, O.BF16
    a, b, exact, mag = _stack_data(np.random.default_rng(6230), dtype, count, n)
    pa, da = gpu.put(a)
    pb, db = gpu.put(b)
    out = T.empty(dtype, [count, n, n])
    bound = 2.0 ** -8 * np.abs(exact) + 1e-5 * mag + 1e-30
    # 64 calls on views of the stacks
    po, _ = gpu.put(out)
    for i in range(count):
        va = G.kdesc(T.HostTensor(a.storage, dtype, [n, n], None, i * n * n), pa)
        vb = G.kdesc(T.HostTensor(b.storage, dtype, [n, n], None, i * n * n), pb)
        vo = G.kdesc(T.HostTensor(out.storage, dtype, [n, n]), po + i * n * n * 2)
        G.run_gpu(gpu, "aixk_matmul", G.ref(va), G.ref(vb), G.ref(vo))
    per_call = O.to_float64(gpu.fetch(po, out.storage), dtype)
    assert np.all(np.abs(per_call - exact) <= bound), "64 calls on select(0, i) views"
    # one call on the stacks
    po2, do2 = gpu.put(out)
    G.run_gpu(gpu, "aixk_matmul_batched", G.ref(da), G.ref(db), G.ref(do2))
    stacked = O.to_float64(gpu.fetch(po2, out.storage), dtype)
    assert np.all(np.abs(stacked - exact) <= bound), "one call on the [64, 512, 512] stacks"
    assert np.all(np.abs(stacked - per_call) <= 2.0 ** -7 * np.abs(exact) + 2e-5 * mag + 1e-30)
    gpu.release()


@pytest.mark.parametrize("dtype", [O.F32, O.BF16], ids=lambda d: NAMES[d])
def test_matmul_identity_at_4096(gpu, dtype):
    """A . I == A exactly at the benchmark size (every product is a * 1 or a * 0, every sum exact)."""
    n = 4096
    rng = np.random.default_rng(6300 + dtype)
    a = T.HostTensor(O.to_storage(rng.uniform(-1, 1, n * n), dtype), dtype, [n, n])
    eye = T.HostTensor(O.to_storage(np.eye(n).reshape(-1), dtype), dtype, [n, n])
    _, da = gpu.put(a)
    _, de = gpu.put(eye)
    po, do = gpu.put(T.empty(dtype, [n, n]))
    G.run_gpu(gpu, "aixk_matmul", G.ref(da), G.ref(de), G.ref(do))
    T.assert_same_bits(gpu.fetch(po, a.storage), a.storage, f"A.I {NAMES[dtype]} at 4096")
    gpu.release()
