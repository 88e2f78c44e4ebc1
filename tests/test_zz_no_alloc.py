"""The entry point that allocates nothing (aixk_reduce_all_noalloc: partial results in a static device array) against
the entry point it is a variant of (aixk_reduce_all), through the C ABI: bit-identical results on two calls in a row,
the second with a smaller input, so that what the first call left in the shared array cannot leak into the second.
Bar: bit-exact for every kind and element type (both run the same kernels with the same launch shape)."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import gpuharness as G
from aix_amd import kernels as K
from oracle import cpuref as O

pytestmark = pytest.mark.gpu
NAMES = O.DTYPE_NAMES
KINDS = [(K.SUM, "sum"), (K.MAX, "max"), (K.ARGMAX, "argmax"), (K.ARGMAX_ONEHOT, "argmax_onehot")]


@pytest.fixture(scope="module")
def gpu():
    g = G.Gpu()
    yield g
    g.close()
    g.ctx.close()


def both_entry_points(gpu, kind, src):
    """Runs the pooled-scratch and the static-scratch entry point on the same device buffer; returns both results."""
    _, ds = gpu.put(src)
    onehot = kind == K.ARGMAX_ONEHOT
    odt = src.dtype if kind in (K.SUM, K.MAX) else O.I32
    like = T.empty(odt, src.shape if onehot else [], fill=5)
    p1, d1 = gpu.put(like)
    p2, d2 = gpu.put(like)
    G.run_gpu(gpu, "aixk_reduce_all", kind, G.ref(ds), G.ref(d1))
    G.run_gpu(gpu, "aixk_reduce_all_noalloc", kind, G.ref(ds), G.ref(d2))
    return gpu.fetch(p1, like.storage), gpu.fetch(p2, like.storage)


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: NAMES[d])
def test_two_calls_in_a_row_match_the_pooled_entry_point(gpu, dtype):
    rng = np.random.default_rng(600 + dtype)
    # first a source that fills thousands of workgroups' partials, then smaller ones (fewer partials than the array
    # still holds from the call before), then a strided view
    sizes = [(3_000_017,), (70_001,), (513,), (1,)]
    for kind, kname in KINDS:
        for shape in sizes:
            src = T.contiguous_tensor(rng, dtype, list(shape), int_span=100)
            want, got = both_entry_points(gpu, kind, src)
            T.assert_same_bits_nan_ok(got, want, src.dtype if kind in (K.SUM, K.MAX) else O.I32, f"{kname} {NAMES[dtype]} {shape}")
            gpu.release()
        src = T.view_tensor(rng, dtype, [301, 257], "transposed", int_span=100)
        want, got = both_entry_points(gpu, kind, src)
        T.assert_same_bits_nan_ok(got, want, src.dtype if kind in (K.SUM, K.MAX) else O.I32, f"{kname} {NAMES[dtype]} transposed")
        gpu.release()


def test_against_the_oracle_and_numpy(gpu):
    """Not only equal to the other entry point: right. f32 sum within 1e-5 x sum|x| of the exact sum, max and argmax
    bit-exact (first maximum wins)."""
    rng = np.random.default_rng(9)
    cpu = O.lib()
    for n in (2_000_003, 4099):
        x = T.contiguous_tensor(rng, O.F32, [n])
        x.storage[[n // 3, n // 2]] = 7.5                                # two equal maxima: the lower index wins
        _, ds = gpu.put(x)
        for kind, odt in ((K.SUM, O.F32), (K.MAX, O.F32), (K.ARGMAX, O.I32)):
            out = T.empty(odt, [])
            po, do = gpu.put(out)
            G.run_gpu(gpu, "aixk_reduce_all_noalloc", kind, G.ref(ds), G.ref(do))
            got = gpu.fetch(po, out.storage)[0]
            if kind == K.SUM:
                s, sa = C.c_double(), C.c_double()
                assert cpu.sum_wide(C.byref(x.desc()), C.byref(s), C.byref(sa)) == 0
                assert abs(float(got) - s.value) <= 1e-5 * sa.value
            elif kind == K.MAX:
                assert got == np.float32(7.5)
            else:
                assert got == n // 3
        gpu.release()


def test_sources_beyond_the_limit_are_refused(gpu):
    """More than 2^31 elements: status 1 and a message, nothing launched (the descriptor is never dereferenced)."""
    p = gpu.raw(256)
    d = K.Tensor()
    d.data, d.dtype, d.rank, d.offset, d.size = p, O.U8, 1, 0, 2 ** 31 + 1
    d.shape[0], d.strides[0] = 2 ** 31 + 1, 1
    out = T.empty(O.U8, [])
    _, do = gpu.put(out)
    rc = gpu.ctx.lib.aixk_reduce_all_noalloc(gpu.ctx.handle, K.SUM, G.ref(d), G.ref(do))
    assert rc == 1
    assert b"at most" in gpu.ctx.lib.aixk_last_error()
    gpu.release()
