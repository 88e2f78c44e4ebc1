"""The accuracy oracles of the float parity tests -- cpuref_sum_wide, cpuref_reduce_to_wide, cpuref_matmul_wide and
the ulp comparison cpuref_ulp_hist_f32 -- against what the mathematics fixes: math.fsum / float64 numpy over the
logical contents of contiguous, transposed, sliced, offset and stride-0 views, every destination shape a caller may
hand to reduceTo (Targets/AIXLib/aixDeviceCPU.cpp:440-453, 627-649), integers stored as floats (exact in any order),
the reference's own sum / reduceTo on such inputs, and hand-built pairs of floats for the ulp rule."""
import ctypes as C
import math

import numpy as np
import pytest

import aixtest as T
from oracle import cpuref as O

CPU = O.lib()
REF = O.ref_lib()

FLOATS = [O.F64, O.F32, O.F16, O.BF16]


def reduced_shapes(rng, shape):
    """Destination shapes reduceTo accepts for a source shape: keep-dim masks, all ones, leading dims dropped."""
    rank = len(shape)
    outs = []
    for _ in range(3):
        mask = [bool(rng.integers(0, 2)) for _ in shape]
        outs.append([1 if m else e for e, m in zip(shape, mask)])
    outs.append([1] * rank)
    k = int(rng.integers(0, rank))
    outs.append(shape[k:])
    outs.append([1 if i % 2 else e for i, e in enumerate(shape[k:])])
    outs.append([])
    return outs


def numpy_reduce(values, dshape):
    """Sum of a float64 array over every dim where the right-aligned destination has extent 1 or no dim at all."""
    rank = values.ndim
    padded = [1] * (rank - len(dshape)) + list(dshape)
    axes = tuple(i for i, (s, d) in enumerate(zip(values.shape, padded)) if d == 1 and s != 1)
    out = values.sum(axis=axes, keepdims=True) if axes else values
    return out.reshape(-1)


def wide_sum(t):
    s, sa = C.c_double(0), C.c_double(0)
    assert CPU.sum_wide(C.byref(t.desc()), C.byref(s), C.byref(sa)) == 0
    return s.value, sa.value


def wide_reduce(src, dshape):
    like = T.empty(src.dtype, dshape)
    n = max(1, O.numel(dshape))
    got, mag = np.zeros(n), np.zeros(n)
    assert CPU.reduce_to_wide(C.byref(src.desc()), C.byref(like.desc()), got.ctypes.data, mag.ctypes.data) == 0
    return got, mag


@pytest.mark.parametrize("dtype", FLOATS, ids=lambda d: O.DTYPE_NAMES[d])
@pytest.mark.parametrize("kind", T.VIEW_KINDS)
def test_sum_wide_is_the_exact_sum_of_the_logical_contents(dtype, kind):
    rng = np.random.default_rng(910 + 10 * dtype + T.VIEW_KINDS.index(kind))
    for trial in range(12):
        shape = T.random_shape(rng, max_rank=4, max_numel=3000, max_extent=12)
        t = T.view_tensor(rng, dtype, shape, kind, lo=-4, hi=4)
        vals = t.values().reshape(-1)
        s, sa = wide_sum(t)
        exact, exact_abs = math.fsum(vals), math.fsum(np.abs(vals))
        # a long double accumulation of n doubles is within n * 2^-64 * sum|x| of the truth
        tol = vals.size * 2.0 ** -60 * exact_abs + 1e-300
        assert abs(s - exact) <= tol, (shape, kind, s, exact)
        assert abs(sa - exact_abs) <= tol, (shape, kind, sa, exact_abs)


@pytest.mark.parametrize("dtype", FLOATS, ids=lambda d: O.DTYPE_NAMES[d])
def test_wide_oracles_are_exact_on_integers_stored_as_floats(dtype):
    """Small integers add exactly in every order and type, so sum_wide, reduce_to_wide, numpy and the reference's
    own sequential sum / reduceTo must all give the same integers."""
    rng = np.random.default_rng(77 + dtype)
    for kind in T.VIEW_KINDS:
        for trial in range(6):
            shape = T.random_shape(rng, max_rank=4, max_numel=200, max_extent=6)
            t = T.view_tensor(rng, dtype, shape, kind)
            ints = rng.integers(-3, 4, size=t.storage.size).astype(np.float64)
            t.storage[:] = O.to_storage(ints, dtype)
            vals = t.values()
            s, sa = wide_sum(t)
            assert s == vals.sum() and sa == np.abs(vals).sum(), (shape, kind)
            if REF is not None:
                out = T.empty(dtype, [])
                assert REF.sum(C.byref(t.desc()), C.byref(out.desc())) == 0
                assert O.to_float64(out.storage, dtype)[0] == s, (shape, kind)
            for dshape in reduced_shapes(rng, shape):
                got, mag = wide_reduce(t, dshape)
                assert np.array_equal(got, numpy_reduce(vals, dshape)), (shape, dshape, kind)
                assert np.array_equal(mag, numpy_reduce(np.abs(vals), dshape)), (shape, dshape, kind)
                if REF is not None:
                    dst = T.empty(dtype, dshape)
                    assert REF.reduce_to(C.byref(t.desc()), C.byref(dst.desc())) == 0
                    assert np.array_equal(O.to_float64(dst.storage, dtype), got), (shape, dshape, kind)


@pytest.mark.parametrize("dtype", FLOATS, ids=lambda d: O.DTYPE_NAMES[d])
def test_reduce_to_wide_against_float64_numpy(dtype):
    rng = np.random.default_rng(4100 + dtype)
    for trial in range(20):
        shape = T.random_shape(rng, max_rank=5, max_numel=4000, max_extent=7)
        kind = T.VIEW_KINDS[trial % len(T.VIEW_KINDS)]
        src = T.view_tensor(rng, dtype, shape, kind, lo=-2, hi=2)
        vals = src.values()
        for dshape in reduced_shapes(rng, shape):
            got, mag = wide_reduce(src, dshape)
            want, want_mag = numpy_reduce(vals, dshape), numpy_reduce(np.abs(vals), dshape)
            assert got.shape == want.shape
            tol = 1e-13 * want_mag + 1e-300
            assert np.all(np.abs(got - want) <= tol), (shape, dshape, kind)
            assert np.all(np.abs(mag - want_mag) <= tol), (shape, dshape, kind)


def test_reduce_to_wide_adds_into_its_output():
    """Like reduceTo itself the wide variant accumulates: a second call doubles the result."""
    rng = np.random.default_rng(3)
    src = T.contiguous_tensor(rng, O.F32, [5, 7])
    like = T.empty(O.F32, [5, 1])
    got, mag = np.zeros(5), np.zeros(5)
    for _ in range(2):
        assert CPU.reduce_to_wide(C.byref(src.desc()), C.byref(like.desc()), got.ctypes.data, mag.ctypes.data) == 0
    assert np.allclose(got, 2 * src.values().sum(axis=1), rtol=1e-15)
    assert np.allclose(mag, 2 * np.abs(src.values()).sum(axis=1), rtol=1e-15)


@pytest.mark.parametrize("dtype", FLOATS, ids=lambda d: O.DTYPE_NAMES[d])
def test_matmul_wide_against_float64_numpy_on_views(dtype):
    rng = np.random.default_rng(620 + dtype)
    for kind_a in ("contig", "transposed", "sliced", "offset"):
        for kind_b in ("contig", "transposed", "sliced", "broadcast"):
            m, k, n = (int(rng.integers(1, 20)) for _ in range(3))
            a = T.view_tensor(rng, dtype, [m, k], kind_a)
            b = T.view_tensor(rng, dtype, [k, n], kind_b)
            got, mag = np.zeros(m * n), np.zeros(m * n)
            assert CPU.matmul_wide(C.byref(a.desc()), C.byref(b.desc()), got.ctypes.data, mag.ctypes.data, 2) == 0
            want, want_mag = a.values() @ b.values(), np.abs(a.values()) @ np.abs(b.values())
            assert np.all(np.abs(got - want.reshape(-1)) <= 1e-13 * want_mag.reshape(-1) + 1e-300), (kind_a, kind_b)
            assert np.all(np.abs(mag - want_mag.reshape(-1)) <= 1e-13 * want_mag.reshape(-1) + 1e-300), (kind_a, kind_b)
    # integers: exact, and a transposed operand must not come out as the untransposed product
    a = T.HostTensor(np.arange(6, dtype=np.float32), O.F32, [2, 3])
    bt = T.HostTensor(np.arange(12, dtype=np.float32), O.F32, [3, 4], [1, 3])       # the transpose of a dense [4, 3]
    got = np.zeros(8)
    assert CPU.matmul_wide(C.byref(a.desc()), C.byref(bt.desc()), got.ctypes.data, None, 1) == 0
    assert np.array_equal(got.reshape(2, 4), np.arange(6.).reshape(2, 3) @ np.arange(12.).reshape(4, 3).T)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.F32], ids=lambda d: O.DTYPE_NAMES[d])
def test_matmul_stack_wide_is_the_exact_product_rounded_once(dtype):
    """cpuref_matmul_stack_wide = float64 numpy products of the logical contents, rounded once to the element type, for
    2-D operands and for stacks whose leading dims are permuted or broadcast views (results dense); a case where the
    reference's running sum in the element type visibly differs (256 terms of 1/256 + 1: bf16 stalls at 1 after the first
    addition, the exact sum is 2) pins that the sum is NOT kept in the element type."""
    rng = np.random.default_rng(640 + dtype)
    for lead in ([], [3], [2, 3]):
        for kind_a, kind_b in (("contig", "contig"), ("transposed", "contig"), ("sliced", "transposed"), ("contig", "broadcast")):
            m, k, n = (int(rng.integers(1, 12)) for _ in range(3))
            a = T.view_tensor(rng, dtype, lead + [m, k], kind_a)
            b = T.view_tensor(rng, dtype, lead + [k, n], kind_b)
            out = T.empty(dtype, lead + [m, n])
            assert CPU.matmul_stack_wide(C.byref(a.desc()), C.byref(b.desc()), C.byref(out.desc()), 2) == 0
            want = O.to_storage(np.matmul(a.values(), b.values()).reshape(-1), dtype)
            # (float64 numpy adds in another order than the oracle: the two exact sums may round to neighbouring values at a tie)
            assert T.ulp_distance(out.storage, want, dtype) <= 1, (lead, kind_a, kind_b)
    if dtype != O.F32:
        a = T.HostTensor(O.to_storage(np.array([1.0] + [1.0 / 256] * 256), dtype), dtype, [1, 257])
        b = T.HostTensor(O.to_storage(np.ones(257), dtype), dtype, [257, 1])
        wide, literal = T.empty(dtype, [1, 1]), T.empty(dtype, [1, 1])
        assert CPU.matmul_stack_wide(C.byref(a.desc()), C.byref(b.desc()), C.byref(wide.desc()), 1) == 0
        assert CPU.matmul(C.byref(a.desc()), C.byref(b.desc()), C.byref(literal.desc())) == 0
        assert O.to_float64(wide.storage, dtype)[0] == 2.0
        if dtype == O.BF16:
            assert O.to_float64(literal.storage, dtype)[0] == 1.0          # the CPU device's own sum never leaves 1


def f32_from_bits(*bits):
    return np.array(bits, dtype=np.uint32).view(np.float32)


def test_ulp_helper_on_hand_built_pairs():
    """The <= 2 ulp rule itself: distance = number of representable floats between the two values."""
    one = np.float32(1.0)
    up1, up2 = np.nextafter(one, np.float32(2)), np.nextafter(np.nextafter(one, np.float32(2)), np.float32(2))
    tiny = f32_from_bits(0x00000001)[0]                  # smallest positive subnormal
    cases = [
        (one, one, 0), (one, up1, 1), (up1, one, 1), (one, up2, 2),
        (np.float32(0.0), np.float32(-0.0), 0),         # +0 and -0 are the same point
        (tiny, -tiny, 2),                               # adjacent to zero on either side: two steps apart
        (np.float32(0.0), tiny, 1), (np.float32(-0.0), tiny, 1),
        (np.float32(np.finfo(np.float32).max), np.float32(np.inf), 1),
        (np.float32(2.0), np.nextafter(np.float32(2.0), np.float32(0)), 1),          # across a power of two
        (np.float32(-1.0), np.nextafter(np.float32(-1.0), np.float32(-2)), 1),
    ]
    for x, y, want in cases:
        worst, hist = O.ulp_hist_f32(np.array([x], np.float32), np.array([y], np.float32), nbins=8)
        assert worst == want, (x, y, worst, want)
        assert hist[min(want, 7)] == 1 and hist.sum() == 1
    nan = np.float32(np.nan)
    other_nan = f32_from_bits(0xFFC12345)[0]
    assert O.ulp_hist_f32(np.array([nan]), np.array([other_nan]), nbins=8)[0] == 0      # NaN matches any NaN
    for x, y in ((nan, one), (one, nan), (nan, np.float32(np.inf))):
        worst, hist = O.ulp_hist_f32(np.array([x], np.float32), np.array([y], np.float32), nbins=8)
        assert worst == 7 and hist[7] == 1              # NaN against a number: the overflow bin, never "close"
    # a histogram over many pairs: k steps along the float line land in bin k
    base = np.linspace(-3, 3, 1001).astype(np.float32)
    bits = base.view(np.int32)
    for k in (0, 1, 2, 5):
        moved = np.where(base >= 0, bits + k, bits - k).astype(np.int32).view(np.float32)   # away from zero
        worst, hist = O.ulp_hist_f32(base, moved, nbins=16)
        assert worst == k and hist[k] == base.size
    # the largest possible distance does not overflow
    worst, _ = O.ulp_hist_f32(np.array([-np.inf], np.float32), np.array([np.inf], np.float32), nbins=4)
    assert worst == 2 * 0x7F800000
