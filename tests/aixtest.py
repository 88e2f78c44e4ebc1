"""Shared helpers for the parity tests: host tensors with arbitrary views, seeded data,
and comparison rules (bit-exact for integers and exact float ops, ulp / relative bounds
elsewhere)."""
import numpy as np

from oracle import cpuref as O

FLOAT_DTYPES = [O.F64, O.F32, O.F16, O.BF16]
INT_DTYPES = [O.I64, O.I32, O.I16, O.I8, O.U8]
ALL_DTYPES = FLOAT_DTYPES + INT_DTYPES


class HostTensor:
    """A view (dtype, shape, element strides, element offset) over a 1-D numpy storage."""

    def __init__(self, storage, dtype, shape, strides=None, offset=0):
        self.storage = np.ascontiguousarray(storage).reshape(-1)
        assert self.storage.dtype == np.dtype(O.NP_STORAGE[dtype]), (self.storage.dtype, dtype)
        self.dtype = dtype
        self.shape = list(shape)
        self.strides = O.row_major(self.shape) if strides is None else list(strides)
        self.offset = offset
        self.size = O.numel(self.shape)
        if self.size:
            last = offset + sum((e - 1) * s for e, s in zip(self.shape, self.strides))
            assert last < self.storage.size, "view exceeds storage"

    def desc(self, ptr=None):
        return O.make_desc(self.storage.ctypes.data if ptr is None else ptr, self.dtype,
                           self.shape, self.strides, self.offset)

    def gather(self):
        """Logical contents as a contiguous numpy array of the storage type."""
        item = self.storage.itemsize
        v = np.lib.stride_tricks.as_strided(self.storage[self.offset:], shape=self.shape,
                                            strides=[s * item for s in self.strides], writeable=False)
        return np.array(v)

    def values(self):
        """Logical contents as float64 (bf16 decoded)."""
        return O.to_float64(self.gather(), self.dtype)

    def clone(self):
        return HostTensor(self.storage.copy(), self.dtype, self.shape, self.strides, self.offset)

    @property
    def is_contiguous(self):
        return self.strides == O.row_major(self.shape)


def random_values(rng, n, dtype, lo=-1.0, hi=1.0, int_span=None):
    """Storage array of n seeded values of an element type."""
    if dtype in FLOAT_DTYPES:
        return O.to_storage(rng.uniform(lo, hi, size=n), dtype)
    info = np.iinfo(O.NP_STORAGE[dtype])
    if int_span is None:
        int_span = 100 if dtype != O.U8 else 200
    a = max(info.min, -int_span)
    b = min(info.max, int_span)
    return rng.integers(a, b + 1, size=n).astype(O.NP_STORAGE[dtype])


def empty(dtype, shape, fill=None):
    n = max(1, O.numel(shape))
    st = np.zeros(n, dtype=O.NP_STORAGE[dtype])
    if fill is not None:
        st[:] = fill
    return HostTensor(st, dtype, shape)


def contiguous_tensor(rng, dtype, shape, **kw):
    return HostTensor(random_values(rng, max(1, O.numel(shape)), dtype, **kw), dtype, shape)


def view_tensor(rng, dtype, shape, kind, **kw):
    """A tensor of the given logical shape laid out as `kind`:
       contig | transposed | sliced | broadcast | offset"""
    shape = list(shape)
    rank = len(shape)
    if kind == "contig" or rank == 0:
        return contiguous_tensor(rng, dtype, shape, **kw)
    if kind == "offset":
        off = int(rng.integers(1, 9))
        st = random_values(rng, O.numel(shape) + off, dtype, **kw)
        return HostTensor(st, dtype, shape, None, off)
    if kind == "transposed":
        perm = list(rng.permutation(rank))
        if rank >= 2 and perm == list(range(rank)):
            perm[-1], perm[-2] = perm[-2], perm[-1]
        phys_shape = [shape[p] for p in perm]            # storage order
        phys_strides = O.row_major(phys_shape)
        strides = [0] * rank
        for pos, p in enumerate(perm):
            strides[p] = phys_strides[pos]
        return HostTensor(random_values(rng, O.numel(shape), dtype, **kw), dtype, shape, strides)
    if kind == "sliced":
        steps = [int(rng.integers(1, 3)) for _ in shape]
        starts = [int(rng.integers(0, 3)) for _ in shape]
        big = [st + (e - 1) * sp + 1 + int(rng.integers(0, 2)) for e, sp, st in zip(shape, steps, starts)]
        base = O.row_major(big)
        strides = [b * sp for b, sp in zip(base, steps)]
        offset = sum(b * st for b, st in zip(base, starts))
        return HostTensor(random_values(rng, O.numel(big), dtype, **kw), dtype, shape, strides, offset)
    if kind == "broadcast":
        keep = [bool(rng.integers(0, 2)) for _ in shape]
        if all(keep):
            keep[int(rng.integers(0, rank))] = False
        small = [e if k else 1 for e, k in zip(shape, keep)]
        base = O.row_major(small)
        strides = [b if k else 0 for b, k in zip(base, keep)]
        return HostTensor(random_values(rng, O.numel(small), dtype, **kw), dtype, shape, strides)
    raise ValueError(kind)


VIEW_KINDS = ["contig", "transposed", "sliced", "broadcast", "offset"]


def random_shape(rng, max_rank=4, max_numel=4096, max_extent=9):
    rank = int(rng.integers(1, max_rank + 1))
    while True:
        shape = [int(rng.integers(1, max_extent + 1)) for _ in range(rank)]
        if O.numel(shape) <= max_numel:
            return shape


def assert_same_bits(got, want, what=""):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    g = got.view(np.uint8) if got.dtype.kind != "V" else got
    w = want.view(np.uint8)
    if not np.array_equal(g, w):
        bad = np.flatnonzero(got.reshape(-1) != want.reshape(-1))
        i = int(bad[0]) if bad.size else -1
        raise AssertionError(f"{what}: {bad.size} of {got.size} elements differ; first at {i}: "
                             f"got {got.reshape(-1)[i]!r} want {want.reshape(-1)[i]!r}")


def assert_same_bits_nan_ok(got, want, dtype, what=""):
    """Bit equality except that any NaN matches any NaN (payloads are not part of parity)."""
    if dtype in FLOAT_DTYPES:
        gv = O.to_float64(got, dtype)
        wv = O.to_float64(want, dtype)
        both_nan = np.isnan(gv) & np.isnan(wv)
        g2 = np.where(both_nan, np.zeros_like(np.asarray(got)), np.asarray(got))
        w2 = np.where(both_nan, np.zeros_like(np.asarray(want)), np.asarray(want))
        return assert_same_bits(g2, w2, what)
    return assert_same_bits(got, want, what)


def ulp_distance(got, want, dtype):
    """Max distance in units of the last place of the element type (floats only)."""
    if dtype == O.F32:
        return O.ulp_hist_f32(got, want)[0]
    if dtype == O.F64:
        a = np.asarray(got, dtype=np.float64).view(np.int64).astype(object)
        b = np.asarray(want, dtype=np.float64).view(np.int64).astype(object)
    else:
        a = np.asarray(got).view(np.int16).astype(np.int64)
        b = np.asarray(want).view(np.int16).astype(np.int64)
    a = np.where(a < 0, -(a & (2 ** (63 if dtype == O.F64 else 15) - 1)), a)
    b = np.where(b < 0, -(b & (2 ** (63 if dtype == O.F64 else 15) - 1)), b)
    gv, wv = O.to_float64(got, dtype), O.to_float64(want, dtype)
    nan = np.isnan(gv) | np.isnan(wv)
    d = np.abs(a - b)
    d = np.where(nan, np.where(np.isnan(gv) & np.isnan(wv), 0, 1 << 20), d)
    return int(d.max()) if d.size else 0
