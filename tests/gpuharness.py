"""GPU-side plumbing for the parity tests: device buffers for HostTensors and comparison rules.

Everything goes through the C ABI of libaixhip_kernels.so (aix_amd.kernels); the oracle is only
ever the checker."""
import ctypes as C

import numpy as np

import aixtest as T
from aix_amd import kernels as K
from oracle import cpuref as O


class Gpu:
    """One context plus the device allocations made for a test; freed on close()."""

    def __init__(self):
        self.ctx = K.Context(0)
        self.live = []

    def close(self):
        self.ctx.sync()
        for p in self.live:
            self.ctx.free(p)
        self.live = []

    def raw(self, nbytes):
        p = self.ctx.alloc(max(nbytes, 1))
        self.live.append(p)
        return p

    def release(self):
        """Free everything allocated so far (between sub-cases of a long test)."""
        self.close()

    def put(self, ht):
        """Upload a HostTensor's storage; returns (device pointer, K.Tensor over it)."""
        p = self.raw(ht.storage.nbytes)
        self.ctx.upload(p, ht.storage)
        return p, kdesc(ht, p)

    def fetch(self, ptr, like):
        out = np.empty_like(like)
        self.ctx.download(out, ptr)
        return out


def kdesc(ht, ptr):
    d = K.Tensor()
    d.data = ptr
    d.dtype = ht.dtype
    d.rank = len(ht.shape)
    d.offset = ht.offset
    d.size = ht.size
    for i, (e, s) in enumerate(zip(ht.shape, ht.strides)):
        d.shape[i] = e
        d.strides[i] = s
    return d


def run_gpu(gpu, fn, *args):
    K.check(getattr(gpu.ctx.lib, fn)(gpu.ctx.handle, *args))


def ref(x):
    return C.byref(x)


# ---- comparison rules ---------------------------------------------------------------------------
EXACT = "exact"


def compare(got, want, dtype, rule, what):
    """rule: EXACT, or an integer = max distance in units of the last place of the element type."""
    if dtype in T.INT_DTYPES or rule == EXACT:
        return T.assert_same_bits_nan_ok(got, want, dtype, what)
    d = T.ulp_distance(got, want, dtype)
    assert d <= rule, f"{what}: {d} ulp apart (allowed {rule})"


def assert_close_to_wide(got_f64, exact, scale, tol, what):
    """|got - exact| <= tol * scale elementwise (scale = sum of |terms| of each result)."""
    got_f64 = np.asarray(got_f64, dtype=np.float64).reshape(-1)
    exact = np.asarray(exact, dtype=np.float64).reshape(-1)
    scale = np.asarray(scale, dtype=np.float64).reshape(-1)
    err = np.abs(got_f64 - exact)
    bound = tol * np.maximum(scale, 1e-300)
    bad = np.flatnonzero(~(err <= bound))
    if bad.size:
        i = int(bad[0])
        raise AssertionError(f"{what}: {bad.size} of {err.size} beyond {tol:g} x scale; first at {i}: "
                             f"got {got_f64[i]!r} exact {exact[i]!r} scale {scale[i]!r}")


class KernelBackend:
    """The golden-case backend over the eager kernel ABI: upload, run, download in place."""
    name = "hip-kernels"

    def __init__(self, gpu):
        self.gpu = gpu

    def _run(self, fn, tensors, pre=(), extra=(), outputs=()):
        ptrs, descs = [], []
        for t in tensors:
            p, d = self.gpu.put(t)
            ptrs.append(p)
            descs.append(d)
        rc = getattr(self.gpu.ctx.lib, fn)(self.gpu.ctx.handle, *pre, *[ref(d) for d in descs], *extra)
        if rc == 0:
            for i in outputs:
                self.gpu.ctx.download(tensors[i].storage, ptrs[i])
        self.gpu.release()
        return rc

    def unary(self, op, a, out):
        return self._run("aixk_unary", [a, out], pre=(op,), outputs=(1,))

    def binary(self, op, a, b, out):
        return self._run("aixk_binary", [a, b, out], pre=(op,), outputs=(2,))

    def copy(self, src, sdt, dst, ddt, n):
        ps, _ = self.gpu.put(src)
        pd, _ = self.gpu.put(dst)
        rc = self.gpu.ctx.lib.aixk_cast(self.gpu.ctx.handle, ps, sdt, pd, ddt, n)
        if rc == 0:
            self.gpu.ctx.download(dst.storage, pd)
        self.gpu.release()
        return rc

    def fill(self, scalar, sdt, out):
        po, do = self.gpu.put(out)
        rc = self.gpu.ctx.lib.aixk_fill(self.gpu.ctx.handle, scalar.ctypes.data, sdt, ref(do))
        if rc == 0:
            self.gpu.ctx.download(out.storage, po)
        self.gpu.release()
        return rc

    def simple(self, name, *tensors, extra=()):
        t = list(tensors)
        table = {
            "argmax": ("aixk_reduce_all", (K.ARGMAX,), (1,)),
            "argmax_indices": ("aixk_reduce_all", (K.ARGMAX_ONEHOT,), (1,)),
            "argmax_to": ("aixk_argmax_to", (0,), (1,)),
            "argmax_indices_to": ("aixk_argmax_to", (1,), (1,)),
            "matmul": ("aixk_matmul", (), (2,)),
            "reduce_to": ("aixk_reduce_to", (K.SUM,), (1,)),
            "max_to": ("aixk_reduce_to", (K.MAX,), (1,)),
            "slice_set": ("aixk_slice_set", (), (1,)),
            "index_select": ("aixk_index_select", (), (1,)),
            "index_add": ("aixk_index_add", (), (1,)),
        }
        fn, pre, outs = table[name]
        return self._run(fn, t, pre=pre, extra=tuple(extra), outputs=outs)
