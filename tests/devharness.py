"""Plumbing for tests of the lazy device (libaixhip.so, include/aixhip.h): device tensors backed by
aixhip_allocate, the golden-case backend, and a tiny recorder that drives the device the way the
AIX front-end does (fresh result allocation per op, temporaries freed before synchronize)."""
import ctypes as C

import numpy as np

import aixtest as T
from aix_amd import device as D
from oracle import cpuref as O


def kdesc(ht, ptr):
    d = D.Tensor()
    d.data = ptr
    d.dtype = ht.dtype
    d.rank = len(ht.shape)
    d.offset = ht.offset
    d.size = ht.size
    for i, (e, s) in enumerate(zip(ht.shape, ht.strides)):
        d.shape[i] = e
        d.strides[i] = s
    return d


class Dev:
    def __init__(self):
        self.dev = D.Device(0)
        self.live = []

    def close(self):
        self.release()
        self.dev.close()

    def release(self):
        for p in self.live:
            self.dev.deallocate(p)
        self.live = []
        self.dev.synchronize()

    def raw(self, nbytes, keep=True):
        p = self.dev.allocate(max(nbytes, 1))
        if keep:
            self.live.append(p)
        return p

    def put(self, ht, keep=True):
        """Device copy of a HostTensor's storage (explicit transfer); returns (ptr, descriptor)."""
        p = self.raw(ht.storage.nbytes, keep)
        self.dev.from_host(p, ht.storage)
        return p, kdesc(ht, p)

    def fetch(self, ptr, like):
        out = np.empty_like(like)
        self.dev.to_host(out, ptr)                # flushes, waits, copies
        return out

    def free(self, ptr):
        if ptr in self.live:
            self.live.remove(ptr)
        self.dev.deallocate(ptr)


def ref(x):
    return C.byref(x)


class DeviceBackend:
    """Golden-case backend over the lazy device ABI."""
    name = "hip-device"

    def __init__(self, dev):
        self.d = dev

    def _run(self, fn, tensors, pre=(), extra=(), outputs=()):
        ptrs, descs = [], []
        for t in tensors:
            p, d = self.d.put(t)
            ptrs.append(p)
            descs.append(d)
        rc = self.d.dev.status(fn, *pre, *[ref(d) for d in descs], *extra)
        if rc == 0:
            for i in outputs:
                self.d.dev.to_host(tensors[i].storage, ptrs[i])
        self.d.release()
        return rc

    def unary(self, op, a, out):
        return self._run(["unary", "sqrt", "sin", "cos", "tanh", "log", "exp"][op], [a, out], outputs=(1,))

    def binary(self, op, a, b, out):
        return self._run(["add", "sub", "mul", "div", "pow"][op], [a, b, out], outputs=(2,))

    def copy(self, src, sdt, dst, ddt, n):
        pd, _ = self.d.put(dst)
        rc = self.d.dev.status("copy", src.storage.ctypes.data, sdt, pd, ddt, n)     # host source, as the front-end passes it
        if rc == 0:
            self.d.dev.to_host(dst.storage, pd)
        self.d.release()
        return rc

    def fill(self, scalar, sdt, out):
        po, do = self.d.put(out)
        rc = self.d.dev.status("fill", scalar.ctypes.data, sdt, ref(do))
        if rc == 0:
            self.d.dev.to_host(out.storage, po)
        self.d.release()
        return rc

    def simple(self, name, *tensors, extra=()):
        outs = {"matmul": (2,)}.get(name, (1,))
        return self._run(name, list(tensors), extra=tuple(extra), outputs=outs)
