"""Random programs over a small pool of buffers, bit for bit against a sequential model.

Small 16-bit products, sliceSet calls and recorded elementwise operators are not enqueued when they are called: products
wait in groups by shape and layout, copies in a list, operators in the planner's window, and each leaves when something
needs it -- a group of products alone, without the other groups (DeviceHIP::issuePending).  Every buffer of the pool is
operand and destination in turn, so the programs are full of read-after-write, write-after-read and write-after-write
hazards between what waits in one place and what is called next; blocks are freed and reallocated while products that
use them wait.  The data are small integers: every product and sum is exact in f32 and rounds to bf16 once, the same
way on any device and in any summation order, so the check is bit equality with a model that runs the calls one after
the other (the order the interface promises, Targets/AIXLib/aixDevice.hpp:30-84)."""
import numpy as np
import pytest

import aixtest as T
import devharness as H
from oracle import cpuref as O

pytestmark = pytest.mark.gpu
N, POOL, ROWS = 64, 10, 3
LIMIT = float(2 ** 20)            # every exact product sum stays below: far inside f32's 24 bits


@pytest.fixture(scope="module")
def dev():
    d = H.Dev()
    yield d
    d.close()


def rounded(x):
    """float64 values rounded to bf16 and widened again"""
    return O.to_float64(O.to_storage(np.asarray(x, np.float64).reshape(-1), O.BF16), O.BF16).reshape(np.shape(x))


def fresh(rng):
    return rng.integers(-1, 2, size=(N, N)).astype(np.float64)


class Pool:
    def __init__(self, dev, rng):
        self.dev, self.rng = dev, rng
        self.model = [fresh(rng) for _ in range(POOL)]
        self.ptr = [None] * POOL
        for i in range(POOL):
            self.ptr[i] = dev.raw(N * N * 2)
            self.upload(i)
        self.row_model = [np.zeros((1, N)) for _ in range(ROWS)]
        self.row_ptr = [dev.raw(N * 2) for _ in range(ROWS)]
        for r in range(ROWS):
            dev.dev.from_host(self.row_ptr[r], O.to_storage(self.row_model[r].reshape(-1), O.BF16))

    def row(self, r, spread=False):
        """the [1, N] row buffer, or its rows-times broadcast view"""
        host = T.HostTensor(np.zeros(N, np.uint16), O.BF16, [N, N] if spread else [1, N], [0, 1] if spread else [N, 1])
        return H.kdesc(host, self.row_ptr[r])

    def upload(self, i):
        self.dev.dev.from_host(self.ptr[i], O.to_storage(self.model[i].reshape(-1), O.BF16))

    def whole(self, i):
        return H.kdesc(T.HostTensor(np.zeros(N * N, np.uint16), O.BF16, [N, N]), self.ptr[i])

    def transposed(self, i):
        return H.kdesc(T.HostTensor(np.zeros(N * N, np.uint16), O.BF16, [N, N], [1, N]), self.ptr[i])

    def half(self, i):
        return H.kdesc(T.HostTensor(np.zeros(N * N, np.uint16), O.BF16, [N // 2, N]), self.ptr[i])

    def top(self, i):
        return float(np.abs(self.model[i]).max())

    def check(self, i, what):
        got = self.dev.fetch(self.ptr[i], np.zeros(N * N, np.uint16))
        T.assert_same_bits(got, O.to_storage(self.model[i].reshape(-1), O.BF16), what)


def run_program(dev, seed, steps):
    rng = np.random.default_rng(seed)
    pool = Pool(dev, rng)
    call = dev.dev.call
    trace = []
    for step in range(steps):
        kind = rng.choice(["mm", "mmT", "mmTT", "add", "transpose", "slice", "fill", "reset", "realloc", "flush", "check", "colsum", "rowadd"],
                          p=[0.20, 0.12, 0.08, 0.12, 0.07, 0.10, 0.05, 0.05, 0.05, 0.03, 0.03, 0.05, 0.05])
        a, b, d = (int(x) for x in rng.choice(POOL, size=3, replace=False))
        trace.append((kind, a, b, d))
        if kind in ("mm", "mmT", "mmTT"):
            if N * pool.top(a) * pool.top(b) >= LIMIT:            # keep the arithmetic exact: one operand starts afresh
                big = a if pool.top(a) >= pool.top(b) else b
                pool.model[big] = fresh(rng)
                pool.upload(big)
            left = pool.model[a].T if kind != "mm" else pool.model[a]
            right = pool.model[b].T if kind == "mmTT" else pool.model[b]
            pool.model[d] = rounded(left @ right)
            call("matmul", H.ref(pool.transposed(a) if kind != "mm" else pool.whole(a)), H.ref(pool.transposed(b) if kind == "mmTT" else pool.whole(b)),
                 H.ref(pool.whole(d)))
        elif kind == "add":
            into = d if rng.random() < 0.6 else a                  # also in place
            pool.model[into] = rounded(pool.model[a] + pool.model[b])
            call("add", H.ref(pool.whole(a)), H.ref(pool.whole(b)), H.ref(pool.whole(into)))
        elif kind == "transpose":
            pool.model[d] = pool.model[a].T.copy()
            call("transpose", H.ref(pool.whole(a)), H.ref(pool.whole(d)), 0, 1)
        elif kind == "slice":
            lo = int(rng.choice([0, N // 2]))
            pool.model[d][lo:lo + N // 2, :] = pool.model[a][:N // 2, :]
            call("slice_set", H.ref(pool.half(a)), H.ref(pool.whole(d)), 0, lo, lo + N // 2, 1)
        elif kind == "fill":
            value = np.array([float(rng.integers(-2, 3))], np.float32)
            pool.model[d][:] = value[0]
            call("fill", value.ctypes.data, O.F32, H.ref(pool.whole(d)))
        elif kind == "reset":
            pool.model[d] = fresh(rng)
            pool.upload(d)
        elif kind == "realloc":                                    # its block goes while products that use it may still wait
            dev.free(pool.ptr[d])
            pool.ptr[d] = dev.raw(N * N * 2)
            pool.model[d] = fresh(rng)
            pool.upload(d)
        elif kind == "flush":
            dev.dev.flush()
        elif kind == "colsum":                                     # fill(0) + reduceTo, as sum(0) issues them: the sums wait in a list of their own
            if N * pool.top(a) > 256:                              # (the CPU device adds in bf16: exact only while the sums are)
                pool.model[a] = fresh(rng)
                pool.upload(a)
            r = int(rng.integers(ROWS))
            pool.row_model[r] = rounded(pool.model[a].sum(axis=0, keepdims=True))
            zero = np.zeros(1, np.float32)
            call("fill", zero.ctypes.data, O.F32, H.ref(pool.row(r)))
            call("reduce_to", H.ref(pool.whole(a)), H.ref(pool.row(r)))
        elif kind == "rowadd":                                     # a broadcast operand that a waiting column sum may still have to write
            r = int(rng.integers(ROWS))
            pool.model[d] = rounded(pool.model[a] + pool.row_model[r])
            call("add", H.ref(pool.whole(a)), H.ref(pool.row(r, spread=True)), H.ref(pool.whole(d)))
        else:
            pool.check(d, f"seed {seed}, buffer {d} after step {step}: {trace[-12:]}")
    for i in range(POOL):
        pool.check(i, f"seed {seed}, buffer {i} at the end; last calls {trace[-12:]}")
    dev.release()


@pytest.mark.parametrize("seed", range(24))
def test_random_programs_equal_the_calls_one_after_the_other(dev, seed):
    run_program(dev, 77000 + seed, 400)


def test_the_model_rounds_like_the_device(dev):
    """One product and one sum at the largest magnitudes the programs reach, so that a failure above is a failure of
    ordering and not of the exact-arithmetic assumption."""
    rng = np.random.default_rng(77900)
    pool = Pool(dev, rng)
    pool.model[0] = rounded(rng.integers(-120, 121, size=(N, N)).astype(np.float64))
    pool.model[1] = rounded(rng.integers(-120, 121, size=(N, N)).astype(np.float64))
    pool.upload(0)
    pool.upload(1)
    assert N * pool.top(0) * pool.top(1) < LIMIT
    pool.model[2] = rounded(pool.model[0] @ pool.model[1])
    dev.dev.call("matmul", H.ref(pool.whole(0)), H.ref(pool.whole(1)), H.ref(pool.whole(2)))
    pool.model[3] = rounded(pool.model[2] + pool.model[2].T)
    dev.dev.call("transpose", H.ref(pool.whole(2)), H.ref(pool.whole(4)), 0, 1)
    dev.dev.call("add", H.ref(pool.whole(2)), H.ref(pool.whole(4)), H.ref(pool.whole(3)))
    pool.check(2, "a product of integers")
    pool.check(3, "a sum of rounded integers")
    dev.release()
