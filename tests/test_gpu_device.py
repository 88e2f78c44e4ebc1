"""The lazy, fusing device (DeviceHIP behind include/aixhip.h) against the CPU oracle.

These drive the device the way the AIX front-end does -- a fresh result allocation per operator,
scalars as fills of rank-0 tensors read through stride-0 views, temporaries deallocated before
synchronize() -- and check results, fusion diagnostics, error behaviour and memory handling.
Patterns follow Targets/AIXTests/DeviceTests.cpp (queue tests :3074-3552, fusion tests :1774-1910).
"""
import ctypes as C
import os

import numpy as np
import pytest

import aixtest as T
import devharness as H
import goldens
from aix_amd import device as D
from aix_amd import kernels as K
from oracle import cpuref as O

pytestmark = pytest.mark.gpu
CPU = O.lib()
NAMES = O.DTYPE_NAMES
EPS32 = 2.0 ** -24


@pytest.fixture(scope="module")
def dev():
    d = H.Dev()
    yield d
    d.close()


def set_diag(dev, **kw):
    cfg = dev.dev.fuse_config()
    cfg.diagnostics = 1
    for k, v in kw.items():
        setattr(cfg, k, v)
    dev.dev.set_fuse_config(cfg)


class Recorder:
    """Builds an expression on the device and, op for op, on the oracle."""

    def __init__(self, dev, dtype, shape):
        self.dev, self.dtype, self.shape = dev, dtype, list(shape)
        self.n = O.numel(shape)
        self.temps = []

    def leaf(self, host):
        p, d = self.dev.put(host)
        return {"host": host, "ptr": p, "desc": d}

    def _result(self):
        host = T.empty(self.dtype, self.shape)
        p = self.dev.raw(host.storage.nbytes)
        node = {"host": host, "ptr": p, "desc": H.kdesc(host, p)}
        self.temps.append(node)
        return node

    def binary(self, op, x, y):
        r = self._result()
        assert CPU.binary(op, C.byref(x["host"].desc()), C.byref(y["host"].desc()), C.byref(r["host"].desc())) == 0
        self.dev.dev.call(["add", "sub", "mul", "div", "pow"][op], H.ref(x["desc"]), H.ref(y["desc"]), H.ref(r["desc"]))
        return r

    def unary(self, op, x):
        r = self._result()
        assert CPU.unary(op, C.byref(x["host"].desc()), C.byref(r["host"].desc())) == 0
        self.dev.dev.call(["unary", "sqrt", "sin", "cos", "tanh", "log", "exp"][op], H.ref(x["desc"]), H.ref(r["desc"]))
        return r

    def scalar(self, value):
        """Tensor-level scalar: a rank-0 tensor filled with the value, read through a stride-0 view
        of the full shape (aixCore.hpp:2384-2388)."""
        host0 = T.empty(self.dtype, [])
        v = np.array([value], dtype=np.float32)
        assert CPU.fill(v.ctypes.data, O.F32, C.byref(host0.desc())) == 0
        p = self.dev.raw(host0.storage.nbytes)
        self.dev.dev.call("fill", v.ctypes.data, O.F32, H.ref(H.kdesc(host0, p)))
        view = T.HostTensor(host0.storage, self.dtype, self.shape, [0] * len(self.shape))
        node = {"host": view, "ptr": p, "desc": H.kdesc(view, p)}
        self.temps.append(node)
        return node

    def free_temps(self, keep=()):
        for t in self.temps:
            if not any(t is k for k in keep):
                self.dev.free(t["ptr"])
        self.temps = [t for t in self.temps if any(t is k for k in keep)]


def build_config0(rec, a, b, c):
    """y = tanh(a*b + c) / (1 + exp(-a)) - 0.5*c"""
    t1 = rec.binary(O.MUL, a, b)
    t2 = rec.binary(O.ADD, t1, c)
    t3 = rec.unary(O.TANH, t2)
    t4 = rec.unary(O.NEG, a)
    t5 = rec.unary(O.EXP, t4)
    t6 = rec.binary(O.ADD, rec.scalar(1.0), t5)
    t7 = rec.binary(O.DIV, t3, t6)
    t8 = rec.binary(O.MUL, rec.scalar(0.5), c)
    y = rec.binary(O.SUB, t7, t8)
    return y, t7


@pytest.mark.parametrize("shape", [[1024, 1024], [4096, 4096]], ids=["1024", "benchmark-size"])
def test_config0_chain_is_one_fused_kernel(dev, shape):
    set_diag(dev)
    rng = np.random.default_rng(0)
    rec = Recorder(dev, O.F32, shape)
    a, b, c = (rec.leaf(T.contiguous_tensor(rng, O.F32, shape)) for _ in range(3))
    y, t7 = build_config0(rec, a, b, c)
    rec.free_temps(keep=(y,))
    got = dev.fetch(y["ptr"], y["host"].storage)
    diag = dev.dev.diagnostics()
    assert diag.fusible_subgraphs == 1 and diag.fused_ops == 9 and diag.fallback_ops == 0, diag.subgraph_summary
    assert diag.fills_absorbed == 2 and diag.ops_recorded == 11
    # chain-level bound: tanh and exp may each differ by 2 ulp from the CPU's libm; the quotient
    # carries that relative error and the final subtraction keeps it absolute.
    want = y["host"].storage.astype(np.float64)
    q = np.abs(t7["host"].storage.astype(np.float64))
    err = np.abs(got.astype(np.float64) - want)
    assert np.all(err <= 8 * EPS32 * (q + np.abs(want)) + 1e-30), float(err.max())
    worst, hist = O.ulp_hist_f32(got, y["host"].storage)
    print("config-0 chain ulp histogram vs CPU chain:", worst, hist[:8].tolist())
    dev.release()


@pytest.mark.parametrize("dtype", T.ALL_DTYPES, ids=lambda d: NAMES[d])
def test_random_exact_expressions(dev, dtype):
    """Random DAGs of exact operators (+ - * negate, scalars, broadcast rows, in-place updates) with
    temporaries freed before the flush: must equal the op-by-op CPU evaluation bit for bit."""
    set_diag(dev)
    rng = np.random.default_rng(31000 + dtype)
    for trial in range(12):
        shape = [int(rng.integers(1, 40)), int(rng.integers(1, 70))]
        rec = Recorder(dev, dtype, shape)
        kw = dict(int_span=7) if dtype in T.INT_DTYPES else dict(lo=-2, hi=2)
        nodes = [rec.leaf(T.contiguous_tensor(rng, dtype, shape, **kw)) for _ in range(3)]
        row = T.HostTensor(T.random_values(rng, shape[1], dtype, **kw), dtype, shape, [0, 1])
        col = T.HostTensor(T.random_values(rng, shape[0], dtype, **kw), dtype, shape, [1, 0])
        nodes += [rec.leaf(row), rec.leaf(col)]
        results = []
        for step in range(int(rng.integers(3, 14))):
            kind = rng.integers(0, 10)
            x = nodes[int(rng.integers(0, len(nodes)))]
            y = nodes[int(rng.integers(0, len(nodes)))]
            if kind < 6:
                r = rec.binary(int(rng.choice([O.ADD, O.SUB, O.MUL])), x, y)
            elif kind < 8:
                r = rec.unary(O.NEG, x)
            else:
                r = rec.binary(int(rng.choice([O.ADD, O.MUL])), rec.scalar(float(rng.integers(-3, 4))), x)
            nodes.append(r)
            results.append(r)
            if rng.integers(0, 4) == 0 and results:      # in-place update of an earlier result: r2 = r2 op x
                tgt = results[int(rng.integers(0, len(results)))]
                op = int(rng.choice([O.ADD, O.SUB, O.MUL]))
                assert CPU.binary(op, C.byref(tgt["host"].desc()), C.byref(x["host"].desc()), C.byref(tgt["host"].desc())) == 0
                dev.dev.call(["add", "sub", "mul"][op], H.ref(tgt["desc"]), H.ref(x["desc"]), H.ref(tgt["desc"]))
        keep = [results[-1]] + [r for r in results[:-1] if rng.integers(0, 3) == 0]
        rec.free_temps(keep=keep)
        for r in keep:
            got = dev.fetch(r["ptr"], r["host"].storage)
            T.assert_same_bits_nan_ok(got, r["host"].storage, dtype, f"{NAMES[dtype]} trial {trial} shape {shape}")
        dev.release()


def test_fusion_on_off_same_bits(dev):
    """The fused kernels and the single-operator replay give identical bits (f32, transcendental ops included)."""
    rng = np.random.default_rng(32000)
    shape = [333, 257]
    outs = []
    for fusion in (1, 0):
        set_diag(dev, elementwise_fusion=fusion)
        rec = Recorder(dev, O.F32, shape)
        r2 = np.random.default_rng(1)
        a, b, c = (rec.leaf(T.contiguous_tensor(r2, O.F32, shape)) for _ in range(3))
        y, _ = build_config0(rec, a, b, c)
        z = rec.unary(O.SIN, rec.binary(O.POW, rec.unary(O.EXP, y), rec.scalar(1.5)))
        rec.free_temps(keep=(z,))
        outs.append(dev.fetch(z["ptr"], z["host"].storage))
        diag = dev.dev.diagnostics()
        assert (diag.fusible_subgraphs >= 1) == bool(fusion)
        dev.release()
    T.assert_same_bits_nan_ok(outs[0], outs[1], O.F32, "fused vs single")
    set_diag(dev, elementwise_fusion=1)


def test_kernel_cache_and_scalar_values(dev):
    """Different immediates reuse the compiled kernel (DeviceTests.cpp:1774-1807)."""
    set_diag(dev)
    rng = np.random.default_rng(33000)
    shape = [64, 100]
    h0, m0 = dev.dev.kernel_cache_stats()
    for k, s in enumerate((0.5, 0.25, 4.0)):
        rec = Recorder(dev, O.F32, shape)
        a = rec.leaf(T.contiguous_tensor(rng, O.F32, shape))
        y = rec.binary(O.ADD, rec.unary(O.COS, rec.binary(O.MUL, rec.scalar(s), a)), rec.scalar(s))
        rec.free_temps(keep=(y,))
        got = dev.fetch(y["ptr"], y["host"].storage)
        assert T.ulp_distance(got, y["host"].storage, O.F32) <= 2
        dev.release()
    h1, m1 = dev.dev.kernel_cache_stats()
    assert m1 - m0 == 1 and h1 - h0 == 2, (h0, m0, h1, m1)


def test_pending_work_is_flushed_before_other_operators(dev):
    """Elementwise work recorded before a reduction / matmul / copy must be visible to it."""
    set_diag(dev)
    rng = np.random.default_rng(34000)
    shape = [96, 160]
    rec = Recorder(dev, O.F32, shape)
    a, b = (rec.leaf(T.contiguous_tensor(rng, O.F32, shape)) for _ in range(2))
    t = rec.binary(O.MUL, a, b)                                    # pending
    # sum(t)
    s_host = T.empty(O.F32, [])
    ps = dev.raw(4)
    dev.dev.call("sum", H.ref(t["desc"]), H.ref(H.kdesc(s_host, ps)))
    exact, scale = C.c_double(), C.c_double()
    assert CPU.sum_wide(C.byref(t["host"].desc()), C.byref(exact), C.byref(scale)) == 0
    got = dev.fetch(ps, s_host.storage)
    assert abs(float(got[0]) - exact.value) <= 1e-5 * scale.value
    # matmul(t, t^T view) after an in-place update of t
    assert CPU.binary(O.ADD, C.byref(t["host"].desc()), C.byref(a["host"].desc()), C.byref(t["host"].desc())) == 0
    dev.dev.call("add", H.ref(t["desc"]), H.ref(a["desc"]), H.ref(t["desc"]))
    tT = T.HostTensor(t["host"].storage, O.F32, [160, 96], [1, 160])
    m_host = T.empty(O.F32, [96, 96])
    pm = dev.raw(m_host.storage.nbytes)
    dev.dev.call("matmul", H.ref(t["desc"]), H.ref(H.kdesc(tT, t["ptr"])), H.ref(H.kdesc(m_host, pm)))
    exact_m = np.zeros(96 * 96)
    scale_m = np.zeros(96 * 96)
    assert CPU.matmul_wide(C.byref(t["host"].desc()), C.byref(tT.desc()), exact_m.ctypes.data, scale_m.ctypes.data, 4) == 0
    got = dev.fetch(pm, m_host.storage).astype(np.float64)
    assert np.all(np.abs(got - exact_m) <= 1e-5 * scale_m + 1e-30)
    # reduceTo into a zero-filled destination (fill recorded, then accumulated into)
    d_host = T.empty(O.F32, [1, 160])
    pd = dev.raw(d_host.storage.nbytes)
    zero = np.zeros(1, np.float32)
    dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(H.kdesc(d_host, pd)))
    dev.dev.call("reduce_to", H.ref(t["desc"]), H.ref(H.kdesc(d_host, pd)))
    exact_r = np.zeros(160)
    scale_r = np.zeros(160)
    assert CPU.reduce_to_wide(C.byref(t["host"].desc()), C.byref(d_host.desc()), exact_r.ctypes.data, scale_r.ctypes.data) == 0
    got = dev.fetch(pd, d_host.storage).astype(np.float64)
    assert np.all(np.abs(got - exact_r) <= 1e-5 * scale_r + 1e-30)
    dev.release()


def test_host_operands_and_error_convention(dev):
    rng = np.random.default_rng(35000)
    a = T.contiguous_tensor(rng, O.F32, [50, 20])
    b = T.view_tensor(rng, O.F32, [50, 20], "transposed")
    want = T.empty(O.F32, [50, 20])
    assert CPU.binary(O.ADD, C.byref(a.desc()), C.byref(b.desc()), C.byref(want.desc())) == 0
    # host tensors handed straight to the device as sources (DeviceTests.cpp:209-215)
    out = T.empty(O.F32, [50, 20])
    po = dev.raw(out.storage.nbytes)
    dev.dev.call("add", H.ref(H.kdesc(a, a.storage.ctypes.data)), H.ref(H.kdesc(b, b.storage.ctypes.data)), H.ref(H.kdesc(out, po)))
    T.assert_same_bits(dev.fetch(po, out.storage), want.storage, "host sources")
    # a host result is refused (aixDeviceMetal.cpp:305-306)
    rc = dev.dev.status("add", H.ref(H.kdesc(a, a.storage.ctypes.data)), H.ref(H.kdesc(b, b.storage.ctypes.data)),
                        H.ref(H.kdesc(out, out.storage.ctypes.data)))
    assert rc == 1 and b"result must have GPU memory" in dev.dev.lib.aixhip_last_error()
    # int32-only argmax results (aixDeviceCPU.cpp:1027-1030)
    pa, da = dev.put(a)
    bad = T.empty(O.F32, [])
    pb = dev.raw(4)
    assert dev.dev.status("argmax", H.ref(da), H.ref(H.kdesc(bad, pb))) == 1
    assert b"int32" in dev.dev.lib.aixhip_last_error()
    # freeing memory the device does not own (aixDeviceMetal.cpp:253-254)
    assert dev.dev.lib.aixhip_deallocate(dev.dev.handle, a.storage.ctypes.data) == 1
    # copy into host memory is refused, copy from host memory converts
    u8 = np.zeros(4, np.uint8)
    src = O.to_storage(np.array([-1.0, 0.0, 42.0, 300.0]), O.BF16)
    assert dev.dev.status("copy", src.ctypes.data, O.BF16, u8.ctypes.data, O.U8, 4) == 1
    pd = dev.raw(4)
    dev.dev.call("copy_immediate", src.ctypes.data, O.BF16, pd, O.U8, 4)
    assert dev.fetch(pd, u8).tolist() == [0, 0, 42, 255]          # DeviceTests.cpp:1282-1305
    dev.release()


def test_host_dereference_of_device_memory(dev):
    """allocate() returns memory the host may write and (slowly) read directly, as the AIX
    front-end does for item(), printing and test set-up (DeviceTests.cpp:185-189)."""
    n = 4096
    pa, pb, po = dev.raw(n * 4, keep=True), dev.raw(n * 4, keep=True), dev.raw(n * 4, keep=True)
    a_host = T.empty(O.F32, [n])
    for round_ in range(3):                                        # same addresses, new data each round
        x = np.random.default_rng(round_).uniform(-1, 1, n).astype(np.float32)
        y = np.random.default_rng(100 + round_).uniform(-1, 1, n).astype(np.float32)
        C.memmove(pa, x.ctypes.data, n * 4)                        # direct host stores into device memory
        C.memmove(pb, y.ctypes.data, n * 4)
        dev.dev.call("mul", H.ref(H.kdesc(a_host, pa)), H.ref(H.kdesc(a_host, pb)), H.ref(H.kdesc(a_host, po)))
        dev.dev.synchronize()
        got = np.empty(n, np.float32)
        C.memmove(got.ctypes.data, po, n * 4)                      # direct host loads from device memory
        T.assert_same_bits(got, x * y, f"round {round_}")
    dev.release()


def test_1024_chained_in_place_adds_without_sync(dev):
    """DeviceTests.cpp:3478-3500: 1024 in-place adds on 1 Mi elements, one synchronize at the end."""
    n = 1 << 20
    x = T.HostTensor(np.zeros(n, np.float32), O.F32, [n])
    one = T.HostTensor(np.ones(n, np.float32), O.F32, [n])
    px, dx = dev.put(x)
    p1, d1 = dev.put(one)
    for _ in range(1024):
        dev.dev.call("add", H.ref(dx), H.ref(d1), H.ref(dx))
    got = dev.fetch(px, x.storage)
    assert np.all(got == 1024.0)
    dev.release()


def test_temporaries_are_recycled(dev):
    """A long allocate / compute / free loop without synchronize keeps memory bounded."""
    dev.dev.synchronize()
    dev.dev.call("empty_cache")                              # blocks cached by earlier tests do not count
    rng = np.random.default_rng(36000)
    n = 1 << 18
    a = T.contiguous_tensor(rng, O.F32, [n])
    pa, da = dev.put(a)
    acc = T.HostTensor(np.zeros(n, np.float32), O.F32, [n])
    pacc, dacc = dev.put(acc)
    for it in range(400):
        pt = dev.raw(n * 4, keep=False)
        dt = H.kdesc(acc, pt)
        dev.dev.call("mul", H.ref(da), H.ref(da), H.ref(dt))
        dev.dev.call("add", H.ref(dacc), H.ref(dt), H.ref(dacc))
        dev.dev.deallocate(pt)
        if it % 50 == 49:
            dev.dev.flush()
    got = dev.fetch(pacc, acc.storage)
    want = np.zeros(n, np.float32)
    sq = a.storage * a.storage
    for _ in range(400):
        want += sq
    T.assert_same_bits(got, want, "accumulated squares")
    live, cached = C.c_uint64(), C.c_uint64()
    D.check(dev.dev.lib.aixhip_memory_stats(dev.dev.handle, C.byref(live), C.byref(cached)))
    assert cached.value <= 160 * n * 4, cached.value
    dev.release()


def test_used_temporaries_are_recycled(dev):
    """The same for temporaries that enqueued work really wrote (an eager operator per iteration):
    they come back once the GPU has passed an event, so 1.6 GiB of them hold a few hundred MiB."""
    dev.dev.synchronize()
    dev.dev.call("empty_cache")
    rng = np.random.default_rng(36001)
    rows, cols = 1024, 1024
    a = T.contiguous_tensor(rng, O.F32, [rows, cols])
    pa, da = dev.put(a)
    acc = T.HostTensor(np.zeros(rows * cols, np.float32), O.F32, [cols, rows])
    pacc, dacc = dev.put(acc)
    loops = 400
    for it in range(loops):
        pt = dev.raw(rows * cols * 4, keep=False)
        dt = H.kdesc(acc, pt)
        dev.dev.call("transpose", H.ref(da), H.ref(dt), 0, 1)          # runs at once: the block is used
        dev.dev.call("add", H.ref(dacc), H.ref(dt), H.ref(dacc))
        dev.dev.deallocate(pt)
    got = dev.fetch(pacc, acc.storage)
    want = np.zeros(rows * cols, np.float32)
    at = np.ascontiguousarray(a.storage.reshape(rows, cols).T).reshape(-1)
    for _ in range(loops):
        want += at
    T.assert_same_bits(got, want, "accumulated transposes")
    live, cached = C.c_uint64(), C.c_uint64()
    D.check(dev.dev.lib.aixhip_memory_stats(dev.dev.handle, C.byref(live), C.byref(cached)))
    info = K.DeviceInfo()
    K.check(K.load().aixk_info(dev.dev.kernel_context(), C.byref(info)))
    floor = max(32 << 20, info.total_mem >> 10)
    assert cached.value <= 3 * floor, (cached.value, floor)
    assert cached.value < loops * rows * cols * 4 // 2
    dev.release()


def test_interior_pointer_operands(dev):
    """Operands and results may point into the middle of an allocation (two tensors carved out of one
    block): the device recognises them as its own memory, orders the work and frees the block once."""
    rng = np.random.default_rng(36500)
    n = 1 << 16
    lo = T.contiguous_tensor(rng, O.F32, [n])
    hi = T.contiguous_tensor(rng, O.F32, [n])
    big = dev.raw(2 * n * 4)
    dev.dev.from_host(big, lo.storage)
    dev.dev.from_host(big + n * 4, hi.storage)
    d_lo, d_hi = H.kdesc(lo, big), H.kdesc(hi, big + n * 4)
    out = dev.raw(n * 4)
    dev.dev.call("add", H.ref(d_lo), H.ref(d_hi), H.ref(H.kdesc(lo, out)))
    T.assert_same_bits(dev.fetch(out, lo.storage), lo.storage + hi.storage, "sum of the two halves")
    dev.dev.call("mul", H.ref(d_lo), H.ref(d_lo), H.ref(d_hi))             # result through an interior pointer
    dev.dev.call("sum", H.ref(d_hi), H.ref(H.kdesc(T.empty(O.F32, [1]), out)))   # an operator that runs at once reads it
    T.assert_same_bits(dev.fetch(big + n * 4, hi.storage), lo.storage * lo.storage, "square written into the upper half")
    got = dev.fetch(out, np.zeros(1, np.float32))
    want = np.float64((lo.storage.astype(np.float64) ** 2).sum())
    assert abs(float(got[0]) - want) <= 1e-5 * want
    dev.release()


def _special_storage(rng, dtype, n):
    if dtype in T.FLOAT_DTYPES:
        with np.errstate(over="ignore", invalid="ignore"):
            vals = np.concatenate([np.array([0.0, -0.0, 1.0, -1.0, 0.5, 255.4, 255.6, -0.4, 300.0, -129.0, 32767.6, -40000.0, 3.0e9, -3.0e9,
                                             1e19, -1e19, 65504.0, 1e-8, np.inf, -np.inf, np.nan]), rng.uniform(-400, 400, n - 21)])
            return O.to_storage(vals, dtype)
    info = np.iinfo(O.NP_STORAGE[dtype])
    return np.concatenate([np.array([info.min, info.max, 0, 1, 2], dtype=O.NP_STORAGE[dtype]),
                           rng.integers(info.min, info.max, n - 5, endpoint=True).astype(O.NP_STORAGE[dtype])])


@pytest.mark.parametrize("src", T.ALL_DTYPES, ids=lambda d: NAMES[d])
def test_recorded_casts_fuse_and_keep_the_conversion_rules(dev, src):
    """Device-to-device copy() is recorded: it runs inside the kernel that consumes its result (converted at
    the load) or produces its operand (converted at the store).  Every pair of element types, special
    values included, against the CPU device operator by operator: y = (x.to(D) + x.to(D)).to(S), both
    intermediate tensors released before the flush, and the plain single cast."""
    set_diag(dev)
    rng = np.random.default_rng(37000 + src)
    n = 2100 + 13                                            # vector body + tail
    st = _special_storage(rng, src, n)
    x = T.HostTensor(st, src, [n])
    px, dx = dev.put(x)
    for dst in T.ALL_DTYPES:
        if dst == src:
            continue
        what = f"{NAMES[src]} -> {NAMES[dst]}"
        # CPU: copy, add, copy back
        xd = T.empty(dst, [n]); yd = T.empty(dst, [n]); back = T.empty(src, [n]); plain = T.empty(dst, [n])
        assert CPU.copy(st.ctypes.data, src, xd.storage.ctypes.data, dst, n) == 0
        with np.errstate(all="ignore"):
            assert CPU.binary(O.ADD, C.byref(xd.desc()), C.byref(xd.desc()), C.byref(yd.desc())) == 0
        assert CPU.copy(yd.storage.ctypes.data, dst, back.storage.ctypes.data, src, n) == 0
        # device: the same stream, temporaries freed before anything runs
        p_xd, p_yd, p_back = dev.raw(xd.storage.nbytes, keep=False), dev.raw(yd.storage.nbytes, keep=False), dev.raw(back.storage.nbytes)
        dev.dev.call("copy", px, src, p_xd, dst, n)
        dev.dev.call("add", H.ref(H.kdesc(xd, p_xd)), H.ref(H.kdesc(xd, p_xd)), H.ref(H.kdesc(yd, p_yd)))
        dev.dev.call("copy", p_yd, dst, p_back, src, n)
        dev.dev.deallocate(p_xd)
        dev.dev.deallocate(p_yd)
        got = dev.fetch(p_back, back.storage)
        diag = dev.dev.diagnostics()
        assert diag.fusible_subgraphs == 1 and diag.fused_ops == 3 and diag.fallback_ops == 0, (what, diag.subgraph_summary, diag.fallback_summary)
        T.assert_same_bits_nan_ok(got, back.storage, src, "fused cast, add, cast back: " + what)
        # a cast on its own runs as the plain conversion kernel
        p_plain = dev.raw(plain.storage.nbytes)
        dev.dev.call("copy", px, src, p_plain, dst, n)
        got = dev.fetch(p_plain, plain.storage)
        T.assert_same_bits_nan_ok(got, xd.storage, dst, "single cast: " + what)
    dev.release()


def test_fill_is_folded_into_slice_set(dev):
    """The backward of a slice: zeros of the input's shape, then the gradient set into the slice.  The pending
    fill becomes the value the one sliceSet pass writes outside the slice (no fill kernel runs); a fill that
    something else has read in between stays a fill."""
    set_diag(dev)
    rng = np.random.default_rng(38000)
    for dtype in (O.F32, O.BF16, O.I32):
        big, part = [40, 96], [40, 32]
        g = T.contiguous_tensor(rng, dtype, part, int_span=50)
        pg, dg = dev.put(g)
        want = T.empty(dtype, big)
        zero = np.zeros(1, np.float32)
        assert CPU.fill(zero.ctypes.data, O.F32, C.byref(want.desc())) == 0
        assert CPU.slice_set(C.byref(g.desc()), C.byref(want.desc()), 1, 32, 64, 1, 1) == 0
        pz = dev.raw(want.storage.nbytes)
        dz = H.kdesc(want, pz)
        dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(dz))
        dev.dev.call("slice_set", H.ref(dg), H.ref(dz), 1, 32, 64, 1)
        got = dev.fetch(pz, want.storage)
        T.assert_same_bits(got, want.storage, f"fill + sliceSet folded, {NAMES[dtype]}")
    dev.release()


def test_runs_of_slice_sets_leave_as_one_launch(dev):
    """cat() is one sliceSet per part (aixCore.hpp:1348-1402), the seed of a sliced tensor one per slice (:2228-2233):
    calls that do not depend on one another wait and leave in one launch.  Every scenario against the oracle applying
    the same calls one after the other: parts of one destination, windows that overlap (the later call wins), a
    destination that is the next call's source, recorded operators before and after, a matmul on the result."""
    set_diag(dev)
    rng = np.random.default_rng(43000)
    dtype = O.BF16
    rows, width, parts = 64, 32, 12

    def oracle_set(src, dst, dim, a, b):
        assert CPU.slice_set(C.byref(src.desc()), C.byref(dst.desc()), dim, a, b, 1, 1) == 0

    # 1. a cat of twelve column blocks and, into another tensor, four row blocks: one launch for all sixteen
    whole, tall = T.empty(dtype, [rows, width * parts], fill=7), T.empty(dtype, [4 * rows, width], fill=7)
    pw, dw = dev.put(whole)
    pt, dt = dev.put(tall)
    srcs = [T.contiguous_tensor(rng, dtype, [rows, width]) for _ in range(parts + 4)]
    ups = [dev.put(x) for x in srcs]
    dev.dev.synchronize()
    before = dev.dev.batched_launch_stats()
    for k in range(parts):
        oracle_set(srcs[k], whole, 1, k * width, (k + 1) * width)
        dev.dev.call("slice_set", H.ref(ups[k][1]), H.ref(dw), 1, k * width, (k + 1) * width, 1)
    for k in range(4):
        oracle_set(srcs[parts + k], tall, 0, k * rows, (k + 1) * rows)
        dev.dev.call("slice_set", H.ref(ups[parts + k][1]), H.ref(dt), 0, k * rows, (k + 1) * rows, 1)
    got_w, got_t = dev.fetch(pw, whole.storage), dev.fetch(pt, tall.storage)
    after = dev.dev.batched_launch_stats()
    assert after[0] - before[0] == 1 and after[1] - before[1] == parts + 4, (before, after)
    T.assert_same_bits(got_w, whole.storage, "twelve column blocks")
    T.assert_same_bits(got_t, tall.storage, "four row blocks")
    # 2. windows that overlap, a strided window, the same window twice: the calls keep their order
    for k, (a, b) in enumerate([(0, 32), (16, 48), (16, 48), (40, 72)]):
        oracle_set(srcs[k], whole, 1, a, b)
        dev.dev.call("slice_set", H.ref(ups[k][1]), H.ref(dw), 1, a, b, 1)
    assert CPU.slice_set(C.byref(srcs[5].desc()), C.byref(whole.desc()), 1, 100, 164, 2, 1) == 0
    dev.dev.call("slice_set", H.ref(ups[5][1]), H.ref(dw), 1, 100, 164, 2)
    oracle_set(srcs[6], whole, 1, 101, 133)
    dev.dev.call("slice_set", H.ref(ups[6][1]), H.ref(dw), 1, 101, 133, 1)
    T.assert_same_bits(dev.fetch(pw, whole.storage), whole.storage, "overlapping windows")
    # 3. a destination that the next call reads, and a source that is overwritten after it was read
    mid, last = T.empty(dtype, [rows, 2 * width], fill=1), T.empty(dtype, [rows, 4 * width], fill=2)
    pm, dm = dev.put(mid)
    pl, dl = dev.put(last)
    oracle_set(srcs[0], mid, 1, 0, width)
    dev.dev.call("slice_set", H.ref(ups[0][1]), H.ref(dm), 1, 0, width, 1)
    oracle_set(mid, last, 1, 2 * width, 4 * width)
    dev.dev.call("slice_set", H.ref(dm), H.ref(dl), 1, 2 * width, 4 * width, 1)
    oracle_set(srcs[1], mid, 1, 0, width)                                         # after `last` took its copy
    dev.dev.call("slice_set", H.ref(ups[1][1]), H.ref(dm), 1, 0, width, 1)
    T.assert_same_bits(dev.fetch(pl, last.storage), last.storage, "chain: the copy of the destination before it changed")
    T.assert_same_bits(dev.fetch(pm, mid.storage), mid.storage, "chain: the destination after its second window")
    # 4. recorded operators on either side: the source is a recorded sum, the destination is negated afterwards
    rec = Recorder(dev, dtype, [rows, width])
    x, y = rec.leaf(srcs[2]), rec.leaf(srcs[3])
    total = rec.binary(O.ADD, x, y)                                               # pending when sliceSet is called
    oracle_set(total["host"], mid, 1, width, 2 * width)
    dev.dev.call("slice_set", H.ref(total["desc"]), H.ref(dm), 1, width, 2 * width, 1)
    rec2 = Recorder(dev, dtype, [rows, 2 * width])
    neg = rec2.unary(O.NEG, {"host": mid, "ptr": pm, "desc": dm})                  # recorded while the sliceSet waits
    oracle_set(srcs[4], mid, 1, 0, width)                                         # and the destination changes again
    dev.dev.call("slice_set", H.ref(ups[4][1]), H.ref(dm), 1, 0, width, 1)
    T.assert_same_bits(dev.fetch(neg["ptr"], neg["host"].storage), neg["host"].storage, "negation of the destination as it was")
    T.assert_same_bits(dev.fetch(pm, mid.storage), mid.storage, "destination after the negation was recorded")
    # 5. a matmul on a destination whose parts are still waiting, and a sliceSet of its result
    a = T.empty(dtype, [64, 64], fill=0)
    pa, da = dev.put(a)
    halves = [T.contiguous_tensor(rng, dtype, [64, 32], lo=-1, hi=1) for _ in range(2)]
    for k, hlf in enumerate(halves):
        _, dh = dev.put(hlf)
        oracle_set(hlf, a, 1, 32 * k, 32 * (k + 1))
        dev.dev.call("slice_set", H.ref(dh), H.ref(da), 1, 32 * k, 32 * (k + 1), 1)
    b = T.contiguous_tensor(rng, dtype, [64, 64], lo=-1, hi=1)
    _, db = dev.put(b)
    prod = T.empty(dtype, [64, 64])
    pp = dev.raw(prod.storage.nbytes)
    dp = H.kdesc(prod, pp)
    dev.dev.call("matmul", H.ref(da), H.ref(db), H.ref(dp))
    wide = T.empty(dtype, [64, 128], fill=5)
    pwd, dwd = dev.put(wide)
    dev.dev.call("slice_set", H.ref(dp), H.ref(dwd), 1, 64, 128, 1)
    raw = dev.fetch(pwd, wide.storage).reshape(64, 128)
    got = O.to_float64(raw[:, 64:], dtype)
    want = O.to_float64(a.storage, dtype).reshape(64, 64) @ O.to_float64(b.storage, dtype).reshape(64, 64)
    assert np.all(raw[:, :64] == 5)
    assert np.max(np.abs(got - want)) <= 2e-2 * np.max(np.abs(want)), "matmul of the assembled operand, set into a window"   # bf16 result: 2e-2 relative
    dev.release()


_CASES = goldens.load_cases()


@pytest.mark.parametrize("case", _CASES, ids=[c["name"] for c in _CASES])
def test_reference_literals_on_device(dev, case):
    goldens.run_case(case, H.DeviceBackend(dev))


def test_matmul_on_stacks_through_the_device(dev):
    """matmul with operands of rank above 2 (beyond the reference's 2-D matmul): a stack of products through the
    device interface -- elementwise work pending on an operand is flushed first, the [batch, heads, seq, d] view of
    a [batch * seq, heads * d] activation is consumed without a copy, a host-memory operand is staged, and
    operands whose leading dims differ are refused with the reference's exception type."""
    rng = np.random.default_rng(36000)
    B, Hd, S, D = 2, 3, 64, 32
    dtype = O.BF16
    rec = Recorder(dev, dtype, [B * S, Hd * D])
    x = rec.leaf(T.contiguous_tensor(rng, dtype, [B * S, Hd * D], lo=-0.3, hi=0.3))
    y = rec.leaf(T.contiguous_tensor(rng, dtype, [B * S, Hd * D], lo=-0.3, hi=0.3))
    q = rec.binary(O.ADD, x, y)                                     # pending when the matmul is called
    heads = [S * Hd * D, D, Hd * D, 1]
    q4 = T.HostTensor(q["host"].storage, dtype, [B, Hd, S, D], heads)
    kT = T.HostTensor(y["host"].storage, dtype, [B, Hd, D, S], [S * Hd * D, D, 1, Hd * D])
    out = T.empty(dtype, [B, Hd, S, S])
    po = dev.raw(out.storage.nbytes)
    dev.dev.call("matmul", H.ref(H.kdesc(q4, q["ptr"])), H.ref(H.kdesc(kT, y["ptr"])), H.ref(H.kdesc(out, po)))
    got = O.to_float64(dev.fetch(po, out.storage), dtype).reshape(B, Hd, S, S)
    want = O.to_float64(q4.gather(), dtype) @ O.to_float64(kT.gather(), dtype)
    scale = np.abs(O.to_float64(q4.gather(), dtype)) @ np.abs(O.to_float64(kT.gather(), dtype))
    assert np.all(np.abs(got - want) <= 1e-5 * scale + 2.0 ** -8 * np.abs(want) + 1e-30)
    # a host-memory second operand (staged into device memory first), f32 stack issued product by product
    a32 = T.contiguous_tensor(rng, O.F32, [3, 40, 24], lo=-1, hi=1)
    b32 = T.contiguous_tensor(rng, O.F32, [3, 24, 56], lo=-1, hi=1)
    pa, da = dev.put(a32)
    o32 = T.empty(O.F32, [3, 40, 56])
    po32 = dev.raw(o32.storage.nbytes)
    dev.dev.call("matmul", H.ref(da), H.ref(H.kdesc(b32, b32.storage.ctypes.data)), H.ref(H.kdesc(o32, po32)))
    got32 = dev.fetch(po32, o32.storage).astype(np.float64).reshape(3, 40, 56)
    want32 = a32.gather().astype(np.float64) @ b32.gather().astype(np.float64)
    assert np.all(np.abs(got32 - want32) <= 1e-5 * (np.abs(a32.gather()).astype(np.float64) @ np.abs(b32.gather()).astype(np.float64)))
    # leading dims that differ: refused
    bad = T.HostTensor(b32.storage, O.F32, [2, 24, 56])
    with pytest.raises(Exception):
        dev.dev.call("matmul", H.ref(da), H.ref(H.kdesc(bad, bad.storage.ctypes.data)), H.ref(H.kdesc(o32, po32)))
    dev.release()


def test_fill_is_folded_into_argmax_indices_to(dev):
    """The mask of a max() backward: an int32 tensor of src's shape filled with 0, then argmaxIndicesTo scatters
    ones into it.  A zero fill still waiting in the window is folded into the operator (over a handful of rows
    the one-hot block is written densely in one pass); any other pending value is put back first, because
    the operator only ever writes the ones."""
    set_diag(dev)
    rng = np.random.default_rng(39000)
    for shape, dim in (([2, 64, 256], 0), ([300, 40], 1), ([5, 1024], 0)):
        src = T.contiguous_tensor(rng, O.F32, shape, lo=-1, hi=1)
        src.storage[:] = np.round(src.storage * 2) / 2                       # ties: the first maximum wins
        _, dsrc = dev.put(src)
        for value in (0.0, 5.0):
            want = T.empty(O.I32, shape)
            v = np.array([value], np.float32)
            assert CPU.fill(v.ctypes.data, O.F32, C.byref(want.desc())) == 0
            assert CPU.argmax_indices_to(C.byref(src.desc()), C.byref(want.desc()), dim) == 0
            pm = dev.raw(want.storage.nbytes)
            dm = H.kdesc(want, pm)
            dev.dev.call("fill", v.ctypes.data, O.F32, H.ref(dm))
            dev.dev.call("argmax_indices_to", H.ref(dsrc), H.ref(dm), dim)
            T.assert_same_bits(dev.fetch(pm, want.storage), want.storage, f"fill({value}) + argmaxIndicesTo {shape} dim={dim}")
    dev.release()


def test_sum_of_everything_joins_the_kernel_that_forms_it(dev):
    """The gradient of a scalar constant (aixCore.hpp:2384-2438, 2030-2036): p = g * x, then fill(0) + reduceTo of p down to
    one element, while the expression goes on (q = p + x, whose own sum starts from 7).  One generated kernel that adds
    p and q up where they are formed, plus aixk_sum_partials per sum; p is never stored once its buffer is gone.
    f32 / f64: 1e-5 / 1e-12 of the sum of |terms| against a float64 sum of the oracle's elementwise results; bf16 / f16
    (summed in f32 here, in the 16-bit type on the CPU): 2e-2 of it.  Sizes from a ragged handful to 3 million, a strided
    operand (the rows shape) and a higher-rank transposed one (the gather shape)."""
    set_diag(dev)
    rng = np.random.default_rng(45000)
    zero, seven = np.zeros(1, np.float32), np.full(1, 7.0, np.float32)
    cases = [(O.F32, [257], None), (O.F32, [1024, 3000], None), (O.BF16, [512, 768], None), (O.F16, [33, 1000], None), (O.F64, [100, 1001], None),
             (O.F32, [64, 96], "rows"), (O.BF16, [6, 40, 24], "gather")]
    for dtype, shape, kind in cases:
        rec = Recorder(dev, dtype, shape)
        g = rec.leaf(T.contiguous_tensor(rng, dtype, shape, lo=-1, hi=1))
        if kind == "rows":
            xh = T.view_tensor(rng, dtype, shape, "sliced", lo=-1, hi=1)
        elif kind == "gather":
            xh = T.view_tensor(rng, dtype, shape, "transposed", lo=-1, hi=1)
        else:
            xh = T.contiguous_tensor(rng, dtype, shape, lo=-1, hi=1)
        x = rec.leaf(xh)
        sums = []
        for _ in range(2):
            host = T.empty(dtype, [])
            sums.append({"host": host, "ptr": dev.raw(host.storage.nbytes)})
        dev.dev.synchronize()
        p = rec.binary(O.MUL, g, x)
        d0 = H.kdesc(sums[0]["host"], sums[0]["ptr"])
        dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(d0))
        dev.dev.call("reduce_to", H.ref(p["desc"]), H.ref(d0))
        q = rec.binary(O.ADD, p, x)
        d1 = H.kdesc(sums[1]["host"], sums[1]["ptr"])
        dev.dev.call("fill", seven.ctypes.data, O.F32, H.ref(d1))
        dev.dev.call("reduce_to", H.ref(q["desc"]), H.ref(d1))
        pv, qv = O.to_float64(p["host"].storage, dtype), O.to_float64(q["host"].storage, dtype)
        rec.free_temps(keep=(q,))
        got_q = dev.fetch(q["ptr"], q["host"].storage)
        diag = dev.dev.diagnostics()
        assert diag.fusible_subgraphs == 1 and diag.fused_ops == 4 and diag.fallback_ops == 0, (NAMES[dtype], shape, kind, diag.subgraph_summary, diag.fallback_summary)
        T.assert_same_bits(got_q, q["host"].storage, f"q = g * x + x beside its sums, {NAMES[dtype]} {shape} {kind}")
        tol = {O.F64: 1e-12, O.F32: 1e-5}.get(dtype, 2e-2)
        for node, exact, scale in ((sums[0], pv.sum(), np.abs(pv).sum()), (sums[1], 7.0 + qv.sum(), 7.0 + np.abs(qv).sum())):
            got = float(O.to_float64(dev.fetch(node["ptr"], node["host"].storage), dtype)[0])
            assert abs(got - exact) <= tol * scale, (NAMES[dtype], shape, kind, got, exact)
        dev.release()
    # a sum whose operand no recorded operator produces runs as before, and so does one taken with fusion switched off
    x = T.contiguous_tensor(rng, O.F32, [1000], lo=-1, hi=1)
    _, dx = dev.put(x)
    host = T.empty(O.F32, [])
    ps = dev.raw(4)
    ds = H.kdesc(host, ps)
    dev.dev.call("fill", seven.ctypes.data, O.F32, H.ref(ds))
    dev.dev.call("reduce_to", H.ref(dx), H.ref(ds))
    got = float(dev.fetch(ps, host.storage)[0])
    assert abs(got - (7.0 + x.storage.astype(np.float64).sum())) <= 1e-5 * (7.0 + np.abs(x.storage).sum())
    dev.release()


def test_runs_of_argmax_indices_to_leave_as_one_launch(dev):
    """The masks of max()'s backward pass, head after head (aixCore.hpp:2170-2175): calls whose zero fill was folded in
    wait and leave in one launch; a recorded operator that reads a mask, a source that a recorded operator produces, and
    a mask whose buffer is also the next call's source keep their order.  Against the oracle call by call."""
    set_diag(dev)
    rng = np.random.default_rng(44000)
    dtype = O.BF16
    shape = [64, 128]
    zero = np.zeros(1, np.float32)

    def mask_of(src_host, src_desc):
        want = T.empty(O.I32, shape)
        assert CPU.fill(zero.ctypes.data, O.F32, C.byref(want.desc())) == 0
        assert CPU.argmax_indices_to(C.byref(src_host.desc()), C.byref(want.desc()), 1) == 0
        pm = dev.raw(want.storage.nbytes)
        dm = H.kdesc(want, pm)
        dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(dm))
        dev.dev.call("argmax_indices_to", H.ref(src_desc), H.ref(dm), 1)
        return pm, dm, want

    srcs = [T.contiguous_tensor(rng, dtype, shape, lo=-1, hi=1) for _ in range(6)]
    ups = [dev.put(x) for x in srcs]
    dev.dev.synchronize()
    before = dev.dev.batched_launch_stats()
    masks = [mask_of(x, d) for x, (_, d) in zip(srcs, ups)]
    got = [dev.fetch(pm, want.storage) for pm, _, want in masks]
    after = dev.dev.batched_launch_stats()
    assert after[0] - before[0] == 1 and after[1] - before[1] == len(srcs), (before, after)
    for g, (_, _, want) in zip(got, masks):
        T.assert_same_bits(g, want.storage, "six masks in one launch")
    # a source that is a recorded sum, and a recorded conversion + product that reads the mask while it waits
    rec = Recorder(dev, dtype, shape)
    x, y = rec.leaf(srcs[0]), rec.leaf(srcs[1])
    total = rec.binary(O.ADD, x, y)
    pm, dm, want = mask_of(total["host"], total["desc"])
    as16 = T.empty(dtype, shape)
    assert CPU.copy(want.storage.ctypes.data, O.I32, as16.storage.ctypes.data, dtype, want.size) == 0
    p16 = dev.raw(as16.storage.nbytes)
    dev.dev.call("copy", pm, O.I32, p16, dtype, want.size)
    prod = rec.binary(O.MUL, {"host": as16, "ptr": p16, "desc": H.kdesc(as16, p16)}, x)
    # the next mask overwrites a buffer that the waiting product still reads: x's own storage is its destination's source
    pm2, dm2, want2 = mask_of(prod["host"], prod["desc"])
    T.assert_same_bits(dev.fetch(prod["ptr"], prod["host"].storage), prod["host"].storage, "mask * x, recorded while the mask waited")
    T.assert_same_bits(dev.fetch(pm, want.storage), want.storage, "mask of a recorded sum")
    T.assert_same_bits(dev.fetch(pm2, want2.storage), want2.storage, "mask of the product")
    dev.release()


def test_tril_and_triu_join_the_fused_kernels(dev):
    """tril / triu recorded as elementwise operators: attention's tril(s) * scale + mask is ONE generated kernel
    (the triangle's extents and diagonal are run-time integers of it), negate -> triu over a dense stack takes the flat
    launch shape, a transposed source the gather shape; results against the CPU oracle operator by operator."""
    set_diag(dev)
    rng = np.random.default_rng(40000)
    for dtype in (O.BF16, O.F32):
        for shape, diag, upper in (([2, 3, 40, 48], 0, 0), ([2, 3, 40, 48], -3, 1), ([5, 33, 20], 4, 0), ([64, 64], 1, 1)):
            rec = Recorder(dev, dtype, shape)
            s = rec.leaf(T.contiguous_tensor(rng, dtype, shape, lo=-2, hi=2))
            mask_store = T.random_values(rng, shape[-2] * shape[-1], dtype, lo=-1, hi=1)
            mask = rec.leaf(T.HostTensor(mask_store, dtype, shape, [0] * (len(shape) - 2) + [shape[-1], 1]))   # uploads flush: before recording
            # oracle: tril, then * scale, then + mask (mask broadcast over the leading dims)
            t_host = T.empty(dtype, shape)
            assert (CPU.triu if upper else CPU.tril)(C.byref(s["host"].desc()), C.byref(t_host.desc()), diag) == 0
            pt = dev.raw(t_host.storage.nbytes)
            t = {"host": t_host, "ptr": pt, "desc": H.kdesc(t_host, pt)}
            dev.dev.call("triu" if upper else "tril", H.ref(s["desc"]), H.ref(t["desc"]), diag)
            scaled = rec.binary(O.MUL, t, rec.scalar(0.125))
            out = rec.binary(O.ADD, scaled, mask)
            got = dev.fetch(out["ptr"], out["host"].storage)
            T.assert_same_bits(got, out["host"].storage, f"tri(upper={upper}, {diag}) * scale + mask {NAMES[dtype]} {shape}")
            diagn = dev.dev.diagnostics()
            assert diagn.fusible_subgraphs == 1 and diagn.fused_ops == 3, diagn.subgraph_summary     # (the scalar's own fill also runs: its tensor is still alive)
            dev.release()
        # negate -> triu on a dense stack (flat launch shape), and tril of a transposed view (gather shape) feeding a negate
        shape = [4, 32, 32]
        rec = Recorder(dev, dtype, shape)
        x = rec.leaf(T.contiguous_tensor(rng, dtype, shape, lo=-1, hi=1))
        e = rec.unary(O.NEG, x)                                         # (exact on both devices)
        z_host = T.empty(dtype, shape)
        assert CPU.triu(C.byref(e["host"].desc()), C.byref(z_host.desc()), -1) == 0
        pz = dev.raw(z_host.storage.nbytes)
        dev.dev.call("triu", H.ref(e["desc"]), H.ref(H.kdesc(z_host, pz)), -1)
        T.assert_same_bits(dev.fetch(pz, z_host.storage), z_host.storage, f"negate -> triu {NAMES[dtype]}")
        xt = T.HostTensor(x["host"].storage, dtype, shape, [32 * 32, 1, 32])
        w_host = T.empty(dtype, shape)
        assert CPU.tril(C.byref(xt.desc()), C.byref(w_host.desc()), 2) == 0
        pw = dev.raw(w_host.storage.nbytes)
        w = {"host": w_host, "ptr": pw, "desc": H.kdesc(w_host, pw)}
        dev.dev.call("tril", H.ref(H.kdesc(xt, x["ptr"])), H.ref(w["desc"]), 2)
        neg = rec.unary(O.NEG, w)
        T.assert_same_bits(dev.fetch(neg["ptr"], neg["host"].storage), neg["host"].storage, f"tril(transposed view) -> negate {NAMES[dtype]}")
        dev.release()


def test_idle_fills_wait_for_their_first_user(dev):
    """zeroGrad() and, a pass later, the accumulation into the gradient: the fill is not launched when the flushes in
    between come (nothing there names its buffer); it becomes an immediate of the accumulation.  Reading the buffer, a
    synchronize(), or an operand pointing into the block bring a waiting fill back in time."""
    set_diag(dev)
    rng = np.random.default_rng(41000)
    n = 50000
    x = T.contiguous_tensor(rng, O.F32, [n])
    other = T.contiguous_tensor(rng, O.F32, [64, 32])
    _, dx = dev.put(x)
    _, dother = dev.put(other)
    pg = dev.raw(n * 4)
    dg = H.kdesc(x, pg)
    zero, three, five, seven = (np.array([v], np.float32) for v in (0.0, 3.0, 5.0, 7.0))
    pt = dev.raw(other.storage.nbytes)
    ptmp = dev.raw(other.storage.nbytes)
    dtmp = H.kdesc(other, ptmp)

    def flush_in_between():
        """A recorded operator and an operator that runs at once and reads its result: the window is flushed (an
        operator that runs at once on operands nothing recorded touches leaves the window alone)."""
        dev.dev.call("add", H.ref(dother), H.ref(dother), H.ref(dtmp))
        dev.dev.call("transpose", H.ref(dtmp), H.ref(H.kdesc(T.empty(O.F32, [32, 64]), pt)), 0, 1)

    dev.dev.synchronize()
    dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(dg))
    flush_in_between()
    diag = dev.dev.diagnostics()
    assert diag.ops_recorded == 2 and diag.fallback_ops + diag.fusible_subgraphs == 1 and diag.fills_absorbed == 0, (diag.ops_recorded, diag.fallback_ops, diag.subgraph_summary)
    dev.dev.call("add", H.ref(dg), H.ref(dx), H.ref(dg))                   # grad = grad + x
    got = dev.fetch(pg, x.storage)
    diag = dev.dev.diagnostics()
    assert diag.ops_recorded == 2 and diag.fusible_subgraphs == 1 and diag.fills_absorbed == 1 and diag.fallback_ops == 0, diag.subgraph_summary
    T.assert_same_bits(got, x.storage + np.float32(0), "0 + x")
    # read back with nothing else recorded / after a synchronize
    ph = dev.raw(n * 4)
    dev.dev.call("fill", three.ctypes.data, O.F32, H.ref(H.kdesc(x, ph)))
    flush_in_between()
    assert np.all(dev.fetch(ph, x.storage) == 3.0)
    dev.dev.call("fill", five.ctypes.data, O.F32, H.ref(H.kdesc(x, ph)))
    flush_in_between()
    dev.dev.synchronize()
    host_view = (C.c_float * n).from_address(ph)                             # device memory is host-visible (large BAR)
    assert host_view[0] == 5.0 and host_view[n - 1] == 5.0
    # a waiting fill whose buffer is released is never launched; the block is reused at once
    pk = dev.raw(1 << 20, keep=False)
    dev.dev.call("fill", seven.ctypes.data, O.F32, H.ref(H.kdesc(T.empty(O.F32, [1 << 18]), pk)))
    flush_in_between()
    dev.dev.deallocate(pk)
    dev.dev.synchronize()
    # operands that point into the middle of a filled block, and a fill through such a pointer
    half = 4096
    big = dev.raw(2 * half * 4)
    whole = T.empty(O.F32, [2 * half])
    upper = T.empty(O.F32, [half])
    dev.dev.call("fill", five.ctypes.data, O.F32, H.ref(H.kdesc(whole, big)))
    flush_in_between()
    pout = dev.raw(half * 4)
    dev.dev.call("unary", H.ref(H.kdesc(upper, big + half * 4)), H.ref(H.kdesc(upper, pout)))
    assert np.all(dev.fetch(pout, upper.storage) == -5.0)
    dev.dev.call("fill", seven.ctypes.data, O.F32, H.ref(H.kdesc(upper, big + half * 4)))
    dev.dev.synchronize()
    got = dev.fetch(big, whole.storage)
    assert np.all(got[:half] == 5.0) and np.all(got[half:] == 7.0)
    dev.release()


def test_runs_of_equal_flat_kernels_leave_as_one_launch(dev):
    """Adam's update of parameter after parameter (aixOptimizer.hpp:112-140), the per-parameter casts of a
    mixed-precision step: generated flat kernels of one signature that do not depend on one another are sent off in one
    launch, each with its own argument block and share of the grid.  Results against the oracle operator by operator
    (exact: multiply and add, correctly rounded on both sides); sizes from one element to a million, ragged tails."""
    set_diag(dev)
    rng = np.random.default_rng(42000)
    sizes = [1, 3, 4, 5, 255, 256, 1000, 4096, 65537, 1 << 20, 7, 300000]
    before = dev.dev.batched_launch_stats()
    nodes = []
    recs = [Recorder(dev, O.F32, [n]) for n in sizes]
    leaves = [rec.leaf(T.contiguous_tensor(rng, O.F32, [n])) for rec, n in zip(recs, sizes)]      # (uploads flush: all of them first)
    for rec, x in zip(recs, leaves):
        y = rec.binary(O.ADD, rec.binary(O.MUL, x, rec.scalar(2.0)), rec.scalar(1.0))
        nodes.append((rec, y))
    for rec, y in nodes:
        rec.free_temps(keep=(y,))
    got = [dev.fetch(y["ptr"], y["host"].storage) for _, y in nodes]
    after = dev.dev.batched_launch_stats()
    assert after[0] - before[0] == 1 and after[1] - before[1] == len(sizes), (before, after)
    for (rec, y), g, n in zip(nodes, got, sizes):
        T.assert_same_bits(g, y["host"].storage, f"2x + 1 over {n} elements, batched")
    dev.release()
    # kernels that depend on one another stay apart: z = 2y + 1 reads the y of the kernel before it
    rec = Recorder(dev, O.F32, [5000])
    x = rec.leaf(T.contiguous_tensor(rng, O.F32, [5000]))
    y = rec.binary(O.ADD, rec.binary(O.MUL, x, rec.scalar(2.0)), rec.scalar(1.0))
    dev.dev.flush()
    before = dev.dev.batched_launch_stats()
    chain = [y]
    for _ in range(3):
        # each link is recorded after a use of the previous result outside the kernel, so that it is a kernel of its own
        chain.append(rec.binary(O.ADD, rec.binary(O.MUL, chain[-1], rec.scalar(2.0)), rec.scalar(1.0)))
    got = dev.fetch(chain[-1]["ptr"], chain[-1]["host"].storage)
    T.assert_same_bits(got, chain[-1]["host"].storage, "three dependent links")
    for link in chain[:-1]:
        T.assert_same_bits(dev.fetch(link["ptr"], link["host"].storage), link["host"].storage, "a link's own result")
    dev.release()
    # casts of several tensors (f32 -> bf16, bf16 -> f32): one launch each way, values as the single operator gives them
    srcs = [T.contiguous_tensor(rng, O.F32, [n], lo=-300, hi=300) for n in (10, 513, 70000, 8)]
    before = dev.dev.batched_launch_stats()
    outs = []
    for s in srcs:
        ps, _ = dev.put(s)
        pd = dev.raw(s.size * 2)
        outs.append(pd)
    dev.dev.synchronize()
    ptrs = [dev.live[-2 * len(srcs) + 2 * k] for k in range(len(srcs))]
    for s, ps, pd in zip(srcs, ptrs, outs):
        dev.dev.call("copy", ps, O.F32, pd, O.BF16, s.size)
    got = [dev.fetch(pd, np.zeros(s.size, np.uint16)) for s, pd in zip(srcs, outs)]
    after = dev.dev.batched_launch_stats()
    assert after[0] - before[0] == 1 and after[1] - before[1] == len(srcs), (before, after)
    for s, g in zip(srcs, got):
        want = np.zeros(s.size, np.uint16)
        assert CPU.copy(s.storage.ctypes.data, O.F32, want.ctypes.data, O.BF16, s.size) == 0
        T.assert_same_bits(g, want, f"f32 -> bf16 over {s.size} elements, batched")
    dev.release()


def test_runs_of_column_sums_leave_as_one_launch(dev):
    """The gradients of biases, layer after layer (aixCore.hpp:2228-2233 sums a gradient to its parameter's shape): reduceTo
    calls down the columns of a dense matrix whose destination's fill was folded in wait and leave together; a source that
    a recorded operator produces, a recorded operator that reads a sum while it waits, a freed source and a second sum
    into the same destination keep their meaning.  Against the oracle's sums in wide arithmetic: 1e-5 of the sum of the
    terms' magnitudes plus one bf16 rounding (2^-8)."""
    set_diag(dev)
    rng = np.random.default_rng(45000)
    dtype = O.BF16
    shape, dshape = [512, 128], [128]
    zero = np.zeros(1, np.float32)

    def close(got_storage, exact, scale, what):
        got = O.to_float64(got_storage, dtype).reshape(-1)
        bound = 1e-5 * np.asarray(scale) + 2.0 ** -8 * np.abs(exact) + 1e-30
        bad = np.flatnonzero(~(np.abs(got - exact) <= bound))
        assert bad.size == 0, f"{what}: {bad.size} of {got.size} beyond the bound; first at {bad[0]}: got {got[bad[0]]!r} exact {exact[bad[0]]!r}"

    def colsum_of(src_host, src_desc):
        filled = T.empty(dtype, dshape)
        assert CPU.fill(zero.ctypes.data, O.F32, C.byref(filled.desc())) == 0
        exact = filled.values().reshape(-1).copy()
        scale = np.abs(exact)
        assert CPU.reduce_to_wide(C.byref(src_host.desc()), C.byref(filled.desc()), exact.ctypes.data, scale.ctypes.data) == 0
        assert CPU.reduce_to(C.byref(src_host.desc()), C.byref(filled.desc())) == 0
        ps = dev.raw(filled.storage.nbytes)
        dd = H.kdesc(filled, ps)
        dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(dd))
        dev.dev.call("reduce_to", H.ref(src_desc), H.ref(dd))
        return {"host": filled, "ptr": ps, "desc": dd, "exact": exact, "scale": scale}

    srcs = [T.contiguous_tensor(rng, dtype, shape, lo=-1, hi=1) for _ in range(6)]
    ups = [dev.put(x) for x in srcs]
    dev.dev.synchronize()
    before = dev.dev.batched_launch_stats()
    sums = [colsum_of(x, d) for x, (_, d) in zip(srcs, ups)]
    dev.free(ups[5][0])                                              # its owner is done with a source while the sum still waits
    spare = [dev.raw(srcs[5].storage.nbytes) for _ in range(3)]      # must not be handed the freed block
    assert all(p != ups[5][0] for p in spare)
    got = [dev.fetch(s["ptr"], s["host"].storage) for s in sums]
    after = dev.dev.batched_launch_stats()
    assert after[0] - before[0] == 1 and after[1] - before[1] == len(srcs), (before, after)
    for g, s in zip(got, sums):
        close(g, s["exact"], s["scale"], "six column sums in one pair of launches")
    # a source that is a recorded sum; a recorded addition that reads two sums while they wait
    rec = Recorder(dev, dtype, shape)
    x, y = rec.leaf(srcs[0]), rec.leaf(srcs[1])
    total = rec.binary(O.ADD, x, y)
    a = colsum_of(total["host"], total["desc"])
    b = colsum_of(x["host"], x["desc"])
    small = Recorder(dev, dtype, dshape)
    both = small.binary(O.ADD, a, b)
    # oracle-side values of a and b are the oracle's own sums; allow both sums' bounds plus the addition's rounding
    exact = a["exact"] + b["exact"]
    close(dev.fetch(both["ptr"], both["host"].storage), exact, a["scale"] + b["scale"] + (2.0 ** -8 / 1e-5) * (np.abs(a["exact"]) + np.abs(b["exact"])), "sum of two waiting column sums")
    close(dev.fetch(a["ptr"], a["host"].storage), a["exact"], a["scale"], "column sums of a recorded sum")
    # a second sum into a destination that a waiting sum writes: the first goes out first
    dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(b["desc"]))
    dev.dev.call("reduce_to", H.ref(y["desc"]), H.ref(b["desc"]))
    c = colsum_of(y["host"], y["desc"])
    close(dev.fetch(b["ptr"], b["host"].storage), c["exact"], c["scale"], "a destination summed into twice")
    dev.release()


def test_operators_at_once_leave_an_unrelated_window_alone(dev):
    """An operator that is enqueued at once (a transpose, a large matmul) goes ahead of the recorded operators when none of
    them writes what it reads or uses what it writes: the window stays whole and what it holds fuses across the call.  One
    that reads a recorded result flushes first.  Results against the oracle, bit for bit (add, multiply, transpose)."""
    set_diag(dev)
    rng = np.random.default_rng(46000)
    shape = [96, 40]
    rec = Recorder(dev, O.F32, shape)
    x, y = rec.leaf(T.contiguous_tensor(rng, O.F32, shape)), rec.leaf(T.contiguous_tensor(rng, O.F32, shape))
    other = T.contiguous_tensor(rng, O.F32, shape)
    _, dother = dev.put(other)
    dev.dev.synchronize()

    def transposed(src_host, src_desc):
        want = T.empty(O.F32, shape[::-1])
        assert CPU.transpose(C.byref(src_host.desc()), C.byref(want.desc()), 0, 1) == 0
        pt = dev.raw(want.storage.nbytes)
        dev.dev.call("transpose", H.ref(src_desc), H.ref(H.kdesc(want, pt)), 0, 1)
        return pt, want

    total = rec.binary(O.ADD, x, y)
    pt, want_t = transposed(other, dother)                                   # nothing recorded touches its operands
    prod = rec.binary(O.MUL, total, x)
    got = dev.fetch(prod["ptr"], prod["host"].storage)
    diag = dev.dev.diagnostics()
    assert diag.ops_recorded == 2 and diag.fusible_subgraphs == 1 and diag.fallback_ops == 0, diag.subgraph_summary
    T.assert_same_bits(got, prod["host"].storage, "(x + y) * x around an unrelated transpose")
    T.assert_same_bits(dev.fetch(pt, want_t.storage), want_t.storage, "the transpose")
    again = rec.binary(O.ADD, prod, y)
    pt2, want_t2 = transposed(again["host"], again["desc"])                  # reads a recorded result: the window goes first
    T.assert_same_bits(dev.fetch(pt2, want_t2.storage), want_t2.storage, "transpose of a recorded sum")
    dev.release()


def test_a_fill_of_the_destination_never_lands_behind_a_call_that_waits(dev):
    """fill(r); matmul(a, b, r); exp(r): the small 16-bit product waits for company, and the recorded fill of its result
    must leave before it, not be set aside as idle and wipe the product later (the reader would then take the fill's
    constant).  The same with a fill through another view of a sliceSet's destination, which cannot be folded into the
    copy.  Both bit for bit against the oracle's operator sequence (the device interface may be driven directly like this,
    as Targets/AIXTests/DeviceTests.cpp does)."""
    rng = np.random.default_rng(47000)
    seven = np.full(1, 7.0, np.float32)
    for dtype in (O.BF16, O.F16):
        a, b = T.contiguous_tensor(rng, dtype, [64, 64]), T.contiguous_tensor(rng, dtype, [64, 64])
        r, o = T.empty(dtype, [64, 64]), T.empty(dtype, [64, 64])
        (_, da), (_, db) = dev.put(a), dev.put(b)
        pr, po = dev.raw(r.storage.nbytes), dev.raw(o.storage.nbytes)
        dr, do = H.kdesc(r, pr), H.kdesc(o, po)
        dev.dev.synchronize()
        dev.dev.call("fill", seven.ctypes.data, O.F32, H.ref(dr))
        dev.dev.call("matmul", H.ref(da), H.ref(db), H.ref(dr))
        dev.dev.call("exp", H.ref(dr), H.ref(do))
        got_r, got_o = dev.fetch(pr, r.storage), dev.fetch(po, o.storage)
        # the product itself is held to the 16-bit bar against exact accumulation; exp is then applied to the device's own product
        exact, scale = np.zeros(64 * 64), np.zeros(64 * 64)
        assert CPU.matmul_wide(C.byref(a.desc()), C.byref(b.desc()), exact.ctypes.data, scale.ctypes.data, 8) == 0
        err = np.abs(O.to_float64(got_r, dtype).ravel() - exact)
        assert (err <= 2e-2 * scale + 1e-30).all(), f"fill + matmul, {NAMES[dtype]}: {err.max()}"
        r.storage[...] = got_r
        assert CPU.unary(O.EXP, C.byref(r.desc()), C.byref(o.desc())) == 0
        bad = T.ulp_distance(got_o, o.storage, dtype)
        assert bad <= 1, f"exp of the product, {NAMES[dtype]}: {bad} ulp"
    for dtype in (O.F32, O.BF16):
        part, whole = T.contiguous_tensor(rng, dtype, [16, 64]), T.contiguous_tensor(rng, dtype, [64, 64])
        upper = T.HostTensor(whole.storage, dtype, [32, 64], [64, 1])
        (_, dp), (pw, dw) = dev.put(part), dev.put(whole)
        dev.dev.synchronize()
        dev.dev.call("fill", seven.ctypes.data, O.F32, H.ref(H.kdesc(upper, pw)))
        dev.dev.call("slice_set", H.ref(dp), H.ref(dw), 0, 8, 24, 1)
        assert CPU.fill(seven.ctypes.data, O.F32, C.byref(upper.desc())) == 0
        assert CPU.slice_set(C.byref(part.desc()), C.byref(whole.desc()), 0, 8, 24, 1, 1) == 0
        T.assert_same_bits(dev.fetch(pw, whole.storage), whole.storage, f"fill through another view + sliceSet, {NAMES[dtype]}")
    dev.release()


def test_generated_kernels_are_kept_on_disk_between_contexts(tmp_path):
    """With AIXHIP_KERNEL_CACHE_DIR set when a device is created, the code object of every kernel it compiles is kept in that
    directory and a later device (a later process) loads it instead of compiling: the second device compiles nothing,
    stores nothing and computes the same bits.  Damaged files -- cut short, a flipped byte, an empty file -- are ignored:
    the third device compiles again, replaces them and computes the same bits."""
    where = tmp_path / "kept" / "kernels"
    rng = np.random.default_rng(34000)
    shape = [96, 130]
    host = T.contiguous_tensor(rng, O.F32, shape)
    klib = K.load()

    def one_device():
        d = H.Dev()
        try:
            rec = Recorder(d, O.F32, shape)
            a = rec.leaf(host)
            y = rec.binary(O.ADD, rec.unary(O.COS, rec.binary(O.MUL, rec.scalar(0.5), a)), rec.scalar(0.25))
            z = rec.unary(O.EXP, rec.binary(O.SUB, y, a))                       # a second kernel after a flush
            rec.free_temps(keep=(y, z))
            got = (d.fetch(y["ptr"], y["host"].storage).copy(), d.fetch(z["ptr"], z["host"].storage).copy())
            assert T.ulp_distance(got[0], y["host"].storage, O.F32) <= 2
            loaded, stored = C.c_uint64(), C.c_uint64()
            assert klib.aixk_rtc_disk_stats(d.dev.kernel_context(), C.byref(loaded), C.byref(stored)) == 0
            return got, loaded.value, stored.value
        finally:
            d.close()

    os.environ["AIXHIP_KERNEL_CACHE_DIR"] = str(where) + "//"
    try:
        first, loaded, stored = one_device()
        files = sorted(where.glob("*.aixk"))
        assert loaded == 0 and stored >= 1 and len(files) == stored, (loaded, stored, files)
        assert not list(where.glob("*.tmp.*"))
        second, loaded, stored2 = one_device()
        assert loaded == stored and stored2 == 0, (loaded, stored, stored2)
        for x, y in zip(first, second):
            T.assert_same_bits(x, y, "a kernel loaded from disk")
        for k, f in enumerate(files):
            blob = f.read_bytes()
            if k % 3 == 0:
                f.write_bytes(blob[:len(blob) // 2])
            elif k % 3 == 1:
                f.write_bytes(blob[:100] + bytes([blob[100] ^ 0x40]) + blob[101:])
            else:
                f.write_bytes(b"")
        third, loaded, stored3 = one_device()
        assert loaded == 0 and stored3 == stored, (loaded, stored3)
        for x, y in zip(first, third):
            T.assert_same_bits(x, y, "a kernel compiled again over a damaged file")
        assert all(f.stat().st_size > 1000 for f in files)
    finally:
        del os.environ["AIXHIP_KERNEL_CACHE_DIR"]
    _, loaded, stored = one_device()
    assert loaded == 0 and stored == 0, "no directory named: nothing is read or written"
