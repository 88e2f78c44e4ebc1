"""Row programs: sums and maxima over the last dimension recorded by the lazy device and fused with the elementwise
operators around them into one generated kernel -- Softmax (Targets/AIXLib/aixNeuralNetwork.hpp:188-192: max -> sub ->
exp -> sum -> div) and the pieces of a LayerNorm.

Each case is driven the way the front-end does (fresh result per operator, fillMin / fill of the destination before
maxTo / reduceTo as in aixCore.hpp:873-891, temporaries freed before the read) three ways: fused, with fusion switched
off (the stand-alone kernels, each checked against the oracle in its own tests), and operator by operator on the CPU
oracle.  Bars: fused and unfused give the SAME BITS wherever there is more than one row (the fused kernel sums a row
in the stand-alone row kernel's order; a single row is a whole-tensor sum there, in another order); against the oracle
chain, whose sums run in index order, 1e-5 of the largest result for f32 and 1e-12 for f64.  The 16-bit types add a row
up in bf16 / f16 on the CPU, one rounding per element (aixDeviceCPU.cpp reduceTo accumulates in the element type), which
loses whole digits over a row; their results are held against the same expression in float64 on the same inputs
instead: 2e-2 of the largest result for softmax (4 rounded operators), 4e-2 for the 11 of a LayerNorm.
"""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import devharness as H
from oracle import cpuref as O

pytestmark = pytest.mark.gpu
CPU = O.lib()
NAMES = O.DTYPE_NAMES
TOL = {O.F64: 1e-12, O.F32: 1e-5, O.F16: 2e-2, O.BF16: 2e-2}


@pytest.fixture(scope="module")
def dev():
    d = H.Dev()
    yield d
    d.close()


def set_fusion(dev, on):
    cfg = dev.dev.fuse_config()
    cfg.diagnostics = 1
    cfg.elementwise_fusion = 1 if on else 0
    dev.dev.set_fuse_config(cfg)


class Front:
    """Records on the device and, operator for operator, on the oracle."""

    def __init__(self, dev, dtype):
        self.dev, self.dtype, self.temps, self.leaves = dev, dtype, [], []

    def leaf(self, host):
        p, d = self.dev.put(host)
        node = {"host": host, "ptr": p, "desc": d}
        self.leaves.append(node)
        return node

    def result(self, shape):
        host = T.empty(self.dtype, shape)
        p = self.dev.raw(host.storage.nbytes)
        node = {"host": host, "ptr": p, "desc": H.kdesc(host, p)}
        self.temps.append(node)
        return node

    def over_rows(self, node, shape):
        """[..., 1] read as [..., L] (stride 0 in the last dim), what broadcastTo hands the device."""
        lead = O.row_major(list(shape[:-1]) + [1])[:-1]
        view = T.HostTensor(node["host"].storage, self.dtype, shape, lead + [0])
        return {"host": view, "ptr": node["ptr"], "desc": H.kdesc(view, node["ptr"])}

    def over_all(self, node, shape):
        view = T.HostTensor(node["host"].storage, self.dtype, shape, [0] * len(shape))
        return {"host": view, "ptr": node["ptr"], "desc": H.kdesc(view, node["ptr"])}

    def row_vector(self, node, shape):
        view = T.HostTensor(node["host"].storage, self.dtype, shape, [0] * (len(shape) - 1) + [1])
        return {"host": view, "ptr": node["ptr"], "desc": H.kdesc(view, node["ptr"])}

    def binary(self, op, x, y, shape):
        r = self.result(shape)
        assert CPU.binary(op, C.byref(x["host"].desc()), C.byref(y["host"].desc()), C.byref(r["host"].desc())) == 0
        self.dev.dev.call(["add", "sub", "mul", "div", "pow"][op], H.ref(x["desc"]), H.ref(y["desc"]), H.ref(r["desc"]))
        return r

    def unary(self, op, x, shape):
        r = self.result(shape)
        assert CPU.unary(op, C.byref(x["host"].desc()), C.byref(r["host"].desc())) == 0
        self.dev.dev.call(["unary", "sqrt", "sin", "cos", "tanh", "log", "exp"][op], H.ref(x["desc"]), H.ref(r["desc"]))
        return r

    def scalar(self, value):
        r = self.result([])
        v = np.array([value], dtype=np.float32)
        assert CPU.fill(v.ctypes.data, O.F32, C.byref(r["host"].desc())) == 0
        self.dev.dev.call("fill", v.ctypes.data, O.F32, H.ref(r["desc"]))
        return r

    def row_max(self, x, shape):
        r = self.result(list(shape[:-1]) + [1])
        assert CPU.fill_min(C.byref(r["host"].desc())) == 0 and CPU.max_to(C.byref(x["host"].desc()), C.byref(r["host"].desc())) == 0
        self.dev.dev.call("fill_min", H.ref(r["desc"]))
        self.dev.dev.call("max_to", H.ref(x["desc"]), H.ref(r["desc"]))
        return r

    def row_sum(self, x, shape):
        r = self.result(list(shape[:-1]) + [1])
        zero = np.zeros(1, np.float32)
        assert CPU.fill(zero.ctypes.data, O.F32, C.byref(r["host"].desc())) == 0 and CPU.reduce_to(C.byref(x["host"].desc()), C.byref(r["host"].desc())) == 0
        self.dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(r["desc"]))
        self.dev.dev.call("reduce_to", H.ref(x["desc"]), H.ref(r["desc"]))
        return r

    def free_temps(self, keep=()):
        for t in self.temps:
            if not any(t is k for k in keep):
                self.dev.free(t["ptr"])
        self.temps = [t for t in self.temps if any(t is k for k in keep)]


def softmax(f, x, shape):
    m = f.row_max(x, shape)
    d = f.binary(O.SUB, x, f.over_rows(m, shape), shape)
    e = f.unary(O.EXP, d, shape)
    s = f.row_sum(e, shape)
    return f.binary(O.DIV, e, f.over_rows(s, shape), shape)


def layer_norm(f, x, gamma, beta, shape):
    col = list(shape[:-1]) + [1]
    length = f.scalar(float(shape[-1]))
    mean = f.binary(O.DIV, f.row_sum(x, shape), f.over_all(length, col), col)
    d = f.binary(O.SUB, x, f.over_rows(mean, shape), shape)
    var = f.binary(O.DIV, f.row_sum(f.binary(O.MUL, d, d, shape), shape), f.over_all(length, col), col)
    std = f.unary(O.SQRT, f.binary(O.ADD, var, f.over_all(f.scalar(1e-5), col), col), col)
    n = f.binary(O.DIV, d, f.over_rows(std, shape), shape)
    return f.binary(O.ADD, f.binary(O.MUL, n, f.row_vector(gamma, shape), shape), f.row_vector(beta, shape), shape)


def close_enough(got, want, dtype, what, tol=None):
    g, w = O.to_float64(got, dtype), O.to_float64(want, dtype)
    both_nan = np.isnan(g) & np.isnan(w)
    assert np.array_equal(np.isnan(g), np.isnan(w)), what
    scale = max(float(np.nanmax(np.abs(w), initial=0.0)), 1e-30)
    err = np.where(both_nan, 0.0, np.abs(g - w))
    tol = TOL[dtype] if tol is None else tol
    assert float(err.max(initial=0.0)) <= tol * scale, f"{what}: {float(err.max())} vs {tol * scale}"


def np_softmax(x):
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def run_both(dev, dtype, shape, build, seed, expect_fused_ops=None, lo=-4.0, hi=4.0, poke=None, exact=None, tol16=2e-2):
    outs, want, leaves = [], None, None
    for fusion in (True, False):
        set_fusion(dev, fusion)
        f = Front(dev, dtype)
        rng = np.random.default_rng(seed)
        host = T.contiguous_tensor(rng, dtype, shape, lo=lo, hi=hi)
        if poke is not None:
            poke(host)
        x = f.leaf(host)
        f.leaves = []
        y = build(f, x, rng)
        f.free_temps(keep=(y,))
        outs.append(dev.fetch(y["ptr"], y["host"].storage))
        if fusion and expect_fused_ops is not None:
            diag = dev.dev.diagnostics()
            assert diag.fusible_subgraphs == 1 and diag.fused_ops == expect_fused_ops and diag.fallback_ops == 0, \
                (diag.fusible_subgraphs, diag.fused_ops, diag.fallback_ops, diag.subgraph_summary, diag.fallback_summary)
        want = y["host"].storage
        leaves = [O.to_float64(host.storage, dtype).reshape(shape)] + [O.to_float64(t["host"].storage, dtype) for t in f.leaves]
        dev.release()
    set_fusion(dev, True)
    what = f"{NAMES[dtype]} {shape}"
    if O.numel(shape[:-1]) > 1:
        T.assert_same_bits_nan_ok(outs[0], outs[1], dtype, "fused vs stand-alone kernels " + what)
    else:
        close_enough(outs[0], outs[1], dtype, "fused vs stand-alone kernels " + what)
    if dtype in (O.F32, O.F64):
        close_enough(outs[0], want, dtype, "fused vs oracle " + what)
    if exact is not None:
        with np.errstate(all="ignore"):
            ideal = exact(*leaves).reshape(-1)
        tol = {O.F64: 1e-12, O.F32: 1e-5}.get(dtype, tol16)
        close_enough(outs[0], O.to_storage(ideal, dtype), dtype, "fused vs float64 " + what, tol)
    return outs[0]


# rows shorter than 2048 elements take a wave each, longer ones a workgroup; [9, 1000] and [3, 520] end inside a lane's
# vector run; 3-D shapes reduce the last dim only
FUSED_SHAPES = [[64, 128], [9, 1000], [33, 2048], [5, 4096], [3, 520], [4, 6, 64], [2, 3, 5, 256], [1, 512], [300, 64]]


@pytest.mark.parametrize("dtype", T.FLOAT_DTYPES, ids=lambda d: NAMES[d])
def test_softmax_is_one_kernel_and_matches(dev, dtype):
    for k, shape in enumerate(FUSED_SHAPES):
        got = run_both(dev, dtype, shape, lambda f, x, rng: softmax(f, x, shape), 500 + k, expect_fused_ops=5, exact=np_softmax)
        rows = O.to_float64(got, dtype).reshape(-1, shape[-1]).sum(axis=1)
        assert np.all(np.abs(rows - 1.0) <= (4e-2 if dtype in (O.F16, O.BF16) else 1e-5)), shape     # what the mathematics fixes


@pytest.mark.parametrize("dtype", [O.F32, O.BF16], ids=lambda d: NAMES[d])
def test_rows_the_row_program_does_not_take(dev, dtype):
    """Too long for the registers of a workgroup, not a whole number of 16-byte vectors, or a handful of elements: the
    reductions run as the stand-alone kernels between fused elementwise kernels; same results."""
    vec = 16 // O.ITEMSIZE[dtype]
    for k, shape in enumerate(([2, 8 * 256 * vec * 2], [16, 100 + vec // 2 + 1], [40, 24], [40, 7], [5, 1])):
        run_both(dev, dtype, shape, lambda f, x, rng: softmax(f, x, shape), 600 + k, exact=np_softmax)


@pytest.mark.parametrize("dtype", T.FLOAT_DTYPES, ids=lambda d: NAMES[d])
def test_layer_norm_pieces_are_one_kernel(dev, dtype):
    for k, shape in enumerate(([48, 768], [7, 4096], [2, 5, 256])):
        def build(f, x, rng):
            gamma = f.leaf(T.contiguous_tensor(rng, dtype, [shape[-1]], lo=0.5, hi=1.5))
            beta = f.leaf(T.contiguous_tensor(rng, dtype, [shape[-1]], lo=-0.5, hi=0.5))
            return layer_norm(f, x, gamma, beta, shape)

        def exact(x, gamma, beta):
            d = x - x.mean(axis=-1, keepdims=True)
            return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + np.float64(np.float32(1e-5))) * gamma + beta
        run_both(dev, dtype, shape, build, 700 + k, expect_fused_ops=11, exact=exact, tol16=4e-2)


def test_special_values_in_rows(dev):
    """A row of -inf (its maximum is -inf, x - max is NaN), a NaN in a row (maxTo skips it as std::max does,
    aixDeviceCPU.cpp maxTo; the sum carries it), +inf, and a row of one repeated value."""
    shape = [8, 256]

    def poke(host):
        v = host.storage.reshape(shape)
        v[1, :] = -np.inf
        v[2, 17] = np.nan
        v[3, 200] = np.inf
        v[4, :] = 3.25
        v[5, 0] = np.nan
    run_both(dev, O.F32, shape, lambda f, x, rng: softmax(f, x, shape), 800, expect_fused_ops=5, poke=poke, exact=np_softmax)


def test_row_results_somebody_still_holds_are_stored(dev):
    """The per-row maximum and sum are read after the window as well: the one kernel stores them too."""
    shape = [37, 512]
    for fusion in (True, False):
        set_fusion(dev, fusion)
        f = Front(dev, O.F32)
        x = f.leaf(T.contiguous_tensor(np.random.default_rng(900), O.F32, shape, lo=-3, hi=3))
        m = f.row_max(x, shape)
        d = f.binary(O.SUB, x, f.over_rows(m, shape), shape)
        s = f.row_sum(d, shape)
        y = f.binary(O.DIV, d, f.over_rows(s, shape), shape)
        f.free_temps(keep=(y, m, s))
        got_y = dev.fetch(y["ptr"], y["host"].storage)
        if fusion:
            diag = dev.dev.diagnostics()
            assert diag.fusible_subgraphs == 1 and diag.fused_ops == 4 and diag.fallback_ops == 0, diag.subgraph_summary
        T.assert_same_bits(dev.fetch(m["ptr"], m["host"].storage), m["host"].storage, "row maxima (exact)")
        close_enough(dev.fetch(s["ptr"], s["host"].storage), s["host"].storage, O.F32, "row sums")
        close_enough(got_y, y["host"].storage, O.F32, "quotients")
        dev.release()
    set_fusion(dev, True)


def test_source_overwritten_after_its_reduction(dev):
    """max over x, then x += 1 in place, then x - max: the maximum is of the old x, the difference of the new one."""
    shape = [20, 384]
    outs = []
    for fusion in (True, False):
        set_fusion(dev, fusion)
        f = Front(dev, O.F32)
        x = f.leaf(T.contiguous_tensor(np.random.default_rng(901), O.F32, shape, lo=-3, hi=3))
        x["host"] = x["host"].clone()
        m = f.row_max(x, shape)
        one = f.scalar(1.0)
        ob = f.over_all(one, shape)
        assert CPU.binary(O.ADD, C.byref(x["host"].desc()), C.byref(ob["host"].desc()), C.byref(x["host"].desc())) == 0
        dev.dev.call("add", H.ref(x["desc"]), H.ref(ob["desc"]), H.ref(x["desc"]))
        y = f.binary(O.SUB, x, f.over_rows(m, shape), shape)
        f.free_temps(keep=(y,))
        outs.append(dev.fetch(y["ptr"], y["host"].storage))
        T.assert_same_bits(outs[-1], y["host"].storage, f"(x + 1) - max(x), fusion={fusion}")     # every step is exact or correctly rounded
        dev.release()
    set_fusion(dev, True)


def test_initial_value_of_the_destination_takes_part(dev):
    """reduceTo adds to, and maxTo compares with, what the destination was filled with (aixDeviceCPU.cpp reduceTo /
    maxTo accumulate into dst): a fill of 10 before the row sum, a fill of 2.5 before the row maximum."""
    shape = [12, 320]
    for fusion in (True, False):
        set_fusion(dev, fusion)
        f = Front(dev, O.F32)
        x = f.leaf(T.contiguous_tensor(np.random.default_rng(902), O.F32, shape, lo=-3, hi=3))
        col = [12, 1]
        s, m = f.result(col), f.result(col)
        for node, value, cpu, name in ((s, 10.0, CPU.reduce_to, "reduce_to"), (m, 2.5, CPU.max_to, "max_to")):
            v = np.array([value], np.float32)
            assert CPU.fill(v.ctypes.data, O.F32, C.byref(node["host"].desc())) == 0 and cpu(C.byref(x["host"].desc()), C.byref(node["host"].desc())) == 0
            dev.dev.call("fill", v.ctypes.data, O.F32, H.ref(node["desc"]))
            dev.dev.call(name, H.ref(x["desc"]), H.ref(node["desc"]))
        y = f.binary(O.MUL, f.binary(O.SUB, x, f.over_rows(s, shape), shape), f.over_rows(m, shape), shape)
        f.free_temps(keep=(y, m))
        close_enough(dev.fetch(y["ptr"], y["host"].storage), y["host"].storage, O.F32, f"(x - (10 + sum)) * max(2.5, max), fusion={fusion}")
        got_m = dev.fetch(m["ptr"], m["host"].storage)
        T.assert_same_bits(got_m, m["host"].storage, "maxima with a floor")
        assert got_m.min() >= 2.5
        dev.release()
    set_fusion(dev, True)


def _random_program(dev, rng, dtype, rows, length, steps, fusion):
    """One random program of exact operators on small integer values (every sum and product stays exactly representable,
    so the order of a sum does not matter and all three evaluations must agree bit for bit): full [rows, length] tensors,
    one-value-per-row tensors from row maxima and row sums (fills folded or not), broadcasts of them, a row vector, scalars,
    in-place updates, operators that run at once in between (which flush the window), temporaries freed along the way."""
    set_fusion(dev, fusion)
    f = Front(dev, dtype)
    shape, col = [rows, length], [rows, 1]
    small = lambda n: O.to_storage(rng.integers(-2, 3, n).astype(np.float64), dtype)            # noqa: E731
    full = [f.leaf(T.HostTensor(small(rows * length), dtype, shape)) for _ in range(3)]
    cols = [f.leaf(T.HostTensor(small(rows), dtype, col))]
    vec = f.leaf(T.HostTensor(small(length), dtype, [length]))
    bound = {id(t): 2.0 for t in full + cols}                        # largest magnitude a tensor can hold
    limit = 2.0 ** (7 if dtype in (O.F16, O.BF16) else 20)           # 16-bit types: integers up to 256 are exact
    kept = []
    for step in range(steps):
        kind = int(rng.integers(0, 12))
        x = full[int(rng.integers(0, len(full)))]
        if kind < 3:                                                 # full op full
            y = full[int(rng.integers(0, len(full)))]
            op = int(rng.choice([O.ADD, O.SUB, O.MUL]))
            b = bound[id(x)] * bound[id(y)] if op == O.MUL else bound[id(x)] + bound[id(y)]
            if b > limit:
                continue
            r = f.binary(op, x, y, shape)
            bound[id(r)] = b
            full.append(r)
        elif kind < 5:                                               # full op (one value per row, broadcast along the row)
            c = cols[int(rng.integers(0, len(cols)))]
            op = int(rng.choice([O.ADD, O.SUB, O.MUL]))
            b = bound[id(x)] * bound[id(c)] if op == O.MUL else bound[id(x)] + bound[id(c)]
            if b > limit:
                continue
            r = f.binary(op, x, f.over_rows(c, shape), shape)
            bound[id(r)] = b
            full.append(r)
        elif kind == 5:                                              # full op row vector / scalar
            if bound[id(x)] + 2 > limit:
                continue
            other = f.row_vector(vec, shape) if rng.integers(0, 2) else f.over_all(f.scalar(float(rng.integers(-2, 3))), shape)
            r = f.binary(int(rng.choice([O.ADD, O.SUB])), x, other, shape)
            bound[id(r)] = bound[id(x)] + 2
            full.append(r)
        elif kind == 6:
            r = f.unary(O.NEG, x, shape)
            bound[id(r)] = bound[id(x)]
            full.append(r)
        elif kind < 9:                                               # row maximum / row sum
            if kind == 7:
                r = f.row_max(x, shape)
                bound[id(r)] = bound[id(x)]
            else:
                if bound[id(x)] * length > limit:
                    continue
                r = f.row_sum(x, shape)
                bound[id(r)] = bound[id(x)] * length
            cols.append(r)
        elif kind == 9:                                              # per-row arithmetic
            a, c = cols[int(rng.integers(0, len(cols)))], cols[int(rng.integers(0, len(cols)))]
            if bound[id(a)] + bound[id(c)] > limit:
                continue
            r = f.binary(int(rng.choice([O.ADD, O.SUB])), a, c, col)
            bound[id(r)] = bound[id(a)] + bound[id(c)]
            cols.append(r)
        elif kind == 10:                                             # in-place update of an earlier result
            y = full[int(rng.integers(0, len(full)))]
            if x is y or bound[id(x)] + bound[id(y)] > limit or not any(x is t for t in f.temps):
                continue
            assert CPU.binary(O.ADD, C.byref(x["host"].desc()), C.byref(y["host"].desc()), C.byref(x["host"].desc())) == 0
            dev.dev.call("add", H.ref(x["desc"]), H.ref(y["desc"]), H.ref(x["desc"]))
            bound[id(x)] += bound[id(y)]
        else:                                                        # an operator that runs at once: contiguous copy of a transposed view
            t_view = T.HostTensor(x["host"].storage, dtype, [length, rows], [1, length])
            r = f.result([length, rows])
            assert CPU.contiguous(C.byref(t_view.desc()), C.byref(r["host"].desc())) == 0
            dev.dev.call("contiguous", H.ref(H.kdesc(t_view, x["ptr"])), H.ref(r["desc"]))
            kept.append(r)
        if rng.integers(0, 5) == 0 and len(f.temps) > 4:             # free a temporary nobody will name again
            victim = f.temps[int(rng.integers(0, len(f.temps)))]
            if not any(victim is k for k in kept) and victim is not full[-1]:
                full = [t for t in full if t is not victim]
                cols = [t for t in cols if t is not victim] or cols
                if any(t is victim for t in full + cols):
                    continue
                f.temps = [t for t in f.temps if t is not victim]
                dev.free(victim["ptr"])
    kept += [t for t in (full[-3:] + cols[-2:]) if any(t is k for k in f.temps)]
    f.free_temps(keep=kept)
    got = [(dev.fetch(t["ptr"], t["host"].storage), t["host"].storage.copy()) for t in kept]
    dev.release()
    return got


@pytest.mark.parametrize("dtype", [O.F32, O.BF16, O.F64], ids=lambda d: NAMES[d])
def test_random_programs_with_row_reductions(dev, dtype):
    for trial in range(10):
        seed = 9000 + 100 * dtype + trial
        rows = int(np.random.default_rng(seed).integers(1, 24))
        length = int(np.random.default_rng(seed + 1).choice([32, 64, 96, 256, 1000 if dtype != O.BF16 else 1024, 2048]))
        fused = _random_program(dev, np.random.default_rng(seed), dtype, rows, length, 30, True)
        plain = _random_program(dev, np.random.default_rng(seed), dtype, rows, length, 30, False)
        assert len(fused) == len(plain) and len(fused) > 0
        for k, ((g1, want), (g2, _)) in enumerate(zip(fused, plain)):
            what = f"{NAMES[dtype]} trial {trial} [{rows}, {length}] tensor {k}"
            T.assert_same_bits(g1, want, "fused vs oracle " + what)
            T.assert_same_bits(g2, want, "unfused vs oracle " + what)
    set_fusion(dev, True)


# ---- triangles and blocks of rows inside a row program -------------------------------------------------------------
def _tri(f, name, x, shape, diagonal):
    r = f.result(shape)
    assert getattr(CPU, name)(C.byref(x["host"].desc()), C.byref(r["host"].desc()), diagonal) == 0
    f.dev.dev.call(name, H.ref(x["desc"]), H.ref(r["desc"]), diagonal)
    return r


def _block(f, node, shape, block_dims):
    """A dense block (the last `block_dims` dims of `shape`) under leading dims of stride 0: the [seq, seq] mask of
    attention under [batch, heads, seq, seq] scores."""
    strides = [0] * (len(shape) - block_dims) + O.row_major(shape[-block_dims:])
    view = T.HostTensor(node["host"].storage, f.dtype, shape, strides)
    return {"host": view, "ptr": node["ptr"], "desc": H.kdesc(view, node["ptr"])}


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.F16], ids=lambda d: NAMES[d])
def test_attention_scores_to_probabilities_is_one_kernel(dev, dtype):
    """softmax(tril(s) * scale + mask) over [batch, heads, seq, seq] scores with a [seq, seq] additive mask
    (frontend/transformer.hpp; aixNeuralNetwork.hpp:188-192 for the softmax): the triangle's rows are the rows the
    program works on and the mask is a block of rows that every seq rows see again, so the eight operators are ONE
    kernel.  Fused = stand-alone kernels bit for bit; both against the oracle's operator chain and float64."""
    for k, (shape, diagonal) in enumerate([([2, 3, 64, 64], 0), ([1, 2, 128, 128], 0), ([3, 32, 256], -1), ([2, 40, 96], 2)]):
        seq = shape[-1]

        def build(f, x, rng, shape=shape, diagonal=diagonal, seq=seq):
            mask_host = T.contiguous_tensor(rng, dtype, shape[-2:], lo=-1.0, hi=0.0)
            upper = np.triu(np.ones(shape[-2:], bool), 1 + diagonal).reshape(-1)
            mask_host.storage[upper] = O.to_storage(np.full(int(upper.sum()), -30000.0), dtype)
            mask = f.leaf(mask_host)
            t = _tri(f, "tril", x, shape, diagonal)
            scaled = f.binary(O.MUL, t, f.over_all(f.scalar(0.125), shape), shape)
            return softmax(f, f.binary(O.ADD, scaled, _block(f, mask, shape, 2), shape), shape)

        def exact(x, m, diagonal=diagonal, shape=shape):
            keep = np.tril(np.ones(shape[-2:]), diagonal)
            return np_softmax(x * keep * 0.125 + m.reshape(shape[-2:]))

        got = run_both(dev, dtype, shape, build, 900 + k, expect_fused_ops=8, exact=exact)
        rows = O.to_float64(got, dtype).reshape(-1, seq).sum(axis=1)
        assert np.all(np.abs(rows - 1.0) <= (4e-2 if dtype in (O.F16, O.BF16) else 1e-5)), shape


@pytest.mark.parametrize("dtype", [O.BF16, O.F32], ids=lambda d: NAMES[d])
def test_triangle_after_a_row_sum_stays_in_the_kernel(dev, dtype):
    """The gradient side: y = triu / tril of (x - rowsum(x) * x) * scale -- a per-row value, two products and a triangle
    in one row program, for matrices stacked under leading dims."""
    for k, (shape, name, diagonal) in enumerate([([4, 64, 64], "tril", 0), ([2, 2, 32, 128], "triu", 1), ([96, 512], "tril", -3)]):
        def build(f, x, rng, shape=shape, name=name, diagonal=diagonal, k=k):
            # the factor: a fill of this window (an immediate of the kernel) or a scalar tensor that lies in memory (the
            # scale of attention, made in the forward pass, when the backward pass uses it): one element seen from
            # everywhere.  (Uploaded first: an upload flushes the window.)
            stored = f.leaf(T.HostTensor(O.to_storage(np.array([0.5]), dtype), dtype, [])) if k == 1 else None
            s = f.row_sum(x, shape)
            d = f.binary(O.SUB, x, f.binary(O.MUL, x, f.over_rows(s, shape), shape), shape)
            half = stored if stored is not None else f.scalar(0.5)
            return _tri(f, name, f.binary(O.MUL, d, f.over_all(half, shape), shape), shape, diagonal)

        def exact(x, *more, shape=shape, name=name, diagonal=diagonal):
            keep = (np.tril if name == "tril" else np.triu)(np.ones(shape[-2:]), diagonal)
            return (x - x * x.sum(axis=-1, keepdims=True)) * 0.5 * keep

        run_both(dev, dtype, shape, build, 950 + k, expect_fused_ops=5, lo=-0.5, hi=0.5, exact=exact, tol16=4e-2)


# ---- the place of every row's first maximum inside a row program ----------------------------------------------------
def _onehot_of_row_maxima(f, x, shape):
    """fill(0) + argmaxIndicesTo along the last dim (aixCore.hpp:927-941), then the cast to the working type that
    `seed * mask` makes (aixCore.hpp:2170-2175, 1616-1630)."""
    mask_host = T.empty(O.I32, shape)
    zero = np.zeros(1, np.float32)
    assert CPU.fill(zero.ctypes.data, O.F32, C.byref(mask_host.desc())) == 0
    assert CPU.argmax_indices_to(C.byref(x["host"].desc()), C.byref(mask_host.desc()), len(shape) - 1) == 0
    pm = f.dev.raw(mask_host.storage.nbytes)
    dm = H.kdesc(mask_host, pm)
    f.temps.append({"host": mask_host, "ptr": pm, "desc": dm})
    f.dev.dev.call("fill", zero.ctypes.data, O.F32, H.ref(dm))
    f.dev.dev.call("argmax_indices_to", H.ref(x["desc"]), H.ref(dm), len(shape) - 1)
    r = f.result(shape)
    assert CPU.copy(mask_host.storage.ctypes.data, O.I32, r["host"].storage.ctypes.data, f.dtype, mask_host.size) == 0
    f.dev.dev.call("copy", pm, O.I32, r["ptr"], f.dtype, mask_host.size)
    return r


@pytest.mark.parametrize("dtype", [O.BF16, O.F32, O.F16], ids=lambda d: NAMES[d])
def test_onehot_of_row_maxima_stays_in_the_kernel(dev, dtype):
    """max()'s backward as the softmax gradient has it: y = x * rowsum(x) + cast(onehot(x)) * rowsum(x) -- the row sum, the
    one-hot of every row's first maximum, its conversion and two products in ONE row program; the int32 mask is gone
    before the read and is never written.  Ties (values on a coarse grid), a row of NaNs, a NaN in column 0 and NaNs
    elsewhere: as the stand-alone operator has them, bit for bit."""
    for k, shape in enumerate([[64, 128], [3, 5, 512], [9, 1000], [4, 2048], [1, 64]]):
        def poke(host, shape=shape):
            vals = O.to_float64(host.storage, dtype).reshape(-1, shape[-1])
            vals = np.round(vals * 2) / 2                                  # many equal maxima: the first one wins
            if vals.shape[0] >= 4:
                vals[1, :] = np.nan                                        # nothing to compare: the leading NaN wins
                vals[2, 0] = np.nan                                        # a leading NaN wins over everything
                vals[3, 5] = np.nan                                        # a NaN elsewhere is no candidate
            host.storage[:] = O.to_storage(vals.reshape(-1), dtype)

        def build(f, x, rng, shape=shape):
            s = f.row_sum(x, shape)
            a = f.binary(O.MUL, x, f.over_rows(s, shape), shape)
            m = _onehot_of_row_maxima(f, x, shape)
            return f.binary(O.ADD, a, f.binary(O.MUL, m, f.over_rows(s, shape), shape), shape)

        got = run_both(dev, dtype, shape, build, 980 + k, expect_fused_ops=6, lo=-2.0, hi=2.0, poke=poke)
        assert got.size == O.numel(shape)
