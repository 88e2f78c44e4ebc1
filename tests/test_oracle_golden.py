"""The oracle against the literal vectors the reference's own tests hold for the operator path
(tests/golden/reference_literals.json), and against closed forms the mathematics fixes."""
import ctypes as C

import numpy as np
import pytest

import aixtest as T
import goldens
from oracle import cpuref as O

CPU = O.lib()
CASES = goldens.load_cases()


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_reference_literals(case):
    goldens.run_case(case, goldens.OracleBackend())


def test_f16_conversions_match_numpy_exhaustively():
    """f16 -> f32 for all 65536 patterns and f32 -> f16 (RNE) around every boundary vs numpy float16."""
    pats = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    up = np.zeros(65536, np.float32)
    assert CPU.copy(pats.ctypes.data, O.F16, up.ctypes.data, O.F32, 65536) == 0
    want = pats.view(np.float16).astype(np.float32)
    T.assert_same_bits_nan_ok(up, want, O.F32, "f16->f32")
    base = want.view(np.uint32).astype(np.int64)
    nxt = np.roll(base, -1)
    cand = (np.concatenate([base, base + 1, base - 1, (base + nxt) // 2, (base + nxt) // 2 + 1]) & 0xFFFFFFFF).astype(np.uint32)
    f = cand.view(np.float32).copy()
    f = f[~np.isnan(f)]
    dn = np.zeros(f.size, np.uint16)
    assert CPU.copy(f.ctypes.data, O.F32, dn.ctypes.data, O.F16, f.size) == 0
    with np.errstate(over="ignore"):
        T.assert_same_bits(dn, f.astype(np.float16).view(np.uint16), "f32->f16")


def test_bf16_conversions_match_bit_model():
    rng = np.random.default_rng(5)
    f = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 1e3,
                        (rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)).view(np.float32)])
    dn = np.zeros(f.size, np.uint16)
    assert CPU.copy(f.ctypes.data, O.F32, dn.ctypes.data, O.BF16, f.size) == 0
    T.assert_same_bits(dn, O.f32_to_bf16_bits(f), "f32->bf16")
    # closed form: truncation error is at most half a unit of the 8-bit significand, ties to even
    finite = np.isfinite(f) & (np.abs(f) < 3e38)
    back = O.bf16_bits_to_f32(dn)[finite].astype(np.float64)
    x = f[finite].astype(np.float64)
    ulp = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(x), 1e-45))) - 7), 2.0 ** -133)
    assert np.all(np.abs(back - x) <= ulp / 2 * (1 + 1e-12))


@pytest.mark.parametrize("dtype", [O.F64, O.F32, O.F16, O.BF16], ids=lambda d: O.DTYPE_NAMES[d])
def test_float_arithmetic_closed_form(dtype):
    """add/sub/mul/div/neg = the IEEE operation in the evaluation type, rounded once to the type."""
    rng = np.random.default_rng(100 + dtype)
    a = T.contiguous_tensor(rng, dtype, [4000], lo=-8, hi=8)
    b = T.contiguous_tensor(rng, dtype, [4000], lo=-8, hi=8)
    av, bv = a.values(), b.values()
    for op, fn in ((O.ADD, np.add), (O.SUB, np.subtract), (O.MUL, np.multiply), (O.DIV, np.divide)):
        out = T.empty(dtype, [4000])
        assert CPU.binary(op, C.byref(a.desc()), C.byref(b.desc()), C.byref(out.desc())) == 0
        if dtype == O.F64:
            want = fn(av, bv)
        else:   # evaluate in f32 (exact inputs), round to the storage type
            want32 = fn(av.astype(np.float32), bv.astype(np.float32))
            want = O.to_storage(want32, dtype)
        T.assert_same_bits(out.storage, np.asarray(want).astype(O.NP_STORAGE[dtype]) if dtype != O.BF16 else want, f"op {op}")


@pytest.mark.parametrize("dtype", T.INT_DTYPES, ids=lambda d: O.DTYPE_NAMES[d])
def test_integer_arithmetic_wraps(dtype):
    rng = np.random.default_rng(200 + dtype)
    info = np.iinfo(O.NP_STORAGE[dtype])
    a = T.HostTensor(rng.integers(info.min, info.max, 3000, endpoint=True).astype(O.NP_STORAGE[dtype]), dtype, [3000])
    b = T.HostTensor(rng.integers(info.min, info.max, 3000, endpoint=True).astype(O.NP_STORAGE[dtype]), dtype, [3000])
    with np.errstate(over="ignore"):
        for op, fn in ((O.ADD, np.add), (O.SUB, np.subtract), (O.MUL, np.multiply)):
            out = T.empty(dtype, [3000])
            assert CPU.binary(op, C.byref(a.desc()), C.byref(b.desc()), C.byref(out.desc())) == 0
            T.assert_same_bits(out.storage, fn(a.storage, b.storage), f"op {op}")       # numpy wraps too
    bsafe = b.clone()
    bsafe.storage[bsafe.storage == 0] = 1
    if info.min < 0:
        bsafe.storage[bsafe.storage == -1] = 2
    out = T.empty(dtype, [3000])
    assert CPU.binary(O.DIV, C.byref(a.desc()), C.byref(bsafe.desc()), C.byref(out.desc())) == 0
    want = np.trunc(a.storage.astype(np.float64) / bsafe.storage.astype(np.float64)) if dtype != O.I64 else None
    if want is not None:
        T.assert_same_bits(out.storage, want.astype(O.NP_STORAGE[dtype]), "div truncates toward zero")


def test_math_is_correctly_rounded_f32():
    """sqrt/exp/log/pow through long double == float64 evaluation rounded to f32 (bar rare double
    rounding, allowed 1 ulp, never observed on these inputs); sin/cos/tanh within 2 ulp of float64."""
    rng = np.random.default_rng(300)
    x = rng.uniform(-20, 20, 100000).astype(np.float32)
    pos = np.abs(x) + np.float32(1e-3)
    a, p = T.HostTensor(x, O.F32, [x.size]), T.HostTensor(pos, O.F32, [x.size])
    for op, src, fn in ((O.EXP, a, np.exp), (O.LOG, p, np.log), (O.SQRT, p, np.sqrt)):
        out = T.empty(O.F32, [x.size])
        assert CPU.unary(op, C.byref(src.desc()), C.byref(out.desc())) == 0
        want = fn(src.storage.astype(np.float64)).astype(np.float32)
        assert T.ulp_distance(out.storage, want, O.F32) <= (0 if op == O.SQRT else 1)
    for op, fn in ((O.SIN, np.sin), (O.COS, np.cos), (O.TANH, np.tanh)):
        out = T.empty(O.F32, [x.size])
        assert CPU.unary(op, C.byref(a.desc()), C.byref(out.desc())) == 0
        assert T.ulp_distance(out.storage, fn(x.astype(np.float64)).astype(np.float32), O.F32) <= 2
    e = T.HostTensor(rng.uniform(-3, 3, x.size).astype(np.float32), O.F32, [x.size])
    out = T.empty(O.F32, [x.size])
    assert CPU.binary(O.POW, C.byref(p.desc()), C.byref(e.desc()), C.byref(out.desc())) == 0
    want = np.power(p.storage.astype(np.float64), e.storage.astype(np.float64)).astype(np.float32)
    assert T.ulp_distance(out.storage, want, O.F32) <= 1


def test_sum_reduce_matmul_invariants():
    """Textbook pins for the order-dependent kernels: exact on integers-as-floats, linear, and
    equal to float64 brute force within the sequential-f32 error bound."""
    rng = np.random.default_rng(400)
    ints = rng.integers(-50, 50, (37, 41)).astype(np.float32)
    a = T.HostTensor(ints, O.F32, [37, 41])
    out = T.empty(O.F32, [])
    assert CPU.sum(C.byref(a.desc()), C.byref(out.desc())) == 0
    assert out.storage[0] == ints.sum(dtype=np.float64)
    for dshape, axis in (([37, 1], 1), ([1, 41], 0), ([41], 0)):
        dst = T.empty(O.F32, dshape)
        assert CPU.reduce_to(C.byref(a.desc()), C.byref(dst.desc())) == 0
        np.testing.assert_array_equal(dst.storage, ints.sum(axis=axis))
        dst = T.empty(O.F32, dshape, fill=-np.inf)
        assert CPU.max_to(C.byref(a.desc()), C.byref(dst.desc())) == 0
        np.testing.assert_array_equal(dst.storage, ints.max(axis=axis))
    # reduceTo accumulates into dst
    dst = T.empty(O.F32, [37, 1], fill=100.0)
    assert CPU.reduce_to(C.byref(a.desc()), C.byref(dst.desc())) == 0
    np.testing.assert_array_equal(dst.storage, ints.sum(axis=1) + 100.0)
    # matmul: integers exact, identity, transposed operand == numpy on the gathered values
    A = rng.integers(-9, 9, (13, 17)).astype(np.float32)
    B = rng.integers(-9, 9, (17, 11)).astype(np.float32)
    ta = T.HostTensor(A, O.F32, [13, 17])
    tbT = T.HostTensor(np.ascontiguousarray(B.T), O.F32, [17, 11], [1, 17])      # B stored transposed
    out = T.empty(O.F32, [13, 11])
    assert CPU.matmul(C.byref(ta.desc()), C.byref(tbT.desc()), C.byref(out.desc())) == 0
    np.testing.assert_array_equal(out.storage.reshape(13, 11), A.astype(np.float64) @ B.astype(np.float64))
    # the wide variants are float64 dot products
    R = rng.standard_normal((19, 23)).astype(np.float32)
    S = rng.standard_normal((23, 7)).astype(np.float32)
    tr, ts = T.HostTensor(R, O.F32, [19, 23]), T.HostTensor(S, O.F32, [23, 7])
    wide = np.zeros(19 * 7)
    assert CPU.matmul_wide(C.byref(tr.desc()), C.byref(ts.desc()), wide.ctypes.data, None, 2) == 0
    np.testing.assert_allclose(wide.reshape(19, 7), R.astype(np.float64) @ S.astype(np.float64), rtol=1e-13, atol=1e-13)
    lit = T.empty(O.F32, [19, 7])
    assert CPU.matmul(C.byref(tr.desc()), C.byref(ts.desc()), C.byref(lit.desc())) == 0
    np.testing.assert_allclose(lit.storage, wide, rtol=0, atol=23 * 2 ** -23 * (np.abs(R) @ np.abs(S)).max())


def test_matmul_stack_is_the_2d_matmul_per_leading_index():
    """cpuref_matmul_stack (an extension: the reference's matmul is 2-D only) adds nothing but the walk over the
    leading dims: integer stacks equal numpy.matmul exactly, through permuted, sliced and stride-0 views, and a
    float stack equals cpuref_matmul on each pair of matrices bit for bit."""
    rng = np.random.default_rng(450)
    # [2, 3, 5, 4] . [2, 3, 4, 6] on int32, operands seen through views of larger arrays
    base_a = rng.integers(-9, 9, (5, 2, 3, 8)).astype(np.int32)            # stored [m, p, q, 2k]: a[p, q, m, k] = base[m, p, q, 2k]
    base_b = rng.integers(-9, 9, (3, 4, 6)).astype(np.int32)               # stored [q, k, n]: the same for every p (stride 0)
    ta = T.HostTensor(base_a, O.I32, [2, 3, 5, 4], [3 * 8, 8, 2 * 3 * 8, 2])
    tb = T.HostTensor(base_b, O.I32, [2, 3, 4, 6], [0, 24, 6, 1])
    out = T.empty(O.I32, [2, 3, 5, 6])
    assert CPU.matmul_stack(C.byref(ta.desc()), C.byref(tb.desc()), C.byref(out.desc()), 2) == 0
    A = base_a[:, :, :, ::2].transpose(1, 2, 0, 3).astype(np.int64)
    B = np.broadcast_to(base_b.astype(np.int64), (2, 3, 4, 6))
    np.testing.assert_array_equal(out.storage.reshape(2, 3, 5, 6), A @ B)
    # an offset moves every matrix of the stack
    tb_off = T.HostTensor(base_b, O.I32, [2, 2, 4, 6], [0, 24, 6, 1], offset=24)
    ta2 = T.HostTensor(base_a, O.I32, [2, 2, 5, 4], [3 * 8, 8, 2 * 3 * 8, 2])
    out = T.empty(O.I32, [2, 2, 5, 6])
    assert CPU.matmul_stack(C.byref(ta2.desc()), C.byref(tb_off.desc()), C.byref(out.desc()), 1) == 0
    np.testing.assert_array_equal(out.storage.reshape(2, 2, 5, 6), A[:, :2] @ B[:, 1:])
    # floats: the bits of the 2-D function, matrix by matrix
    for dtype in (O.F32, O.BF16):
        fa = O.to_storage(rng.uniform(-1, 1, 4 * 7 * 9), dtype)
        fb = O.to_storage(rng.uniform(-1, 1, 4 * 9 * 5), dtype)
        sa, sb = T.HostTensor(fa, dtype, [4, 7, 9]), T.HostTensor(fb, dtype, [4, 9, 5])
        stack = T.empty(dtype, [4, 7, 5])
        assert CPU.matmul_stack(C.byref(sa.desc()), C.byref(sb.desc()), C.byref(stack.desc()), 3) == 0
        for i in range(4):
            one = T.empty(dtype, [7, 5])
            a2 = T.HostTensor(fa, dtype, [7, 9], offset=i * 63)
            b2 = T.HostTensor(fb, dtype, [9, 5], offset=i * 45)
            assert CPU.matmul(C.byref(a2.desc()), C.byref(b2.desc()), C.byref(one.desc())) == 0
            T.assert_same_bits(stack.storage[i * 35:(i + 1) * 35], one.storage, f"stack matrix {i}")
    # ranks must agree, leading dims must agree
    bad = T.HostTensor(base_b, O.I32, [3, 4, 6])
    assert CPU.matmul_stack(C.byref(ta.desc()), C.byref(bad.desc()), C.byref(out.desc()), 1) != 0


def test_argmax_first_maximum_brute_force():
    rng = np.random.default_rng(500)
    for _ in range(50):
        shape = [int(v) for v in rng.integers(1, 6, 3)]
        x = rng.integers(0, 3, shape).astype(np.float32)
        a = T.HostTensor(x, O.F32, shape)
        out = T.empty(O.I32, [])
        assert CPU.argmax(C.byref(a.desc()), C.byref(out.desc())) == 0
        assert out.storage[0] == int(np.argmax(x))                   # numpy: first occurrence
        for dim in range(3):
            keep = list(shape)
            keep[dim] = 1
            dst = T.empty(O.I32, keep)
            assert CPU.argmax_to(C.byref(a.desc()), C.byref(dst.desc()), dim) == 0
            np.testing.assert_array_equal(dst.storage.reshape(keep), np.argmax(x, axis=dim).reshape(keep))
            hot = T.empty(O.I32, shape)
            assert CPU.argmax_indices_to(C.byref(a.desc()), C.byref(hot.desc()), dim) == 0
            want = np.zeros(shape, np.int32)
            np.put_along_axis(want, np.expand_dims(np.argmax(x, axis=dim), dim), 1, axis=dim)
            np.testing.assert_array_equal(hot.storage.reshape(shape), want)
