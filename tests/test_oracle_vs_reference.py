"""Bit-exact A/B of the CPU checker against the real reference CPU backend
(oracle/_ref, built in place from /root/reference where that is mounted).

The reference build has no 16-bit float kernels (they need <stdfloat>), so this
covers the integer, fp32, fp64 and complex paths: flat, broadcast, strided,
transposed and batched forms of every entry point.
"""
import itertools

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import ops, types

INTS = [ta.int8, ta.int16, ta.int32, ta.int64]
REALS = [ta.float32, ta.float64]
SEED = 11


def run_both(oracle, reference, fn):
    with support.use_functions(oracle):
        a = fn()
    with support.use_functions(reference):
        b = fn()
    return a, b


def check(oracle, reference, fn, what):
    a, b = run_both(oracle, reference, fn)
    support.assert_bit_exact(a.storage(), b.storage(), what)


def make(dtype, tid, shape, low=-4, high=4):
    return support.host_tensor(support.values_for(dtype, SEED, tid, shape, low, high), dtype)


BINARY_LAYOUTS = {
    "flat": ((4, 5, 6), (4, 5, 6), [], []),
    "broadcast": ((2, 1, 3), (1, 4, 3), [], []),
    "rank_mismatch": ((3,), (2, 4, 3), [], []),
    "scalar_operand": ((4, 5), (1,), [], []),
    "transposed": ((5, 4), (4, 5), [("transpose", (0, 1))], []),
    "expanded": ((1, 6), (5, 6), [("expand", (5, 6))], []),
    "sliced": ((6, 8), (3, 4), [("index", (slice(0, 6, 2), slice(1, 8, 2)))], []),
    "singleton": ((1, 1), (1,), [], []),
}
PAIRS = ([(d, d) for d in INTS + REALS + [ta.complex64, ta.complex128]] +
         [(ta.int8, ta.int32), (ta.int64, ta.int16), (ta.int32, ta.float32), (ta.float64, ta.int32), (ta.float32, ta.float64)])


@pytest.mark.parametrize("layout", list(BINARY_LAYOUTS))
@pytest.mark.parametrize("pair", PAIRS, ids=lambda p: f"{p[0]}-{p[1]}")
@pytest.mark.parametrize("op", ["add", "sub", "mul"])
def test_binary(oracle, reference, op, pair, layout):
    sa, sb, va, vb = BINARY_LAYOUTS[layout]
    a = support.apply_view(make(pair[0], 1, sa), va)
    b = support.apply_view(make(pair[1], 2, sb), vb)
    check(oracle, reference, lambda: getattr(ops, op)(a, b), f"{op} {pair} {layout}")


@pytest.mark.parametrize("pair", [(ta.float32, ta.float32), (ta.float64, ta.float64), (ta.int32, ta.float32), (ta.float32, ta.float64)],
                         ids=lambda p: f"{p[0]}-{p[1]}")
def test_pow(oracle, reference, pair):
    a = make(pair[0], 3, (3, 1, 5), 0, 4)
    b = make(pair[1], 4, (1, 4, 5), -3, 3)
    check(oracle, reference, lambda: ops.pow(a, b), f"pow {pair}")


UNARY = ["log", "exp", "sqrt", "abs", "sin", "cos", "tan", "sinh", "cosh", "tanh", "neg", "repack"]


@pytest.mark.parametrize("view", ["contiguous", "transposed", "sliced", "singleton"])
@pytest.mark.parametrize("dtype", REALS, ids=str)
@pytest.mark.parametrize("op", UNARY + ["rsqrt"])
def test_unary(oracle, reference, op, dtype, view):
    x = make(dtype, 5, (6, 8), 0.25, 4) if view != "singleton" else make(dtype, 5, (1, 1), 0.25, 4)
    if view == "transposed":
        x = x.transpose(0, 1)
    elif view == "sliced":
        x = x[1:6:2, ::3]
    fn = (lambda: ops.rsqrt(x, 1e-5)) if op == "rsqrt" else (lambda: getattr(ops, op)(x))
    check(oracle, reference, fn, f"{op} {dtype} {view}")


@pytest.mark.parametrize("dtype", INTS + [ta.complex64, ta.complex128], ids=str)
@pytest.mark.parametrize("op", ["neg", "repack"])
def test_unary_other_types(oracle, reference, op, dtype):
    x = make(dtype, 6, (3, 5, 2)).transpose(0, 2)
    check(oracle, reference, lambda: getattr(ops, op)(x), f"{op} {dtype}")


@pytest.mark.parametrize("dtype", [ta.int32, ta.int64], ids=str)
def test_abs_integers(oracle, reference, dtype):
    x = make(dtype, 7, (4, 9), -100, 100)
    check(oracle, reference, lambda: ops.abs(x), f"abs {dtype}")


@pytest.mark.parametrize("view", ["contiguous", "transposed", "singleton"])
@pytest.mark.parametrize("dtype", INTS + REALS, ids=str)
def test_scale(oracle, reference, dtype, view):
    x = make(dtype, 8, (1,) if view == "singleton" else (5, 7), -100, 100)
    if view == "transposed":
        x = x.transpose(0, 1)
    check(oracle, reference, lambda: ops.scale(x, 3), f"scale {dtype} {view}")


@pytest.mark.parametrize("dtype", INTS + REALS, ids=str)
@pytest.mark.parametrize("op", ["eq", "ne", "gt", "ge", "lt", "le"])
def test_compare(oracle, reference, op, dtype):
    a = support.values_for(dtype, SEED, 9, (3, 7, 5), -3, 3)
    b = support.values_for(dtype, SEED, 10, (3, 7, 5), -3, 3)
    if dtype.is_floating:
        a = np.round(a)
        b = np.round(b)
        a[0, 0, 0] = np.nan
        b[1, 1, 1] = np.nan
        a[2, 2, 2] = b[2, 2, 2] = np.nan
    ta_, tb_ = support.host_tensor(a, dtype), support.host_tensor(b, dtype)
    check(oracle, reference, lambda: getattr(ops, op)(ta_, tb_), f"{op} {dtype}")
    va, vb = ta_.transpose(0, 2), support.host_tensor(np.ascontiguousarray(b.transpose(2, 1, 0)), dtype)
    check(oracle, reference, lambda: getattr(ops, op)(va, vb), f"{op} {dtype} strided")


@pytest.mark.parametrize("view", ["contiguous", "transposed", "singleton_axis"])
@pytest.mark.parametrize("axis", [0, 1, 2])
@pytest.mark.parametrize("dtype", INTS + REALS, ids=str)
@pytest.mark.parametrize("op", ["sum", "mean", "argmax", "argmin"])
def test_reduce(oracle, reference, op, dtype, axis, view):
    if op == "mean" and dtype.is_integral:
        pytest.skip("mean has no integer kernel")
    shape = (4, 1, 6) if view == "singleton_axis" else (4, 5, 6)
    x = make(dtype, 12, shape, -3, 3)
    if view == "transposed":
        x = x.transpose(0, 2)
    check(oracle, reference, lambda: getattr(ops, op)(x, axis, True), f"{op} {dtype} axis={axis} {view}")


def test_argmax_ties_nan_and_infinities(oracle, reference):
    x = np.array([[1, 5, 5, 2], [np.nan, np.nan, np.nan, np.nan], [-np.inf, -np.inf, -np.inf, -np.inf],
                  [np.nan, 3, 3, np.nan], [np.inf, 1, np.inf, 0]], dtype=np.float32)
    t = support.host_tensor(x, ta.float32)
    for op in ("argmax", "argmin"):
        for axis in (0, 1):
            check(oracle, reference, lambda: getattr(ops, op)(t, axis), f"{op} edge axis={axis}")
    i = support.host_tensor(np.array([[-128, -128, -128], [127, 127, 3]], dtype=np.int8), ta.int8)
    for op in ("argmax", "argmin"):
        check(oracle, reference, lambda: getattr(ops, op)(i, 1), f"{op} int8 limits")


GEMM_PAIRS = [(ta.float32, ta.float32), (ta.float64, ta.float64), (ta.int8, ta.int8), (ta.int16, ta.int32), (ta.int32, ta.int32),
              (ta.int64, ta.int8), (ta.int32, ta.float32), (ta.float64, ta.float32)]
GEMM_LAYOUTS = {
    "nn": ((5, 7), (7, 3), [], []),
    "nt": ((5, 7), (3, 7), [], [("transpose", (-1, -2))]),
    "tn": ((7, 5), (7, 3), [("transpose", (-1, -2))], []),
    "tt": ((7, 5), (3, 7), [("transpose", (-1, -2))], [("transpose", (-1, -2))]),
    "batched": ((2, 3, 5, 7), (2, 3, 7, 4), [], []),
    "batch_broadcast": ((2, 1, 5, 7), (1, 3, 7, 4), [], []),
    "rank4_rank2_nt": ((2, 3, 4, 6), (5, 6), [], [("transpose", (-1, -2))]),
    "rank3_rank4": ((3, 5, 7), (2, 3, 7, 4), [], []),
    "single_row": ((1, 9), (9, 4), [], []),
    "single_column": ((6, 9), (1, 9), [], [("transpose", (-1, -2))]),
}


@pytest.mark.parametrize("layout", list(GEMM_LAYOUTS))
@pytest.mark.parametrize("pair", GEMM_PAIRS, ids=lambda p: f"{p[0]}-{p[1]}")
def test_gemm(oracle, reference, pair, layout):
    sa, sb, va, vb = GEMM_LAYOUTS[layout]
    a = support.apply_view(make(pair[0], 13, sa), va)
    b = support.apply_view(make(pair[1], 14, sb), vb)
    check(oracle, reference, lambda: ops.matmul(a, b), f"gemm {pair} {layout}")


CONV_CASES = {
    "k3_s1_p1": ((2, 3, 6, 7), (4, 3, 3, 3), (1, 1), (1, 1)),
    "k7_s2_p3": ((1, 3, 16, 16), (2, 3, 7, 7), (2, 2), (3, 3)),
    "k1_s2_p0": ((2, 4, 8, 8), (3, 4, 1, 1), (2, 2), (0, 0)),
    "rect": ((1, 2, 7, 5), (3, 2, 3, 2), (2, 1), (0, 2)),
}


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("dtype", [ta.float32, ta.float64, ta.int32, ta.int8], ids=str)
@pytest.mark.parametrize("name", list(CONV_CASES))
def test_conv2d(oracle, reference, name, dtype, bias):
    xs, ws, stride, pad = CONV_CASES[name]
    x, w = make(dtype, 15, xs), make(dtype, 16, ws)
    b = make(dtype, 17, (ws[0],)) if bias else None
    check(oracle, reference, lambda: ops.convolve2d(x, w, b, stride, pad), f"conv2d {name} {dtype} bias={bias}")


def test_conv2d_strided_signal(oracle, reference):
    x = make(ta.float32, 18, (2, 6, 7, 3)).permute(0, 3, 1, 2)
    w = make(ta.float32, 19, (4, 3, 3, 3))
    check(oracle, reference, lambda: ops.convolve2d(x, w, None, 1, 1), "conv2d NHWC view")


def test_conv2d_status_codes(oracle, reference):
    x, w = make(ta.float32, 20, (1, 3, 5, 5)), make(ta.float32, 21, (2, 4, 3, 3))
    for lib in (oracle, reference):
        f = lib.functions["conv2d"]
        y = ta.Tensor(ta.float32, (1, 2, 3, 3)).initialize(ta.Host())
        dx, dw, dy = x.descriptor(), w.descriptor(), y.descriptor()
        import ctypes as C
        from tannic_amd import abi
        assert f(C.byref(dx), C.byref(dw), C.byref(dy), abi.SIZE2(0, 0), abi.SIZE2(1, 1)) == abi.ERROR  # channel mismatch
        dw16 = make(ta.int32, 22, (2, 3, 3, 3)).descriptor()
        assert f(C.byref(dx), C.byref(dw16), C.byref(dy), abi.SIZE2(0, 0), abi.SIZE2(1, 1)) == abi.UNSUPPORTED_DTYPE


@pytest.mark.parametrize("pair", [(ta.float32, ta.float32), (ta.float64, ta.float64), (ta.float32, ta.float64), (ta.int32, ta.float32),
                                  (ta.int8, ta.int16)], ids=lambda p: f"{p[0]}-{p[1]}")
@pytest.mark.parametrize("op", ["view_as_cartesian", "view_as_polar"])
def test_complex_construction(oracle, reference, op, pair):
    a = make(pair[0], 23, (4, 1, 3), 0, 3)
    b = make(pair[1], 24, (4, 5, 3), -3, 3)
    comp = ta.float64 if ta.float64 in pair else ta.float32
    ctype = ta.complex64 if comp is ta.float32 else ta.complex128

    def fn():
        out = ta.Tensor(ctype, (4, 5, 3)).initialize(ta.Host())
        return ops._call(op, ta.Host(), [a, b], out)
    check(oracle, reference, fn, f"{op} {pair}")


@pytest.mark.parametrize("dtype", INTS + REALS + [ta.complex64], ids=str)
def test_cpy_into_strided_destination(oracle, reference, dtype):
    src = make(dtype, 25, (3, 1, 4)).transpose(0, 2)

    def fn():
        dst = make(dtype, 26, (8, 2, 6))
        ops.copy_into(dst[::2, 0:1, ::2], src)
        return dst
    check(oracle, reference, fn, f"cpy {dtype}")


def test_allclose(oracle, reference):
    a = make(ta.float32, 27, (5, 6))
    b = support.host_tensor(a.numpy() * (1 + 5e-6), ta.float32)
    c = support.host_tensor(a.numpy() + 1e-3, ta.float32)
    n = support.host_tensor(np.full((5, 6), np.nan), ta.float32)
    for lib in (oracle, reference):
        with support.use_functions(lib):
            assert ops.allclose(a, b) is True
            assert ops.allclose(a, c) is False
            assert ops.allclose(a, c, atol=2e-3) is True
            assert ops.allclose(a.transpose(), support.host_tensor(a.numpy().T.copy(), ta.float32)) is True
            assert ops.allclose(a, n) is True  # NaN differences never trip the test
            with pytest.raises(ta.TannicError):
                ops.allclose(make(ta.int32, 28, (2,)), make(ta.int32, 28, (2,)))


REPEAT_VIEWS = {
    "plain": ((2, 3, 4), []),
    "permuted": ((2, 3, 4), [("permute", (2, 0, 1))]),
    "sliced": ((4, 6, 5), [("index", (slice(0, 4, 2), slice(1, 6, 2), slice(0, 5, 1)))]),
    "expanded": ((1, 3, 1), [("expand", (2, 3, 4))]),
    "vector": ((5,), []),
}


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
@pytest.mark.parametrize("view", list(REPEAT_VIEWS))
@pytest.mark.parametrize("dtype", INTS + REALS, ids=str)
def test_repeat(oracle, reference, dtype, view, axis):
    shape, spec = REPEAT_VIEWS[view]
    x = support.apply_view(make(dtype, 31, shape), spec)
    if axis >= x.rank:
        pytest.skip("axis beyond the rank")
    check(oracle, reference, lambda: ops.repeat(x, 3, axis), f"repeat {dtype} {view} axis {axis}")


@pytest.mark.parametrize("k", [0, 1, 3, -1, -2, 7, -7])
@pytest.mark.parametrize("view", ["plain", "transposed", "sliced"])
@pytest.mark.parametrize("op", ["triu", "tril"])
@pytest.mark.parametrize("dtype", [ta.int32, ta.int64] + REALS, ids=str)
def test_triangular(oracle, reference, dtype, op, view, k):
    x = make(dtype, 32, (5, 6))
    if view == "transposed":
        x = x.transpose(0, 1)
    elif view == "sliced":
        x = x[1:5, 0:6:2]
    check(oracle, reference, lambda: getattr(ops, op)(x, k), f"{op} {dtype} {view} k={k}")


def test_triangular_rejects_other_ranks(oracle, reference):
    x = make(ta.float32, 33, (2, 3, 4))
    for lib in (oracle, reference):
        with support.use_functions(lib):
            with pytest.raises(ops.TannicError):
                ops.triu(x, 0)


CONV1D_CASES = {
    "plain": ((2, 3, 17), (4, 3, 5), 1, 0),
    "stride_pad": ((1, 2, 20), (3, 2, 4), 3, 2),
    "wide_pad": ((2, 1, 4), (2, 1, 3), 1, 4),
    "one_output": ((1, 4, 6), (5, 4, 6), 1, 0),
}


@pytest.mark.parametrize("name", list(CONV1D_CASES))
@pytest.mark.parametrize("dtype", INTS + REALS, ids=str)
def test_conv1d(oracle, reference, dtype, name):
    xs, ws, stride, pad = CONV1D_CASES[name]
    x, w = make(dtype, 41, xs, -3, 3), make(dtype, 42, ws, -3, 3)
    check(oracle, reference, lambda: ops.convolve1d(x, w, stride, pad), f"conv1d {dtype} {name}")


def test_conv1d_strided_signal_and_status(oracle, reference):
    x = make(ta.float32, 43, (2, 12, 3)).transpose(1, 2)          # [2, 3, 12] with the length stride 3
    w = make(ta.float32, 44, (4, 3, 5))
    check(oracle, reference, lambda: ops.convolve1d(x, w, 2, 1), "conv1d strided signal")
    bad = ta.Tensor(ta.float32, (1, 4, 2)).initialize(ta.Host())
    for lib in (oracle, reference):
        with support.use_functions(lib):
            with pytest.raises(ops.TannicError):      # destination of the wrong shape: ERROR
                ops._call("conv1d", ta.Host(), [x, w], bad, extra=(ops.C.c_size_t(1), ops.C.c_size_t(2)))


# concat: the reference addresses the block behind the axis with one stride, so the A/B covers what it gets right —
# at most one dimension behind the axis — with every kind of view in front of it
CONCAT_CASES = {
    "rows": ((2, 3), (4, 3), 0, [], []),
    "columns": ((3, 2), (3, 5), 1, [], []),
    "last_axis_rank3": ((2, 3, 4), (2, 3, 2), 2, [], []),
    "middle_axis_rank3": ((2, 3, 4), (2, 5, 4), 1, [], []),
    "transposed_operand": ((2, 4, 3), (2, 5, 3), 1, [("transpose", (1, 2))], []),   # first becomes [2, 3, 4]... see below
    "expanded_operand": ((1, 1, 3), (2, 4, 3), 1, [("expand", (2, 1, 3))], []),
    "sliced_operands": ((4, 6), (4, 8), 1, [("index", (slice(0, 4, 2), slice(0, 6, 2)))], [("index", (slice(1, 4, 2), slice(0, 8, 2)))]),
    "vectors": ((5,), (3,), 0, [], []),
}


@pytest.mark.parametrize("name", [n for n in CONCAT_CASES if n != "transposed_operand"])
@pytest.mark.parametrize("dtype", INTS + REALS, ids=str)
def test_concat(oracle, reference, dtype, name):
    sa, sb, axis, va, vb = CONCAT_CASES[name]
    a = support.apply_view(make(dtype, 51, sa), va)
    b = support.apply_view(make(dtype, 52, sb), vb)
    check(oracle, reference, lambda: ops.concatenate(a, b, axis), f"concat {dtype} {name}")


def test_concat_transposed_operands(oracle, reference):
    a = make(ta.float32, 53, (2, 3, 4)).transpose(1, 2)     # [2, 4, 3], strides (12, 1, 4)
    b = make(ta.float32, 54, (2, 3, 5)).transpose(1, 2)     # [2, 5, 3]
    check(oracle, reference, lambda: ops.concatenate(a, b, 1), "concat transposed")


OUTER_PAIRS = [(ta.int8, ta.int64), (ta.int64, ta.int16), (ta.int32, ta.int64), (ta.int64, ta.int64),
               (ta.int8, ta.int32), (ta.int32, ta.int8), (ta.int16, ta.int32), (ta.int32, ta.int16),
               (ta.float32, ta.float32), (ta.float32, ta.float64), (ta.float64, ta.float32), (ta.float64, ta.float64),
               (ta.int32, ta.float32), (ta.float32, ta.int32), (ta.int32, ta.float64), (ta.float64, ta.int32)]


@pytest.mark.parametrize("pair", OUTER_PAIRS, ids=lambda p: f"{p[0]}-{p[1]}")
def test_outer(oracle, reference, pair):
    a, b = make(pair[0], 55, (7,), -3, 3), make(pair[1], 56, (5,), -3, 3)
    check(oracle, reference, lambda: ops.outer(a, b), f"outer {pair}")
