"""Pins for the parts of the CPU checker that no reference build in this image
covers (16-bit floats, comparisons' bit packing, value max/min), against numpy
arithmetic, closed forms and brute force."""
import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import ops, types

SEED = 23


def f16(tid, shape, low=-4, high=4):
    return support.values_for(ta.float16, SEED, tid, shape, low, high)


def bf16(tid, shape, low=-4, high=4):
    return support.values_for(ta.bfloat16, SEED, tid, shape, low, high)


def round_bf16(x):
    return types.bfloat16_bits_to_float32(types.float32_to_bfloat16_bits(np.asarray(x, dtype=np.float32)))


@pytest.mark.parametrize("op,fn", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply)])
def test_f16_arithmetic_is_correctly_rounded(oracle, op, fn):
    a, b = f16(1, (64, 33)), f16(2, (64, 33))
    got = getattr(ops, op)(support.host_tensor(a, ta.float16), support.host_tensor(b, ta.float16)).storage()
    want = fn(a.astype(np.float64), b.astype(np.float64)).astype(np.float16)  # exact in fp64, one rounding
    support.assert_bit_exact(got, want, op)


@pytest.mark.parametrize("op,fn", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply)])
def test_bf16_arithmetic_is_float_then_one_rounding(oracle, op, fn):
    a, b = bf16(3, (64, 33)), bf16(4, (64, 33))
    got = getattr(ops, op)(support.host_tensor(a, ta.bfloat16), support.host_tensor(b, ta.bfloat16)).storage()
    want = types.float32_to_bfloat16_bits(fn(a.astype(np.float64), b.astype(np.float64)).astype(np.float32))
    # fp64 -> fp32 -> bf16 double rounding can only differ from the checker's fp32 evaluation on fp32 ties
    assert np.mean(got != want) < 1e-3
    assert np.max(np.abs(got.astype(np.int32) - want.astype(np.int32))) <= 1


def test_f16_mixed_with_f32_promotes(oracle):
    a, b = f16(5, (8, 9)), support.uniform(SEED, 6, (8, 9))
    got = ops.mul(support.host_tensor(a, ta.float16), support.host_tensor(b, ta.float32))
    assert got.dtype is ta.float32
    support.assert_bit_exact(got.storage(), a.astype(np.float32) * b, "f16*f32")


@pytest.mark.parametrize("name,fn", [("log", np.log), ("exp", np.exp), ("sqrt", np.sqrt), ("sin", np.sin), ("cos", np.cos),
                                      ("tanh", np.tanh), ("abs", np.abs)])
def test_f16_functions_compute_in_float_and_round_once(oracle, name, fn):
    x = f16(7, (50, 40), 0.125, 4)
    got = getattr(ops, name)(support.host_tensor(x, ta.float16)).storage()
    want = fn(x.astype(np.float64)).astype(np.float16)
    assert support.ulp_distance_f16(got, want).max() <= 1  # libm's float result vs the exact value: at most one f16 ulp
    if name in ("sqrt", "abs"):
        support.assert_bit_exact(got, want, name)


def test_rsqrt_is_evaluated_in_double(oracle):
    x = support.uniform(SEED, 8, (1000,), 0.5, 4)
    got = ops.rsqrt(support.host_tensor(x, ta.float32), 1e-5).storage()
    want = (1.0 / np.sqrt(x.astype(np.float64) + np.float64(np.float32(1e-5)))).astype(np.float32)
    support.assert_bit_exact(got, want, "rsqrt")


def test_wide_f16_gemm_is_fp32_gemm_rounded_once(oracle):
    a, b = f16(9, (17, 64), -1, 1), f16(10, (13, 64), -1, 1)
    A, B = support.host_tensor(a, ta.float16), support.host_tensor(b, ta.float16)
    got = ops.matmul(A, B.transpose()).storage()
    wide = ops.matmul(support.host_tensor(a, ta.float32), support.host_tensor(b, ta.float32).transpose()).storage()
    support.assert_bit_exact(got, wide.astype(np.float16), "f16 gemm, wide")
    # and the mixed entry of the reference's table gives the un-rounded fp32 value
    mixed = ops.matmul(A, support.host_tensor(b, ta.float32).transpose())
    assert mixed.dtype is ta.float32
    support.assert_bit_exact(mixed.storage(), wide, "f16 x f32 gemm")


def test_wide_bf16_gemm_and_reductions(oracle):
    a, b = bf16(11, (9, 128), -1, 1), bf16(12, (128, 5), -1, 1)
    got = ops.matmul(support.host_tensor(a, ta.bfloat16), support.host_tensor(b, ta.bfloat16)).numpy()
    wide = ops.matmul(support.host_tensor(a, ta.float32), support.host_tensor(b, ta.float32)).numpy()
    support.assert_bit_exact(got, round_bf16(wide), "bf16 gemm, wide")
    s = ops.sum(support.host_tensor(a, ta.bfloat16), -1).numpy()
    w = ops.sum(support.host_tensor(a, ta.float32), -1).numpy()
    support.assert_bit_exact(s, round_bf16(w), "bf16 sum, wide")
    m = ops.mean(support.host_tensor(a, ta.bfloat16), 0).numpy()
    wm = ops.mean(support.host_tensor(a, ta.float32), 0).numpy()
    support.assert_bit_exact(m, round_bf16(wm), "bf16 mean, wide")


def test_wide_f16_conv_is_fp32_conv_rounded_once(oracle):
    x, w, b = f16(13, (2, 3, 9, 8), -1, 1), f16(14, (4, 3, 3, 3), -1, 1), f16(15, (4,), -1, 1)
    got = ops.convolve2d(*(support.host_tensor(v, ta.float16) for v in (x, w, b)), stride=2, padding=1).storage()
    wide = ops.convolve2d(*(support.host_tensor(v, ta.float32) for v in (x, w, b)), stride=2, padding=1).storage()
    support.assert_bit_exact(got, wide.astype(np.float16), "f16 conv, wide")


def test_native_16bit_accumulation_rounds_every_step(oracle):
    """Native mode restated independently: fold with a float16 accumulator."""
    a = f16(16, (3, 200), -1, 1)
    try:
        oracle.set_accumulate(False)
        got = ops.sum(support.host_tensor(a, ta.float16), -1).storage()
    finally:
        oracle.set_accumulate(True)
    want = np.zeros(3, dtype=np.float16)
    for k in range(a.shape[1]):
        want = (want.astype(np.float32) + a[:, k].astype(np.float32)).astype(np.float16)
    support.assert_bit_exact(got, want, "native f16 sum")


@pytest.mark.parametrize("dtype", [ta.int32, ta.float32, ta.float16, ta.bfloat16, ta.int8], ids=str)
def test_comparisons_pack_bits_lsb_first(oracle, dtype):
    a = np.round(support.values_for(dtype, SEED, 17, (5, 7, 3), -2, 2).astype(np.float64))
    b = np.round(support.values_for(dtype, SEED, 18, (5, 7, 3), -2, 2).astype(np.float64))
    A, B = support.host_tensor(a, dtype), support.host_tensor(b, dtype)
    table = {"eq": a == b, "ne": a != b, "gt": a > b, "ge": a >= b, "lt": a < b, "le": a <= b}
    for name, want in table.items():
        out = getattr(ops, name)(A, B)
        raw = out.raw()[: (a.size + 7) // 8]
        support.assert_bit_exact(raw, np.packbits(want.reshape(-1), bitorder="little"), name)
    # identities: exactly one of lt/eq/gt holds without NaN; ne = not eq; ge = not lt
    lt, eq, gt = (getattr(ops, n)(A, B).storage() for n in ("lt", "eq", "gt"))
    assert (lt.astype(int) + eq + gt == 1).all()
    assert (ops.ne(A, B).storage() == ~eq).all() and (ops.ge(A, B).storage() == ~lt).all()


def test_comparison_of_rank0_accumulates_into_the_byte(oracle):
    a, b = support.host_tensor(np.array(2.0), ta.float32), support.host_tensor(np.array(1.0), ta.float32)
    assert ops.gt(a, b).storage() == True  # noqa: E712
    assert ops.lt(a, b).storage() == False  # noqa: E712


def test_integer_gemm_is_exact_and_identity_is_neutral(oracle):
    a = support.integers(SEED, 19, (6, 37), -9, 9)
    b = support.integers(SEED, 20, (37, 5), -9, 9)
    for dtype in (ta.float32, ta.int32, ta.float64, ta.float16):
        got = ops.matmul(support.host_tensor(a, dtype), support.host_tensor(b, dtype)).numpy()
        support.assert_bit_exact(got.astype(np.int64), a @ b, f"integer-valued gemm {dtype}")
    x = support.uniform(SEED, 21, (7, 7))
    got = ops.matmul(support.host_tensor(x, ta.float32), support.host_tensor(np.eye(7), ta.float32)).storage()
    support.assert_bit_exact(got, x, "A @ I")


def test_transposed_view_equals_repacked_copy(oracle):
    a, b = support.uniform(SEED, 22, (5, 9)), support.uniform(SEED, 23, (4, 9))
    A, B = support.host_tensor(a, ta.float32), support.host_tensor(b, ta.float32)
    via_view = ops.matmul(A, B.transpose()).storage()
    via_copy = ops.matmul(A, ops.repack(B.transpose())).storage()
    support.assert_bit_exact(via_view, via_copy, "view vs copy")


def test_conv1x1_is_a_gemm_and_padding_taps_add_nothing(oracle):
    x = support.integers(SEED, 24, (2, 5, 4, 3), -4, 4).astype(np.float32)
    w = support.integers(SEED, 25, (6, 5, 1, 1), -4, 4).astype(np.float32)
    got = ops.convolve2d(support.host_tensor(x, ta.float32), support.host_tensor(w, ta.float32)).numpy()
    want = np.einsum("nchw,oc->nohw", x, w[:, :, 0, 0])
    support.assert_bit_exact(got, want.astype(np.float32), "1x1 conv")
    # brute force with zero padding, integer-valued data so every order of summation agrees
    w3 = support.integers(SEED, 26, (2, 5, 3, 3), -2, 2).astype(np.float32)
    got = ops.convolve2d(support.host_tensor(x, ta.float32), support.host_tensor(w3, ta.float32), None, (2, 1), (1, 1)).numpy()
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    ho, wo = (4 + 2 - 3) // 2 + 1, (3 + 2 - 3) // 1 + 1
    want = np.zeros((2, 2, ho, wo), dtype=np.float32)
    for oh in range(ho):
        for ow in range(wo):
            patch = xp[:, :, oh * 2: oh * 2 + 3, ow: ow + 3]
            want[:, :, oh, ow] = np.einsum("nchw,ochw->no", patch, w3)
    support.assert_bit_exact(got, want, "3x3 conv brute force")


@pytest.mark.parametrize("dtype", [ta.float32, ta.int32, ta.float16], ids=str)
def test_value_max_min_against_numpy(oracle, dtype):
    x = support.values_for(dtype, SEED, 27, (4, 9, 5), -3, 3)
    X = support.host_tensor(x, dtype)
    for axis in (0, 1, 2):
        support.assert_bit_exact(ops.max(X, axis).storage(), x.max(axis=axis), f"max {axis}")
        support.assert_bit_exact(ops.min(X, axis).storage(), x.min(axis=axis), f"min {axis}")
        idx = ops.argmax(X, axis).storage()
        support.assert_bit_exact(idx, x.argmax(axis=axis), f"argmax {axis}")  # numpy also returns the first occurrence
        support.assert_bit_exact(ops.argmin(X, axis).storage(), x.argmin(axis=axis), f"argmin {axis}")


def test_value_max_min_signed_zeros_and_nan(oracle):
    """+0 is above -0 wherever they stand, NaNs are skipped, and a slice where nothing exceeds the start gives back its
    first element: checked against the definition written out by hand."""
    x = np.array([[0.0, -0.0, 0.0], [-0.0, 0.0, -0.0], [np.nan, -0.0, 0.0], [np.nan, np.nan, np.nan], [-np.inf, np.nan, -np.inf],
                  [np.nan, -2.0, 5.0], [np.inf, np.nan, np.inf]], dtype=np.float32)
    X = support.host_tensor(x, ta.float32)
    got_max, got_min = ops.max(X, 1).storage().view(np.uint32), ops.min(X, 1).storage().view(np.uint32)
    bits = lambda v: np.array(v, dtype=np.float32).view(np.uint32)
    assert (got_max[:3] == bits(0.0)).all() and (got_min[:3] == bits(-0.0)).all()
    assert got_max[3] == x[3, 0].view(np.uint32) and got_min[3] == x[3, 0].view(np.uint32)      # all NaN: the first element
    assert got_max[4] == bits(-np.inf) and got_min[4] == bits(-np.inf)
    assert got_max[5] == bits(5.0) and got_min[5] == bits(-2.0)
    assert got_max[6] == bits(np.inf) and got_min[6] == bits(np.inf)                            # nothing below +inf: the first element


def test_polar_has_the_radius_as_modulus(oracle):
    rho = support.uniform(SEED, 28, (6, 5), 0.5, 3)
    theta = support.uniform(SEED, 29, (6, 5), -3, 3)
    z = ops.polar(support.host_tensor(rho, ta.float32), support.host_tensor(theta, ta.float32)).numpy()
    support.assert_close(np.abs(z), rho, 1e-6, 0, "|polar|")
    z0 = ops.polar(support.host_tensor(rho, ta.float32), support.host_tensor(np.zeros((6, 5)), ta.float32)).numpy()
    support.assert_bit_exact(z0.real, rho, "theta = 0")
    assert (z0.imag == 0).all()


# ---- repeat, triu, tril against numpy ---------------------------------------------------------------------------
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_repeat_is_numpy_repeat(oracle, axis):
    x = support.values_for(ta.float32, 5, 41, (3, 4, 5), -2, 2)
    with support.use_functions(oracle):
        got = ops.repeat(support.host_tensor(x, ta.float32).transpose(0, 2).transpose(0, 2), 3, axis).numpy()
    np.testing.assert_array_equal(got, np.repeat(x, 3, axis=axis))


@pytest.mark.parametrize("k", [0, 1, 2, 5])
def test_triangular_is_numpy_for_non_negative_offsets(oracle, k):
    x = support.values_for(ta.float64, 5, 42, (6, 4), 1, 2)
    with support.use_functions(oracle):
        up = ops.triu(support.host_tensor(x, ta.float64), k).numpy()
        lo = ops.tril(support.host_tensor(x, ta.float64), k).numpy()
    np.testing.assert_array_equal(up, np.triu(x, k))
    np.testing.assert_array_equal(lo, np.tril(x, k))


def test_triangular_negative_offset_wraps_for_the_first_rows(oracle):
    # i + k is formed in unsigned arithmetic (src/cpu/triang.cpp:12,20): for i < -k the edge is huge,
    # so triu clears those rows and tril keeps them whole; from row -k on both agree with numpy
    x = support.values_for(ta.float32, 5, 43, (5, 5), 1, 2)
    with support.use_functions(oracle):
        up = ops.triu(support.host_tensor(x, ta.float32), -2).numpy()
        lo = ops.tril(support.host_tensor(x, ta.float32), -2).numpy()
    assert not up[:2].any()
    np.testing.assert_array_equal(up[2:], np.triu(x, -2)[2:])
    np.testing.assert_array_equal(lo[:2], x[:2])
    np.testing.assert_array_equal(lo[2:], np.tril(x, -2)[2:])


# ---- concat and outer against numpy --------------------------------------------------------------------------------
@pytest.mark.parametrize("axis", [1, 2])
def test_concat_is_numpy_concatenate_for_the_last_two_axes(oracle, axis):
    a = support.values_for(ta.float32, 5, 44, (2, 3, 4), -2, 2)
    shape_b = (2, 5, 4) if axis == 1 else (2, 3, 6)
    b = support.values_for(ta.float32, 5, 45, shape_b, -2, 2)
    with support.use_functions(oracle):
        got = ops.concatenate(support.host_tensor(a, ta.float32), support.host_tensor(b, ta.float32), axis).numpy()
    np.testing.assert_array_equal(got, np.concatenate([a, b], axis=axis))


def test_outer_is_numpy_outer_and_unsupported_pairs_say_so(oracle):
    a = support.values_for(ta.float64, 5, 46, (6,), -2, 2)
    b = support.values_for(ta.float32, 5, 47, (4,), -2, 2)
    with support.use_functions(oracle):
        got = ops.outer(support.host_tensor(a, ta.float64), support.host_tensor(b, ta.float32)).numpy()
        np.testing.assert_array_equal(got, np.outer(a, b.astype(np.float64)))
        # int8 x int8: the reference's kernel writes int32 into the int8 destination the front end made
        with pytest.raises(ops.TannicError):
            ops.outer(support.host_tensor(np.ones(3), ta.int8), support.host_tensor(np.ones(3), ta.int8))


def test_pairs_whose_table_type_is_not_the_destinations_are_refused(oracle):
    """The reference's tables write float for an integer with a 16-bit float (binary operations, matmul with int8 / int16)
    while its front end sizes the destination as the 16-bit type: it overruns the destination.  The checker refuses
    those pairs, like the device; so it does a comparison or allclose of two dtypes, whose second operand the
    reference reads as the first's type."""
    i8 = support.host_tensor(np.ones((2, 2)), ta.int8)
    i64 = support.host_tensor(np.ones((2, 2)), ta.int64)
    f16 = support.host_tensor(np.ones((2, 2)), ta.float16)
    bf16 = support.host_tensor(np.ones((2, 2)), ta.bfloat16)
    f64 = support.host_tensor(np.ones((2, 2)), ta.float64)
    for op in (ops.add, ops.sub, ops.mul):
        for a, b in ((i8, f16), (f16, i64), (bf16, i8), (i64, bf16)):
            with pytest.raises(ta.TannicError):
                op(a, b)
    with pytest.raises(ta.TannicError):
        ops.matmul(i8, f16)
    for cmp in (ops.eq, ops.gt, ops.le):
        with pytest.raises(ta.TannicError):
            cmp(i64, i8)
    with pytest.raises(ta.TannicError):
        ops.allclose(f64, f16)
    assert ops.allclose(f64, f64)
