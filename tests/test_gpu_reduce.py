"""Axis reductions on the device against the CPU checker.

Bars: bit-exact for integer sums (wrap-around included), for argmax/argmin
indices (ties, NaN, infinities) and for value max/min; floating sums/means
within R*eps*sum|x| of the sequential CPU sum (the device adds partial sums as
a tree); 16-bit sums accumulate in fp32 on both sides and differ by at most
one rounding of the 16-bit result.
"""
import numpy as np
import pytest

import golden_cases
import support
import tannic_amd as ta
from tannic_amd import ops

pytestmark = pytest.mark.gpu
SEED = 9
REDUCE_GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] in ("sum", "mean", "argmax", "argmin", "mean_sq")]

# (shape, axis): which kernel the launcher picks for a contiguous source
SHAPES = {
    "rows_short": ((300, 17), 1),
    "rows_vector": ((512, 1024), 1),
    "rows_odd": ((77, 1001), 1),
    "rows_block_wide": ((3, 40000), 1),
    # rows that start anywhere / whose length no vector divides: the aligned middle as vectors, its ends one element per lane
    "rows_odd_1025": ((70, 1025), 1),
    "rows_odd_2051": ((9, 2051), 1),
    "rows_odd_block_wide": ((3, 8195), 1),
    # a handful of very long rows: several blocks per row (vocabulary logits); odd and even lengths, one and many rows
    "rows_split_one_odd": ((1, 50257), 1),
    "rows_split_sixteen_odd": ((16, 50257), 1),
    "rows_split_even": ((5, 32768), 1),
    "rows_split_long": ((2, 300003), 1),
    "one_row": ((9000,), 0),
    "columns_wide": ((4, 300, 1024), 1),
    "columns_split": ((2, 4096, 256), 1),
    "columns_narrow": ((5, 200, 20), 1),
    "columns_tiny": ((7, 33, 3), 1),
    "first_axis": ((1000, 96), 0),
    "middle_of_4d": ((3, 50, 4, 32), 1),
    "reduced_extent_one": ((6, 1, 40), 1),
}


@pytest.mark.parametrize("case", REDUCE_GOLDEN, ids=lambda c: c["name"])
def test_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    rtol, atol = golden_cases.tolerance(case)
    support.assert_close(got, golden_cases.expected_of(case), rtol, atol, case["name"])


def sum_tolerance(x, axis, dtype):
    eps = {ta.float32: 2.0 ** -24, ta.float64: 2.0 ** -53}[dtype]
    r = x.shape[axis]
    return r * eps * np.abs(x.astype(np.float64)).sum(axis=axis).max()


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("dtype", [ta.float32, ta.float64], ids=str)
def test_float_sum_and_mean(device, dtype, name):
    shape, axis = SHAPES[name]
    x = support.values_for(dtype, SEED, 1, shape)
    h, d = support.both(x, dtype, device)
    atol = sum_tolerance(x, axis, dtype)
    for op in ("sum", "mean"):
        for keepdim in (False, True):
            want, got = getattr(ops, op)(h, axis, keepdim), getattr(ops, op)(d, axis, keepdim)
            assert got.shape == want.shape
            support.assert_close(got.numpy(), want.numpy(), 1e-6 if dtype is ta.float32 else 1e-14, atol, f"{op} {name} {dtype}")


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_16bit_sum_and_mean_accumulate_in_fp32(device, dtype, name):
    shape, axis = SHAPES[name]
    x = support.values_for(dtype, SEED, 2, shape, -1, 1)
    h, d = support.both(x, dtype, device)
    for op in ("sum", "mean"):
        want, got = getattr(ops, op)(h, axis).numpy(), getattr(ops, op)(d, axis).numpy()
        ulp = 2.0 ** -10 if dtype is ta.float16 else 2.0 ** -7
        support.assert_close(got, want, ulp, ulp * 2.0 ** -3, f"{op} {name} {dtype}")


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("dtype", [ta.int8, ta.int16, ta.int32, ta.int64], ids=str)
def test_integer_sum_is_bit_exact_with_wrap_around(device, dtype, name):
    shape, axis = SHAPES[name]
    h, d = support.both(support.values_for(dtype, SEED, 3, shape, -120, 120), dtype, device)
    support.assert_bit_exact(ops.sum(d, axis).storage(), ops.sum(h, axis).storage(), f"sum {name} {dtype}")


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("dtype", [ta.float32, ta.float16, ta.bfloat16, ta.float64, ta.int32, ta.int8, ta.int64], ids=str)
def test_argmax_argmin_max_min_bit_exact(device, dtype, name):
    shape, axis = SHAPES[name]
    # few distinct values: ties everywhere, the lowest index must win
    x = np.round(support.values_for(dtype, SEED, 4, shape, -3, 3).astype(np.float64))
    h, d = support.both(x, dtype, device)
    for op in ("argmax", "argmin", "max", "min"):
        want, got = getattr(ops, op)(h, axis), getattr(ops, op)(d, axis)
        assert got.dtype is want.dtype and got.shape == want.shape
        support.assert_bit_exact(got.storage(), want.storage(), f"{op} {name} {dtype}")


@pytest.mark.parametrize("extent", [3, 4, 15, 16, 17, 31, 32, 33, 47, 48, 49, 64, 65])
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_index_search_over_16bit_columns_at_the_group_boundaries(device, dtype, extent):
    """[3, extent, 512]: 64 lanes across the columns, four rows of lanes, no sharing of R, so a lane walks rows
    ty, ty + 4, ...: extents around 16, 32, 48 and 64 are one to four whole groups of four rows (the loop that folds a
    group while the next is loading takes them in turn from two register sets), with and without rows left over."""
    x = np.round(support.values_for(dtype, SEED, 11, (3, extent, 512), -4, 4).astype(np.float64))
    x[1, extent // 2, 7] = np.nan
    x[2, :, 9] = -np.inf
    h, d = support.both(x, dtype, device)
    for op in ("argmax", "argmin", "max", "min"):
        want, got = getattr(ops, op)(h, 1), getattr(ops, op)(d, 1)
        support.assert_bit_exact(got.storage(), want.storage(), f"{op} extent {extent} {dtype}")


def test_argmax_with_nan_and_infinities(device):
    x = support.uniform(SEED, 5, (64, 700))
    x[0, :] = np.nan
    x[1, :] = -np.inf
    x[2, 5] = np.nan
    x[3, 10] = np.inf
    x[3, 600] = np.inf
    x[4, :] = np.inf
    h, d = support.both(x, ta.float32, device)
    for op in ("argmax", "argmin"):
        for axis in (0, 1):
            support.assert_bit_exact(getattr(ops, op)(d, axis).storage(), getattr(ops, op)(h, axis).storage(), f"{op} axis={axis}")
    hi, di = support.both(np.full((5, 300), -128), ta.int8, device)
    support.assert_bit_exact(ops.argmax(di, 1).storage(), ops.argmax(hi, 1).storage(), "int8 all lowest")


@pytest.mark.parametrize("extent", [8, 64, 504, 512, 520, 1024, 1032, 1536, 2048])
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_index_of_extreme_in_many_short_rows_of_16_bit_floats(device, dtype, extent):
    """Thousands of rows of at most 2048 16-bit floats (whole 16-byte pieces) are searched by a kernel of their own:
    ties, NaNs, infinities, signed zeros and rows in which nothing beats the start value, at every piece count."""
    rows = 1027
    x = np.round(support.values_for(dtype, SEED, 40 + extent, (rows, extent), -4, 4).astype(np.float64))
    rng = np.random.default_rng(extent)
    x[0, :] = np.nan                                   # nothing but NaN: index 0
    x[1, :] = -np.inf                                  # argmax never leaves 0; argmin ties everywhere
    x[2, :] = np.inf
    x[3, :] = np.nan; x[3, extent - 1] = -7.0          # the only number is the last element
    x[4, :] = 0.0; x[4, ::3] = -0.0                    # zeros of both signs tie
    x[5, :] = 1.0; x[5, extent // 2] = np.nan          # the same value everywhere: lowest index
    x[6, :] = -2.0; x[6, extent - 1] = 9.0; x[6, extent // 2] = 9.0   # two holders in different lanes or pieces
    x[7, :] = np.nan; x[7, extent - 3:] = [-np.inf, np.inf, -np.inf][:3]
    for row in range(8, 200):                          # one or two planted extremes at random places
        where = rng.integers(0, extent, 2)
        x[row, where] = 50.0
        x[row, rng.integers(0, extent, 2)] = -50.0
        if row % 5 == 0:
            x[row, rng.integers(0, extent, max(1, extent // 7))] = np.nan
    h, d = support.both(x, dtype, device)
    for op in ("argmax", "argmin"):
        want, got = getattr(ops, op)(h, 1), getattr(ops, op)(d, 1)
        assert got.dtype is ta.int64 and got.shape == want.shape
        support.assert_bit_exact(got.storage(), want.storage(), f"{op} {dtype} [{rows},{extent}]")
    clean = ~np.isnan(x).any(axis=1)                   # and against numpy where its answer is defined the same way
    np.testing.assert_array_equal(ops.argmax(d, 1).numpy()[clean & (x.max(axis=1) > -np.inf)],
                                  x.argmax(axis=1)[clean & (x.max(axis=1) > -np.inf)])


@pytest.mark.parametrize("dtype", [ta.float32, ta.float64, ta.float16, ta.bfloat16], ids=str)
def test_value_max_min_order_signed_zeros_and_skip_nan(device, dtype):
    """max / min are the largest / smallest NUMBER of a slice with +0 above -0, whichever lane, wavefront or block
    holds which zero; NaNs only show where nothing exceeds the start value (then the slice's first element comes back)."""
    rows, n = 6, 5000
    x = np.zeros((rows, n))
    x[0, :] = 0.0; x[0, 4321] = -0.0           # one -0 among +0
    x[1, :] = -0.0; x[1, 77] = 0.0             # one +0 among -0
    x[2, ::2] = -0.0                           # alternating
    x[3, :] = np.nan; x[3, 1234] = -0.0; x[3, 4000] = 0.0
    x[4, :] = np.nan                           # nothing but NaN: the first element
    x[5, :] = -3.0; x[5, 9] = np.nan; x[5, 4999] = -0.0
    h, d = support.both(x, dtype, device)
    for axis in (1, 0):
        for op in ("max", "min"):
            want, got = getattr(ops, op)(h, axis), getattr(ops, op)(d, axis)
            support.assert_bit_exact(got.storage(), want.storage(), f"{op} axis={axis} {dtype}")
    got_max, got_min = ops.max(d, 1).numpy().astype(np.float64), ops.min(d, 1).numpy().astype(np.float64)
    assert not np.signbit(got_max[:4]).any() and np.signbit(got_min[:4]).all()      # +0 is the maximum, -0 the minimum
    assert np.isnan(got_max[4]) and np.isnan(got_min[4])
    assert got_max[5] == 0 and np.signbit(got_max[5]) and got_min[5] == -3.0


@pytest.mark.parametrize("dtype", [ta.float32, ta.int32, ta.float16], ids=str)
def test_strided_sources(device, dtype):
    h, d = support.both(np.round(support.values_for(dtype, SEED, 6, (12, 30, 20)).astype(np.float64)), dtype, device)
    for spec in ([("transpose", (0, 2))], [("index", (slice(1, 12, 2), slice(None), slice(0, 20, 3)))], [("permute", (1, 2, 0))]):
        hv, dv = support.apply_view(h, spec), support.apply_view(d, spec)
        for axis in range(3):
            for op in ("sum", "argmax", "min"):
                want, got = getattr(ops, op)(hv, axis), getattr(ops, op)(dv, axis)
                support.assert_bit_exact(got.storage(), want.storage(), f"{op} {dtype} {spec} axis={axis}")  # integer-valued: sums exact


@pytest.mark.parametrize("dtype", [ta.float32, ta.int32, ta.float16, ta.float64], ids=str)
def test_views_that_are_dense_in_another_order_and_rows_of_a_few_elements(device, dtype):
    """A transposed matrix summed along its rows is the column sum of the matrix as it lies: views whose dims are a
    dense tensor's in another order reduce as [outer, R, inner] when the dims that stay keep their order (and element by
    element otherwise: a lane per result, or a wavefront when the results are few and the reduced dim long); rows of up
    to 16 elements, of one when the reduced dim has extent 1, take a lane each."""
    cases = [((700, 300), [("transpose", (0, 1))]), ((40, 300, 64), [("transpose", (1, 2))]), ((40, 64, 300), [("transpose", (0, 1))]),
             ((12, 64, 300), [("permute", (2, 0, 1))]), ((9, 1, 300, 70), [("transpose", (2, 3))]), ((5000, 1), []), ((4000, 7), []), ((30, 40, 1), []),
             ((3000, 16), []), ((1, 900), [("transpose", (0, 1))]),
             # views that are not dense: few results over a long reduced dim take a wavefront each
             ((40, 600, 6), [("index", (slice(0, 40, 2),))]), ((50, 2000), [("index", (slice(None), slice(1, 1999)))]),
             ((6, 3, 1000), [("index", (slice(None), slice(None), slice(0, 1000, 3)))]),
             # a large view whose neighbouring results lie far apart is copied into a contiguous tensor first
             ((40, 50, 12, 20), [("transpose", (0, 1))]), ((300, 1100), [("index", (slice(None), slice(0, 1100, 2))), ("transpose", (0, 1))])]
    for shape, spec in cases:
        h, d = support.both(np.round(support.values_for(dtype, SEED, 9, shape, -3, 3).astype(np.float64)), dtype, device)
        hv, dv = support.apply_view(h, spec), support.apply_view(d, spec)
        for axis in range(len(shape)):
            for op in ("sum", "argmax", "max"):
                want, got = getattr(ops, op)(hv, axis), getattr(ops, op)(dv, axis)
                assert got.shape == want.shape
                support.assert_bit_exact(got.storage(), want.storage(), f"{op} {dtype} {shape} {spec} axis={axis}")  # integer-valued: sums exact


def test_rms_norm_statistics(device):
    """mean(X*X, -1, keepdim) then rsqrt: the reduction pattern of an RMSNorm row (R = 4096)."""
    h, d = support.both(support.values_for(ta.bfloat16, SEED, 7, (1, 64, 4096)), ta.bfloat16, device)

    def stat(x):
        return ops.rsqrt(ops.mean(ops.mul(x, x), -1, True), 1e-5)
    support.assert_close(stat(d).numpy(), stat(h).numpy(), 2.0 ** -7, 0, "rms statistics")


def test_softmax_statistics(device):
    """max and sum over the last axis (R = 512), as a softmax row needs them."""
    h, d = support.both(support.values_for(ta.float32, SEED, 8, (4, 64, 512)), ta.float32, device)

    def softmax_den(x):
        m = ops.max(x, -1, True)
        return ops.sum(ops.exp(ops.sub(x, m)), -1, True)
    support.assert_close(softmax_den(d).numpy(), softmax_den(h).numpy(), 1e-5, 0, "softmax denominator")
