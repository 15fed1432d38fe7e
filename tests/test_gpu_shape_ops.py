"""repeat, triu and tril on the device against the CPU checker: bit-exact (elements are only moved)."""
import numpy as np
import pytest

import golden_cases
import support
import tannic_amd as ta
from tannic_amd import ops

pytestmark = pytest.mark.gpu
SEED = 21
GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] == "repeat"]
DTYPES = [ta.int8, ta.int16, ta.int32, ta.int64, ta.float16, ta.bfloat16, ta.float32, ta.float64]

# (shape, view): plain, strided, and shapes whose last dimension is moved 16 bytes at a time
VIEWS = {
    "plain": ((2, 3, 4), []),
    "permuted": ((2, 3, 4), [("permute", (2, 0, 1))]),
    "sliced": ((4, 6, 5), [("index", (slice(0, 4, 2), slice(1, 6, 2), slice(0, 5, 1)))]),
    "expanded": ((1, 3, 1), [("expand", (2, 3, 4))]),
    "vector": ((37,), []),
    "wide_rows": ((3, 5, 64), []),
    "heads": ((1, 8, 40, 128), []),
    "heads_transposed": ((1, 40, 8, 128), [("transpose", (1, 2))]),
}


@pytest.mark.parametrize("case", GOLDEN, ids=lambda c: c["name"])
def test_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    np.testing.assert_array_equal(got, golden_cases.expected_of(case))


@pytest.mark.parametrize("axis", [0, 1, 2, -1])
@pytest.mark.parametrize("view", list(VIEWS))
@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_repeat_bit_exact(device, dtype, view, axis):
    shape, spec = VIEWS[view]
    hx, dx = support.both(support.values_for(dtype, SEED, 1, shape, -4, 4), dtype, device)
    hx, dx = support.apply_view(hx, spec), support.apply_view(dx, spec)
    if axis >= hx.rank:
        pytest.skip("axis beyond the rank")
    want, got = ops.repeat(hx, 4, axis), ops.repeat(dx, 4, axis)
    assert got.shape == want.shape
    support.assert_bit_exact(got.storage(), want.storage(), f"repeat {dtype} {view} axis {axis}")


@pytest.mark.parametrize("k", [0, 1, 3, -1, -2, 9, -9])
@pytest.mark.parametrize("view", ["plain", "transposed", "sliced"])
@pytest.mark.parametrize("op", ["triu", "tril"])
@pytest.mark.parametrize("dtype", [ta.int32, ta.int64, ta.float16, ta.bfloat16, ta.float32, ta.float64], ids=str)
def test_triangular_bit_exact(device, dtype, op, view, k):
    hx, dx = support.both(support.values_for(dtype, SEED, 2, (7, 6), -4, 4), dtype, device)
    if view == "transposed":
        hx, dx = hx.transpose(0, 1), dx.transpose(0, 1)
    elif view == "sliced":
        hx, dx = hx[1:7, 0:6:2], dx[1:7, 0:6:2]
    want, got = getattr(ops, op)(hx, k), getattr(ops, op)(dx, k)
    support.assert_bit_exact(got.storage(), want.storage(), f"{op} {dtype} {view} k={k}")


@pytest.mark.parametrize("k", [0, 1, 5, -1, -7, 40, -40])
@pytest.mark.parametrize("op", ["triu", "tril"])
@pytest.mark.parametrize("dtype", [ta.int64, ta.float16, ta.float32], ids=str)
def test_triangular_of_rows_in_16_byte_pieces(device, dtype, op, k):
    """Rows of 32 columns (whole 16-byte pieces, some wholly kept, some wholly zeroed, some cut by the diagonal), from a
    plain matrix and from rows 3.. of a taller one."""
    hx, dx = support.both(support.values_for(dtype, SEED, 3, (37, 32), -4, 4), dtype, device)
    for first in (0, 3):
        want, got = getattr(ops, op)(hx[first:], k), getattr(ops, op)(dx[first:], k)
        support.assert_bit_exact(got.storage(), want.storage(), f"{op} {dtype} rows from {first} k={k}")


def test_causal_mask_shape(device):
    n = 512
    hx, dx = support.both(np.ones((n, n), dtype=np.float32), ta.float32, device)
    got = ops.tril(dx, 0).numpy()
    np.testing.assert_array_equal(got, np.tril(np.ones((n, n), dtype=np.float32)))


def test_status_codes(device):
    x = ta.Tensor(ta.float32, (2, 3, 4)).initialize(device)
    with pytest.raises(ops.TannicError):
        ops.triu(x, 0)                      # rank 2 only
    b = ta.Tensor(ta.boolean, (8,)).initialize(device)
    with pytest.raises(ops.TannicError):
        ops.repeat(b, 2, 0)                 # no boolean repeat


# ---- concat and outer ---------------------------------------------------------------------------------------------------
MORE_GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] in ("concat", "outer")]


@pytest.mark.parametrize("case", MORE_GOLDEN, ids=lambda c: c["name"])
def test_concat_outer_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    np.testing.assert_array_equal(got, golden_cases.expected_of(case))


CONCAT = {
    "rows": ((2, 3), (4, 3), 0, [], []),
    "columns": ((3, 2), (3, 5), 1, [], []),
    "last_axis_rank3": ((2, 3, 4), (2, 3, 2), 2, [], []),
    "middle_axis_rank3": ((2, 3, 4), (2, 5, 4), 1, [], []),
    "expanded_operand": ((1, 1, 3), (2, 4, 3), 1, [("expand", (2, 1, 3))], []),
    "transposed_operands": ((2, 3, 4), (2, 3, 5), 1, [("transpose", (1, 2))], [("transpose", (1, 2))]),
    "sequence_with_token": ((4, 1, 64), (4, 50, 64), 1, [], []),
}


@pytest.mark.parametrize("name", list(CONCAT))
@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_concat_bit_exact(device, dtype, name):
    sa, sb, axis, va, vb = CONCAT[name]
    ha, da = support.both(support.values_for(dtype, SEED, 3, sa, -4, 4), dtype, device)
    hb, db = support.both(support.values_for(dtype, SEED, 4, sb, -4, 4), dtype, device)
    ha, da, hb, db = support.apply_view(ha, va), support.apply_view(da, va), support.apply_view(hb, vb), support.apply_view(db, vb)
    want, got = ops.concatenate(ha, hb, axis), ops.concatenate(da, db, axis)
    assert got.shape == want.shape
    support.assert_bit_exact(got.storage(), want.storage(), f"concat {dtype} {name}")


@pytest.mark.parametrize("axis", [0, 1])
def test_concat_leading_axes_follow_numpy(device, axis):
    """More than one dimension behind the axis: every dimension is indexed by its own stride (the CPU path is not)."""
    a = support.values_for(ta.float32, SEED, 5, (2, 3, 4, 5), -4, 4)
    b = support.values_for(ta.float32, SEED, 6, (3, 3, 4, 5) if axis == 0 else (2, 2, 4, 5), -4, 4)
    got = ops.concatenate(ta.tensor(a, ta.float32, device), ta.tensor(b, ta.float32, device), axis).numpy()
    np.testing.assert_array_equal(got, np.concatenate([a, b], axis=axis))


OUTER = [(ta.int8, ta.int64), (ta.int64, ta.int32), (ta.int64, ta.int64), (ta.int8, ta.int32), (ta.int32, ta.int8), (ta.int16, ta.int32), (ta.int32, ta.int16), (ta.float32, ta.float32), (ta.float32, ta.float64),
         (ta.float64, ta.float64), (ta.int32, ta.float32), (ta.float64, ta.int32), (ta.float16, ta.float32), (ta.float32, ta.bfloat16)]


@pytest.mark.parametrize("pair", OUTER, ids=lambda p: f"{p[0]}-{p[1]}")
def test_outer_bit_exact(device, pair):
    ha, da = support.both(support.values_for(pair[0], SEED, 7, (300,), -3, 3), pair[0], device)
    hb, db = support.both(support.values_for(pair[1], SEED, 8, (77,), -3, 3), pair[1], device)
    want, got = ops.outer(ha, hb), ops.outer(da, db)
    assert got.shape == want.shape == (300, 77) and got.dtype is want.dtype
    support.assert_bit_exact(got.storage(), want.storage(), f"outer {pair}")


def test_outer_pairs_that_overrun_their_destination_are_refused(device):
    a = ta.tensor(np.ones(4), ta.float16, device)
    with pytest.raises(ops.TannicError):
        ops.outer(a, a)     # the table says fp32, the destination is fp16


def test_outer_of_strided_vectors(device, oracle):
    """Every other element of a vector is a vector: both operands are read through their strides (the reference reads
    them as contiguous, src/cpu/outer.cpp:18-40)."""
    a, b = np.arange(40, dtype=np.float64) - 20, np.arange(30, dtype=np.float64) - 7
    for dtype in (ta.float32, ta.float64, ta.int64):
        want = np.outer(a[::2], b[1::3])
        (ha, da), (hb, db) = support.both(a, dtype, device), support.both(b, dtype, device)
        np.testing.assert_array_equal(ops.outer(da[::2], db[1::3]).numpy().astype(np.float64), want)
        np.testing.assert_array_equal(ops.outer(ha[::2], hb[1::3]).numpy().astype(np.float64), want)
