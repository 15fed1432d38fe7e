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
