"""Elementwise device kernels against the CPU checker on identical seeded inputs.

Bars: bit-exact for integers, comparisons and every correctly-rounded float
operation (add, sub, mul, neg, abs, sqrt, scale, copies); rel 1e-5 for fp32
transcendental functions (device libm vs glibc); one ulp of the 16-bit type for
fp16/bf16 functions.
"""
import numpy as np
import pytest

import golden_cases
import support
import tannic_amd as ta
from tannic_amd import ops

pytestmark = pytest.mark.gpu
SEED = 5
INTS = [ta.int8, ta.int16, ta.int32, ta.int64]
FLOATS = [ta.float16, ta.bfloat16, ta.float32, ta.float64]
ELEMENTWISE_GOLDEN = [c for c in golden_cases.TENSOR_CASES if c["op"] not in ("matmul", "conv2d", "sum", "mean", "argmax", "argmin", "mean_sq")]


def pair_of(dtype, tid, shape, device, low=-4, high=4):
    return support.both(support.values_for(dtype, SEED, tid, shape, low, high), dtype, device)


@pytest.mark.parametrize("case", ELEMENTWISE_GOLDEN, ids=lambda c: c["name"])
def test_reference_vectors_on_device(device, case):
    got = golden_cases.run(case, device)
    rtol, atol = golden_cases.tolerance(case)
    support.assert_close(got, golden_cases.expected_of(case), rtol, max(atol, 1e-30), case["name"])


LAYOUTS = {
    "flat_vector": ((64, 4096), (64, 4096), [], []),
    "flat_odd": ((1031, 517), (1031, 517), [], []),
    "broadcast_row_scalar": ((16, 384, 128), (1, 384, 1), [], []),
    "broadcast_last": ((6, 50, 256), (256,), [], []),
    "broadcast_mid": ((2, 1, 3), (1, 4, 3), [], []),
    "one_element": ((300, 129), (1,), [], []),
    "transposed": ((70, 40), (40, 70), [("transpose", (0, 1))], []),
    "expanded": ((1, 96), (50, 96), [("expand", (50, 96))], []),
    "sliced_misaligned": ((64, 130), (64, 128), [("index", (slice(None), slice(1, 129)))], []),
    "singleton": ((1, 1), (1,), [], []),
    # rows whose length no vector divides next to an operand that is constant along the row (softmax's x - max): vectors
    # over the flat index that run over row ends; the constant operand with its own outer strides; rows shorter than a
    # vector; an odd number of elements in all; the constant operand first
    "odd_rows_column": ((37, 197), (37, 1), [], []),
    "odd_rows_column_outer_broadcast": ((3, 5, 21, 19), (3, 1, 21, 1), [], []),
    "short_odd_rows_column": ((50, 5), (50, 1), [], []),
    "odd_count_column": ((9, 31), (9, 1), [], []),
    "column_first_odd_rows": ((23, 1), (23, 45), [], []),
    "rank8": ((2, 1, 2, 3, 1, 2, 2, 3), (1, 3, 2, 1, 2, 2, 1, 3), [], []),
}
PAIRS = ([(d, d) for d in INTS + FLOATS + [ta.complex64, ta.complex128]] +
         [(ta.int8, ta.int32), (ta.int64, ta.int16), (ta.int32, ta.float32), (ta.float64, ta.int32), (ta.float32, ta.float64),
          (ta.float16, ta.float32), (ta.float32, ta.bfloat16), (ta.bfloat16, ta.float64)])


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("pair", PAIRS, ids=lambda p: f"{p[0]}-{p[1]}")
def test_add_sub_mul_bit_exact(device, pair, layout):
    sa, sb, va, vb = LAYOUTS[layout]
    ha, da = pair_of(pair[0], 1, sa, device)
    hb, db = pair_of(pair[1], 2, sb, device)
    for op in ("add", "sub", "mul"):
        want = getattr(ops, op)(support.apply_view(ha, va), support.apply_view(hb, vb))
        got = getattr(ops, op)(support.apply_view(da, va), support.apply_view(db, vb))
        assert got.dtype is want.dtype and got.shape == want.shape
        support.assert_bit_exact(got.storage(), want.storage(), f"{op} {pair} {layout}")


@pytest.mark.parametrize("pair", [(ta.float32, ta.float32), (ta.float64, ta.float64), (ta.int32, ta.float32), (ta.float32, ta.float64),
                                  (ta.float16, ta.float32)], ids=lambda p: f"{p[0]}-{p[1]}")
def test_pow(device, pair):
    ha, da = pair_of(pair[0], 3, (33, 1, 65), device, 0, 4)
    hb, db = pair_of(pair[1], 4, (1, 17, 65), device, -3, 3)
    want, got = ops.pow(ha, hb), ops.pow(da, db)
    rtol = 1e-5 if want.dtype is ta.float32 else 1e-12
    support.assert_close(got.numpy(), want.numpy(), rtol, 1e-30, f"pow {pair}")


def test_unsupported_binary_pairs(device):
    _, a = pair_of(ta.float16, 5, (4,), device)
    _, b = pair_of(ta.int8, 6, (4,), device)
    with pytest.raises(ta.TannicError):
        ops.add(a, b)     # 16-bit float with integer: destination sized for 2 bytes, kernel would write 4
    with pytest.raises(ta.TannicError):
        ops.pow(a, a)     # same for pow of two 16-bit operands


EXACT_UNARY = ["neg", "abs", "sqrt", "repack"]
LIBM_UNARY = ["log", "exp", "sin", "cos", "tan", "sinh", "cosh", "tanh"]
VIEWS = {
    "contiguous": ((257, 1030), []),
    "transposed": ((130, 70), [("transpose", (0, 1))]),
    "sliced": ((40, 66), [("index", (slice(1, 40, 3), slice(2, 66, 2)))]),
    "singleton": ((1, 1, 1), []),
    "permuted_4d": ((3, 8, 5, 16), [("permute", (0, 2, 1, 3))]),
}


def tolerance_of(dtype):
    return {ta.float32: (1e-5, 1e-30), ta.float64: (1e-12, 1e-300)}[dtype]


@pytest.mark.parametrize("view", list(VIEWS))
@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_unary_functions(device, dtype, view):
    shape, spec = VIEWS[view]
    h, d = pair_of(dtype, 7, shape, device, 0.125, 4)
    hv, dv = support.apply_view(h, spec), support.apply_view(d, spec)
    for op in EXACT_UNARY:
        support.assert_bit_exact(getattr(ops, op)(dv).storage(), getattr(ops, op)(hv).storage(), f"{op} {dtype} {view}")
    for op in LIBM_UNARY + ["rsqrt"]:
        fn = (lambda t: ops.rsqrt(t, 1e-5)) if op == "rsqrt" else getattr(ops, op)
        want, got = fn(hv), fn(dv)
        if dtype in (ta.float16, ta.bfloat16):
            w, g = want.storage().view(np.int16).astype(np.int32), got.storage().view(np.int16).astype(np.int32)
            assert np.abs(w - g).max() <= 1, f"{op} {dtype} {view}: more than one ulp apart"
        else:
            support.assert_close(got.numpy(), want.numpy(), *tolerance_of(dtype), f"{op} {dtype} {view}")


def test_rsqrt_of_bfloat16_subnormals_without_epsilon(device):
    """A bfloat16 subnormal is a float subnormal, which the hardware's reciprocal square root reads as zero: the device
    scales such inputs first.  The CPU path evaluates in double (src/cpu/ops-unary.cpp:141-149); one ulp apart at most."""
    bits = np.array([0x0001, 0x0002, 0x0040, 0x007F, 0x0080, 0x0081, 0x0100, 0x3F80], dtype=np.uint16)
    h = ta.Tensor(ta.bfloat16, bits.shape).initialize(ta.Host())
    h.write_raw(bits)
    d = h.to(device)
    want, got = ops.rsqrt(h, 0.0).storage().astype(np.int32), ops.rsqrt(d, 0.0).storage().astype(np.int32)
    assert np.isfinite(ta.types.bfloat16_bits_to_float32(got.astype(np.uint16))).all()
    assert np.abs(want - got).max() <= 1, (want, got)


def test_rsqrt_fp32_is_bit_exact(device):
    """The double-precision evaluation makes the fp32 result correctly rounded on both sides."""
    h, d = pair_of(ta.float32, 8, (100, 333), device, 0.01, 100)
    support.assert_bit_exact(ops.rsqrt(d, 1e-6).storage(), ops.rsqrt(h, 1e-6).storage(), "rsqrt")


@pytest.mark.parametrize("dtype", INTS + [ta.complex64, ta.complex128], ids=str)
def test_neg_repack_abs_other_types(device, dtype):
    h, d = pair_of(dtype, 9, (31, 5, 12), device, -100, 100)
    for spec in ([], [("transpose", (0, 2))]):
        hv, dv = support.apply_view(h, spec), support.apply_view(d, spec)
        names = ["neg", "repack"] + (["abs"] if dtype in (ta.int32, ta.int64) else [])
        for op in names:
            support.assert_bit_exact(getattr(ops, op)(dv).storage(), getattr(ops, op)(hv).storage(), f"{op} {dtype}")


TRANSPOSING_COPIES = {
    "matrix": ((130, 70), [("transpose", (0, 1))]),
    "matrix_ragged_tiles": ((65, 193), [("transpose", (0, 1))]),
    "batched_matrices": ((5, 40, 72), [("transpose", (1, 2))]),
    "heads_to_front_of_columns": ((2, 33, 4, 20), [("permute", (0, 3, 1, 2))]),
    "nchw_as_nhwc": ((3, 17, 9, 21), [("permute", (0, 2, 3, 1))]),
    "first_axis_last": ((40, 3, 50), [("permute", (1, 2, 0))]),
    "column_slice_of_a_transposed_matrix": ((90, 64), [("transpose", (0, 1)), ("index", (slice(3, 60), slice(5, 88)))]),
}


@pytest.mark.parametrize("name", list(TRANSPOSING_COPIES))
@pytest.mark.parametrize("dtype", [ta.int8, ta.float16, ta.float32, ta.float64, ta.complex128], ids=str)
def test_repack_of_views_that_are_contiguous_along_another_dimension(device, dtype, name):
    """Copies whose source runs contiguously along another dimension than the result's last one move 64 x 64 tiles
    through LDS: tiles that end inside the matrix, batches before and between the two dimensions, views that start
    inside the storage, every element size."""
    shape, spec = TRANSPOSING_COPIES[name]
    h, d = pair_of(dtype, 12, shape, device, -100, 100)
    hv, dv = support.apply_view(h, spec), support.apply_view(d, spec)
    want, got = ops.repack(hv), ops.repack(dv)
    assert got.shape == want.shape
    support.assert_bit_exact(got.storage(), want.storage(), f"repack {name} {dtype}")


@pytest.mark.parametrize("view", ["contiguous", "transposed", "singleton"])
@pytest.mark.parametrize("dtype", INTS + FLOATS, ids=str)
def test_scale(device, dtype, view):
    h, d = pair_of(dtype, 10, (1,) if view == "singleton" else (129, 260), device, -100, 100)
    if view == "transposed":
        h, d = h.transpose(), d.transpose()
    for k in (3, -7, 0.333):
        support.assert_bit_exact(ops.scale(d, k).storage(), ops.scale(h, k).storage(), f"scale {dtype} {view} {k}")


@pytest.mark.parametrize("dtype", INTS + FLOATS, ids=str)
def test_comparisons(device, dtype):
    for shape in [(3, 7, 5), (64, 1024), (1001,), (8,), (1,)]:
        a = np.round(support.values_for(dtype, SEED, 11, shape, -3, 3).astype(np.float64))
        b = np.round(support.values_for(dtype, SEED, 12, shape, -3, 3).astype(np.float64))
        if dtype.is_floating:
            a.reshape(-1)[0] = np.nan
            b.reshape(-1)[-1] = np.nan
        ha, da = support.both(a, dtype, device)
        hb, db = support.both(b, dtype, device)
        for op in ("eq", "ne", "gt", "ge", "lt", "le"):
            want, got = getattr(ops, op)(ha, hb), getattr(ops, op)(da, db)
            n = (want.nelements + 7) // 8
            support.assert_bit_exact(got.raw()[:n], want.raw()[:n], f"{op} {dtype} {shape}")
    # strided operands are walked with their own strides
    ha, da = pair_of(dtype, 13, (20, 30), device, -2, 2)
    hb, db = pair_of(dtype, 14, (30, 20), device, -2, 2)
    want, got = ops.le(ha.transpose(), hb), ops.le(da.transpose(), db)
    support.assert_bit_exact(got.raw()[:75], want.raw()[:75], f"le strided {dtype}")


def test_comparison_rank0(device):
    ha, da = support.both(np.array(2.0), ta.float32, device)
    hb, db = support.both(np.array(1.0), ta.float32, device)
    assert ops.gt(da, db).storage() == ops.gt(ha, hb).storage() == True  # noqa: E712
    assert ops.lt(da, db).storage() == ops.lt(ha, hb).storage() == False  # noqa: E712


@pytest.mark.parametrize("pair", [(ta.float32, ta.float32), (ta.float64, ta.float64), (ta.float32, ta.float64), (ta.int32, ta.float32),
                                  (ta.int8, ta.int16)], ids=lambda p: f"{p[0]}-{p[1]}")
def test_complex_construction(device, pair):
    ha, da = pair_of(pair[0], 15, (40, 1, 33), device, 0, 3)
    hb, db = pair_of(pair[1], 16, (40, 5, 33), device, -3, 3)
    comp = ta.float64 if ta.float64 in pair else ta.float32
    ctype = ta.complex64 if comp is ta.float32 else ta.complex128
    for op in ("view_as_cartesian", "view_as_polar"):
        want = ops._call(op, ta.Host(), [ha, hb], ta.Tensor(ctype, (40, 5, 33)).initialize(ta.Host()))
        got = ops._call(op, device, [da, db], ta.Tensor(ctype, (40, 5, 33)).initialize(device))
        if op == "view_as_cartesian":
            support.assert_bit_exact(got.storage(), want.storage(), f"{op} {pair}")
        else:
            rtol = 1e-5 if comp is ta.float32 else 1e-12
            support.assert_close(got.numpy(), want.numpy(), rtol, 1e-6 if comp is ta.float32 else 1e-14, f"{op} {pair}")


def test_rotary_embedding_through_complex_multiply(device):
    """The llama-style path of tests/cpu/test-complex.cpp:64-91: view pairs as complex, multiply, view back."""
    hq, dq = pair_of(ta.float32, 17, (1, 4, 16, 32), device)
    hr, dr = pair_of(ta.float32, 18, (16, 16), device, 1, 1.0000001)
    ht, dt = pair_of(ta.float32, 19, (16, 16), device, -3, 3)

    def rope(q, rho, theta):
        freqs = ops.polar(rho, theta)
        z = ops.complexify(q.view(1, 4, 16, 16, 2))
        return ops.realify(ops.mul(z, freqs)).view(1, 4, 16, 32)
    support.assert_close(rope(dq, dr, dt).numpy(), rope(hq, hr, ht).numpy(), 1e-5, 1e-6, "rope")


@pytest.mark.parametrize("dtype", INTS + FLOATS + [ta.complex64, ta.complex128], ids=str)
def test_cpy_into_strided_destination(device, dtype):
    hs, ds = pair_of(dtype, 20, (33, 1, 40), device)
    hd, dd = pair_of(dtype, 21, (80, 2, 66), device)
    ops.copy_into(hd[::2, 0:1, ::2], hs.transpose(0, 2))
    ops.copy_into(dd[::2, 0:1, ::2], ds.transpose(0, 2))
    support.assert_bit_exact(dd.storage(), hd.storage(), f"cpy {dtype}")


@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_allclose(device, dtype):
    h, d = pair_of(dtype, 22, (55, 66), device)
    near = h.numpy().astype(np.float64) * (1 + 1e-9)
    far = h.numpy().astype(np.float64) + 0.5
    for other, rtol, atol in ((near, 1e-5, 1e-8), (far, 1e-5, 1e-8), (far, 1e-5, 1.0)):
        ho, do = support.both(other, dtype, device)
        assert ops.allclose(d, do, rtol, atol) == ops.allclose(h, ho, rtol, atol)
    assert ops.allclose(d.transpose(), support.both(h.numpy().T.copy(), dtype, device)[1])
    hn, dn = support.both(np.full((55, 66), np.nan), dtype, device)
    assert ops.allclose(d, dn) == ops.allclose(h, hn)


@pytest.mark.parametrize("dtype", [ta.float32, ta.float16], ids=str)
def test_broadcast_chain_reduced_size(device, dtype):
    """Y = log(|X| + 1) + Z*Z - exp(X) + 3*X, evaluated operator by operator as the front end does."""
    hx, dx = pair_of(dtype, 23, (8, 512, 128), device)
    hz, dz = pair_of(dtype, 24, (1, 512, 1), device)
    h1, d1 = support.both(np.ones(1), dtype, device)

    def chain(x, z, one):
        return ops.add(ops.sub(ops.add(ops.log(ops.add(ops.abs(x), one)), ops.mul(z, z)), ops.exp(x)), ops.scale(x, 3))
    want, got = chain(hx, hz, h1).numpy(), chain(dx, dz, d1).numpy()
    if dtype is ta.float32:
        # cancellation between the terms amplifies libm's last-bit differences: bound them by the largest term
        support.assert_close(got, want, 1e-5, 1e-5 * 64, "chain fp32")
    else:
        support.assert_close(got, want, 2e-3, 0.07, "chain fp16")  # one fp16 ulp at |y| ~ 64 is 0.03


def test_int32_add_and_compare_reduced_size(device):
    hx, dx = pair_of(ta.int32, 25, (8, 512, 128), device)
    hz, dz = pair_of(ta.int32, 26, (1, 512, 1), device)
    want, got = ops.add(hx, hz), ops.add(dx, dz)
    support.assert_bit_exact(got.storage(), want.storage(), "int32 broadcast add")
    # comparisons do not broadcast: the sum is compared with X itself
    n = want.nelements // 8
    support.assert_bit_exact(ops.gt(got, dx).raw()[:n], ops.gt(want, hx).raw()[:n], "int32 compare")
