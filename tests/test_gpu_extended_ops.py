"""The operators without a twin in the reference (div, cast, swiglu, rms_norm, softmax, rope) on the device.

There is no reference implementation to compare with, so each is checked against its defining formula in
float64 numpy, to one rounding of the result type, and against the chain of reference-defined operators a
Tannic program would write for it: in the 16-bit types the chain rounds at every node, so it may only be
further from the float64 value than the one-pass result, never closer.
"""
import math

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import ops, types

pytestmark = pytest.mark.gpu
SEED = 33
FLOATS = [ta.float16, ta.bfloat16, ta.float32, ta.float64]
REALS = [ta.int8, ta.int16, ta.int32, ta.int64] + FLOATS
# relative size of one rounding of the type (half an ulp at the top of a binade), with head-room for the float arithmetic
ROUNDING = {ta.float16: 2.0 ** -11, ta.bfloat16: 2.0 ** -8, ta.float32: 2.0 ** -23, ta.float64: 2.0 ** -52}
TINY = {ta.float16: 2.0 ** -24, ta.bfloat16: 1e-30, ta.float32: 1e-37, ta.float64: 0.0}


def values(dtype, tensor_id, shape, low=-4.0, high=4.0):
    return support.values_for(dtype, SEED, tensor_id, shape, low, high)


def f64(t):
    return np.asarray(t.numpy(), dtype=np.float64)


# float arithmetic behind a result: rounding errors of the float (double) steps, in units of the result type's rounding
ARITHMETIC = {ta.float16: 1.1, ta.bfloat16: 1.1, ta.float32: 8.0, ta.float64: 64.0}


def check(got, want, dtype, what, slack=1.0, atol=0.0):
    support.assert_close(got, want, slack * 1.01 * ROUNDING[dtype], atol + TINY[dtype] + 1e-300, what)


# ---- div -----------------------------------------------------------------------------
@pytest.mark.parametrize("shapes", [((5, 7), (5, 7)), ((3, 4, 64), (1, 4, 1)), ((64,), (2, 3, 64)), ((), ())], ids=str)
@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_div_same_type(device, dtype, shapes):
    a = values(dtype, 1, shapes[0])
    b = values(dtype, 2, shapes[1], 0.5, 4.0)
    got = ops.div(ta.tensor(a, dtype, device), ta.tensor(b, dtype, device))
    want = a.astype(np.float64) / b.astype(np.float64)
    assert got.dtype is dtype and got.shape == want.shape
    check(f64(got), want, dtype, f"div {dtype} {shapes}")


@pytest.mark.parametrize("pair", [(ta.float16, ta.float32), (ta.float32, ta.bfloat16), (ta.float32, ta.float64), (ta.float64, ta.float16)], ids=str)
def test_div_mixed_types(device, pair):
    a, b = values(pair[0], 3, (6, 40)), values(pair[1], 4, (6, 40), 0.5, 4.0)
    got = ops.div(ta.tensor(a, pair[0], device), ta.tensor(b, pair[1], device))
    wide = ta.float64 if ta.float64 in pair else ta.float32
    assert got.dtype is wide
    check(f64(got), a.astype(np.float64) / b.astype(np.float64), wide, f"div {pair}")


def test_div_exact_cases(device):
    """Quotients that are representable come out exactly; division by zero follows IEEE."""
    a = np.array([1.0, -6.0, 0.0, 1.0, -1.0, 0.0], dtype=np.float32)
    b = np.array([4.0, 3.0, 5.0, 0.0, 0.0, 0.0], dtype=np.float32)
    got = ops.div(ta.tensor(a, ta.float32, device), ta.tensor(b, ta.float32, device)).numpy()
    np.testing.assert_array_equal(got[:5], np.array([0.25, -2.0, 0.0, np.inf, -np.inf], dtype=np.float32))
    assert np.isnan(got[5])


def test_div_rejects_integers(device):
    a = ta.tensor(np.arange(4), ta.int32, device)
    with pytest.raises(ops.TannicError):
        ops.div(a, a)


# ---- cast ----------------------------------------------------------------------------
def expected_cast(x, src, dst):
    """numpy's conversion is the definition wherever it is defined: in-range values, any pair of real types."""
    wide = x.astype(np.float64) if src.is_floating else x.astype(np.int64)
    if dst is ta.bfloat16:
        if src is ta.float64:
            return round_f64_to_bf16(wide)
        return types.bfloat16_bits_to_float32(types.float32_to_bfloat16_bits(wide.astype(np.float32))).astype(np.float64)
    if dst.is_integral and src.is_floating:
        return np.trunc(wide).astype(dst.storage)
    return wide.astype(dst.storage)


def round_f64_to_bf16(x):
    """Nearest bfloat16 (ties to even) of float64 values with one rounding: chosen between the two neighbours."""
    bits = x.astype(np.float32).view(np.uint32) & np.uint32(0xFFFF0000)
    over = np.abs(bits.view(np.float32).astype(np.float64)) > np.abs(x)     # float32 rounding crossed a grid point
    bits = np.where(over, bits - np.uint32(0x10000), bits).astype(np.uint32)
    lo = bits.view(np.float32).astype(np.float64)
    hi = (bits + np.uint32(0x10000)).astype(np.uint32).view(np.float32).astype(np.float64)
    d_lo, d_hi = np.abs(x - lo), np.abs(hi - x)
    even_lo = ((bits >> np.uint32(16)) & np.uint32(1)) == 0
    return np.where((d_lo < d_hi) | ((d_lo == d_hi) & even_lo), lo, hi)


@pytest.mark.parametrize("dst", REALS, ids=str)
@pytest.mark.parametrize("src", REALS, ids=str)
def test_cast_pairs(device, src, dst):
    x = values(src, 5, (5, 66), -100.0, 100.0) if src.is_floating else values(src, 5, (5, 66), -100, 100)
    got = ops.cast(ta.tensor(x, src, device), dst)
    assert got.dtype is dst and got.shape == (5, 66)
    want = expected_cast(x, src, dst)
    np.testing.assert_array_equal(np.asarray(got.numpy(), dtype=np.float64), np.asarray(want, dtype=np.float64), err_msg=f"cast {src}->{dst}")


def test_cast_double_to_16bit_rounds_once(device):
    """Values a hair above a tie of the 16-bit grid: rounding through float32 first would land on the tie and go to even."""
    ties16 = np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, -(2.0 + 2.0 ** -10)], dtype=np.float64)   # float16 ties
    ties_bf = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, -(2.0 + 2.0 ** -7)], dtype=np.float64)     # bfloat16 ties
    for nudge in (2.0 ** -40, -(2.0 ** -40), 0.0):
        x16, xbf = ties16 * (1.0 + nudge), ties_bf * (1.0 + nudge)
        got16 = ops.cast(ta.tensor(x16, ta.float64, device), ta.float16).numpy()
        np.testing.assert_array_equal(got16, x16.astype(np.float16), err_msg=f"f64->f16 nudge {nudge}")
        gotbf = np.asarray(ops.cast(ta.tensor(xbf, ta.float64, device), ta.bfloat16).numpy(), dtype=np.float64)
        np.testing.assert_array_equal(gotbf, round_f64_to_bf16(xbf), err_msg=f"f64->bf16 nudge {nudge}")


def test_cast_float_to_integer_edges(device):
    x = np.array([3.9, -3.9, 127.9, -128.9, 1e10, -1e10, np.nan, np.inf, -np.inf, 0.0], dtype=np.float32)
    got8 = ops.cast(ta.tensor(x, ta.float32, device), ta.int8).numpy()
    np.testing.assert_array_equal(got8, np.array([3, -3, 127, -128, 127, -128, 0, 127, -128, 0], dtype=np.int8))
    got32 = ops.cast(ta.tensor(x, ta.float32, device), ta.int32).numpy()
    np.testing.assert_array_equal(got32, np.array([3, -3, 127, -128, 2 ** 31 - 1, -2 ** 31, 0, 2 ** 31 - 1, -2 ** 31, 0], dtype=np.int32))
    got64 = ops.cast(ta.tensor(x, ta.float32, device), ta.int64).numpy()
    np.testing.assert_array_equal(got64, np.array([3, -3, 127, -128, 10 ** 10, -10 ** 10, 0, 2 ** 63 - 1, -2 ** 63, 0], dtype=np.int64))


def test_cast_strided_source(device):
    x = values(ta.float32, 6, (6, 10))
    t = ta.tensor(x, ta.float32, device).transpose(0, 1)[1:9:2]
    got = ops.cast(t, ta.float16)
    np.testing.assert_array_equal(got.numpy(), x.T[1:9:2].astype(np.float16))


# ---- swiglu ----------------------------------------------------------------------------
def silu_mul(g, u):
    g, u = g.astype(np.float64), u.astype(np.float64)
    return g / (1.0 + np.exp(-g)) * u


@pytest.mark.parametrize("shape", [(3, 5), (4, 512), (2, 3, 14336 // 8)], ids=str)
@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_swiglu(device, dtype, shape):
    g, u = values(dtype, 7, shape, -8.0, 8.0), values(dtype, 8, shape)
    got = ops.swiglu(ta.tensor(g, dtype, device), ta.tensor(u, dtype, device))
    check(f64(got), silu_mul(g, u), dtype, f"swiglu {dtype} {shape}", ARITHMETIC[dtype])


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_swiglu_not_worse_than_the_chain(device, dtype):
    """g * rsqrt(exp(-g) + 1)^2 * u, the way a program without division writes it."""
    g, u = values(dtype, 9, (8, 256), -6.0, 6.0), values(dtype, 10, (8, 256))
    dg, du = ta.tensor(g, dtype, device), ta.tensor(u, dtype, device)
    one = ta.tensor(np.ones(1), dtype, device)
    sg = ops.rsqrt(ops.add(ops.exp(ops.neg(dg)), one))
    chain = f64(ops.mul(ops.mul(ops.mul(dg, sg), sg), du))
    fused = f64(ops.swiglu(dg, du))
    want = silu_mul(g, u)
    assert np.abs(fused - want).max() <= np.abs(chain - want).max() + 1e-12


# ---- rms_norm ----------------------------------------------------------------------------
def rms_norm_definition(x, g, eps):
    x, g = x.astype(np.float64), g.astype(np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * g


# rows in registers of one wavefront, of a block, misaligned / ragged rows, rows longer than the registers hold
RMS_SHAPES = [(3, 64), (2000, 256), (5, 4096), (1, 512, 4096), (7, 33), (3, 4100), (2, 40000), (4096,)]


@pytest.mark.parametrize("shape", RMS_SHAPES, ids=str)
@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_rms_norm(device, dtype, shape):
    if dtype is ta.float64 and shape == (2, 40000):
        shape = (2, 10000)
    x, g = values(dtype, 11, shape), values(dtype, 12, shape[-1:], 0.5, 1.5)
    got = ops.rms_norm(ta.tensor(x, dtype, device), ta.tensor(g, dtype, device), 1e-5)
    check(f64(got), rms_norm_definition(x, g, np.float32(1e-5)), dtype, f"rms_norm {dtype} {shape}", ARITHMETIC[dtype])


def test_rms_norm_scale_invariance(device):
    """Without eps the result does not change when the row is scaled by a power of two."""
    x, g = values(ta.float32, 13, (9, 1024)), values(ta.float32, 14, (1024,))
    dg = ta.tensor(g, ta.float32, device)
    a = ops.rms_norm(ta.tensor(x, ta.float32, device), dg, 0.0).numpy()
    b = ops.rms_norm(ta.tensor(x * 8.0, ta.float32, device), dg, 0.0).numpy()
    np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_rms_norm_not_worse_than_the_chain(device, dtype):
    x, g = values(dtype, 15, (64, 4096)), values(dtype, 16, (4096,), 0.5, 1.5)
    dx, dg = ta.tensor(x, dtype, device), ta.tensor(g, dtype, device)
    chain = f64(ops.mul(ops.mul(dx, ops.rsqrt(ops.mean(ops.mul(dx, dx), -1, True), 1e-5)), dg))
    fused = f64(ops.rms_norm(dx, dg, 1e-5))
    want = rms_norm_definition(x, g, np.float32(1e-5))
    assert np.abs(fused - want).max() <= np.abs(chain - want).max() + 1e-12


def test_rms_norm_rejects_strided(device):
    x = ta.tensor(values(ta.float32, 17, (8, 8)), ta.float32, device).transpose(0, 1)
    g = ta.tensor(np.ones(8), ta.float32, device)
    with pytest.raises(ops.TannicError):
        ops.rms_norm(x, g)


# ---- softmax -------------------------------------------------------------------------------
def softmax_definition(x, mask, scale):
    s = x.astype(np.float64) * np.float64(np.float32(scale))
    if mask is not None:
        s = s + mask.astype(np.float64)
    with np.errstate(invalid="ignore"):
        e = np.exp(s - s.max(axis=-1, keepdims=True))
        return e / e.sum(axis=-1, keepdims=True)


def causal(n, dtype):
    return np.where(np.tril(np.ones((n, n), dtype=bool)), 0.0, -np.inf).astype(np.float32)


# the last five: rows no 16-byte access fits, a wavefront per row (4, 8, 16 and 32 elements per lane), and too few of them for that
SOFTMAX_SHAPES = [(4, 64), (3, 40, 512), (2, 4, 128, 128), (1300, 200), (5, 4096), (3, 37), (2, 1028), (2, 70000),
                  (300, 197), (2, 130, 511), (260, 1025), (257, 2047), (100, 197),
                  # a handful of very long rows shared by several blocks: odd and even lengths, one and many rows
                  (1, 50257), (16, 50257), (3, 32768), (64, 16385),
                  # thousands of rows of at most 16 elements (of one element): a lane per row
                  (5000, 1), (4100, 7), (70, 60, 16), (4200, 13)]


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES, ids=str)
@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_softmax(device, dtype, shape):
    if dtype is ta.float64 and shape == (2, 70000):
        shape = (2, 9000)
    x = values(dtype, 18, shape, -6.0, 6.0)
    got = ops.softmax(ta.tensor(x, dtype, device), None, 0.25)
    want = softmax_definition(x, None, 0.25)
    # exp of a float argument near -3: an ulp of the argument is 2^-22, so the quotient carries a few 1e-7 of relative error
    slack = {ta.float16: 1.5, ta.bfloat16: 1.5, ta.float32: 16.0, ta.float64: 256.0}[dtype]
    check(f64(got), want, dtype, f"softmax {dtype} {shape}", slack)
    np.testing.assert_allclose(f64(got).sum(axis=-1), 1.0, rtol=0, atol=shape[-1] * ROUNDING[dtype])


@pytest.mark.parametrize("n", [16, 128, 512, 100, 197])
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16, ta.float32], ids=str)
def test_softmax_causal_mask(device, dtype, n):
    x = values(dtype, 19, (2, 3, n, n), -8.0, 8.0)
    m = causal(n, dtype)
    got = f64(ops.softmax(ta.tensor(x, dtype, device), ta.tensor(m, dtype, device), 1.0 / math.sqrt(128)))
    want = softmax_definition(x, m, 1.0 / math.sqrt(128))
    slack = {ta.float16: 1.5, ta.bfloat16: 1.5, ta.float32: 16.0}[dtype]
    check(got, want, dtype, f"softmax causal {dtype} {n}", slack)
    upper = np.triu(np.ones((n, n), dtype=bool), 1)
    assert (got[..., upper] == 0.0).all()                      # masked entries are exactly zero
    np.testing.assert_array_equal(got[..., 0, 0], 1.0)         # the first row attends to one entry


@pytest.mark.parametrize("dtype", [ta.float16, ta.float32], ids=str)
def test_softmax_causal_mask_over_many_short_rows(device, dtype):
    """300 heads of 16 x 16 scores under a causal mask: rows of 16 elements, a lane each."""
    x = values(dtype, 20, (300, 16, 16), -8.0, 8.0)
    m = causal(16, dtype)
    got = f64(ops.softmax(ta.tensor(x, dtype, device), ta.tensor(m, dtype, device), 0.5))
    want = softmax_definition(x, m, 0.5)
    check(got, want, dtype, f"softmax causal short rows {dtype}", {ta.float16: 1.5, ta.float32: 16.0}[dtype])
    assert (got[..., np.triu(np.ones((16, 16), dtype=bool), 1)] == 0.0).all()


def test_softmax_shift_invariance(device):
    """Adding a constant to a row changes nothing: the maximum is subtracted first (values chosen so the sum is exact)."""
    x = np.array([[0.0, 1.0, 2.0, 3.0] * 16], dtype=np.float32)
    a = ops.softmax(ta.tensor(x, ta.float32, device)).numpy()
    b = ops.softmax(ta.tensor(x + 64.0, ta.float32, device)).numpy()
    np.testing.assert_array_equal(a, b)
    big = ops.softmax(ta.tensor(np.array([[1e4, 1e4 - 1.0, -1e4, 0.0] * 16], dtype=np.float32), ta.float32, device)).numpy()
    assert np.isfinite(big).all()


def test_softmax_fully_masked_row_is_nan(device):
    x = np.zeros((2, 64), dtype=np.float32)
    m = np.zeros((2, 64), dtype=np.float32)
    m[1] = -np.inf
    got = ops.softmax(ta.tensor(x, ta.float32, device), ta.tensor(m, ta.float32, device)).numpy()
    np.testing.assert_array_equal(got[0], np.float32(1.0 / 64))
    assert np.isnan(got[1]).all()


def test_softmax_over_long_rows_with_masked_ranges(device):
    """Rows shared by several blocks: a block whose whole range is masked adds nothing, a row masked everywhere is NaN, and
    the other entries are what the definition gives."""
    length = 40000
    x = values(ta.float32, 23, (3, length), -4.0, 4.0)
    m = np.zeros((3, length), dtype=np.float32)
    m[0, :20000] = -np.inf      # the first blocks of row 0 see -inf only
    m[1, 12345:] = -np.inf
    m[2] = -np.inf
    got = ops.softmax(ta.tensor(x, ta.float32, device), ta.tensor(m, ta.float32, device)).numpy().astype(np.float64)
    want = softmax_definition(x[:2], m[:2], 1.0)
    np.testing.assert_allclose(got[:2], want, rtol=2e-5, atol=1e-12)
    assert (got[0, :20000] == 0.0).all() and (got[1, 12345:] == 0.0).all()
    assert np.isnan(got[2]).all()


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16], ids=str)
def test_softmax_not_worse_than_the_chain(device, dtype):
    x = values(dtype, 20, (8, 64, 64), -8.0, 8.0)
    m = causal(64, dtype)
    dx, dm = ta.tensor(x, dtype, device), ta.tensor(m, dtype, device)
    s = ops.add(ops.scale(dx, 0.125), dm)
    e = ops.exp(ops.sub(s, ops.max(s, -1, True)))
    r = ops.rsqrt(ops.sum(e, -1, True))
    chain = f64(ops.mul(ops.mul(e, r), r))
    fused = f64(ops.softmax(dx, dm, 0.125))
    want = softmax_definition(x, m, 0.125)
    assert np.abs(fused - want).max() <= np.abs(chain - want).max() + 1e-12


def test_softmax_rejects_bad_mask(device):
    x = ta.tensor(np.zeros((2, 8, 8)), ta.float32, device)
    with pytest.raises(ops.TannicError):
        ops.softmax(x, ta.tensor(np.zeros((4, 8)), ta.float32, device))


# ---- rope ------------------------------------------------------------------------------------
def rope_definition(x, cos, sin):
    x, cos, sin = x.astype(np.float64), cos.astype(np.float64), sin.astype(np.float64)
    out = np.empty_like(x)
    out[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
    out[..., 1::2] = x[..., 0::2] * sin + x[..., 1::2] * cos
    return out


def tables(n, d, dtype):
    inv = 500000.0 ** (-np.arange(0, d, 2, dtype=np.float64) / d)
    ang = np.outer(np.arange(n, dtype=np.float64), inv)
    c, s = ta.tensor(np.cos(ang), dtype, ta.Host()), ta.tensor(np.sin(ang), dtype, ta.Host())
    return c.numpy(), s.numpy()


@pytest.mark.parametrize("layout", ["plain", "heads_transposed", "sliced"])
@pytest.mark.parametrize("shape", [(1, 4, 24, 128), (2, 3, 10, 6), (5, 64), (2, 2, 7, 16)], ids=str)
@pytest.mark.parametrize("dtype", FLOATS, ids=str)
def test_rope(device, dtype, shape, layout):
    n, d = shape[-2], shape[-1]
    c, s = tables(n, d, dtype)
    dc, ds = ta.tensor(c, dtype, device), ta.tensor(s, dtype, device)
    if layout == "heads_transposed":
        if len(shape) != 4:
            pytest.skip("needs a head axis")
        stored = values(dtype, 21, (shape[0], shape[2], shape[1], shape[3]))
        x, dx = stored.transpose(0, 2, 1, 3), ta.tensor(stored, dtype, device).transpose(1, 2)
    elif layout == "sliced":
        stored = values(dtype, 22, shape[:-1] + (2 * d,))
        x, dx = stored[..., 1::2], ta.tensor(stored, dtype, device)[(Ellipsis, slice(1, 2 * d, 2))]
    else:
        x = values(dtype, 23, shape)
        dx = ta.tensor(x, dtype, device)
    got = ops.rope(dx, dc, ds)
    assert got.shape == shape and got.is_contiguous
    # a difference of products: the float steps err relative to the operands (|x| <= 4), not to the result
    steps = 16 * (2.0 ** -53 if dtype is ta.float64 else 2.0 ** -24)
    check(f64(got), rope_definition(x, c, s), dtype, f"rope {dtype} {shape} {layout}", atol=steps)


def test_rope_keeps_pair_norms(device):
    """A rotation: x[2i]^2 + x[2i+1]^2 is unchanged (to float32 rounding), and position 0 is the identity."""
    x = values(ta.float32, 24, (2, 9, 64))
    c, s = tables(9, 64, ta.float32)
    got = ops.rope(ta.tensor(x, ta.float32, device), ta.tensor(c, ta.float32, device), ta.tensor(s, ta.float32, device)).numpy()
    before = x[..., 0::2].astype(np.float64) ** 2 + x[..., 1::2].astype(np.float64) ** 2
    after = got[..., 0::2].astype(np.float64) ** 2 + got[..., 1::2].astype(np.float64) ** 2
    np.testing.assert_allclose(after, before, rtol=1e-6, atol=1e-9)
    np.testing.assert_array_equal(got[:, 0, :], x[:, 0, :])


def test_rope_rejects_odd_width(device):
    x = ta.tensor(np.zeros((2, 3, 5)), ta.float32, device)
    t = ta.tensor(np.zeros((3, 2)), ta.float32, device)
    with pytest.raises(ops.TannicError):
        ops.rope(x, t, t)
