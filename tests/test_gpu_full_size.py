"""The benchmark configurations at their full sizes.

The CPU checker cannot finish these sizes in seconds, so each case is checked three ways that do not depend on the
size: (1) slices the checker CAN finish (rows of a product, images of a batch, slabs of a tensor) are cut out of
the full-size device result and compared with the checker at the usual bars; (2) float64 numpy on more of the
result; (3) a property of the operation itself (scaling an operand by two scales the product exactly, a
reduction of a repeated tensor repeats, a checksum of a product equals the product of checksums).
Inputs are seeded; a tensor repeats a block of 2^22 values so that the host side stays short.
"""
import gc
import math

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import ops, types

pytestmark = pytest.mark.gpu
BLOCK = 1 << 22


def tiled(kind, tensor_id, shape, dtype, scale):
    n = int(np.prod(shape))
    period = min(n, BLOCK)
    base = support.normal(0, tensor_id, (period,), scale) if kind == "normal" else support.uniform(0, tensor_id, (period,), -scale, scale)
    # the block is rounded to the tensor's type first: the array returned is what the tensor will hold
    if dtype.is_integral:
        base = np.floor(base).astype(dtype.storage)
    elif dtype is ta.float16:
        base = base.astype(np.float16)
    elif dtype is ta.bfloat16:
        base = types.bfloat16_bits_to_float32(types.float32_to_bfloat16_bits(base))
    else:
        base = base.astype(dtype.storage)
    return np.resize(base, n).reshape(shape)


def cut(t, index):
    """A slice of a device tensor as numbers, copied on the device first so that only the slice travels."""
    return ops.repack(t[index]).numpy()


@pytest.fixture(autouse=True)
def release_memory():
    yield
    gc.collect()


# ---- fp16 GEMM at the Llama-3-8B projection shapes and the square case -------------------------------------
GEMM_SHAPES = [(m, n) for n in (4096, 14336) for m in (1, 16, 128, 2048)] + [(4096, 4096)]


@pytest.mark.parametrize("m,n", GEMM_SHAPES, ids=lambda v: str(v))
def test_fp16_gemm_full_size(device, oracle, m, n):
    k = 4096
    x = tiled("normal", 1, (m, k), ta.float16, 1.0)
    w = tiled("normal", 2, (n, k), ta.float16, 0.02)
    dx, dw = ta.tensor(x, ta.float16, device), ta.tensor(w, ta.float16, device)
    got = ops.matmul(dx, dw.transpose()).numpy()
    assert got.shape == (m, n) and np.isfinite(got).all()
    # (1) the checker on a few rows (fp32 accumulation on both sides)
    rows = sorted({0, m // 2, m - 1})
    hw = ta.tensor(w, ta.float16, ta.Host())
    want = ops.matmul(ta.tensor(x[rows], ta.float16, ta.Host()), hw.transpose()).numpy()
    support.assert_close(got[rows], want, 2e-3, 1e-3, f"gemm rows {rows} of [{m},{k}].[{n},{k}]^T")
    # (2) float64 on one row of every 64-row band: every tile of the result is touched
    band = np.arange(0, m, 64)
    exact = x[band].astype(np.float64) @ w.astype(np.float64).T
    support.assert_close(got[band], exact, 2e-3, 1e-3, "gemm against float64")
    # (3a) doubling X doubles the product exactly (powers of two commute with every rounding here)
    #      away from the subnormal range of the result type, where the two roundings sit on different grids
    twice = ops.matmul(ta.tensor(x * np.float16(2.0), ta.float16, device), dw.transpose()).numpy()
    normal = np.abs(got) >= 2.0 ** -13
    np.testing.assert_array_equal(twice[normal], (got * np.float16(2.0))[normal])
    support.assert_close(twice[~normal], got[~normal].astype(np.float64) * 2.0, 0, 2.0 ** -23, "doubling, subnormal results")
    # (3b) checksum of checksums: 1^T (X W^T) 1 = (1^T X)(W^T 1); the fp16 rounding of each entry averages out
    total = got.astype(np.float64).sum()
    expect = x.astype(np.float64).sum(axis=0) @ w.astype(np.float64).sum(axis=0)
    spread = math.sqrt(m * n) * 2.0 ** -11 * np.abs(got).astype(np.float64).mean() * 8
    assert abs(total - expect) <= spread + 1e-6 * abs(expect), (total, expect, spread)


def test_fp32_gemm_512_is_the_reference_configuration(device, oracle):
    """fp32 [512,512] . [512,512], uniform [-1,1) from seed 0, against the checker within rel 1e-5."""
    a, b = support.uniform(0, 0, (512, 512)), support.uniform(0, 1, (512, 512))
    got = ops.matmul(ta.tensor(a, ta.float32, device), ta.tensor(b, ta.float32, device)).numpy()
    want = ops.matmul(ta.tensor(a, ta.float32, ta.Host()), ta.tensor(b, ta.float32, ta.Host())).numpy()
    support.assert_close(got, want, 1e-5, 512 * 2.0 ** -24 * 4, "fp32 gemm 512^3")


# ---- conv2d, batch 32, the three ResNet-50-style layers ------------------------------------------------------
CONV_LAYERS = {
    "3_to_64_k7_s2_p3_at_224": ((32, 3, 224, 224), (64, 3, 7, 7), 2, 3),
    "64_to_64_k3_s1_p1_at_56": ((32, 64, 56, 56), (64, 64, 3, 3), 1, 1),
    "256_to_512_k1_s2_at_56": ((32, 256, 56, 56), (512, 256, 1, 1), 2, 0),
}


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16, ta.float32], ids=str)
@pytest.mark.parametrize("layer", list(CONV_LAYERS))
def test_conv2d_full_size(device, oracle, layer, dtype):
    xs, ws, stride, pad = CONV_LAYERS[layer]
    fan_in = ws[1] * ws[2] * ws[3]
    x = tiled("normal", 3, xs, dtype, 1.0)
    w = tiled("normal", 4, ws, dtype, math.sqrt(2.0 / fan_in))
    bias = np.zeros(ws[0], dtype=np.float32)
    dx, dw, db = ta.tensor(x, dtype, device), ta.tensor(w, dtype, device), ta.tensor(bias, dtype, device)
    got = ops.convolve2d(dx, dw, db, stride, pad)
    ho = (xs[2] + 2 * pad - ws[2]) // stride + 1
    assert got.shape == (xs[0], ws[0], ho, ho)
    hw, hb = ta.tensor(w, dtype, ta.Host()), ta.tensor(bias, dtype, ta.Host())
    rtol, atol = (1e-5, fan_in * 2.0 ** -24 * 8) if dtype is ta.float32 else (2e-3 if dtype is ta.float16 else 2.0 ** -7, 1e-3)
    # (1) the checker on the first and the last image
    for image in (0, xs[0] - 1):
        want = ops.convolve2d(ta.tensor(x[image:image + 1], dtype, ta.Host()), hw, hb, stride, pad).numpy()
        support.assert_close(cut(got, slice(image, image + 1)), want, rtol, atol, f"conv {layer} {dtype} image {image}")
    # (3) images are independent of their place in the batch: the reversed batch gives the reversed result, bit for bit
    reversed_result = ops.convolve2d(ta.tensor(np.ascontiguousarray(x[::-1]), dtype, device), dw, db, stride, pad)
    np.testing.assert_array_equal(cut(reversed_result, slice(0, 1)), cut(got, slice(xs[0] - 1, xs[0])))
    np.testing.assert_array_equal(cut(reversed_result, slice(20, 21)), cut(got, slice(xs[0] - 21, xs[0] - 20)))


# ---- the broadcasting elementwise chain on [64, 4096, 1024] ------------------------------------------------------
SHAPE = (64, 4096, 1024)
SLABS = (0, 31, 63)


def chain(x, z):
    three_x = ops.scale(x, 3)
    one = ta.tensor(np.ones(1), x.dtype, x.environment)
    return ops.add(ops.sub(ops.add(ops.log(ops.add(ops.abs(x), one)), ops.mul(z, z)), ops.exp(x)), three_x)


@pytest.mark.parametrize("dtype", [ta.float32, ta.float16], ids=str)
def test_elementwise_chain_full_size(device, oracle, dtype):
    x = tiled("uniform", 5, SHAPE, dtype, 4.0)
    z = tiled("uniform", 6, (1, 4096, 1), dtype, 4.0)
    dx, dz = ta.tensor(x, dtype, device), ta.tensor(z, dtype, device)
    got = chain(dx, dz)
    assert got.shape == SHAPE
    hz = ta.tensor(z, dtype, ta.Host())
    # every node rounds once on both sides; exp and log differ from the host's by an ulp of float here and there
    # (exp(4) = 55: an ulp of the fp16 exponential is 0.03, of the float one 4e-6) and the sum can cancel to near zero
    rtol, atol = (1e-5, 2e-4) if dtype is ta.float32 else (4e-3, 7e-2)
    for k in SLABS:
        want = chain(ta.tensor(x[k:k + 1], dtype, ta.Host()), hz).numpy()
        support.assert_close(cut(got, slice(k, k + 1)), want, rtol, atol, f"chain {dtype} slab {k}")
    # the tensor repeats every BLOCK elements = one slab: so does the result, bit for bit
    np.testing.assert_array_equal(cut(got, slice(5, 6)), cut(got, slice(6, 7)))
    del got, dx
    # float64 definition on one slab
    k = 17
    x64, z64 = x[k].astype(np.float64), z[0].astype(np.float64)
    exact = np.log(np.abs(x64) + 1.0) + z64 * z64 - np.exp(x64) + 3.0 * x64
    got_k = cut(chain(ta.tensor(x[k:k + 1], dtype, device), dz), slice(0, 1))[0]
    support.assert_close(got_k, exact, 1e-5 if dtype is ta.float32 else 6e-3, 2e-4 if dtype is ta.float32 else 0.15, "chain against float64")


def test_int32_add_and_compare_full_size_bit_exact(device, oracle):
    a = tiled("uniform", 7, SHAPE, ta.int32, 4.0)
    b = tiled("uniform", 8, SHAPE, ta.int32, 4.0)
    z = tiled("uniform", 9, (1, 4096, 1), ta.int32, 4.0)
    da, db, dz = ta.tensor(a, ta.int32, device), ta.tensor(b, ta.int32, device), ta.tensor(z, ta.int32, device)
    total, wider, greater = ops.add(da, db), ops.add(da, dz), ops.gt(da, db)
    for k in SLABS:
        ha, hb = ta.tensor(a[k:k + 1], ta.int32, ta.Host()), ta.tensor(b[k:k + 1], ta.int32, ta.Host())
        np.testing.assert_array_equal(cut(total, slice(k, k + 1)), ops.add(ha, hb).numpy())
        np.testing.assert_array_equal(cut(wider, slice(k, k + 1)), ops.add(ha, ta.tensor(z, ta.int32, ta.Host())).numpy())
    # the bit-packed comparison: the whole mask against numpy, one slab against the checker
    mask = greater.storage()
    np.testing.assert_array_equal(mask, a > b)
    np.testing.assert_array_equal(mask[0], ops.gt(ta.tensor(a[0:1], ta.int32, ta.Host()), ta.tensor(b[0:1], ta.int32, ta.Host())).storage()[0])


# ---- reductions of [64, 4096, 1024] ------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [ta.float32, ta.float16], ids=str)
def test_reductions_full_size(device, oracle, dtype):
    x = tiled("uniform", 10, SHAPE, dtype, 4.0)
    dx = ta.tensor(x, dtype, device)
    sum_tol = (1e-5, 1e-3) if dtype is ta.float32 else (2e-3, 2e-2)
    for axis in (2, 1):
        results = {name: getattr(ops, name)(dx, axis).numpy() for name in ("sum", "mean", "max", "min", "argmax", "argmin")}
        # (1) the checker on a slab (the slab keeps its axes: [1, 4096, 1024])
        for k in (0, 63):
            hx = ta.tensor(x[k:k + 1], dtype, ta.Host())
            for name in ("max", "min", "argmax", "argmin"):
                np.testing.assert_array_equal(results[name][k], getattr(ops, name)(hx, axis).numpy()[0], err_msg=f"{name} axis {axis} slab {k}")
            for name in ("sum", "mean"):
                support.assert_close(results[name][k], getattr(ops, name)(hx, axis).numpy()[0], *sum_tol, f"{name} axis {axis} slab {k}")
        # (2) numpy on three slabs (the tensor repeats slab by slab, so more of them add nothing)
        for k in SLABS:
            np.testing.assert_array_equal(results["argmax"][k], x[k].argmax(axis=axis - 1))
            np.testing.assert_array_equal(results["argmin"][k], x[k].argmin(axis=axis - 1))
            np.testing.assert_array_equal(results["max"][k], x[k].max(axis=axis - 1))
            support.assert_close(results["sum"][k], x[k].astype(np.float64).sum(axis=axis - 1), *sum_tol, f"sum axis {axis} against float64")
            support.assert_close(results["mean"][k], x[k].astype(np.float64).mean(axis=axis - 1), *sum_tol, f"mean axis {axis} against float64")
        # (3) every slab holds the same block: so does every slab of every result
        for name, values in results.items():
            np.testing.assert_array_equal(values[1:], np.broadcast_to(values[0], values[1:].shape), err_msg=f"{name} axis {axis} across slabs")
    # axis 0 crosses the slabs: float64 numpy and the repetition property (every slab is the same block, so the maximum
    # over slabs is the block itself, first found in slab 0)
    np.testing.assert_array_equal(ops.max(dx, 0).numpy(), x[0])
    np.testing.assert_array_equal(ops.argmax(dx, 0).numpy(), np.zeros(SHAPE[1:], dtype=np.int64))
    support.assert_close(ops.sum(dx, 0).numpy(), x[0].astype(np.float64) * SHAPE[0], *sum_tol, "sum axis 0 against float64")


def test_byte_offsets_beyond_4_gib(device):
    """Tensors of 4.4 GB (element counts under 2^31, byte offsets over 2^32): elementwise, broadcast, both reduction
    directions, argmax and a transposing copy index them with 64-bit offsets."""
    n = 1_100_000_000
    x = (np.arange(n, dtype=np.int64) % 1000).astype(np.float32)
    dx = ta.tensor(x, ta.float32, device)
    got = ops.add(dx, dx).numpy()
    assert (got[-1_000_000:] == 2 * x[-1_000_000:]).all() and (got[::4097] == 2 * x[::4097]).all()
    del got
    cube = dx.view(1100, 1000, 1000)
    got = ops.mul(cube, ta.tensor(np.full((1, 1000, 1), 3.0), ta.float32, device)).numpy().reshape(-1)
    assert (got[-1_000_000:] == 3 * x[-1_000_000:]).all() and (got[::4099] == 3 * x[::4099]).all()
    del got
    blocks = x.reshape(1100, 1000, 1000)
    np.testing.assert_allclose(ops.sum(cube, 2).numpy(), blocks.sum(axis=2, dtype=np.float64), rtol=1e-6)
    np.testing.assert_allclose(ops.sum(cube, 0).numpy(), blocks.sum(axis=0, dtype=np.float64), rtol=1e-6)
    assert (ops.argmax(cube, 1).numpy() == blocks.argmax(axis=1)).all()
    turned = ops.repack(cube.transpose(0, 2)).numpy()
    assert (turned[:, :, -3:] == blocks.transpose(2, 1, 0)[:, :, -3:]).all() and (turned[::7, ::11] == blocks.transpose(2, 1, 0)[::7, ::11]).all()


def test_more_than_two_to_the_31_elements(device):
    """An int8 tensor of 2^31 + 2^21 elements (the reference indexes with size_t throughout, src/cpu/ops-binary.cpp:48-61):
    the elementwise engine counts 16-byte vectors, not elements, so add, a broadcast multiply, neg and a copy of a
    transposed view take it; reductions index their source with 64-bit offsets and take it too.  Bit-exact."""
    rows, width = 2048 + 2, 1 << 20
    n = rows * width
    assert n > 1 << 31
    block = ((np.arange(1 << 22, dtype=np.int64) * 37 + 11) % 251 - 125).astype(np.int8)
    x = np.resize(block, n)
    dx = ta.tensor(x, ta.int8, device)
    got = ops.add(dx, dx).numpy()
    want = (x.astype(np.int16) * 2).astype(np.int8)
    assert (got[-3_000_000:] == want[-3_000_000:]).all() and (got[:: 4099] == want[:: 4099]).all() and (got[1 << 31: (1 << 31) + 4096] == want[1 << 31: (1 << 31) + 4096]).all()
    del got, want
    got = ops.neg(dx).numpy()
    assert (got[-3_000_000:] == -x[-3_000_000:]).all() and (got[:: 4099] == -x[:: 4099]).all()
    del got
    grid = dx.view(rows, 1024, 1024)
    three = ta.tensor(np.full((1, 1024, 1), 3), ta.int8, device)
    got = ops.mul(grid, three).numpy().reshape(-1)
    want = (x.astype(np.int16) * 3).astype(np.int8)
    assert (got[-3_000_000:] == want[-3_000_000:]).all() and (got[:: 4099] == want[:: 4099]).all()
    del got, want
    blocks = x.reshape(rows, 1024, 1024)
    got = ops.sum(grid, 2).numpy()
    np.testing.assert_array_equal(got, blocks.sum(axis=2, dtype=np.int64).astype(np.int8))
    got = ops.argmax(grid, 0).numpy()
    np.testing.assert_array_equal(got, blocks.argmax(axis=0))
