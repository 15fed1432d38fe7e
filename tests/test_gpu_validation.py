"""Descriptors that do not fit each other are refused with ERROR before anything is launched: the kernels index one
operand by another's coordinates, so a mismatch would read or write outside a tensor."""
import ctypes as C

import numpy as np
import pytest

import tannic_amd as ta
from tannic_amd import abi, ops

pytestmark = pytest.mark.gpu


def call(name, device, sources, dst, extra=()):
    lib = ta.library()
    dvc = device.structure()
    stream = lib.pop_stream(C.byref(dvc))
    descs = [s.descriptor() for s in sources]
    out = dst.descriptor()
    status = lib.kernels[name](*[C.byref(d) for d in descs], C.byref(out), stream, *extra)
    lib.put_stream(C.byref(dvc), stream)
    return status, lib.error_message()


def zeros(shape, dtype, device):
    return ta.tensor(np.zeros(shape), dtype, device)


@pytest.mark.parametrize("name", ["add", "mul", "div", "swiglu"])
def test_binary_operand_must_broadcast_to_the_destination(device, name):
    a, b = zeros((4, 6), ta.float32, device), zeros((5, 6), ta.float32, device)
    status, message = call(name, device, [a, b], zeros((4, 6), ta.float32, device))
    assert status == abi.ERROR and "broadcast" in message
    # rank above the destination's
    status, _ = call(name, device, [zeros((2, 4, 6), ta.float32, device), a], zeros((4, 6), ta.float32, device))
    assert status == abi.ERROR


@pytest.mark.parametrize("name,extra", [("exp", ()), ("neg", ()), ("rsqrt", (C.c_float(0.0),)), ("cast", ())])
def test_unary_shapes_must_match(device, name, extra):
    status, message = call(name, device, [zeros((4, 6), ta.float32, device)], zeros((4, 7), ta.float32, device), extra)
    assert status == abi.ERROR and "shapes differ" in message


def test_compare_shapes_must_match(device):
    a, b = zeros((4, 8), ta.int32, device), zeros((1, 8), ta.int32, device)
    status, message = call("gt", device, [a, b], zeros((4, 8), ta.boolean, device))
    assert status == abi.ERROR and "shapes differ" in message


def test_allclose_shapes_must_match(device):
    lib = ta.library()
    dvc = device.structure()
    stream = lib.pop_stream(C.byref(dvc))
    a, b = zeros((4, 8), ta.float32, device).descriptor(), zeros((4, 9), ta.float32, device).descriptor()
    r = lib.kernels["allclose"](C.byref(a), C.byref(b), stream, 1e-5, 1e-8)
    lib.put_stream(C.byref(dvc), stream)
    assert r == -1


def test_well_formed_calls_still_succeed(device):
    a, b = zeros((4, 6), ta.float32, device), zeros((1, 6), ta.float32, device)
    status, _ = call("add", device, [a, b], zeros((4, 6), ta.float32, device))
    assert status == abi.SUCCESS
    assert ops.add(a, b).shape == (4, 6)


@pytest.mark.parametrize("name", ["argsum", "argmax", "max"])
def test_reduction_destination_must_hold_one_element_per_slice(device, name):
    src = zeros((4, 6, 8), ta.float32, device)
    dtype = ta.int64 if name == "argmax" else ta.float32
    status, message = call(name, device, [src], zeros((4, 6), dtype, device), (C.c_uint8(1),))
    assert status == abi.ERROR and "destination" in message
    status, _ = call(name, device, [src], zeros((4, 8), dtype, device), (C.c_uint8(1),))
    assert status == abi.SUCCESS
    status, _ = call(name, device, [src], zeros((4, 1, 8), dtype, device), (C.c_uint8(1),))   # kept dimension
    assert status == abi.SUCCESS


def test_gemm_operand_extents_must_fit_the_destination(device):
    """The kernels take M and N from the destination and K from the first operand: operands that are smaller than that
    would be read past their end."""
    f = lambda *shape: zeros(shape, ta.float16, device)
    for a, b, dst in ((f(8, 8), f(8, 8), f(16, 16)),                 # destination larger than the product
                      (f(64, 32), f(64, 64), f(64, 64)),             # K of the second operand
                      (f(64, 64), f(64, 32), f(64, 64)),             # N of the second operand
                      (f(32, 64), f(64, 64), f(64, 64)),             # M of the first operand
                      (f(2, 64, 64), f(64, 64), f(3, 64, 64)),       # batch extent neither 1 nor the destination's
                      (f(2, 3, 8, 8), f(8, 8), f(3, 8, 8))):         # operand of higher rank than the destination
        status, message = call("gemm", device, [a, b], dst)
        assert status == abi.ERROR and "gemm" in message, (a.shape, b.shape, dst.shape, status, message)
    status, _ = call("gemm", device, [f(1, 64, 32), f(32, 64)], f(3, 64, 64))
    assert status == abi.SUCCESS


def test_copy_and_complex_operands_must_fit_the_destination(device):
    status, message = call("cpy", device, [zeros((4, 6), ta.float32, device)], zeros((4, 8), ta.float32, device))
    assert status == abi.ERROR and "cpy" in message
    status, message = call("cpy", device, [zeros((4, 6), ta.float32, device)], zeros((2, 4, 6), ta.float32, device))
    assert status == abi.ERROR and "cpy" in message
    status, _ = call("cpy", device, [zeros((1, 6), ta.float32, device)], zeros((4, 6), ta.float32, device))     # extent 1 repeats
    assert status == abi.SUCCESS
    for name in ("view_as_cartesian", "view_as_polar"):
        status, message = call(name, device, [zeros((4, 6), ta.float32, device), zeros((4, 5), ta.float32, device)], zeros((4, 6), ta.complex64, device))
        assert status == abi.ERROR and "complex" in message
        status, _ = call(name, device, [zeros((4, 6), ta.float32, device), zeros((1, 6), ta.float32, device)], zeros((4, 6), ta.complex64, device))
        assert status == abi.SUCCESS


# ---- dtypes that do not fit each other -----------------------------------------------------------------------------------
# A kernel writes elements of one type: a destination described with another dtype would be over- or under-run, and a
# second operand read as the first's type (what the reference's comparison and allclose do) would be read past its end.
def test_destination_dtype_must_be_the_result_type(device):
    f32, f16, i32 = (lambda s: zeros(s, ta.float32, device)), (lambda s: zeros(s, ta.float16, device)), (lambda s: zeros(s, ta.int32, device))
    cases = [
        ("exp", [f32((4, 8))], f16((4, 8)), ()),
        ("neg", [i32((4, 8))], zeros((4, 8), ta.int64, device), ()),
        ("add", [f32((4, 8)), f32((4, 8))], zeros((4, 8), ta.float64, device), ()),
        ("mul", [i32((4, 8)), f32((4, 8))], i32((4, 8)), ()),
        ("div", [f32((4, 8)), f32((4, 8))], f16((4, 8)), ()),
        ("argsum", [f32((4, 8))], f16((4,)), (C.c_uint8(1),)),
        ("argmax", [f32((4, 8))], zeros((4,), ta.int32, device), (C.c_uint8(1),)),
        ("max", [f16((4, 8))], f32((4,)), (C.c_uint8(1),)),
        ("gemm", [f16((8, 8)), f16((8, 8))], f32((8, 8)), ()),
        ("gemm", [f32((8, 8)), f32((8, 8))], f16((8, 8)), ()),
        ("conv2d", [f16((1, 2, 6, 6)), f16((3, 2, 3, 3))], f32((1, 3, 4, 4)), (abi.SIZE2(0, 0), abi.SIZE2(1, 1))),
        ("repeat", [f32((4, 8))], f16((8, 8)), (C.c_int(0), C.c_int(2))),
        ("triu", [f32((4, 8))], zeros((4, 8), ta.float64, device), (C.c_int(0),)),
        ("gt", [f32((4, 8)), f32((4, 8))], zeros((4, 8), ta.int8, device), ()),
        ("cpy", [f32((4, 8))], f16((4, 8)), ()),
        ("view_as_polar", [f32((4, 8)), f32((4, 8))], zeros((4, 8), ta.complex128, device), ()),
    ]
    for name, sources, dst, extra in cases:
        status, message = call(name, device, sources, dst, extra)
        assert status == abi.ERROR and message, (name, status, message)


def test_scale_destination_dtype(device):
    lib = ta.library()
    dvc = device.structure()
    stream = lib.pop_stream(C.byref(dvc))
    src, dst = zeros((4, 8), ta.float32, device).descriptor(), zeros((4, 8), ta.float16, device).descriptor()
    value = C.c_float(2.0)
    scalar = abi.scalar_t(C.cast(C.pointer(value), C.c_void_p), ta.float32.code)
    status = lib.kernels["scale"](C.byref(src), C.byref(scalar), C.byref(dst), stream)
    lib.put_stream(C.byref(dvc), stream)
    assert status == abi.ERROR


def test_comparison_and_allclose_want_one_dtype(device):
    """The reference reads the second operand as the first's type (src/cpu/cmps.cpp:108-202, src/cpu/val.cpp:73-83): with
    a narrower second operand that runs past its end, so the pair is refused."""
    wide, narrow = zeros((64, 64), ta.int64, device), zeros((64, 64), ta.int8, device)
    for name in ("eq", "ne", "gt", "ge", "lt", "le"):
        status, message = call(name, device, [wide, narrow], zeros((64, 64), ta.boolean, device))
        assert status == abi.UNSUPPORTED_DTYPE and "different dtypes" in message, name
    lib = ta.library()
    dvc = device.structure()
    stream = lib.pop_stream(C.byref(dvc))
    a, b = zeros((64, 64), ta.float64, device).descriptor(), zeros((64, 64), ta.float16, device).descriptor()
    r = lib.kernels["allclose"](C.byref(a), C.byref(b), stream, 1e-5, 1e-8)
    lib.put_stream(C.byref(dvc), stream)
    assert r == -1
    with pytest.raises(ta.TannicError):
        ops.gt(wide, narrow)


# ---- nothing to do ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(0,), (3, 0), (0, 4), (2, 0, 5)])
def test_empty_tensors_go_through_every_family(device, oracle, shape):
    """A tensor without elements is a valid operand: the call succeeds, launches nothing and agrees with the CPU path
    (an empty index space once divided by zero on the host while the launch was planned)."""
    import support
    for dtype in (ta.float32, ta.float16, ta.int32):
        h, d = support.both(np.zeros(shape), dtype, device)
        for op in (ops.neg, ops.repack, lambda t: ops.add(t, t), lambda t: ops.mul(t, t), lambda t: ops.scale(t, 2), lambda t: ops.gt(t, t)):
            want, got = op(h), op(d)
            assert got.shape == want.shape and got.dtype is want.dtype
        for axis in range(len(shape)):
            for name in ("sum", "argmax", "max", "min"):
                want, got = getattr(ops, name)(h, axis), getattr(ops, name)(d, axis)
                assert got.shape == want.shape
                support.assert_bit_exact(got.storage(), want.storage(), f"{name} {dtype} {shape} axis={axis}")
    # value max / min over an axis without elements: the start value of the fold
    h, d = support.both(np.zeros((0, 4)), ta.float32, device)
    assert np.isneginf(ops.max(d, 0).numpy()).all() and np.isposinf(ops.min(d, 0).numpy()).all()
    # (the last two: extents that meet the tiled kernels' alignment conditions, whose loaders would fetch a first tile)
    for sa, sb in (((0, 4), (4, 3)), ((3, 4), (4, 0)), ((3, 0), (0, 5)), ((64, 0), (0, 512)), ((512, 0), (0, 512))):
        for dtype in (ta.float16, ta.float32):
            ha, da = support.both(np.ones(sa), dtype, device)
            hb, db = support.both(np.ones(sb), dtype, device)
            want, got = ops.matmul(ha, hb), ops.matmul(da, db)
            assert got.shape == want.shape
            support.assert_bit_exact(got.storage(), want.storage(), f"matmul {dtype} {sa} x {sb}")


def test_a_tensor_without_storage_is_refused(device):
    """A descriptor with elements and a null address is turned away at the entry (a kernel reading it would fault the
    device); one without elements needs no storage."""
    good = zeros((4, 8), ta.float32, device)
    for name, n_sources, extra in (("exp", 1, ()), ("add", 2, ()), ("gt", 2, ()), ("argsum", 1, (C.c_uint8(1),)), ("gemm", 2, ()), ("cpy", 1, ()), ("div", 2, ())):
        lib = ta.library()
        dvc = device.structure()
        stream = lib.pop_stream(C.byref(dvc))
        sources = [zeros((8, 8) if name == "gemm" else (4, 8), ta.float32, device) for _ in range(n_sources)]
        shape = {"gt": (4, 8), "argsum": (4,), "gemm": (8, 8)}.get(name, (4, 8))
        dst = zeros(shape, ta.boolean if name == "gt" else ta.float32, device)
        descs = [s.descriptor() for s in sources]
        out = dst.descriptor()
        descs[0].address = None
        status = lib.kernels[name](*[C.byref(d) for d in descs], C.byref(out), stream, *extra)
        message = lib.error_message()
        lib.put_stream(C.byref(dvc), stream)
        assert status == abi.ERROR and "no storage" in message, (name, status, message)
    del good
