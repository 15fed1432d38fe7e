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
