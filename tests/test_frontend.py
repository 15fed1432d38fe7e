"""Host-side logic above the ABI: descriptors, views, dtype and shape rules."""
import numpy as np
import pytest

import tannic_amd as ta
from tannic_amd import abi, ops


def test_descriptor_follows_node_rules():
    t = ta.tensor(np.arange(24).reshape(2, 3, 4), ta.float32)
    d = t.descriptor()
    assert (d.rank, d.size, d.dtype, d.layout) == (3, 24, abi.FLOAT32, abi.CONTIGUOUS)
    assert list(d.shape.sizes[:3]) == [2, 3, 4] and list(d.strides.sizes[:3]) == [12, 4, 1]
    assert d.environment.kind == abi.HOST and d.environment.resource.host.traits == abi.PAGEABLE
    v = t.transpose(0, 2)
    dv = v.descriptor()
    assert list(dv.shape.sizes[:3]) == [4, 3, 2] and list(dv.strides.sizes[:3]) == [1, 4, 12] and dv.layout == abi.STRIDED
    s = t[1, 2]
    assert s.shape == (4,) and s.descriptor().address == t.address + (12 + 8) * 4   # offsets are in bytes
    one = ta.tensor(np.ones((1, 1)), ta.int8)
    assert one.descriptor().layout == abi.SINGLETON
    e = ta.tensor(np.ones((1, 5)), ta.float16).expand(3, 5)
    assert e.strides == (0, 1) and e.descriptor().layout == abi.STRIDED


def test_boolean_tensors_are_bit_packed():
    b = ta.Tensor(ta.boolean, (3, 7))
    assert b.nbytes == 3 and ta.types.nbytesof(ta.boolean, 8) == 1 and ta.types.nbytesof(ta.boolean, 9) == 2


def test_broadcast_and_promotion_rules():
    assert ops.broadcast((2, 1, 3), (1, 4, 3)) == (2, 4, 3)
    assert ops.broadcast((3,), (2, 4, 3)) == (2, 4, 3)
    with pytest.raises(ta.TannicError):
        ops.broadcast((2, 3), (4, 3))
    assert ops.promote(ta.float16, ta.float32) is ta.float32
    assert ops.promote(ta.int64, ta.float16) is ta.float16      # larger enum wins, whatever the width
    assert ops._composition_dtype(ta.int32, ta.int32) is ta.int64
    assert ops._composition_dtype(ta.int8, ta.int16) is ta.int32
    assert ops._composition_dtype(ta.bfloat16, ta.bfloat16) is ta.bfloat16
    assert ops._composition_dtype(ta.float16, ta.float32) is ta.float32


def test_reduction_shapes():
    assert ops._reduced_shape((2, 3, 4), 1, False) == (2, 4)
    assert ops._reduced_shape((2, 3, 4), 1, True) == (2, 1, 4)
    assert ops._reduced_shape((5,), 0, False) == ()


def test_bfloat16_round_trip_is_nearest_even():
    x = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.0e38, np.inf], dtype=np.float32)
    bits = ta.types.float32_to_bfloat16_bits(x)
    assert list(bits[:3]) == [0x3F80, 0x3F80, 0x3F82]   # ties go to the even mantissa
    assert ta.types.bfloat16_bits_to_float32(bits)[3] == -2.5 and np.isinf(ta.types.bfloat16_bits_to_float32(bits)[5])


def test_scalars_are_cast_the_reference_way():
    assert ops.scalar_bytes(3, ta.int32) == (3).to_bytes(4, "little")
    assert ops.scalar_bytes(1.00390625, ta.bfloat16) == (0x3F80).to_bytes(2, "little")  # truncation
    assert ops.scalar_bytes(0.333, ta.float16) == int(ops.float_to_half_bits(0.333)).to_bytes(2, "little")
    # 1 + 2^-11 is a tie: half-up gives the next value, nearest-even would keep 1.0
    assert ops.float_to_half_bits(1.0 + 2.0 ** -11) == 0x3C01
