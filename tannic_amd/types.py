"""Element types of the backend and their host-side storage.

Codes follow ``enum type`` (``include/tannic/runtime/types.h:29-44``); sizes
follow ``dsizeof``/``nbytesof`` (``include/tannic/types.hpp:100-154``): booleans
are bit-packed, eight to a byte, and report an element size of 0.
"""
import numpy as np

from . import abi


class DType:
    __slots__ = ("code", "name", "itemsize", "storage")

    def __init__(self, code, name, itemsize, storage):
        self.code, self.name, self.itemsize, self.storage = code, name, itemsize, storage

    def __repr__(self):
        return self.name

    @property
    def is_floating(self):
        return self.code in (abi.FLOAT16, abi.BFLOAT16, abi.FLOAT32, abi.FLOAT64)

    @property
    def is_integral(self):
        return self.code in (abi.INT8, abi.INT16, abi.INT32, abi.INT64)

    @property
    def is_complex(self):
        return self.code in (abi.COMPLEX64, abi.COMPLEX128)


boolean = DType(abi.BOOLEAN, "boolean", 0, np.uint8)
int8 = DType(abi.INT8, "int8", 1, np.int8)
int16 = DType(abi.INT16, "int16", 2, np.int16)
int32 = DType(abi.INT32, "int32", 4, np.int32)
int64 = DType(abi.INT64, "int64", 8, np.int64)
float16 = DType(abi.FLOAT16, "float16", 2, np.float16)
# numpy has no bfloat16: host copies hold the raw 16 bits
bfloat16 = DType(abi.BFLOAT16, "bfloat16", 2, np.uint16)
float32 = DType(abi.FLOAT32, "float32", 4, np.float32)
float64 = DType(abi.FLOAT64, "float64", 8, np.float64)
complex64 = DType(abi.COMPLEX64, "complex64", 8, np.complex64)
complex128 = DType(abi.COMPLEX128, "complex128", 16, np.complex128)

ALL = [boolean, int8, int16, int32, int64, float16, bfloat16, float32, float64, complex64, complex128]
BY_CODE = {d.code: d for d in ALL}
BY_NAME = {d.name: d for d in ALL}


def nbytesof(dtype, nelements):
    """Bytes needed for ``nelements`` of ``dtype`` (``types.hpp:149-154``)."""
    if dtype is boolean:
        return (nelements + 7) // 8
    return dtype.itemsize * nelements


def float32_to_bfloat16_bits(x):
    """Round-to-nearest-even fp32 -> bf16, returned as uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    rounded = np.where(nan, (u >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def bfloat16_bits_to_float32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_storage(values, dtype):
    """Host values (any numeric array-like) -> array in ``dtype``'s storage form."""
    if dtype is bfloat16:
        a = np.asarray(values)
        if a.dtype == np.uint16:
            return a
        return float32_to_bfloat16_bits(a.astype(np.float32))
    if dtype is boolean:
        return np.packbits(np.asarray(values, dtype=bool).reshape(-1), bitorder="little")
    return np.asarray(values).astype(dtype.storage)


def to_numeric(storage, dtype):
    """Storage-form array -> array numpy can compute with (bf16 -> float32)."""
    if dtype is bfloat16:
        return bfloat16_bits_to_float32(storage)
    return storage
