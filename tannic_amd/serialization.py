"""Reader and writer of Tannic's tensor file layout (``include/tannic/serialization.hpp:26-66``).

The reference defines the records and how they are filled, not the I/O itself; a file is, in order and without
padding (``#pragma pack(1)``, little endian):

    Header            magic u32 = 0x43495245, version u8 = 1, checksum u16 = 0xABCD, nbytes u64
                      (nbytes = everything after the header: metadata + shape + data)            15 bytes
    Metadata<Tensor>  dcode u8 (``dcodeof``, ``include/tannic/types.hpp:206-221``), offset u64,
                      nbytes u64 (of the data), rank u8                                            18 bytes
    shape             rank x u64
    data              the tensor's elements, row-major (bit-packed for booleans)

``read`` places the data on the host or straight on a device (one bulk upload), which is how real weights reach
the device backend.
"""
import struct

import numpy as np

from . import types
from .tensor import Device, Host, Tensor

MAGIC = 0x43495245
VERSION = 1
CHECKSUM = 0xABCD
HEADER = struct.Struct("<IBHQ")
METADATA = struct.Struct("<BQQB")

# dcodeof / dtypeof (include/tannic/types.hpp:206-249)
DCODES = {
    types.boolean: 1, types.int8: 12, types.int16: 13, types.int32: 14, types.int64: 15, types.float16: 23,
    types.bfloat16: 231, types.float32: 24, types.float64: 25, types.complex64: 35, types.complex128: 36,
}
DTYPES = {code: dtype for dtype, code in DCODES.items()}


class FormatError(ValueError):
    pass


def dumps(tensor):
    """The file image of ``tensor`` (made contiguous first; a view's offset is not kept: the data starts at 0)."""
    if not tensor.is_contiguous():
        raise FormatError("only contiguous tensors are written; repack a view first")
    raw = tensor.raw()[: tensor.nbytes].tobytes()
    meta = METADATA.pack(DCODES[tensor.dtype], 0, len(raw), tensor.rank)
    shape = struct.pack(f"<{tensor.rank}Q", *tensor.shape)
    body = meta + shape + raw
    return HEADER.pack(MAGIC, VERSION, CHECKSUM, len(body)) + body


def loads(image, environment=None):
    """The tensor a file image holds, on ``environment`` (host by default)."""
    environment = environment or Host()
    if len(image) < HEADER.size:
        raise FormatError("shorter than a header")
    magic, version, checksum, nbytes = HEADER.unpack_from(image, 0)
    if magic != MAGIC:
        raise FormatError(f"bad magic 0x{magic:08X}")
    if version != VERSION:
        raise FormatError(f"unknown version {version}")
    if checksum != CHECKSUM:
        raise FormatError(f"bad checksum 0x{checksum:04X}")
    if len(image) - HEADER.size < nbytes or nbytes < METADATA.size:
        raise FormatError("truncated: the header announces more bytes than follow")
    dcode, offset, data_bytes, rank = METADATA.unpack_from(image, HEADER.size)
    if dcode not in DTYPES:
        raise FormatError(f"unknown dtype code {dcode}")
    if rank > 8:
        raise FormatError(f"rank {rank} exceeds the 8 dimensions a tensor can have")
    at = HEADER.size + METADATA.size
    if nbytes != METADATA.size + 8 * rank + data_bytes:
        raise FormatError("sizes in header and metadata disagree")
    shape = struct.unpack_from(f"<{rank}Q", image, at)
    at += 8 * rank
    dtype = DTYPES[dcode]
    tensor = Tensor(dtype, shape)
    if tensor.nbytes != data_bytes:
        raise FormatError(f"shape {shape} of {dtype} needs {tensor.nbytes} bytes, the file holds {data_bytes}")
    if offset != 0:
        raise FormatError("a non-zero storage offset is not supported")
    tensor.initialize(environment)
    data = np.frombuffer(image, dtype=np.uint8, count=data_bytes, offset=at)
    tensor.write_raw(data)
    return tensor


def save(tensor, path):
    with open(path, "wb") as f:
        f.write(dumps(tensor))


def load(path, environment=None):
    with open(path, "rb") as f:
        return loads(f.read(), environment)
