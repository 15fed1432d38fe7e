"""Tannic's tensor file layout (include/tannic/serialization.hpp:26-66): the byte layout is pinned by an image written
out by hand from the packed records, the reader/writer by round trips over every dtype, the reader's checks by
damaged images."""
import struct

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import serialization as ser


def test_layout_known_answer():
    """int32 [2,3] = 0..5: Header{0x43495245, 1, 0xABCD, 18 + 16 + 24}, Metadata{14, 0, 24, 2}, shape, data."""
    t = ta.tensor(np.arange(6).reshape(2, 3), ta.int32, ta.Host())
    want = (bytes.fromhex("45524943") + b"\x01" + bytes.fromhex("cdab") + struct.pack("<Q", 58)      # ERIC in memory order
            + b"\x0e" + struct.pack("<QQ", 0, 24) + b"\x02" + struct.pack("<QQ", 2, 3) + np.arange(6, dtype="<i4").tobytes())
    assert len(want) == 15 + 18 + 16 + 24
    assert ser.dumps(t) == want
    back = ser.loads(want)
    assert back.dtype is ta.int32 and back.shape == (2, 3)
    np.testing.assert_array_equal(back.numpy(), np.arange(6).reshape(2, 3))


def test_record_sizes_follow_pack_1():
    assert ser.HEADER.size == 4 + 1 + 2 + 8 and ser.METADATA.size == 1 + 8 + 8 + 1


def test_dtype_codes():
    """dcodeof (include/tannic/types.hpp:206-221)."""
    assert [ser.DCODES[d] for d in (ta.boolean, ta.int8, ta.int16, ta.int32, ta.int64, ta.float16, ta.bfloat16, ta.float32,
                                    ta.float64, ta.complex64, ta.complex128)] == [1, 12, 13, 14, 15, 23, 231, 24, 25, 35, 36]


@pytest.mark.parametrize("shape", [(), (7,), (3, 5), (2, 3, 4, 5), (0, 4)], ids=str)
@pytest.mark.parametrize("dtype", [d for d in ta.types.ALL], ids=str)
def test_round_trip_on_the_host(dtype, shape, tmp_path):
    if dtype is ta.boolean:
        values = support.uniform(3, 1, shape) > 0
    else:
        values = support.values_for(dtype, 3, 1, shape)
    t = ta.tensor(np.asarray(values).reshape(shape), dtype, ta.Host())
    path = tmp_path / "t.tannic"
    ser.save(t, path)
    back = ser.load(path)
    assert back.dtype is dtype and back.shape == tuple(shape)
    support.assert_bit_exact(back.storage(), t.storage(), f"round trip {dtype} {shape}")
    assert path.stat().st_size == 15 + 18 + 8 * len(shape) + t.nbytes


def test_views_are_refused():
    t = ta.tensor(np.arange(12).reshape(3, 4), ta.float32, ta.Host()).transpose(0, 1)
    with pytest.raises(ser.FormatError):
        ser.dumps(t)


@pytest.mark.parametrize("damage", ["magic", "version", "checksum", "short", "size", "dcode", "rank", "shape"])
def test_damaged_images_are_refused(damage):
    image = bytearray(ser.dumps(ta.tensor(np.arange(6).reshape(2, 3), ta.float32, ta.Host())))
    if damage == "magic":
        image[0] ^= 0xFF
    elif damage == "version":
        image[4] = 2
    elif damage == "checksum":
        image[5] ^= 0xFF
    elif damage == "short":
        image = image[:-4]
    elif damage == "size":
        image[7:15] = struct.pack("<Q", 57)
    elif damage == "dcode":
        image[15] = 99
    elif damage == "rank":
        image[32] = 9
    elif damage == "shape":
        image[33:41] = struct.pack("<Q", 5)
    with pytest.raises(ser.FormatError):
        ser.loads(bytes(image))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16, ta.float32, ta.int64, ta.boolean], ids=str)
def test_load_straight_onto_the_device(device, dtype, tmp_path):
    values = support.uniform(4, 2, (5, 33)) > 0 if dtype is ta.boolean else support.values_for(dtype, 4, 2, (5, 33))
    host = ta.tensor(values, dtype, ta.Host())
    ser.save(host, tmp_path / "w.tannic")
    dev = ser.load(tmp_path / "w.tannic", device)
    assert isinstance(dev.environment, ta.Device)
    support.assert_bit_exact(dev.storage(), host.storage(), f"device load {dtype}")
    # and back: a device tensor is written from its bytes
    assert ser.dumps(dev) == ser.dumps(host)
