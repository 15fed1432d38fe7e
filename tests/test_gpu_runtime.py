"""Memory, streams and copies of the device library, called through the C ABI."""
import ctypes as C

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import abi, ops

pytestmark = pytest.mark.gpu


def test_device_count_and_invalid_ids(device):
    lib = ta.library()
    assert lib.get_device_count() >= 1
    assert lib.arch() == b"gfx950"
    with pytest.raises(IndexError):  # std::out_of_range in the reference (src/resources.cpp:46-48)
        ta.Device(lib.get_device_count())
    with pytest.raises(IndexError):
        ta.Device(-1)


def test_stream_pool_is_lifo(device):
    lib = ta.library()
    dvc = device.structure()
    s1 = lib.pop_stream(C.byref(dvc))
    s2 = lib.pop_stream(C.byref(dvc))
    assert s1.address != 0 and s2.address != 0 and s1.address != s2.address
    lib.put_stream(C.byref(dvc), s2)
    lib.put_stream(C.byref(dvc), s1)
    again = lib.pop_stream(C.byref(dvc))
    assert again.address == s1.address  # last put, first popped (src/cuda/streams.cu:23-38)
    lib.put_stream(C.byref(dvc), again)


def test_allocate_copy_compare(device):
    lib = ta.library()
    dvc = device.structure()
    data = np.arange(1000, dtype=np.float32)
    ptr = lib.allocate(C.byref(dvc), data.nbytes)
    assert ptr
    assert lib.copy_from_host(C.byref(dvc), data.ctypes.data, ptr, data.nbytes) == abi.SUCCESS
    assert lib.compare_from_host(C.byref(dvc), data.ctypes.data, ptr, data.nbytes) == 1
    other = data.copy()
    other[500] += 1
    assert lib.compare_from_host(C.byref(dvc), other.ctypes.data, ptr, data.nbytes) == 0
    back = np.empty_like(data)
    assert lib.copy_device_to_host(C.byref(dvc), ptr, back.ctypes.data, data.nbytes) == abi.SUCCESS
    assert (back == data).all()
    assert lib.deallocate(C.byref(dvc), ptr) is None


def test_element_assignment_and_read_back(device):
    """`X[i, j] = v` and `X[i, j] == v` go through copyFromHost / compareFromHost one element
    at a time (src/tensor.cpp:34-75)."""
    lib = ta.library()
    dvc = device.structure()
    x = ta.Tensor(ta.float32, (2, 3)).initialize(device)
    for i in range(6):
        v = C.c_float(i * 1.5)
        assert lib.copy_from_host(C.byref(dvc), C.byref(v), x.address + 4 * i, 4) == abi.SUCCESS
    for i in range(6):
        v = C.c_float(i * 1.5)
        assert lib.compare_from_host(C.byref(dvc), C.byref(v), x.address + 4 * i, 4) == 1
    assert (x.numpy() == np.arange(6).reshape(2, 3) * 1.5).all()


def test_tensor_copies_between_environments(device, oracle):
    h = support.host_tensor(support.uniform(1, 1, (33, 65)), ta.float32)
    d = h.to(device)
    d2 = d.to(device)          # device -> device
    back = d2.to(ta.Host())    # device -> host
    support.assert_bit_exact(back.storage(), h.storage(), "H2D, D2D, D2H")
    v = d.transpose()          # a view keeps its strides across the copy
    support.assert_bit_exact(v.to(ta.Host()).storage(), h.storage().T, "view")


def test_mixed_environments_are_rejected(device, oracle):
    h = support.host_tensor(np.ones((2, 2)), ta.float32)
    d = h.to(device)
    with pytest.raises(ta.TannicError):
        ops.add(h, d)


def test_unsupported_dtypes_report_status(device):
    lib = ta.library()
    dvc = device.structure()
    b = ta.Tensor(ta.boolean, (8,)).initialize(device)
    c = ta.Tensor(ta.complex64, (8,)).initialize(device)
    out = ta.Tensor(ta.float32, (8,)).initialize(device)
    stream = lib.pop_stream(C.byref(dvc))
    try:
        db, dc, do = b.descriptor(), c.descriptor(), out.descriptor()
        assert lib.kernels["log"](C.byref(db), C.byref(do), stream) == abi.UNSUPPORTED_DTYPE
        assert lib.kernels["log"](C.byref(dc), C.byref(do), stream) == abi.UNSUPPORTED_DTYPE
        assert lib.kernels["add"](C.byref(dc), C.byref(do), C.byref(do), stream) == abi.UNSUPPORTED_DTYPE
        assert lib.kernels["gemm"](C.byref(dc), C.byref(dc), C.byref(do), stream) == abi.UNSUPPORTED_DTYPE
        assert lib.kernels["argmean"](C.byref(db), C.byref(do), stream, 0) == abi.UNSUPPORTED_DTYPE
        assert lib.kernels["allclose"](C.byref(db), C.byref(db), stream, 1e-5, 1e-8) == -1
    finally:
        lib.put_stream(C.byref(dvc), stream)
    with pytest.raises(ta.TannicError):
        ops.exp(ta.Tensor(ta.int32, (4,)).initialize(device))


def test_released_blocks_are_reused_on_their_stream_only(device):
    """A released block goes to a later fitting request on the same stream (stream order already separates the
    two users); a request on another stream, or of a very different size, does not get it."""
    lib = ta.library()
    dvc = device.structure()
    size = 3 << 20

    def take_until(wanted, limit=256):
        """Allocates blocks of `size` until `wanted` comes back (earlier tests may have left other blocks of this size)."""
        taken = []
        while len(taken) < limit:
            ptr = lib.allocate(C.byref(dvc), size)
            taken.append(ptr)
            if ptr == wanted:
                break
        return taken

    first = lib.allocate(C.byref(dvc), size)
    lib.deallocate(C.byref(dvc), first)
    taken = take_until(first)
    assert taken[-1] == first and len(set(taken)) == len(taken)
    for ptr in taken:
        lib.deallocate(C.byref(dvc), ptr)
    small = lib.allocate(C.byref(dvc), size // 4)       # the kept block would waste three quarters
    assert small not in taken
    lib.deallocate(C.byref(dvc), small)
    # take the pool's stream away: allocations now ride on another stream and must not see the kept blocks
    held = lib.pop_stream(C.byref(dvc))
    elsewhere = lib.allocate(C.byref(dvc), size)
    assert elsewhere and elsewhere not in taken
    lib.deallocate(C.byref(dvc), elsewhere)
    lib.put_stream(C.byref(dvc), held)
    back = take_until(first)
    assert back[-1] == first
    for ptr in back:
        lib.deallocate(C.byref(dvc), ptr)


def test_temporaries_reusing_blocks_keep_results_right(device, oracle):
    """A chain of operators whose temporaries are released and handed out again at once: every result is still right."""
    x = support.values_for(ta.float32, 5, 1, (64, 257))
    dx, hx = ta.tensor(x, ta.float32, device), ta.tensor(x, ta.float32, ta.Host())
    got, want = dx, hx
    for step in range(40):
        got = ops.add(ops.mul(got, dx), ops.neg(got)) if step % 2 else ops.sub(ops.abs(got), dx)
        want = ops.add(ops.mul(want, hx), ops.neg(want)) if step % 2 else ops.sub(ops.abs(want), hx)
        got, want = ops.tanh(got), ops.tanh(want)
    support.assert_close(got.numpy(), want.numpy(), 1e-5, 1e-6, "forty operators over reused blocks")


def test_copies_with_nothing_to_copy_or_nowhere_to_go(device):
    """Zero bytes succeed without touching the addresses; a null address with bytes to move is an error, not a crash."""
    lib = ta.library()
    dvc = device.structure()
    assert lib.copy_from_host(C.byref(dvc), None, None, 0) == abi.SUCCESS
    assert lib.copy_device_to_host(C.byref(dvc), None, None, 0) == abi.SUCCESS
    assert lib.compare_from_host(C.byref(dvc), None, None, 0) == 1
    ptr = lib.allocate(C.byref(dvc), 0)          # an empty tensor still owns an address
    assert ptr
    buf = (C.c_char * 16)()
    assert lib.copy_from_host(C.byref(dvc), None, ptr, 16) == abi.ERROR
    assert lib.copy_device_to_host(C.byref(dvc), ptr, None, 16) == abi.ERROR
    assert lib.compare_from_host(C.byref(dvc), None, ptr, 16) == -1
    assert lib.copy_from_host(C.byref(dvc), buf, ptr, 16) == abi.SUCCESS
    lib.deallocate(C.byref(dvc), ptr)
    assert lib.deallocate(C.byref(dvc), None) is None
    assert lib.allocate(None, 64) is None
    empty = ta.Tensor(ta.float32, (0, 4)).initialize(device)
    assert empty.numpy().shape == (0, 4) and empty.to(ta.Host()).numpy().shape == (0, 4)
