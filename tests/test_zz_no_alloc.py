"""tannic_hip_gemm_noalloc: the matrix product for callers that must not allocate.  Its results equal tannic_hip_gemm's bit
for bit, on two calls in a row that both take the kernels sharing K between workgroups (the ones that use scratch
memory), the second smaller than the first so that it finds the first call's partial sums in the shared array."""
import ctypes as C

import numpy as np
import pytest

import support
import tannic_amd as ta
from tannic_amd import abi

pytestmark = pytest.mark.gpu
SCRATCH_BYTES = 8 << 20   # TANNIC_GEMM_NOALLOC_SCRATCH_BYTES


def counters():
    """(kernel-scratch acquisitions, tensor allocations and releases, workgroups sharing K in the last product that shared it)"""
    out = (C.c_uint64 * 3)()
    ta.library().counters(out)
    return tuple(out)


def product(name, device, a, b, shape, dtype):
    """Returns (status, message, destination, what the counters moved by during the call itself)."""
    lib = ta.library()
    stream = device.stream()      # the stream every operator of this harness runs on; nothing is popped and held
    dst = ta.Tensor(dtype, shape).initialize(device)
    da, db, dd = a.descriptor(), b.descriptor(), dst.descriptor()
    before = counters()
    status = lib.kernels[name](C.byref(da), C.byref(db), C.byref(dd), stream)
    after = counters()
    message = lib.error_message()
    return status, message, dst, (after[0] - before[0], after[1] - before[1], after[2])


# (M, N, K, layout): few output tiles and a long K, so that several workgroups share a tile's K (and more than the 8192
# results up to which a product that is not K-contiguous runs the kernel for few results, which needs no scratch)
CALLS = [(128, 4096, 4096, "nt"), (72, 192, 2048, "nn")]


@pytest.mark.parametrize("dtype", [ta.float16, ta.bfloat16, ta.float32], ids=str)
def test_two_calls_in_a_row_equal_the_allocating_entry_point(device, dtype):
    for call, (m, n, k, layout) in enumerate(CALLS):
        x = support.values_for(dtype, 21, 2 * call, (m, k), -1, 1)
        w = support.values_for(dtype, 21, 2 * call + 1, (n, k) if layout == "nt" else (k, n), -1, 1)
        dx, dw = ta.tensor(x, dtype, device), ta.tensor(w, dtype, device)
        if layout == "nt":
            dw = dw.transpose()
        status, message, want, moved = product("gemm", device, dx, dw, (m, n), dtype)
        assert status == abi.SUCCESS, message
        # the shapes of CALLS take the kernels that share K (the ones that need scratch memory): the allocating entry
        # point asks the scratch cache for it ...
        assert moved[0] == 1 and moved[2] > 1, moved
        status, message, got, moved = product("gemm_noalloc", device, dx, dw, (m, n), dtype)
        assert status == abi.SUCCESS, message
        # ... and this one shares K as many ways without asking anybody for memory
        assert moved[0] == 0 and moved[1] == 0 and moved[2] > 1, moved
        support.assert_bit_exact(got.storage(), want.storage(), f"gemm_noalloc {dtype} call {call}: [{m},{k}] x [{k},{n}] {layout}")
        # and the product is the right one
        exact = x.astype(np.float64) @ (w.astype(np.float64).T if layout == "nt" else w.astype(np.float64))
        support.assert_close(got.numpy(), exact, 2.0 ** -7 if dtype is ta.bfloat16 else 2e-3, 1e-3 * k ** 0.5, f"gemm_noalloc {dtype} against float64")


def test_products_without_shared_k_need_no_scratch(device):
    x = support.values_for(ta.float16, 22, 0, (300, 128), -1, 1)
    w = support.values_for(ta.float16, 22, 1, (520, 128), -1, 1)
    dx, dw = ta.tensor(x, ta.float16, device), ta.tensor(w, ta.float16, device).transpose()
    _, _, want, _ = product("gemm", device, dx, dw, (300, 520), ta.float16)
    status, message, got, moved = product("gemm_noalloc", device, dx, dw, (300, 520), ta.float16)
    assert moved[0] == 0 and moved[1] == 0, moved
    assert status == abi.SUCCESS, message
    support.assert_bit_exact(got.storage(), want.storage(), "gemm_noalloc, whole K per workgroup")


def test_a_product_whose_partial_sums_do_not_fit_is_refused(device):
    """[128,16384] x [16384,8192]: 64 tiles of 128 x 128 with K shared at least four ways: 4 x 128 x 8192 fp32 partial sums are 16 MiB already."""
    dx = ta.Tensor(ta.float16, (128, 16384)).initialize(device)
    dw = ta.Tensor(ta.float16, (8192, 16384)).initialize(device).transpose()
    status, message, _, _ = product("gemm_noalloc", device, dx, dw, (128, 8192), ta.float16)
    assert status == abi.ERROR and "partial sums" in message and str(SCRATCH_BYTES) in message, (status, message)
    status, message, _, _ = product("gemm", device, dx, dw, (128, 8192), ta.float16)
    assert status == abi.SUCCESS, message
