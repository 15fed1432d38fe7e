"""Shared test plumbing: the CPU checker's loader, seeded inputs, comparisons.

Only the test-suite, the smoke check and the benchmark's cpu_baseline leg use
the libraries under oracle/.
"""
import ctypes as C
import os
import subprocess

import numpy as np

import tannic_amd as ta
from tannic_amd import abi, types

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")


class HostLibrary:
    """A library of stream-less entry points with a common prefix."""

    def __init__(self, path, prefix):
        self.path = path
        self.cdll = C.CDLL(path)
        self.functions = {}
        for name, (res, args) in abi.kernel_signatures(with_stream=False).items():
            try:
                fn = getattr(self.cdll, prefix + name)
            except AttributeError:
                continue
            fn.restype, fn.argtypes = res, args
            self.functions[name] = fn

    def set_accumulate(self, wide):
        self.cdll.oracle_set_accumulate(1 if wide else 0)


_oracle = None
_reference = False


def oracle_library():
    global _oracle
    if _oracle is None:
        path = os.path.join(ORACLE_DIR, "liboracle.so")
        if not os.path.exists(path):
            subprocess.run(["make", "-C", ORACLE_DIR, "liboracle.so"], check=True, capture_output=True)
        _oracle = HostLibrary(path, "oracle_")
    return _oracle


def reference_library():
    global _reference
    if _reference is False:
        path = os.path.join(ORACLE_DIR, "_ref", "libtannic_ref.so")
        _reference = HostLibrary(path, "ref_") if os.path.exists(path) else None
    return _reference


class use_functions:
    """Temporarily routes host operands of ``tannic_amd.ops`` to ``library``."""

    def __init__(self, library):
        self.library = library

    def __enter__(self):
        self.previous = ta.ops._host_functions
        ta.ops.set_host_functions(self.library.functions)

    def __exit__(self, *exc):
        ta.ops.set_host_functions(self.previous)


# ---- seeded inputs: counter-based, identical on every host -----------------
def _splitmix64(x):
    x = (x + np.uint64(0x9E3779B97F4A7C15))
    z = x
    z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def random_bits(seed, tensor_id, n):
    with np.errstate(over="ignore"):
        base = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(tensor_id))
        return _splitmix64(base + np.arange(n, dtype=np.uint64))


def uniform(seed, tensor_id, shape, low=-1.0, high=1.0):
    n = int(np.prod(shape, dtype=np.int64))
    u = (random_bits(seed, tensor_id, n) >> np.uint64(40)).astype(np.float64) * 2.0 ** -24
    return (low + (high - low) * u).astype(np.float32).reshape(shape)


def normal(seed, tensor_id, shape, sigma=1.0):
    n = int(np.prod(shape, dtype=np.int64))
    bits = random_bits(seed, tensor_id, 2 * n)
    u1 = ((bits[:n] >> np.uint64(11)).astype(np.float64) + 1.0) * 2.0 ** -53
    u2 = (bits[n:] >> np.uint64(11)).astype(np.float64) * 2.0 ** -53
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (sigma * z).astype(np.float32).reshape(shape)


def integers(seed, tensor_id, shape, low=-4, high=4):
    return np.floor(uniform(seed, tensor_id, shape, low, high)).astype(np.int64)


def values_for(dtype, seed, tensor_id, shape, low=-4.0, high=4.0):
    """Seeded values representable in ``dtype`` (as a numeric numpy array)."""
    if dtype.is_integral:
        return integers(seed, tensor_id, shape, int(low), int(high)).astype(dtype.storage)
    if dtype.is_complex:
        re = uniform(seed, tensor_id, shape, low, high)
        im = uniform(seed, tensor_id + 7919, shape, low, high)
        return (re + 1j * im).astype(dtype.storage)
    x = uniform(seed, tensor_id, shape, low, high)
    if dtype is types.float16:
        return x.astype(np.float16)
    if dtype is types.bfloat16:
        return types.bfloat16_bits_to_float32(types.float32_to_bfloat16_bits(x))
    return x.astype(dtype.storage)


def host_tensor(values, dtype):
    return ta.tensor(values, dtype, ta.Host())


def both(values, dtype, device):
    """The same data as a host tensor and as a device tensor."""
    h = host_tensor(values, dtype)
    return h, h.to(device)


def apply_view(t, spec):
    """spec: list of (method, args) applied in order, e.g. [("transpose", (-1, -2))]."""
    for method, args in spec:
        if method == "index":
            t = t[args]
        else:
            t = getattr(t, method)(*args)
    return t


def ulp_distance_f16(a, b):
    ia = a.view(np.int16).astype(np.int32)
    ib = b.view(np.int16).astype(np.int32)
    ia = np.where(ia < 0, -32768 - ia, ia)
    ib = np.where(ib < 0, -32768 - ib, ib)
    return np.abs(ia - ib)


def assert_bit_exact(got, want, what=""):
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert got.dtype == want.dtype, (what, got.dtype, want.dtype)
    if got.dtype.kind in "fc":
        same = (got.view(np.uint8) == want.view(np.uint8)).all() if got.size else True
        if not same:
            bad = np.argwhere(~((got == want) | (np.isnan(got) & np.isnan(want))))
            assert bad.size == 0, f"{what}: {bad.shape[0]} elements differ, first at {bad[0]}: {got[tuple(bad[0])]} vs {want[tuple(bad[0])]}"
    else:
        bad = np.argwhere(got != want)
        assert bad.size == 0, f"{what}: {bad.shape[0]} elements differ, first at {bad[0]}: {got[tuple(bad[0])]} vs {want[tuple(bad[0])]}"


def assert_close(got, want, rtol, atol, what=""):
    """|got - want| <= atol + rtol*|want| (the reference's allclose form, src/cpu/val.cpp:34-36)."""
    got = np.asarray(got).astype(np.complex128 if np.iscomplexobj(got) else np.float64)
    want = np.asarray(want).astype(got.dtype)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    both_nan = np.isnan(got) & np.isnan(want)
    both_inf = np.isinf(got) & np.isinf(want) & (np.sign(got.real) == np.sign(want.real))
    err = np.abs(got - want)
    bad = ~((err <= atol + rtol * np.abs(want)) | both_nan | both_inf)
    if bad.any():
        i = tuple(np.argwhere(bad)[0])
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} elements out of tolerance "
                             f"(rtol={rtol}, atol={atol}); first at {i}: got {got[i]} want {want[i]}")
