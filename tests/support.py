"""Shared test plumbing: the CPU checker's loader, seeded inputs, comparisons.

Only the test-suite, the smoke check and the benchmark's cpu_baseline leg use
the libraries under oracle/.
"""
import ctypes as C
import os
import sys

import numpy as np

import tannic_amd as ta
from tannic_amd import abi, types

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
sys.path.insert(0, ORACLE_DIR)


from host_library import HostLibrary, oracle_library, reference_library  # noqa: E402,F401


class use_functions:
    """Temporarily routes host operands of ``tannic_amd.ops`` to ``library``."""

    def __init__(self, library):
        self.library = library

    def __enter__(self):
        self.previous = ta.ops._host_functions
        ta.ops.set_host_functions(self.library.functions)

    def __exit__(self, *exc):
        ta.ops.set_host_functions(self.previous)


# ---- seeded inputs (tannic_amd.synthetic) -----------------
from tannic_amd.synthetic import random_bits, uniform, normal, integers, values_for  # noqa: E402,F401


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
