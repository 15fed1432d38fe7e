"""Loader of the CPU checker (oracle/liboracle.so) and, where it was built, of the reference's own CPU backend
(oracle/_ref/libtannic_ref.so).  Test infrastructure: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg only; nothing in the product path loads these libraries."""
import ctypes as C
import os
import subprocess

from tannic_amd import abi

ORACLE_DIR = os.path.dirname(os.path.abspath(__file__))


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
