"""Loader of the device library ``csrc/libtannic_hip.so`` (C ABI of ``include/tannic_hip.h``).

There is no CPU fallback behind this module: if the library is missing or does
not load, every use raises.
"""
import ctypes as C
import os

from . import abi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "csrc", "libtannic_hip.so")


class BackendError(RuntimeError):
    pass


class DeviceLibrary:
    """The ``tannic_hip_*`` symbols with their signatures attached."""

    def __init__(self, path=LIBRARY_PATH):
        if not os.path.exists(path):
            raise BackendError(
                f"{path} is missing: build it with `python -m tannic_amd.build` "
                "(hipcc --offload-arch=gfx950); tannic_amd has no CPU fallback"
            )
        self.path = path
        self.cdll = C.CDLL(path)
        self.kernels = {}
        for name, (res, args) in abi.kernel_signatures(with_stream=True).items():
            fn = getattr(self.cdll, "tannic_hip_" + name)
            fn.restype, fn.argtypes = res, args
            self.kernels[name] = fn
        for name, (res, args) in abi.runtime_signatures().items():
            fn = getattr(self.cdll, "tannic_hip_" + name)
            fn.restype, fn.argtypes = res, args
            setattr(self, name, fn)

    def error_message(self):
        msg = self.last_error()
        return msg.decode() if msg else ""


_library = None


def library():
    global _library
    if _library is None:
        _library = DeviceLibrary()
    return _library


def exported_symbols():
    """Every symbol ``include/tannic_hip.h`` declares, as the library must export it."""
    names = list(abi.kernel_signatures(True)) + list(abi.runtime_signatures())
    return ["tannic_hip_" + n for n in names]
