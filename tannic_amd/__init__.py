"""tannic_amd — MI355X (gfx950) device backend for the Tannic tensor library.

``csrc/`` holds the hand-written HIP kernels and the C ABI (``include/tannic_hip.h``);
the Python modules mirror the part of the reference's front end that sits
directly above that ABI: descriptors, views, dtype/shape rules and the
one-call-per-operator dispatch.
"""
from . import abi, types
from .types import (boolean, int8, int16, int32, int64, float16, bfloat16, float32, float64,
                    complex64, complex128)
from .backend import BackendError, library, LIBRARY_PATH
from .tensor import Tensor, Host, Device, tensor
from . import ops
from .ops import TannicError
from .graph import Graph
