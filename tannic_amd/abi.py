"""ctypes mirror of ``include/tannic_hip.h``.

The structures restate the reference's runtime structs field for field
(``include/tannic/runtime/tensor.h:45-73``, ``resources.h:35-60``,
``streams.h:32-34``); the layout is asserted at import time against the sizes
and offsets the reference headers give on x86-64.
"""
import ctypes as C

DIMENSIONS = 8

# enum type (include/tannic/runtime/types.h:29-44)
ANY, BOOLEAN, INT8, INT16, INT32, INT64, FLOAT16, BFLOAT16, FLOAT32, FLOAT64, COMPLEX64, COMPLEX128, UNKNOWN, TYPES = range(14)
# enum status (include/tannic/runtime/status.h:26-32)
SUCCESS, ERROR, UNSUPPORTED_DTYPE, NULL_ALLOCATOR, INCOMPATIBLE_DEVICES = range(5)
STATUS_NAMES = ["SUCCESS", "ERROR", "UNSUPPORTED_DTYPE", "NULL_ALLOCATOR", "INCOMPATIBLE_DEVICES"]
# enum layout (include/tannic/runtime/tensor.h:39-43)
SINGLETON, CONTIGUOUS, STRIDED = range(3)
# enum environment / host (include/tannic/runtime/resources.h:35-43)
HOST, DEVICE = 0, 1
PAGEABLE, PINNED = 1, 2


class host_t(C.Structure):
    _fields_ = [("traits", C.c_int)]


class device_t(C.Structure):
    _fields_ = [("id", C.c_int)]


class _resource(C.Union):
    _fields_ = [("host", host_t), ("device", device_t)]


class environment_t(C.Structure):
    _fields_ = [("kind", C.c_int), ("resource", _resource)]


class scalar_t(C.Structure):
    _fields_ = [("address", C.c_void_p), ("dtype", C.c_int)]


class shape_t(C.Union):
    _fields_ = [("address", C.c_void_p), ("sizes", C.c_size_t * DIMENSIONS)]


class strides_t(C.Union):
    _fields_ = [("address", C.c_void_p), ("sizes", C.c_int64 * DIMENSIONS)]


class tensor_t(C.Structure):
    _fields_ = [
        ("address", C.c_void_p),
        ("rank", C.c_uint8),
        ("shape", shape_t),
        ("strides", strides_t),
        ("dtype", C.c_int),
        ("environment", environment_t),
        ("size", C.c_size_t),
        ("layout", C.c_int),
    ]


class stream_t(C.Structure):
    _fields_ = [("address", C.c_size_t)]


def _check_layout():
    assert C.sizeof(tensor_t) == 176
    want = {"address": 0, "rank": 8, "shape": 16, "strides": 80, "dtype": 144, "environment": 148, "size": 160, "layout": 168}
    for name, off in want.items():
        assert getattr(tensor_t, name).offset == off, name
    assert C.sizeof(shape_t) == 64 and C.sizeof(strides_t) == 64
    assert C.sizeof(scalar_t) == 16 and scalar_t.dtype.offset == 8
    assert C.sizeof(environment_t) == 8 and environment_t.resource.offset == 4
    assert C.sizeof(stream_t) == 8 and C.sizeof(device_t) == 4 and C.sizeof(host_t) == 4


_check_layout()

TP = C.POINTER(tensor_t)
SP = C.POINTER(scalar_t)
DP = C.POINTER(device_t)
SIZE2 = C.c_size_t * 2

UNARY_OPS = ["neg", "repack", "log", "exp", "sqrt", "abs", "sin", "cos", "tan", "sinh", "cosh", "tanh"]
BINARY_OPS = ["add", "sub", "mul", "pow"]
COMPARE_OPS = ["eq", "ne", "gt", "ge", "lt", "le"]
COMPLEX_OPS = ["view_as_cartesian", "view_as_polar"]
REDUCE_OPS = ["argsum", "argmean", "argmax", "argmin", "max", "min"]


def kernel_signatures(with_stream):
    """name -> (restype, argtypes) of every compute entry point.

    With ``with_stream`` the device library's signatures (``tannic_hip_*``);
    without, the stream-less form the CPU twins of the reference use
    (``src/cpu/*.hpp``).
    """
    s = [stream_t] if with_stream else []
    sig = {}
    for n in UNARY_OPS:
        sig[n] = (C.c_int, [TP, TP] + s)
    sig["rsqrt"] = (C.c_int, [TP, TP] + s + [C.c_float])
    for n in BINARY_OPS + COMPARE_OPS + COMPLEX_OPS + ["gemm"] + (["gemm_noalloc"] if with_stream else []):
        sig[n] = (C.c_int, [TP, TP, TP] + s)
    sig["scale"] = (C.c_int, [TP, SP, TP] + s)
    for n in REDUCE_OPS:
        sig[n] = (C.c_int, [TP, TP] + s + [C.c_uint8])
    sig["cpy"] = (C.c_int, [TP, TP] + s)
    sig["repeat"] = (C.c_int, [TP, TP] + s + [C.c_int, C.c_int])
    sig["concat"] = (C.c_int, [TP, TP, TP] + s + [C.c_int])
    sig["outer"] = (C.c_int, [TP, TP, TP] + s)
    sig["triu"] = (C.c_int, [TP, TP] + s + [C.c_int])
    sig["tril"] = (C.c_int, [TP, TP] + s + [C.c_int])
    sig["allclose"] = (C.c_int, [TP, TP] + s + [C.c_double, C.c_double])
    sig["conv1d"] = (C.c_int, [TP, TP, TP] + s + [C.c_size_t, C.c_size_t])
    sig["conv2d"] = (C.c_int, [TP, TP, TP] + s + [SIZE2, SIZE2])
    sig["conv2d_biased"] = (C.c_int, [TP, TP, TP, TP] + s + [SIZE2, SIZE2])
    # operators without a twin in the reference
    sig["div"] = (C.c_int, [TP, TP, TP] + s)
    sig["swiglu"] = (C.c_int, [TP, TP, TP] + s)
    sig["cast"] = (C.c_int, [TP, TP] + s)
    sig["rms_norm"] = (C.c_int, [TP, TP, TP] + s + [C.c_float])
    sig["softmax"] = (C.c_int, [TP, TP, TP] + s + [C.c_float])   # the second operand (mask) may be NULL
    sig["rope"] = (C.c_int, [TP, TP, TP, TP] + s)
    return sig


def runtime_signatures():
    """name -> (restype, argtypes) of the memory / stream / event entry points."""
    return {
        "last_error": (C.c_char_p, []),
        "arch": (C.c_char_p, []),
        "get_device_count": (C.c_int, []),
        "set_device": (C.c_int, [C.c_int]),
        "allocate": (C.c_void_p, [DP, C.c_size_t]),
        "deallocate": (C.c_void_p, [DP, C.c_void_p]),
        "copy_from_host": (C.c_int, [DP, C.c_void_p, C.c_void_p, C.c_size_t]),
        "copy_device_to_host": (C.c_int, [DP, C.c_void_p, C.c_void_p, C.c_size_t]),
        "compare_from_host": (C.c_int, [DP, C.c_void_p, C.c_void_p, C.c_size_t]),
        "copy": (C.c_int, [TP, TP, C.c_size_t, stream_t]),
        "pop_stream": (stream_t, [DP]),
        "put_stream": (None, [DP, stream_t]),
        "stream_synchronize": (C.c_int, [stream_t]),
        "device_synchronize": (C.c_int, []),
        "graph_begin": (C.c_void_p, [DP]),
        "graph_end": (C.c_int, [C.c_void_p]),
        "graph_launch": (C.c_int, [C.c_void_p]),
        "graph_destroy": (None, [C.c_void_p]),
        "graph_stream": (stream_t, [C.c_void_p]),
        "counters": (None, [C.POINTER(C.c_uint64)]),
        "event_create": (C.c_void_p, []),
        "event_destroy": (None, [C.c_void_p]),
        "event_record": (C.c_int, [C.c_void_p, stream_t]),
        "event_elapsed_ms": (C.c_float, [C.c_void_p, C.c_void_p]),
        "probe_mfma": (C.c_int, [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, stream_t]),
    }
