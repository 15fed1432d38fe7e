"""Operator interface of the reference, dispatching to the device backend.

Each function applies the front end's own dtype/shape rule to size the
destination, allocates it where the operands live, pops a stream, makes ONE
backend call and puts the stream back, raising on any status but SUCCESS —
the contract of ``Callback::operator()`` (``include/tannic/callback.hpp:46-178``).

Device operands go to ``libtannic_hip.so``.  Host operands have no kernels in
this package: they raise unless a host function table was registered with
``set_host_functions`` (the test-suite registers its CPU checker there, the way
the reference pairs ``cpu::f`` with ``cuda::f``).
"""
import builtins
import ctypes as C
import struct

import numpy as np

from . import abi, types
from .backend import BackendError, library
from .tensor import Device, Host, Tensor

_host_functions = None


def set_host_functions(table):
    """``table[name](*descriptors_and_args)`` -> status, stream-less signatures; None unsets."""
    global _host_functions
    _host_functions = table


class TannicError(RuntimeError):
    pass


def _resolve(*tensors):
    """``resolve_two_environment`` / ``resolve_three_environment`` (``src/bindings.cpp:118-188``)."""
    if len(tensors) == 2:
        first, second = tensors[0].buffer, tensors[1].buffer
        if first is not None and second is not None and first.environment is second.environment:
            return first.environment
    envs = [t.environment for t in tensors]
    devices = [e for e in envs if isinstance(e, Device)]
    if not devices:
        return Host()
    if len(devices) != len(envs) or any(d.id != devices[0].id for d in devices):
        raise TannicError("Environment issue!")  # INCOMPATIBLE_DEVICES
    return devices[0]


def _call(name, env, sources, dst, extra=(), scalar=None):
    """One backend call in the order the ABI expects: sources, [scalar], dst, [stream], extra."""
    args = [s.reference() for s in sources]
    if scalar is not None:
        args.append(C.byref(scalar))
    args.append(dst.reference())
    if env.kind == abi.DEVICE:
        lib = library()
        status = lib.kernels[name](*args, env.stream(), *extra)
        if status == abi.SUCCESS:
            return dst
        detail = lib.error_message() if status == abi.ERROR else ""
    else:
        if _host_functions is None:
            raise BackendError(f"{name}: operands are on the host and tannic_amd holds device kernels only")
        status = _host_functions[name](*args, *extra)
        detail = ""
    if status != abi.SUCCESS:
        # callback.hpp:67-69 reports every failure with this message
        raise TannicError(f"Unsupported dtype ({name}: {abi.STATUS_NAMES[status]}{' ' + detail if detail else ''})")
    return dst


def _new(dtype, shape, env):
    return Tensor.fresh(dtype, shape, env)


# ---- dtype / shape rules ------------------------------------------------
def promote(first, second):
    """``operation::promote``: the larger enum wins (``include/tannic/operations.hpp:133-135``)."""
    return first if first.code > second.code else second


def broadcast(first, second):
    """``operation::broadcast`` (``include/tannic/operations.hpp:137-152``)."""
    if first == second:
        return tuple(first)
    known = _BROADCASTS.get((first, second))
    if known is not None:
        return known
    rank = builtins.max(len(first), len(second))
    out = []
    for d in range(rank):
        a = 1 if d < rank - len(first) else first[d - (rank - len(first))]
        b = 1 if d < rank - len(second) else second[d - (rank - len(second))]
        if not (a == b or a == 1 or b == 1):
            raise TannicError("Shapes are not broadcast-compatible.")
        out.append(builtins.max(a, b))
    if len(_BROADCASTS) > 4096:
        _BROADCASTS.clear()
    known = _BROADCASTS[(tuple(first), tuple(second))] = tuple(out)
    return known


_BROADCASTS = {}    # (shape, shape) -> broadcast shape: the pairs of a program recur


# ---- unary functions (include/tannic/functions.hpp:52-57: contiguous target) ----
def _unary(name):
    def fn(x):
        return _call(name, x.environment, [x], _new(x.dtype, x.shape, x.environment))
    fn.__name__ = name
    return fn


neg = _unary("neg")
repack = _unary("repack")
log = _unary("log")
exp = _unary("exp")
sqrt = _unary("sqrt")
abs = _unary("abs")
sin = _unary("sin")
cos = _unary("cos")
tan = _unary("tan")
sinh = _unary("sinh")
cosh = _unary("cosh")
tanh = _unary("tanh")


def rsqrt(x, eps=0.0):
    """``1/sqrt(x + eps)`` (``include/tannic/functions.hpp``, ``src/cpu/ops-unary.cpp:141-149``)."""
    return _call("rsqrt", x.environment, [x], _new(x.dtype, x.shape, x.environment), extra=(C.c_float(eps),))


# ---- binary operations (include/tannic/tensor.hpp:358-363) ---------------
def _binary(name):
    def fn(a, b):
        env = _resolve(a, b)
        return _call(name, env, [a, b], _new(promote(a.dtype, b.dtype), broadcast(a.shape, b.shape), env))
    fn.__name__ = name
    return fn


add = _binary("add")
sub = _binary("sub")
mul = _binary("mul")
pow = _binary("pow")


def float_to_half_bits(value):
    """fp32 -> fp16 bits the way ``float16_t(float)`` does it (``src/types.cpp:6-40``):
    the dropped mantissa bits round half UP, not half to even."""
    bits = struct.unpack("<I", struct.pack("<f", value))[0]
    sign = (bits >> 16) & 0x8000
    raw_exponent = (bits >> 23) & 0xFF
    exponent = raw_exponent - 127 + 15
    mantissa = bits & 0x7FFFFF
    if raw_exponent == 0xFF:
        if mantissa == 0:
            return sign | 0x7C00
        half = sign | 0x7C00 | (mantissa >> 13)
        return half | 1 if (half & 0x3FF) == 0 else half
    if exponent <= 0:
        if exponent < -10:
            return sign
        mantissa |= 0x800000
        shift = 14 - exponent
        sub = mantissa >> shift
        if mantissa & (1 << (shift - 1)):
            sub += 1
        return sign | sub
    if exponent >= 31:
        return sign | 0x7C00
    half = sign | (exponent << 10) | (mantissa >> 13)
    return half + 1 if mantissa & 0x1000 else half


def scalar_bytes(value, dtype):
    """Host bytes of a scalar cast to the tensor's dtype (``include/tannic/scalars.hpp:36-52``):
    fp16 rounds half up, bf16 truncates (``src/types.cpp:74-78``)."""
    if dtype is types.float16:
        return struct.pack("<H", float_to_half_bits(float(value)) & 0xFFFF)
    if dtype is types.bfloat16:
        return struct.pack("<H", struct.unpack("<I", struct.pack("<f", float(value)))[0] >> 16)
    return np.array(value).astype(dtype.storage).tobytes()


def scale(x, value):
    """``k * X`` (``include/tannic/operations.hpp:295-313``)."""
    raw = C.create_string_buffer(scalar_bytes(value, x.dtype), 16)
    sc = abi.scalar_t(C.cast(raw, C.c_void_p), x.dtype.code)
    return _call("scale", x.environment, [x], _new(x.dtype, x.shape, x.environment), scalar=sc)


# ---- comparisons (include/tannic/comparisons.hpp:29-68) -------------------
def _compare(name):
    def fn(a, b):
        if a.shape != b.shape:
            raise TannicError("Shapes must match for comparison")
        env = _resolve(a, b)
        return _call(name, env, [a, b], _new(types.boolean, a.shape, env))
    fn.__name__ = name
    return fn


eq = _compare("eq")
ne = _compare("ne")
gt = _compare("gt")
ge = _compare("ge")
lt = _compare("lt")
le = _compare("le")


# ---- complex (include/tannic/complex.hpp:46-192) --------------------------
def _complex_of(dtype):
    if dtype is types.float32:
        return types.complex64
    if dtype is types.float64:
        return types.complex128
    raise TannicError("complex needs float32 or float64 components")


def cartesian(real, imaginary):
    env = _resolve(real, imaginary)
    dtype = _complex_of(promote(real.dtype, imaginary.dtype))
    return _call("view_as_cartesian", env, [real, imaginary], _new(dtype, broadcast(real.shape, imaginary.shape), env))


def polar(rho, theta):
    env = _resolve(rho, theta)
    dtype = _complex_of(promote(rho.dtype, theta.dtype))
    return _call("view_as_polar", env, [rho, theta], _new(dtype, broadcast(rho.shape, theta.shape), env))




def _retype(x, dtype):
    if dtype.is_complex:
        v = Tensor(dtype, x.shape[:-1], [s // 2 for s in x.strides[:-1]], x.offset)
    else:
        v = Tensor(dtype, tuple(x.shape) + (2,), [s * 2 for s in x.strides] + [1], x.offset)
    v.buffer = x.buffer
    return v


def complexify(x):
    """f32[..., 2] -> complex64[...] zero-copy (``complex.hpp:46-110``)."""
    if x.shape[-1] != 2 or x.strides[-1] != 1:
        raise TannicError("last dimension must hold (re, im) pairs")
    return _retype(x, _complex_of(x.dtype))


def realify(z):
    """complex64[...] -> f32[..., 2] zero-copy (``complex.hpp:112-192``)."""
    return _retype(z, types.float32 if z.dtype is types.complex64 else types.float64)


# ---- reductions (include/tannic/reductions.hpp:63-193) --------------------
def _reduced_shape(shape, axis, keepdim):
    return tuple(s if d != axis else 1 for d, s in enumerate(shape) if d != axis or keepdim)


def _reduce(name, x, axis, keepdim, dtype):
    if x.rank == 0:
        raise TannicError("Cannot reduce scalar tensors")
    axis = axis % x.rank
    dst = _new(dtype, _reduced_shape(x.shape, axis, keepdim), x.environment)
    return _call(name, x.environment, [x], dst, extra=(C.c_uint8(axis),))


def sum(x, axis=-1, keepdim=False):
    return _reduce("argsum", x, axis, keepdim, x.dtype)


def mean(x, axis=-1, keepdim=False):
    return _reduce("argmean", x, axis, keepdim, x.dtype)


def argmax(x, axis=-1, keepdim=False):
    return _reduce("argmax", x, axis, keepdim, types.int64)


def argmin(x, axis=-1, keepdim=False):
    # Argmin::reduce drops the axis whatever keepdim says (reductions.hpp:133-143)
    return _reduce("argmin", x, axis, False, types.int64)


def max(x, axis=-1, keepdim=False):
    """Largest number along ``axis`` (+0 above -0, NaNs skipped; the first element where nothing exceeds -inf);
    the reference has no such reduction."""
    return _reduce("max", x, axis, keepdim, x.dtype)


def min(x, axis=-1, keepdim=False):
    """Smallest number along ``axis`` (-0 below +0, NaNs skipped; the first element where nothing is below +inf);
    the reference has no such reduction."""
    return _reduce("min", x, axis, keepdim, x.dtype)


# ---- matmul (include/tannic/transformations.hpp:87-202) -------------------
def _composition_dtype(a, b):
    I8, I16, I32, I64 = types.int8, types.int16, types.int32, types.int64
    F16, BF16, F32, F64 = types.float16, types.bfloat16, types.float32, types.float64
    if a.is_integral and b.is_integral:
        if I64 in (a, b) or (a is I32 and b is I32):
            return I64
        return I32
    for half in (F16, BF16):
        if half in (a, b):
            other = b if a is half else a
            if other is half:
                return half
            if other in (I8, I16):
                return half
            if other is I32 or other is F32:
                return F32
            if other is I64 or other is F64:
                return F64
            if other in (F16, BF16):
                return F16  # bf16 x f16 -> f16 in the table; no kernel exists for it
    if a.is_floating and b.is_floating:
        return F64 if F64 in (a, b) else F32
    if {a, b} <= {I32, F32, F64}:
        return F64 if F64 in (a, b) else F32
    raise TannicError("Unsuported dtypes")


def matmul(a, b):
    """``matmul(A, B)``: batch dims broadcast, transposed views reach the kernel as strides."""
    if a.rank < 2 or b.rank < 2:
        raise TannicError("Inputs must have rank >= 2")
    if a.shape[-1] != b.shape[-2]:
        raise TannicError("Inner dimensions must match for matmul")
    shape = broadcast(a.shape[:-2], b.shape[:-2]) + (a.shape[-2], b.shape[-1])
    env = _resolve(a, b)
    return _call("gemm", env, [a, b], _new(_composition_dtype(a.dtype, b.dtype), shape, env))


# ---- convolution (include/tannic/convolutions.hpp:71-120) -----------------
def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def convolve2d(signal, kernel, bias=None, stride=1, padding=0):
    stride, padding = _pair(stride), _pair(padding)
    if signal.dtype is not kernel.dtype or (bias is not None and bias.dtype is not signal.dtype):
        raise TannicError("Dtypes must match in convolutions.")
    if signal.rank != 4 or kernel.rank != 4:
        raise TannicError("Only rank 4 tensors supported.")
    n, c_in, h, w = signal.shape
    c_out, k_in, kh, kw = kernel.shape
    if c_in != k_in:
        raise TannicError("Input channels must match kernel channels.")
    if bias is not None and (bias.rank != 1 or bias.shape[0] != c_out):
        raise TannicError("Bias shape must be [C_out].")
    shape = (n, c_out, (h + 2 * padding[0] - kh) // stride[0] + 1, (w + 2 * padding[1] - kw) // stride[1] + 1)
    operands = [signal, kernel] + ([bias] if bias is not None else [])
    env = _resolve(*operands)
    extra = (abi.SIZE2(*padding), abi.SIZE2(*stride))
    return _call("conv2d_biased" if bias is not None else "conv2d", env, operands, _new(signal.dtype, shape, env), extra=extra)


def convolve1d(signal, kernel, stride=1, padding=0):
    """``convolve1D(signal, kernel, stride, padding)`` (``include/tannic/convolutions.hpp:38-68, 135-145``)."""
    if stride == 0:
        raise TannicError("Stride must be non-zero for Conv1D.")
    if signal.dtype is not kernel.dtype:
        raise TannicError("Dtypes must match in convolutions.")
    if signal.rank != 3 or kernel.rank != 3:
        raise TannicError("Only rank 3 tensors supported for Conv1D.")
    n, c_in, length = signal.shape
    c_out, k_in, k_len = kernel.shape
    if c_in != k_in:
        raise TannicError("Input channels must match kernel channels.")
    shape = (n, c_out, (length + 2 * padding - k_len) // stride + 1)
    env = _resolve(signal, kernel)
    return _call("conv1d", env, [signal, kernel], _new(signal.dtype, shape, env), extra=(C.c_size_t(padding), C.c_size_t(stride)))


# ---- copies and checks ---------------------------------------------------
def repeat(x, repeats, axis=0):
    """``repeat(source, repeats, axis)``: every index along ``axis`` ``repeats`` times in place
    (``include/tannic/transformations.hpp:221-240, 325-329``; kernel ``src/cpu/reps.cpp:18-54``)."""
    axis = axis + x.rank if axis < 0 else axis
    if not 0 <= axis < x.rank:
        raise TannicError("repeat: axis out of range")
    shape = list(x.shape)
    shape[axis] *= repeats
    env = _resolve(x)
    dst = _new(x.dtype, shape, env)
    _call("repeat", env, [x], dst, (C.c_int(axis), C.c_int(repeats)))
    return dst


def concatenate(first, second, axis=0):
    """``concatenate(first, second, axis)`` (``include/tannic/transformations.hpp:241-262, 344-352``)."""
    if axis < 0:
        raise TannicError("Negative index not supported in concat")
    if first.dtype is not second.dtype:
        raise TannicError("Cannot concatenate tensors of different dtypes")
    if first.rank != second.rank or axis >= first.rank:
        raise TannicError("Ranks must match for concatenation")
    shape = list(first.shape)
    for d in range(first.rank):
        if d == axis:
            shape[d] = first.shape[d] + second.shape[d]
        elif first.shape[d] != second.shape[d]:
            raise TannicError("All dimensions except concat axis must match")
    env = _resolve(first, second)
    dst = _new(first.dtype, shape, env)
    _call("concat", env, [first, second], dst, (C.c_int(axis),))
    return dst


def outer(first, second):
    """``outer(first, second)``: vectors only; the destination takes the dtype with the larger code
    (``include/tannic/transformations.hpp:208-221, 306-312``)."""
    if first.rank != 1 or second.rank != 1:
        raise TannicError("Outer product of tensors with rank more than 1 not supported")
    dtype = first.dtype if first.dtype.code > second.dtype.code else second.dtype
    env = _resolve(first, second)
    dst = _new(dtype, (first.shape[0], second.shape[0]), env)
    return _call("outer", env, [first, second], dst)


def _triangular(name, x, k):
    env = _resolve(x)
    dst = _new(x.dtype, x.shape, env)
    _call(name, env, [x], dst, (C.c_int(k),))
    return dst


def triu(x, k=0):
    """``triangular(x, Position::Upper, k)`` (``include/tannic/filter.hpp:63-76``, ``src/filter.cpp:20-37``)."""
    return _triangular("triu", x, k)


def tril(x, k=0):
    """``triangular(x, Position::Lower, k)`` (``include/tannic/filter.hpp:63-76``, ``src/filter.cpp:20-37``)."""
    return _triangular("tril", x, k)


def copy_into(dst, src):
    """``slice = expr``: strided copy into an existing view (``include/tannic/tensor.hpp:447-456``)."""
    return _call("cpy", _resolve(dst, src), [src], dst)


def allclose(a, b, rtol=1e-5, atol=1e-8):
    """``allclose`` (``src/cpu/val.cpp:73-83``, ``src/cuda/val.cu:82-89``): waits for the device."""
    env = _resolve(a, b)
    da, db = a.descriptor(), b.descriptor()
    if isinstance(env, Device):
        lib = library()
        dvc = env.structure()
        stream = lib.pop_stream(C.byref(dvc))
        r = lib.kernels["allclose"](C.byref(da), C.byref(db), stream, rtol, atol)
        lib.put_stream(C.byref(dvc), stream)
    else:
        if _host_functions is None:
            raise BackendError("allclose: operands are on the host and tannic_amd holds device kernels only")
        r = _host_functions["allclose"](C.byref(da), C.byref(db), rtol, atol)
    if r < 0:
        raise TannicError("Unsupported dtype")
    return bool(r)


# ---- operators without a twin in the reference ---------------------------------------
# A Tannic program has no division, cast, softmax or normalisation (``include/tannic/functions.hpp``,
# ``include/tannic/operations.hpp``) and spells them as chains; these are the one-pass forms the device library adds.
def div(a, b):
    """``a / b`` with the broadcasting and promotion of the other binary operations; floating types only."""
    env = _resolve(a, b)
    return _call("div", env, [a, b], _new(promote(a.dtype, b.dtype), broadcast(a.shape, b.shape), env))


def cast(x, dtype):
    """``x`` in ``dtype`` (real types), contiguous."""
    return _call("cast", x.environment, [x], _new(dtype, x.shape, x.environment))


def swiglu(gate, up):
    """``gate / (1 + exp(-gate)) * up``."""
    env = _resolve(gate, up)
    return _call("swiglu", env, [gate, up], _new(gate.dtype, broadcast(gate.shape, up.shape), env))


def rms_norm(x, gain, eps=1e-5):
    """``x / sqrt(mean(x**2, -1) + eps) * gain`` over the last axis of a contiguous ``x``."""
    env = _resolve(x, gain)
    return _call("rms_norm", env, [x, gain], _new(x.dtype, x.shape, env), extra=(C.c_float(eps),))


def softmax(x, mask=None, scale=1.0):
    """Softmax over the last axis of ``x * scale + mask``; ``mask`` is ``None`` or ``[x.shape[-2], x.shape[-1]]``."""
    env = _resolve(x) if mask is None else _resolve(x, mask)
    if not isinstance(env, Device):
        raise BackendError("softmax: operands are on the host and tannic_amd holds device kernels only")
    dst = _new(x.dtype, x.shape, env)
    dx, dd = x.descriptor(), dst.descriptor()
    dm = None if mask is None else mask.descriptor()
    lib = library()
    dvc = env.structure()
    stream = lib.pop_stream(C.byref(dvc))
    status = lib.kernels["softmax"](C.byref(dx), None if dm is None else C.byref(dm), C.byref(dd), stream, C.c_float(scale))
    lib.put_stream(C.byref(dvc), stream)
    if status != abi.SUCCESS:
        detail = lib.error_message() if status == abi.ERROR else ""
        raise TannicError(f"Unsupported dtype (softmax: {abi.STATUS_NAMES[status]}{' ' + detail if detail else ''})")
    return dst


def rope(x, cos, sin):
    """Rotary embedding of ``x [.., n, d]`` by ``cos, sin [n, d/2]`` on the pairs ``(2i, 2i+1)``; contiguous result."""
    env = _resolve(x, cos, sin)
    return _call("rope", env, [x, cos, sin], _new(x.dtype, x.shape, env))
