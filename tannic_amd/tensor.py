"""Host-side mirror of the reference's ``Tensor``/``Buffer``/``Node`` for the device path.

A ``Tensor`` is dtype + shape + element strides + byte offset over a shared
``Buffer`` (``include/tannic/tensor.hpp:45-70``, ``src/buffer.cpp:11-43``).  Views
are zero-copy stride arithmetic (``include/tannic/views.hpp``).  ``descriptor()``
fills a ``tensor_t`` exactly the way ``Node::Node`` does (``src/graph.cpp:9-64``):
address = buffer + offset, strides in elements, size = element count,
layout SINGLETON / CONTIGUOUS / STRIDED.
"""
import ctypes as C
import math
import struct

import numpy as np

from . import abi, types
from .backend import BackendError, library


class Host:
    """Pageable host memory (``include/tannic/resources.hpp``, ``Host``)."""

    kind = abi.HOST

    def __eq__(self, other):
        return isinstance(other, Host)

    def __hash__(self):
        return 0

    def __repr__(self):
        return "Host()"


_STREAMS = {}      # device id -> its stream (see Device.stream)


class Device:
    """One GPU.  Mirrors ``Device::Device`` (``src/resources.cpp:44-49``): ids outside
    ``[0, getDeviceCount())`` raise ``IndexError`` (``std::out_of_range`` there)."""

    kind = abi.DEVICE

    def __init__(self, id=0):
        count = library().get_device_count()
        if id < 0 or id >= count:
            raise IndexError("Invalid device ID")
        self.id = id
        self._structure = abi.device_t(id)
        self.reference = C.byref(self._structure)    # what every backend call on this device passes

    def structure(self):
        return self._structure

    def stream(self):
        """The stream this device's backend calls run on.  The reference pops a stream from a per-device LIFO pool
        before every call and puts it back after (``src/bindings.cpp:22-42``, ``src/cuda/streams.cu:23-38``), which hands
        a host thread the same stream every time; this mirror asks the pool once per device and keeps the answer."""
        stream = _STREAMS.get(self.id)
        if stream is None:
            lib = library()
            stream = lib.pop_stream(self.reference)
            lib.put_stream(self.reference, stream)
            _STREAMS[self.id] = stream
        return stream

    def __eq__(self, other):
        return isinstance(other, Device) and other.id == self.id

    def __hash__(self):
        return 1 + self.id

    def __repr__(self):
        return f"Device({self.id})"


class Buffer:
    """Owns one allocation; device memory goes back through ``deallocate``
    (``src/buffer.cpp:37-43`` -> ``Device::deallocate`` -> ``cuda::deallocate``)."""

    def __init__(self, nbytes, environment):
        self.nbytes = nbytes
        self.environment = environment
        self.array, self.address = None, 0     # (what __del__ looks at, should the allocation raise)
        if environment.kind == abi.DEVICE:
            self.address = library().allocate(environment.reference, max(nbytes, 1))
            if not self.address:
                raise BackendError("device allocation failed: " + library().error_message())
            self.array = None
        else:
            self.array = np.zeros(max(nbytes, 1), dtype=np.uint8)
            self.address = self.array.ctypes.data

    def __del__(self):
        if self.array is None and self.address:
            try:
                library().deallocate(self.environment.reference, self.address)
            except Exception:
                pass
            self.address = None


# tensor_t: address, rank, shape[8], strides[8], dtype, environment (kind, device id or host traits), size, layout
_TENSOR_T = struct.Struct("<QB7x8Q8qiii4xQi4x")
_PAD = [(0,) * (abi.DIMENSIONS - r) for r in range(abi.DIMENSIONS + 1)]
assert _TENSOR_T.size == C.sizeof(abi.tensor_t)


_IMAGES = {}      # (shape, strides, dtype, environment) -> packed tensor_t without the address
_STRIDES = {}     # shape -> (contiguous strides, number of elements); shapes recur, the table stays small


def _shape_facts(shape):
    facts = _STRIDES.get(shape)
    if facts is None:
        strides, expected = [0] * len(shape), 1
        for i in range(len(shape) - 1, -1, -1):
            strides[i] = expected
            expected *= shape[i]
        if len(_STRIDES) > 4096:
            _STRIDES.clear()
        facts = _STRIDES[shape] = (tuple(strides), math.prod(shape))
    return facts


def contiguous_strides(shape):
    return _shape_facts(tuple(shape))[0]


class Tensor:
    def __init__(self, dtype, shape, strides=None, offset=0):
        shape = tuple(int(s) for s in shape)
        if len(shape) > abi.DIMENSIONS:
            raise ValueError("rank limited to 8")
        self.dtype = dtype
        self.shape = shape
        self.strides = contiguous_strides(shape) if strides is None else tuple(int(s) for s in strides)
        self.offset = int(offset)  # bytes
        self.buffer = None
        self.nelements = math.prod(shape)

    # ---- metadata -------------------------------------------------------
    @property
    def rank(self):
        return len(self.shape)

    @property
    def nbytes(self):
        return types.nbytesof(self.dtype, self.nelements)

    def is_initialized(self):
        return self.buffer is not None

    def is_contiguous(self):
        # include/tannic/tensor.hpp:60-69: every stride must equal the running product
        known = self.__dict__.get("_contiguous")
        if known is None:
            known = self._contiguous = self.strides == contiguous_strides(self.shape)
        return known

    @classmethod
    def fresh(cls, dtype, shape, environment):
        """A new contiguous tensor with its own buffer: what an operator allocates for its result."""
        t = cls.__new__(cls)
        t.dtype = dtype
        t.shape = shape = tuple(shape)
        t.strides, t.nelements = _shape_facts(shape)
        t.offset = 0
        t._contiguous = True
        t.buffer = Buffer(types.nbytesof(dtype, t.nelements), environment)
        return t

    def is_singleton(self):
        return self.nelements == 1

    @property
    def environment(self):
        if self.buffer is None:
            raise BackendError("tensor is not initialized")
        return self.buffer.environment

    @property
    def address(self):
        return self.buffer.address + self.offset

    # ---- storage --------------------------------------------------------
    def initialize(self, data=None, environment=None):
        """``Tensor::initialize(Environment)`` (``src/tensor.cpp:29-32``); with ``data``
        the values are stored row-major first (bulk upload, not per element)."""
        if environment is None and isinstance(data, (Host, Device)):
            data, environment = None, data
        environment = environment or Host()
        if self.strides != contiguous_strides(self.shape) and data is not None:
            raise ValueError("initialize with data needs a contiguous tensor")
        self.buffer = Buffer(self.nbytes + self.offset, environment)
        if data is not None:
            self.write(data)
        return self

    def write(self, values):
        """Stores ``values`` (row-major, numeric) into a contiguous tensor."""
        raw = types.to_storage(values, self.dtype)
        if self.dtype is not types.boolean:
            raw = np.ascontiguousarray(raw.reshape(self.shape))
        self.write_raw(raw)

    def write_raw(self, raw):
        """Stores ``raw`` (the tensor's bytes in storage form, row-major) into a contiguous tensor: one bulk copy."""
        raw = np.ascontiguousarray(raw)
        assert raw.nbytes == self.nbytes, (raw.nbytes, self.nbytes)
        if isinstance(self.environment, Device):
            dvc = self.environment.structure()
            rc = library().copy_from_host(C.byref(dvc), raw.ctypes.data, self.address, raw.nbytes)
            if rc != abi.SUCCESS:
                raise BackendError(library().error_message())
            # the upload is stream-ordered; the host array must outlive it
            library().device_synchronize()
        else:
            C.memmove(self.address, raw.ctypes.data, raw.nbytes)

    def raw(self):
        """The whole underlying buffer from this view's offset on, as host bytes."""
        n = self.buffer.nbytes - self.offset
        out = np.empty(n, dtype=np.uint8)
        if isinstance(self.environment, Device):
            dvc = self.environment.structure()
            rc = library().copy_device_to_host(C.byref(dvc), self.address, out.ctypes.data, n)
            if rc != abi.SUCCESS:
                raise BackendError(library().error_message())
        else:
            C.memmove(out.ctypes.data, self.address, n)
        return out

    def storage(self):
        """Logical contents in storage form (bf16 as uint16 bits, booleans as bool)."""
        raw = self.raw()
        if self.dtype is types.boolean:
            bits = np.unpackbits(raw, bitorder="little")[: self.nelements]
            return bits.astype(bool).reshape(self.shape)
        flat = raw[: (len(raw) // self.dtype.itemsize) * self.dtype.itemsize].view(self.dtype.storage)
        if self.nelements == 0:
            return np.empty(self.shape, dtype=self.dtype.storage)
        view = np.lib.stride_tricks.as_strided(
            flat, shape=self.shape, strides=tuple(s * self.dtype.itemsize for s in self.strides), writeable=False
        )
        return np.array(view)

    def numpy(self):
        """Logical contents as a numeric array (bf16 widened to float32)."""
        return types.to_numeric(self.storage(), self.dtype)

    def to(self, environment):
        """``Tensor::to`` (``src/tensor.cpp:84-140``) for H2D, D2H and D2D through ``copy``."""
        out = Tensor(self.dtype, self.shape, self.strides)
        out.buffer = Buffer(self.buffer.nbytes - self.offset, environment)
        dev = environment if isinstance(environment, Device) else self.environment
        if not isinstance(dev, Device):
            C.memmove(out.address, self.address, out.buffer.nbytes)
            return out
        lib = library()
        dvc = dev.structure()
        stream = lib.pop_stream(C.byref(dvc))
        src, dst = self.descriptor(), out.descriptor()
        rc = lib.copy(C.byref(src), C.byref(dst), out.buffer.nbytes, stream)
        lib.put_stream(C.byref(dvc), stream)
        if rc != abi.SUCCESS:
            raise BackendError(lib.error_message())
        return out

    # ---- the descriptor handed to the backend ---------------------------
    def descriptor(self):
        """The ``tensor_t`` of this view; built once (a view's shape, strides, offset and buffer never change)."""
        cached = self.__dict__.get("_descriptor")
        if cached is not None:
            return cached
        # One packed image of ``tensor_t`` per (shape, strides, dtype, environment), kept; a tensor's own descriptor is a copy
        # of it with the address filled in (offsets checked against the structure when ``abi`` is imported).
        env = self.buffer.environment
        key = (self.shape, self.strides, self.dtype.code, env.kind, env.id if env.kind == abi.DEVICE else -1)
        image = _IMAGES.get(key)
        if image is None:
            rank = len(self.shape)
            pad = _PAD[rank]
            layout = abi.SINGLETON if self.nelements == 1 else abi.CONTIGUOUS if self.is_contiguous() else abi.STRIDED
            resource = env.id if env.kind == abi.DEVICE else abi.PAGEABLE
            if len(_IMAGES) > 4096:
                _IMAGES.clear()
            image = _IMAGES[key] = _TENSOR_T.pack(0, rank, *self.shape, *pad, *self.strides, *pad, self.dtype.code, env.kind, resource, self.nelements, layout)
        t = abi.tensor_t.from_buffer_copy(image)
        t.address = self.buffer.address + self.offset
        self._descriptor = t
        self._reference = C.byref(t)
        return t

    def reference(self):
        """``byref(descriptor())``, kept with it: the argument a backend call takes."""
        r = self.__dict__.get("_reference")
        if r is None:
            self.descriptor()
            r = self._reference
        return r

    # ---- views (include/tannic/views.hpp) --------------------------------
    def _view(self, shape, strides, offset=None):
        v = Tensor.__new__(Tensor)
        v.dtype = self.dtype
        v.shape = shape = tuple(shape)
        v.strides = tuple(strides)
        v.offset = self.offset if offset is None else offset
        v.nelements = math.prod(shape)
        v.buffer = self.buffer
        return v

    def transpose(self, first=-1, second=-2):
        """Swaps two dims' sizes and strides (``views.hpp:126-161``)."""
        a, b = first % self.rank, second % self.rank
        shape, strides = list(self.shape), list(self.strides)
        shape[a], shape[b] = shape[b], shape[a]
        strides[a], strides[b] = strides[b], strides[a]
        return self._view(shape, strides)

    def permute(self, *dims):
        dims = [d % self.rank for d in dims]
        return self._view([self.shape[d] for d in dims], [self.strides[d] for d in dims])

    def expand(self, *sizes):
        """Broadcast view with stride 0 on expanded dims (``views.hpp:212-279``)."""
        rank = len(sizes)
        off = rank - self.rank
        shape, strides = [], []
        for d in range(rank):
            have = self.shape[d - off] if d >= off else 1
            want = have if sizes[d] == -1 else sizes[d]
            if have == want:
                shape.append(have)
                strides.append(self.strides[d - off] if d >= off else 0)
            elif have == 1:
                shape.append(want)
                strides.append(0)
            else:
                raise ValueError("expand: incompatible size")
        return self._view(shape, strides)

    def view(self, *shape):
        """Reinterprets a contiguous tensor's shape (``views.hpp:46-105``)."""
        if not self.is_contiguous():
            raise ValueError("view needs a contiguous tensor")
        shape = list(shape)
        if -1 in shape:
            known = math.prod(s for s in shape if s != -1)
            shape[shape.index(-1)] = self.nelements // known
        if math.prod(shape) != self.nelements:
            raise ValueError("view: element count differs")
        return self._view(shape, contiguous_strides(shape))

    def unsqueeze(self, axis):
        axis = axis % (self.rank + 1)
        shape, strides = list(self.shape), list(self.strides)
        stride = strides[axis] * shape[axis] if axis < self.rank else 1
        shape.insert(axis, 1)
        strides.insert(axis, stride)
        return self._view(shape, strides)

    def squeeze(self):
        keep = [i for i, s in enumerate(self.shape) if s != 1]
        return self._view([self.shape[i] for i in keep], [self.strides[i] for i in keep])

    def __getitem__(self, index):
        """Integer and range indexing; offsets accumulate in bytes (``slices.hpp:97,103``)."""
        if not isinstance(index, tuple):
            index = (index,)
        shape, strides, offset = [], [], self.offset
        dim = 0
        for ix in index:
            if ix is Ellipsis:
                skip = self.rank - (len(index) - 1) - dim
                for _ in range(skip):
                    shape.append(self.shape[dim]); strides.append(self.strides[dim]); dim += 1
                continue
            if isinstance(ix, slice):
                start, stop, step = ix.indices(self.shape[dim])
                n = max(0, (stop - start + step - 1) // step) if step > 0 else 0
                offset += start * self.strides[dim] * self.dtype.itemsize
                shape.append(n); strides.append(self.strides[dim] * step)
            else:
                i = int(ix) % self.shape[dim]
                offset += i * self.strides[dim] * self.dtype.itemsize
            dim += 1
        while dim < self.rank:
            shape.append(self.shape[dim]); strides.append(self.strides[dim]); dim += 1
        return self._view(shape, strides, offset)

    def __repr__(self):
        return f"Tensor({self.dtype}, shape={self.shape}, strides={self.strides}, offset={self.offset})"


def tensor(values, dtype, environment=None):
    """Contiguous tensor holding ``values`` (shape taken from the array)."""
    a = np.asarray(values)
    t = Tensor(dtype, a.shape)
    return t.initialize(a, environment or Host())
