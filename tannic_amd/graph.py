"""Backend calls recorded once and replayed as one HIP graph (``tannic_hip_graph_*``).

The reference's front end evaluates every expression where it is written, one backend call per node; for a sequence
of short kernels (a decoder layer is some sixty) issuing the calls takes longer than running them.  A ``Graph`` records
the calls made inside its ``with`` block on a device and replays them with one launch::

    x = tensor(..., Device())
    with Graph(x.environment) as g:
        y = layer.forward(x, ...)        # recorded, not run
    g.launch()                           # y now holds forward(x)
    ops.copy_into(x, new_input)          # (any eager call that writes x's memory)
    g.launch()                           # y holds forward(new_input)

Tensors created inside the block keep their addresses for the life of the graph and are rewritten by every launch;
tensors that existed before (inputs, weights) must stay allocated while the graph is launched.  Calls that wait for
the device (``numpy()``, ``allclose``) cannot be recorded and raise.
"""
from . import abi
from .backend import BackendError, library
from .tensor import Device


class Graph:
    def __init__(self, device=None):
        self.device = device if device is not None else Device()
        if not isinstance(self.device, Device):
            raise TypeError("Graph records calls on a Device")
        self.handle = None
        self.ready = False

    def __enter__(self):
        lib = library()
        self.handle = lib.graph_begin(self.device.reference)
        if not self.handle:
            raise BackendError(lib.error_message())
        # the operators of this harness launch on the stream the device handed out once (Device.stream); a recording on
        # any other stream would record nothing and the calls would run eagerly
        if lib.graph_stream(self.handle).address != self.device.stream().address:
            self.close()
            raise BackendError("Graph: the backend records another stream than the one this device's operators use (a stream popped and not put back?)")
        return self

    def __exit__(self, kind, value, trace):
        lib = library()
        if kind is not None:
            # the block failed: drop the recording, let the exception through
            self.close()
            return False
        if lib.graph_end(self.handle) != abi.SUCCESS:
            message = lib.error_message()
            self.close()
            raise BackendError(message)
        self.ready = True
        return False

    def launch(self):
        """Queue one replay on the device's stream (asynchronous, like every backend call)."""
        if not self.ready:
            raise BackendError("Graph.launch: nothing recorded")
        lib = library()
        if lib.graph_launch(self.handle) != abi.SUCCESS:
            raise BackendError(lib.error_message())

    def close(self):
        """Wait for the stream and release the recording and the memory it owns."""
        if self.handle:
            library().graph_destroy(self.handle)
        self.handle, self.ready = None, False

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
