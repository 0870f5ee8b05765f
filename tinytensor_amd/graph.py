"""HIP streams and graphs for the Python mirror: run a sequence of backend calls on a stream of its own, or record it
once into a HIP graph and replay it with one launch.

No counterpart in the reference (its CUDA backend launches everything on the default stream,
tinytensor/tensor/backend/cuda/kernel_launch.cuh:19-29).  Every entry point of the C ABI takes the stream it
launches on and only records kernels (no memset or copy nodes), so a step that has run once on the stream — which
sets the kernels' attributes, grows the per-stream scratch and leaves its result blocks in the allocator's cache —
can be captured without allocating.  The graph replays with the addresses it was recorded with: the tensors the
captured function reads are refreshed in place (Graph.copy_in), and every block the function allocated while it was
being recorded -- results and temporaries alike -- stays pinned to the Graph object until Graph.close(), so that no
later allocation can receive a block that a replay still writes.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _capi
from .tensor import Tensor, TTException, get_backend, kAMD, pin_allocations

_hip = None


def _runtime():
    global _hip
    if _hip is None:
        lib = C.CDLL("libamdhip64.so")
        vp = C.c_void_p
        for name, args in {
            "hipStreamCreate": [C.POINTER(vp)], "hipStreamCreateWithFlags": [C.POINTER(vp), C.c_uint],
            "hipStreamSynchronize": [vp], "hipStreamDestroy": [vp], "hipStreamQuery": [vp],
            "hipStreamBeginCapture": [vp, C.c_int], "hipStreamEndCapture": [vp, C.POINTER(vp)],
            "hipGraphInstantiate": [C.POINTER(vp), vp, C.POINTER(vp), C.c_char_p, C.c_size_t],
            "hipGraphLaunch": [vp, vp], "hipGraphExecDestroy": [vp], "hipGraphDestroy": [vp],
            "hipGraphGetNodes": [vp, C.POINTER(vp), C.POINTER(C.c_size_t)],
            "hipStreamIsCapturing": [vp, C.POINTER(C.c_int)],
        }.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = args, C.c_int
        _hip = lib
    return _hip


def _call(name: str, *args) -> None:
    rc = getattr(_runtime(), name)(*args)
    if rc != 0:
        raise TTException(f"{name} failed with HIP error {rc}")


def stream_is_capturing(handle) -> bool:
    """Whether the stream with this hipStream_t handle (None or 0: the default stream) is recording a graph."""
    if not handle:
        return False
    status = C.c_int(0)
    _call("hipStreamIsCapturing", C.c_void_p(handle), C.byref(status))
    return status.value != 0  # hipStreamCaptureStatusNone == 0


class Stream:
    """A HIP stream at the default priority.  `non_blocking`: the stream does not synchronise implicitly with the
    default stream (hipStreamNonBlocking), so work on the two may overlap."""

    def __init__(self, non_blocking: bool = False):
        self._h = C.c_void_p()
        if non_blocking:
            _call("hipStreamCreateWithFlags", C.byref(self._h), 1)  # hipStreamNonBlocking
        else:
            _call("hipStreamCreate", C.byref(self._h))

    @property
    def handle(self) -> int:
        return self._h.value

    def synchronize(self) -> None:
        _call("hipStreamSynchronize", self._h)

    def is_idle(self) -> bool:
        """Whether everything enqueued on the stream so far has finished (hipStreamQuery; not during a capture)."""
        rc = _runtime().hipStreamQuery(self._h)
        if rc not in (0, 600):  # hipSuccess, hipErrorNotReady
            raise TTException(f"hipStreamQuery failed with HIP error {rc}")
        return rc == 0

    def run(self, fn):
        """Calls fn() with every backend launch going to this stream (asynchronously); returns fn's result."""
        with get_backend(kAMD).on_stream(self.handle):
            return fn()

    def close(self) -> None:
        """Waits for the stream's work and takes the handle off the allocator's books (blocks allocated or freed for
        this stream stay usable; nothing will wait on the stream again), then destroys it."""
        if self._h.value:
            rc = _capi.lib.ttamd_stream_release(kAMD.id, self._h)
            if rc != 0:
                raise TTException(_capi.lib.ttamd_last_error_string().decode())
            _call("hipStreamDestroy", self._h)
            self._h = C.c_void_p()


class Graph:
    """fn's launches recorded once; launch() replays them on the stream they were captured from."""

    def __init__(self, stream: Stream, fn, warmup: int = 2):
        self.stream = stream
        self._graph, self._exec = C.c_void_p(), C.c_void_p()
        # The warm-up runs keep their allocations until they end, as the recorded run will: afterwards the allocator's
        # cache holds one block for every tensor the function creates, temporaries included, and the capture below
        # finds them all there.
        for _ in range(warmup):
            keep: list = []
            with pin_allocations(keep):
                stream.run(fn)
            stream.synchronize()
            with get_backend(kAMD).on_stream(stream.handle):
                del keep[:]  # returned for this stream
        stream.synchronize()
        # Global capture mode: an allocation or a blocking call anywhere in the process would invalidate the capture,
        # which is the guarantee wanted here.
        self._pinned: list = []  # every storage allocated during the capture, held until close()
        _call("hipStreamBeginCapture", stream._h, 0)
        try:
            with pin_allocations(self._pinned):
                self.outputs = stream.run(fn)
        finally:
            rc = _runtime().hipStreamEndCapture(stream._h, C.byref(self._graph))
        if rc != 0 or not self._graph.value:
            raise TTException(f"HIP graph capture failed (hipStreamEndCapture returned {rc})")
        _call("hipGraphInstantiate", C.byref(self._exec), self._graph, None, None, 0)

    def num_nodes(self) -> int:
        n = C.c_size_t(0)
        _call("hipGraphGetNodes", self._graph, None, C.byref(n))
        return n.value

    def launch(self) -> None:
        _call("hipGraphLaunch", self._exec, self.stream._h)

    @staticmethod
    def copy_in(dst: Tensor, src: np.ndarray) -> None:
        """Blocking copy of new values into a dense tensor the graph reads (same dtype and size)."""
        src = np.ascontiguousarray(src)
        if src.nbytes != dst.numel() * dst.itemsize or dst.offset != 0:
            raise TTException("copy_in needs a dense tensor of the same byte size")
        rc = _capi.lib.ttamd_memcpy_h2d(dst.device.id, C.c_void_p(dst.storage.ptr), src.ctypes.data_as(C.c_void_p), src.nbytes)
        if rc != 0:
            raise TTException(_capi.lib.ttamd_last_error_string().decode())

    def close(self) -> None:
        if self._exec.value:
            _call("hipGraphExecDestroy", self._exec)
            self._exec = C.c_void_p()
        if self._graph.value:
            _call("hipGraphDestroy", self._graph)
            self._graph = C.c_void_p()
        self._pinned = []  # the blocks go back to the allocator (for the stream current now)
