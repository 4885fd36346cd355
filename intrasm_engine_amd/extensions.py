"""Counterpart of the reference's pybind module ``intrasm_engine_extensions``
(pytorch/csrc/extensions/pybind.cu:483-616): same class and method names, thin
wrappers over the ``iex_graph_*`` C ABI.  Usual import: ``import
intrasm_engine_amd.extensions as iex``.  Handles cross as Python ints.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib


def _L():
    return _lib.load()


def print_cudastream(stream):
    """Round-trips one stream handle (or a list) through the native library and prints
    it; returns what the library saw (pybind.cu:17-33)."""
    if isinstance(stream, (list, tuple)):
        return [print_cudastream(s) for s in stream]
    seen = _L().iex_echo_stream(int(stream))
    if seen < 0:
        raise RuntimeError(_lib.last_error())
    print(f"stream {seen:#x}")
    return seen


def print_cudaevent(event):
    """Same for an event handle; a null handle is an error (pybind.cu:35-45)."""
    seen = _L().iex_echo_event(int(event) if event else None)
    if seen < 0:
        raise RuntimeError(_lib.last_error())
    print(f"event {seen:#x}")
    return seen


class CUDAGraphCaptureNotifier:
    """Keeps PyTorch consistent while a capture that torch did not start is running on
    the current stream (pybind.cu:163-333): allocations made during the capture go to a
    private memory pool that outlives the capture, so tensors created inside it keep
    their addresses for every replay.

    RNG bookkeeping: no operator of this path consumes Philox random numbers, so the
    seed/offset tensors of the reference are not needed; ``replay`` is kept as the hook
    that ``execute_graph`` calls.
    """

    def __init__(self):
        self._device = None
        self._pool = None
        self._capture_stream = None
        self._active = False

    def capture_begin(self, pool=None):
        stream = torch.cuda.current_stream()
        if stream == torch.cuda.default_stream(stream.device):
            raise RuntimeError(
                "CUDA graphs must be captured on a non-default stream. (However, after capture, "
                "it's ok to replay them on the default stream.)")
        if self._active:
            raise RuntimeError("capture_begin called twice without capture_end")
        self._device = stream.device.index
        if pool is not None:
            self._pool = tuple(pool)
        elif self._pool is None:
            self._pool = torch.cuda.graph_pool_handle()
        self._capture_stream = stream
        # before the capture starts, as in the reference (pybind.cu:221-237)
        torch._C._cuda_beginAllocateCurrentStreamToPool(self._device, self._pool)
        self._active = True

    def assert_capture_has_begun(self):
        if not _L().iex_stream_is_capturing(torch.cuda.current_stream().cuda_stream):
            raise RuntimeError("the current stream is not capturing")

    def capture_end(self):
        if not self._active:
            raise RuntimeError("capture_end without capture_begin")
        if torch.cuda.current_stream() != self._capture_stream:
            raise RuntimeError("Capture must end on the same stream it began on.")
        torch._C._cuda_endAllocateToPool(self._device, self._pool)
        self._active = False

    def abort(self):
        """Undo capture_begin after a failed begin (keeps the allocator usable)."""
        if self._active:
            torch._C._cuda_endAllocateToPool(self._device, self._pool)
            self._active = False

    def replay(self):
        return None

    def pool(self):
        return self._pool

    def release_pool(self):
        """Let the allocator reclaim the capture's pool once its tensors are gone."""
        if self._pool is not None and self._device is not None:
            torch._C._cuda_releasePool(self._device, self._pool)
            self._pool = None

    def __del__(self):
        try:
            if not self._active:
                self.release_pool()
        except Exception:
            pass


class CudaGraphWrapper:
    """Owns a graph handle and its executable graph (helper_CUDAGraphConstructor.cu.h:106-166)."""

    def __init__(self, graph, _builder=None):
        """``graph``: a hipGraph_t as an integer (ownership passes to the wrapper).
        ``_builder`` (internal): an ``iex_graph*`` this module already created."""
        if _builder is not None:
            self._g = _builder
        else:
            self._g = _L().iex_graph_wrap(int(graph))
        if not self._g:
            raise RuntimeError(_lib.last_error())
        self._added_as_child = False

    def _check(self, rc):
        _lib.check(rc, "graph")

    def notify_added_as_child_graph(self):
        self._added_as_child = True

    def add_graph_as_child_node(self, child):
        self._check(_L().iex_graph_add_child_graph(self._g, child._g))
        child.notify_added_as_child_graph()

    def instantiate_graph_exec(self):
        self._check(_L().iex_graph_instantiate(self._g))

    def execute_graph(self, stream):
        self._check(_L().iex_graph_launch(self._g, int(stream) if stream else None))

    def destroy_graph_exec(self):
        self._check(_L().iex_graph_destroy_exec(self._g))

    def graph_handle(self) -> int:
        return _L().iex_graph_handle(self._g) or 0

    def num_nodes(self) -> int:
        return _L().iex_graph_num_nodes(self._g)

    def num_edges(self) -> int:
        return _L().iex_graph_num_edges(self._g)

    def edges(self):
        n = self.num_edges()
        if n <= 0:
            return []
        a = (ctypes.c_longlong * n)()
        b = (ctypes.c_longlong * n)()
        _L().iex_graph_get_edges(self._g, a, b, n)
        return list(zip(a, b))

    def node_types(self):
        return [_L().iex_graph_node_type(self._g, i) for i in range(self.num_nodes())]

    def dump_graph(self, path: str):
        self._check(_L().iex_graph_dump_dot(self._g, path.encode()))

    def __del__(self):
        g, self._g = getattr(self, "_g", None), None
        if g:
            try:
                _L().iex_graph_destroy(g)
            except Exception:
                pass


class CUDAExperimentalGraphConstructor(CudaGraphWrapper):
    """Per-stream captures -> branches of one graph
    (helper_CUDAGraphConstructor.cu.h:406-486; bound at pybind.cu:530-615)."""

    def __init__(self):
        g = _L().iex_graph_create()
        if not g:
            raise RuntimeError(_lib.last_error())
        super().__init__(None, _builder=g)

    def register_stream(self, stream):
        self._check(_L().iex_graph_register_stream(self._g, int(stream) if stream else None))

    def notify_before_invoking_library_call(self, stream):
        self._check(_L().iex_graph_begin_capture(self._g, int(stream) if stream else None))

    def notify_after_invoking_library_call(self, stream):
        self._check(_L().iex_graph_end_capture(self._g, int(stream) if stream else None))

    def add_event_record_node(self, event, stream):
        self._check(_L().iex_graph_add_event_record_node(self._g, int(event) if event else None,
                                                         int(stream) if stream else None))

    def add_stream_wait_event_node(self, stream, event):
        self._check(_L().iex_graph_add_stream_wait_event_node(self._g, int(stream) if stream else None,
                                                              int(event) if event else None))

    def join(self, streams, dst_stream):
        arr = (ctypes.c_void_p * len(streams))(*[int(s) for s in streams])
        self._check(_L().iex_graph_join(self._g, arr, len(streams), int(dst_stream) if dst_stream else None))

    def print_graph(self):
        for a, b in self.edges():
            print(f"Node {a} has edge to {b}")

    def combine_graphs(self, other) -> CudaGraphWrapper:
        """Both graphs as sibling child nodes of a new graph (helper_cuda_graph.cu.h:34-62)."""
        arr = (ctypes.c_void_p * 2)(self._g, other._g)
        g = _L().iex_graph_combine(arr, 2)
        if not g:
            raise RuntimeError(_lib.last_error())
        self.notify_added_as_child_graph()
        other.notify_added_as_child_graph()
        return CudaGraphWrapper(None, _builder=g)
