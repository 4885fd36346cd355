"""``TorchCUDAGraphConstructor`` -- Python facade of the graph builder, same public
methods as the reference (pytorch/cpp_extensions/cuda_graph_constructor.py:12-147):
a list of registered streams (the first is where branches join and where the graph is
launched), a capture notifier that keeps torch's allocator consistent, and the native
builder that turns each ``capture_library_call_begin/end`` pair into a branch.
"""
from __future__ import annotations

import torch

import intrasm_engine_amd
from ... import extensions as iex
from ...common.compound_streams import CompoundStream


class TorchCUDAGraphConstructor:
    def __init__(self, device=None):
        if device is None:
            device = torch.device(f"cuda:{torch.cuda.current_device()}")
        self.device = torch.device(device)
        if self.device not in intrasm_engine_amd.current_stream:
            intrasm_engine_amd.initialize_current_streams()
        self.registeredStreams: list[CompoundStream] = [intrasm_engine_amd.current_stream[self.device]]
        self.notifier = iex.CUDAGraphCaptureNotifier()
        self.constructor = iex.CUDAExperimentalGraphConstructor()
        self.constructor.register_stream(self.registeredStreams[0].handle)

    def get_primary_stream(self) -> CompoundStream:
        """The first stream: where streams join and where the graph is executed."""
        return self.registeredStreams[0]

    def register_new_stream(self) -> CompoundStream:
        # default priority on purpose: mixed stream priorities must not be used here
        stream = CompoundStream(torch.cuda.stream(torch.cuda.Stream(device=self.device)))
        self.registeredStreams.append(stream)
        self.constructor.register_stream(stream.handle)
        return stream

    def register_new_streams(self, num_streams: int) -> list[CompoundStream]:
        return [self.register_new_stream() for _ in range(num_streams)]

    def print_graph(self):
        self.constructor.print_graph()

    def dump_graph(self, path: str):
        self.constructor.dump_graph(path)

    def assert_current_stream_registered(self):
        assert torch.cuda.current_stream() in {
            context.torch_stream.stream for context in self.registeredStreams
        }, "Current stream is not registered."

    @staticmethod
    def _event_handle(event: torch.cuda.Event) -> int:
        # torch creates the underlying event lazily, at the first record()
        assert event.cuda_event != 0, (
            "Event uninitialized! PyTorch initialize the event lazily. Please"
            " call event.record() after creating the event object and before"
            " the real recording to make sure the event is initialized."
        )
        return event.cuda_event

    def add_event_record_node(self, event: torch.cuda.Event, torch_stream):
        self.constructor.add_event_record_node(self._event_handle(event), torch_stream.stream.cuda_stream)

    def add_stream_wait_event_node(self, torch_stream, event: torch.cuda.Event):
        self.constructor.add_stream_wait_event_node(torch_stream.stream.cuda_stream, self._event_handle(event))

    def capture_library_call_begin(self):
        self.assert_current_stream_registered()
        self.notifier.capture_begin(None)
        try:
            self.constructor.notify_before_invoking_library_call(torch.cuda.current_stream().cuda_stream)
        except Exception:
            self.notifier.abort()
            raise
        self.notifier.assert_capture_has_begun()

    def capture_library_call_end(self):
        try:
            self.constructor.notify_after_invoking_library_call(torch.cuda.current_stream().cuda_stream)
        finally:
            self.notifier.capture_end()

    def instantiate_graph_exec(self):
        self.constructor.instantiate_graph_exec()

    def execute_graph(self):
        self.notifier.replay()
        self.constructor.execute_graph(self.registeredStreams[0].handle)

    def join(self, streams: list[CompoundStream], dest_stream: CompoundStream):
        self.constructor.join([s.handle for s in streams], dest_stream.handle)

    def synchronize(self):
        torch.cuda.synchronize(device=self.device)

    def destroy_graph_exec(self):
        self.constructor.destroy_graph_exec()

    # context-manager form, as torch.cuda.graph: `with stream_ctx: with constructor: ...`
    def __enter__(self):
        self.capture_library_call_begin()
        return self

    def __exit__(self, *args):
        self.capture_library_call_end()
