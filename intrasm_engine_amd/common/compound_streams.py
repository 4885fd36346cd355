"""Stream context used by the graph builder.

The reference bundles three views of one CUDA stream (pycuda, torch, cupy) because its
dense companions are launched through three different Python libraries
(common/compound_streams.py:7-58).  Here every kernel is launched on torch's current
stream, so the bundle holds the torch ``StreamContext`` only; the attribute names the
callers use (``torch_stream``, ``device``, context-manager protocol) are kept.
"""
from __future__ import annotations

import torch


class CompoundStream:
    def __init__(self, torch_stream: "torch.cuda.StreamContext"):
        self.torch_stream = torch_stream
        self.device = torch_stream.stream.device

    @property
    def stream(self) -> "torch.cuda.Stream":
        return self.torch_stream.stream

    @property
    def handle(self) -> int:
        """The hipStream_t as an integer."""
        return self.torch_stream.stream.cuda_stream

    def __enter__(self):
        self.torch_stream.__enter__()
        return self

    def __exit__(self, *args):
        self.torch_stream.__exit__(*args)
