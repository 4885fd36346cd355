"""intrasm_engine_amd -- the sparse-plus-dense GEMM path of intrasm_engine, gfx950-native.

Importing the package (mirrors ``intrasm_engine/__init__.py:17-85`` of the reference)
  * loads ``libiex_hip.so`` through ctypes and fails loudly if it is not built,
  * registers the ``torch.ops.iex_ops.*`` operators,
  * when a GPU is visible, creates one non-default HIP stream per device, makes it
    torch's current stream and publishes it as ``current_stream[device]`` (captures
    cannot run on the legacy default stream).
"""
from __future__ import annotations

import torch

from . import _lib

_lib.load()

from .common.compound_streams import CompoundStream  # noqa: E402
from .pytorch import ops as _ops  # noqa: E402

_ops.register()

#: device -> CompoundStream that was current when the package initialised that device
current_stream: dict = {}


def initialize_current_streams() -> None:
    """One fresh stream per visible device, set as torch's current stream
    (reference: ``initialize_current_streams``, intrasm_engine/__init__.py:17-51)."""
    if not torch.cuda.is_available():
        return
    for idx in range(torch.cuda.device_count()):
        device = torch.device(f"cuda:{idx}")
        if device in current_stream:
            continue
        stream = torch.cuda.Stream(device=device)
        current_stream[device] = CompoundStream(torch.cuda.stream(stream))
    torch.cuda.set_device(0)
    torch.cuda.set_stream(current_stream[torch.device("cuda:0")].torch_stream.stream)


initialize_current_streams()
