"""Co-run measurement harness: "each kernel list alone" against "one list per stream in
one graph".

Same protocol as the reference's harness (tests/test_interleaving.py:21-23, 348-369,
434-476): every list of zero-argument callables ("execs") is captured through
``TorchCUDAGraphConstructor``; the serialized figure captures all lists on ONE stream,
the co-run figure captures one list per registered stream and joins the branches; a
graph launch is timed with events recorded on the primary stream.  Unlike the reference
(one launch, one sample) the launch is repeated and the median is reported.
"""
from __future__ import annotations

import statistics
from typing import Callable, Sequence

import torch

from .pytorch.cpp_extensions.cuda_graph_constructor import TorchCUDAGraphConstructor


def gemm_tflops(m: int, n: int, k: int, time_ms: float) -> float:
    """2*m*n*k / time, counting A*B only (tests/test_interleaving.py:21-23)."""
    return 2.0 * m * n * k / (time_ms * 1e-3) / 1e12


def _time_graph(constructor: TorchCUDAGraphConstructor, repeats: int, warmup: int) -> list[float]:
    constructor.instantiate_graph_exec()
    times = []
    try:
        for _ in range(warmup):
            constructor.execute_graph()
        constructor.synchronize()
        for _ in range(repeats):
            start = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            start.record()
            constructor.execute_graph()
            end.record()
            constructor.synchronize()
            times.append(start.elapsed_time(end))
    finally:
        constructor.destroy_graph_exec()
    return times


def capture_serialized(*exec_lists: Sequence[Callable[[], object]]):
    """All lists on the primary stream, interleaved element by element
    (the body of run_non_interleaving, tests/test_interleaving.py:348-359)."""
    constructor = TorchCUDAGraphConstructor()
    keep = []
    with constructor.get_primary_stream():
        constructor.capture_library_call_begin()
        try:
            for idx in range(len(exec_lists[0])):
                for execs in exec_lists:
                    keep.append(execs[idx]())
        finally:
            constructor.capture_library_call_end()
    return constructor, keep


def capture_interleaved(*exec_lists: Sequence[Callable[[], object]], constructor: TorchCUDAGraphConstructor | None = None):
    """One list per stream, branches joined on the primary stream
    (the body of run_interleaving, tests/test_interleaving.py:451-464)."""
    if constructor is None:
        constructor = TorchCUDAGraphConstructor()
        constructor.register_new_streams(len(exec_lists) - 1)
    assert len(constructor.registeredStreams) == len(exec_lists)
    keep = []
    for stream, execs in zip(constructor.registeredStreams, exec_lists):
        with stream:
            constructor.capture_library_call_begin()
            try:
                for fn in execs:
                    keep.append(fn())
            finally:
                constructor.capture_library_call_end()
    constructor.join(constructor.registeredStreams[1:], constructor.registeredStreams[0])
    return constructor, keep


def run_non_interleaving(*exec_lists, repeats: int = 5, warmup: int = 1) -> float:
    """Median milliseconds of one launch of the single-stream graph."""
    constructor, keep = capture_serialized(*exec_lists)
    times = _time_graph(constructor, repeats, warmup)
    del keep
    return statistics.median(times)


def run_interleaving(*exec_lists, constructor: TorchCUDAGraphConstructor | None = None, repeats: int = 5,
                     warmup: int = 1) -> float:
    """Median milliseconds of one launch of the multi-branch graph."""
    constructor, keep = capture_interleaved(*exec_lists, constructor=constructor)
    times = _time_graph(constructor, repeats, warmup)
    del keep
    return statistics.median(times)


def time_execs(execs: Sequence[Callable[[], object]], repeats: int = 5, warmup: int = 1) -> float:
    """Median milliseconds of one graph holding ``execs`` back to back on one stream."""
    return run_non_interleaving(list(execs), repeats=repeats, warmup=warmup)
