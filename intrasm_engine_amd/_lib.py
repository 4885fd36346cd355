"""ctypes binding of ``libiex_hip.so`` (the C ABI declared in ``include/iex_hip.h``).

The library is the only compute path of the package: if it is missing, or a call
fails, an exception is raised -- there is no Python or CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libiex_hip.so")

F32, F16, BF16 = 0, 1, 2
I32, I16 = 0, 1

SPMM_PER_BATCH_VALUES = 0x1
SPMM_ACCUMULATE = 0x2
SPMM_RELU = 0x4
SPMM_TABLES_READY = 0x8
SPMM_LISTS_READY = 0x10
SPMM_BESIDE_GATHER_KERNEL = 0x40
SPMM_ANY_COLUMN_ORDER = 0x20
SDDMM_SUM_OVER_BATCH = 0x1
SDDMM_ACCUMULATE = 0x2
SDDMM_TABLES_READY = 0x4
SDDMM_LISTS_READY = 0x8
SDDMM_ANY_COLUMN_ORDER = 0x10
CSR_BAD_OFFSETS, CSR_COLUMN_OUT_OF_RANGE, CSR_NOT_ASCENDING = 0x1, 0x2, 0x4

_c = ctypes
_vp, _i, _ll, _f = _c.c_void_p, _c.c_int, _c.c_longlong, _c.c_float

# name -> (restype, argtypes).  Kept in one table so that the symbol-export test can
# walk it against the header.
SIGNATURES = {
    "iex_abi_version": (_i, []),
    "iex_last_error": (_c.c_char_p, []),
    "iex_last_kernels": (_c.c_char_p, []),
    "iex_device_ok": (_i, []),
    "iex_copy_bytes": (_i, [_vp, _vp, _c.c_size_t, _vp]),
    "iex_spmm_ex": (_i, [_i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_spmm_ws": (_i, [_i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _c.c_size_t]),
    "iex_spmm_sched": (_i, [_i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _c.c_size_t, _c.POINTER(_i)]),
    "iex_csr_row_histogram": (_i, [_i, _vp, _vp, _vp]),
    "iex_csr_dense_share": (_i, [_i, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _c.c_size_t, _vp]),
    "iex_csr_dense_share_scratch_bytes": (_c.c_size_t, [_i, _i]),
    "iex_spmm_workspace_bytes": (_c.c_size_t, [_i, _i, _i, _i, _i, _i, _i, _i]),
    "iex_spmm_workspace_kind": (_i, [_i, _i, _i, _i, _i, _i, _i, _i]),
    "iex_spmm_static": (_i, [_i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_spmm_static_scratch_bytes": (_c.c_size_t, []),
    "iex_CudaSpmm2": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_CudaSpmm3": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_CudaSpmm5": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_csr_check": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "iex_sddmm_ex": (_i, [_i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_sddmm_ws": (_i, [_i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _c.c_size_t]),
    "iex_sddmm_workspace_bytes": (_c.c_size_t, [_i, _i, _i, _i, _i, _i, _i]),
    "iex_sddmm_workspace_kind": (_i, [_i, _i, _i, _i, _i, _i, _i]),
    "iex_pattern_tables_bytes": (_c.c_size_t, [_i, _i, _i]),
    "iex_pattern_tables": (_i, [_i, _i, _i, _vp, _vp, _vp, _c.c_size_t, _vp]),
    "iex_CudaSddmm2": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i]),
    "iex_csr_softmax": (_i, [_i, _i, _i, _vp, _vp, _vp, _f, _vp, _i]),
    "iex_gemm": (_i, [_i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _ll, _ll, _ll, _vp]),
    "iex_gemm_ws": (_i, [_i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _ll, _ll, _ll, _vp, _vp, _c.c_size_t]),
    "iex_gemm_workspace_bytes": (_c.c_size_t, [_i, _i, _i, _i, _i, _i]),
    "iex_fused_spmm_gemm": (_i, [_i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp,
                                 _i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _ll, _ll, _ll, _i, _vp]),
    "iex_fused_role": (_i, [_i, _i, _i, _i, _c.POINTER(_i), _c.POINTER(_i)]),
    "iex_fused_timeline": (_i, [_vp]),
    "iex_graph_create": (_vp, []),
    "iex_graph_wrap": (_vp, [_vp]),
    "iex_graph_destroy": (None, [_vp]),
    "iex_graph_handle": (_vp, [_vp]),
    "iex_graph_register_stream": (_i, [_vp, _vp]),
    "iex_graph_begin_capture": (_i, [_vp, _vp]),
    "iex_graph_end_capture": (_i, [_vp, _vp]),
    "iex_graph_add_event_record_node": (_i, [_vp, _vp, _vp]),
    "iex_graph_add_stream_wait_event_node": (_i, [_vp, _vp, _vp]),
    "iex_graph_join": (_i, [_vp, _c.POINTER(_vp), _i, _vp]),
    "iex_graph_instantiate": (_i, [_vp]),
    "iex_graph_launch": (_i, [_vp, _vp]),
    "iex_graph_destroy_exec": (_i, [_vp]),
    "iex_graph_add_child_graph": (_i, [_vp, _vp]),
    "iex_graph_combine": (_vp, [_c.POINTER(_vp), _i]),
    "iex_graph_dump_dot": (_i, [_vp, _c.c_char_p]),
    "iex_graph_num_nodes": (_ll, [_vp]),
    "iex_graph_num_edges": (_ll, [_vp]),
    "iex_graph_get_edges": (_ll, [_vp, _c.POINTER(_ll), _c.POINTER(_ll), _ll]),
    "iex_graph_node_type": (_i, [_vp, _ll]),
    "iex_stream_is_capturing": (_i, [_vp]),
    "iex_echo_stream": (_ll, [_vp]),
    "iex_echo_event": (_ll, [_vp]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library and bind every entry point.  Raises ImportError when the
    shared object has not been built (``python -c 'import __graft_entry__ as g; g.build()'``,
    ``python intrasm_engine_amd/csrc/build.py`` or ``make -C intrasm_engine_amd/csrc``)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(hipcc, --offload-arch=gfx950).  There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library disagree
        fn.restype = res
        fn.argtypes = args
    if lib.iex_abi_version() != 1:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.iex_abi_version()} != 1")
    _lib = lib
    return lib


def last_kernels() -> str:
    """Kernels launched by the most recent compute entry point on this thread."""
    return load().iex_last_kernels().decode("utf-8", "replace")


def last_error() -> str:
    return load().iex_last_error().decode("utf-8", "replace")


def check(rc: int, what: str = "") -> None:
    """Turn a non-zero return code into RuntimeError carrying the library's message
    (the reference raises through AT_CUDA_CHECK / TORCH_CHECK, sputnik_kernels.cpp:93)."""
    if rc != 0:
        msg = last_error()
        raise RuntimeError(f"{what + ': ' if what else ''}{msg or 'error'} (code {rc})")
