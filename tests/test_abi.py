"""The C-ABI library loads on a machine without a GPU and exports every symbol that
include/iex_hip.h declares (no compute calls here)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "iex_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(iex_[A-Za-z0-9_]+)\s*\(", text)))


def test_header_declares_the_reference_launchers():
    names = _declared_symbols()
    for required in ("iex_CudaSpmm2", "iex_CudaSpmm3", "iex_CudaSpmm5", "iex_CudaSddmm2", "iex_spmm_ex",
                     "iex_sddmm_ex", "iex_gemm", "iex_fused_spmm_gemm", "iex_graph_create", "iex_graph_join"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from intrasm_engine_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in _declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_binding_table_matches_header():
    from intrasm_engine_amd import _lib
    declared = set(_declared_symbols())
    bound = set(_lib.SIGNATURES)
    assert bound == declared, f"only in header: {declared - bound}; only in binding: {bound - declared}"


def test_version_and_error_text():
    from intrasm_engine_amd import _lib
    lib = _lib.load()
    assert lib.iex_abi_version() == 1
    # argument errors are detected on the host, before any launch
    rc = lib.iex_spmm_ex(_lib.F32, _lib.I32, 0, -1, 4, 4, 0, None, None, None, None, None, None, None, None, 1)
    assert rc == -1 and "negative dimension" in _lib.last_error()
    rc = lib.iex_gemm(_lib.F32, 0, 8, 8, 8, 1, 1, 1, 1, 0, 0, 0, None)
    assert rc == -2 and "fp16 or bf16" in _lib.last_error()
    rc = lib.iex_gemm(_lib.F16, 0, 8, 8, 7, 16, 16, 16, 1, 0, 0, 0, None)
    assert rc == -2 and "multiple of 8" in _lib.last_error()
    rc = lib.iex_graph_instantiate(None)
    assert rc == -1


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from intrasm_engine_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libiex_hip.so"))
    try:
        _lib.load()
    except ImportError as e:
        assert "no fallback" in str(e).lower()
    else:
        raise AssertionError("load() must raise when the shared object is absent")
