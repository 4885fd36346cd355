"""numpy front-end of the CPU oracle (``oracle.c``).

TEST INFRASTRUCTURE ONLY.  Importers are limited to ``tests/``, the smoke check
and the benchmark's CPU-baseline leg; the shipped package never imports this
module.  Every function converts its operands to float32 / int32 C arrays, calls
the C restatement and returns float64 (or float32 for the ``*_f32`` timing
variants) numpy arrays.  fp16 / bf16 operands are widened exactly before the
call, so the oracle always sees the same rounded inputs as the device kernels.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``oracle.c`` with gcc (a second or two)."""
    src = os.path.join(_HERE, "oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _f32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


def _i32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.int32))


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct)) if a is not None else None


_F = ctypes.c_float
_D = ctypes.c_double
_I = ctypes.c_int


def spmm(b, row_indices, values, row_offsets, column_indices, m, *, out_init=None,
         bias=None, relu=False):
    """float64 ``out[z] = A @ b[z]``.  ``values`` 1-D (shared by the batch) or 2-D
    (batch, nnz).  ``out_init`` turns on accumulate mode (``out = out_init + A @ b``)."""
    b = _f32(b)
    assert b.ndim == 3
    batch, k, n = b.shape
    values = _f32(values)
    ri, ro, ci = _i32(row_indices), _i32(row_offsets), _i32(column_indices)
    nnz = ci.shape[0]
    per_batch = int(values.ndim == 2)
    if out_init is not None:
        out = np.ascontiguousarray(np.asarray(out_init, dtype=np.float64)).copy()
    else:
        out = np.zeros((batch, m, n), dtype=np.float64)
    bias_a = _f32(bias) if bias is not None else None
    lib().oracle_spmm_f64(m, k, n, nnz, _p(ri, _I), _p(values, _F), _p(ro, _I), _p(ci, _I),
                          _p(b, _F), _p(out, _D), batch, per_batch, int(out_init is not None),
                          _p(bias_a, _F), int(relu))
    return out


def spmm_f32(b, row_indices, values, row_offsets, column_indices, m):
    """float32-accumulate variant (the single-core CPU port timed by the benchmark)."""
    b = _f32(b)
    batch, k, n = b.shape
    values = _f32(values)
    ri, ro, ci = _i32(row_indices), _i32(row_offsets), _i32(column_indices)
    out = np.zeros((batch, m, n), dtype=np.float32)
    lib().oracle_spmm_f32(m, k, n, ci.shape[0], _p(ri, _I), _p(values, _F), _p(ro, _I),
                          _p(ci, _I), _p(b, _F), _p(out, _F), batch, int(values.ndim == 2), 0)
    return out


def spmm_abs_scale(b, row_indices, values, row_offsets, column_indices, m):
    """sum_j |a_j| * |b[col_j, :]| per output element: the condition scale used to
    bound the error of outputs that cancel towards zero."""
    return spmm(np.abs(_f32(b)), row_indices, np.abs(_f32(values)), row_offsets, column_indices, m)


def sddmm(a, b, row_indices, row_offsets, column_indices, *, sum_over_batch=True, out_init=None):
    """float64 sampled ``a @ b^T`` at the CSR pattern.  a: (batch,m,k); b: (batch,n,k)."""
    a, b = _f32(a), _f32(b)
    assert a.ndim == 3 and b.ndim == 3
    batch, m, k = a.shape
    n = b.shape[1]
    ri, ro, ci = _i32(row_indices), _i32(row_offsets), _i32(column_indices)
    nnz = ci.shape[0]
    shape = (nnz,) if sum_over_batch else (batch, nnz)
    if out_init is not None:
        out = np.ascontiguousarray(np.asarray(out_init, dtype=np.float64)).copy()
        assert out.shape == shape
    else:
        out = np.zeros(shape, dtype=np.float64)
    lib().oracle_sddmm_f64(m, k, n, nnz, _p(ri, _I), _p(ro, _I), _p(ci, _I), _p(a, _F), _p(b, _F),
                           _p(out, _D), batch, int(sum_over_batch), int(out_init is not None))
    return out


def sddmm_f32(a, b, row_indices, row_offsets, column_indices, *, sum_over_batch=True):
    a, b = _f32(a), _f32(b)
    batch, m, k = a.shape
    n = b.shape[1]
    ri, ro, ci = _i32(row_indices), _i32(row_offsets), _i32(column_indices)
    nnz = ci.shape[0]
    out = np.zeros((nnz,) if sum_over_batch else (batch, nnz), dtype=np.float32)
    lib().oracle_sddmm_f32(m, k, n, nnz, _p(ri, _I), _p(ro, _I), _p(ci, _I), _p(a, _F), _p(b, _F),
                           _p(out, _F), batch, int(sum_over_batch))
    return out


def sddmm_abs_scale(a, b, row_indices, row_offsets, column_indices, *, sum_over_batch=True):
    return sddmm(np.abs(_f32(a)), np.abs(_f32(b)), row_indices, row_offsets, column_indices,
                 sum_over_batch=sum_over_batch)


def gemm(a, b, *, trans_b=False):
    """float64 ``a @ b`` (b is (K,N)) or ``a @ b.T`` (b is (N,K))."""
    a, b = _f32(a), _f32(b)
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    assert (b.shape[1] if trans_b else b.shape[0]) == K
    out = np.zeros((M, N), dtype=np.float64)
    lib().oracle_gemm_f64(M, N, K, _p(a, _F), _p(b, _F), int(trans_b), _p(out, _D))
    return out


def dense_to_csr(matrix):
    """(values, row_indices, row_offsets, column_indices), the reference's tuple order."""
    mat = _f32(matrix)
    m, k = mat.shape
    nnz = lib().oracle_dense_to_csr(m, k, _p(mat, _F), None, None, None, None)
    values = np.zeros(nnz, dtype=np.float32)
    ri = np.zeros(m, dtype=np.int32)
    ro = np.zeros(m + 1, dtype=np.int32)
    ci = np.zeros(nnz, dtype=np.int32)
    lib().oracle_dense_to_csr(m, k, _p(mat, _F), _p(values, _F), _p(ri, _I), _p(ro, _I), _p(ci, _I))
    return values, ri, ro, ci


def csr_to_dense(m, k, values, row_offsets, column_indices):
    out = np.zeros((m, k), dtype=np.float64)
    ro = np.asarray(row_offsets)
    rows = np.repeat(np.arange(m), np.diff(ro))
    out[rows, np.asarray(column_indices).astype(np.int64)] = np.asarray(values, dtype=np.float64)
    return out


def csr_transpose(m, k, row_offsets, column_indices):
    """(row_offsets_t, column_indices_t, perm): values_t = values[perm]."""
    ro, ci = _i32(row_offsets), _i32(column_indices)
    nnz = ci.shape[0]
    ro_t = np.zeros(k + 1, dtype=np.int32)
    ci_t = np.zeros(nnz, dtype=np.int32)
    perm = np.zeros(nnz, dtype=np.int32)
    lib().oracle_csr_transpose(m, k, nnz, _p(ro, _I), _p(ci, _I), _p(ro_t, _I), _p(ci_t, _I),
                               _p(perm, _I))
    return ro_t, ci_t, perm


def csr_softmax(values, row_offsets):
    """Row-wise softmax over the stored entries of a CSR matrix (float64), the
    middle step of sparse attention between SDDMM and SpMM.  values: (..., nnz)."""
    v = np.asarray(values, dtype=np.float64)
    ro = np.asarray(row_offsets)
    out = np.empty_like(v)
    for r in range(len(ro) - 1):
        s, e = ro[r], ro[r + 1]
        if e > s:
            seg = v[..., s:e]
            ex = np.exp(seg - seg.max(axis=-1, keepdims=True))
            out[..., s:e] = ex / ex.sum(axis=-1, keepdims=True)
    return out
