"""The on-disk CSR pattern format of the DLMC collection (``.smtx``) and its MatrixMarket
companion, as the reference's benchmark tooling reads and writes them (benchmark/utils.py:11-44).

``.smtx`` holds a sparsity pattern without values, three lines of text:

    num_rows, num_cols, num_nonzeros          (comma separated)
    row_ptrs                                  (num_rows + 1 integers, blank separated)
    col_idxs                                  (num_nonzeros integers, blank separated, 0-based)

The reference parses it leniently (extra blanks are skipped, :30-33) and never validates it; this
reader validates what the kernels rely on (monotone row pointers ending at nnz, columns inside
the matrix and strictly ascending inside a row) because a pattern that breaks those would make a
device kernel read out of bounds.  Everything here is host-side integer work on numpy arrays; the
arrays it returns are what ``workloads.CSR`` and the operators take.
"""
from __future__ import annotations

import os

import numpy as np

from .workloads import CSR, swizzle_from_offsets


class SmtxError(ValueError):
    pass


def _ints(line: str, what: str, path: str) -> np.ndarray:
    try:
        return np.array([int(tok) for tok in line.split()], dtype=np.int64)
    except ValueError as e:
        raise SmtxError(f"{path}: {what} holds a token that is not an integer ({e})") from None


def read_smtx(path: str):
    """``(num_rows, num_cols, row_offsets int32 (m+1), column_indices int32 (nnz))``."""
    with open(path, "r") as f:
        lines = [ln for ln in f.read().split("\n")]
    while lines and lines[-1].strip() == "":
        lines.pop()
    if len(lines) < 2:
        raise SmtxError(f"{path}: expected 3 lines (header, row_ptrs, col_idxs), found {len(lines)}")
    header = [tok.strip() for tok in lines[0].strip().split(",")]
    if len(header) != 3:
        raise SmtxError(f"{path}: header must be 'num_rows, num_cols, num_nonzeros', got {lines[0]!r}")
    try:
        m, k, nnz = (int(tok) for tok in header)
    except ValueError:
        raise SmtxError(f"{path}: header must hold three integers, got {lines[0]!r}") from None
    if m < 0 or k < 0 or nnz < 0:
        raise SmtxError(f"{path}: negative size in header {lines[0]!r}")
    row_ptrs = _ints(lines[1], "row_ptrs", path)
    col_idxs = _ints(lines[2], "col_idxs", path) if len(lines) > 2 else np.zeros(0, np.int64)
    if len(lines) > 3:
        raise SmtxError(f"{path}: {len(lines) - 3} unexpected line(s) after col_idxs")
    if row_ptrs.shape[0] != m + 1:
        raise SmtxError(f"{path}: row_ptrs has {row_ptrs.shape[0]} entries, header says {m} rows")
    if col_idxs.shape[0] != nnz:
        raise SmtxError(f"{path}: col_idxs has {col_idxs.shape[0]} entries, header says {nnz} nonzeros")
    check_pattern(m, k, row_ptrs, col_idxs, path)
    return m, k, row_ptrs.astype(np.int32), col_idxs.astype(np.int32)


def check_pattern(m: int, k: int, row_offsets, column_indices, where: str = "pattern") -> None:
    """Raises :class:`SmtxError` unless the arrays form a canonical CSR pattern."""
    ro = np.asarray(row_offsets, dtype=np.int64)
    ci = np.asarray(column_indices, dtype=np.int64)
    if ro.shape[0] != m + 1 or ro[0] != 0 or ro[-1] != ci.shape[0]:
        raise SmtxError(f"{where}: row_ptrs must start at 0 and end at the number of nonzeros")
    if np.any(np.diff(ro) < 0):
        raise SmtxError(f"{where}: row_ptrs decrease at row {int(np.argmax(np.diff(ro) < 0))}")
    if ci.shape[0] >= 2 ** 31 or m >= 2 ** 31 or k >= 2 ** 31:
        raise SmtxError(f"{where}: sizes beyond int32")
    if ci.shape[0] == 0:
        return
    if ci.min() < 0 or ci.max() >= k:
        raise SmtxError(f"{where}: column index outside [0, {k})")
    same_row = np.ones(ci.shape[0] - 1, dtype=bool)
    starts = ro[1:-1]
    starts = starts[(starts > 0) & (starts < ci.shape[0])]
    same_row[starts - 1] = False                       # pairs that straddle a row boundary
    bad = same_row & (np.diff(ci) <= 0)
    if np.any(bad):
        j = int(np.argmax(bad))
        row = int(np.searchsorted(ro, j, side="right") - 1)
        raise SmtxError(f"{where}: column indices of row {row} are not strictly ascending")


def write_smtx(path: str, m: int, k: int, row_offsets, column_indices) -> None:
    """The three-line format above; ``read_smtx(write_smtx(x)) == x``."""
    check_pattern(m, k, row_offsets, column_indices, "write_smtx")
    ro = np.asarray(row_offsets, dtype=np.int64)
    ci = np.asarray(column_indices, dtype=np.int64)
    with open(path, "w") as f:
        f.write(f"{m}, {k}, {ci.shape[0]}\n")
        f.write(" ".join(map(str, ro.tolist())) + "\n")
        f.write(" ".join(map(str, ci.tolist())) + "\n")


def smtx_to_csr(path: str, seed: int = 0, sigma: float = 0.02) -> CSR:
    """Pattern from ``path`` with values N(0, sigma) drawn from ``seed`` (the files carry none;
    exact zeros are re-drawn so that nnz stays what the pattern says) and the row swizzle."""
    m, k, ro, ci = read_smtx(path)
    rng = np.random.default_rng(seed)
    values = (rng.standard_normal(ci.shape[0]) * sigma).astype(np.float32)
    small = np.abs(values) < 6.2e-5                     # would vanish or go subnormal in fp16
    values[small] = np.where(rng.random(int(small.sum())) < 0.5, -sigma, sigma).astype(np.float32)
    return CSR(m, k, values, swizzle_from_offsets(ro), ro, ci, {"source": os.path.basename(path), "seed": seed})


def generate_mtx_from_smtx(smtx_filename: str, seed: int | None = None) -> str:
    """Writes ``<name>.mtx`` beside ``<name>.smtx``: MatrixMarket coordinate real general, 1-based
    ``row col value`` lines in row-major order, values uniform in [0, 1) (benchmark/utils.py:35-44;
    the reference draws from the global ``random`` module, here a seed may be given).  Returns the
    path written."""
    m, k, ro, ci = read_smtx(smtx_filename)
    rng = np.random.default_rng(seed)
    values = rng.random(ci.shape[0])
    out = smtx_filename[: smtx_filename.rfind(".")] + ".mtx"
    rows = np.repeat(np.arange(m, dtype=np.int64), np.diff(ro.astype(np.int64)))
    with open(out, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n")
        f.write(f"{m} {k} {ci.shape[0]}\n")
        for r, c, v in zip(rows.tolist(), ci.tolist(), values.tolist()):
            f.write(f"{r + 1} {c + 1} {v!r}\n")
    return out


def find_smtx(root: str) -> list[str]:
    """Every ``.smtx`` below ``root``, sorted (the walk of benchmark/utils.py:54-60)."""
    found = []
    for d, _, files in os.walk(root):
        found.extend(os.path.join(d, f) for f in files if f.endswith(".smtx"))
    return sorted(found)
