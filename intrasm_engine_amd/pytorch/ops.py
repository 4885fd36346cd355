"""``torch.ops.iex_ops.*`` -- the operator registry of the path.

Same operator names, argument order, shape rules and error texts as the reference's
``TORCH_LIBRARY(iex_ops)`` (pytorch/csrc/extensions/sputnik_kernels.cpp:32-193); the
body of every operator is: validate, allocate the output with ``torch.empty`` on the
operand's device (so a surrounding graph capture routes it to the capture's pool),
look up torch's *current* stream (never an argument, sputnik_kernels.cpp:81,151) and
call the C ABI of ``libiex_hip.so``.  Nothing here computes on the CPU.

Registered operators
    spmm_sputnik_reuse_weight        fp32, values (nnz)                     [reference :173-175]
    spmm_sputnik_atomic              fp32, values (batch, nnz)              [reference :170-172]
    spmm_sputnik_reuse_weight_half   fp16, int16 or int32 column indices    [reference :179-181, unregistered there]
    sddmm_sputnik_atomic_upd_weight  fp32, output (nnz) summed over batch   [reference :182-184]
    sddmm_sputnik_half               fp16/bf16/fp32, output (batch, nnz)    [new: reference :185-187 is commented out]
    spmm_sputnik_batched_values      fp16/fp32, values (batch, nnz), written (not accumulated) [new]
    csr_softmax_                     in-place softmax over CSR rows         [new]
    gemm_mfma                        bf16/fp16 dense companion GEMM         [replaces torch.matmul / CUTLASS / Triton companions]
    fused_spmm_gemm                  single-launch sparse + dense           [new]
"""
from __future__ import annotations

import contextlib
import ctypes
import threading
import weakref

import torch

from .. import _lib

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}
_IT = {torch.int32: _lib.I32, torch.int16: _lib.I16}


_TUNING = threading.local()
_SPMM_KEYS = ("force_wpr", "force_variant", "force_rpw", "force_nt", "force_lpg")


@contextlib.contextmanager
def kernel_params(*, spmm: dict | None = None, sddmm: dict | None = None, gemm: dict | None = None):
    """Kernel choices for the operators called inside the block (this thread only), for tuning:
    ``spmm`` = any of force_variant / force_rpw / force_nt / force_lpg / force_wpr (the tuning
    bits of ``iex_spmm_ex``) and beside_gather_kernel (true: the calls will share the chip with a gather-bound launch,
    ``IEX_SPMM_BESIDE_GATHER_KERNEL``), ``sddmm`` = force_wpr / force_variant, ``gemm`` = tile (the shape code of
    ``iex_gemm``: 5 = 128x128, 6 = 128x256, 7 = 256x256 tiles, 8 = 128x128 and 9 = 64x128 by eight waves with K steps of 64, 10 = 128x256 by eight waves, 12 = 256x256 with K split over two workgroups per tile, 13 = 256x256 by eight waves in alternating phases, 14 = 64x128 with K split over two to eight workgroups per tile; 1..4 = the
    register-staged kernels).
    Without a block, or for a key left out, the library chooses; a category left out (None) keeps
    what an enclosing block set for it.  A kernel family that cannot
    take the operands at hand (a matrix-core family for an n that is not a multiple of 8, say)
    falls back to a gather kernel, as the C entry points document: results stay correct, the
    timing is then that of the fallback."""
    for name, given, known in (("spmm", spmm, _SPMM_KEYS + ("beside_gather_kernel",)), ("sddmm", sddmm, ("force_wpr", "force_variant")), ("gemm", gemm, ("tile",))):
        unknown = set(given or {}) - set(known)
        if unknown:
            raise TypeError(f"unknown {name} kernel parameters: {sorted(unknown)}")
    before = {k: getattr(_TUNING, k, None) for k in ("spmm", "sddmm", "gemm")}
    # only the categories that were passed are replaced: a nested block for one category keeps
    # what an outer block set for the others (an empty dict hands that category back to the library)
    for name, given in (("spmm", spmm), ("sddmm", sddmm), ("gemm", gemm)):
        if given is not None:
            setattr(_TUNING, name, given or None)
    try:
        yield
    finally:
        _TUNING.spmm, _TUNING.sddmm, _TUNING.gemm = before["spmm"], before["sddmm"], before["gemm"]


def _version(t) -> int:
    """In-place-change counter of a tensor; tensors created under ``torch.inference_mode()`` keep none (reading it
    raises) and cannot be changed in place either, so 0 serves."""
    if t.is_inference():
        return 0
    return t._version


def _chk(cond: bool, msg: str = "") -> None:
    if not cond:
        raise RuntimeError(msg or "Expected condition to be true (operator argument check failed)")


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _check_csr_common(first, row_indices, row_offsets, column_indices, names):
    """The dimension / device / contiguity / layout checks shared by both launcher
    macros (sputnik_kernels.cpp:41-79 and :109-149), same order and texts."""
    _chk(row_indices.dim() == 1)
    _chk(row_offsets.dim() == 1)
    _chk(column_indices.dim() == 1)
    tensors = list(names) + [("row_indices", row_indices), ("row_offsets", row_offsets),
                             ("column_offsets", column_indices)]
    for name, t in tensors:
        _chk(t.is_cuda, f"{name} must be a CUDA tensor")
    for name, t in tensors:
        _chk(t.is_contiguous(), f"{name} must be a contiguous tensor")
    for name, t in tensors:
        _chk(not t.is_sparse and t.layout == torch.strided, f"{name} must be a dense tensor")


def _check_index_dtypes(row_indices, row_offsets, column_indices, allow_i16=False):
    _chk(row_indices.dtype == torch.int32, "row_indices must be int32")
    _chk(row_offsets.dtype == torch.int32, "row_offsets must be int32")
    ok = (torch.int32, torch.int16) if allow_i16 else (torch.int32,)
    _chk(column_indices.dtype in ok, "column_indices must be " + " or ".join(str(d) for d in ok))


# From this share of nonzeros in dense blocks the kernels for patterns with structure are taken (SddmmPlan.analyze's
# rule).  A block counts as dense here from 2048 nonzeros (an eighth of 128 x 128): the kernels themselves lay a block
# out for the matrix cores from 1536, but a mask whose blocks all sit at that mark runs no faster through them than
# through the gather kernels (16 heads x 4096 x 4096, columns at random, MI355X: 10 % dense 172 against 151 us for the
# SDDMM, 166 against 147 for the SpMM; 20 % dense 172 against 286 and 164 against 278).
_STRUCTURE_SHARE = 0.5
_STRUCTURE_BLOCK_NONZEROS = 2048


def _row_histogram_host(row_offsets):
    """The 16 counts of ``iex_csr_row_histogram`` as a tuple of ints (one small launch, one synchronising read)."""
    hist = torch.zeros(16, dtype=torch.int32, device=row_offsets.device)
    with torch.cuda.device(row_offsets.device):
        rc = _lib.load().iex_csr_row_histogram(row_offsets.numel() - 1, row_offsets.data_ptr(), hist.data_ptr(),
                                               _stream_ptr(row_offsets.device))
    _lib.check(rc, "csr_row_histogram")
    return tuple(int(x) for x in hist.tolist())


def _share_scratch(lib, row_offsets, k):
    """Zeroed memory with which ``iex_csr_dense_share`` counts a block of rows by several workgroups (None: not needed)."""
    need = lib.iex_csr_dense_share_scratch_bytes(row_offsets.numel() - 1, int(k))
    return torch.zeros(need, dtype=torch.uint8, device=row_offsets.device) if need else None


def _dense_share_host(row_offsets, column_indices, k, dense_min=None):
    """Share of the nonzeros that sit in 128 x 128 blocks holding ``dense_min`` of them or more (``iex_csr_dense_share``;
    one small launch and a synchronising read), or None where the kernel does not apply (more than 65536 columns)."""
    nonzeros = column_indices.numel()
    if nonzeros == 0 or int(k) > 65536:
        return None
    dense_min = _STRUCTURE_BLOCK_NONZEROS if dense_min is None else dense_min
    count = torch.zeros(1, dtype=torch.int32, device=row_offsets.device)
    with torch.cuda.device(row_offsets.device):
        lib = _lib.load()
        scratch = _share_scratch(lib, row_offsets, k)
        rc = lib.iex_csr_dense_share(1 if column_indices.dtype == torch.int16 else 0, row_offsets.numel() - 1, int(k), nonzeros,
                                     row_offsets.data_ptr(), column_indices.data_ptr(), int(dense_min), count.data_ptr(),
                                     scratch.data_ptr() if scratch is not None else None, scratch.numel() if scratch is not None else 0,
                                     _stream_ptr(row_offsets.device))
    _lib.check(rc, "csr_dense_share")
    return int(count.item()) / nonzeros


def _pattern_tables_host(row_offsets, column_indices, k):
    """The tables and lists of the kernels for patterns with structure, written once (``iex_pattern_tables``) into a
    tensor that lives as long as the pattern's note; the stream is waited for, so every later call on any stream finds
    them complete and only reads them.  None where those kernels do not apply."""
    m, nonzeros = row_offsets.numel() - 1, column_indices.numel()
    lib = _lib.load()
    nbytes = lib.iex_pattern_tables_bytes(m, int(k), nonzeros) if column_indices.dtype == torch.int32 else 0
    if nbytes == 0:
        return None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=row_offsets.device)
    with torch.cuda.device(row_offsets.device):
        rc = lib.iex_pattern_tables(m, int(k), nonzeros, row_offsets.data_ptr(), column_indices.data_ptr(), ws.data_ptr(), nbytes,
                                    _stream_ptr(row_offsets.device))
        _lib.check(rc, "pattern_tables")
        torch.cuda.current_stream(row_offsets.device).synchronize()
    return ws


def _set_note(row_offsets, column_indices, k, status, hist, share=None):
    # (last field: the tables of the kernels for patterns with structure, made by the first call that wants them)
    column_indices.__dict__["_iex_csr"] = (weakref.ref(row_offsets), _version(row_offsets), _version(column_indices), int(k), status, hist, share,
                                           None)


def mark_canonical(row_offsets, column_indices, k, measure=True):
    """Record that ``(row_offsets, column_indices)`` is canonical CSR with ``k`` columns (what ``dense_to_sparse`` and
    ``transpose_info`` build), so that the operators need not look: see :func:`_pattern_note`.  Set-up code: reads the
    pattern's row-length histogram and the share of its nonzeros in dense blocks back (two small kernels, two
    synchronising reads).  ``measure=False`` skips that -- no kernel, no synchronisation, allowed under stream capture:
    for patterns that change from call to call (a mask made on the device every step) and are canonical by
    construction; the library's rules then go by the shape and the density alone."""
    hist = share = None
    if measure and row_offsets.is_cuda and row_offsets.numel() > 1:
        _, hist, share = _look(row_offsets, column_indices, k)      # (the check runs along: one launch more, no read more)
    _set_note(row_offsets, column_indices, k, 0, hist, share)
    return column_indices


def _pattern_note(row_offsets, column_indices, k):
    """``(status, histogram)`` of a pattern: the bits of ``iex_csr_check`` and the 16 counts of ``iex_csr_row_histogram``
    (rows with more than 64 << j nonzeros), or ``(None, None)`` when they are not known and cannot be found out now
    (a stream capture is running: looking ends in a synchronising read).

    The reference's kernels take the columns of a row in any order, and repeated (Sputnik: sputnik_spmm.cu.inc:229-243,
    sputnik_sddmm.cu.inc:137); most kernel families here are faster because they do not.  So every operator looks at a
    pattern the first time it sees it -- two small launches and one read -- and remembers the answer on the
    ``column_indices`` tensor object, together with the ``row_offsets`` object it belongs to and both version
    counters: a pattern costs one look, in-place changes and other pairings cost another.  The histogram lets the
    row kernel give every row the number of wavefronts its own length deserves (``iex_spmm_sched``)."""
    note = column_indices.__dict__.get("_iex_csr")
    if note is not None and note[0]() is row_offsets and note[1:4] == (_version(row_offsets), _version(column_indices), int(k)):
        return note[4], note[5]
    if torch.cuda.is_current_stream_capturing():
        return None, None
    status, hist, share = _look(row_offsets, column_indices, k)
    _set_note(row_offsets, column_indices, k, status, hist, share)
    return status, hist


def _look(row_offsets, column_indices, k):
    """One look at a pattern: ``iex_csr_check``, ``iex_csr_row_histogram`` and ``iex_csr_dense_share`` launched one after
    the other into one small buffer and read back at once (one synchronisation).  Histogram and share are None for a
    pattern whose offsets are unsound (the kernels cut such offsets to the arrays, so launching them is safe)."""
    for name, t in (("row_offsets", row_offsets), ("column_indices", column_indices)):
        _chk(t.is_cuda, f"{name} must be a CUDA tensor")
        _chk(t.is_contiguous(), f"{name} must be a contiguous tensor")
    _chk(row_offsets.dtype == torch.int32, "row_offsets must be int32")
    _chk(column_indices.dtype in (torch.int32, torch.int16), "column_indices must be int32 or int16")
    _chk(row_offsets.device == column_indices.device, "row_offsets should be in the same device as column_indices")
    _chk(row_offsets.numel() >= 1, "row_offsets must have m + 1 entries")
    m, nonzeros = row_offsets.numel() - 1, column_indices.numel()
    itype = 1 if column_indices.dtype == torch.int16 else 0
    buf = torch.zeros(18, dtype=torch.int32, device=row_offsets.device)      # status | 16 counts | nonzeros in dense blocks
    lib = _lib.load()
    with_share = nonzeros > 0 and int(k) <= 65536 and m > 0
    with torch.cuda.device(row_offsets.device):
        stream = _stream_ptr(row_offsets.device)
        _lib.check(lib.iex_csr_check(itype, m, int(k), nonzeros, row_offsets.data_ptr(), column_indices.data_ptr(), buf.data_ptr(), stream), "csr_check")
        if m > 0:
            _lib.check(lib.iex_csr_row_histogram(m, row_offsets.data_ptr(), buf.data_ptr() + 4, stream), "csr_row_histogram")
        if with_share:
            scratch = _share_scratch(lib, row_offsets, k)
            _lib.check(lib.iex_csr_dense_share(itype, m, int(k), nonzeros, row_offsets.data_ptr(), column_indices.data_ptr(),
                                               _STRUCTURE_BLOCK_NONZEROS, buf.data_ptr() + 68,
                                               scratch.data_ptr() if scratch is not None else None,
                                               scratch.numel() if scratch is not None else 0, stream), "csr_dense_share")
    got = buf.tolist()
    status = int(got[0])
    if status & _lib.CSR_BAD_OFFSETS:
        return status, None, None
    return status, tuple(int(x) for x in got[1:17]), (got[17] / nonzeros if with_share else None)


def _csr_status(row_offsets, column_indices, k):
    return _pattern_note(row_offsets, column_indices, k)[0]


def _known_dense_share(row_offsets, column_indices, k):
    """What an earlier look at the pattern found for the share of nonzeros in dense 128 x 128 blocks, or None."""
    note = column_indices.__dict__.get("_iex_csr")
    if note is not None and note[0]() is row_offsets and note[1:4] == (_version(row_offsets), _version(column_indices), int(k)):
        return note[6]
    return None


def _known_tables(row_offsets, column_indices, k):
    """The tables of the kernels for patterns with structure for a pattern that is known to be canonical: made by the
    first call that asks (never under stream capture: making them ends in a wait for the stream) and kept with the
    pattern's note.  None where nothing is known about the pattern, or the tables cannot be made now."""
    note = column_indices.__dict__.get("_iex_csr")
    if note is None or note[0]() is not row_offsets or note[1:4] != (_version(row_offsets), _version(column_indices), int(k)) or note[4] != 0:
        return None
    if note[7] is None and not torch.cuda.is_current_stream_capturing():
        tables = _pattern_tables_host(row_offsets, column_indices, k)
        if tables is not None:
            column_indices.__dict__["_iex_csr"] = note[:7] + (tables,)
        return tables
    return note[7]


def structured_tables(row_offsets, column_indices, k):
    """:func:`_known_tables` for a pattern whose look found structure (at least ``_STRUCTURE_SHARE`` of its nonzeros in
    dense blocks), None for any other."""
    share = _known_dense_share(row_offsets, column_indices, k)
    return _known_tables(row_offsets, column_indices, k) if share is not None and share >= _STRUCTURE_SHARE else None


def prepare_pattern(row_offsets, column_indices, k, tables=True):
    """Look at a pattern now (see :func:`_csr_status`) so that later calls -- under stream capture too, where nothing can
    be looked at -- take every kernel family for canonical CSR.  Returns the status bits; raises for offsets or columns
    that point outside the arrays.  Set-up code for patterns that do not come from ``dense_to_sparse``.
    ``tables``: also make, for a pattern with structure, the tables that the kernels for such patterns work from (an
    attention mask wants them; a weight matrix, whose products never take those kernels, does not: about 8 bytes a nonzero)."""
    status = _csr_status(row_offsets, column_indices, k)
    _chk(status is not None, "prepare_pattern: cannot look at a pattern while the current stream is being captured")
    _chk(not (status & (_lib.CSR_BAD_OFFSETS | _lib.CSR_COLUMN_OUT_OF_RANGE)),
         f"row_offsets must ascend from 0 to the number of nonzeros and every column index must lie in [0, {int(k)})")
    if tables and status == 0:
        structured_tables(row_offsets, column_indices, k)
    return status


def carry_pattern_note(column_indices, copy):
    """``copy`` holds the same column indices as ``column_indices`` (another integer type, a clone): what is known about
    the one holds for the other."""
    note = column_indices.__dict__.get("_iex_csr")
    if note is not None and note[2] == _version(column_indices):
        # (the tables were made from int32 indices: a copy of another integer type does not inherit them)
        copy.__dict__["_iex_csr"] = note[:2] + (_version(copy),) + note[3:7] + (note[7] if copy.dtype == column_indices.dtype else None,)
    return copy


def _any_order(row_offsets, column_indices, k, what):
    """True when the call must keep to the kernels that take columns in any order: the pattern is known to need it, or
    nothing is known about it.  Offsets or columns that point outside the arrays are refused: no kernel may follow them."""
    status = _csr_status(row_offsets, column_indices, k)
    if status is None:
        return True
    _chk(not (status & (_lib.CSR_BAD_OFFSETS | _lib.CSR_COLUMN_OUT_OF_RANGE)),
         f"{what}: row_offsets must ascend from 0 to the number of nonzeros and every column index must lie in [0, {int(k)})")
    return bool(status & _lib.CSR_NOT_ASCENDING)


def _spmm(b, row_indices, values, row_offsets, column_indices, m, *, per_batch_values,
          accumulate, dtypes, allow_i16, out=None, bias=None, relu=False, force_wpr=0, force_variant=0, force_rpw=0,
          force_nt=0, force_lpg=0, no_workspace=False, plan=None):
    tuned = getattr(_TUNING, "spmm", None)
    if tuned and not (force_wpr or force_variant or force_rpw or force_nt or force_lpg):
        force_wpr, force_variant, force_rpw, force_nt, force_lpg = (tuned.get(key, 0) for key in _SPMM_KEYS)
    beside_gather = bool(tuned and tuned.get("beside_gather_kernel"))
    if plan is not None and plan.variant and not force_variant:
        # settled by SddmmPlan.analyze(): the dense-blocks kernel for masks with structure (it still has to fit dtype and
        # shape: checked below), else the row kernel
        force_variant = 10 if plan.variant == 3 else 1
    _chk(b.dim() == 3)
    if per_batch_values:
        _chk(values.dim() == 2)
        _chk(b.size(0) == values.size(0))
        _chk(values.size(1) == column_indices.size(0))
    else:
        _chk(values.dim() == 1)
        _chk(values.size(0) == column_indices.size(0))
    _check_csr_common(b, row_indices, row_offsets, column_indices, [("b", b), ("values", values)])
    _chk(values.device == b.device, "values should be in the same device as b")
    _chk(values.device == row_indices.device, "a should be in the same device as row_indices")
    _chk(values.device == row_offsets.device, "a should be in the same device as row_offsets")
    _chk(values.device == column_indices.device, "a should be in the same device as column_indices")
    _chk(b.dtype in dtypes, f"b must be one of {dtypes}")
    _chk(values.dtype == b.dtype, "values must have the dtype of b")
    _check_index_dtypes(row_indices, row_offsets, column_indices, allow_i16)
    _chk(column_indices.dtype != torch.int16 or b.dtype == torch.float16, "int16 column_indices go with float16 values only")
    batch, k, n = b.shape
    nonzeros = column_indices.size(0)
    m = int(m)
    _chk(row_indices.size(0) == m, "row_indices must have m entries")
    _chk(row_offsets.size(0) == m + 1, "row_offsets must have m + 1 entries")
    if per_batch_values and accumulate:
        # the one shape rule of the reference that is about data, not layout (:87-89)
        _chk(batch == 1 or nonzeros % 4 == 0,
             "If batch size > 1 then number of nonzeros should be a multiple of 4")
    if out is None:
        # "atomic" store mode adds into the output; the reference leaves it uninitialised
        # (at::empty, :91) -- here the operator is defined as zero, then accumulate.
        out = (torch.zeros if accumulate else torch.empty)((batch, m, n), dtype=b.dtype, device=b.device)
    else:
        _chk(out.shape == (batch, m, n) and out.dtype == b.dtype and out.is_contiguous()
             and out.device == b.device, "out must be a contiguous (batch, m, n) tensor like b")
    if bias is not None:
        _chk(bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == m
             and bias.device == b.device, "bias must be a contiguous fp32 tensor with m entries")
    any_order = nonzeros > 0 and not force_variant and _any_order(row_offsets, column_indices, k, "spmm")
    if per_batch_values and not accumulate and not any_order and not force_variant and nonzeros > 0 and b.dtype in (torch.float16, torch.bfloat16):
        # values per batch entry = attention probabilities: the library's own rule for the dense-blocks kernel sees
        # the density only; what the first look at the pattern found about its structure decides here
        share = _known_dense_share(row_offsets, column_indices, k)
        if share is not None and batch * m * k >= (1 << 25):
            force_variant = 10 if share >= _STRUCTURE_SHARE else 1
            if force_variant == 10 and _lib.load().iex_spmm_workspace_kind(
                    _DT[b.dtype], _IT[column_indices.dtype], _lib.SPMM_PER_BATCH_VALUES | (10 << 16), m, k, n, nonzeros, batch) != 10:
                force_variant = 0      # (the kernel does not serve this call: another n, int16 indices)
    flags = (_lib.SPMM_PER_BATCH_VALUES if per_batch_values else 0) | (_lib.SPMM_ANY_COLUMN_ORDER if any_order else 0) | \
            (_lib.SPMM_BESIDE_GATHER_KERNEL if beside_gather else 0) | \
            (_lib.SPMM_ACCUMULATE if accumulate else 0) | (_lib.SPMM_RELU if relu else 0) | \
            ((int(force_wpr) & 0xff) << 8) | ((int(force_variant) & 0xf) << 16) | ((int(force_rpw) & 0xf) << 20) | \
            ((int(force_nt) & 0xf) << 24) | ({0: 0, 8: 1, 16: 2, 32: 3, 64: 4}[int(force_lpg)] << 28)
    lib = _lib.load()
    with torch.cuda.device(b.device):
        # room for the dense form of the sparse operand where the library would rather hand the
        # product to its dense GEMM (large 16-bit products): from torch's allocator, on the current
        # stream, released (stream-ordered) when this call returns
        shape = (_DT[b.dtype], _IT[column_indices.dtype], flags, m, k, n, nonzeros, batch)
        if plan is not None and plan.variant == 3 and ((flags >> 16) & 0xf) == 10 and lib.iex_spmm_workspace_kind(*shape) != 10:
            flags &= ~((0xf << 16) | (0xff << 8))      # the planned kernel does not serve this call (fp32, another n): the library's rule
            shape = shape[:2] + (flags,) + shape[3:]
        ws_bytes = 0 if no_workspace else lib.iex_spmm_workspace_bytes(*shape)
        if plan is not None and ws_bytes and lib.iex_spmm_workspace_kind(*shape) == 10:
            # the tables of the dense-blocks kernel depend on the pattern only and are those of the SDDMM for masks
            # with structure: a plan shared with that operator's calls on the pattern serves both
            key = (row_offsets.data_ptr(), column_indices.data_ptr(), _version(row_offsets), _version(column_indices),
                   m, k, nonzeros)
            if plan._ready(key, ws_bytes, b.device, (row_offsets, column_indices)):
                flags |= _lib.SPMM_TABLES_READY
                code = (flags >> 8) & 0xff if ((flags >> 16) & 0xf) == 10 else 0    # (what counts as a dense block: the lists depend on it)
                if plan.lists_key == (key, code):
                    flags |= _lib.SPMM_LISTS_READY
            plan.lists_key = (key, (flags >> 8) & 0xff if ((flags >> 16) & 0xf) == 10 else 0)
            ws = plan.workspace
        else:
            tables = _known_tables(row_offsets, column_indices, k) if ws_bytes and lib.iex_spmm_workspace_kind(*shape) == 10 and \
                (((flags >> 16) & 0xf) != 10 or ((flags >> 8) & 0xff) == 0) else None
            if tables is not None and tables.numel() >= ws_bytes and tables.device == b.device:
                # written when the pattern was first looked at, with the built-in threshold, and read-only since
                ws = tables
                flags |= _lib.SPMM_TABLES_READY | _lib.SPMM_LISTS_READY
            else:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=b.device) if ws_bytes else None
        # what is known about the pattern's row lengths (only what an earlier look left, unless the kernel that needs
        # it was asked for by name)
        if ((flags >> 16) & 0xf) == 11 and nonzeros > 0:
            _pattern_note(row_offsets, column_indices, k)
        note = column_indices.__dict__.get("_iex_csr")
        hist = note[5] if nonzeros > 0 and note is not None and note[0]() is row_offsets and \
            note[1:4] == (_version(row_offsets), _version(column_indices), int(k)) else None
        rc = lib.iex_spmm_sched(
            _DT[b.dtype], _IT[column_indices.dtype], flags, m, k, n, nonzeros,
            row_indices.data_ptr(), values.data_ptr(), row_offsets.data_ptr(),
            column_indices.data_ptr(), b.data_ptr(), bias.data_ptr() if bias is not None else None,
            out.data_ptr(), _stream_ptr(b.device), batch, ws.data_ptr() if ws is not None else None, ws_bytes,
            (ctypes.c_int * 16)(*hist) if hist is not None else None)
    _lib.check(rc, "spmm")
    return out


class SddmmPlan:
    """Memory that per-entry SDDMM calls on one CSR pattern (and the SpMM calls with per-entry values on the same pattern:
    the two products of sparse attention) keep between calls.

    The kernel for masks with structure (``iex_sddmm_ws``, variant 3) works from tables that a setup kernel derives
    from the pattern alone (m, n, row_offsets, column_indices).  A caller whose mask does not change passes the same
    plan to every call: the first call writes the tables and lists into the plan's workspace, later calls skip the setup
    kernels (``IEX_SDDMM_TABLES_READY``, ``IEX_SDDMM_LISTS_READY``).  The plan notices other index tensors, other shapes and in-place changes of the index
    tensors (their version counters) and then lets the tables be written again.  Calls that share a plan must be
    ordered on one stream (the workspace is theirs for the duration of the work)."""

    def __init__(self):
        self.workspace = None
        self.key = None
        self.lists_key = None   # (the lists behind the tables also depend on what counts as a dense block)
        self.variant = 0        # 0: the library's rule (by density); 1 / 3 after analyze()
        self._index_tensors = ()
        self.dense_share = None

    def analyze(self, row_offsets, column_indices, n, dense_min=None):
        """Look at the pattern once (copies the index arrays to the host: a synchronisation, so not under capture and
        not per call) and settle which kernel the plan's calls use: the one for masks with structure when at least
        half of the nonzeros sit in 128 x 128 blocks that hold ``dense_min`` or more of them, else the gather kernel.
        The library's own rule only knows the overall density, which a band and a random mask can share."""
        import numpy as np
        dense_min = _STRUCTURE_BLOCK_NONZEROS if dense_min is None else dense_min
        ro = row_offsets.detach().cpu().numpy().astype(np.int64)
        ci = column_indices.detach().cpu().numpy().astype(np.int64)
        m = ro.shape[0] - 1
        rows = np.repeat(np.arange(m, dtype=np.int64), np.diff(ro))
        tiles_n = (int(n) + 127) // 128
        counts = np.bincount((rows // 128) * tiles_n + np.minimum(ci // 128, tiles_n - 1), minlength=((m + 127) // 128) * tiles_n)
        self.dense_share = float(counts[counts >= dense_min].sum()) / max(1, ci.shape[0])
        self.variant = 3 if self.dense_share >= _STRUCTURE_SHARE else 1
        return self.variant

    def _ready(self, key, nbytes, device, index_tensors=()):
        """Workspace of nbytes for this key; True when it already holds the key's tables.  The plan keeps the index
        tensors of its key alive: the key names them by address and version, and an address that the allocator has
        handed to another tensor since would pass for the old pattern."""
        if self.workspace is None or self.workspace.numel() < nbytes or self.workspace.device != device:
            self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
            self.key = None
            self.lists_key = None
        ready = self.key == key
        self.key = key
        self._index_tensors = tuple(index_tensors)
        return ready


def _sddmm(a, b, row_indices, row_offsets, column_indices, *, sum_over_batch, dtypes,
           out=None, accumulate=False, force_wpr=0, force_variant=0, no_workspace=False, plan=None):
    tuned = getattr(_TUNING, "sddmm", None)
    if tuned and not (force_wpr or force_variant):
        force_wpr, force_variant = tuned.get("force_wpr", 0), tuned.get("force_variant", 0)
    if plan is not None and plan.variant and not force_variant:
        force_variant = plan.variant      # settled by SddmmPlan.analyze(); variant 3 still has to fit (dtype, k): checked below
    _chk(a.dim() == b.dim())
    _chk(a.dim() == 3)
    _chk(a.size(0) == b.size(0))
    _chk(a.size(2) == b.size(2))
    _check_csr_common(a, row_indices, row_offsets, column_indices, [("a", a), ("b", b)])
    _chk(a.device == b.device, "a should be in the same device as b")
    _chk(a.device == row_indices.device, "a should be in the same device as row_indices")
    _chk(a.device == row_offsets.device, "a should be in the same device as row_offsets")
    _chk(a.device == column_indices.device, "a should be in the same device as column_indices")
    _chk(a.dtype in dtypes, f"a must be one of {dtypes}")
    _chk(b.dtype == a.dtype, "b must have the dtype of a")
    _check_index_dtypes(row_indices, row_offsets, column_indices)
    batch, m, k = a.shape
    n = b.size(1)
    nonzeros = column_indices.size(0)
    _chk(row_indices.size(0) == m, "row_indices must have m entries")
    _chk(row_offsets.size(0) == m + 1, "row_offsets must have m + 1 entries")
    shape = (nonzeros,) if sum_over_batch else (batch, nonzeros)
    if out is None:
        out = torch.empty(shape, dtype=a.dtype, device=a.device)
    else:
        _chk(tuple(out.shape) == shape and out.dtype == a.dtype and out.is_contiguous()
             and out.device == a.device, "out has the wrong shape, dtype, layout or device")
    any_order = nonzeros > 0 and not force_variant and _any_order(row_offsets, column_indices, n, "sddmm")
    if not sum_over_batch and not accumulate and not any_order and not force_variant and nonzeros > 0 and a.dtype in (torch.float16, torch.bfloat16):
        # per-entry SDDMM = attention scores: by the pattern's structure where a look at it has told, not by its density
        share = _known_dense_share(row_offsets, column_indices, n)
        if share is not None and batch * m * n >= (1 << 25):
            force_variant = 3 if share >= _STRUCTURE_SHARE else 1
            if force_variant == 3 and _lib.load().iex_sddmm_workspace_kind(_DT[a.dtype], 3 << 16, m, k, n, nonzeros, batch) != 3:
                force_variant = 0      # (the kernel does not serve this call: another k)
    flags = (_lib.SDDMM_SUM_OVER_BATCH if sum_over_batch else 0) | (_lib.SDDMM_ANY_COLUMN_ORDER if any_order else 0) | \
            (_lib.SDDMM_ACCUMULATE if accumulate else 0) | ((int(force_wpr) & 0xff) << 8) | \
            ((int(force_variant) & 0xf) << 16)
    lib = _lib.load()
    if plan is not None and plan.variant == 3 and force_variant == 3 and \
            lib.iex_sddmm_workspace_kind(_DT[a.dtype], flags, m, k, n, nonzeros, batch) != 3:
        flags &= ~(0xf << 16)            # the planned kernel does not serve this call (fp32, another k): the library's rule
    with torch.cuda.device(a.device):
        # room for the dense product where the library would rather compute all of it on the matrix
        # cores and pick the nonzeros (16-bit, long k): from torch's allocator, on the current stream
        ws_bytes = 0 if no_workspace else lib.iex_sddmm_workspace_bytes(_DT[a.dtype], flags, m, k, n, nonzeros, batch)
        if plan is not None and ws_bytes and lib.iex_sddmm_workspace_kind(_DT[a.dtype], flags, m, k, n, nonzeros, batch) == 3:
            key = (row_offsets.data_ptr(), column_indices.data_ptr(), _version(row_offsets), _version(column_indices),
                   m, n, nonzeros)
            code = (flags >> 8) & 0xff if ((flags >> 16) & 0xf) == 3 else 0     # (what counts as a dense block: the lists depend on it)
            if plan._ready(key, ws_bytes, a.device, (row_offsets, column_indices)):
                flags |= _lib.SDDMM_TABLES_READY
                if plan.lists_key == (key, code):
                    flags |= _lib.SDDMM_LISTS_READY
            plan.lists_key = (key, code)
            ws = plan.workspace
        else:
            kind3 = ws_bytes and lib.iex_sddmm_workspace_kind(_DT[a.dtype], flags, m, k, n, nonzeros, batch) == 3
            tables = _known_tables(row_offsets, column_indices, n) if kind3 and (((flags >> 16) & 0xf) != 3 or ((flags >> 8) & 0xff) == 0) else None
            if tables is not None and tables.numel() >= ws_bytes and tables.device == a.device:
                # written when the pattern was first looked at, with the built-in threshold, and read-only since
                ws = tables
                flags |= _lib.SDDMM_TABLES_READY | _lib.SDDMM_LISTS_READY
            else:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
        rc = lib.iex_sddmm_ws(
            _DT[a.dtype], flags, m, k, n, nonzeros, row_indices.data_ptr(), row_offsets.data_ptr(),
            column_indices.data_ptr(), a.data_ptr(), b.data_ptr(), out.data_ptr(),
            _stream_ptr(a.device), batch, ws.data_ptr() if ws is not None else None, ws_bytes)
    _lib.check(rc, "sddmm")
    return out


# ----------------------------------------------------------------- operators
def spmm_sputnik_reuse_weight(b, row_indices, values, row_offsets, column_indices, m):
    return _spmm(b, row_indices, values, row_offsets, column_indices, m, per_batch_values=False,
                 accumulate=False, dtypes=(torch.float32,), allow_i16=False)


def spmm_sputnik_atomic(b, row_indices, values, row_offsets, column_indices, m):
    return _spmm(b, row_indices, values, row_offsets, column_indices, m, per_batch_values=True,
                 accumulate=True, dtypes=(torch.float32,), allow_i16=False)


def spmm_sputnik_reuse_weight_half(b, row_indices, values, row_offsets, column_indices, m):
    return _spmm(b, row_indices, values, row_offsets, column_indices, m, per_batch_values=False,
                 accumulate=False, dtypes=(torch.float16, torch.bfloat16), allow_i16=True)


def spmm_sputnik_batched_values(b, row_indices, values, row_offsets, column_indices, m):
    return _spmm(b, row_indices, values, row_offsets, column_indices, m, per_batch_values=True,
                 accumulate=False, dtypes=(torch.float32, torch.float16, torch.bfloat16),
                 allow_i16=True)


def spmm_batched_values_planned(b, row_indices, values, row_offsets, column_indices, m, plan: "SddmmPlan"):
    """``spmm_sputnik_batched_values`` for a caller that keeps an :class:`SddmmPlan` for the pattern (not a registered
    operator: the plan is a Python object).  The plan may be the one that the pattern's SDDMM calls use: the tables are
    the same, the SpMM keeps two lists of its own behind them."""
    return _spmm(b, row_indices, values, row_offsets, column_indices, m, per_batch_values=True,
                 accumulate=False, dtypes=(torch.float32, torch.float16, torch.bfloat16),
                 allow_i16=True, plan=plan)


def sddmm_sputnik_atomic_upd_weight(a, b, row_indices, row_offsets, column_indices):
    return _sddmm(a, b, row_indices, row_offsets, column_indices, sum_over_batch=True,
                  dtypes=(torch.float32,))


def sddmm_sputnik_half(a, b, row_indices, row_offsets, column_indices):
    return _sddmm(a, b, row_indices, row_offsets, column_indices, sum_over_batch=False,
                  dtypes=(torch.float32, torch.float16, torch.bfloat16))


def sddmm_half_planned(a, b, row_indices, row_offsets, column_indices, plan: SddmmPlan):
    """``sddmm_sputnik_half`` for a caller that keeps an :class:`SddmmPlan` for the pattern (not a registered operator:
    the plan is a Python object)."""
    return _sddmm(a, b, row_indices, row_offsets, column_indices, sum_over_batch=False,
                  dtypes=(torch.float32, torch.float16, torch.bfloat16), plan=plan)


def csr_check(row_offsets, column_indices, k):
    """What is wrong with a CSR pattern of ``k`` columns, as the bits of ``iex_csr_check`` (0 = canonical: offsets from 0
    to nnz ascending, columns inside [0, k) and strictly ascending inside a row -- what every kernel family but the
    row / gather kernels takes for granted, and what ``dense_to_sparse`` produces).  One small launch and a
    synchronising read of its result: for set-up code, not per call.  The reference's kernels take columns in any
    order (Sputnik), so a pattern from elsewhere is worth one check."""
    for name, t in (("row_offsets", row_offsets), ("column_indices", column_indices)):
        _chk(t.is_cuda, f"{name} must be a CUDA tensor")
        _chk(t.is_contiguous(), f"{name} must be a contiguous tensor")
    _chk(row_offsets.dtype == torch.int32, "row_offsets must be int32")
    _chk(column_indices.dtype in (torch.int32, torch.int16), "column_indices must be int32 or int16")
    _chk(row_offsets.device == column_indices.device, "row_offsets should be in the same device as column_indices")
    _chk(row_offsets.numel() >= 1, "row_offsets must have m + 1 entries")
    status = torch.zeros(1, dtype=torch.int32, device=row_offsets.device)
    with torch.cuda.device(row_offsets.device):
        rc = _lib.load().iex_csr_check(1 if column_indices.dtype == torch.int16 else 0, row_offsets.numel() - 1, int(k),
                                       column_indices.numel(), row_offsets.data_ptr(), column_indices.data_ptr(),
                                       status.data_ptr(), _stream_ptr(row_offsets.device))
    _lib.check(rc, "csr_check")
    return int(status.item())


def csr_softmax_(values, row_indices, row_offsets, scale):
    _chk(values.dim() == 2, "values must be (batch, nnz)")
    for name, t in (("values", values), ("row_indices", row_indices), ("row_offsets", row_offsets)):
        _chk(t.is_cuda, f"{name} must be a CUDA tensor")
        _chk(t.is_contiguous(), f"{name} must be a contiguous tensor")
    _chk(values.dtype in _DT, "values must be fp32, fp16 or bf16")
    _chk(row_indices.dtype == torch.int32 and row_offsets.dtype == torch.int32,
         "row_indices / row_offsets must be int32")
    m = row_indices.size(0)
    _chk(row_offsets.size(0) == m + 1, "row_offsets must have m + 1 entries")
    with torch.cuda.device(values.device):
        rc = _lib.load().iex_csr_softmax(_DT[values.dtype], m, values.size(1), row_indices.data_ptr(),
                                         row_offsets.data_ptr(), values.data_ptr(), float(scale),
                                         _stream_ptr(values.device), values.size(0))
    _lib.check(rc, "csr_softmax")
    return values


def gemm_mfma(a, b, trans_b=False, out=None):
    """``a @ b`` (or ``a @ b.T`` with ``trans_b``) for fp16/bf16, 2-D or batched 3-D."""
    _chk(a.is_cuda and b.is_cuda, "a and b must be CUDA tensors")
    _chk(a.dtype in (torch.float16, torch.bfloat16), "a must be fp16 or bf16")
    _chk(b.dtype == a.dtype, "b must have the dtype of a")
    _chk(a.device == b.device, "a should be in the same device as b")
    _chk(a.dim() in (2, 3) and b.dim() in (2, 3), "a and b must be 2-D or 3-D")
    _chk(a.is_contiguous(), "a must be a contiguous tensor")
    _chk(b.is_contiguous(), "b must be a contiguous tensor")
    M, K = a.shape[-2], a.shape[-1]
    N = b.shape[-2] if trans_b else b.shape[-1]
    _chk((b.shape[-1] if trans_b else b.shape[-2]) == K, "inner dimensions of a and b differ")
    batch = a.shape[0] if a.dim() == 3 else (b.shape[0] if b.dim() == 3 else 1)
    if a.dim() == 3 and b.dim() == 3:
        _chk(a.shape[0] == b.shape[0], "batch sizes of a and b differ")
    sa = M * K if a.dim() == 3 else 0
    sb = N * K if b.dim() == 3 else 0
    batched = a.dim() == 3 or b.dim() == 3
    shape = (batch, M, N) if batched else (M, N)
    if out is None:
        out = torch.empty(shape, dtype=a.dtype, device=a.device)
    else:
        _chk(tuple(out.shape) == shape and out.dtype == a.dtype and out.is_contiguous()
             and out.device == a.device, "out has the wrong shape, dtype, layout or device")
    with torch.cuda.device(a.device):
        tile = (getattr(_TUNING, "gemm", None) or {}).get("tile", 0)
        lib = _lib.load()
        code = int(bool(trans_b)) | ((int(tile) & 0xf) << 4)
        # room for the partial sums where the library would split K over two workgroups per tile (few tiles, long K)
        ws_bytes = lib.iex_gemm_workspace_bytes(_DT[a.dtype], code, M, N, K, batch)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
        rc = lib.iex_gemm_ws(_DT[a.dtype], code, M, N, K, a.data_ptr(), b.data_ptr(), out.data_ptr(), batch, sa, sb, M * N,
                             _stream_ptr(a.device), ws.data_ptr() if ws is not None else None, ws_bytes)
    _lib.check(rc, "gemm")
    return out


def fused_spmm_gemm(b, row_indices, values, row_offsets, column_indices, m, ga, gb, trans_b=False,
                    interleave=None):
    """One launch computing ``(A_csr @ b[0], ga @ gb)``; fp16 SpMM, fp16/bf16 GEMM (2-D, or
    3-D batched with equal batch sizes).
    ``interleave``: the order of the two kinds of workgroup in the grid, as ``iex_fused_spmm_gemm`` takes it (0: GEMM
    tiles first, g > 0: in groups of g through the grid, < 0: SpMM tiles first).  None: the kind with the longer inner
    dimension first -- a CU runs one tile at a time, the tiles of both kinds have the same outline and last as long as
    their inner dimension, and a schedule that starts its long tasks first ends soonest (config 4 on MI355X: SpMM
    tiles first 0.279 ms, GEMM tiles first 0.344 ms, in groups of 64 0.323 ms, against 0.325 ms for one after the other)."""
    _chk(b.dim() == 3 and b.size(0) == 1, "fused launch takes one batch entry")
    _chk(values.dim() == 1 and values.size(0) == column_indices.size(0))
    _check_csr_common(b, row_indices, row_offsets, column_indices, [("b", b), ("values", values)])
    _chk(b.dtype == torch.float16 and values.dtype == torch.float16, "fused SpMM operands must be fp16")
    _check_index_dtypes(row_indices, row_offsets, column_indices, allow_i16=True)
    _chk(ga.is_cuda and gb.is_cuda and ga.device == b.device and gb.device == b.device,
         "GEMM operands must be on the device of b")
    _chk(ga.dtype in (torch.float16, torch.bfloat16) and gb.dtype == ga.dtype, "GEMM operands must be fp16 or bf16")
    _chk(ga.dim() == gb.dim() and ga.dim() in (2, 3) and ga.is_contiguous() and gb.is_contiguous(),
         "GEMM operands must be contiguous, both 2-D or both 3-D")
    m = int(m)
    _chk(row_indices.size(0) == m and row_offsets.size(0) == m + 1, "CSR arrays do not match m")
    _, k, n = b.shape
    M, K = ga.shape[-2], ga.shape[-1]
    N = gb.shape[-2] if trans_b else gb.shape[-1]
    _chk((gb.shape[-1] if trans_b else gb.shape[-2]) == K, "inner dimensions of the GEMM differ")
    gbatch = ga.shape[0] if ga.dim() == 3 else 1
    _chk(ga.dim() == 2 or gb.shape[0] == gbatch, "batch sizes of the GEMM operands differ")
    _chk(column_indices.size(0) == 0 or not _any_order(row_offsets, column_indices, k, "fused_spmm_gemm"),
         "fused_spmm_gemm needs canonical CSR (columns of a row ascending and distinct) that has been seen outside a capture")
    if interleave is None:
        interleave = -1 if k >= K else 0
    out = torch.empty((1, m, n), dtype=b.dtype, device=b.device)
    c = torch.empty((gbatch, M, N) if ga.dim() == 3 else (M, N), dtype=ga.dtype, device=b.device)
    with torch.cuda.device(b.device):
        rc = _lib.load().iex_fused_spmm_gemm(
            _IT[column_indices.dtype], m, k, n, column_indices.size(0), row_indices.data_ptr(),
            values.data_ptr(), row_offsets.data_ptr(), column_indices.data_ptr(), b.data_ptr(),
            out.data_ptr(), _DT[ga.dtype], int(bool(trans_b)), M, N, K, ga.data_ptr(), gb.data_ptr(),
            c.data_ptr(), gbatch, M * K, N * K, M * N, int(interleave), _stream_ptr(b.device))
    _lib.check(rc, "fused_spmm_gemm")
    return out, c


_SPMM_SCHEMA = "(Tensor b, Tensor row_indices, Tensor values, Tensor row_offsets, Tensor column_indices, int m) -> Tensor"
_SDDMM_SCHEMA = "(Tensor a, Tensor b, Tensor row_indices, Tensor row_offsets, Tensor column_indices) -> Tensor"
_registered = False
_library = None


def register() -> None:
    """Define the operators under ``torch.ops.iex_ops`` (idempotent)."""
    global _registered, _library
    if _registered:
        return
    lib = torch.library.Library("iex_ops", "DEF")
    table = [
        ("spmm_sputnik_reuse_weight", _SPMM_SCHEMA, spmm_sputnik_reuse_weight),
        ("spmm_sputnik_atomic", _SPMM_SCHEMA, spmm_sputnik_atomic),
        ("spmm_sputnik_reuse_weight_half", _SPMM_SCHEMA, spmm_sputnik_reuse_weight_half),
        ("spmm_sputnik_batched_values", _SPMM_SCHEMA, spmm_sputnik_batched_values),
        ("sddmm_sputnik_atomic_upd_weight", _SDDMM_SCHEMA, sddmm_sputnik_atomic_upd_weight),
        ("sddmm_sputnik_half", _SDDMM_SCHEMA, sddmm_sputnik_half),
        ("csr_softmax_", "(Tensor(a!) values, Tensor row_indices, Tensor row_offsets, float scale) -> Tensor(a!)",
         csr_softmax_),
        ("gemm_mfma", "(Tensor a, Tensor b, bool trans_b=False) -> Tensor",
         lambda a, b, trans_b=False: gemm_mfma(a, b, trans_b)),
        ("fused_spmm_gemm",
         "(Tensor b, Tensor row_indices, Tensor values, Tensor row_offsets, Tensor column_indices, int m, "
         "Tensor ga, Tensor gb, bool trans_b=False, int? interleave=None) -> (Tensor, Tensor)",
         fused_spmm_gemm),
    ]
    for name, schema, fn in table:
        lib.define(name + schema)
        # one implementation for every backend: the body itself rejects non-device
        # tensors with the reference's message ("b must be a CUDA tensor")
        lib.impl(name, fn, "CompositeExplicitAutograd")
    _library = lib
    _registered = True
