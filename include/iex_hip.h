/*
 * libiex_hip.so -- C ABI of the gfx950 sparse-plus-dense GEMM path.
 *
 * Conventions (they replace the reference's launcher ABI, csrc/extensions.h:10-31):
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is allocated,
 *     freed or synchronised inside the library (except the iex_graph_* host objects);
 *   - `stream` is a hipStream_t passed as void* (NULL = the legacy default stream);
 *   - functions return 0 (hipSuccess) on success, a positive hipError_t when the HIP
 *     runtime refused something, or a negative IEX_ERR_* code when an argument is
 *     rejected before any launch; iex_last_error() holds the text of the last failure
 *     on the calling thread;
 *   - matrices are row-major and contiguous; the batch dimension is outermost;
 *   - a CSR matrix is (row_indices, values, row_offsets, column_indices): row_offsets
 *     has m+1 int32 entries, column_indices are ascending inside a row, row_indices is
 *     the scheduling swizzle (a permutation of 0..m-1, heavy rows first).  The swizzle
 *     only orders the work: output row r is always written from CSR row r.
 */
#ifndef IEX_HIP_H_
#define IEX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IEX_ABI_VERSION 1

/* element types of values / dense operands */
enum { IEX_F32 = 0, IEX_F16 = 1, IEX_BF16 = 2 };
/* element types of column_indices (IEX_I16: SpMM with IEX_F16 values only, the combination of the reference's
 * CudaSpmm5; every other product takes IEX_I32 and fails with IEX_ERR_UNSUPPORTED otherwise) */
enum { IEX_I32 = 0, IEX_I16 = 1 };

/* negative return codes (argument errors detected on the host) */
enum {
  IEX_ERR_BAD_ARGUMENT = -1,   /* null pointer, negative size, unknown enum */
  IEX_ERR_UNSUPPORTED = -2,    /* combination the library has no kernel for */
  IEX_ERR_TOO_LARGE = -3,      /* a dimension exceeds what the grid / index type can hold */
  IEX_ERR_STATE = -4           /* graph object used out of order */
};

int iex_abi_version(void);
/* Text of the most recent failure on this thread ("" when none). */
const char* iex_last_error(void);
/* Names (with template arguments) of the kernels that the most recent SpMM / SDDMM / GEMM / fused entry point
 * launched on this thread, joined by " + " ("" before the first call or when nothing was launched): what a
 * profile of the same call lists, read from the library instead of re-derived from its selection rules.
 * No counterpart in the reference. */
const char* iex_last_kernels(void);
/* 1 when a gfx950 device is visible to the HIP runtime, else 0. */
int iex_device_ok(void);

/* Does a CSR pattern meet what the faster kernel families take for granted?  ORs into *status (device memory,
 * an int that the caller has set to 0; the launch is asynchronous on `stream`):                              */
#define IEX_CSR_BAD_OFFSETS 0x1         /* row_offsets does not start at 0, end at nonzeros or ascend            */
#define IEX_CSR_COLUMN_OUT_OF_RANGE 0x2 /* a column index outside [0, k)                                         */
#define IEX_CSR_NOT_ASCENDING 0x4       /* columns of a row not strictly ascending (unsorted, or a duplicate)    */
/* Status 0 = canonical CSR: every SpMM / SDDMM family applies.  With IEX_CSR_NOT_ASCENDING alone the pattern is
 * still valid input for the row kernel and the SDDMM gather kernel (IEX_SPMM_FORCE_VARIANT(1),
 * IEX_SDDMM_FORCE_VARIANT(1)), as it is for the reference, whose Sputnik kernels take columns in any order; the
 * other families would compute something else without saying so.  One pass over the index arrays (a wavefront per
 * row).  itype = the type of column_indices (IEX_I32 or IEX_I16).  No counterpart in the reference. */
int iex_csr_check(int itype, int m, int k, int nonzeros, const int* row_offsets, const void* column_indices,
                  int* status, void* stream);

/* Row lengths of a pattern on a coarse scale, for iex_spmm_sched: adds to histogram[j] (device memory, 16 ints that the
 * caller has set to 0; the launch is asynchronous on `stream`) the number of rows with more than 64 << j nonzeros,
 * j = 0 .. 15.  A function of row_offsets alone; a caller reads it back once per pattern, as set-up.
 * No counterpart in the reference (its launchers know the mean row length only: nonzeros / m). */
int iex_csr_row_histogram(int m, const int* row_offsets, int* histogram, void* stream);

/* How much of a pattern sits in dense blocks: adds to *dense_nonzeros (device memory, an int that the caller has set
 * to 0; asynchronous on `stream`) the number of nonzeros that lie in 128 x 128 blocks (rows and columns counted from
 * 0 in steps of 128) holding at least dense_min of them.  The kernels for patterns with structure (SDDMM variant 3,
 * SpMM family 10) put such blocks on the matrix cores and count a block as dense from 1536 nonzeros; they pay off when
 * about half of the nonzeros or more sit in such blocks (bands, windows, block diagonals), whatever the overall
 * density -- which is all that the 0 = choose rule of those entry points can see.  A caller reads the figure back
 * once per pattern, as set-up, and forces the variant.  k <= 65536.  Offsets that point outside the arrays are cut to
 * [0, nonzeros] and columns outside [0, k) are counted nowhere, so the kernel may be launched together with
 * iex_csr_check and the two results read back at once.
 * scratch (device memory, may be NULL): with iex_csr_dense_share_scratch_bytes(m, k) bytes that the caller has set to
 * 0, a block of 128 rows is counted by several workgroups (a pattern of 4096 rows has 32 such blocks, and one
 * workgroup per block leaves seven eighths of the chip idle: 8.4 M nonzeros 130 us); without it, or with fewer bytes,
 * by one.  The call may overwrite the scratch memory until the work it puts on `stream` has run; the counts are the
 * same either way.  iex_csr_dense_share_scratch_bytes returns 0 where one workgroup per block fills the chip anyway.
 * No counterpart in the reference. */
int iex_csr_dense_share(int itype, int m, int k, int nonzeros, const int* row_offsets, const void* column_indices,
                        int dense_min, int* dense_nonzeros, void* scratch, size_t scratch_bytes, void* stream);
size_t iex_csr_dense_share_scratch_bytes(int m, int k);

/* dst[0:nbytes] = src[0:nbytes] with a plain 128-bit-per-lane streaming kernel (nbytes and both
 * pointers multiples of 16).  Measurement aid with no counterpart in the reference: hardware
 * traffic counters are scaled by what they read for this copy of known size. */
int iex_copy_bytes(void* dst, const void* src, size_t nbytes, void* stream);

/* ------------------------------------------------------------------ SpMM ---- */
/* flags for iex_spmm_ex */
#define IEX_SPMM_PER_BATCH_VALUES 0x1 /* values is (batch, nnz) instead of (nnz)            */
#define IEX_SPMM_ACCUMULATE 0x2       /* out += A*b (reference "atomic" store mode)         */
#define IEX_SPMM_RELU 0x4             /* out = max(0, A*b + bias)                           */
/* iex_spmm_ws, family 10 only (ignored elsewhere): the workspace still holds the tables that an earlier
 * call with the same m, k, nonzeros and index arrays wrote there -- a family-10 SpMM, or an SDDMM of
 * variant 3 on the same pattern (iex_sddmm_ws with n = this call's k): the tables are the same.   */
#define IEX_SPMM_TABLES_READY 0x8
/* ... and the lists that family 10 itself derives from the tables (which blocks count as dense, the nonzeros
 * outside them) are still there too, from a family-10 call with the same bits 8..15.  Only with
 * IEX_SPMM_TABLES_READY.                                                                              */
#define IEX_SPMM_LISTS_READY 0x10
/* The column indices of a row may come in any order and repeat (what the reference's Sputnik kernels accept,
 * sputnik_spmm.cu.inc:229-243): with nothing forced the call keeps to the families that take such input (1 and 8).
 * The drop-ins iex_CudaSpmm2 / 3 / 5 below always set it: they know nothing about where their arrays come from.
 * Ignored when bits 16..19 force a family.                                                             */
#define IEX_SPMM_ANY_COLUMN_ORDER 0x20
/* The launch will share the chip with a launch that is bound by gathers from L2 (the row kernel on a parallel branch
 * of a graph or on another stream).  Where the fp32 matrix-core kernel (family 5) and the row kernel are close for this
 * product (fp32, int32 indices, density from 19.5 %, n a multiple of 4 from 128 up; alone the matrix-core kernel is 5-7 %
 * slower there and the library would not take it) the call then runs on the matrix cores and leaves the L2 -> CU path to
 * its neighbour: the config-2 sweep on two branches 654 -> 600 us on MI355X.  The reference pairs kernels of different
 * units by hand (tests/test_interleaving.py:434-476); this is the same choice, made by the callee.  Ignored when bits
 * 16..19 force a family, with IEX_SPMM_ANY_COLUMN_ORDER, and for every other element type.                      */
#define IEX_SPMM_BESIDE_GATHER_KERNEL 0x40
/* bits 8..15: force waves-per-row (1, 4 or 8); 0 = choose from nnz/m.  For tuning.    */
#define IEX_SPMM_FORCE_WPR(w) (((w) & 0xff) << 8)
/* bits 16..19: force the kernel family: 1 = row kernel gathering from L2, 2 = LDS-staged
 * gather, 3 / 4 = matrix-core kernels (fp16 / bf16: A expanded to dense tiles in LDS; 4 waves
 * and 128 x 256 tiles / 8 waves and 128 x 512 tiles), 5 = matrix-core kernel for fp32
 * (v_mfma_f32_32x32x2, 32-row tiles), 6 = family 4's tile with the dense operand loaded from
 * global memory straight into LDS and A expanded 64 columns at a time (fp16 / bf16), 7 = dense
 * form of A in the caller's workspace, then the dense GEMM (iex_spmm_ws only), 8 = A with at most
 * 128 columns and an output at least one tile (64 128-bit vectors) wide: the dense operand's tile
 * in LDS, rows streamed in natural order (bit-equal to family 1 with one wavefront per row; fails
 * on other shapes), 9 = unused,
 * 10 = sparse operands with structure (attention probabilities: bands, blocks, windows) times a dense
 * operand of 64, 128, ... columns (served 64 at a time): per 128 rows, the dense 128 x 128 blocks of A are laid out in LDS and
 * multiplied on the matrix cores, the nonzeros elsewhere are gathered row by row (fp16 / bf16, int32 indices,
 * n a multiple of 64 up to 1024, k <= 65536, plain store without bias or ReLU, values shared or per batch entry;
 * chosen by itself for values per batch entry on patterns at least 3 % dense with batch * m * k >= 2^25, on request
 * elsewhere; iex_spmm_ws only, with
 * the workspace iex_spmm_workspace_bytes reports: the tables of SDDMM variant 3 for the pattern, which a small
 * kernel writes first, and behind them lists that one more small kernel derives from the tables -- see
 * IEX_SPMM_TABLES_READY / IEX_SPMM_LISTS_READY; bits 8..15 set the number of nonzeros from which a block counts
 * as dense: 0 = built in (1536), 1 = every block, 255 = none, else 64 * value); fails on other shapes.
 * 0 = choose.
 * 11 = the row kernel with wavefronts per row by the row's own length (iex_spmm_sched only: see there).
 * Families 2-6 and 10 rely on strictly ascending column indices inside a row (canonical CSR, what
 * dense_to_sparse produces); family 1 accepts any order and duplicates -- force it for such
 * input.  Families 3-6 and 10 multiply explicit zeros with the dense operand, so a non-finite entry
 * in a row of `dense` that no nonzero references still reaches the output (0 * inf = NaN).
 * bits 20..23: rows per wavefront of family 2 (2, 4 or 8); windows of nonzeros held in
 * registers per row of family 4 (1, 2, 4 or 5 windows of 16), 5 (2, 4 or 8 windows of 8) and
 * 6 (1, 2 or 4 windows of 16).  0 = choose.                                              */
#define IEX_SPMM_FORCE_VARIANT(v) (((v) & 0xf) << 16)
#define IEX_SPMM_FORCE_RPW(r) (((r) & 0xf) << 20)
/* bits 24..27: adjacent 64-lane column tiles per wavefront of the row kernel (1 or 2); tile
 * arrangement of family 5 (1 = 32 x 64, 2 = 32 x 128 as two 64-column waves, 4 = 32 x 128,
 * 5 = 16 x 64, 6 = 16 x 128 as two 64-column waves).                                        */
#define IEX_SPMM_FORCE_NT(t) (((t) & 0xf) << 24)
/* bits 28..30: lanes per nonzero of the row kernel, coded 1..4 = 8, 16, 32, 64 lanes; for
 * family 3 the lanes that share a row during expansion (8 or 16); for family 5 code 1 turns
 * the separate expanding wavefronts off (every wave then expands and multiplies in turn).  */
#define IEX_SPMM_FORCE_LPG_CODE(c) (((c) & 0x7) << 28)

/* out[z, r, :] = sum_j values[(z,) j] * dense[z, column_indices[j], :]  (+ bias[r], ReLU)
 * dense is (batch, k, n), out is (batch, m, n), both of `dtype`; accumulation is fp32.
 * bias (fp32, length m) may be NULL.
 * Generalises CudaSpmmBiasRelu (sputnik_spmm_host_func.cu.inc:118-204). */
int iex_spmm_ex(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                const int* row_indices, const void* values, const int* row_offsets,
                const void* column_indices, const void* dense, const float* bias,
                void* out, void* stream, int batch);

/* iex_spmm_ex with a workspace in device memory that the call may use (and overwrite) until the
 * work it puts on `stream` has run.  With `workspace_bytes` >= iex_spmm_workspace_bytes(...) and a
 * 16-byte aligned `workspace`, fp16 / bf16 products that would run on a matrix-core SpMM kernel
 * (families 3, 4, 6) instead write the dense form of A (m * k * 2 bytes) into the workspace and
 * hand it to the dense GEMM (iex_gemm): the matrix-core SpMM kernels rebuild the dense form of
 * their rows of A in LDS once per column tile of the output, the GEMM reads it ready-made (family
 * 7; the caveat of families 3-6 about explicit zeros holds, and column indices inside a row must
 * be distinct).  Needs values shared by the batch and k and n multiples of 8 (bias, ReLU and
 * accumulation ride in the GEMM's epilogue); anything else, and a NULL or short workspace, runs
 * exactly as iex_spmm_ex.  Where the product has few tiles and a long k (iex_gemm_ws) the size asked for includes,
 * behind the dense form rounded up to 256 bytes, the room the GEMM wants for splitting k over several workgroups per
 * tile; a 16-byte aligned workspace of m * k * 2 bytes still runs the path, without the split.
 * IEX_SPMM_FORCE_VARIANT(7) asks for that path and fails where it cannot run.
 * iex_spmm_workspace_bytes returns the size with which the call described would use the workspace,
 * 0 when it would not whatever the size.  Neither call allocates.
 * No counterpart in the reference: its launchers (csrc/extensions.h:28-30) take no workspace. */
int iex_spmm_ws(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                const int* row_indices, const void* values, const int* row_offsets,
                const void* column_indices, const void* dense, const float* bias,
                void* out, void* stream, int batch, void* workspace, size_t workspace_bytes);
size_t iex_spmm_workspace_bytes(int dtype, int itype, int flags, int m, int k, int n,
                                int nonzeros, int batch);
/* iex_spmm_ws for a caller that knows the pattern's row lengths: `row_histogram` is HOST memory, the 16 counts of
 * iex_csr_row_histogram for row_offsets (NULL: exactly iex_spmm_ws).  Where the call runs on the row kernel (family 1)
 * with full 128-bit vectors and would split rows over wavefronts, the split then follows each row's own length
 * instead of the mean (the reference's remedy for uneven rows is the swizzle alone, sputnik_spmm.cu.inc:109-114):
 * row_indices lists the rows by decreasing length, so the rows that get 16, 8, 4, 2 wavefronts and 1 are five
 * consecutive ranges of it, a workgroup of 16 wavefronts serves 1, 2, 4, 8 or 16 rows of one range, and the partial
 * sums of a row meet in LDS in a fixed order (no atomics: same bits from call to call).  The histogram and the
 * order of row_indices settle how many wavefronts a row HAS; into how many parts its sum is cut follows from the
 * row's own length, and a row with fewer wavefronts than parts lets one of them take all the parts.  So every row is
 * summed completely, and to the same bits, whatever the histogram and whatever the order of row_indices: a wrong
 * histogram or another order costs time only.  IEX_SPMM_FORCE_VARIANT(11) asks for this kernel and fails without a histogram
 * (bits 20..23 then force the chunks of 64 nonzeros a wavefront may get: 1 + log2, 0 = choose).
 * No counterpart in the reference. */
int iex_spmm_sched(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                   const int* row_indices, const void* values, const int* row_offsets,
                   const void* column_indices, const void* dense, const float* bias,
                   void* out, void* stream, int batch, void* workspace, size_t workspace_bytes,
                   const int* row_histogram);
/* What that workspace would hold: 0 = nothing (not used), 7 = the dense form of A,
 * 10 = the tables and lists of family 10 (functions of the pattern only: a caller that keeps the workspace for a
 * pattern may say so with IEX_SPMM_TABLES_READY / IEX_SPMM_LISTS_READY on later calls). */
int iex_spmm_workspace_kind(int dtype, int itype, int flags, int m, int k, int n, int nonzeros, int batch);

/* iex_spmm_ws for callers that cannot allocate device memory (code under hipGraph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments as iex_spmm_ex, same results as iex_spmm_ws with a
 * workspace of the size iex_spmm_workspace_bytes asks for, but the workspace is an array of
 * IEX_SPMM_STATIC_SCRATCH_BYTES that the library itself holds on every GPU it runs on, from the moment the
 * library is loaded there until the process ends.  The call allocates and frees nothing (the first call on a
 * device looks the array's address up once).  A call whose workspace would exceed the array fails with
 * IEX_ERR_TOO_LARGE before anything is launched; a call that would not use a workspace runs as iex_spmm_ex.
 * All calls on one GPU share that GPU's array: two calls whose work may overlap in time (different streams,
 * different threads) race on it -- order them, or give one of them iex_spmm_ws with memory of its own.  The
 * array keeps the previous call's contents; every kernel that reads it writes what it reads first
 * (IEX_SPMM_TABLES_READY / IEX_SPMM_LISTS_READY are ignored here: the array is nobody's to keep).
 * No counterpart in the reference (its launchers take no workspace, csrc/extensions.h:28-30). */
#define IEX_SPMM_STATIC_SCRATCH_BYTES ((size_t)96 << 20)
int iex_spmm_static(int dtype, int itype, int flags, int m, int k, int n, int nonzeros,
                    const int* row_indices, const void* values, const int* row_offsets,
                    const void* column_indices, const void* dense, const float* bias,
                    void* out, void* stream, int batch);
size_t iex_spmm_static_scratch_bytes(void);

/* Drop-ins for the three launchers the reference declares in csrc/extensions.h:28-30.  Like the reference's they accept
 * column indices in any order inside a row, and duplicates (IEX_SPMM_ANY_COLUMN_ORDER is always set: the row kernel,
 * or the few-columns kernel); a caller that knows its CSR arrays to be canonical gets every family from iex_spmm_ex.
 * CudaSpmm2: fp32, per-batch values (batch, nnz), accumulates into `out`
 *            (spmm_sputnik_atomic, sputnik_kernels.cpp:170-172);
 * CudaSpmm3: fp32, values shared by the batch (spmm_sputnik_reuse_weight, :173-175);
 * CudaSpmm5: fp16 values / dense / out, int16 column indices, values shared
 *            (spmm_sputnik_reuse_weight_half, :179-181). */
int iex_CudaSpmm2(int m, int k, int n, int nonzeros, const int* row_indices,
                  const float* values, const int* row_offsets, const int* column_indices,
                  const float* dense_matrix, float* output_matrix, void* stream,
                  int batch_size);
int iex_CudaSpmm3(int m, int k, int n, int nonzeros, const int* row_indices,
                  const float* values, const int* row_offsets, const int* column_indices,
                  const float* dense_matrix, float* output_matrix, void* stream,
                  int batch_size);
int iex_CudaSpmm5(int m, int k, int n, int nonzeros, const int* row_indices,
                  const uint16_t* values, const int* row_offsets,
                  const int16_t* column_indices, const uint16_t* dense_matrix,
                  uint16_t* output_matrix, void* stream, int batch_size);

/* ----------------------------------------------------------------- SDDMM ---- */
#define IEX_SDDMM_SUM_OVER_BATCH 0x1 /* one (nnz) output summed over the batch            */
#define IEX_SDDMM_ACCUMULATE 0x2     /* out += ... instead of out = ...                   */
/* iex_sddmm_ws, variant 3 only (ignored elsewhere): the workspace still holds the tables that an
 * earlier call with the same m, n, nonzeros and index arrays (and a kind-3 workspace) wrote there;
 * the kernel that writes them is skipped.  For callers whose mask does not change from call to call. */
#define IEX_SDDMM_TABLES_READY 0x4
/* ... and the lists that variant 3 derives from the tables (which blocks count as dense, the nonzeros outside them)
 * are still there too, from a call with the same bits 8..15 -- of iex_sddmm_ws, or of iex_spmm_ws family 10 on the same
 * pattern: the lists are the same.  Only with IEX_SDDMM_TABLES_READY.                                              */
#define IEX_SDDMM_LISTS_READY 0x8
/* The column indices of a row may come in any order and repeat (sputnik_sddmm.cu.inc:137 reads them as they come):
 * with nothing forced the call keeps to the gather kernel and the dense-product path, which take such input.
 * Ignored when bits 16..19 force a variant.                                                            */
#define IEX_SDDMM_ANY_COLUMN_ORDER 0x10
/* bits 8..15: force wavefronts per row (1 or 4); 0 = choose from nnz/m.  For tuning.
 * With variant 3 the same bits set the number of nonzeros from which a 128 x 128 block of the
 * mask counts as dense: 0 = built in, 1 = every block, 255 = none, else 64 * value.       */
#define IEX_SDDMM_FORCE_WPR(w) (((w) & 0xff) << 8)
/* bits 16..19: 1 = the gather kernel; 3 = the kernel for masks with structure (attention: bands,
 * blocks, windows): per 128 rows, the dense 128 x 128 blocks of the mask get their scores from the
 * matrix cores, sampled inside the workgroup and never stored, the nonzeros elsewhere one dot
 * product each (fp16 / bf16, k = 32, 64 or 128, n <= 65536, plain store, one output per batch
 * entry, strictly ascending columns inside a row; iex_sddmm_ws only: the workspace holds
 * (6 ceil(n / 128) + 1) * m words of tables -- per row and block of columns a cursor, a packed word and a
 * 128-bit mask -- and behind them 2 * nonzeros + m words and a few more of lists -- the dense blocks
 * of every 128 rows, the nonzeros outside them row by row -- that two small kernels write first, once
 * for all batch entries: iex_sddmm_workspace_bytes gives the total); 7 = dense
 * product in the caller's workspace, then sampling (iex_sddmm_ws only).
 * 3 and 7 fail where they cannot run.  0 = choose: 3 when the mask is at least 3 % dense and
 * batch * m * n is at least 2^25, else 7 or 1 by a time model.                              */
#define IEX_SDDMM_FORCE_VARIANT(v) (((v) & 0xf) << 16)

/* out[(z,) j] = sum_c lhs[z, row(j), c] * rhs[z, column_indices[j], c]
 * lhs is (batch, m, k), rhs is (batch, n, k) -- rhs rows are the sampled columns.
 * out is (nnz) with IEX_SDDMM_SUM_OVER_BATCH, else (batch, nnz); fp32 accumulation.
 * Generalises CudaSddmm2 (sputnik_sddmm.cu.inc:206-233) to fp16 and per-batch output. */
int iex_sddmm_ex(int dtype, int flags, int m, int k, int n, int nonzeros,
                 const int* row_indices, const int* row_offsets, const int* column_indices,
                 const void* lhs_matrix, const void* rhs_matrix, void* output_values,
                 void* stream, int batch);

/* iex_sddmm_ex with a workspace in device memory that the call may use (and overwrite) until
 * the work it puts on `stream` has run.  With `workspace_bytes` >= iex_sddmm_workspace_bytes(...)
 * and a 16-byte aligned `workspace`, fp16 / bf16 calls with a long k and a mask that is not very
 * sparse compute the whole product lhs * rhs^T (m * n * 2 bytes per batch entry, one entry at a
 * time) with the dense GEMM and pick the nonzeros' entries: the gather kernel reads k * 2 bytes of
 * rhs per nonzero, which costs more than all m * n dot products on the matrix cores (weight
 * gradients of a sparse linear layer: k = tokens).  Same arithmetic per output (fp32 accumulation,
 * one rounding).  Needs plain store, (batch, nnz) output or batch 1, k and n multiples of 8;
 * anything else, and a NULL or short workspace, runs exactly as iex_sddmm_ex.
 * The workspace also serves variant 3 above (short k, masks with structure), which 0 = choose picks first.
 * iex_sddmm_workspace_bytes returns the size with which the call described would use the
 * workspace, 0 when it would not whatever the size.  Neither call allocates.
 * No counterpart in the reference: CudaSddmm2 (csrc/extensions.h:31) takes no workspace. */
int iex_sddmm_ws(int dtype, int flags, int m, int k, int n, int nonzeros,
                 const int* row_indices, const int* row_offsets, const int* column_indices,
                 const void* lhs_matrix, const void* rhs_matrix, void* output_values,
                 void* stream, int batch, void* workspace, size_t workspace_bytes);
size_t iex_sddmm_workspace_bytes(int dtype, int flags, int m, int k, int n, int nonzeros, int batch);
/* What the workspace would hold: 0 = nothing (not used), 3 = the tables of variant 3 (a function of m, n
 * and the index arrays only: see IEX_SDDMM_TABLES_READY), 7 = the dense product. */
int iex_sddmm_workspace_kind(int dtype, int flags, int m, int k, int n, int nonzeros, int batch);

/* The tables and lists that SDDMM variant 3 and SpMM family 10 derive from a pattern (m rows, n columns: the SpMM's k),
 * written into the caller's workspace by their two setup kernels, with the built-in threshold for dense blocks: for a
 * caller that prepares a pattern once, waits for the stream, and then passes the workspace with both READY flags
 * (IEX_SDDMM_TABLES_READY | IEX_SDDMM_LISTS_READY, IEX_SPMM_TABLES_READY | IEX_SPMM_LISTS_READY) to every call on the
 * pattern -- the workspace is only read from then on, so calls on different streams may share it.
 * iex_pattern_tables_bytes: the size (what iex_sddmm_workspace_bytes reports for variant 3 and
 * iex_spmm_workspace_bytes for family 10 on the pattern), 0 where those kernels do not apply (n > 65536).
 * int32 column indices, strictly ascending inside a row.  No counterpart in the reference. */
size_t iex_pattern_tables_bytes(int m, int n, int nonzeros);
int iex_pattern_tables(int m, int n, int nonzeros, const int* row_offsets, const int* column_indices, void* workspace,
                       size_t workspace_bytes, void* stream);

/* Drop-in for CudaSddmm2 (csrc/extensions.h:31; sddmm_sputnik_atomic_upd_weight,
 * sputnik_kernels.cpp:182-184): fp32, output (nnz) = sum over the batch, written
 * (not accumulated), so the caller need not zero it. */
int iex_CudaSddmm2(int m, int k, int n, int nonzeros, const int* row_indices,
                   const int* row_offsets, const int* column_indices,
                   const float* lhs_matrix, const float* rhs_matrix, float* output_values,
                   void* stream, int batch_size);

/* In-place row-wise softmax over the stored entries of a CSR matrix:
 * values[z, j] = exp(scale*values[z, j] - max_row) / sum_row.  values is (batch, nnz).
 * The middle step of sparse attention between SDDMM and SpMM (no reference
 * counterpart in tree; the reference leaves it to xformers). */
int iex_csr_softmax(int dtype, int m, int nonzeros, const int* row_indices,
                    const int* row_offsets, void* values, float scale, void* stream,
                    int batch);

/* ------------------------------------------------------------------ GEMM ---- */
/* C[z] = A[z] * B[z] (trans_b == 0, B is (K,N)) or A[z] * B[z]^T (trans_b == 1, B is
 * (N,K), the torch.nn.Linear weight layout used by MyLinear, layers_and_funcs/torch.py:17).
 * dtype is IEX_F16 or IEX_BF16 for A, B and C; accumulation is fp32 on the matrix cores.
 * stride_* are element strides between batch entries (0 = operand shared by the batch).
 * Bits 4..7 of trans_b force the kernel for tuning: 5 = 128x128, 6 = 128x256, 7 = 256x256 tiles,
 * 8 = 128x128 and 9 = 64x128 by eight waves with K steps of 64 (few tiles, long K), 10 = 128x256 by eight waves
 * (11: with K steps of 64), 12 = 256x256 with K split over two workgroups per tile (iex_gemm_ws only), 13 = 256x256 by
 * eight waves in two groups that take turns: one reads operand fragments and issues loads while the other multiplies,
 * 14 = 64x128 by eight waves with K split over two to eight workgroups per tile (iex_gemm_ws only),
 * all with the operands loaded from global memory straight into LDS (0 = choose picks among 5, 8, 9, 10 and 13, and
 * 14 where iex_gemm_ws got the room iex_gemm_workspace_bytes asks for);
 * 1 = 128x128, 2 = 128x256, 3 = 256x256, 4 = 128x128 with K steps of 64, operands staged through
 * registers.  K % 8 == 0, N % 8 == 0 for a (K,N) B, 16-byte aligned operands.
 * Replaces the cuBLAS / CUTLASS / Triton companions of tests/test_interleaving.py:26-345. */
int iex_gemm(int dtype, int trans_b, int M, int N, int K, const void* A, const void* B,
             void* C, int batch, long long stride_a, long long stride_b,
             long long stride_c, void* stream);

/* iex_gemm with a workspace in device memory that the call may use (and overwrite) until the work it
 * puts on `stream` has run.  Used by the kernels that split K over several workgroups per tile.
 * Shape code 14 (bits 4..7 of trans_b): 64 x 128 tiles with K in two to eight parts, which the library also picks by
 * itself for products with few tiles and a long K (64 tiles or fewer, or 128 or fewer and K >= 4096; every part at
 * least 1024 of K; as many parts as give every CU a workgroup: 4096 x 128 x 4096 23.8 -> 17.1 us in 4 parts, 512 x 512 x
 * 8192 42.5 -> 17.6 us in 8).  Every workgroup leaves its fp32 partial sums in the workspace and draws a ticket; the one
 * that draws a tile's last ticket adds the parts up in the order of the parts and stores the tile, so the result does
 * not depend on which workgroup was last, and nobody waits for anybody.  Workspace: tiles * parts * 64 * 128 * 4 bytes,
 * then a ticket word per tile; 256-byte aligned.
 * Shape code 12: 256 x 256 tiles with K in two halves, on request only (measured on the product it was built for, 4096 x
 * 2048 x 4096: slower than what iex_gemm picks by itself).  The first of a tile's two workgroups to finish leaves its
 * partial sums in the workspace (M * N * 4 bytes rounded up to whole tiles, plus two words per tile), the other adds
 * them to its own and stores.  The second workgroup's wait is bounded; if it ever gave up, the tile is left unwritten and
 * its "written" word (the second half of the words behind the partial sums) reads -1 after the launch instead of 1:
 * stale sums are never added.
 * Both exchange through the L2 of the XCD that the workgroups of a tile run on (workgroup ids that differ by multiples
 * of 8: ids are dealt round-robin to the 8 XCDs in the mode this library is built for, one partition spanning the whole
 * GPU).  Plain store; a K step for every part.  Codes 12 and 14 fail without the workspace; code 0 without it (or with one
 * too small) runs exactly as iex_gemm; every other code ignores it.  iex_gemm_workspace_bytes returns 0 where the
 * workspace would not be used.  Neither call allocates.
 * No counterpart in the reference (its dense companions are library calls). */
int iex_gemm_ws(int dtype, int trans_b, int M, int N, int K, const void* A, const void* B,
                void* C, int batch, long long stride_a, long long stride_b,
                long long stride_c, void* stream, void* workspace, size_t workspace_bytes);
size_t iex_gemm_workspace_bytes(int dtype, int trans_b, int M, int N, int K, int batch);

/* ----------------------------------------------- horizontally fused launch ---- */
/* One launch whose workgroups are split between tiles of the dense GEMM C[z] = A[z]*B[z]
 * (as iex_gemm: gemm_batch entries, element strides stride_*) and row blocks of the fp16 CSR
 * SpMM (as iex_spmm_ex with dtype IEX_F16, batch 1, no flags).  interleave == 0: the GEMM
 * workgroups come first; interleave == g > 0: they are spread through the grid in groups of
 * g, each group followed by an even share of the SpMM blocks (any g >= 1 is valid); interleave < 0: the SpMM
 * workgroups come first (the longer jobs first: the GEMM tiles then fill the CUs that the SpMM's last round leaves
 * idle).  Both results are identical to the separate launches.  No counterpart in the reference
 * (the name survives only as the unused HORIZONTAL_GRAINED flag, tests/test_interleaving.py:441). */
int iex_fused_spmm_gemm(int spmm_itype, int m, int k, int n, int nonzeros,
                        const int* row_indices, const void* values, const int* row_offsets,
                        const void* column_indices, const void* dense, void* spmm_out,
                        int gemm_dtype, int trans_b, int M, int N, int K, const void* A,
                        const void* B, void* C, int gemm_batch, long long stride_a,
                        long long stride_b, long long stride_c, int interleave, void* stream);
/* The workgroup-id -> role map of that launch, evaluated on the host: for a grid of gemm_blocks +
 * spmm_blocks workgroups and group size `interleave`, workgroup `id` runs GEMM tile *index
 * (*is_gemm = 1) or SpMM block *index (*is_gemm = 0).  Every tile and every block is the role of
 * exactly one id for any counts and any interleave; the device code calls the same function.
 * No launch, no GPU needed.  No counterpart in the reference. */
int iex_fused_role(int gemm_blocks, int spmm_blocks, int interleave, int id, int* is_gemm, int* index);
/* Diagnostic: where and when every workgroup of a fused launch ran.  After iex_fused_timeline(buffer) the calls of
 * iex_fused_spmm_gemm that this thread makes and that run on the matrix-core kernel write, per workgroup id, four
 * 64-bit words into `buffer` (device memory, 32 bytes x workgroups of the launch, the caller's): the constant-rate
 * clock (100 MHz) when the workgroup began and when its last wavefront ended, the place ((XCD << 16) | the low 16 bits
 * of the hardware id word: compute unit, shader array and shader engine in bits 8..15), and (1 << 32 for a GEMM tile) |
 * the tile or block index.  Costs a workgroup barrier and four stores per workgroup; results are unchanged.
 * iex_fused_timeline(NULL) switches it off.  No counterpart in the reference. */
int iex_fused_timeline(void* buffer);

/* ------------------------------------------------------------ graph builder ---- */
/* Opaque builder of ONE hipGraph from per-stream captures; mirrors
 * CUDAExperimentalGraphConstructor<cudaStream_t> + CudaGraphWrapper
 * (common/include/helper_CUDAGraphConstructor.cu.h:106-166, 268-486) as bound by
 * pybind.cu:337-471.  Not internally synchronised: one thread per object. */
typedef struct iex_graph iex_graph;

iex_graph* iex_graph_create(void);                 /* graph + empty root node            */
iex_graph* iex_graph_wrap(void* hip_graph);        /* CudaGraphWrapper(long)             */
void iex_graph_destroy(iex_graph* g);
void* iex_graph_handle(iex_graph* g);              /* the hipGraph_t                     */
int iex_graph_register_stream(iex_graph* g, void* stream);   /* last activity := root  */
int iex_graph_begin_capture(iex_graph* g, void* stream);     /* notify_before_invoking_library_call */
int iex_graph_end_capture(iex_graph* g, void* stream);       /* notify_after_invoking_library_call  */
int iex_graph_add_event_record_node(iex_graph* g, void* event, void* stream);
int iex_graph_add_stream_wait_event_node(iex_graph* g, void* stream, void* event);
int iex_graph_join(iex_graph* g, void* const* streams, int num_streams, void* dst_stream);
int iex_graph_instantiate(iex_graph* g);           /* error if already instantiated      */
int iex_graph_launch(iex_graph* g, void* stream);
int iex_graph_destroy_exec(iex_graph* g);
int iex_graph_add_child_graph(iex_graph* parent, iex_graph* child);
/* N graphs as sibling child nodes of a fresh graph (helper_cuda_graph.cu.h:34-62). */
iex_graph* iex_graph_combine(iex_graph* const* graphs, int num_graphs);
int iex_graph_dump_dot(iex_graph* g, const char* path);
/* Structure queries used by tests and print_graph. */
long long iex_graph_num_nodes(iex_graph* g);
long long iex_graph_num_edges(iex_graph* g);
/* Fills up to `cap` (from,to) pairs as indices into the node order of
 * hipGraphGetNodes; returns the number of edges. */
long long iex_graph_get_edges(iex_graph* g, long long* from, long long* to, long long cap);
/* Node type (hipGraphNodeType) of node `index`, or negative on error. */
int iex_graph_node_type(iex_graph* g, long long index);
/* 1 while `stream` is being captured. */
int iex_stream_is_capturing(void* stream);

/* Handle round-trip checks (pybind.cu:17-45 print_cudastream / print_cudaevent):
 * return the pointer value they were given after querying it with the runtime. */
long long iex_echo_stream(void* stream);
long long iex_echo_event(void* event);

#ifdef __cplusplus
}
#endif
#endif /* IEX_HIP_H_ */
