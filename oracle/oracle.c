/*
 * CPU oracle for the sparse-plus-dense GEMM path.  TEST INFRASTRUCTURE ONLY:
 * nothing under the shipped package may include, link or call this file; the
 * parity tests, the smoke check and the benchmark's CPU-baseline leg are its
 * only users.
 *
 * Each function restates, as plain loops, what one reference operator computes.
 * The arithmetic of the reference lives in the Sputnik headers (an absent,
 * unpinned submodule), so the restatement follows the reference's own call
 * sites and wrappers:
 *   shapes, batch dimension, output shapes ...... pytorch/csrc/extensions/sputnik_kernels.cpp:7-168
 *   argument meaning and order ................... pytorch/csrc/extensions.h:10-31
 *   row swizzle, per-batch offsets, reuse flags .. pytorch/csrc/extensions/sputnik_spmm.cu.inc:109-133,160-164,176-180
 *   bias + ReLU epilogue, store mode ............. pytorch/csrc/extensions/sputnik_spmm.cu.inc:272-293
 *   SDDMM operand layout and batch summation ..... pytorch/csrc/extensions/sputnik_sddmm.cu.inc:63-79,92-101,124-130,177-181
 *
 * Pinning status (what checks each function against something other than its
 * own formula is listed in tests/test_oracle_pinning.py):
 *   oracle_spmm_*   : pinned (scipy CSR, torch.sparse, dense float64 matmul, brute force,
 *                     identity / permutation / dense special cases, the 3x4 example of
 *                     tests/test_cuda_python_interop.py:79-86).
 *   oracle_sddmm_*  : pinned (dense float64 a @ b^T gathered at the mask, full and diagonal
 *                     masks, gradient duality with SpMM).
 *   oracle_gemm_f64 : pinned (numpy float64 matmul, integer-input exactness).
 *   oracle_dense_to_csr / oracle_csr_transpose : pinned (scipy csr_matrix / .T.tocsr()).
 * The floating-point summation ORDER of the reference's kernels is not recoverable
 * here (sources absent); the oracle therefore accumulates in double and parity is
 * asserted to the stated relative tolerances, not bit-for-bit.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* out[z, r, :] (+)= sum_j values[(z,) j] * dense[z, col[j], :]  for r = row_indices[i].
 * sputnik_kernels.cpp:34-102 (b is (batch,k,n), out is (batch,m,n)),
 * sputnik_spmm.cu.inc:114 (row = row_indices[block]), :160-164 (values shared by the batch
 * unless per_batch_values), :287-293 (accumulate = atomic store mode, defined here as
 * "add to what out already holds").  bias (may be NULL) and relu follow :272-282.
 * Accumulates in double; rows that row_indices never names are left untouched. */
void oracle_spmm_f64(int m, int k, int n, int nnz, const int *row_indices,
                     const float *values, const int *row_offsets,
                     const int *column_indices, const float *dense, double *out,
                     int batch, int per_batch_values, int accumulate,
                     const float *bias, int relu) {
  (void)k;
  for (int z = 0; z < batch; ++z) {
    const float *vals = per_batch_values ? values + (size_t)z * nnz : values;
    const float *b = dense + (size_t)z * k * n;
    double *o = out + (size_t)z * m * n;
    for (int i = 0; i < m; ++i) {
      int r = row_indices[i];
      double *orow = o + (size_t)r * n;
      for (int c = 0; c < n; ++c) {
        double acc = 0.0;
        for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j)
          acc += (double)vals[j] * (double)b[(size_t)column_indices[j] * n + c];
        if (bias) acc += (double)bias[r];
        if (relu && acc < 0.0) acc = 0.0;
        orow[c] = accumulate ? orow[c] + acc : acc;
      }
    }
  }
}

/* Same operator with float accumulators in nonzero order, the precision the
 * reference kernel keeps (sputnik_spmm.cu.inc:185-187).  Row-at-a-time axpy
 * form so that a -O3 build vectorises it: this is the variant the benchmark
 * times as the single-core CPU port. */
void oracle_spmm_f32(int m, int k, int n, int nnz, const int *row_indices,
                     const float *values, const int *row_offsets,
                     const int *column_indices, const float *dense, float *out,
                     int batch, int per_batch_values, int accumulate) {
  (void)k;
  for (int z = 0; z < batch; ++z) {
    const float *vals = per_batch_values ? values + (size_t)z * nnz : values;
    const float *b = dense + (size_t)z * k * n;
    float *o = out + (size_t)z * m * n;
    for (int i = 0; i < m; ++i) {
      int r = row_indices[i];
      float *restrict orow = o + (size_t)r * n;
      if (!accumulate) memset(orow, 0, sizeof(float) * (size_t)n);
      for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j) {
        const float v = vals[j];
        const float *restrict brow = b + (size_t)column_indices[j] * n;
        for (int c = 0; c < n; ++c) orow[c] += v * brow[c];
      }
    }
  }
}

/* out[(z,) j] = sum_c lhs[z, row(j), c] * rhs[z, col(j), c].
 * sputnik_kernels.cpp:104-168 (a is (batch,m,k), b is (batch,n,k): rhs rows are the
 * sampled COLUMNS of the product), sputnik_sddmm.cu.inc:92-101 (batch offsets),
 * :124-130 (sum_over_batch: one (nnz) output summed over z), :177-181 (accumulate).
 * Accumulates in double. */
void oracle_sddmm_f64(int m, int k, int n, int nnz, const int *row_indices,
                      const int *row_offsets, const int *column_indices,
                      const float *lhs, const float *rhs, double *out, int batch,
                      int sum_over_batch, int accumulate) {
  (void)n;
  if (!accumulate) {
    size_t total = sum_over_batch ? (size_t)nnz : (size_t)nnz * batch;
    for (size_t t = 0; t < total; ++t) out[t] = 0.0;
  }
  for (int z = 0; z < batch; ++z) {
    const float *a = lhs + (size_t)z * m * k;
    const float *b = rhs + (size_t)z * n * k;
    double *o = sum_over_batch ? out : out + (size_t)z * nnz;
    for (int i = 0; i < m; ++i) {
      int r = row_indices[i];
      for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j) {
        const float *ar = a + (size_t)r * k;
        const float *br = b + (size_t)column_indices[j] * k;
        double acc = 0.0;
        for (int c = 0; c < k; ++c) acc += (double)ar[c] * (double)br[c];
        o[j] += acc;
      }
    }
  }
}

/* float-accumulate SDDMM for the single-core CPU timing leg. */
void oracle_sddmm_f32(int m, int k, int n, int nnz, const int *row_indices,
                      const int *row_offsets, const int *column_indices,
                      const float *lhs, const float *rhs, float *out, int batch,
                      int sum_over_batch) {
  (void)n;
  size_t total = sum_over_batch ? (size_t)nnz : (size_t)nnz * batch;
  memset(out, 0, sizeof(float) * total);
  for (int z = 0; z < batch; ++z) {
    const float *a = lhs + (size_t)z * m * k;
    const float *b = rhs + (size_t)z * n * k;
    float *o = sum_over_batch ? out : out + (size_t)z * nnz;
    for (int i = 0; i < m; ++i) {
      int r = row_indices[i];
      const float *restrict ar = a + (size_t)r * k;
      for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j) {
        const float *restrict br = b + (size_t)column_indices[j] * k;
        float acc = 0.f;
        for (int c = 0; c < k; ++c) acc += ar[c] * br[c];
        o[j] += acc;
      }
    }
  }
}

/* C = A * B (trans_b == 0, B is (K,N) row-major) or A * B^T (trans_b == 1, B is (N,K)
 * row-major, the torch.nn.Linear weight layout of layers_and_funcs/torch.py:17).
 * Double accumulation.  gemm_tflops counts 2*M*N*K (tests/test_interleaving.py:21-23). */
void oracle_gemm_f64(int M, int N, int K, const float *A, const float *B,
                     int trans_b, double *C) {
  for (int i = 0; i < M; ++i) {
    double *crow = C + (size_t)i * N;
    for (int j = 0; j < N; ++j) crow[j] = 0.0;
    if (trans_b) {
      for (int j = 0; j < N; ++j) {
        double acc = 0.0;
        for (int p = 0; p < K; ++p)
          acc += (double)A[(size_t)i * K + p] * (double)B[(size_t)j * K + p];
        crow[j] = acc;
      }
    } else {
      for (int p = 0; p < K; ++p) {
        double a = (double)A[(size_t)i * K + p];
        const float *brow = B + (size_t)p * N;
        for (int j = 0; j < N; ++j) crow[j] += a * (double)brow[j];
      }
    }
  }
}

/* Dense (m,k) -> CSR in the tuple order of pytorch/utils.py:147-153:
 * values = row-major matrix[matrix != 0]; row_offsets = [0, cumsum(nnz per row)];
 * column_indices ascending inside each row; row_indices = rows ordered by
 * decreasing nnz (the load-balancing swizzle consumed at sputnik_spmm.cu.inc:114),
 * ties kept in ascending row order (stable).  Call once with values == NULL to get
 * nnz, then again with buffers.  Returns nnz. */
int oracle_dense_to_csr(int m, int k, const float *matrix, float *values,
                        int *row_indices, int *row_offsets, int *column_indices) {
  int nnz = 0;
  for (int r = 0; r < m; ++r) {
    if (row_offsets) row_offsets[r] = nnz;
    for (int c = 0; c < k; ++c) {
      float v = matrix[(size_t)r * k + c];
      if (v != 0.0f) {
        if (values) {
          values[nnz] = v;
          column_indices[nnz] = c;
        }
        ++nnz;
      }
    }
  }
  if (row_offsets) row_offsets[m] = nnz;
  if (row_indices && row_offsets) {
    /* stable insertion by decreasing length: counting sort on length */
    int maxlen = 0;
    for (int r = 0; r < m; ++r) {
      int len = row_offsets[r + 1] - row_offsets[r];
      if (len > maxlen) maxlen = len;
    }
    int pos = 0;
    for (int len = maxlen; len >= 0; --len)
      for (int r = 0; r < m; ++r)
        if (row_offsets[r + 1] - row_offsets[r] == len) row_indices[pos++] = r;
  }
  return nnz;
}

/* CSR (m,k) -> CSR of the transpose (k,m); perm[t] = position in the source arrays of
 * the t-th nonzero of the transpose (the "transpose by a precomputed permutation" that
 * layers_and_funcs/sputnik.py:117-122 relies on). */
void oracle_csr_transpose(int m, int k, int nnz, const int *row_offsets,
                          const int *column_indices, int *row_offsets_t,
                          int *column_indices_t, int *perm) {
  for (int c = 0; c <= k; ++c) row_offsets_t[c] = 0;
  for (int j = 0; j < nnz; ++j) row_offsets_t[column_indices[j] + 1]++;
  for (int c = 0; c < k; ++c) row_offsets_t[c + 1] += row_offsets_t[c];
  /* fill in source order => ascending source row inside each transposed row */
  for (int r = 0; r < m; ++r) {
    for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j) {
      int c = column_indices[j];
      int dst = row_offsets_t[c]++;
      column_indices_t[dst] = r;
      perm[dst] = j;
    }
  }
  for (int c = k; c > 0; --c) row_offsets_t[c] = row_offsets_t[c - 1];
  row_offsets_t[0] = 0;
}
