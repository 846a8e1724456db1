/*
 * CPU oracle for the RoDe hot path: row-decomposition preprocessing, SDDMM and SpMM.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the bench's cpu_baseline leg may load it; the shipped
 * library never links or calls anything in this file.
 *
 * Every function restates, in plain C, a CPU routine that the reference keeps
 * inside its own test programs (cited per function).  What pins each one:
 *   - oracle_preprocess: hand-worked vectors, the independent per-row closed
 *     form of Preprocess_opt/_preprocess.cu:262-270 plus a prefix sum, the
 *     exact-once coverage invariant, ordering invariants, analytic cases and
 *     brute force on tiny inputs (tests/test_oracle_preprocess.py).
 *   - oracle_sddmm_*: fp64 numpy einsum, special cases (all-ones operands,
 *     zero values, one-hot rows) and brute force (tests/test_oracle_numeric.py).
 *   - oracle_spmm_*: the reference has NO CPU SpMM; this is the textbook CSR
 *     product, pinned by scipy.sparse (library routine), B=1 row sums,
 *     identity pattern and linearity (tests/test_oracle_numeric.py).
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -shared).
 */
#include <stddef.h>
#include <stdint.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* Number of threads the *_mt variants will use (1 without OpenMP). */
int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/*
 * Sequential row decomposition.
 * Follows RoDe_SDDMM/main.cu:114-163 (identical text at RoDe_SDDMM/test.cu:73-116,
 * RoDe_SDDMM/rode_sddmm_cuda.cu:80-110 and, without the sentinel,
 * Preprocess_opt/_preprocess.cu:340-373).
 *
 * Argument order is that of _preprocess.cu:340 (seg, kblock, veclen); main.cu
 * passes (seg, veclen, kblock).  st_off gets the sentinel st_off[n_blk] =
 * row_ptr[M] (main.cu:161-162), which the kernels read (RoDeSpmm.cu:213).
 *
 * Capacity the caller must provide: block_r_ind >= nnz/seg + M entries,
 * st_off one more, residue_r_ind >= M.
 */
void oracle_preprocess(int seg, int kblock, int veclen, int M, const int *row_ptr,
                       int *block_r_ind, int *st_off, int *residue_r_ind,
                       int *n_blk_out, int *n_res_out)
{
    int n_blk = 0, n_res = 0;
    for (int i = 0; i < M; ++i) {
        int row_offset = row_ptr[i];
        int n_padding = row_offset % veclen;
        int nnz = row_ptr[i + 1] - row_offset + n_padding;

        if (nnz > seg) { /* first segment keeps the unaligned start */
            block_r_ind[n_blk] = i;
            st_off[n_blk++] = row_offset;
            row_offset = (row_offset + seg) - n_padding;
            nnz -= seg;
        }
        while (nnz > seg) {
            block_r_ind[n_blk] = i;
            st_off[n_blk++] = row_offset;
            row_offset += seg;
            nnz -= seg;
        }
        if (nnz > 0) {
            if (nnz >= kblock) {
                block_r_ind[n_blk] = i;
                st_off[n_blk++] = row_offset;
            }
            if (nnz % kblock)
                residue_r_ind[n_res++] = i;
        }
    }
    st_off[n_blk] = row_ptr[M];
    *n_blk_out = n_blk;
    *n_res_out = n_res;
}

/*
 * SDDMM, fp32 accumulate, the reference's own CPU check.
 * Follows RoDe_SDDMM/main.cu:65-91 (same loop at test.cu:44-68):
 * out[idx] = values[idx] * sum_k lhs[row,k] * rhs[col,k], accumulated left to
 * right in float.
 */
void oracle_sddmm_f32(int m, int k, const int *row_offsets, const int *column_indices,
                      const float *values, const float *lhs, const float *rhs, float *out)
{
    for (int row = 0; row < m; ++row) {
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            int col = column_indices[idx];
            float dot = 0.0f;
            for (int kk = 0; kk < k; ++kk)
                dot += lhs[(size_t)row * k + kk] * rhs[(size_t)col * k + kk];
            out[idx] = values[idx] * dot;
        }
    }
}

/* Same loop, rows shared between threads (static schedule balanced by nnz is
 * left to the runtime's guided schedule).  Used only as the all-cores leg of
 * the bench's CPU baseline. */
void oracle_sddmm_f32_mt(int m, int k, const int *row_offsets, const int *column_indices,
                         const float *values, const float *lhs, const float *rhs, float *out)
{
#pragma omp parallel for schedule(guided, 64)
    for (int row = 0; row < m; ++row) {
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            int col = column_indices[idx];
            float dot = 0.0f;
            for (int kk = 0; kk < k; ++kk)
                dot += lhs[(size_t)row * k + kk] * rhs[(size_t)col * k + kk];
            out[idx] = values[idx] * dot;
        }
    }
}

/*
 * SDDMM with fp64 accumulation: the value the tolerance is measured against.
 * Same formula as main.cu:65-91, with the sum and the final product in double.
 * abs_out (optional) receives |values[idx]| * sum_k |lhs*rhs|, the scale a
 * per-element error bound is normalised by.
 */
void oracle_sddmm_f64(int m, int k, const int *row_offsets, const int *column_indices,
                      const float *values, const float *lhs, const float *rhs,
                      double *out, double *abs_out)
{
#pragma omp parallel for schedule(guided, 64)
    for (int row = 0; row < m; ++row) {
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            int col = column_indices[idx];
            double dot = 0.0, adot = 0.0;
            for (int kk = 0; kk < k; ++kk) {
                double p = (double)lhs[(size_t)row * k + kk] * (double)rhs[(size_t)col * k + kk];
                dot += p;
                adot += p < 0 ? -p : p;
            }
            double v = (double)values[idx];
            out[idx] = v * dot;
            if (abs_out)
                abs_out[idx] = (v < 0 ? -v : v) * adot;
        }
    }
}

/*
 * SpMM C[m x n] = A_csr * B[k x n], fp32.  The reference ships no CPU SpMM;
 * this is the textbook CSR product that RoDeSpmm.cu:197-476 / :41-195 compute
 * piecewise (every nonzero contributes values[idx] * B[col,:] to C[row,:]
 * exactly once).  Rows without nonzeros are written as zeros.
 */
void oracle_spmm_f32(int m, int n, const int *row_offsets, const int *column_indices,
                     const float *values, const float *B, float *C)
{
    for (int row = 0; row < m; ++row) {
        float *c = C + (size_t)row * n;
        for (int j = 0; j < n; ++j)
            c[j] = 0.0f;
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            const float *b = B + (size_t)column_indices[idx] * n;
            float v = values[idx];
            for (int j = 0; j < n; ++j)
                c[j] += v * b[j];
        }
    }
}

void oracle_spmm_f32_mt(int m, int n, const int *row_offsets, const int *column_indices,
                        const float *values, const float *B, float *C)
{
#pragma omp parallel for schedule(guided, 64)
    for (int row = 0; row < m; ++row) {
        float *c = C + (size_t)row * n;
        for (int j = 0; j < n; ++j)
            c[j] = 0.0f;
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            const float *b = B + (size_t)column_indices[idx] * n;
            float v = values[idx];
            for (int j = 0; j < n; ++j)
                c[j] += v * b[j];
        }
    }
}

/* fp64-accumulated SpMM plus, per row, L1 = sum_idx |values[idx]| * sum_j |B[col,j]|
 * accumulated per output column into abs_out (optional, m x n): the scale the
 * error bound is normalised by. */
void oracle_spmm_f64(int m, int n, const int *row_offsets, const int *column_indices,
                     const float *values, const float *B, double *C, double *abs_out)
{
#pragma omp parallel for schedule(guided, 64)
    for (int row = 0; row < m; ++row) {
        double *c = C + (size_t)row * n;
        double *a = abs_out ? abs_out + (size_t)row * n : 0;
        for (int j = 0; j < n; ++j) {
            c[j] = 0.0;
            if (a)
                a[j] = 0.0;
        }
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            const float *b = B + (size_t)column_indices[idx] * n;
            double v = (double)values[idx];
            for (int j = 0; j < n; ++j) {
                double p = v * (double)b[j];
                c[j] += p;
                if (a)
                    a[j] += p < 0 ? -p : p;
            }
        }
    }
}

/* SpMM with fp64 values, B and C: the arithmetic of the double overloads
 * RoDe_SpMM/RoDeSpmm.cu:521-529 (same kernels instantiated for double). */
void oracle_spmm_d(int m, int n, const int *row_offsets, const int *column_indices,
                   const double *values, const double *B, double *C)
{
#pragma omp parallel for schedule(guided, 64)
    for (int row = 0; row < m; ++row) {
        double *c = C + (size_t)row * n;
        for (int j = 0; j < n; ++j)
            c[j] = 0.0;
        for (int idx = row_offsets[row]; idx < row_offsets[row + 1]; ++idx) {
            const double *b = B + (size_t)column_indices[idx] * n;
            double v = values[idx];
            for (int j = 0; j < n; ++j)
                c[j] += v * b[j];
        }
    }
}
