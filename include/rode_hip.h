/*
 * C ABI of librode_hip.so -- RoDe row-decomposition preprocessing, SpMM and
 * SDDMM for AMD MI355X (gfx950).
 *
 * Plain pointers and sizes only.  Every pointer named d_* is DEVICE memory
 * owned by the caller; nothing here allocates or frees, and nothing
 * synchronises with the host: all work is queued on the streams passed in
 * (a `void*` stream is a hipStream_t; NULL is HIP's default stream).
 * Return value: 0 on success, otherwise a hipError_t value
 * (rode_hip_error_string() turns it into text).
 *
 * C of the SpMM calls must be ordinary (coarse-grained) device memory, as hipMalloc
 * returns: long rows are summed with hardware floating-point atomics, which
 * fine-grained or host-coherent allocations do not support.
 *
 * Layout and alignment contract (same as the reference kernels, which use
 * 128-bit accesses throughout, e.g. RoDe_SpMM/RoDeSpmm.cu:89,247-248 and
 * RoDe_SDDMM/RoDeSddmm.cu:75,80,88): all arrays row-major and 16-byte aligned.
 */
#ifndef RODE_HIP_H_
#define RODE_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Library version, (major << 16) | minor. */
int rode_hip_version(void);

/* Text for a code returned by the functions below. */
const char* rode_hip_error_string(int code);

/*
 * Scratch bytes rode_hip_preprocess() needs for a matrix of M rows
 * (replaces the cudaMalloc/cudaFree of CUB temp storage inside the reference's
 * GPU preprocess, Preprocess_opt/_preprocess.cu:325-335).
 */
size_t rode_hip_preprocess_workspace_bytes(int M);

/*
 * Row decomposition on the GPU.
 * Replaces RoDe_preprocess (GPU), Preprocess_opt/_preprocess.cu:323-339, and
 * produces the arrays of the CPU routine RoDe_SDDMM/main.cu:114-163 bit for
 * bit, sentinel d_st_off[n_blk] = row_ptr[M] included.
 *   seg_length, k_block, vec_len : decomposition parameters, order of
 *                                  _preprocess.cu:323 (512,32,4 or 32,32,4 in the reference)
 *   d_row_ptr        int[M+1]    CSR row pointer
 *   d_block_r_ind    int[cap]    out: row of every block segment
 *   d_st_off         int[cap+1]  out: first nonzero of every block segment, then the sentinel
 *   d_residue_r_ind  int[>=M]    out: rows that own a residue
 *   d_n_blk, d_n_res int[1] each out: segment / residue counts
 *   capacity_blocks  cap above; (nnz + (vec_len-1)*M)/seg_length + M always suffices
 *                    (the reference sizes it nnz/seg + M, _preprocess.cu:426).  If it is
 *                    too small nothing is written past it and *d_n_blk still reports
 *                    the true count, so the caller can detect the overflow.
 *   d_workspace      rode_hip_preprocess_workspace_bytes(M) bytes, 8-byte aligned (8 bytes per
 *                    1024 rows: the status words of the scan across workgroups)
 * Two launches: a fill of the scratch, then one kernel that reads row_ptr once, scans and
 * writes the lists.  Should a workgroup ever wait in vain for an earlier one (bounded; it
 * cannot happen while the GPU runs workgroups it has started), *d_n_blk = *d_n_res = -1.
 */
int rode_hip_preprocess(int seg_length, int k_block, int vec_len, int M, const int* d_row_ptr,
                        int* d_block_r_ind, int* d_st_off, int* d_residue_r_ind, int* d_n_blk, int* d_n_res,
                        int capacity_blocks, void* d_workspace, size_t workspace_bytes, void* stream);

/*
 * The same decomposition for a caller that holds the row pointer in HOST memory and wants
 * HOST arrays back.  Replaces the CPU routines RoDe_preprocess_cpu,
 * Preprocess_opt/_preprocess.cu:340-373, and RoDe_preprocess, RoDe_SDDMM/main.cu:114-163
 * (argument order here: seg_length, k_block, vec_len; main.cu has vec_len before k_block).
 * Every pointer is host memory; h_block_r_ind needs n_blk entries, h_st_off n_blk + 1
 * (sentinel), h_residue_r_ind n_res; (nnz + (vec_len-1)*M)/seg_length + M (+1) and M always
 * suffice.  Unlike everything else in this header the call allocates (and frees) device
 * memory, copies, runs the kernels of rode_hip_preprocess on the default stream of the
 * current device and waits for them.
 */
int rode_hip_preprocess_host(int seg_length, int k_block, int vec_len, int M, const int* h_row_ptr,
                             int* h_block_r_ind, int* h_st_off, int* h_residue_r_ind, int* h_n_blk, int* h_n_res);

/*
 * rode_hip_preprocess() without a workspace argument and without any allocation, for
 * callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its GPU
 * routine allocates and frees CUB scratch on every call, _preprocess.cu:331-335).
 * Same arguments, same kernels and byte-identical results; the scan scratch is a fixed
 * array inside the library (128 KB of device memory per GPU, held until the process
 * ends), so M is limited to RODE_HIP_STATIC_MAX_ROWS: a larger M returns
 * hipErrorOutOfMemory (2) before anything is launched.  The first call on a device looks
 * up the array's address (no allocation; make that call outside stream capture).  Every
 * call on one GPU uses that GPU's one array: calls that overlap in time on the same GPU
 * (different streams) race; calls queued on one stream do not, from whichever host threads
 * they come (the launches of a call are queued under a lock).  The
 * caller clears nothing between calls: each call begins with a fill kernel over the part
 * of the array it is going to use (a kernel, not a memset, so the call can be captured).
 */
#define RODE_HIP_STATIC_MAX_ROWS 4194304
int rode_hip_preprocess_static(int seg_length, int k_block, int vec_len, int M, const int* d_row_ptr,
                               int* d_block_r_ind, int* d_st_off, int* d_residue_r_ind, int* d_n_blk, int* d_n_res,
                               int capacity_blocks, void* stream);

/*
 * SpMM  C[M x n] += A_csr[M x k] * B[k x n]  (fp32 values, fp32 or fp16 dense B,
 * fp32 accumulate and output).
 * Replaces RoDeSpmm_n32 / RoDeSpmm_n128 (fp32), RoDe_SpMM/RoDeSpmm.h:4-8,
 * RoDeSpmm.cu:511-519: the block-segment kernel runs on stream1 over m1
 * segments, the residue kernel on stream2 over m2 rows.  As in the reference
 * C must be zero on entry: segments and tails of long rows are added with
 * atomics, short rows are stored, rows without nonzeros are not touched.
 * n: any positive multiple of 4 (the reference needs a multiple of its 32- or
 * 64-wide tile and does not guard the edge); multiples of 32 take the unguarded
 * fast path.  The decomposition must have been made with k_block 32, vec_len 4 and a
 * seg_length that is a positive multiple of 32 (rode_hip_preprocess itself accepts any
 * parameters).  This holds for every SpMM and SDDMM entry point below.  With lists made
 * for another seg_length the kernels still stay inside the arrays and inside each row,
 * but - like the reference's kernels - they leave some nonzeros of a row out, and which
 * ones may differ between entry points.
 */
int rode_hip_spmm_f32(int m1, int m2, int k, int n, const float* d_values, const int* d_column_indices,
                      const int* d_row_offsets, const int* d_row_indices1, const int* d_row_indices2,
                      const int* d_row_seg_st_offsets, const float* d_B, float* d_C, void* stream1,
                      void* stream2);

/*
 * SpMM with a promise.  dtype selects the element type of B (RODE_DENSE_F32: fp32 values
 * and C; RODE_DENSE_F16: fp32 values and C, fp16 B; RODE_DENSE_F64: fp64 values, B, C);
 * flags = 0 behaves exactly like the typed functions above.  RODE_SPMM_WHOLE_LISTS
 * promises that row_indices1 / row_seg_st_offsets / row_indices2 are the COMPLETE
 * decomposition of the matrix (not a slice of it): a row of 32..1024 aligned slots may
 * then be summed - all its segments and its tail - by one wavefront with a single
 * update of C instead of one atomic update per work item.  Same results; no counterpart
 * in the reference.
 */
#define RODE_DENSE_F32 0
#define RODE_DENSE_F16 1
#define RODE_DENSE_F64 2
#define RODE_SPMM_WHOLE_LISTS 1
/* With RODE_SPMM_WHOLE_LISTS: a row of C that a single work item produces is STORED instead
 * of added to, so that C need not be zero there on entry (C = A B instead of C += A B):
 *   - rows of fewer than 32 aligned slots (stored by every entry point, as in the reference);
 *   - rows of at most rode_hip_spmm_overwrite_limit() aligned slots;
 *   - the rows of the kept groups of a group plan, whatever their length.
 * Longer rows are still added to by several work items and must be zero on entry, and rows
 * without slots are not touched: a caller whose matrix has neither calls no
 * rode_hip_spmm_clear_rows() at all.  (Aligned slots of a row: its nonzeros plus
 * row_offsets[r] % 4.)  No counterpart in the reference. */
#define RODE_SPMM_OVERWRITE 16
/* Launch only the block-segment kernel / only the residue kernel / only the kernels of a
 * hub plan, with every other decision (which rows a single wavefront sums whole, which rows
 * the hub kernels take) made as if all were launched: for measuring one kernel, and for
 * callers that order them themselves.  m1, m2, all lists and plans are passed as for a
 * normal call; at most one of the three bits. */
#define RODE_SPMM_ONLY_BLOCK 2
#define RODE_SPMM_ONLY_RESIDUE 4
#define RODE_SPMM_ONLY_HUB 8
int rode_hip_spmm_ex(int dtype, int flags, int m1, int m2, int k, int n, const void* d_values,
                     const int* d_column_indices, const int* d_row_offsets, const int* d_row_indices1,
                     const int* d_row_indices2, const int* d_row_seg_st_offsets, const void* d_B, void* d_C,
                     void* stream1, void* stream2);

/*
 * Locality plan (no counterpart in the reference, whose kernels gather every dense row
 * from memory: RoDe_SpMM/RoDeSpmm.cu:140-160, RoDe_SDDMM/RoDeSddmm.cu:96-140).
 * The residue list is cut into chunks of RODE_HIP_PLAN_RESIDUE_CHUNK entries.  For every
 * chunk the plan records whether the dense rows its nonzeros reference cluster in a window
 * of at most RODE_HIP_WINDOW_ROWS consecutive rows (banded matrices: FEM, stencils).  The
 * *_planned entry points below process such a chunk with kernels that stage the window in
 * LDS once per 128-byte column tile and read it from there; nonzeros outside the window
 * are still gathered from memory, so a plan never changes a result, only the speed.
 * A plan is made in two steps; the second, larger part is only worth making when the first
 * finds windows (h_counts[1] > 0):
 *
 * 1. rode_hip_window_plan: the descriptors.
 *   dense_rows   rows of the dense operand the column indices point into (B of SpMM,
 *                rhs of SDDMM): the number of columns of the sparse matrix
 *   d_plan       rode_hip_window_plan_bytes(m2) bytes, 16-byte aligned, out.  Layout:
 *                int[4] header {residue chunks, residue chunks with a window, 0, 0},
 *                then int[4] per chunk {first window row, window rows (0: none),
 *                nonzeros, nonzeros outside the window}
 *   h_counts     NULL, or HOST int[4] that receives the header; the call then waits for
 *                the kernels (three small launches, each nonzero's column index read once)
 * 2. rode_hip_window_rows: for every residue row of a chunk with a window, where in the
 *    window each of its nonzeros is (what the window kernels would otherwise work out per
 *    call), in the order they will be read.
 *   d_rows       rode_hip_window_rows_bytes(m2) bytes (10 KiB per chunk of 128 residue
 *                rows), 16-byte aligned, out
 *
 * A plan belongs to exactly the residue list it was made from (same m2, same arrays).
 */
#define RODE_HIP_PLAN_RESIDUE_CHUNK 128
#define RODE_HIP_WINDOW_ROWS 512
size_t rode_hip_window_plan_bytes(int m2);
int rode_hip_window_plan(int m2, int dense_rows, const int* d_row_indices_residue, const int* d_row_offsets,
                         const int* d_column_indices, void* d_plan, size_t plan_bytes, int* h_counts, void* stream);
size_t rode_hip_window_rows_bytes(int m2);
int rode_hip_window_rows(int m2, const int* d_row_indices_residue, const int* d_row_offsets,
                         const int* d_column_indices, const void* d_plan, void* d_rows, size_t rows_bytes, void* stream);

/*
 * Hub plan (no counterpart in the reference either).  For matrices with a few very long
 * rows (hubs of a power-law graph) whose dense operand is far larger than the caches: the
 * rows of at least min_len aligned nonzero slots are cut into pieces by column slab
 * (RODE_HIP_HUB_SLAB_ROWS dense rows) and worked on slab after slab - a few neighbouring
 * slabs, about 4 MB of the dense operand, at a time - by kernels of their own, so that the
 * hub rows' nonzeros of those slabs meet in one L2 and a dense row is fetched from memory
 * once for all of them.  The other kernels leave those rows out.  Results are
 * the same up to the order of the fp32 additions inside a hub row.
 *   dense_rows   rows of the dense operand (columns of the sparse matrix)
 *   min_len      >= RODE_HIP_HUB_MIN_LEN; a piece should hold dozens of nonzeros: 4096 and
 *                dense_rows / 512 are sensible lower bounds (measured on a 2 M x 2 M
 *                power-law matrix: 4096 is best, 2048 and 8192 gain less, 1024 loses)
 *   d_plan       rode_hip_hub_plan_bytes(M, dense_rows, nnz, min_len) bytes, 16-byte aligned, out
 *   h_counts     HOST int[8], out (the call waits for its two kernels): [0] hub rows,
 *                [1] slabs, [2] min_len, [3] 1 if the plan is usable - every hub row's column
 *                indices ascend and lie inside the operand - else 0, [4] room for hub rows;
 *                the *_planned entry points need it and ignore a plan with [3] == 0 or [0] == 0
 * A hub plan belongs to the pattern it was made from, and excludes a locality plan: the
 * *_planned entry points refuse to take both.
 */
#define RODE_HIP_HUB_SLAB_ROWS 2048
#define RODE_HIP_HUB_MIN_LEN 64
size_t rode_hip_hub_plan_bytes(int M, int dense_rows, int nnz, int min_len);
size_t rode_hip_hub_workspace_bytes(const int* h_hub_counts, int n, int elem_bytes);
int rode_hip_hub_plan(int M, int dense_rows, int nnz, int min_len, const int* d_row_offsets,
                      const int* d_column_indices, void* d_plan, size_t plan_bytes, int* h_counts, void* stream);

/*
 * Group plan (no counterpart in the reference either).  For matrices whose adjacent rows
 * share long runs of consecutive column indices (sliding-window attention masks, dense
 * bands, block structure): groups of RODE_HIP_GROUP_ROWS adjacent rows whose longest runs
 * have at least 64 columns in common, holding at least three quarters of their nonzeros,
 * and start and end within 255 columns of each other, are processed by kernels of their
 * own.  Those walk the columns that all the runs hold once, load every dense row of that
 * shared run once for all rows of the group (its address follows from the run, no column
 * index is read), and then take each row's other nonzeros, the ends of its own run
 * included, the usual way: a row never meets a dense row that it does not reference.  The
 * other kernels leave those rows out.  Same results up to the order of the fp32 additions.
 *   d_plan       rode_hip_group_plan_bytes(M) bytes, 16-byte aligned, out
 *   h_counts     HOST int[4], out (the call waits for its kernels): [0] groups (M / 4,
 *                whole groups only), [1] groups with a run, [2] rows outside those groups
 *                (0: the other kernels have nothing to do and are not launched); the
 *                *_planned entry points need it and ignore a plan with [1] == 0
 * A group plan belongs to the pattern it was made from and excludes the other two plans.
 * SDDMM uses it for k <= 128 elements (fp32 and fp16 alike: rows of one 128-element slab; wider
 * rows go through the list kernels, plan or not), SpMM for any width.
 */
#define RODE_HIP_GROUP_ROWS 4
size_t rode_hip_group_plan_bytes(int M);
int rode_hip_group_plan(int M, const int* d_row_offsets, const int* d_column_indices, void* d_plan, size_t plan_bytes,
                        int* h_counts, void* stream);

/*
 * The plans of one matrix, as the *_planned entry points take them: a struct in HOST
 * memory, read during the call only.  Every member may be NULL / 0; a struct of zeros (or
 * a NULL struct pointer) makes the planned calls exactly the unplanned ones.
 *   window, window_rows   both parts of a locality plan made from the lists of the call
 *   window_counts         NULL, or the HOST int[4] header rode_hip_window_plan returned;
 *                         with it, kernels that would find no chunk to work on are not
 *                         launched at all.  fp64 operands, and dense rows of at most 128
 *                         bytes, ignore the locality plan.
 *   hub, hub_counts       a hub plan of this matrix and its HOST int[8] header (required
 *                         with it).  Needs the complete decomposition: for SpMM the
 *                         RODE_SPMM_WHOLE_LISTS promise, for SDDMM simply whole lists.
 *                         Excludes a locality plan.
 *   hub_workspace, hub_workspace_bytes   SpMM only: rode_hip_hub_workspace_bytes(hub_counts,
 *                         n, 4 or 8) bytes of scratch, 16-byte aligned, that the hub kernels
 *                         of this call may write and read (one partial row of C per hub
 *                         row and slab group, summed by a second kernel), or NULL: the
 *                         pieces are then added to C atomically, slower for wide rows.
 *   groups, group_counts  a group plan of this matrix and its HOST int[4] header (required
 *                         with it).  Needs the complete decomposition, like a hub plan,
 *                         and excludes both other plans.
 *   seg_length            0, or the segment length the lists were made with (the first
 *                         argument of the preprocessing call).  Not a plan, but knowledge
 *                         the launch can use: a decomposition with short segments (the
 *                         reference's K = 128 set has 32) is walked several segments per
 *                         wavefront, and with the length known the grid is sized for that.
 *                         Without it the kernels read the length off the lists and the
 *                         grid is capped instead.  A wrong value costs time, never a result.
 * Same results as without a plan, up to the order of the fp32 additions inside a row.
 */
typedef struct rode_hip_plans {
    const void* window;
    const void* window_rows;
    const int* window_counts;
    const void* hub;
    const int* hub_counts;
    void* hub_workspace;
    size_t hub_workspace_bytes;
    const void* groups;
    const int* group_counts;
    int seg_length;
} rode_hip_plans;

/* rode_hip_spmm_ex with plans. */
int rode_hip_spmm_planned(int dtype, int flags, int m1, int m2, int k, int n, const void* d_values,
                          const int* d_column_indices, const int* d_row_offsets, const int* d_row_indices1,
                          const int* d_row_indices2, const int* d_row_seg_st_offsets, const void* d_B, void* d_C,
                          const rode_hip_plans* plans, void* stream1, void* stream2);

/* The longest row, in aligned slots, that rode_hip_spmm_planned(..., RODE_SPMM_WHOLE_LISTS |
 * RODE_SPMM_OVERWRITE, m1, ..., plans, ...) stores with one work item; 0: none of the rows
 * with 32 aligned slots or more (few block segments: every work item adds; a hub plan).
 * plans may be NULL.  Host arithmetic, no GPU work. */
int rode_hip_spmm_overwrite_limit(int m1, const rode_hip_plans* plans);

/*
 * Prepares an uninitialised C[M x n] for one of the SpMM calls: zeroes exactly the rows
 * that SpMM adds to (aligned length >= 32) or never touches (rows in no list) and
 * leaves alone the rows it stores.  A cheaper replacement for clearing all of C; the
 * reference has no counterpart (its callers memset C).  elem_bytes is 4 (f32, f16
 * variants) or 8 (f64).  Must be ordered before both SpMM streams.
 */
int rode_hip_spmm_clear_rows(int M, int n, int elem_bytes, const int* d_row_offsets, void* d_C, void* stream);

/* fp64 values, B and C.  Replaces the double overloads of RoDeSpmm_n32 / RoDeSpmm_n128,
 * RoDe_SpMM/RoDeSpmm.h:10-14, RoDeSpmm.cu:521-529.  Same contract as rode_hip_spmm_f32
 * (n a multiple of 2). */
int rode_hip_spmm_f64(int m1, int m2, int k, int n, const double* d_values, const int* d_column_indices,
                      const int* d_row_offsets, const int* d_row_indices1, const int* d_row_indices2,
                      const int* d_row_seg_st_offsets, const double* d_B, double* d_C, void* stream1,
                      void* stream2);

/* Same with B stored as IEEE fp16, n a multiple of 8 (no reference entry point; operand semantics of the
 * unused helper VectorCompute<half4>::FMA, RoDe_SpMM/common_utils.h:183-230:
 * widen to fp32, fp32 FMA). */
int rode_hip_spmm_f16(int m1, int m2, int k, int n, const float* d_values, const int* d_column_indices,
                      const int* d_row_offsets, const int* d_row_indices1, const int* d_row_indices2,
                      const int* d_row_seg_st_offsets, const void* d_B_half, float* d_C, void* stream1,
                      void* stream2);

/*
 * SDDMM  out[idx] = values[idx] * <lhs[row(idx),:], rhs[col(idx),:]>.
 * Replaces RoDeSDDMM_n32 / RoDeSDDMM_n128, RoDe_SDDMM/RoDeSddmm.h:4-9,
 * RoDeSddmm.cu:496-545.  k: any positive multiple of 4 up to 512 (the reference
 * has 32 and 128); 32, 64 and 128 take the unguarded fast path.  Segments may have any length that the decomposition produced, so one
 * entry point serves both reference parameter sets (512,32,4) and (32,32,4).
 * Every out[idx], idx < nnz, is written exactly once; out needs no clearing.
 * A launch is skipped only when its count is zero (the reference also skips it
 * when the stream handle is NULL, RoDeSddmm.cu:503,509; here NULL is the
 * default stream).
 */
int rode_hip_sddmm_f32(int m1, int m2, int n, int k, const int* d_row_indices_block,
                       const int* d_row_indices_residue, const int* d_st_offsets, const int* d_row_offsets,
                       const int* d_column_indices, const float* d_values, const float* d_lhs_matrix,
                       const float* d_rhs_matrix, float* d_out, void* stream1, void* stream2);

/* Same with lhs / rhs stored as IEEE fp16, fp32 accumulate, k a multiple of 8 (no reference entry point). */
int rode_hip_sddmm_f16(int m1, int m2, int n, int k, const int* d_row_indices_block,
                       const int* d_row_indices_residue, const int* d_st_offsets, const int* d_row_offsets,
                       const int* d_column_indices, const float* d_values, const void* d_lhs_half,
                       const void* d_rhs_half, float* d_out, void* stream1, void* stream2);

/*
 * SDDMM with plans: dtype RODE_DENSE_F32 or RODE_DENSE_F16 selects the element type of
 * lhs / rhs; plans as for rode_hip_spmm_planned (NULL: exactly the typed functions above).
 * flags: 0, or one of the RODE_SPMM_ONLY_* bits (one kernel family of the call).
 * Same results up to the order of the fp32 additions of a dot product.  No counterpart in
 * the reference.
 */
int rode_hip_sddmm_planned(int dtype, int flags, int m1, int m2, int n, int k, const int* d_row_indices_block,
                           const int* d_row_indices_residue, const int* d_st_offsets, const int* d_row_offsets,
                           const int* d_column_indices, const float* d_values, const void* d_lhs_matrix,
                           const void* d_rhs_matrix, float* d_out, const rode_hip_plans* plans, void* stream1,
                           void* stream2);

/*
 * Row softmax over the values of a CSR pattern, out[idx] = softmax over the row of
 * scale * in[idx]; rows without nonzeros are skipped; out may alias in.  No
 * counterpart in the reference: it is the step between its SDDMM and SpMM when
 * the two are chained as sparse attention (the reference op is forward-only SDDMM,
 * RoDe_SDDMM/rode_sddmm.py:194-248).
 */
int rode_hip_csr_softmax_f32(int M, const int* d_row_offsets, const float* d_in, float* d_out, float scale,
                             void* stream);

/* Its gradient: ds[idx] = scale * p[idx] * (dp[idx] - sum over the row of dp * p); ds may alias dp. */
int rode_hip_csr_softmax_backward_f32(int M, const int* d_row_offsets, const float* d_p, const float* d_dp,
                                      float* d_ds, float scale, void* stream);

/*
 * Sparse attention in one kernel: out[r, :] = sum over the row's nonzeros of
 * p[idx] * v[col(idx), :] with p = softmax over the row of
 * scale * values[idx] * <q[r, :], k[col(idx), :]> -- the results of SDDMM, the row softmax
 * above and SpMM chained, without their intermediate arrays.  No counterpart in the
 * reference (its op is the forward SDDMM alone, RoDe_SDDMM/rode_sddmm.py:194-248).
 *   dtype        RODE_DENSE_F32 or RODE_DENSE_F16: element type of q, k and v
 *   M            rows of the pattern (= rows of q and of out)
 *   d            width of q, k and v: 32, 64 or 128
 *   d_row_offsets, d_column_indices, d_values   the CSR pattern; the row decomposition is
 *                not used: one wave takes a whole row, whatever its length
 *   d_q [M x d], d_k, d_v [columns x d]   row-major, 16-byte aligned
 *   d_out        float [M x d]; rows without nonzeros are written as zeros
 *   d_probs      NULL, or float [nnz] that receives p (what a gradient needs)
 *   plans        NULL, or the plans of this pattern: a group plan with at least 1024 groups
 *                with a run (2048 for fp16 operands) is used (the rows of a group then share
 *                one wave, and every k and v row of the group's run is loaded once for its
 *                four rows; with fewer groups a wave per row keeps more of the GPU busy); the
 *                other plans are ignored
 */
int rode_hip_attention_forward(int dtype, int M, int d, const int* d_row_offsets, const int* d_column_indices,
                               const float* d_values, const void* d_q, const void* d_k, const void* d_v,
                               float scale, float* d_out, float* d_probs, const rode_hip_plans* plans, void* stream);

/*
 * The same for `heads` problems on one pattern in one launch (the heads of an attention
 * layer share their mask): d_q and d_out hold heads x M x d elements, d_k and d_v
 * heads x N x d, d_probs (if not NULL) heads x nnz, each head after the other.  N: columns
 * of the pattern, nnz: its nonzeros (they say where the next head's operands start).  The
 * pattern, its values and the plan are read by every head.
 *   d_row_stats  NULL, or float [heads x M x 2], 8-byte aligned (needs d_probs): d_probs then
 *                receives the scaled SCORES scale * values * <q, k> instead of p, and
 *                d_row_stats the pair (maximum score, 1 / sum of exp(score - maximum)) of
 *                every row, so that p = exp(score - maximum) * (1 / sum).  Cheaper than
 *                normalised probabilities (no second pass over the row);
 *                rode_hip_attention_backward_rows takes the two arrays as they are.
 */
int rode_hip_attention_forward_batched(int dtype, int heads, int M, int N, int nnz, int d, const int* d_row_offsets,
                                       const int* d_column_indices, const float* d_values, const void* d_q, const void* d_k,
                                       const void* d_v, float scale, float* d_out, float* d_probs, float* d_row_stats,
                                       const rode_hip_plans* plans, void* stream);

/*
 * The gradient of rode_hip_attention_forward in two kernels (no counterpart in the
 * reference, whose op is forward-only, RoDe_SDDMM/rode_sddmm.py:194-248).  With g the
 * gradient of the loss with respect to out:
 *   rode_hip_attention_backward_rows  walks the pattern: per nonzero dp = <g[r, :], v[col, :]>
 *       and dz = scale * values * p * (dp - <g[r, :], out[r, :]>), the gradient with respect
 *       to <q[r, :], k[col, :]>; writes grad_q[r, :] = sum dz * k[col, :] and, to the nonzero's
 *       slot in the transposed pattern, the pair (p, dz);
 *   rode_hip_attention_backward_cols  walks the transposed pattern (rode_hip_csr_transpose):
 *       grad_k[c, :] = sum dz * q[row, :] and grad_v[c, :] = sum p * g[row, :] over the
 *       nonzeros of column c, with the pairs the first call left in its order.
 *   dtype        RODE_DENSE_F32 or RODE_DENSE_F16: element type of q, k and v (g, out and the
 *                three gradients are float; with fp16 operands g is rounded to fp16 relative to
 *                the largest magnitude of its row where it meets rows of v)
 *   heads        problems on the one pattern (1: a single head); every operand below except
 *                the pattern, d_t_slot and the plans holds `heads` arrays, one after the other
 *   M, N, nnz    rows / columns / nonzeros of the pattern; d: 32, 64 or 128
 *   d_probs      float [nnz]: p as rode_hip_attention_forward wrote it
 *   d_row_stats  NULL, or what rode_hip_attention_forward_batched wrote beside the scores
 *                it then left in d_probs
 *   d_out        float [M x d]: the forward result
 *   d_t_slot     int [nnz]: for every nonzero its index in the transposed pattern, i.e. the
 *                inverse of the d_perm that rode_hip_csr_transpose returns
 *   d_pairs      float [2 * nnz], 16-byte aligned: written by the first call, read by the second
 *   plans / t_plans   NULL, or the plans of the pattern / of the transposed pattern (a group
 *                plan is used from the same number of groups on as in the forward call,
 *                t_plans from 1024 groups on)
 * Rows (columns) without nonzeros get zero gradients.  Both calls queue on `stream`.
 */
int rode_hip_attention_backward_rows(int dtype, int heads, int M, int N, int nnz, int d, const int* d_row_offsets,
                                     const int* d_column_indices, const float* d_values, const float* d_probs,
                                     const float* d_row_stats, const float* d_grad_out, const float* d_out, const void* d_k,
                                     const void* d_v, float scale, const int* d_t_slot, float* d_grad_q, float* d_pairs,
                                     const rode_hip_plans* plans, void* stream);
int rode_hip_attention_backward_cols(int dtype, int heads, int M, int N, int nnz, int d, const int* d_t_row_offsets,
                                     const int* d_t_column_indices, const float* d_pairs, const float* d_grad_out,
                                     const void* d_q, float* d_grad_k, float* d_grad_v, const rode_hip_plans* t_plans, void* stream);

/*
 * The transposed pattern of a CSR matrix (M rows, N columns, nnz nonzeros): what the
 * gradients with respect to the column-side operands (SDDMM's rhs, SpMM's B) run on.  No
 * counterpart in the reference (forward-only, RoDe_SDDMM/rode_sddmm.py:194-248).
 *   d_perm               int[nnz] out: the nonzero indices ordered by (column, index), so
 *                        values_t = values[perm]; nonzeros of one column keep their input
 *                        order (rows ascending), the result is the same on every run
 *   d_t_row_offsets      int[N + 1] out
 *   d_t_column_indices   int[nnz] out: the row of nonzero perm[j]
 *   d_workspace          rode_hip_csr_transpose_workspace_bytes(nnz) bytes, 16-byte aligned
 * Column indices must lie in [0, N).  A stable radix sort, 4 bits per pass.
 */
size_t rode_hip_csr_transpose_workspace_bytes(int nnz);
int rode_hip_csr_transpose(int M, int N, int nnz, const int* d_row_offsets, const int* d_column_indices,
                           int* d_t_row_offsets, int* d_t_column_indices, int* d_perm, void* d_workspace,
                           size_t workspace_bytes, void* stream);

/*
 * d_dst[i] = d_src[d_index[i]] for i < n: the values of the transposed pattern,
 * values_t = values[perm], with perm from rode_hip_csr_transpose.  d_index and d_dst
 * 16-byte aligned, d_dst must not be d_src, every index in range of d_src.  No counterpart in
 * the reference (see rode_hip_csr_transpose).
 */
int rode_hip_permute_f32(int n, const float* d_src, const int* d_index, float* d_dst, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* RODE_HIP_H_ */
