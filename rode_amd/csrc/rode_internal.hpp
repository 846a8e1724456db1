// Launch functions behind the C ABI (one per kernel family).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stddef.h>

namespace rode {

size_t preprocess_workspace_bytes(int M);

// Largest matrix the allocation-free preprocessing entry point takes (RODE_HIP_STATIC_MAX_ROWS).
constexpr int kPreprocessStaticMaxRows = 4 * 1024 * 1024;
// Device address of the current GPU's static preprocessing scratch.
hipError_t preprocess_static_workspace(void** ptr);

hipError_t preprocess_launch(int seg, int kblock, int veclen, int M, const int* row_ptr, int* block_r_ind,
                             int* st_off, int* residue_r_ind, int* n_blk, int* n_res, void* workspace,
                             int capacity_blocks, hipStream_t stream);

// T = dense operand type; values, accumulators and C are float for T = float / __half
// and double for T = double.
template <typename T> struct SpmmAcc { using type = float; };
template <> struct SpmmAcc<double> { using type = double; };

// flags: the RODE_SPMM_* bits of the C ABI
constexpr int kSpmmWholeLists = 1, kSpmmOnlyBlock = 2, kSpmmOnlyResidue = 4, kSpmmOnlyHub = 8, kSpmmOverwrite = 16;
constexpr int kOnlyMask = kSpmmOnlyBlock | kSpmmOnlyResidue | kSpmmOnlyHub;

// A locality plan (rode_plan.hip): device array, and optionally a host copy of its four
// header ints (chunk counts), with which launches that have nothing to do are left out.
struct PlanRef {
    const int* dev = nullptr;         // descriptors
    const void* rows = nullptr;       // planned rows of the chunks with a window
    const int* host_counts = nullptr;
    // A hub plan (rode_hub.hip) and the host copy of its eight header ints (required with it).
    const int* hub = nullptr;
    const int* hub_counts = nullptr;
    // SpMM only: room for one partial row of C per (slab, hub row), or null (atomics instead).
    void* hub_workspace = nullptr;
    size_t hub_workspace_bytes = 0;
    // A group plan (rode_group.hip) and the host copy of its four header ints (required with it).
    const int* groups = nullptr;
    const int* group_counts = nullptr;
    // SDDMM: the RODE_SPMM_ONLY_* bits of the call (SpMM carries them in its flags)
    int only = 0;
    // Segment length of the decomposition the lists were made with, 0: not known
    int seg_length = 0;
};

hipError_t group_plan_launch(int M, const int* row_ptr, const int* col, int* plan, hipStream_t stream);

// The attention kernels take nheads problems on one pattern of M rows, N columns and nnz
// nonzeros per launch (operands head after head).  (plan: only a group plan is used)
template <typename T>
hipError_t attention_launch(int nheads, int M, int N, int nnz, int d, const int* row_ptr, const int* col, const float* val,
                            const T* q, const T* k, const T* v, float scale, float* out, float* probs, float* row_stats,
                            PlanRef plan, hipStream_t stream);

// Gradient of the attention kernel (rode_attention_backward.hip): the row pass over the
// pattern, then the column pass over the transposed pattern (plan: only a group plan is used,
// of the pattern the pass walks).  pz: nheads x 2 * nnz floats, written by the first in the
// order of the transposed pattern (t_slot: every nonzero's slot there), read by the second.
// row_stats: NULL when probs holds probabilities, else what attention_launch wrote beside the
// scores in probs.
template <typename T>
hipError_t attention_backward_rows_launch(int nheads, int M, int N, int nnz, int d, const int* row_ptr, const int* col,
                                          const float* val, const float* probs, const float* row_stats, const float* g,
                                          const float* out, const T* k, const T* v, float scale, const int* t_slot, float* dq,
                                          float* pz, PlanRef plan, hipStream_t stream);
template <typename T>
hipError_t attention_backward_cols_launch(int nheads, int M, int N, int nnz, int d, const int* t_row_ptr, const int* t_col,
                                          const float* pz, const float* g, const T* q, float* dk, float* dv, PlanRef plan,
                                          hipStream_t stream);

hipError_t hub_plan_launch(int M, int dense_rows, int nnz, int min_len, const int* row_ptr, int* plan, hipStream_t stream);
hipError_t hub_pieces_launch(int hub_rows, int dense_rows, const int* row_ptr, const int* col, int* plan, hipStream_t stream);

size_t window_plan_ints(int m2);
size_t window_plan_rows_bytes(int m2);
hipError_t window_plan_launch(int m2, int dense_rows, const int* residue_rows, const int* row_ptr, const int* col,
                              int* plan, hipStream_t stream);
hipError_t window_plan_rows_launch(int m2, const int* residue_rows, const int* row_ptr, const int* col, const int* plan,
                                   void* rows, hipStream_t stream);

// (rode_spmm.hip) which rows an SpMM call under kSpmmOverwrite stores instead of adding to
int spmm_overwrite_limit(int m1, bool hub_plan);
template <typename T>
hipError_t spmm_launch(int m1, int m2, int n, const int* block_rows, const int* residue_rows, const int* st_off,
                       const int* row_ptr, const int* col, const typename SpmmAcc<T>::type* val, const T* B,
                       typename SpmmAcc<T>::type* C, int flags, PlanRef plan, hipStream_t s1, hipStream_t s2);

// the window kernel of SpMM over the planned chunks of the residue list (T = float or __half)
template <typename T>
hipError_t spmm_window_launch(int m2, int n, int owned_slots, const int* col, const float* val, const T* B, float* C,
                              const int* plan, const void* plan_rows, hipStream_t stream);

hipError_t spmm_clear_rows_launch(int M, size_t row_bytes, const int* row_ptr, void* C, hipStream_t stream);

template <typename T>
hipError_t sddmm_launch(int m1, int m2, int k, const int* block_rows, const int* residue_rows, const int* st_off,
                        const int* row_ptr, const int* col, const float* val, const T* lhs, const T* rhs,
                        float* out, PlanRef plan, hipStream_t s1, hipStream_t s2);

// the window kernel of SDDMM over the planned chunks of the residue list
template <typename T>
hipError_t sddmm_window_launch(int m2, int k, const int* col, const float* val, const T* lhs, const T* rhs, float* out,
                               const int* plan, const void* plan_rows, hipStream_t stream);

hipError_t permute_launch(int n, const float* src, const int* index, float* dst, hipStream_t stream);
size_t csr_transpose_workspace_bytes(int nnz);
hipError_t csr_transpose_launch(int M, int N, int nnz, const int* row_ptr, const int* col, int* t_row_ptr, int* t_col,
                                int* perm, void* workspace, hipStream_t stream);
hipError_t csr_softmax_launch(int M, const int* row_ptr, const float* in, float* out, float scale,
                              hipStream_t stream);
hipError_t csr_softmax_backward_launch(int M, const int* row_ptr, const float* p, const float* dp, float* ds,
                                       float scale, hipStream_t stream);

} // namespace rode
