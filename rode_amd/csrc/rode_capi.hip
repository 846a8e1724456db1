// extern "C" boundary of librode_hip.so plus the C++ entry points that keep the
// reference's signatures.  No kernel code here.
#include "../../include/rode_hip.h"
#include "../../include/RoDePreprocess.h"
#include "../../include/RoDeSddmm.h"
#include "../../include/RoDeSpmm.h"
#include "rode_internal.hpp"
#include "rode_items.hpp"

#include <cstdio>
#include <mutex>

static_assert(RODE_HIP_STATIC_MAX_ROWS == rode::kPreprocessStaticMaxRows, "header and library disagree");
static_assert(RODE_HIP_PLAN_RESIDUE_CHUNK == rode::kPlanResidueChunk && RODE_HIP_WINDOW_ROWS == rode::kResidueWindowRowsMax,
              "header and library disagree");

namespace {

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

} // namespace

extern "C" {

int rode_hip_version(void) { return (0 << 16) | 2; }

const char* rode_hip_error_string(int code) { return hipGetErrorString(static_cast<hipError_t>(code)); }

size_t rode_hip_preprocess_workspace_bytes(int M) { return rode::preprocess_workspace_bytes(M); }

int rode_hip_preprocess(int seg_length, int k_block, int vec_len, int M, const int* d_row_ptr, int* d_block_r_ind,
                        int* d_st_off, int* d_residue_r_ind, int* d_n_blk, int* d_n_res, int capacity_blocks,
                        void* d_workspace, size_t workspace_bytes, void* stream)
{
    if (seg_length <= 0 || k_block <= 0 || vec_len <= 0 || M < 0 || capacity_blocks < 0) return hipErrorInvalidValue;
    if (!d_row_ptr || !d_block_r_ind || !d_st_off || !d_residue_r_ind || !d_n_blk || !d_n_res || !d_workspace)
        return hipErrorInvalidValue;
    if (workspace_bytes < rode::preprocess_workspace_bytes(M) || (reinterpret_cast<uintptr_t>(d_workspace) & 7u))
        return hipErrorInvalidValue;
    return rode::preprocess_launch(seg_length, k_block, vec_len, M, d_row_ptr, d_block_r_ind, d_st_off,
                                   d_residue_r_ind, d_n_blk, d_n_res, d_workspace, capacity_blocks, as_stream(stream));
}

int rode_hip_preprocess_static(int seg_length, int k_block, int vec_len, int M, const int* d_row_ptr,
                               int* d_block_r_ind, int* d_st_off, int* d_residue_r_ind, int* d_n_blk, int* d_n_res,
                               int capacity_blocks, void* stream)
{
    if (seg_length <= 0 || k_block <= 0 || vec_len <= 0 || M < 0 || capacity_blocks < 0) return hipErrorInvalidValue;
    if (!d_row_ptr || !d_block_r_ind || !d_st_off || !d_residue_r_ind || !d_n_blk || !d_n_res)
        return hipErrorInvalidValue;
    if (M > RODE_HIP_STATIC_MAX_ROWS) return hipErrorOutOfMemory; // the fixed scratch cannot hold the scan of more rows
    void* ws = nullptr;
    const hipError_t e = rode::preprocess_static_workspace(&ws);
    if (e != hipSuccess) return e;
    // The two launches of a call (the fill of the scratch, then the kernel that uses it) are
    // queued together: host threads that call at the same time for one stream - the default
    // stream of RoDe_preprocess, say - get their calls one after the other on the GPU.
    static std::mutex queueing;
    std::lock_guard<std::mutex> lock(queueing);
    return rode::preprocess_launch(seg_length, k_block, vec_len, M, d_row_ptr, d_block_r_ind, d_st_off,
                                   d_residue_r_ind, d_n_blk, d_n_res, ws, capacity_blocks, as_stream(stream));
}

int rode_hip_preprocess_host(int seg_length, int k_block, int vec_len, int M, const int* h_row_ptr,
                             int* h_block_r_ind, int* h_st_off, int* h_residue_r_ind, int* h_n_blk, int* h_n_res)
{
    if (seg_length <= 0 || k_block <= 0 || vec_len <= 0 || M < 0) return hipErrorInvalidValue;
    if (!h_row_ptr || !h_block_r_ind || !h_st_off || !h_residue_r_ind || !h_n_blk || !h_n_res)
        return hipErrorInvalidValue;
    const long long nnz = h_row_ptr[M];
    const long long cap64 = (nnz + (long long)(vec_len - 1) * M) / seg_length + M;
    if (nnz < 0 || cap64 > 0x7ffffff0ll) return hipErrorInvalidValue;
    const int cap = (int)cap64;
    const size_t ws_bytes = rode::preprocess_workspace_bytes(M);
    // one device allocation: [workspace | row_ptr | block_r_ind | st_off | residue_r_ind | counts]
    const size_t ws_slots = (ws_bytes + 3) / 4;
    const size_t slots = ws_slots + (size_t)(M + 1) + (size_t)cap + 1 + (size_t)cap + 2 + (size_t)(M > 0 ? M : 1) + 2;
    int* d = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&d), slots * sizeof(int));
    if (e != hipSuccess) return e;
    int* d_rp = d + ws_slots;
    int* d_blk = d_rp + (M + 1);
    int* d_st = d_blk + cap + 1;
    int* d_res = d_st + cap + 2;
    int* d_cnt = d_res + (M > 0 ? M : 1);
    int cnt[2] = {0, 0};
    e = hipMemcpy(d_rp, h_row_ptr, sizeof(int) * (size_t)(M + 1), hipMemcpyHostToDevice);
    if (e == hipSuccess)
        e = rode::preprocess_launch(seg_length, k_block, vec_len, M, d_rp, d_blk, d_st, d_res, d_cnt, d_cnt + 1, d, cap,
                                    nullptr);
    if (e == hipSuccess) e = hipMemcpy(cnt, d_cnt, sizeof(cnt), hipMemcpyDeviceToHost); // waits for the kernels
    if (e == hipSuccess && cnt[0] > 0)
        e = hipMemcpy(h_block_r_ind, d_blk, sizeof(int) * (size_t)cnt[0], hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemcpy(h_st_off, d_st, sizeof(int) * ((size_t)cnt[0] + 1), hipMemcpyDeviceToHost);
    if (e == hipSuccess && cnt[1] > 0)
        e = hipMemcpy(h_residue_r_ind, d_res, sizeof(int) * (size_t)cnt[1], hipMemcpyDeviceToHost);
    (void)hipFree(d);
    if (e == hipSuccess) {
        *h_n_blk = cnt[0];
        *h_n_res = cnt[1];
    }
    return e;
}

size_t rode_hip_window_plan_bytes(int m2) { return m2 < 0 ? 0 : rode::window_plan_ints(m2) * sizeof(int); }

int rode_hip_window_plan(int m2, int dense_rows, const int* d_row_indices_residue, const int* d_row_offsets,
                         const int* d_column_indices, void* d_plan, size_t plan_bytes, int* h_counts, void* stream)
{
    if (m2 < 0 || dense_rows < 0 || !d_plan || !aligned16(d_plan)) return hipErrorInvalidValue;
    if (plan_bytes < rode_hip_window_plan_bytes(m2)) return hipErrorInvalidValue;
    if (m2 > 0 && (!d_row_indices_residue || !d_row_offsets || !d_column_indices)) return hipErrorInvalidValue;
    hipError_t e = rode::window_plan_launch(m2, dense_rows, d_row_indices_residue, d_row_offsets, d_column_indices,
                                            static_cast<int*>(d_plan), as_stream(stream));
    if (e == hipSuccess && h_counts) {
        e = hipMemcpyAsync(h_counts, d_plan, 4 * sizeof(int), hipMemcpyDeviceToHost, as_stream(stream));
        if (e == hipSuccess) e = hipStreamSynchronize(as_stream(stream));
    }
    return e;
}

size_t rode_hip_window_rows_bytes(int m2) { return m2 < 0 ? 0 : rode::window_plan_rows_bytes(m2); }

int rode_hip_window_rows(int m2, const int* d_row_indices_residue, const int* d_row_offsets,
                         const int* d_column_indices, const void* d_plan, void* d_rows, size_t rows_bytes, void* stream)
{
    if (m2 < 0 || !d_plan || !aligned16(d_plan)) return hipErrorInvalidValue;
    if (m2 == 0) return hipSuccess;
    if (!d_rows || !aligned16(d_rows) || rows_bytes < rode_hip_window_rows_bytes(m2)) return hipErrorInvalidValue;
    if (!d_row_indices_residue || !d_row_offsets || !d_column_indices) return hipErrorInvalidValue;
    return rode::window_plan_rows_launch(m2, d_row_indices_residue, d_row_offsets, d_column_indices,
                                         static_cast<const int*>(d_plan), d_rows, as_stream(stream));
}

size_t rode_hip_hub_plan_bytes(int M, int dense_rows, int nnz, int min_len)
{
    if (M < 0 || dense_rows < 0 || nnz < 0 || min_len < RODE_HIP_HUB_MIN_LEN) return 0;
    return rode::hub_plan_ints(M, dense_rows, nnz, min_len) * sizeof(int);
}

int rode_hip_hub_plan(int M, int dense_rows, int nnz, int min_len, const int* d_row_offsets,
                      const int* d_column_indices, void* d_plan, size_t plan_bytes, int* h_counts, void* stream)
{
    if (M < 0 || dense_rows < 0 || nnz < 0 || min_len < RODE_HIP_HUB_MIN_LEN || !d_plan || !aligned16(d_plan) || !h_counts)
        return hipErrorInvalidValue;
    if (plan_bytes < rode_hip_hub_plan_bytes(M, dense_rows, nnz, min_len)) return hipErrorInvalidValue;
    if (M > 0 && (!d_row_offsets || (nnz > 0 && !d_column_indices))) return hipErrorInvalidValue;
    // the hub rows first; once their number is known, a workgroup per hub row cuts it into pieces
    // (and may still mark the plan unusable: the header is read again afterwards)
    int* plan = static_cast<int*>(d_plan);
    hipError_t e = rode::hub_plan_launch(M, dense_rows, nnz, min_len, d_row_offsets, plan, as_stream(stream));
    for (int pass = 0; pass < 2 && e == hipSuccess; ++pass) {
        e = hipMemcpyAsync(h_counts, d_plan, 8 * sizeof(int), hipMemcpyDeviceToHost, as_stream(stream));
        if (e == hipSuccess) e = hipStreamSynchronize(as_stream(stream));
        if (e == hipSuccess && pass == 0) {
            if (h_counts[3] == 0 || h_counts[0] <= 0 || nnz == 0) break; // nothing to cut up
            e = rode::hub_pieces_launch(h_counts[0], dense_rows, d_row_offsets, d_column_indices, plan, as_stream(stream));
        }
    }
    return e;
}

size_t rode_hip_hub_workspace_bytes(const int* h_hub_counts, int n, int elem_bytes)
{
    if (!h_hub_counts || n <= 0 || (elem_bytes != 4 && elem_bytes != 8) || h_hub_counts[0] <= 0 || h_hub_counts[1] <= 0)
        return 0;
    const int merge = rode::hub_merge(n * elem_bytes / 4);
    return (size_t)h_hub_counts[0] * rode::hub_groups(h_hub_counts[1], merge) * n * elem_bytes;
}

size_t rode_hip_group_plan_bytes(int M) { return M < 0 ? 0 : rode::group_plan_ints(M) * sizeof(int); }

int rode_hip_group_plan(int M, const int* d_row_offsets, const int* d_column_indices, void* d_plan, size_t plan_bytes,
                        int* h_counts, void* stream)
{
    if (M < 0 || !d_plan || !aligned16(d_plan) || !h_counts || plan_bytes < rode_hip_group_plan_bytes(M))
        return hipErrorInvalidValue;
    if (M > 0 && (!d_row_offsets || !d_column_indices)) return hipErrorInvalidValue;
    hipError_t e = rode::group_plan_launch(M, d_row_offsets, d_column_indices, static_cast<int*>(d_plan), as_stream(stream));
    if (e == hipSuccess) e = hipMemcpyAsync(h_counts, d_plan, 4 * sizeof(int), hipMemcpyDeviceToHost, as_stream(stream));
    if (e == hipSuccess) e = hipStreamSynchronize(as_stream(stream));
    return e;
}

namespace {
// The caller's plans as the launchers take them; false if they cannot belong to these lists.
bool plan_ref(const rode_hip_plans* p, int m2, rode::PlanRef& plan)
{
    if (!p) return true;
    if (p->seg_length < 0) return false;
    plan.seg_length = p->seg_length;
    const bool window = p->window && p->window_rows; // (one without rows: the standard kernels do everything)
    if (p->groups) {
        // a group plan needs its header on the host, and excludes the other plans (their
        // kernels do not know which rows the group kernels have taken)
        if (!p->group_counts || !aligned16(p->groups) || window || p->hub) return false;
        if (p->group_counts[0] < 0 || p->group_counts[1] < 0 || p->group_counts[1] > p->group_counts[0]) return false;
        plan.groups = static_cast<const int*>(p->groups);
        plan.group_counts = p->group_counts;
    }
    if (p->hub) {
        // a hub plan needs its header on the host, and excludes a locality plan (the window
        // kernels do not know which rows the hub kernels have taken)
        if (!p->hub_counts || !aligned16(p->hub) || window) return false;
        if (p->hub_counts[0] < 0 || p->hub_counts[0] > p->hub_counts[4] || p->hub_counts[1] < 0 ||
            p->hub_counts[2] < RODE_HIP_HUB_MIN_LEN)
            return false;
        plan.hub = static_cast<const int*>(p->hub);
        plan.hub_counts = p->hub_counts;
        if (p->hub_workspace && aligned16(p->hub_workspace)) {
            plan.hub_workspace = p->hub_workspace;
            plan.hub_workspace_bytes = p->hub_workspace_bytes;
        }
    }
    if (!window) return true;
    if (!aligned16(p->window) || !aligned16(p->window_rows)) return false;
    if (p->window_counts && p->window_counts[0] != rode::plan_residue_chunks(m2)) return false;
    plan.dev = static_cast<const int*>(p->window);
    plan.rows = p->window_rows;
    plan.host_counts = p->window_counts;
    return true;
}
} // namespace

int rode_hip_spmm_ex(int dtype, int flags, int m1, int m2, int k, int n, const void* d_values,
                     const int* d_column_indices, const int* d_row_offsets, const int* d_row_indices1,
                     const int* d_row_indices2, const int* d_row_seg_st_offsets, const void* d_B, void* d_C,
                     void* stream1, void* stream2)
{
    return rode_hip_spmm_planned(dtype, flags, m1, m2, k, n, d_values, d_column_indices, d_row_offsets, d_row_indices1,
                                 d_row_indices2, d_row_seg_st_offsets, d_B, d_C, nullptr, stream1, stream2);
}

int rode_hip_spmm_planned(int dtype, int flags, int m1, int m2, int k, int n, const void* d_values,
                          const int* d_column_indices, const int* d_row_offsets, const int* d_row_indices1,
                          const int* d_row_indices2, const int* d_row_seg_st_offsets, const void* d_B, void* d_C,
                          const rode_hip_plans* plans, void* stream1, void* stream2)
{
    (void)k;
    constexpr int kKnown = RODE_SPMM_WHOLE_LISTS | RODE_SPMM_ONLY_BLOCK | RODE_SPMM_ONLY_RESIDUE | RODE_SPMM_ONLY_HUB |
                           RODE_SPMM_OVERWRITE;
    static_assert(RODE_SPMM_WHOLE_LISTS == rode::kSpmmWholeLists && RODE_SPMM_ONLY_BLOCK == rode::kSpmmOnlyBlock &&
                      RODE_SPMM_ONLY_RESIDUE == rode::kSpmmOnlyResidue && RODE_SPMM_ONLY_HUB == rode::kSpmmOnlyHub &&
                      RODE_SPMM_OVERWRITE == rode::kSpmmOverwrite,
                  "header and library disagree");
    if (m1 < 0 || m2 < 0 || (flags & ~kKnown)) return hipErrorInvalidValue;
    if ((flags & RODE_SPMM_OVERWRITE) && !(flags & RODE_SPMM_WHOLE_LISTS)) return hipErrorInvalidValue; // (one owner per row needs whole lists)
    const int only = flags & rode::kOnlyMask;
    if (only & (only - 1)) return hipErrorInvalidValue; // at most one ONLY bit
    if (m1 == 0 && m2 == 0) return hipSuccess;
    if (!aligned16(d_B) || !aligned16(d_C)) return hipErrorInvalidValue;
    hipStream_t s1 = as_stream(stream1), s2 = as_stream(stream2);
    rode::PlanRef plan;
    if (!plan_ref(plans, m2, plan)) return hipErrorInvalidValue;
    // the hub and group kernels replace work items of both lists: only with the complete decomposition
    if ((plan.hub || plan.groups) && !(flags & RODE_SPMM_WHOLE_LISTS)) return hipErrorInvalidValue;
    switch (dtype) {
    case RODE_DENSE_F32:
        return rode::spmm_launch<float>(m1, m2, n, d_row_indices1, d_row_indices2, d_row_seg_st_offsets, d_row_offsets,
                                        d_column_indices, static_cast<const float*>(d_values),
                                        static_cast<const float*>(d_B), static_cast<float*>(d_C), flags, plan, s1, s2);
    case RODE_DENSE_F16:
        return rode::spmm_launch<__half>(m1, m2, n, d_row_indices1, d_row_indices2, d_row_seg_st_offsets,
                                         d_row_offsets, d_column_indices, static_cast<const float*>(d_values),
                                         static_cast<const __half*>(d_B), static_cast<float*>(d_C), flags, plan, s1, s2);
    case RODE_DENSE_F64:
        return rode::spmm_launch<double>(m1, m2, n, d_row_indices1, d_row_indices2, d_row_seg_st_offsets,
                                         d_row_offsets, d_column_indices, static_cast<const double*>(d_values),
                                         static_cast<const double*>(d_B), static_cast<double*>(d_C), flags, plan, s1, s2);
    default: return hipErrorInvalidValue;
    }
}

int rode_hip_spmm_overwrite_limit(int m1, const rode_hip_plans* plans)
{
    const bool hub = plans && plans->hub && plans->hub_counts && plans->hub_counts[3] != 0 && plans->hub_counts[0] > 0;
    return m1 < 0 ? 0 : rode::spmm_overwrite_limit(m1, hub);
}

int rode_hip_spmm_f32(int m1, int m2, int k, int n, const float* d_values, const int* d_column_indices,
                      const int* d_row_offsets, const int* d_row_indices1, const int* d_row_indices2,
                      const int* d_row_seg_st_offsets, const float* d_B, float* d_C, void* stream1, void* stream2)
{
    return rode_hip_spmm_ex(RODE_DENSE_F32, 0, m1, m2, k, n, d_values, d_column_indices, d_row_offsets, d_row_indices1,
                            d_row_indices2, d_row_seg_st_offsets, d_B, d_C, stream1, stream2);
}

int rode_hip_spmm_clear_rows(int M, int n, int elem_bytes, const int* d_row_offsets, void* d_C, void* stream)
{
    if (M < 0 || n <= 0 || (elem_bytes != 4 && elem_bytes != 8) || ((size_t)n * elem_bytes) % 16 != 0)
        return hipErrorInvalidValue;
    if (M == 0) return hipSuccess;
    if (!d_row_offsets || !d_C || !aligned16(d_C)) return hipErrorInvalidValue;
    return rode::spmm_clear_rows_launch(M, (size_t)n * elem_bytes, d_row_offsets, d_C, as_stream(stream));
}

int rode_hip_spmm_f64(int m1, int m2, int k, int n, const double* d_values, const int* d_column_indices,
                      const int* d_row_offsets, const int* d_row_indices1, const int* d_row_indices2,
                      const int* d_row_seg_st_offsets, const double* d_B, double* d_C, void* stream1, void* stream2)
{
    return rode_hip_spmm_ex(RODE_DENSE_F64, 0, m1, m2, k, n, d_values, d_column_indices, d_row_offsets, d_row_indices1,
                            d_row_indices2, d_row_seg_st_offsets, d_B, d_C, stream1, stream2);
}

int rode_hip_spmm_f16(int m1, int m2, int k, int n, const float* d_values, const int* d_column_indices,
                      const int* d_row_offsets, const int* d_row_indices1, const int* d_row_indices2,
                      const int* d_row_seg_st_offsets, const void* d_B_half, float* d_C, void* stream1,
                      void* stream2)
{
    return rode_hip_spmm_ex(RODE_DENSE_F16, 0, m1, m2, k, n, d_values, d_column_indices, d_row_offsets, d_row_indices1,
                            d_row_indices2, d_row_seg_st_offsets, d_B_half, d_C, stream1, stream2);
}

int rode_hip_sddmm_planned(int dtype, int flags, int m1, int m2, int n, int k, const int* d_row_indices_block,
                           const int* d_row_indices_residue, const int* d_st_offsets, const int* d_row_offsets,
                           const int* d_column_indices, const float* d_values, const void* d_lhs_matrix,
                           const void* d_rhs_matrix, float* d_out, const rode_hip_plans* plans, void* stream1,
                           void* stream2)
{
    (void)n;
    if (m1 < 0 || m2 < 0 || (flags & ~rode::kOnlyMask) || (flags & (flags - 1))) return hipErrorInvalidValue;
    if (m1 == 0 && m2 == 0) return hipSuccess;
    if (!aligned16(d_lhs_matrix) || !aligned16(d_rhs_matrix)) return hipErrorInvalidValue;
    rode::PlanRef plan;
    if (!plan_ref(plans, m2, plan)) return hipErrorInvalidValue;
    plan.only = flags;
    switch (dtype) {
    case RODE_DENSE_F32:
        return rode::sddmm_launch<float>(m1, m2, k, d_row_indices_block, d_row_indices_residue, d_st_offsets,
                                         d_row_offsets, d_column_indices, d_values,
                                         static_cast<const float*>(d_lhs_matrix), static_cast<const float*>(d_rhs_matrix),
                                         d_out, plan, as_stream(stream1), as_stream(stream2));
    case RODE_DENSE_F16:
        return rode::sddmm_launch<__half>(m1, m2, k, d_row_indices_block, d_row_indices_residue, d_st_offsets,
                                          d_row_offsets, d_column_indices, d_values,
                                          static_cast<const __half*>(d_lhs_matrix),
                                          static_cast<const __half*>(d_rhs_matrix), d_out, plan, as_stream(stream1),
                                          as_stream(stream2));
    default: return hipErrorInvalidValue;
    }
}

int rode_hip_sddmm_f32(int m1, int m2, int n, int k, const int* d_row_indices_block, const int* d_row_indices_residue,
                       const int* d_st_offsets, const int* d_row_offsets, const int* d_column_indices,
                       const float* d_values, const float* d_lhs_matrix, const float* d_rhs_matrix, float* d_out,
                       void* stream1, void* stream2)
{
    return rode_hip_sddmm_planned(RODE_DENSE_F32, 0, m1, m2, n, k, d_row_indices_block, d_row_indices_residue, d_st_offsets,
                                  d_row_offsets, d_column_indices, d_values, d_lhs_matrix, d_rhs_matrix, d_out, nullptr,
                                  stream1, stream2);
}

int rode_hip_sddmm_f16(int m1, int m2, int n, int k, const int* d_row_indices_block, const int* d_row_indices_residue,
                       const int* d_st_offsets, const int* d_row_offsets, const int* d_column_indices,
                       const float* d_values, const void* d_lhs_half, const void* d_rhs_half, float* d_out,
                       void* stream1, void* stream2)
{
    return rode_hip_sddmm_planned(RODE_DENSE_F16, 0, m1, m2, n, k, d_row_indices_block, d_row_indices_residue, d_st_offsets,
                                  d_row_offsets, d_column_indices, d_values, d_lhs_half, d_rhs_half, d_out, nullptr,
                                  stream1, stream2);
}

int rode_hip_csr_softmax_f32(int M, const int* d_row_offsets, const float* d_in, float* d_out, float scale,
                             void* stream)
{
    if (M < 0 || !d_row_offsets || (M > 0 && (!d_in || !d_out))) return hipErrorInvalidValue;
    return rode::csr_softmax_launch(M, d_row_offsets, d_in, d_out, scale, as_stream(stream));
}

int rode_hip_csr_softmax_backward_f32(int M, const int* d_row_offsets, const float* d_p, const float* d_dp,
                                      float* d_ds, float scale, void* stream)
{
    if (M < 0 || !d_row_offsets || (M > 0 && (!d_p || !d_dp || !d_ds))) return hipErrorInvalidValue;
    return rode::csr_softmax_backward_launch(M, d_row_offsets, d_p, d_dp, d_ds, scale, as_stream(stream));
}

// (only a group plan means anything to the attention kernels)
static bool group_plan_only(const rode_hip_plans* plans, int rows, rode::PlanRef& plan)
{
    if (!plans || !plans->groups) return true;
    rode_hip_plans only_groups = {};
    only_groups.groups = plans->groups;
    only_groups.group_counts = plans->group_counts;
    return plan_ref(&only_groups, 0, plan) && plan.group_counts[0] == rode::row_groups(rows);
}

int rode_hip_attention_forward_batched(int dtype, int heads, int M, int N, int nnz, int d, const int* d_row_offsets,
                                       const int* d_column_indices, const float* d_values, const void* d_q, const void* d_k,
                                       const void* d_v, float scale, float* d_out, float* d_probs, float* d_row_stats,
                                       const rode_hip_plans* plans, void* stream)
{
    if (heads < 0 || M < 0 || N < 0 || nnz < 0 || !d_row_offsets) return hipErrorInvalidValue;
    if (d_row_stats && (!d_probs || ((uintptr_t)d_row_stats & 7) != 0)) return hipErrorInvalidValue;
    rode::PlanRef plan;
    if (!group_plan_only(plans, M, plan)) return hipErrorInvalidValue;
    if (d != 32 && d != 64 && d != 128) return hipErrorInvalidValue;
    if (M > 0 && heads > 0 && (!d_column_indices || !d_values || !d_q || !d_k || !d_v || !d_out)) return hipErrorInvalidValue;
    if (!aligned16(d_q) || !aligned16(d_k) || !aligned16(d_v) || !aligned16(d_out)) return hipErrorInvalidValue;
    if (dtype == RODE_DENSE_F32)
        return rode::attention_launch<float>(heads, M, N, nnz, d, d_row_offsets, d_column_indices, d_values,
                                             static_cast<const float*>(d_q), static_cast<const float*>(d_k),
                                             static_cast<const float*>(d_v), scale, d_out, d_probs, d_row_stats, plan,
                                             as_stream(stream));
    if (dtype == RODE_DENSE_F16)
        return rode::attention_launch<__half>(heads, M, N, nnz, d, d_row_offsets, d_column_indices, d_values,
                                              static_cast<const __half*>(d_q), static_cast<const __half*>(d_k),
                                              static_cast<const __half*>(d_v), scale, d_out, d_probs, d_row_stats, plan,
                                              as_stream(stream));
    return hipErrorInvalidValue;
}

int rode_hip_attention_forward(int dtype, int M, int d, const int* d_row_offsets, const int* d_column_indices,
                               const float* d_values, const void* d_q, const void* d_k, const void* d_v,
                               float scale, float* d_out, float* d_probs, const rode_hip_plans* plans, void* stream)
{
    // (one head: nobody asks where the next head's operands start)
    return rode_hip_attention_forward_batched(dtype, 1, M, 0, 0, d, d_row_offsets, d_column_indices, d_values, d_q, d_k, d_v,
                                              scale, d_out, d_probs, nullptr, plans, stream);
}

int rode_hip_attention_backward_rows(int dtype, int heads, int M, int N, int nnz, int d, const int* d_row_offsets,
                                     const int* d_column_indices, const float* d_values, const float* d_probs,
                                     const float* d_row_stats, const float* d_grad_out, const float* d_out, const void* d_k,
                                     const void* d_v, float scale, const int* d_t_slot, float* d_grad_q, float* d_pairs,
                                     const rode_hip_plans* plans, void* stream)
{
    if (heads < 0 || M < 0 || N < 0 || nnz < 0 || !d_row_offsets) return hipErrorInvalidValue;
    if (((uintptr_t)d_row_stats & 7) != 0) return hipErrorInvalidValue;
    rode::PlanRef plan;
    if (!group_plan_only(plans, M, plan)) return hipErrorInvalidValue;
    if (d != 32 && d != 64 && d != 128) return hipErrorInvalidValue;
    if (M > 0 && heads > 0 && (!d_column_indices || !d_values || !d_probs || !d_grad_out || !d_out || !d_k || !d_v || !d_t_slot ||
                               !d_grad_q || !d_pairs))
        return hipErrorInvalidValue;
    if (!aligned16(d_grad_out) || !aligned16(d_out) || !aligned16(d_k) || !aligned16(d_v) || !aligned16(d_grad_q) ||
        !aligned16(d_pairs))
        return hipErrorInvalidValue;
    if (dtype == RODE_DENSE_F32)
        return rode::attention_backward_rows_launch<float>(heads, M, N, nnz, d, d_row_offsets, d_column_indices, d_values, d_probs,
                                                           d_row_stats, d_grad_out, d_out, static_cast<const float*>(d_k),
                                                           static_cast<const float*>(d_v), scale, d_t_slot, d_grad_q, d_pairs,
                                                           plan, as_stream(stream));
    if (dtype == RODE_DENSE_F16)
        return rode::attention_backward_rows_launch<__half>(heads, M, N, nnz, d, d_row_offsets, d_column_indices, d_values, d_probs,
                                                            d_row_stats, d_grad_out, d_out, static_cast<const __half*>(d_k),
                                                            static_cast<const __half*>(d_v), scale, d_t_slot, d_grad_q, d_pairs,
                                                            plan, as_stream(stream));
    return hipErrorInvalidValue;
}

int rode_hip_attention_backward_cols(int dtype, int heads, int M, int N, int nnz, int d, const int* d_t_row_offsets,
                                     const int* d_t_column_indices, const float* d_pairs, const float* d_grad_out,
                                     const void* d_q, float* d_grad_k, float* d_grad_v, const rode_hip_plans* t_plans, void* stream)
{
    if (heads < 0 || M < 0 || N < 0 || nnz < 0 || !d_t_row_offsets) return hipErrorInvalidValue;
    rode::PlanRef plan;
    if (!group_plan_only(t_plans, N, plan)) return hipErrorInvalidValue;
    if (d != 32 && d != 64 && d != 128) return hipErrorInvalidValue;
    if (N > 0 && heads > 0 && (!d_t_column_indices || !d_pairs || !d_grad_out || !d_q || !d_grad_k || !d_grad_v))
        return hipErrorInvalidValue;
    if (!aligned16(d_grad_out) || !aligned16(d_q) || !aligned16(d_grad_k) || !aligned16(d_grad_v) || !aligned16(d_pairs))
        return hipErrorInvalidValue;
    if (dtype == RODE_DENSE_F32)
        return rode::attention_backward_cols_launch<float>(heads, M, N, nnz, d, d_t_row_offsets, d_t_column_indices, d_pairs,
                                                           d_grad_out, static_cast<const float*>(d_q), d_grad_k, d_grad_v, plan,
                                                           as_stream(stream));
    if (dtype == RODE_DENSE_F16)
        return rode::attention_backward_cols_launch<__half>(heads, M, N, nnz, d, d_t_row_offsets, d_t_column_indices, d_pairs,
                                                            d_grad_out, static_cast<const __half*>(d_q), d_grad_k, d_grad_v, plan,
                                                            as_stream(stream));
    return hipErrorInvalidValue;
}

size_t rode_hip_csr_transpose_workspace_bytes(int nnz) { return rode::csr_transpose_workspace_bytes(nnz); }

int rode_hip_permute_f32(int n, const float* d_src, const int* d_index, float* d_dst, void* stream)
{
    if (n < 0 || (n > 0 && (!d_src || !d_index || !d_dst || !aligned16(d_index) || !aligned16(d_dst) || d_src == d_dst)))
        return hipErrorInvalidValue;
    return rode::permute_launch(n, d_src, d_index, d_dst, as_stream(stream));
}

int rode_hip_csr_transpose(int M, int N, int nnz, const int* d_row_offsets, const int* d_column_indices,
                           int* d_t_row_offsets, int* d_t_column_indices, int* d_perm, void* d_workspace,
                           size_t workspace_bytes, void* stream)
{
    if (M < 0 || N < 0 || nnz < 0 || !d_t_row_offsets) return hipErrorInvalidValue;
    if (nnz > 0 && (!d_row_offsets || !d_column_indices || !d_t_column_indices || !d_perm || !d_workspace || N == 0 ||
                    M == 0 || !aligned16(d_workspace) || workspace_bytes < rode::csr_transpose_workspace_bytes(nnz)))
        return hipErrorInvalidValue;
    return rode::csr_transpose_launch(M, N, nnz, d_row_offsets, d_column_indices, d_t_row_offsets, d_t_column_indices,
                                      d_perm, d_workspace, as_stream(stream));
}

} // extern "C"

// ---- reference-signature C++ entry points ----------------------------------
// The reference functions return void and check nothing (RoDeSpmm.cu:505-508,
// RoDeSddmm.cu:503-512); a failure here is at least reported on stderr.
namespace {
void report(const char* fn, int code)
{
    if (code != 0) std::fprintf(stderr, "%s: %s\n", fn, rode_hip_error_string(code));
}
} // namespace

void RoDeSpmm_n32(int m1, int m2, int k, int n, const float* values, const int* column_indices, const int* row_offsets,
                  const int* row_indices1, const int* row_indices2, const int* row_seg_st_offsets, const float* B,
                  float* C, hipStream_t stream1, hipStream_t stream2)
{
    report("RoDeSpmm_n32", rode_hip_spmm_f32(m1, m2, k, n, values, column_indices, row_offsets, row_indices1,
                                             row_indices2, row_seg_st_offsets, B, C, stream1, stream2));
}

void RoDeSpmm_n128(int m1, int m2, int k, int n, const float* values, const int* column_indices, const int* row_offsets,
                   const int* row_indices1, const int* row_indices2, const int* row_seg_st_offsets, const float* B,
                   float* C, hipStream_t stream1, hipStream_t stream2)
{
    report("RoDeSpmm_n128", (n % 64) ? (int)hipErrorInvalidValue
                                     : rode_hip_spmm_f32(m1, m2, k, n, values, column_indices, row_offsets,
                                                         row_indices1, row_indices2, row_seg_st_offsets, B, C,
                                                         stream1, stream2));
}

void RoDeSpmm_n32(int m1, int m2, int k, int n, const double* values, const int* column_indices,
                  const int* row_offsets, const int* row_indices1, const int* row_indices2,
                  const int* row_seg_st_offsets, const double* B, double* C, hipStream_t stream1, hipStream_t stream2)
{
    report("RoDeSpmm_n32", rode_hip_spmm_f64(m1, m2, k, n, values, column_indices, row_offsets, row_indices1,
                                             row_indices2, row_seg_st_offsets, B, C, stream1, stream2));
}

void RoDeSpmm_n128(int m1, int m2, int k, int n, const double* values, const int* column_indices,
                   const int* row_offsets, const int* row_indices1, const int* row_indices2,
                   const int* row_seg_st_offsets, const double* B, double* C, hipStream_t stream1, hipStream_t stream2)
{
    report("RoDeSpmm_n128", (n % 64) ? (int)hipErrorInvalidValue
                                     : rode_hip_spmm_f64(m1, m2, k, n, values, column_indices, row_offsets,
                                                         row_indices1, row_indices2, row_seg_st_offsets, B, C,
                                                         stream1, stream2));
}

void RoDeSDDMM_n32(int m1, int m2, int n, int k, const int* row_indices_block, const int* row_indices_residue,
                   const int* st_offsets, const int* row_offsets, const int* column_indices, const float* values,
                   const float* lhs_matrix, const float* rhs_matrix, float* out, hipStream_t stream1,
                   hipStream_t stream2)
{
    report("RoDeSDDMM_n32", k != 32 ? (int)hipErrorInvalidValue
                                    : rode_hip_sddmm_f32(m1, m2, n, k, row_indices_block, row_indices_residue,
                                                         st_offsets, row_offsets, column_indices, values, lhs_matrix,
                                                         rhs_matrix, out, stream1, stream2));
}

void RoDeSDDMM_n128(int m1, int m2, int n, int k, const int* row_indices_block, const int* row_indices_residue,
                    const int* st_offsets, const int* row_offsets, const int* column_indices, const float* values,
                    const float* lhs_matrix, const float* rhs_matrix, float* out, hipStream_t stream1,
                    hipStream_t stream2)
{
    report("RoDeSDDMM_n128", k != 128 ? (int)hipErrorInvalidValue
                                      : rode_hip_sddmm_f32(m1, m2, n, k, row_indices_block, row_indices_residue,
                                                           st_offsets, row_offsets, column_indices, values,
                                                           lhs_matrix, rhs_matrix, out, stream1, stream2));
}

void RoDe_preprocess_cpu(int N_SEG, int blockX, int vecLen, int M, const int* row_ptr, int* block_r_ind, int* st_off,
                         int* residue_r_ind, int& n_blk, int& n_res)
{
    n_blk = n_res = 0;
    report("RoDe_preprocess_cpu", rode_hip_preprocess_host(N_SEG, blockX, vecLen, M, row_ptr, block_r_ind, st_off,
                                                           residue_r_ind, &n_blk, &n_res));
}

void RoDe_preprocess(int SegmentLength, int vectorLen, int KBLOCK, int M, const int* row_ptr, int* block_r_ind,
                     int* st_off, int* residue_r_ind, int& n_blk, int& n_res)
{
    n_blk = n_res = 0;
    report("RoDe_preprocess", rode_hip_preprocess_host(SegmentLength, KBLOCK, vectorLen, M, row_ptr, block_r_ind, st_off,
                                                       residue_r_ind, &n_blk, &n_res));
}

void RoDe_preprocess(int N_SEG, int blockX, int vecLen, int M, const int* row_ptr, int* block_r_ind, int* st_off,
                     int* residue_r_ind, int* n_blk, int* n_res)
{
    // The signature carries no capacity: the caller's arrays are trusted to hold
    // the result, as in the reference.  Nor does it carry scratch: the library's own fixed
    // array serves every matrix it can hold (no allocation, the call only queues kernels on
    // the default stream, where calls run one after the other whichever host thread made
    // them), a larger one gets scratch for the call.
    if (M <= RODE_HIP_STATIC_MAX_ROWS) {
        report("RoDe_preprocess", rode_hip_preprocess_static(N_SEG, blockX, vecLen, M, row_ptr, block_r_ind, st_off,
                                                             residue_r_ind, n_blk, n_res, 0x7fffffff, nullptr));
        return;
    }
    void* ws = nullptr;
    const size_t bytes = rode_hip_preprocess_workspace_bytes(M);
    hipError_t e = hipMalloc(&ws, bytes);
    if (e != hipSuccess) {
        report("RoDe_preprocess", (int)e);
        return;
    }
    report("RoDe_preprocess", rode_hip_preprocess(N_SEG, blockX, vecLen, M, row_ptr, block_r_ind, st_off,
                                                  residue_r_ind, n_blk, n_res, 0x7fffffff, ws, bytes, nullptr));
    (void)hipFree(ws); // waits for the queued kernels
}
