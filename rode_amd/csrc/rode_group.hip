// Group plan: groups of kGroupRows adjacent rows whose longest runs of consecutive column
// indices overlap for the most part (sliding-window attention masks, dense bands, block
// structure).  The group kernels (spmm_group_kernel, sddmm_group_kernel,
// attention_group_kernel) walk the range of columns the runs cover between them once for
// all rows of a group: one load of a dense row serves every row of the group, and the dense
// rows of the range are consecutive in memory, so no column index is read for them.  The
// nonzeros of a row outside its run are processed as usual, by the same workgroup; the
// standard kernels leave grouped rows out.  No counterpart in the reference, whose kernels
// gather the dense row of every nonzero of every row (RoDe_SpMM/RoDeSpmm.cu:140-160,
// RoDe_SDDMM/RoDeSddmm.cu:96-140).  The plan changes no result.
//
//   group_runs_kernel   per row: its longest run of consecutive columns (first column,
//                       length, position in the row); one wave per row.
//   group_desc_kernel   per group: the columns its rows' runs have in common and the range
//                       they cover between them; the group is kept if the common part has
//                       at least kGroupMinRun columns and holds at least three quarters of
//                       the group's nonzeros, and the runs start and end within 255 columns
//                       of each other.
#include "rode_items.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

constexpr int kGroupMinRun = 64;

// One wave per row, 64 nonzeros per step: lane e flags its nonzero when a run starts there
// (its column is not its predecessor's plus one); the ballot of the flags is walked bit by
// bit - the same in every lane, on the scalar unit - closing a run at every flag.  Of runs
// of equal length the first counts.
__global__ void __launch_bounds__(kWgThreads)
group_runs_kernel(int M, const int* __restrict__ row_ptr, const int* __restrict__ col, int* __restrict__ runs)
{
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
    const long long row_ll = (long long)blockIdx.x * kWavesPerWg + wave;
    if (row_ll >= M) return;
    const int row = (int)row_ll;
    const int s = row_ptr[row], e = row_ptr[row + 1];
    int best_first = 0, best_len = 0, best_pos = 0;
    int run_first = 0, run_pos = 0; // the run that is open: its first column, its position in the row
    for (int base = s; base < e; base += kWave) {
        const int i = base + lane;
        const bool live = i < e;
        const int c = live ? col[i] : 0;
        const bool starts = live && (i == s || col[i - 1] + 1 != c);
        unsigned long long flags = __ballot(starts);
        while (flags) {
            const int f = __builtin_ctzll(flags);
            flags &= flags - 1;
            const int pos = base - s + f;
            if (pos - run_pos > best_len) {
                best_first = run_first;
                best_len = pos - run_pos;
                best_pos = run_pos;
            }
            run_first = __builtin_amdgcn_readlane(c, f);
            run_pos = pos;
        }
    }
    if (e - s - run_pos > best_len) {
        best_first = run_first;
        best_len = e - s - run_pos;
        best_pos = run_pos;
    }
    if (lane == 0) {
        runs[3 * row] = best_first;
        runs[3 * row + 1] = best_len;
        runs[3 * row + 2] = best_pos;
    }
}

__global__ void __launch_bounds__(kWgThreads)
group_desc_kernel(int groups, const int* __restrict__ row_ptr, const int* __restrict__ runs, int* __restrict__ plan)
{
    const int g = blockIdx.x * kWgThreads + threadIdx.x;
    if (g >= groups) return;
    RowGroup d;
    int lo = 0, hi = 0x7fffffff;           // the columns all four runs hold
    int first = 0x7fffffff, last = 0;      // the columns any of them holds
    long long slots = 0;
#pragma unroll
    for (int r = 0; r < kGroupRows; ++r) {
        const int row = g * kGroupRows + r;
        const int a = runs[3 * row], b = a + runs[3 * row + 1];
        lo = max(lo, a);
        hi = min(hi, b);
        first = min(first, a);
        last = max(last, b);
        slots += row_ptr[row + 1] - row_ptr[row];
    }
    const int common = hi - lo;
    // kept: a long common part that holds most of the group's nonzeros, and runs that start and
    // end within 255 columns of each other (what a byte per row can say)
    const bool keep = common >= kGroupMinRun && 4ll * kGroupRows * common >= 3 * slots && lo - first <= 255 && last - hi <= 255;
    d.lo = keep ? first : 0;
    d.len = keep ? last - first : 0;
    d.heads = d.tails = 0u;
#pragma unroll
    for (int r = 0; r < kGroupRows; ++r) {
        const int row = g * kGroupRows + r;
        const int a = runs[3 * row], b = a + runs[3 * row + 1];
        d.pos[r] = keep ? runs[3 * row + 2] : 0;
        if (keep) {
            d.heads |= (unsigned)(a - first) << (8 * r);
            d.tails |= (unsigned)(last - b) << (8 * r);
        }
    }
    reinterpret_cast<RowGroup*>(plan + kGroupHeaderInts)[g] = d;
    if (keep) {
        atomicAdd(plan + 1, 1);
        atomicSub(plan + 2, kGroupRows);
    }
}

__global__ void group_header_kernel(int M, int groups, int* __restrict__ plan)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        plan[0] = groups;
        plan[1] = 0;
        plan[2] = M; // rows outside the groups with a run: counted down as groups are kept
        plan[3] = 0;
    }
}

} // namespace

hipError_t group_plan_launch(int M, const int* row_ptr, const int* col, int* plan, hipStream_t stream)
{
    const int groups = row_groups(M);
    group_header_kernel<<<1, kWave, 0, stream>>>(M, groups, plan);
    if (groups > 0) {
        int* runs = plan + kGroupHeaderInts + (size_t)groups * (sizeof(RowGroup) / sizeof(int)); // scratch behind the table
        group_runs_kernel<<<(M + kWavesPerWg - 1) / kWavesPerWg, kWgThreads, 0, stream>>>(M, row_ptr, col, runs);
        group_desc_kernel<<<(groups + kWgThreads - 1) / kWgThreads, kWgThreads, 0, stream>>>(groups, row_ptr, runs, plan);
    }
    return hipGetLastError();
}

} // namespace rode
