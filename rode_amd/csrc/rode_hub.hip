// Hub plan: the rows with at least `min_len` nonzero slots, and for each of them where
// its nonzeros of every column slab start (see the hub plan in rode_items.hpp for what the
// kernels do with it).  No counterpart in the reference: its kernels gather every dense
// row from memory whenever a nonzero references it (RoDe_SpMM/RoDeSpmm.cu:140-160,
// RoDe_SDDMM/RoDeSddmm.cu:96-140).  The plan changes no result.
//
//   hub_count_kernel, hub_scan_kernel, hub_write_kernel
//                      the hub rows, in ascending order: counted per block of 2048 rows, a
//                      prefix sum over the blocks (one workgroup; it also fills in the
//                      header), then every block writes its hub rows to its place.
//   hub_pieces_kernel  one workgroup per hub row: a binary search per slab boundary in the
//                      row's column indices, and a pass over the row that checks that its
//                      columns ascend (if one does not, the plan is marked unusable).
#include "rode_items.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

constexpr int kSelectThreads = 1024;

__device__ __forceinline__ bool is_hub(const int* __restrict__ row_ptr, int row, int min_len)
{
    const int s = row_ptr[row];
    return row_ptr[row + 1] - s + (s & (kVecLen - 1)) >= min_len;
}

// Hub rows among the rows [first, first + 256 * kSelectRows) of one workgroup, thread t
// looking at kSelectRows consecutive rows: counted, or written in order to their place.
constexpr int kSelectRows = kHubSelectBlockRows / kWgThreads;

__global__ void __launch_bounds__(kWgThreads)
hub_count_kernel(int M, int min_len, const int* __restrict__ row_ptr, int* __restrict__ block_counts)
{
    __shared__ int wave_sum[kWavesPerWg];
    const int first = (blockIdx.x * kWgThreads + threadIdx.x) * kSelectRows;
    int count = 0;
    for (int r = first; r < min(M, first + kSelectRows); ++r) count += is_hub(row_ptr, r, min_len) ? 1 : 0;
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) count += __shfl_xor(count, d, kWave);
    if (threadIdx.x % kWave == 0) wave_sum[threadIdx.x / kWave] = count;
    __syncthreads();
    if (threadIdx.x == 0) {
        int total = 0;
        for (int w = 0; w < kWavesPerWg; ++w) total += wave_sum[w];
        block_counts[blockIdx.x] = total;
    }
}

// One workgroup: exclusive prefix over the block counts (in place) and the header.
__global__ void __launch_bounds__(kSelectThreads)
hub_scan_kernel(int nblocks, int dense_rows, int room, int min_len, int* __restrict__ block_counts, int* __restrict__ plan)
{
    __shared__ int partial[kSelectThreads];
    const int per = (nblocks + kSelectThreads - 1) / kSelectThreads;
    const int lo = min(nblocks, (int)threadIdx.x * per), hi = min(nblocks, lo + per);
    int count = 0;
    for (int i = lo; i < hi; ++i) count += block_counts[i];
    partial[threadIdx.x] = count;
    __syncthreads();
    for (int d = 1; d < kSelectThreads; d <<= 1) {
        const int add = (int)threadIdx.x >= d ? partial[threadIdx.x - d] : 0;
        __syncthreads();
        partial[threadIdx.x] += add;
        __syncthreads();
    }
    int run = partial[threadIdx.x] - count;
    for (int i = lo; i < hi; ++i) {
        const int c = block_counts[i];
        block_counts[i] = run;
        run += c;
    }
    if (threadIdx.x == kSelectThreads - 1) {
        const int total = partial[kSelectThreads - 1];
        plan[0] = min(total, room);
        plan[1] = hub_slabs(dense_rows);
        plan[2] = min_len;
        plan[3] = total <= room ? 1 : 0; // (room = hub_room(nnz, min_len) always suffices)
        plan[4] = room;
        plan[5] = plan[6] = plan[7] = 0;
    }
}

__global__ void __launch_bounds__(kWgThreads)
hub_write_kernel(int M, int room, int min_len, const int* __restrict__ row_ptr, const int* __restrict__ block_starts,
                 int* __restrict__ plan)
{
    __shared__ int thread_count[kWgThreads];
    const int first = (blockIdx.x * kWgThreads + threadIdx.x) * kSelectRows;
    int count = 0;
    for (int r = first; r < min(M, first + kSelectRows); ++r) count += is_hub(row_ptr, r, min_len) ? 1 : 0;
    thread_count[threadIdx.x] = count;
    __syncthreads();
    if (count == 0) return;
    int at = block_starts[blockIdx.x];
    for (int t = 0; t < (int)threadIdx.x; ++t) at += thread_count[t]; // (hub rows are few: hardly any thread gets here)
    int* rows = plan + kHubHeaderInts;
    for (int r = first; r < min(M, first + kSelectRows); ++r)
        if (is_hub(row_ptr, r, min_len)) {
            if (at < room) rows[at] = r;
            ++at;
        }
}

__global__ void __launch_bounds__(kWgThreads)
hub_pieces_kernel(int dense_rows, const int* __restrict__ row_ptr, const int* __restrict__ col, int* __restrict__ plan)
{
    const int h = blockIdx.x;
    if (h >= plan[0]) return;
    const int slabs = plan[1];
    const int row = plan[kHubHeaderInts + h];
    const int s = row_ptr[row], e = row_ptr[row + 1];
    int* pieces = plan + kHubHeaderInts + plan[4] + (size_t)h * (slabs + 1);
    // start of slab b: the first nonzero of the row whose column is >= b * kHubSlabRows
    for (int b = threadIdx.x; b <= slabs; b += kWgThreads) {
        const long long bound = (long long)b * kHubSlabRows;
        int lo = s, hi = e; // columns before lo are < bound, columns from hi on are >= bound
        while (lo < hi) {
            const int mid = lo + ((hi - lo) >> 1);
            if (col[mid] < bound) lo = mid + 1; else hi = mid;
        }
        pieces[b] = b == slabs ? e : lo;
    }
    bool ascending = true;
    for (int i = s + threadIdx.x; i + 1 < e; i += kWgThreads) ascending = ascending && col[i] <= col[i + 1];
    // also: every column is inside the operand (else a piece past the last slab would be lost)
    for (int i = s + threadIdx.x; i < e; i += kWgThreads) ascending = ascending && (unsigned)col[i] < (unsigned)dense_rows;
    if (!ascending) plan[3] = 0;
}

} // namespace

// First the hub rows (their number is then in plan[0]), then - for that many rows - their pieces.
hipError_t hub_plan_launch(int M, int dense_rows, int nnz, int min_len, const int* row_ptr, int* plan, hipStream_t stream)
{
    const int room = hub_room(nnz, min_len);
    const int nblocks = (M + kHubSelectBlockRows - 1) / kHubSelectBlockRows;
    int* block_counts = plan + hub_table_ints(dense_rows, nnz, min_len); // scratch behind the tables
    hub_count_kernel<<<max(nblocks, 1), kWgThreads, 0, stream>>>(M, min_len, row_ptr, block_counts);
    hub_scan_kernel<<<1, kSelectThreads, 0, stream>>>(nblocks, dense_rows, room, min_len, block_counts, plan);
    hub_write_kernel<<<max(nblocks, 1), kWgThreads, 0, stream>>>(M, room, min_len, row_ptr, block_counts, plan);
    return hipGetLastError();
}

hipError_t hub_pieces_launch(int hub_rows, int dense_rows, const int* row_ptr, const int* col, int* plan, hipStream_t stream)
{
    if (hub_rows <= 0) return hipSuccess;
    hub_pieces_kernel<<<hub_rows, kWgThreads, 0, stream>>>(dense_rows, row_ptr, col, plan);
    return hipGetLastError();
}

} // namespace rode
