// Transposed pattern of a CSR matrix: the nonzeros ordered by (column, row), as a
// permutation of their indices, with the row offsets and column indices of the
// transposed matrix.  The gradients with respect to the column-side operands of SDDMM and
// SpMM are products on that pattern.  No counterpart in the reference (its op is
// forward-only, RoDe_SDDMM/rode_sddmm.py:194-248).
//
// A stable least-significant-digit radix sort of (column, nonzero index) pairs, 4 bits
// per pass, as many passes as the column count has hex digits.  Stable, so nonzeros of one
// column stay in index order (= row order, and the input order of duplicates): the
// result is unique, the same on every run.  Per pass:
//   1. digit_count_kernel  - per block of 2048 pairs, how many carry each of the 16 digits;
//   2. digit_scan_kernel   - exclusive prefix over (digit, block): where each block's
//                            pairs of each digit start in the output;
//   3. digit_scatter_kernel- every pair to that start + the number of pairs of the same
//                            digit before it in its block (ballot ranks inside a wave, a
//                            small LDS table across the steps and waves of the block).
// Then the rows of the permuted nonzeros (a binary search in the row offsets each) are the
// transposed column indices, and the places where the sorted column changes are the
// transposed row offsets.
#include "rode_device.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

constexpr int kSortItems = 8;                        // pairs per thread
constexpr int kSortBlock = kWgThreads * kSortItems;  // pairs per workgroup
constexpr int kRadixBits = 4;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kScanThreads = 1024;

// Pair i of thread t of a block is element block * 2048 + i * 256 + t: loads are
// coalesced, and element order is (step i, wave, lane).
__device__ __forceinline__ int pair_index(int block, int i) { return block * kSortBlock + i * kWgThreads + (int)threadIdx.x; }

__global__ void __launch_bounds__(kWgThreads)
digit_count_kernel(const int* __restrict__ keys, int n, int shift, int nblocks, int* __restrict__ hist)
{
    __shared__ int wave_count[kWavesPerWg][kRadix];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    int count[kRadix]; // the same in every lane of the wave
#pragma unroll
    for (int b = 0; b < kRadix; ++b) count[b] = 0;
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
        const int e = pair_index(blockIdx.x, i);
        const int digit = e < n ? (keys[e] >> shift) & (kRadix - 1) : -1;
#pragma unroll
        for (int b = 0; b < kRadix; ++b) count[b] += __popcll(__ballot(digit == b));
    }
    if (lane < kRadix) {
        int mine = 0;
#pragma unroll
        for (int b = 0; b < kRadix; ++b) mine = lane == b ? count[b] : mine;
        wave_count[wave][lane] = mine;
    }
    __syncthreads();
    if (threadIdx.x < kRadix) {
        int total = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerWg; ++w) total += wave_count[w][threadIdx.x];
        hist[threadIdx.x * nblocks + blockIdx.x] = total;
    }
}

// Exclusive prefix sum of `len` ints in place, one workgroup.
__global__ void __launch_bounds__(kScanThreads)
digit_scan_kernel(int* __restrict__ data, int len)
{
    __shared__ int partial[kScanThreads];
    const int per = (len + kScanThreads - 1) / kScanThreads;
    const int lo = min(len, (int)threadIdx.x * per), hi = min(len, lo + per);
    int sum = 0;
    for (int i = lo; i < hi; ++i) sum += data[i];
    partial[threadIdx.x] = sum;
    __syncthreads();
    // Hillis-Steele over the 1024 partial sums
    for (int d = 1; d < kScanThreads; d <<= 1) {
        const int add = (int)threadIdx.x >= d ? partial[threadIdx.x - d] : 0;
        __syncthreads();
        partial[threadIdx.x] += add;
        __syncthreads();
    }
    int run = partial[threadIdx.x] - sum; // exclusive
    for (int i = lo; i < hi; ++i) {
        const int v = data[i];
        data[i] = run;
        run += v;
    }
}

// vals_in == nullptr: the value of pair e is e (first pass).
__global__ void __launch_bounds__(kWgThreads)
digit_scatter_kernel(const int* __restrict__ keys_in, const int* __restrict__ vals_in, int n, int shift, int nblocks,
                     const int* __restrict__ starts, int* __restrict__ keys_out, int* __restrict__ vals_out)
{
    // before[i][w][b]: pairs of digit b in the steps and waves of this block that come before (step i, wave w)
    __shared__ int before[kSortItems][kWavesPerWg][kRadix];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    int key[kSortItems], digit[kSortItems], rank[kSortItems];
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
        const int e = pair_index(blockIdx.x, i);
        key[i] = e < n ? keys_in[e] : 0;
        digit[i] = e < n ? (key[i] >> shift) & (kRadix - 1) : -1;
        int my_rank = 0, my_count = 0;
#pragma unroll
        for (int b = 0; b < kRadix; ++b) {
            const unsigned long long mask = __ballot(digit[i] == b);
            if (digit[i] == b) my_rank = __popcll(mask & ((1ull << lane) - 1ull));
            if (lane == b) my_count = __popcll(mask);
        }
        rank[i] = my_rank;
        if (lane < kRadix) before[i][wave][lane] = my_count; // counts for now
    }
    __syncthreads();
    if (threadIdx.x < kRadix) {
        int run = starts[threadIdx.x * nblocks + blockIdx.x];
        for (int i = 0; i < kSortItems; ++i) {
            for (int w = 0; w < kWavesPerWg; ++w) {
                const int c = before[i][w][threadIdx.x];
                before[i][w][threadIdx.x] = run;
                run += c;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
        const int e = pair_index(blockIdx.x, i);
        if (e < n) {
            const int to = before[i][wave][digit[i]] + rank[i];
            keys_out[to] = key[i];
            vals_out[to] = vals_in ? vals_in[e] : e;
        }
    }
}

// t_col[j] = row of nonzero perm[j]; t_row_ptr from the places where the sorted column changes.
__global__ void __launch_bounds__(kWgThreads)
transposed_arrays_kernel(int M, int N, int nnz, const int* __restrict__ row_ptr, const int* __restrict__ sorted_cols,
                         const int* __restrict__ perm, int* __restrict__ t_row_ptr, int* __restrict__ t_col)
{
    const int j = blockIdx.x * kWgThreads + threadIdx.x;
    if (j >= nnz) return;
    const int idx = perm[j];
    int lo = 0, hi = M; // row_ptr[lo] <= idx < row_ptr[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (row_ptr[mid] <= idx) lo = mid; else hi = mid;
    }
    t_col[j] = lo;
    // transposed rows (c_prev, c] start at j; the last nonzero also closes the rows after its column
    const int c = sorted_cols[j];
    const int c_prev = j > 0 ? sorted_cols[j - 1] : -1;
    for (int r = c_prev + 1; r <= c; ++r) t_row_ptr[r] = j;
    if (j == nnz - 1)
        for (int r = c + 1; r <= N; ++r) t_row_ptr[r] = nnz;
}

__global__ void fill_kernel(int* __restrict__ p, int n, int v)
{
    const int i = blockIdx.x * kWgThreads + threadIdx.x;
    if (i < n) p[i] = v;
}

inline int sort_blocks(int nnz) { return (nnz + kSortBlock - 1) / kSortBlock; }

inline size_t round16(size_t b) { return (b + 15) & ~(size_t)15; }

} // namespace

size_t csr_transpose_workspace_bytes(int nnz)
{
    // two key buffers, one value buffer (the other one is the caller's perm), digit table
    return 3 * round16((size_t)max(nnz, 1) * 4) + round16((size_t)kRadix * max(sort_blocks(nnz), 1) * 4);
}

namespace {

// dst[i] = src[index[i]]: four outputs per thread, the indices and the results as 128-bit
// accesses, the four reads wherever the indices point.
__global__ void __launch_bounds__(kWgThreads)
permute_kernel(int n, const float* __restrict__ src, const int* __restrict__ index, float* __restrict__ dst)
{
    // (neighbouring outputs read neighbouring places of src when the pattern has any locality:
    // a contiguous range of workgroups per XCD keeps those re-reads in one L2)
    const long long i0 = ((long long)xcd_logical_block(blockIdx.x, gridDim.x) * kWgThreads + threadIdx.x) * 4;
    if (i0 + 3 < n) {
        const int4 at = *reinterpret_cast<const int4*>(index + i0);
        *reinterpret_cast<float4*>(dst + i0) = make_float4(src[at.x], src[at.y], src[at.z], src[at.w]);
    } else {
        for (long long i = i0; i < n; ++i) dst[i] = src[index[i]];
    }
}

} // namespace

// The values of a transposed pattern: values_t = values[perm] (perm from csr_transpose_launch).
hipError_t permute_launch(int n, const float* src, const int* index, float* dst, hipStream_t stream)
{
    if (n <= 0) return hipSuccess;
    const long long threads = ((long long)n + 3) / 4;
    const long long wgs = ((threads + kWgThreads - 1) / kWgThreads + kXcds - 1) / kXcds * kXcds;
    permute_kernel<<<(int)wgs, kWgThreads, 0, stream>>>(n, src, index, dst);
    return hipGetLastError();
}

hipError_t csr_transpose_launch(int M, int N, int nnz, const int* row_ptr, const int* col, int* t_row_ptr, int* t_col,
                                int* perm, void* workspace, hipStream_t stream)
{
    if (nnz <= 0) {
        const int g = (N + 1 + kWgThreads - 1) / kWgThreads;
        fill_kernel<<<g, kWgThreads, 0, stream>>>(t_row_ptr, N + 1, 0);
        return hipGetLastError();
    }
    const size_t buf = round16((size_t)nnz * 4);
    char* ws = static_cast<char*>(workspace);
    int* keys[2] = {reinterpret_cast<int*>(ws), reinterpret_cast<int*>(ws + buf)};
    int* vals_ws = reinterpret_cast<int*>(ws + 2 * buf);
    int* hist = reinterpret_cast<int*>(ws + 3 * buf);
    const int nblocks = sort_blocks(nnz);
    int bits = 1;
    while (bits < 31 && (N - 1) >> bits) ++bits; // columns are < N
    const int passes = (bits + kRadixBits - 1) / kRadixBits;
    // the values ping-pong between the workspace and perm so that the last pass writes perm
    const int* keys_in = col;
    const int* vals_in = nullptr;
    for (int p = 0; p < passes; ++p) {
        int* keys_out = keys[p & 1];
        int* vals_out = ((passes - 1 - p) & 1) ? vals_ws : perm;
        const int shift = p * kRadixBits;
        digit_count_kernel<<<nblocks, kWgThreads, 0, stream>>>(keys_in, nnz, shift, nblocks, hist);
        digit_scan_kernel<<<1, kScanThreads, 0, stream>>>(hist, kRadix * nblocks);
        digit_scatter_kernel<<<nblocks, kWgThreads, 0, stream>>>(keys_in, vals_in, nnz, shift, nblocks, hist, keys_out,
                                                                 vals_out);
        keys_in = keys_out;
        vals_in = vals_out;
    }
    const int g = (nnz + kWgThreads - 1) / kWgThreads;
    transposed_arrays_kernel<<<g, kWgThreads, 0, stream>>>(M, N, nnz, row_ptr, keys_in, perm, t_row_ptr, t_col);
    return hipGetLastError();
}

} // namespace rode
