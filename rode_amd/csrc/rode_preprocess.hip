// Row-decomposition preprocessing on the GPU: count -> scan -> compaction/fill.
//
// Output contract (bit-exact): the arrays the reference's sequential CPU routine
// produces, RoDe_SDDMM/main.cu:114-163 (same text in test.cu:73-116,
// rode_sddmm_cuda.cu:80-110, Preprocess_opt/_preprocess.cu:340-373), including
// the sentinel st_off[n_blk] = row_ptr[M] (main.cu:161-162).  The reference's
// own GPU pipeline (_preprocess.cu:244-339: RoDe_get_bn_rn -> 2x ExclusiveSum
// -> RoDe_fill_data) scatters into the arrays other workgroups are still
// reading and has one thread emit all segments of its row; here the scan
// results live in caller-provided scratch and the fill runs one thread per
// *segment*, so a 200 K-nonzero row costs the same as 400 short ones.
#include "rode_device.hpp"
#include "rode_internal.hpp"

#include <mutex>

namespace rode {

namespace {

constexpr int kRowsPerThread = 4;
constexpr int kTileRows = kWgThreads * kRowsPerThread; // rows scanned by one workgroup

// Scratch layout: [tile_sum | tile_prefix | row_blk_prefix], the 8-byte arrays first.
constexpr size_t workspace_bytes_for(size_t rows)
{
    return (2 * ((rows + kTileRows - 1) / kTileRows) + 2) * sizeof(unsigned long long) + (rows + 2) * sizeof(int);
}

// Scratch of the allocation-free entry point: one copy per GPU, held until the process
// ends (16.1 MiB).  In host code this name is only a handle for hipGetSymbolAddress; the
// kernels receive the address that call returns.
constexpr size_t kStaticScratchBytes = (workspace_bytes_for(kPreprocessStaticMaxRows) + 255) / 256 * 256;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Per-row counts in closed form.  With p = s % vec_len and N = len + p the
// sequential routine peels t = (N-1)/seg whole segments until 1 <= N' <= seg is
// left, then emits one more segment iff N' >= k_block and one residue iff
// N' % k_block != 0.  (For seg % k_block == 0 this equals RoDe_get_bn_rn,
// _preprocess.cu:262-270; for other parameters it still follows the sequential
// text, which is the contract.)
__device__ __forceinline__ unsigned long long row_counts(int seg, int kblock, int veclen, int s, int e)
{
    const int N = e - s + s % veclen;
    if (N <= 0) return 0ull;
    const int t = (N - 1) / seg;
    const int rest = N - t * seg;
    const unsigned bn = (unsigned)t + (rest >= kblock ? 1u : 0u);
    const unsigned rn = (rest % kblock) ? 1u : 0u;
    return ((unsigned long long)bn << 32) | rn; // both sums stay below 2^31, no carry between halves
}

__device__ __forceinline__ unsigned long long wave_inclusive_scan(unsigned long long v, int lane)
{
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const unsigned long long up = __shfl_up(v, d, kWave);
        if (lane >= d) v += up;
    }
    return v;
}

// Exclusive scan over the 256 threads of a workgroup; returns the exclusive
// prefix of `v` and the workgroup total.
__device__ __forceinline__ unsigned long long wg_exclusive_scan(unsigned long long v, unsigned long long* total)
{
    __shared__ unsigned long long wave_tot[kWavesPerWg];
    const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
    const unsigned long long incl = wave_inclusive_scan(v, lane);
    __syncthreads(); // wave_tot may still be read from a previous call
    if (lane == kWave - 1) wave_tot[w] = incl;
    __syncthreads();
    unsigned long long base = 0, tot = 0;
#pragma unroll
    for (int i = 0; i < kWavesPerWg; ++i) {
        if (i < w) base += wave_tot[i];
        tot += wave_tot[i];
    }
    *total = tot;
    return base + incl - v;
}

__global__ void __launch_bounds__(kWgThreads)
tile_reduce_kernel(int seg, int kblock, int veclen, int M, const int* __restrict__ row_ptr,
                   unsigned long long* __restrict__ tile_sum)
{
    const int r0 = blockIdx.x * kTileRows + threadIdx.x * kRowsPerThread;
    unsigned long long acc = 0;
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int r = r0 + i;
        if (r < M) acc += row_counts(seg, kblock, veclen, row_ptr[r], row_ptr[r + 1]);
    }
    unsigned long long total;
    wg_exclusive_scan(acc, &total);
    if (threadIdx.x == 0) tile_sum[blockIdx.x] = total;
}

// One workgroup: exclusive scan of the tile sums, totals, sentinel.
__global__ void __launch_bounds__(kWgThreads)
tile_scan_kernel(int M, int ntiles, int capacity, const int* __restrict__ row_ptr,
                 const unsigned long long* __restrict__ tile_sum, unsigned long long* __restrict__ tile_prefix,
                 int* __restrict__ row_blk_prefix, int* __restrict__ st_off, int* __restrict__ n_blk,
                 int* __restrict__ n_res)
{
    unsigned long long carry = 0;
    for (int base = 0; base < ntiles; base += kWgThreads) {
        const int i = base + threadIdx.x;
        const unsigned long long v = i < ntiles ? tile_sum[i] : 0ull;
        unsigned long long total;
        const unsigned long long excl = wg_exclusive_scan(v, &total);
        if (i < ntiles) tile_prefix[i] = carry + excl;
        carry += total;
    }
    if (threadIdx.x == 0) {
        const int nb = (int)(carry >> 32);
        *n_blk = nb;
        *n_res = (int)(carry & 0xffffffffull);
        row_blk_prefix[M] = nb;
        // a caller whose arrays are too small still gets the true counts, and nothing is
        // written past `capacity` segments (st_off holds capacity + 1 entries)
        if (nb <= capacity) st_off[nb] = row_ptr[M];
    }
}

// Per-row exclusive prefixes; residue rows are compacted right here.
__global__ void __launch_bounds__(kWgThreads)
row_scan_kernel(int seg, int kblock, int veclen, int M, const int* __restrict__ row_ptr,
                const unsigned long long* __restrict__ tile_prefix, int* __restrict__ row_blk_prefix,
                int* __restrict__ residue_r_ind)
{
    const int r0 = blockIdx.x * kTileRows + threadIdx.x * kRowsPerThread;
    unsigned long long c[kRowsPerThread];
    unsigned long long acc = 0;
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int r = r0 + i;
        c[i] = r < M ? row_counts(seg, kblock, veclen, row_ptr[r], row_ptr[r + 1]) : 0ull;
        acc += c[i];
    }
    unsigned long long total;
    unsigned long long run = tile_prefix[blockIdx.x] + wg_exclusive_scan(acc, &total);
#pragma unroll
    for (int i = 0; i < kRowsPerThread; ++i) {
        const int r = r0 + i;
        if (r < M) {
            row_blk_prefix[r] = (int)(run >> 32);
            if (c[i] & 1ull) residue_r_ind[(int)(run & 0xffffffffull)] = r;
        }
        run += c[i];
    }
}

// One thread per block segment j: its row is the last r with prefix[r] <= j.
__global__ void __launch_bounds__(kWgThreads)
fill_segments_kernel(int seg, int veclen, int M, int capacity, const int* __restrict__ row_ptr,
                     const int* __restrict__ row_blk_prefix, int* __restrict__ block_r_ind,
                     int* __restrict__ st_off)
{
    const int n_blk = min(row_blk_prefix[M], capacity);
    for (int j = blockIdx.x * kWgThreads + threadIdx.x; j < n_blk; j += gridDim.x * kWgThreads) {
        int lo = 0, hi = M; // invariant: prefix[lo] <= j < prefix[hi]
        while (hi - lo > 1) {
            const int mid = lo + (hi - lo) / 2;
            if (row_blk_prefix[mid] <= j) lo = mid; else hi = mid;
        }
        const int s = row_ptr[lo];
        const int jj = j - row_blk_prefix[lo];
        block_r_ind[j] = lo;
        st_off[j] = jj == 0 ? s : (s - s % veclen) + jj * seg;
    }
}

} // namespace

size_t preprocess_workspace_bytes(int M) { return workspace_bytes_for((size_t)(M > 0 ? M : 0)); }

// Device address of this GPU's copy of `scratch`, looked up once per device.
hipError_t preprocess_static_workspace(void** ptr)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* per_device[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mu);
    if (!per_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        per_device[dev] = p;
    }
    *ptr = per_device[dev];
    return hipSuccess;
}

hipError_t preprocess_launch(int seg, int kblock, int veclen, int M, const int* row_ptr, int* block_r_ind,
                             int* st_off, int* residue_r_ind, int* n_blk, int* n_res, void* workspace,
                             int capacity_blocks, hipStream_t stream)
{
    const int ntiles = (int)(((size_t)M + kTileRows - 1) / kTileRows);
    unsigned long long* tile_sum = static_cast<unsigned long long*>(workspace);
    unsigned long long* tile_prefix = tile_sum + ntiles + 1;
    int* row_blk_prefix = reinterpret_cast<int*>(tile_prefix + ntiles + 1);

    if (ntiles > 0)
        tile_reduce_kernel<<<ntiles, kWgThreads, 0, stream>>>(seg, kblock, veclen, M, row_ptr, tile_sum);
    tile_scan_kernel<<<1, kWgThreads, 0, stream>>>(M, ntiles, capacity_blocks, row_ptr, tile_sum, tile_prefix,
                                                    row_blk_prefix, st_off, n_blk, n_res);
    if (ntiles > 0) {
        row_scan_kernel<<<ntiles, kWgThreads, 0, stream>>>(seg, kblock, veclen, M, row_ptr, tile_prefix,
                                                            row_blk_prefix, residue_r_ind);
        // n_blk is only known on the device: size the grid from the caller's
        // capacity bound and let the kernel stride.
        long long want = ((long long)capacity_blocks + kWgThreads - 1) / kWgThreads;
        const int grid = (int)(want < 1 ? 1 : (want > 4096 ? 4096 : want));
        fill_segments_kernel<<<grid, kWgThreads, 0, stream>>>(seg, veclen, M, capacity_blocks, row_ptr,
                                                               row_blk_prefix, block_r_ind, st_off);
    }
    return hipGetLastError();
}

} // namespace rode
