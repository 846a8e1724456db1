// Row-decomposition preprocessing on the GPU: count -> scan -> compaction/fill.
//
// Output contract (bit-exact): the arrays the reference's sequential CPU routine
// produces, RoDe_SDDMM/main.cu:114-163 (same text in test.cu:73-116,
// rode_sddmm_cuda.cu:80-110, Preprocess_opt/_preprocess.cu:340-373), including
// the sentinel st_off[n_blk] = row_ptr[M] (main.cu:161-162).  The reference's
// own GPU pipeline (_preprocess.cu:244-339: RoDe_get_bn_rn -> 2x ExclusiveSum
// -> RoDe_fill_data) scatters into the arrays other workgroups are still
// reading and has one thread emit all segments of its row; here one kernel
// reads row_ptr once, scans across its workgroups through a small scratch
// array and writes the lists from the scanned offsets, a row with many
// segments by a whole wave.
#include "rode_device.hpp"
#include "rode_internal.hpp"

#include <mutex>

namespace rode {

namespace {

// Rows per tile (one workgroup), from the number of rows: few tiles keep the scan across
// tiles short (a round trip to memory per 512 tiles when all tiles run at once, and a
// ticket each), many threads keep the memory system busy.
struct TileShape {
    int threads, rows_per_thread;
    int rows() const { return threads * rows_per_thread; }
};
inline TileShape tile_shape_for(size_t rows)
{
    if (rows <= 128 * 1024) return {256, 1};
    if (rows <= 512 * 1024) return {256, 4};
    if (rows <= 1024 * 1024) return {1024, 4};
    return {1024, 8};
}
constexpr int kMinTileRows = 256;

// Scratch layout: [ticket counter, unused | one status word per tile].  (Sized for the
// smallest tile, whatever tile a call uses.)
constexpr size_t workspace_bytes_for(size_t rows)
{
    return (2 + (rows + kMinTileRows - 1) / kMinTileRows) * sizeof(unsigned long long);
}

// Scratch of the allocation-free entry point: one copy per GPU, held until the process
// ends (128 KB).  In host code this name is only a handle for hipGetSymbolAddress; the
// kernels receive the address that call returns.
constexpr size_t kStaticScratchBytes = (workspace_bytes_for(kPreprocessStaticMaxRows) + 255) / 256 * 256;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Decomposition parameters as the kernels use them: divisions by a power of two (every
// parameter set of the reference: 512 or 32, 32, 4) are shifts and masks.
struct Params {
    int seg, kblock, veclen;
    int seg_shift;   // log2(seg), or -1
    int kblock_mask; // kblock - 1 if a power of two, or -1
    int veclen_mask; // veclen - 1 if a power of two, or -1
};
inline Params make_params(int seg, int kblock, int veclen)
{
    auto pow2 = [](int v) { return v > 0 && (v & (v - 1)) == 0; };
    int shift = -1;
    if (pow2(seg))
        for (shift = 0; (1 << shift) < seg; ++shift) {}
    return Params{seg, kblock, veclen, shift, pow2(kblock) ? kblock - 1 : -1, pow2(veclen) ? veclen - 1 : -1};
}
__device__ __forceinline__ int pad_of(const Params& p, int s) { return p.veclen_mask >= 0 ? (s & p.veclen_mask) : s % p.veclen; }

// Per-row counts in closed form.  With p = s % vec_len and N = len + p the
// sequential routine peels t = (N-1)/seg whole segments until 1 <= N' <= seg is
// left, then emits one more segment iff N' >= k_block and one residue iff
// N' % k_block != 0.  (For seg % k_block == 0 this equals RoDe_get_bn_rn,
// _preprocess.cu:262-270; for other parameters it still follows the sequential
// text, which is the contract.)  Packed: segments << 32 | residue.
__device__ __forceinline__ unsigned long long row_counts(const Params& p, int s, int e)
{
    const int N = e - s + pad_of(p, s);
    if (N <= 0) return 0ull;
    const int t = p.seg_shift >= 0 ? (N - 1) >> p.seg_shift : (N - 1) / p.seg;
    const int rest = N - t * p.seg;
    const unsigned bn = (unsigned)t + (rest >= p.kblock ? 1u : 0u);
    const unsigned rn = (p.kblock_mask >= 0 ? (rest & p.kblock_mask) : rest % p.kblock) ? 1u : 0u;
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

// Exclusive scan over the THREADS threads of a workgroup; returns the exclusive
// prefix of `v` and the workgroup total.
template <int THREADS>
__device__ __forceinline__ unsigned long long wg_exclusive_scan(unsigned long long v, unsigned long long* total)
{
    constexpr int kWaves = THREADS / kWave;
    __shared__ unsigned long long wave_tot[kWaves];
    const int lane = threadIdx.x % kWave, w = threadIdx.x / kWave;
    const unsigned long long incl = wave_inclusive_scan(v, lane);
    if (lane == kWave - 1) wave_tot[w] = incl;
    __syncthreads();
    unsigned long long base = 0, tot = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) {
        if (i < w) base += wave_tot[i];
        tot += wave_tot[i];
    }
    *total = tot;
    return base + incl - v;
}

// Status word of a tile: bits 62-63 say what the rest is - 0 nothing yet, 1 the tile's own
// counts, 2 the counts of all tiles up to and including it, 3 a wait gave up somewhere before
// this tile - then 31 bits of segments and 31 bits of residues (both totals are below 2^31).
// One 64-bit word, so that a reader never sees half of an update.
constexpr unsigned long long kOwnSum = 1ull << 62, kPrefixSum = 2ull << 62, kGaveUp = 3ull << 62, kStateMask = 3ull << 62;
__device__ __forceinline__ unsigned long long pack_status(unsigned long long state, unsigned long long counts)
{
    return state | ((counts >> 32) << 31) | (counts & 0x7fffffffull);
}
__device__ __forceinline__ unsigned long long unpack_counts(unsigned long long status)
{
    return (((status >> 31) & 0x7fffffffull) << 32) | (status & 0x7fffffffull);
}

__global__ void __launch_bounds__(kWgThreads) clear_status_kernel(int words, unsigned long long* __restrict__ status)
{
    const int i = blockIdx.x * kWgThreads + threadIdx.x;
    if (i < words) status[i] = 0ull;
}

// A wait that cannot be met (it never happened in testing: a tile only waits for tiles that
// took their ticket before it and therefore run) ends after this many polls instead of
// holding the GPU; every later tile hears of it through the status words and the call reports
// n_blk = n_res = -1.
constexpr int kMaxPolls = 1 << 22;

// One pass over row_ptr: counts per row, a decoupled look-back scan across the tiles (a tile
// publishes its own counts, then adds up the published counts of the tiles before it until it
// meets one that already knows its prefix), and the compaction - residue rows and block
// segments are written straight from the scanned offsets, the segments one per thread and
// step (a binary search in the tile's own offsets finds the row), so that a row with
// thousands of segments costs what as many short rows would.  Tiles are numbered by a ticket
// in the order they start, so a tile only ever waits for tiles that are already running.
// THREADS per workgroup, RPT rows per thread; a thread's rows are consecutive.
template <int THREADS, int RPT>
__global__ void __launch_bounds__(THREADS)
decompose_kernel(Params p, int M, int ntiles, int capacity, const int* __restrict__ row_ptr,
                 unsigned long long* __restrict__ ws, int* __restrict__ block_r_ind, int* __restrict__ st_off,
                 int* __restrict__ residue_r_ind, int* __restrict__ n_blk, int* __restrict__ n_res)
{
    constexpr int kTile = THREADS * RPT;
    // (one unused word after every 32, so that threads reading rows RPT apart use different banks)
    constexpr auto at = [](int i) { return i + (i >> 5); };
    __shared__ int lds_rp[kTile + 1 + (kTile >> 5) + 1];
    __shared__ int lds_first[kTile + 1 + (kTile >> 5) + 1]; // first segment of every row, counted from the tile's first
    __shared__ unsigned long long lds_prefix;
    __shared__ int lds_tile;
    __shared__ bool lds_failed;
    unsigned long long* counter = ws;       // [0] tickets
    unsigned long long* status = ws + 2;    // one word per tile
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    if (tid == 0) lds_tile = (int)atomicAdd(counter, 1ull);
    __syncthreads();
    const int tile = lds_tile;
    const long long row0 = (long long)tile * kTile;
    for (int i = tid; i <= kTile; i += THREADS) lds_rp[at(i)] = row0 + i <= M ? row_ptr[row0 + i] : 0;
    __syncthreads();

    unsigned long long c[RPT], acc = 0;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int r = tid * RPT + i;
        c[i] = row0 + r < M ? row_counts(p, lds_rp[at(r)], lds_rp[at(r + 1)]) : 0ull;
        acc += c[i];
    }
    unsigned long long total;
    const unsigned long long within = wg_exclusive_scan<THREADS>(acc, &total);

    // look-back, by the first wave
    if (wave == 0) {
        if (lane == 0)
            __hip_atomic_store(status + tile, pack_status(tile == 0 ? kPrefixSum : kOwnSum, total), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        unsigned long long before = 0;
        bool gave_up = false, done = false;
        // kLookBack * 64 earlier tiles per step, all asked for at once: when every tile of a
        // matrix is running at the same time, prefixes spread no faster than one step of this
        // loop per round trip to memory
        constexpr int kLookBack = 8;
        for (int last = tile - 1; last >= 0 && !gave_up && !done; last -= kLookBack * kWave) {
            unsigned long long st[kLookBack];
#pragma unroll
            for (int w = 0; w < kLookBack; ++w) {
                const int t = last - w * kWave - lane;
                st[w] = t >= 0 ? __hip_atomic_load(status + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : kPrefixSum;
            }
#pragma unroll
            for (int w = 0; w < kLookBack; ++w) {
                if (done || gave_up) break; // (the same in all lanes)
                const int t = last - w * kWave - lane;
                int polls = 0;
                while (t >= 0 && (st[w] & kStateMask) == 0 && ++polls < kMaxPolls)
                    st[w] = __hip_atomic_load(status + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                gave_up = __any((st[w] & kStateMask) == 0 || (st[w] & kStateMask) == kGaveUp);
                // the nearest tile that knows its prefix ends the walk; the tiles after it add their own counts
                // (lanes before tile 0 say "prefix 0")
                const unsigned long long knows = __ballot((st[w] & kStateMask) == kPrefixSum);
                const int stop = knows ? __builtin_ctzll(knows) : kWave; // lanes 0 .. stop take part
                unsigned long long part = t >= 0 && lane <= stop ? unpack_counts(st[w]) : 0ull;
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1) part += __shfl_xor(part, d, kWave);
                before += part;
                done = knows != 0ull;
            }
        }
        if (lane == 0) {
            if (tile > 0 || gave_up)
                __hip_atomic_store(status + tile, gave_up ? kGaveUp : pack_status(kPrefixSum, before + total), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            lds_prefix = before;
            lds_failed = gave_up;
        }
    }
    __syncthreads();
    const int tile_first = (int)(lds_prefix >> 32); // the tile's first segment
    unsigned long long run = lds_prefix + within;

    // residue rows, and where every row's segments start
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int r = tid * RPT + i;
        lds_first[at(r)] = (int)(run >> 32) - tile_first;
        if (c[i] & 1ull) residue_r_ind[(int)(run & 0xffffffffull)] = (int)(row0 + r);
        run += c[i];
    }
    __syncthreads();
    // block segments: segment j of the tile belongs to the last row that starts at or before it
    const int segments = (int)(total >> 32);
    for (int j = tid; j < segments; j += THREADS) {
        int lo = 0, hi = kTile; // invariant: first[lo] <= j, and first[hi] > j or hi == kTile
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (lds_first[at(mid)] <= j) lo = mid; else hi = mid;
        }
        const int s = lds_rp[at(lo)], jj = j - lds_first[at(lo)];
        if (tile_first + j < capacity) {
            block_r_ind[tile_first + j] = (int)(row0 + lo);
            st_off[tile_first + j] = jj == 0 ? s : (s - pad_of(p, s)) + jj * p.seg;
        }
    }
    // the last tile knows the totals: counts and the sentinel
    if (tile == ntiles - 1 && tid == 0) {
        const unsigned long long all = lds_prefix + total;
        const int nb = (int)(all >> 32);
        *n_blk = lds_failed ? -1 : nb;
        *n_res = lds_failed ? -1 : (int)(all & 0xffffffffull);
        // a caller whose arrays are too small still gets the true counts, and nothing is
        // written past `capacity` segments (st_off holds capacity + 1 entries)
        if (nb <= capacity) st_off[nb] = row_ptr[M];
    }
}

// M == 0: no tile runs; counts and sentinel all the same.
__global__ void empty_matrix_kernel(const int* __restrict__ row_ptr, int* __restrict__ st_off, int* __restrict__ n_blk,
                                    int* __restrict__ n_res)
{
    *n_blk = 0;
    *n_res = 0;
    st_off[0] = row_ptr[0];
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
    const TileShape shape = tile_shape_for((size_t)(M > 0 ? M : 0));
    const int ntiles = (int)(((size_t)M + shape.rows() - 1) / shape.rows());
    if (ntiles == 0) {
        empty_matrix_kernel<<<1, 1, 0, stream>>>(row_ptr, st_off, n_blk, n_res);
        return hipGetLastError();
    }
    unsigned long long* ws = static_cast<unsigned long long*>(workspace);
    // (a fill kernel, not a memset: the call may be recorded into a HIP graph)
    clear_status_kernel<<<(ntiles + 2 + kWgThreads - 1) / kWgThreads, kWgThreads, 0, stream>>>(ntiles + 2, ws);
#define RODE_DECOMPOSE(THREADS, RPT)                                                                                      \
    decompose_kernel<THREADS, RPT><<<ntiles, THREADS, 0, stream>>>(make_params(seg, kblock, veclen), M, ntiles, capacity_blocks, row_ptr, \
                                                                   ws, block_r_ind, st_off, residue_r_ind, n_blk, n_res)
    if (shape.threads == 256 && shape.rows_per_thread == 1) RODE_DECOMPOSE(256, 1);
    else if (shape.threads == 256) RODE_DECOMPOSE(256, 4);
    else if (shape.rows_per_thread == 4) RODE_DECOMPOSE(1024, 4);
    else RODE_DECOMPOSE(1024, 8);
#undef RODE_DECOMPOSE
    return hipGetLastError();
}

} // namespace rode
