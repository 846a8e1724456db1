// Locality plan: for every chunk of 128 consecutive residue-list entries, decide whether
// the dense rows its nonzeros reference cluster in a window of consecutive rows small
// enough to be staged in LDS (banded matrices), and which window.
//
// No counterpart in the reference: its kernels gather every dense row from memory
// (RoDe_SpMM/RoDeSpmm.cu:140-160, RoDe_SDDMM/RoDeSddmm.cu:96-140).  The plan changes no
// result; it only tells the window kernels where most of a chunk's dense rows are.
//
// One workgroup per chunk:
//   1. slot range of every entry (the ranges of RoDeSpmm.cu:71-82);
//   2. 256 column samples spread evenly over the chunk's slots; their quartiles q25 and
//      q75 place the window: if they are further apart than the window is long, the chunk
//      has no window; otherwise the window is centred on their midpoint;
//   3. every slot is tested against that window: hit count and the extent of the hits
//      (the window shrinks to [smallest hit, largest hit]);
//   4. the chunk gets its window if the hits are at least half of its slots and at least
//      twice the window's rows (staging a row has to be repaid by about two reads).
#include "rode_items.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

__global__ void plan_header_kernel(int m2, int* __restrict__ plan)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        plan[0] = plan_residue_chunks(m2);
        plan[1] = 0;
        plan[2] = 0;
        plan[3] = 0;
    }
}

__device__ __forceinline__ int wave_reduce_add(int v)
{
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}
__device__ __forceinline__ int wave_reduce_min(int v)
{
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v = min(v, __shfl_xor(v, d, kWave));
    return v;
}
__device__ __forceinline__ int wave_reduce_max(int v)
{
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v = max(v, __shfl_xor(v, d, kWave));
    return v;
}

__global__ void __launch_bounds__(kWgThreads)
plan_chunks_kernel(int m2, int dense_rows, const int* __restrict__ residue_rows, const int* __restrict__ row_ptr,
                   const int* __restrict__ col, int* __restrict__ plan)
{
    constexpr int CH = kPlanResidueChunk;
    constexpr int ROWS_MAX = kResidueWindowRowsMax;
    static_assert(CH <= kWgThreads, "one thread per entry");
    __shared__ int first[CH];
    __shared__ int prefix[CH + 1];
    __shared__ int samples[kWgThreads];
    __shared__ int quart[2];
    __shared__ int red[3][kWavesPerWg];

    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const int chunk = blockIdx.x;
    const int e0 = chunk * CH;
    const int ne = min(CH, m2 - e0);
    int* desc = plan + kPlanHeaderInts + kPlanDescInts * chunk;

    // 1. slot range of every entry
    int my_len = 0;
    if (tid < ne) {
        const ResidueItem it = residue_item(residue_rows[e0 + tid], row_ptr);
        first[tid] = it.first;
        my_len = it.cnt;
    }
    if (tid < CH) prefix[tid + 1] = my_len; // lengths for now
    if (tid == 0) prefix[0] = 0;
    __syncthreads();
    if (tid == 0) {
        int run = 0;
        for (int i = 1; i <= CH; ++i) {
            run += prefix[i];
            prefix[i] = run;
        }
    }
    __syncthreads();
    const int total = prefix[CH];
    if (total <= 0) {
        if (tid == 0) *reinterpret_cast<int4*>(desc) = make_int4(0, 0, 0, 0);
        return;
    }
    // entry that holds slot p of the chunk: the last e with prefix[e] <= p
    auto entry_of = [&](int p) {
        int lo = 0, hi = CH; // prefix[lo] <= p < prefix[hi]
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (prefix[mid] <= p) lo = mid; else hi = mid;
        }
        return lo;
    };

    // 2. samples and their quartiles
    {
        const int p = (int)(((long long)tid * total + total / 2) / kWgThreads);
        const int e = entry_of(p);
        samples[tid] = col[first[e] + (p - prefix[e])];
    }
    __syncthreads();
    {
        const int mine = samples[tid];
        int rank = 0;
        for (int j = 0; j < kWgThreads; ++j) {
            const int other = samples[j];
            rank += (other < mine || (other == mine && j < tid)) ? 1 : 0;
        }
        if (rank == kWgThreads / 4) quart[0] = mine;
        if (rank == kWgThreads * 3 / 4 - 1) quart[1] = mine;
    }
    __syncthreads();
    const int q25 = quart[0], q75 = quart[1];
    if ((long long)q75 - q25 + 1 > ROWS_MAX || dense_rows <= 0) {
        if (tid == 0) *reinterpret_cast<int4*>(desc) = make_int4(0, 0, total, total);
        return;
    }
    int w0 = q25 + (q75 - q25) / 2 - ROWS_MAX / 2;
    w0 = max(0, min(w0, dense_rows - ROWS_MAX));
    const int wend = min(dense_rows, w0 + ROWS_MAX);

    // 3. hits and their extent
    int hits = 0, lo_hit = 0x7fffffff, hi_hit = -1;
    for (int p = tid; p < total; p += kWgThreads) {
        const int e = entry_of(p);
        const int c = col[first[e] + (p - prefix[e])];
        if (c >= w0 && c < wend) {
            ++hits;
            lo_hit = min(lo_hit, c);
            hi_hit = max(hi_hit, c);
        }
    }
    hits = wave_reduce_add(hits);
    lo_hit = wave_reduce_min(lo_hit);
    hi_hit = wave_reduce_max(hi_hit);
    if (lane == 0) {
        red[0][wave] = hits;
        red[1][wave] = lo_hit;
        red[2][wave] = hi_hit;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kWavesPerWg; ++w) {
            hits += red[0][w];
            lo_hit = min(lo_hit, red[1][w]);
            hi_hit = max(hi_hit, red[2][w]);
        }
        // 4. decision
        const int wn = hi_hit - lo_hit + 1;
        const bool take = hits > 0 && 2ll * hits >= total && hits >= 2ll * wn;
        *reinterpret_cast<int4*>(desc) = take ? make_int4(lo_hit, wn, total, total - hits) : make_int4(0, 0, total, total - hits);
        if (take) atomicAdd(plan + 1, 1);
    }
}

// Fills the PlannedChunk of every chunk that has a window: 8 threads per residue row.
__global__ void __launch_bounds__(kPlanResidueChunk * 8)
plan_rows_kernel(int m2, const int* __restrict__ residue_rows, const int* __restrict__ row_ptr,
                 const int* __restrict__ col, const int* __restrict__ plan, PlannedChunk* __restrict__ rows)
{
    constexpr int L = 8, OWN = kBlockItems / L;
    __shared__ unsigned char keys[kPlanResidueChunk][kBlockItems];
    const int chunk = blockIdx.x;
    const WindowDesc d = plan_residue_desc(plan, chunk);
    PlannedChunk& out = rows[chunk];
    if (threadIdx.x == 0) {
        out.w0 = d.w0;
        out.wn = d.wn;
        out.reserved[0] = out.reserved[1] = 0;
    }
    if (d.wn <= 0) return;
    const int local = threadIdx.x / L, ls = threadIdx.x % L;
    const int entry = chunk * kPlanResidueChunk + local;
    int row = -1, first = 0, cnt = 0, aligned = 0;
    bool accumulate = false;
    if (entry < m2) {
        row = residue_rows[entry];
        const ResidueItem it = residue_item(row, row_ptr);
        first = it.first;
        cnt = it.cnt;
        aligned = it.aligned;
        accumulate = it.accumulate;
    }
    // which lane group of the window kernels takes this row: groups 2, 3, 6, 7 list odd window rows first
    const int odd_first = (local >> 1) & 1;
    unsigned u[OWN];
    unsigned best = 0xffffu;
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        const int s = ls + i * L;
        u[i] = 0xffffu;
        unsigned char key = 3; // not a slot of the row
        if (s < cnt) {
            const unsigned dw = (unsigned)(col[first + s] - d.w0);
            if (dw < (unsigned)d.wn) {
                u[i] = dw;
                key = ((dw & 1u) != (unsigned)odd_first) ? 1 : 0;
            } else {
                key = 2; // outside the window: after the ones inside
            }
        }
        keys[local][s] = key;
        best = min(best, u[i]);
    }
#pragma unroll
    for (int m = 1; m < L; m <<= 1) best = min(best, (unsigned)__shfl_xor((int)best, m, kWave));
    if (best == 0xffffu) best = 0; // no slot inside the window: every read is replaced anyway
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); // the 8 threads of a row are lanes of one wave
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    unsigned missbits = 0;
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        const int s = ls + i * L;
        const int key = keys[local][s];
        int rank = 0; // position: slots with a smaller key, or the same key and a smaller index, come first
        for (int o = 0; o < kBlockItems; ++o) {
            const int other = keys[local][o];
            rank += (other < key || (other == key && o < s)) ? 1 : 0;
        }
        const unsigned where = key == 0 || key == 1 ? u[i] : best;
        out.entry[local][rank] = (unsigned short)(where | (key <= 2 ? (unsigned)s << 9 : 0u));
        if (key == 2) missbits |= 1u << rank;
    }
#pragma unroll
    for (int m = 1; m < L; m <<= 1) missbits |= (unsigned)__shfl_xor((int)missbits, m, kWave);
    if (ls == 0) {
        PlannedRowMeta meta;
        meta.row = row;
        meta.first = first;
        meta.packed = cnt | (accumulate ? 1 << 8 : 0) | (min(aligned, 0xffff) << 16);
        meta.missmask = missbits;
        out.meta[local] = meta;
    }
}

} // namespace

size_t window_plan_ints(int m2) { return plan_ints(m2); }
size_t window_plan_rows_bytes(int m2) { return (size_t)plan_residue_chunks(m2) * sizeof(PlannedChunk); }

hipError_t window_plan_launch(int m2, int dense_rows, const int* residue_rows, const int* row_ptr, const int* col,
                              int* plan, hipStream_t stream)
{
    plan_header_kernel<<<1, kWave, 0, stream>>>(m2, plan);
    const int chunks = plan_residue_chunks(m2);
    if (chunks > 0) {
        plan_chunks_kernel<<<chunks, kWgThreads, 0, stream>>>(m2, dense_rows, residue_rows, row_ptr, col, plan);
    }
    return hipGetLastError();
}

hipError_t window_plan_rows_launch(int m2, const int* residue_rows, const int* row_ptr, const int* col, const int* plan,
                                   void* rows, hipStream_t stream)
{
    const int chunks = plan_residue_chunks(m2);
    if (chunks > 0)
        plan_rows_kernel<<<chunks, kPlanResidueChunk * 8, 0, stream>>>(m2, residue_rows, row_ptr, col, plan,
                                                                       static_cast<PlannedChunk*>(rows));
    return hipGetLastError();
}

} // namespace rode
