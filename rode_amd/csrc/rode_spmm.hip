// SpMM over a row-decomposed CSR matrix:  C[row, :] += sum_idx values[idx] * B[col(idx), :]
// Same work split, index arithmetic and store/accumulate rules as the
// reference's SparseKernel::Kernel4Block (RoDe_SpMM/RoDeSpmm.cu:197-476) and
// Kernel4Residue (:41-195); the execution shape is written for 64-lane
// wavefronts:
//
//   * the dense tile is TN columns wide; LPR = TN / (elements per 128-bit load)
//     lanes cover one B row, so one load instruction of a wave gathers 64 / LPR
//     different B rows, each as full 128-bit coalesced reads;
//   * (col, value) pairs of up to 64 nonzero slots are staged in LDS with one
//     coalesced load per lane and read back four at a time as broadcasts;
//   * block kernel: one wave per block segment; its lane groups take
//     interleaved slot quads, the partial rows are combined with a butterfly
//     over the groups and added to C with hardware fp32 atomics (always, as in
//     RoDeSpmm.cu:464-474: a long row has several segments and usually a residue).
//     Rows of 32..1024 slots are an exception in the execution, not in the result:
//     the wave of the row's first segment sums the whole row, tail included, and
//     adds it to C once; the row's other work items return at once;
//   * residue kernel: one group of LPR lanes per residue row, 64 / LPR rows per
//     wave (short rows are latency-bound and need many rows in flight); rows
//     shorter than 32 slots are stored with plain 128-bit stores, tails of
//     longer rows are added atomically (RoDeSpmm.cu:76-82, 173-194).
//
// Slots that belong to the previous row (the `start & 3` head of an unaligned
// segment) are neutralised with value 0 *and* the column of the first real slot,
// so a non-finite B row can never leak into a row that does not reference it
// (the reference multiplies B[0, :] by zero there, RoDeSpmm.cu:271-274).
#include "rode_items.hpp"
#include "rode_units.hpp"
#include "rode_internal.hpp"

#include <type_traits>

namespace rode {

namespace {

// Rows of at most `owned_slots` aligned slots (and at least 32, i.e. rows that have block
// segments) are summed by a single wave of the block kernel (spmm_block_item).  The
// launcher passes kOwnedRowSlots when the caller promises that the two lists are the
// complete decomposition of the matrix (a row's first segment and its residue entry are
// then both in this call) and there are enough block segments to keep every CU busy
// anyway; else 0 (every work item on its own wave: small matrices need the parallelism
// more than they mind the extra atomics).  Measured on both sides: with 3936 segments
// (168 K nonzeros, width 128) the step takes 0.025 ms with whole rows and 0.030 ms without,
// with 9152 segments (1 M nonzeros, fp16 rows of 128) 0.104 against 0.120 ms; from 200 K
// segments on the difference is below 1 %.
constexpr int kOwnedRowSlots = 1024;
constexpr int kOwnedMinSegments = 1024;
// Without the promise the block kernel may still merge the short segments of a row that
// the list it was given holds, when there are this many of them.
constexpr int kMergeMinSegments = 16384;

// Up to this many workgroups, and when both kernels go to the same stream, the two lists
// are processed by one launch (spmm_pair_kernel).  Above it the residue kernel runs on its
// own: it needs a quarter of the block kernel's registers and keeps twice the waves per CU.
constexpr int kPairMaxWorkgroups = 16384;

// A row of C that is written once and not read again by the kernel that writes it: stored
// with the non-temporal hint, so that it does not push the gathered rows of B out of the
// caches on its way (config 4, K=128: residue kernel 1.19 -> 1.09 ms; the same hint on the
// loads of B, on SDDMM's loads of rhs or on its stores of `out` made those kernels slower).
template <int VEC>
__device__ __forceinline__ void store_row(float* dst, const float (&acc)[VEC])
{
    typedef float Quad __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int x = 0; x < VEC; x += 4) {
        const Quad v = {acc[x], acc[x + 1], acc[x + 2], acc[x + 3]};
        __builtin_nontemporal_store(v, reinterpret_cast<Quad*>(dst + x));
    }
}

template <int VEC>
__device__ __forceinline__ void store_row(double* dst, const double (&acc)[VEC])
{
    typedef double Pair __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int x = 0; x < VEC; x += 2) {
        const Pair v = {acc[x], acc[x + 1]};
        __builtin_nontemporal_store(v, reinterpret_cast<Pair*>(dst + x));
    }
}

// Sum over the aligned slots [base, base + cnt) of values * B rows, for this lane's columns
// of the tile; the first `mask` slots (the previous row's) and the slots past cnt in the
// last quad are neutralised.  Every lane of the wave returns the wave's total.
// (split, jump: the slots are [base, base + split) followed by [base + split + jump, ...):
// a row with a hole that somebody else works on; split >= cnt for one plain range.)
template <typename T, int TN>
__device__ __forceinline__ void spmm_sum_slots(int base, int mask, int cnt, int split, int jump, int lane, int* my_c,
                                               typename DenseVec<T>::Acc* my_v, const T* b_lane, int n,
                                               const int* __restrict__ col,
                                               const typename DenseVec<T>::Acc* __restrict__ val,
                                               typename DenseVec<T>::Acc (&total)[SpmmShape<T, TN>::kVec])
{
    using S = SpmmShape<T, TN>;
    using A = typename S::Acc;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    const int group = lane / LPR;
    A acc[VEC];
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = A(0);

    for (int off = 0; off < cnt; off += kWave) {
        const int slot = off + lane;
        const int live = min(cnt - off, kWave); // 64, or less on the last step
        int c = 0;
        A v = A(0);
        if (lane < ((live + 3) & ~3)) {
            // slots of the previous row (head) and slots past the end (last quad) are
            // neutralised: value 0, column of a real slot
            const bool head = slot < mask, past = slot >= cnt;
            const int at = head ? mask : (past ? cnt - 1 : slot);
            const int idx = base + at + (at >= split ? jump : 0);
            c = col[idx];
            v = (head || past) ? A(0) : val[idx];
        }
        my_c[lane] = c;
        my_v[lane] = v;
        wave_lds_sync();
        if (live == kWave)
            spmm_gather<T, TN, 16 / G, true>(b_lane, (size_t)n, acc, my_c, my_v, group, G, 16);
        else
            spmm_gather<T, TN, 16 / G, false>(b_lane, (size_t)n, acc, my_c, my_v, group, G, (live + 3) / 4);
        wave_lds_sync();
    }
#pragma unroll
    for (int x = 0; x < VEC; ++x) total[x] = butterfly_sum<LPR, kWave>(acc[x]);
}

// One wave per block segment (see sddmm_block_kernel for the slot arithmetic,
// identical at RoDeSpmm.cu:210-234).
// (bid of nblocks: the workgroup's position in the part of the grid that works on block segments)
// WALK: 0 one wave per segment only, 1 chunks only (chunk_hint > 1), 2 either, found out here.
// (Kernels of their own, so that the code of one way does not cost the other registers.)
// STORE: a row's only work item stores its sum instead of adding it (owners.overwrite; a
// kernel of its own as well: as a run-time branch it slowed the fp16 kernel of width 128
// that never takes it from 0.97 to 1.13 ms on the power-law benchmark).
template <typename T, int TN, bool EDGE, int WALK, bool STORE>
__device__ __forceinline__ void
spmm_block_body(int bid, int nblocks, int m1, int n, int owned_slots, int chunk_hint, RowOwners owners,
                const int* __restrict__ block_rows,
                const int* __restrict__ st_off, const int* __restrict__ row_ptr, const int* __restrict__ col,
                const typename DenseVec<T>::Acc* __restrict__ val, const T* __restrict__ B,
                typename DenseVec<T>::Acc* __restrict__ C)
{
    using S = SpmmShape<T, TN>;
    using A = typename S::Acc;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) A lds_v[kWavesPerWg * kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    // Lists with short segments (and enough of them that merging is on): a wave walks a chunk
    // of consecutive segments from leader to leader, adds up what it finds for one row and
    // updates that row of C once (the sums of the items, not one long sum: same rounding as
    // the combine of neighbouring waves below).
    int chunk = 1;
    if constexpr (WALK == 1) chunk = chunk_hint;
    if constexpr (WALK == 2)
        chunk = block_chunk_for_grid(owned_slots != 0 && m1 >= kWalkMinSegments ? block_chunk(m1, block_rows, st_off) : 1, m1,
                                     nblocks);
    if (WALK != 0 && chunk > 1) {
        const long long first = chunk_first_segment(bid, wave, m1, chunk);
        if (first < 0) return;
        const int last = (int)min(first + chunk, (long long)m1);
        const int ls = lane % LPR, group = lane / LPR;
        const int tile = blockIdx.y * TN;
        const bool col_ok = !EDGE || tile + ls * VEC < n;
        const T* b_lane = B + tile + (col_ok ? ls * VEC : 0);
        constexpr int EPG = VEC / G > 0 ? VEC / G : 1; // elements each lane group adds to C
        A row_total[VEC];
        int pending = -1;           // the row that row_total belongs to
        bool pending_whole = false; // ... is that row's one work item
        auto flush = [&]() {
            A* c_lane = C + (size_t)pending * n + tile + ls * VEC;
            if (STORE && pending_whole) { // (the same in every lane)
#pragma unroll
                for (int x = 0; x < VEC; ++x)
                    if (group == x / EPG && col_ok) c_lane[x] = row_total[x];
                return;
            }
#pragma unroll
            for (int x = 0; x < VEC; ++x)
                if (group == x / EPG && col_ok) atomicAdd(c_lane + x, row_total[x]);
        };
        for (int from = (int)first; from < last; from += kScanSegments) {
            const ChunkScan scan = scan_chunk(kSpmmMergeSlots, from, m1, owned_slots, owners, lane, block_rows, st_off, row_ptr);
            const int count = min(last - from, kScanSegments);
            for (unsigned long long todo = scan.items & ((1ull << count) - 1ull); todo; todo &= todo - 1ull) {
                const BlockItem it = chunk_item(scan, __builtin_ctzll(todo));
                A total[VEC];
                spmm_sum_slots<T, TN>(it.base, it.mask, it.cnt, it.cnt, 0, lane, lds_c + wave * kWave, lds_v + wave * kWave,
                                      b_lane, n, col, val, total);
                if (it.row != pending) {
                    if (pending >= 0) flush();
                    pending = it.row;
                    pending_whole = it.whole;
#pragma unroll
                    for (int x = 0; x < VEC; ++x) row_total[x] = total[x];
                } else {
#pragma unroll
                    for (int x = 0; x < VEC; ++x) row_total[x] += total[x];
                }
            }
        }
        if (pending >= 0) flush();
        return;
    }
    const int seg0 = xcd_logical_block(bid, nblocks) * kWavesPerWg;
    const int seg = seg0 + wave;
    BlockItem it{-1, 0, 0, 0};
    const bool active = seg < m1 && spmm_block_item(seg, m1, owned_slots, owners, lane, block_rows, st_off, row_ptr, it);
    // A wave without a work item leaves at once (with the reference's 32-slot segments that
    // is most waves); the barrier below then counts only the waves that are still running
    // (S_BARRIER waits on the surviving waves of a workgroup).
    if (!active) return;
    // Do two work items of this workgroup add to the same row (neighbouring segments of a
    // long row that are not merged into one leader)?  Every wave finds the same answer.  If
    // so, the waves add their sums up in LDS and the row of C gets one update per run of
    // such work items instead of one each.
    int item_row[kWavesPerWg]; // the row of each wave's work item, -1: that wave has none (and has left)
    bool shared_row = false;
#pragma unroll
    for (int i = 0; i < kWavesPerWg; ++i) {
        item_row[i] = spmm_block_leader_row(seg0 + i, m1, owned_slots, owners, block_rows, st_off, row_ptr);
        if (i > 0) shared_row = shared_row || (item_row[i] >= 0 && item_row[i] == item_row[i - 1]);
    }
    const int row = it.row, mask = it.mask, base = it.base, cnt = it.cnt;

    const int ls = lane % LPR, group = lane / LPR;
    const int tile = blockIdx.y * TN;
    // EDGE: n is not a multiple of TN; lanes past the last column re-read the tile's
    // first columns (a valid address) and never write
    const bool col_ok = !EDGE || tile + ls * VEC < n;
    const T* b_lane = B + tile + (col_ok ? ls * VEC : 0);
    int* my_c = lds_c + wave * kWave;
    A* my_v = lds_v + wave * kWave;

    // combine the lane groups, then spread the atomics over them
    constexpr int EPG = VEC / G > 0 ? VEC / G : 1; // elements each group adds
    A total[VEC];
    spmm_sum_slots<T, TN>(base, mask, cnt, cnt, 0, lane, my_c, my_v, b_lane, n, col, val, total);
    if (shared_row) {
        __shared__ __attribute__((aligned(16))) A wg_sum[kWavesPerWg][TN];
        if (group == 0) {
#pragma unroll
            for (int x = 0; x < VEC; ++x) wg_sum[wave][ls * VEC + x] = total[x];
        }
        __syncthreads();
        // the first wave of a run of equal rows takes the sums of the others
        bool first_of_run = true, run_goes_on = true;
#pragma unroll
        for (int w = 0; w < kWavesPerWg; ++w) {
            if (w + 1 == wave && item_row[w] == row) first_of_run = false;
            if (w > wave) {
                run_goes_on = run_goes_on && item_row[w] == row;
                if (run_goes_on && first_of_run) {
#pragma unroll
                    for (int x = 0; x < VEC; ++x) total[x] += wg_sum[w][ls * VEC + x];
                }
            }
        }
        if (!first_of_run) return;
    }
    A* c_lane = C + (size_t)row * n + tile + ls * VEC;
    if (STORE && it.whole) { // the row's only work item (the same in every lane): nothing to add to
#pragma unroll
        for (int x = 0; x < VEC; ++x)
            if (group == x / EPG && col_ok) c_lane[x] = total[x];
        return;
    }
#pragma unroll
    for (int x = 0; x < VEC; ++x)
        if (group == x / EPG && col_ok) atomicAdd(c_lane + x, total[x]);
}

// One group of LPR lanes per residue row (tail selection: RoDeSpmm.cu:71-82); the
// group walks its row's slot quads one after the other, no cross-lane reduction.
template <typename T, int TN, bool EDGE>
__device__ __forceinline__ void
spmm_residue_body(int bid, int nblocks, int m2, int n, int owned_slots, RowOwners owners,
                  const int* __restrict__ residue_rows,
                  const int* __restrict__ row_ptr, const int* __restrict__ col,
                  const typename DenseVec<T>::Acc* __restrict__ val, const T* __restrict__ B,
                  typename DenseVec<T>::Acc* __restrict__ C, const int* __restrict__ plan)
{
    using S = SpmmShape<T, TN>;
    using A = typename S::Acc;
    constexpr int VEC = S::kVec, LPR = S::kLpr;
    constexpr int RPW = kWave / LPR;        // rows per wave
    constexpr int OWN = kBlockItems / LPR;  // slots staged by one lane
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * RPW * kBlockItems];
    __shared__ __attribute__((aligned(16))) A lds_v[kWavesPerWg * RPW * kBlockItems];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int group = lane / LPR, ls = lane % LPR;
    const int item = (xcd_logical_block(bid, nblocks) * kWavesPerWg + wave) * RPW + group;
    if (item >= m2) return;

    if (plan && plan_residue_desc(plan, item / kPlanResidueChunk).wn > 0) return; // the window kernel has this chunk

    const int row = residue_rows[item];
    const ResidueItem it = residue_item(row, row_ptr);
    const bool accumulate = it.accumulate; // the row also has block segments
    if (accumulate && it.aligned <= owned_slots) return; // summed entirely, tail included, by the block kernel
    if (owned_elsewhere(owners, row, it.aligned)) return; // another kernel has the whole row
    const int first = it.first, cnt = it.cnt;

    const int tile = blockIdx.y * TN;
    const bool col_ok = !EDGE || tile + ls * VEC < n;
    int* my_c = lds_c + (wave * RPW + group) * kBlockItems;
    A* my_v = lds_v + (wave * RPW + group) * kBlockItems;

    A acc[VEC];
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = A(0);

    if (cnt > 0) {
        const int padded = (cnt + 3) & ~3; // slots past the tail repeat its last column with value 0
#pragma unroll
        for (int i = 0; i < OWN; ++i) {
            const int slot = ls + i * LPR;
            if (slot < padded) {
                my_c[slot] = col[first + min(slot, cnt - 1)];
                my_v[slot] = slot < cnt ? val[first + slot] : A(0);
            }
        }
        wave_lds_sync();
        // (two quads in flight where their dense rows fit 32 registers: config 4 K=64 0.550 -> 0.535 ms, K=32
        // 0.305 -> 0.292; with fp16's eight elements per load it costs waves per SIMD instead: 0.66 -> 0.76 ms)
        if constexpr (VEC <= 4)
            spmm_gather_pairs<T, TN, kBlockItems / 4>(B + tile + (col_ok ? ls * VEC : 0), (size_t)n, acc, my_c, my_v, padded / 4);
        else
            spmm_gather<T, TN, kBlockItems / 4, false>(B + tile + (col_ok ? ls * VEC : 0), (size_t)n, acc, my_c, my_v, 0, 1,
                                                       padded / 4);
    }

    A* c_lane = C + (size_t)row * n + tile + ls * VEC;
    if (!col_ok) return;
    if (accumulate) {
#pragma unroll
        for (int x = 0; x < VEC; ++x) atomicAdd(c_lane + x, acc[x]);
    } else {
        store_row<VEC>(c_lane, acc);
    }
}

template <typename T, int TN, bool EDGE, int WALK, bool STORE>
__global__ void __launch_bounds__(kWgThreads)
spmm_block_kernel(int m1, int n, int owned_slots, int chunk_hint, RowOwners owners, const int* __restrict__ block_rows,
                  const int* __restrict__ st_off,
                  const int* __restrict__ row_ptr, const int* __restrict__ col,
                  const typename DenseVec<T>::Acc* __restrict__ val, const T* __restrict__ B,
                  typename DenseVec<T>::Acc* __restrict__ C)
{
    spmm_block_body<T, TN, EDGE, WALK, STORE>(blockIdx.x, gridDim.x, m1, n, owned_slots, chunk_hint, owners, block_rows, st_off,
                                       row_ptr, col, val, B, C);
}

template <typename T, int TN, bool EDGE>
__global__ void __launch_bounds__(kWgThreads)
spmm_residue_kernel(int m2, int n, int owned_slots, RowOwners owners, const int* __restrict__ residue_rows,
                    const int* __restrict__ row_ptr, const int* __restrict__ col,
                    const typename DenseVec<T>::Acc* __restrict__ val, const T* __restrict__ B,
                    typename DenseVec<T>::Acc* __restrict__ C, const int* __restrict__ plan)
{
    spmm_residue_body<T, TN, EDGE>(blockIdx.x, gridDim.x, m2, n, owned_slots, owners, residue_rows, row_ptr, col, val, B,
                                   C, plan);
}

// Both lists in one launch: the first g1 workgroups of a grid row work on block segments,
// the others on residue rows.  For matrices so small that a launch costs as much as its
// kernel (a kernel of a few microseconds); the two parts then also fill the GPU together.
template <typename T, int TN, bool EDGE, bool STORE>
__global__ void __launch_bounds__(kWgThreads)
spmm_pair_kernel(int g1, int m1, int m2, int n, int owned_slots, int chunk_hint, RowOwners owners,
                 const int* __restrict__ block_rows,
                 const int* __restrict__ residue_rows, const int* __restrict__ st_off, const int* __restrict__ row_ptr,
                 const int* __restrict__ col, const typename DenseVec<T>::Acc* __restrict__ val,
                 const T* __restrict__ B, typename DenseVec<T>::Acc* __restrict__ C, const int* __restrict__ plan)
{
    if ((int)blockIdx.x < g1)
        spmm_block_body<T, TN, EDGE, 2, STORE>(blockIdx.x, g1, m1, n, owned_slots, 0, owners, block_rows, st_off, row_ptr, col, val,
                                        B, C);
    else
        spmm_residue_body<T, TN, EDGE>(blockIdx.x - g1, gridDim.x - g1, m2, n, max(owned_slots, 0), owners, residue_rows,
                                       row_ptr, col, val,
                                       B, C, plan);
}

// The groups of a group plan (rode_group.hip): four adjacent rows with runs of consecutive
// columns that overlap in a long shared run (shared_run).  One wave per group (WPG = 1), or a
// workgroup whose four waves split the shared run.  Every dense row of it is loaded once
// and multiplied into the sums of all four rows (its address follows from the run, no
// column index is read).  Then the rows' other nonzeros: with one wave per group, of the four rows together;
// with a workgroup, wave w adds row w's, the waves' sums meet in LDS, and wave w adds the
// total of row w to C.  A row is in no other work item: no atomics.
template <typename T, int TN, bool EDGE, int WPG>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
spmm_group_kernel(int n, int n_groups, const RowGroup* __restrict__ groups, const int* __restrict__ row_ptr,
                  const int* __restrict__ col, const typename DenseVec<T>::Acc* __restrict__ val,
                  const T* __restrict__ B, typename DenseVec<T>::Acc* __restrict__ C, bool overwrite)
{
    using S = SpmmShape<T, TN>;
    using A = typename S::Acc;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave, R = kGroupRows;
    constexpr int GPW = kWavesPerWg / WPG; // groups per workgroup
    static_assert(WPG == 1 || WPG == kWavesPerWg, "a group has one wave, or one workgroup");
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg][WPG == 1 ? R : 1][kWave];
    __shared__ __attribute__((aligned(16))) A lds_v[kWavesPerWg][R][kWave];
    __shared__ __attribute__((aligned(16))) A sums[WPG > 1 ? kWavesPerWg : 1][R][TN];
    // (the wave's number is the same in all its lanes; saying so keeps the group's description,
    // the position in the run and the addresses of its dense rows in scalar registers)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
    const int g = xcd_logical_block(blockIdx.x, gridDim.x) * GPW + wave / WPG;
    if (g >= n_groups) return;
    if (groups[g].len <= 0) return; // not a group: its rows are in the lists
    const RowGroup d = shared_run(groups[g]); // the columns [lo, lo + len) that all four runs hold
    const int w = wave % WPG; // this wave among the waves of its group
    const int ls = lane % LPR, group = lane / LPR;
    const int tile = blockIdx.y * TN;
    const bool col_ok = !EDGE || tile + ls * VEC < n;
    const T* b_lane = B + tile + (col_ok ? ls * VEC : 0);
    const int row0 = g * R;
    // per row: the slot of column j of the shared run is at[r] + j
    int at[R];
#pragma unroll
    for (int r = 0; r < R; ++r) at[r] = row_ptr[row0 + r] + d.pos[r];

    // this wave's share of the run, in quads of columns
    const int quads = (d.len + 3) / 4;
    const int q_begin = quads * w / WPG, q_end = quads * (w + 1) / WPG;
    const int j_end = min(d.len, 4 * q_end);
    A acc[R][VEC];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[r][x] = A(0);
    // a dense row of the run = a scalar address (start of the run, step, quad) + this lane's
    // 32-bit offset (its lane group's quad, its elements of the tile, the row in the quad)
    const T* b_run = B + tile + (size_t)d.lo * n;
    const unsigned row_bytes = (unsigned)n * (unsigned)sizeof(T);
    const unsigned lane_off = 4u * group * row_bytes + (col_ok ? ls * VEC * (unsigned)sizeof(T) : 0u); // in bytes
    A v_next[R]; // the values of the next step are loaded while this one is computed
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int j = 4 * q_begin + lane;
        v_next[r] = j < j_end ? val[at[r] + j] : A(0);
    }
    for (int j0 = 4 * q_begin; j0 < j_end; j0 += kWave) {
#pragma unroll
        for (int r = 0; r < R; ++r) lds_v[wave][r][lane] = v_next[r];
        wave_lds_sync();
        {
            const int j = j0 + kWave + lane;
#pragma unroll
            for (int r = 0; r < R; ++r) v_next[r] = j < j_end ? val[at[r] + j] : A(0);
        }
        const int nq = min(kWave / 4, (j_end - j0 + 3) / 4);
#pragma unroll
        for (int i = 0; i < kWave / 4 / G; ++i) {
            const int q = group + i * G;
            if (q < nq) {
                // four consecutive rows of B (the last quad of a run may be cut short: its rows
                // past the run repeat the run's last row, which every row of the group
                // references; their values are zero)
                const char* b_quad = reinterpret_cast<const char*>(b_run + (size_t)(j0 + 4 * i * G) * n);
                const int room = d.len - 1 - (j0 + 4 * q);
                const unsigned o1 = room >= 1 ? row_bytes : 0u;
                const unsigned o2 = room >= 2 ? 2u * row_bytes : o1;
                const unsigned o3 = room >= 3 ? 3u * row_bytes : o2;
                const unsigned off[4] = {lane_off, lane_off + o1, lane_off + o2, lane_off + o3};
                A b[4][VEC];
#pragma unroll
                for (int t = 0; t < 4; ++t) DenseVec<T>::load(reinterpret_cast<const T*>(b_quad + off[t]), b[t]);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    A v[4];
                    load_quad(&lds_v[wave][r][4 * q], v);
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int x = 0; x < VEC; ++x) acc[r][x] = fma(v[t], b[t][x], acc[r][x]);
                }
            }
        }
        wave_lds_sync();
    }
    if constexpr (WPG == 1) {
        // the nonzeros outside the run, of the four rows at once: their columns and values are
        // loaded together and their gathers follow each other without a wait in between (row
        // after row, a wave would sit through two memory round trips per row and step)
        int row_first[R], split[R], jump[R], cnt[R], max_cnt = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            row_first[r] = at[r] - d.pos[r];
            split[r] = d.pos[r];
            jump[r] = d.len;
            cnt[r] = split[r] + (row_ptr[row0 + r + 1] - (at[r] + d.len)); // the slots before the run + those after it
            max_cnt = max(max_cnt, cnt[r]);
        }
        for (int off = 0; off < max_cnt; off += kWave) {
            const int slot = off + lane;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int live = min(cnt[r] - off, kWave); // this row's slots in this step (may be <= 0)
                int c = 0;
                A v = A(0);
                if (lane < ((live + 3) & ~3)) { // (slots past the end of the last quad: value 0, column of a real slot)
                    const bool past = slot >= cnt[r];
                    const int slot_at = past ? cnt[r] - 1 : slot;
                    const int idx = row_first[r] + slot_at + (slot_at >= split[r] ? jump[r] : 0);
                    c = col[idx];
                    v = past ? A(0) : val[idx];
                }
                lds_c[wave][r][lane] = c;
                lds_v[wave][r][lane] = v;
            }
            wave_lds_sync();
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int live = min(cnt[r] - off, kWave);
                if (live >= kWave)
                    spmm_gather<T, TN, 16 / G, true>(b_lane, (size_t)n, acc[r], lds_c[wave][r], lds_v[wave][r], group, G, 16);
                else if (live > 0)
                    spmm_gather<T, TN, 16 / G, false>(b_lane, (size_t)n, acc[r], lds_c[wave][r], lds_v[wave][r], group, G,
                                                      (live + 3) / 4);
            }
            wave_lds_sync();
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int x = 0; x < VEC; ++x) acc[r][x] = butterfly_sum<LPR, kWave>(acc[r][x]);
            if (group == 0 && col_ok) {
                A* c_lane = C + (size_t)(row0 + r) * n + tile + ls * VEC;
#pragma unroll
                for (int x = 0; x < VEC; ++x) c_lane[x] = overwrite ? acc[r][x] : c_lane[x] + acc[r][x]; // (added by contract, unless told to store)
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int x = 0; x < VEC; ++x) acc[r][x] = butterfly_sum<LPR, kWave>(acc[r][x]);
            if (group == 0) {
#pragma unroll
                for (int x = 0; x < VEC; ++x) sums[wave][r][ls * VEC + x] = acc[r][x];
            }
        }
        __syncthreads();
        // the row this wave finishes: its nonzeros before and after the run, then the update of C
#pragma unroll
        for (int r = w; r < R; r += WPG) {
            const int row = row0 + r, s = row_ptr[row], e = row_ptr[row + 1];
            const int run_first = s + d.pos[r], run_end = run_first + d.run(r);
            A outside[VEC]; // the slots before the run and, in the same pass, those after it
            spmm_sum_slots<T, TN>(s, 0, (run_first - s) + (e - run_end), run_first - s, d.run(r), lane, lds_c[wave][0],
                                  &lds_v[wave][0][0], b_lane, n, col, val, outside);
            if (group == 0 && col_ok) {
                A* c_lane = C + (size_t)row * n + tile + ls * VEC;
#pragma unroll
                for (int x = 0; x < VEC; ++x) {
                    A total = outside[x];
#pragma unroll
                    for (int v = 0; v < WPG; ++v) total += sums[v][r][ls * VEC + x];
                    c_lane[x] = overwrite ? total : c_lane[x] + total; // (added by contract, unless told to store)
                }
            }
        }
    }
}

// The rows of a hub plan, cut into pieces by column slab (rode_items.hpp): one wave per
// piece, slab after slab, so that the hub rows' nonzeros of one slab of B are worked on at
// the same time on one XCD and find B's rows in its L2.  A piece's sum goes to its own row
// of `partial` (piece = slab group * hub rows + hub row; spmm_hub_reduce_kernel adds a row's
// pieces up), or, without that workspace, is added to its row of C atomically (a hub row
// then gets one atomic row update per slab: slower than the plain kernels at 512-byte rows).
template <typename T, int TN, bool EDGE>
__global__ void __launch_bounds__(kWgThreads)
spmm_hub_kernel(int n, int merge, const int* __restrict__ hub, const int* __restrict__ col,
                const typename DenseVec<T>::Acc* __restrict__ val, const T* __restrict__ B,
                typename DenseVec<T>::Acc* __restrict__ C, typename DenseVec<T>::Acc* __restrict__ partial)
{
    using S = SpmmShape<T, TN>;
    using A = typename S::Acc;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) A lds_v[kWavesPerWg * kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const HubPlan hp = hub_plan_view(hub);
    const long long item = (long long)xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (item >= (long long)hp.n_hub * hub_groups(hp.slabs, merge)) return;
    const int slab = (int)(item / hp.n_hub) * merge, h = (int)(item % hp.n_hub);
    const int* piece = hp.pieces + (size_t)h * (hp.slabs + 1);
    const int base = piece[slab], cnt = piece[min(slab + merge, hp.slabs)] - base;
    if (cnt <= 0) return; // (the reduction skips empty pieces too)
    const int row = hp.rows[h];
    const int ls = lane % LPR, group = lane / LPR;
    const int tile = blockIdx.y * TN;
    const bool col_ok = !EDGE || tile + ls * VEC < n;
    const T* b_lane = B + tile + (col_ok ? ls * VEC : 0);
    constexpr int EPG = VEC / G > 0 ? VEC / G : 1; // elements each group adds
    A total[VEC];
    spmm_sum_slots<T, TN>(base, 0, cnt, cnt, 0, lane, lds_c + wave * kWave, lds_v + wave * kWave, b_lane, n, col, val, total);
    if (partial) {
        if (group == 0 && col_ok) store_row<VEC>(partial + (size_t)item * n + tile + ls * VEC, total);
        return;
    }
    A* c_lane = C + (size_t)row * n + tile + ls * VEC;
#pragma unroll
    for (int x = 0; x < VEC; ++x)
        if (group == x / EPG && col_ok) atomicAdd(c_lane + x, total[x]);
}

// C[hub row, :] += sum of the row's pieces (a hub row is in no other work item, so no
// atomics; added, not stored, because long rows are accumulated into C by contract).  One workgroup per hub row: a group of n * sizeof / 16 threads reads a
// piece's partial row 16 bytes per thread, the groups take the slabs in turn and their
// sums are added up through LDS in a fixed order.
template <typename A>
__global__ void __launch_bounds__(kWgThreads)
spmm_hub_reduce_kernel(int n, int merge, const int* __restrict__ hub, const A* __restrict__ partial, A* __restrict__ C)
{
    constexpr int V = 16 / sizeof(A);
    __shared__ __attribute__((aligned(16))) A sums[kWgThreads * V];
    const HubPlan hp = hub_plan_view(hub);
    const int h = blockIdx.x;
    if (h >= hp.n_hub) return;
    const int* piece = hp.pieces + (size_t)h * (hp.slabs + 1);
    A* c_row = C + (size_t)hp.rows[h] * n;
    const int vecs = n / V; // 16-byte pieces of a row (n * sizeof(A) is a multiple of 16)
    for (int v0 = 0; v0 < vecs; v0 += kWgThreads) {
        const int width = min(vecs - v0, kWgThreads); // threads side by side on one partial row
        const int groups = kWgThreads / width;
        const int group = threadIdx.x / width, v = v0 + threadIdx.x % width;
        A sum[V];
#pragma unroll
        for (int x = 0; x < V; ++x) sum[x] = A(0);
        if (group < groups) {
            for (int sg = group; sg * merge < hp.slabs; sg += groups) {
                if (piece[min(sg * merge + merge, hp.slabs)] > piece[sg * merge]) {
                    const A* src = partial + ((size_t)sg * hp.n_hub + h) * n + (size_t)v * V;
#pragma unroll
                    for (int x = 0; x < V; ++x) sum[x] += src[x];
                }
            }
        }
#pragma unroll
        for (int x = 0; x < V; ++x) sums[threadIdx.x * V + x] = sum[x];
        __syncthreads();
        if (group == 0) {
            for (int g = 1; g < groups; ++g) {
#pragma unroll
                for (int x = 0; x < V; ++x) sum[x] += sums[(g * width + threadIdx.x) * V + x];
            }
#pragma unroll
            for (int x = 0; x < V; ++x) c_row[(size_t)v * V + x] += sum[x];
        }
        __syncthreads();
    }
}

constexpr int kClearRowsPerGroup = 8;

// Zeroes exactly the rows of C that the two SpMM kernels do not overwrite: rows whose
// aligned length N = len + (start & 3) is >= 32 are accumulated into, rows with N == 0
// belong to no work item; rows with 0 < N < 32 are stored by the residue kernel and
// are left alone.  16 lanes x 16 bytes per step and row.
__global__ void __launch_bounds__(kWgThreads)
spmm_clear_rows_kernel(int M, size_t row_bytes, const int* __restrict__ row_ptr, char* __restrict__ C)
{
    constexpr int kLanes = 16, kGroups = kWgThreads / kLanes;
    const int group = threadIdx.x / kLanes, lane = threadIdx.x % kLanes;
    const int first = xcd_logical_block(blockIdx.x, gridDim.x) * (kGroups * kClearRowsPerGroup);
    // batch b of a workgroup covers kGroups consecutive rows, one per lane group
    int s[kClearRowsPerGroup], e[kClearRowsPerGroup];
#pragma unroll
    for (int b = 0; b < kClearRowsPerGroup; ++b) {
        const int row = first + b * kGroups + group;
        s[b] = row < M ? row_ptr[row] : 1;
        e[b] = row < M ? row_ptr[row + 1] : 2; // N = 2: a row that is left alone
    }
#pragma unroll
    for (int b = 0; b < kClearRowsPerGroup; ++b) {
        const int N = e[b] - s[b] + (s[b] & (kVecLen - 1));
        if (N > 0 && N < kBlockItems) continue;
        char* dst = C + (size_t)(first + b * kGroups + group) * row_bytes;
        for (size_t off = lane * 16; off < row_bytes; off += kLanes * 16)
            *reinterpret_cast<uint4*>(dst + off) = make_uint4(0, 0, 0, 0);
    }
}

inline int grid_for_waves(long long nwaves)
{
    long long wgs = (nwaves + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds; // xcd_logical_block needs a multiple of kXcds
    // a launch dimension holds fewer than 2^32 threads; more work items than that (over
    // 16 M workgroups) are refused instead of being launched wrongly
    return wgs * kWgThreads < (1ll << 32) ? (int)wgs : -1;
}

template <typename T, int TN, bool EDGE>
hipError_t launch(int m1, int m2, int n, const int* block_rows, const int* residue_rows, const int* st_off,
                  const int* row_ptr, const int* col, const typename DenseVec<T>::Acc* val, const T* B,
                  typename DenseVec<T>::Acc* C, int flags, PlanRef plan, hipStream_t s1, hipStream_t s2)
{
    const int tiles = (n + TN - 1) / TN;
    const int owned_slots = (flags & kSpmmWholeLists) && m1 >= kOwnedMinSegments ? kOwnedRowSlots : 0;
    // what the block kernel is told: rows it owns, or (negative) only that it may merge short
    // segments - which needs no promise, and with this many segments costs no parallelism
    const int block_owned = owned_slots > 0 ? owned_slots : (m1 >= kMergeMinSegments ? -1 : 0);
    // a usable hub plan takes its rows out of both lists (the caller promised whole lists with it)
    const bool hub_plan = plan.hub != nullptr && plan.hub_counts != nullptr && plan.hub_counts[3] != 0 &&
                          plan.hub_counts[0] > 0;
    const bool group_plan = plan.groups != nullptr && plan.group_counts != nullptr && plan.group_counts[1] > 0;
    RowOwners owners;
    owners.hub_min_len = hub_plan ? plan.hub_counts[2] : 0;
    if (group_plan) {
        owners.groups = reinterpret_cast<const RowGroup*>(plan.groups + kGroupHeaderInts);
        owners.n_groups = plan.group_counts[0];
    }
    // rows with a single work item are stored instead of added (spmm_overwrite_limit says which)
    const bool overwrite = (flags & kSpmmOverwrite) != 0;
    owners.overwrite = overwrite && spmm_overwrite_limit(m1, hub_plan) > 0;
    const int only = flags & kOnlyMask; // one kernel family of the call (timing each on its own)
    const bool hubs = hub_plan && (only == 0 || only == kSpmmOnlyHub);
    const bool grouped = group_plan && (only == 0 || only == kSpmmOnlyHub); // (timed with the hub kernels)
    constexpr int RPW = kWave / SpmmShape<T, TN>::kLpr;
    // (segments per wave: known only when the caller said how long its segments are and merging is on)
    const int chunk_hint = block_owned != 0 ? chunk_for_segments(plan.seg_length, m1) : (plan.seg_length > 0 ? 1 : 0);
    const int g1 = chunk_hint > 0 ? grid_for_waves((m1 + chunk_hint - 1) / chunk_hint) : grid_for_waves(min(m1, kBlockGridWaves));
    const int g2 = grid_for_waves(((long long)m2 + RPW - 1) / RPW);
    if (g1 < 0 || g2 < 0 || tiles > 65535) return hipErrorInvalidConfiguration;
    // With a host copy of the plan's header, a kernel that would find every chunk taken by
    // the other one is not launched at all.
    bool standard_residue = true, window_residue = plan.dev != nullptr;
    if (plan.dev && plan.host_counts) {
        standard_residue = plan.host_counts[1] < plan.host_counts[0];
        window_residue = plan.host_counts[1] > 0;
    }
    // (every row in a group with a run: the lists' kernels would find nothing to do)
    const bool lists = !(group_plan && plan.group_counts[2] == 0);
    const bool block = lists && m1 > 0 && (only == 0 || only == kSpmmOnlyBlock);
    const bool residue = lists && m2 > 0 && (only == 0 || only == kSpmmOnlyResidue);
    hipError_t e = hipSuccess;
    if (block && residue && standard_residue && s1 == s2 && (long long)(g1 + g2) * tiles <= kPairMaxWorkgroups) {
        dim3 grid(g1 + g2, tiles);
        auto kernel = owners.overwrite ? spmm_pair_kernel<T, TN, EDGE, true> : spmm_pair_kernel<T, TN, EDGE, false>;
        kernel<<<grid, kWgThreads, 0, s1>>>(g1, m1, m2, n, block_owned, chunk_hint, owners, block_rows, residue_rows, st_off,
                                            row_ptr, col, val, B, C, plan.dev);
        e = hipGetLastError();
    } else {
        if (block) {
            dim3 grid(g1, tiles);
            auto kernel = spmm_block_kernel<T, TN, EDGE, 2, false>;
            if (chunk_hint == 1)
                kernel = owners.overwrite ? spmm_block_kernel<T, TN, EDGE, 0, true> : spmm_block_kernel<T, TN, EDGE, 0, false>;
            else if (chunk_hint > 1)
                kernel = owners.overwrite ? spmm_block_kernel<T, TN, EDGE, 1, true> : spmm_block_kernel<T, TN, EDGE, 1, false>;
            else if (owners.overwrite)
                kernel = spmm_block_kernel<T, TN, EDGE, 2, true>;
            kernel<<<grid, kWgThreads, 0, s1>>>(m1, n, block_owned, chunk_hint, owners, block_rows, st_off, row_ptr, col, val, B, C);
            e = hipGetLastError();
        }
        if (residue && standard_residue) {
            dim3 grid(g2, tiles);
            spmm_residue_kernel<T, TN, EDGE><<<grid, kWgThreads, 0, s2>>>(m2, n, owned_slots, owners, residue_rows, row_ptr, col,
                                                                          val, B, C, plan.dev);
            if (e == hipSuccess) e = hipGetLastError();
        }
    }
    if (e == hipSuccess && hubs) {
        using A = typename DenseVec<T>::Acc;
        const int merge = hub_merge(n * (int)sizeof(A) / 4);
        const long long pieces = (long long)plan.hub_counts[0] * hub_groups(plan.hub_counts[1], merge);
        const int gh = grid_for_waves(pieces);
        if (gh < 0) return hipErrorInvalidConfiguration;
        dim3 grid(gh, tiles);
        const size_t need = (size_t)pieces * n * sizeof(A);
        A* partial = plan.hub_workspace && plan.hub_workspace_bytes >= need ? static_cast<A*>(plan.hub_workspace) : nullptr;
        spmm_hub_kernel<T, TN, EDGE><<<grid, kWgThreads, 0, s1>>>(n, merge, plan.hub, col, val, B, C, partial);
        if (partial) spmm_hub_reduce_kernel<A><<<plan.hub_counts[0], kWgThreads, 0, s1>>>(n, merge, plan.hub, partial, C);
        e = hipGetLastError();
    }
    if (e == hipSuccess && grouped) {
        // one wave per group when there are groups enough to fill the GPU that way (measured on
        // the attention-mask benchmark, 4096 groups: 0.042 against 0.062 ms), else a workgroup
        if (plan.group_counts[1] >= kGroupWaveEach) {
            const int wgs = (owners.n_groups + kWavesPerWg - 1) / kWavesPerWg;
            dim3 grid((wgs + kXcds - 1) / kXcds * kXcds, tiles);
            spmm_group_kernel<T, TN, EDGE, 1><<<grid, kWgThreads, 0, s1>>>(n, owners.n_groups, owners.groups, row_ptr, col,
                                                                           val, B, C, overwrite);
        } else {
            dim3 grid((owners.n_groups + kXcds - 1) / kXcds * kXcds, tiles);
            spmm_group_kernel<T, TN, EDGE, kWavesPerWg><<<grid, kWgThreads, 0, s1>>>(n, owners.n_groups, owners.groups, row_ptr,
                                                                                     col, val, B, C, overwrite);
        }
        e = hipGetLastError();
    }
    if constexpr (!std::is_same<T, double>::value) {
        if (e == hipSuccess && residue && window_residue)
            e = spmm_window_launch<T>(m2, n, owned_slots, col, val, B, C, plan.dev, plan.rows, s2);
    }
    return e;
}

template <typename T, int TN>
hipError_t launch_edge(int m1, int m2, int n, const int* block_rows, const int* residue_rows, const int* st_off,
                       const int* row_ptr, const int* col, const typename DenseVec<T>::Acc* val, const T* B,
                       typename DenseVec<T>::Acc* C, int flags, PlanRef plan, hipStream_t s1, hipStream_t s2)
{
    return n % TN ? launch<T, TN, true>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C,
                                        flags, plan, s1, s2)
                  : launch<T, TN, false>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C,
                                         flags, plan, s1, s2);
}

} // namespace

// The longest row (in aligned slots) that an SpMM call with m1 block segments, the whole-lists
// promise and kSpmmOverwrite stores with a single work item instead of adding to it; 0: none
// of the rows that have block segments (rows of fewer than 32 aligned slots are always
// stored, rows of kept groups of a group plan under kSpmmOverwrite as well).
int spmm_overwrite_limit(int m1, bool hub_plan) { return m1 >= kOwnedMinSegments && !hub_plan ? kOwnedRowSlots : 0; }

// n: any positive multiple of the 128-bit vector width (4 fp32, 8 fp16, 2 fp64).  The
// dense row is cut into tiles of 32, 64 or 128 columns (at most 32 lanes per tile row);
// the tile width with the least padding wins, the widest on a tie.  Multiples of 32 (all
// the reference supports) run without any bounds test.  Chunks of the residue list for
// which `plan` holds a window go to the window kernel (fp32 and fp16 operands wider than
// one 128-byte tile; fp64 and narrower operands ignore the plan: with a single tile the
// window is not reused often enough to repay its staging).
template <typename T>
hipError_t spmm_launch(int m1, int m2, int n, const int* block_rows, const int* residue_rows, const int* st_off,
                       const int* row_ptr, const int* col, const typename SpmmAcc<T>::type* val, const T* B,
                       typename SpmmAcc<T>::type* C, int flags, PlanRef plan, hipStream_t s1, hipStream_t s2)
{
    static_assert(std::is_same<typename SpmmAcc<T>::type, typename DenseVec<T>::Acc>::value, "accumulation type");
    if (n <= 0 || n % DenseVec<T>::kElems != 0) return hipErrorInvalidValue;
    // the window kernels are for fp32 / fp16 operands with more than one 128-byte tile per row
    if (std::is_same<T, double>::value || (size_t)n * sizeof(T) <= 128) {
        plan.dev = nullptr;
        plan.rows = nullptr;
        plan.host_counts = nullptr;
    }
    constexpr int kMaxTile = 32 * DenseVec<T>::kElems >= 128 ? 128 : 32 * DenseVec<T>::kElems;
    auto padded = [n](int tn) { return (n + tn - 1) / tn * tn; };
    int best = 32;
    if (padded(64) <= padded(best)) best = 64;
    if (kMaxTile >= 128 && padded(128) <= padded(best)) best = 128;
    if constexpr (kMaxTile >= 128) {
        if (best == 128)
            return launch_edge<T, 128>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C, flags,
                                       plan, s1, s2);
    }
    if (best == 64)
        return launch_edge<T, 64>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C, flags, plan,
                                  s1, s2);
    return launch_edge<T, 32>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C, flags, plan, s1, s2);
}

hipError_t spmm_clear_rows_launch(int M, size_t row_bytes, const int* row_ptr, void* C, hipStream_t stream)
{
    if (M <= 0) return hipSuccess;
    constexpr int kRowsPerWg = kWgThreads / 16 * kClearRowsPerGroup;
    long long wgs = ((long long)M + kRowsPerWg - 1) / kRowsPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds;
    if (wgs * kWgThreads >= (1ll << 32)) return hipErrorInvalidConfiguration;
    spmm_clear_rows_kernel<<<(int)wgs, kWgThreads, 0, stream>>>(M, row_bytes, row_ptr, static_cast<char*>(C));
    return hipGetLastError();
}

template hipError_t spmm_launch<float>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                       const float*, const float*, float*, int, PlanRef, hipStream_t, hipStream_t);
template hipError_t spmm_launch<__half>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                        const float*, const __half*, float*, int, PlanRef, hipStream_t, hipStream_t);
template hipError_t spmm_launch<double>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                        const double*, const double*, double*, int, PlanRef, hipStream_t, hipStream_t);

} // namespace rode
