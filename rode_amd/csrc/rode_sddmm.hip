// SDDMM over a row-decomposed CSR pattern:
//     out[idx] = values[idx] * < lhs[row(idx), :], rhs[col(idx), :] >
// Same work split and index arithmetic as the reference's SDDMMKernel4Block
// (RoDe_SDDMM/RoDeSddmm.cu:15-203) and SDDMMKernel4Residue (:206-494); the
// execution shape is written for 64-lane wavefronts:
//
//   * block kernel: a "unit" is 32 consecutive nonzero slots handled by one 32-lane
//     half of a wave: lane e of the half owns slot e (its column index, its value,
//     its output), so sparse loads and the final store are fully coalesced;
//   * inside a half, groups of LPR = KT / (elements per 128-bit load) lanes read one
//     dense rhs row (KT = 32, 64 or 128 elements of it at a time; K up to 4 such
//     slabs) per load instruction, LPR rows per group per unit;
//   * the K-slices of four rows at a time are combined with a transpose-reduce
//     (DPP quad_perm for xor 1/2, ds_swizzle for xor 4/8/16) that leaves the dot
//     product of slot e in lane e;
//   * one wave walks one block segment, 64 slots per step, the lhs row slice stays
//     in registers for the whole segment;
//   * residue kernel: each group of LPR lanes takes one residue row (< 32 slots),
//     so a wave works on 64 / LPR rows at once (2 at K=128 fp32, 8 at K=32):
//     short rows are latency-bound and need many rows in flight per wave.
#include "rode_items.hpp"
#include "rode_units.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

// out[idx] = values[idx] * <lhs[row, :], rhs[col(idx), :]> for the aligned slots
// [base, base + cnt) of one row, 64 slots per step; the first `mask` slots (the previous
// row's) are computed but not stored.
// (split, jump: the slots are [base, base + split) followed by [base + split + jump, ...):
// a row with a hole that somebody else works on; split >= cnt for one plain range.)
template <typename T, int KT, int NS, bool EDGE>
__device__ __forceinline__ void sddmm_row_slots(int row, int base, int mask, int cnt, int split, int jump, int k, int lane,
                                                int* lds_cols,
                                                const int* __restrict__ col, const float* __restrict__ val,
                                                const T* __restrict__ lhs, const T* __restrict__ rhs,
                                                float* __restrict__ out)
{
    using S = SddmmShape<T, KT>;
    typename S::Reg a[NS][S::kRegs];
    load_lhs_slice<T, KT, NS, EDGE>(lhs, row, k, lane, a);
    const T* rhs_lane = rhs + (lane % S::kLpr) * S::kVec;

    for (int off = 0; off < cnt; off += kWave) {
        if (off + (lane & 32) < cnt) { // the upper half sits out a trailing 32-slot step
            const int slot = off + lane;
            // cnt is a multiple of 32 for every decomposition the kernels are specified for
            // (segment length a multiple of 32).  Lists made with another segment length must
            // still never make a lane read or write beyond its row's block part: such lanes
            // repeat the last slot and store nothing.
            const bool live = slot < cnt;
            const int at = live ? slot : cnt - 1;
            const int idx = base + at + (at >= split ? jump : 0);
            const int c = col[idx];
            const float v = val[idx];
            const float d = sddmm_unit<T, KT, NS, EDGE>(rhs_lane, a, c, k, lds_cols, lane);
            if (slot >= mask && live) out[idx] = v * d;
        }
    }
}

// One wave per block segment.  Segment s covers the aligned slots
// [base, base + cnt) with base = st_off[s] & ~3 and cnt = floor((len + mask) / 32) * 32
// (RoDeSddmm.cu:35-54); the first `mask` slots belong to the previous row and are
// computed but never stored (RoDeSddmm.cu:56-58, 197).
// (bid of nblocks: the workgroup's position in the part of the grid that works on block segments)
template <typename T, int KT, int NS, bool EDGE>
__device__ __forceinline__ void
sddmm_block_body(int bid, int nblocks, int m1, int k, int chunk_hint, RowOwners owners, const int* __restrict__ block_rows,
                 const int* __restrict__ st_off,
                 const int* __restrict__ row_ptr, const int* __restrict__ col, const float* __restrict__ val,
                 const T* __restrict__ lhs, const T* __restrict__ rhs, float* __restrict__ out)
{
    __shared__ __attribute__((aligned(16))) int lds[kWavesPerWg * kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    // Lists with short segments, and many of them: a wave walks a chunk of consecutive
    // segments from leader to leader, with windows of kWalkSlots slots (rode_items.hpp).
    const int chunk = chunk_hint > 0 ? chunk_hint
                                     : block_chunk_for_grid(m1 >= kWalkMinSegments ? block_chunk(m1, block_rows, st_off) : 1, m1, nblocks);
    if (chunk > 1) {
        const long long first = chunk_first_segment(bid, wave, m1, chunk);
        if (first < 0) return;
        const int last = (int)min(first + chunk, (long long)m1);
        for (int from = (int)first; from < last; from += kScanSegments) {
            const ChunkScan scan = scan_chunk(kWalkSlots, from, m1, 0, owners, lane, block_rows, st_off, row_ptr);
            const int count = min(last - from, kScanSegments);
            for (unsigned long long todo = scan.items & ((1ull << count) - 1ull); todo; todo &= todo - 1ull) {
                const BlockItem it = chunk_item(scan, __builtin_ctzll(todo));
                sddmm_row_slots<T, KT, NS, EDGE>(it.row, it.base, it.mask, it.cnt, it.cnt, 0, k, lane, lds + wave * kWave, col,
                                                 val, lhs, rhs, out);
            }
        }
        return;
    }
    const int seg = xcd_logical_block(bid, nblocks) * kWavesPerWg + wave;
    if (seg >= m1) return;

    // Consecutive segments of one row whose starts fall into the same window of
    // kSddmmMergeSlots slots are handled by the wave of the first of them, so a decomposition
    // with short segments (32 in the reference's K=128 parameter set) still fills whole
    // 64-slot steps and loads the lhs row once.  Longer segments are unaffected.  (Outputs
    // are pure functions of the inputs, so this is safe even when a caller passes a slice of
    // the lists: the worst case is an output computed twice.)
    BlockItem it;
    if (!sddmm_block_item(seg, m1, owners, lane, block_rows, st_off, row_ptr, it)) return;
    const int row = it.row, mask = it.mask, base = it.base, cnt = it.cnt;

    sddmm_row_slots<T, KT, NS, EDGE>(row, base, mask, cnt, cnt, 0, k, lane, lds + wave * kWave, col, val, lhs, rhs, out);
}

// One group of LPR lanes per residue row.  Tail selection follows RoDeSddmm.cu:237-243:
// with N = len + (s & 3), rows with N >= 32 keep only their last N % 32 slots
// starting at (s & ~3) + floor(N / 32) * 32; shorter rows are taken whole.
// Lane ls of the group owns the slots ls, ls + LPR, ... (value, result, store).
template <typename T, int KT, int NS, bool EDGE>
__device__ __forceinline__ void
sddmm_residue_body(int bid, int nblocks, int m2, int k, RowOwners owners, const int* __restrict__ residue_rows,
                   const int* __restrict__ row_ptr, const int* __restrict__ col, const float* __restrict__ val,
                   const T* __restrict__ lhs, const T* __restrict__ rhs, float* __restrict__ out,
                   const int* __restrict__ plan)
{
    using S = SddmmShape<T, KT>;
    constexpr int VEC = S::kVec, LPR = S::kLpr;
    constexpr int RPW = kWave / LPR;          // rows per wave
    constexpr int OWN = kBlockItems / LPR;    // slots owned by one lane
    constexpr int LQ = LPR / 4;               // lane quads per group
    __shared__ __attribute__((aligned(16))) int lds[kWavesPerWg * RPW * kBlockItems];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int group = lane / LPR, ls = lane % LPR;
    const int item = (xcd_logical_block(bid, nblocks) * kWavesPerWg + wave) * RPW + group;
    if (item >= m2) return;
    if (plan && plan_residue_desc(plan, item / kPlanResidueChunk).wn > 0) return; // the window kernel has this chunk

    const int row = residue_rows[item];
    const ResidueItem it = residue_item(row, row_ptr);
    const int first = it.first, cnt = it.cnt;
    if (cnt <= 0) return; // an empty, unaligned row is listed as a residue but owns no slot
    if (owned_elsewhere(owners, row, it.aligned)) return; // another kernel has the whole row

    int* my_cols = lds + (wave * RPW + group) * kBlockItems;
    float v[OWN];
    const int padded = (cnt + 3) & ~3; // slots past the tail repeat its last column
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        const int slot = ls + i * LPR;
        v[i] = 0.f;
        if (slot < padded) {
            const int idx = first + min(slot, cnt - 1);
            my_cols[slot] = col[idx];
            v[i] = val[idx];
        }
    }
    typename S::Reg a[NS][S::kRegs];
    load_lhs_slice<T, KT, NS, EDGE, true>(lhs, row, k, lane, a);
    const T* rhs_lane = rhs + ls * VEC;
    wave_lds_sync();

    float res[OWN];
#pragma unroll
    for (int i = 0; i < OWN; ++i) res[i] = 0.f;
    const int nquads = padded / 4;
#pragma unroll
    for (int q = 0; q < kBlockItems / 4; ++q) {
        if (q < nquads) {
            const int4 c4 = *reinterpret_cast<const int4*>(my_cols + 4 * q);
            const int c[4] = {c4.x, c4.y, c4.z, c4.w};
            float p[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                p[j] = lane_dot<T, KT, NS, EDGE>(a, rhs_lane + (size_t)c[j] * k, k, ls * VEC);
            const bool hi2 = ls & 2, hi1 = ls & 1;
            const float q0 = (hi2 ? p[2] : p[0]) + lane_xor2(hi2 ? p[0] : p[2]);
            const float q1 = (hi2 ? p[3] : p[1]) + lane_xor2(hi2 ? p[1] : p[3]);
            float r = (hi1 ? q1 : q0) + lane_xor1(hi1 ? q0 : q1);
            r = butterfly_sum<4, LPR>(r);
            // slot 4q + (ls & 3) belongs to lane (4q + (ls & 3)) % LPR, register (4q) / LPR
            if ((ls >> 2) == q % LQ) res[q / LQ] = r;
        }
    }
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        const int slot = ls + i * LPR;
        if (slot < cnt) out[first + slot] = v[i] * res[i];
    }
}

template <typename T, int KT, int NS, bool EDGE>
__global__ void __launch_bounds__(kWgThreads)
sddmm_block_kernel(int m1, int k, int chunk_hint, RowOwners owners, const int* __restrict__ block_rows,
                   const int* __restrict__ st_off,
                   const int* __restrict__ row_ptr, const int* __restrict__ col, const float* __restrict__ val,
                   const T* __restrict__ lhs, const T* __restrict__ rhs, float* __restrict__ out)
{
    sddmm_block_body<T, KT, NS, EDGE>(blockIdx.x, gridDim.x, m1, k, chunk_hint, owners, block_rows, st_off, row_ptr, col, val,
                                      lhs, rhs, out);
}

template <typename T, int KT, int NS, bool EDGE>
__global__ void __launch_bounds__(kWgThreads)
sddmm_residue_kernel(int m2, int k, RowOwners owners, const int* __restrict__ residue_rows, const int* __restrict__ row_ptr,
                     const int* __restrict__ col, const float* __restrict__ val, const T* __restrict__ lhs,
                     const T* __restrict__ rhs, float* __restrict__ out, const int* __restrict__ plan)
{
    sddmm_residue_body<T, KT, NS, EDGE>(blockIdx.x, gridDim.x, m2, k, owners, residue_rows, row_ptr, col, val, lhs, rhs,
                                        out, plan);
}

// Both lists in one launch: the first g1 workgroups work on block segments, the others on
// residue rows.  For matrices so small that a launch costs as much as its kernel.
template <typename T, int KT, int NS, bool EDGE>
__global__ void __launch_bounds__(kWgThreads)
sddmm_pair_kernel(int g1, int m1, int m2, int k, int chunk_hint, RowOwners owners, const int* __restrict__ block_rows,
                  const int* __restrict__ residue_rows,
                  const int* __restrict__ st_off, const int* __restrict__ row_ptr, const int* __restrict__ col,
                  const float* __restrict__ val, const T* __restrict__ lhs, const T* __restrict__ rhs,
                  float* __restrict__ out, const int* __restrict__ plan)
{
    if ((int)blockIdx.x < g1)
        sddmm_block_body<T, KT, NS, EDGE>(blockIdx.x, g1, m1, k, chunk_hint, owners, block_rows, st_off, row_ptr, col, val, lhs,
                                          rhs, out);
    else
        sddmm_residue_body<T, KT, NS, EDGE>(blockIdx.x - g1, gridDim.x - g1, m2, k, owners, residue_rows, row_ptr, col, val, lhs,
                                            rhs, out, plan);
}

// The nonzeros of a kept group outside its run, of the four rows at once: 64 slots per row
// and step, their columns and values loaded together, their dot products one row after the
// other without a wait in between (row after row, a wave sits through the memory round trips
// of every row).  lds_cols: kGroupRows * 64 ints of this wave.
template <typename T, int KT, bool EDGE>
__device__ __forceinline__ void sddmm_group_leftovers(const RowGroup& d, int row0, int k, int lane,
                                                      int* lds_cols, const int* __restrict__ row_ptr,
                                                      const int* __restrict__ col, const float* __restrict__ val,
                                                      const T* __restrict__ lhs, const T* __restrict__ rhs,
                                                      float* __restrict__ out)
{
    using S = SddmmShape<T, KT>;
    constexpr int R = kGroupRows;
    typename S::Reg a[R][1][S::kRegs];
    int row_first[R], split[R], jump[R], cnt[R], max_cnt = 0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        load_lhs_slice<T, KT, 1, EDGE>(lhs, row0 + r, k, lane, a[r]);
        row_first[r] = row_ptr[row0 + r];
        split[r] = d.pos[r];
        jump[r] = d.run(r);
        cnt[r] = row_ptr[row0 + r + 1] - row_first[r] - jump[r]; // the slots before the run + those after it
        max_cnt = max(max_cnt, cnt[r]);
    }
    const T* rhs_lane = rhs + (lane % S::kLpr) * S::kVec;
    for (int off = 0; off < max_cnt; off += kWave) {
        const int slot = off + lane;
        int idx[R];
        float v[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            idx[r] = -1;
            v[r] = 0.f;
            int c = 0;
            if (off + (lane & 32) < cnt[r]) { // (a row without slots in this half of the step reads nothing)
                const bool live = slot < cnt[r];
                const int at = live ? slot : cnt[r] - 1; // (lanes past the end repeat the last slot and store nothing)
                const int i = row_first[r] + at + (at >= split[r] ? jump[r] : 0);
                c = col[i];
                if (live) {
                    idx[r] = i;
                    v[r] = val[i];
                }
            }
            lds_cols[r * kWave + lane] = c;
        }
        wave_lds_sync();
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (off + (lane & 32) < cnt[r]) {
                const float dot = sddmm_unit_staged<T, KT, 1, EDGE>(rhs_lane, a[r], k, lds_cols + r * kWave, lane);
                if (idx[r] >= 0) out[idx[r]] = v[r] * dot;
            }
        }
        wave_lds_sync();
    }
}

// The groups of a group plan (rode_group.hip): four adjacent rows with runs of consecutive
// columns that overlap in a long shared run (shared_run).  One wave per group (WPG = 1), or a
// workgroup whose four waves split the shared run.  Every rhs row of it is loaded once
// (its address follows from the run, no column index is read) and multiplied with the lhs
// rows of all four rows of the group, which stay in registers.  Then the rows' other nonzeros: with one wave per
// group, of the four rows together (sddmm_group_leftovers); with a workgroup, wave w takes
// row w's.  Single-slab rows only (k <= 128 elements per lane tile): four lhs slices of more
// slabs would not fit.
// (A variant in which the four waves of a workgroup took four consecutive groups and read
// the union of their runs through LDS tiles, loaded once per workgroup, ran in the same
// time on config 5 - 0.049 ms fp32, 0.035 against 0.033 ms fp16 - and was taken out.)
template <typename T, int KT, bool EDGE, int WPG>
__global__ void __launch_bounds__(kWgThreads)
sddmm_group_kernel(int k, int n_groups, const RowGroup* __restrict__ groups, const int* __restrict__ row_ptr,
                   const int* __restrict__ col, const float* __restrict__ val, const T* __restrict__ lhs,
                   const T* __restrict__ rhs, float* __restrict__ out)
{
    using S = SddmmShape<T, KT>;
    constexpr int LPR = S::kLpr, VEC = S::kVec, R = kGroupRows;
    static_assert(WPG == 1 || WPG == kWavesPerWg, "a group has one wave, or one workgroup");
    __shared__ __attribute__((aligned(16))) int lds[kWavesPerWg * (WPG == 1 ? R : 1) * kWave];
    // (the wave's number is the same in all its lanes; saying so keeps the group's description,
    // the position in the run and the base address of its rhs rows in scalar registers)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
    const int g = xcd_logical_block(blockIdx.x, gridDim.x) * (kWavesPerWg / WPG) + wave / WPG;
    if (g >= n_groups) return;
    if (groups[g].len <= 0) return; // not a group: its rows are in the lists
    const RowGroup d = shared_run(groups[g]); // the columns [lo, lo + len) that all four runs hold
    const int w = wave % WPG; // this wave among the waves of its group
    const int row0 = g * R;
    // per row: the slot of column j of the shared run is at[r] + j
    int at[R];
#pragma unroll
    for (int r = 0; r < R; ++r) at[r] = row_ptr[row0 + r] + d.pos[r];
    // this wave's share of the run, in quads of columns; lane e of a step has column j0 + e
    const int quads = (d.len + 3) / 4;
    const int q_begin = quads * w / WPG, q_end = quads * (w + 1) / WPG;
    const int j_end = min(d.len, 4 * q_end);
    // an rhs row of the run = a scalar address (the run's first row at this step) + this lane's
    // 32-bit offset (row within the step, the lane's elements)
    const unsigned row_bytes = (unsigned)k * (unsigned)sizeof(T);
    const T* rhs_run = rhs + (size_t)d.lo * k;
    // LP lanes per rhs row, each with E of its 16-byte vectors (LP lanes apart): half as many lanes
    // as a row has vectors, so that a dot product crosses half as many lanes as in the list
    // kernels, and the lhs rows of the group still fit 32 registers.  (With four lanes per row
    // at fp32 rows of 64 - 64 registers of lhs rows, 164 in all, a wave less per SIMD - config 5
    // took 0.075 ms instead of 0.059; from an LDS copy of the lhs rows the compiler spends the
    // registers on loads in flight instead; two passes of two rows each: 0.078 ms.)
    constexpr int LP = LPR >= 8 ? LPR / 2 : LPR, E = LPR / LP;
    const int lp = lane % LP; // this lane among the lanes of its rhs row
    typename S::Reg a[R][E][S::kRegs];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int i = 0; i < E; ++i) {
            DotVec<T>::zero(a[r][i]);
            if (!EDGE || (lp + LP * i) * VEC < k) DotVec<T>::load(lhs + (size_t)(row0 + r) * k + (lp + LP * i) * VEC, a[r][i]);
        }
    const int group_first = lane - lp; // first column (within the step) of this lane group
    for (int j0 = 4 * q_begin; j0 < j_end; j0 += kWave) {
        if (j0 + (lane & 32) < j_end) { // the upper half sits out a step that has nothing for it
            const char* step_rows = reinterpret_cast<const char*>(rhs_run + (size_t)j0 * k);
            float result[R];
#pragma unroll
            for (int r = 0; r < R; ++r) result[r] = 0.f;
#pragma unroll
            for (int q = 0; q < LP / 4; ++q) {
                float p[R][4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const unsigned at = __umul24(min(group_first + 4 * q + t, d.len - 1 - j0), row_bytes) + lp * VEC * (unsigned)sizeof(T);
#pragma unroll
                    for (int r = 0; r < R; ++r) p[r][t] = 0.f;
#pragma unroll
                    for (int i = 0; i < E; ++i) {
                        uint4 b = make_uint4(0u, 0u, 0u, 0u);
                        if (!EDGE || (lp + LP * i) * VEC < k)
                            b = *reinterpret_cast<const uint4*>(step_rows + (at + LP * i * VEC * (unsigned)sizeof(T)));
#pragma unroll
                        for (int r = 0; r < R; ++r) p[r][t] = DotVec<T>::dot_raw(a[r][i], b, p[r][t]);
                    }
                }
                // transpose-reduce per row: afterwards lane (lp & 3) == t holds column t of the quad
                const bool hi2 = lp & 2, hi1 = lp & 1;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float q0 = (hi2 ? p[r][2] : p[r][0]) + lane_xor2(hi2 ? p[r][0] : p[r][2]);
                    const float q1 = (hi2 ? p[r][3] : p[r][1]) + lane_xor2(hi2 ? p[r][1] : p[r][3]);
                    float v = (hi1 ? q1 : q0) + lane_xor1(hi1 ? q0 : q1);
                    v = butterfly_sum<4, LP>(v);
                    if ((lp >> 2) == q) result[r] = v;
                }
            }
            const int j = j0 + lane;
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (j < j_end) out[at[r] + j] = val[at[r] + j] * result[r];
        }
    }
    if constexpr (WPG == 1) {
        sddmm_group_leftovers<T, KT, EDGE>(d, row0, k, lane, lds + wave * kGroupRows * kWave, row_ptr, col, val, lhs, rhs, out);
    } else {
        // the rows this wave finishes: their nonzeros before and after the run
#pragma unroll
        for (int r = w; r < R; r += WPG) {
            const int row = row0 + r, s = row_ptr[row], e = row_ptr[row + 1];
            const int run_first = s + d.pos[r], run_end = run_first + d.run(r);
            // (the slots before the run and, in the same pass, those after it)
            sddmm_row_slots<T, KT, 1, EDGE>(row, s, 0, (run_first - s) + (e - run_end), run_first - s, d.run(r), k, lane,
                                            lds + wave * kWave, col, val, lhs, rhs, out);
        }
    }
}

// The rows of a hub plan, cut into pieces by column slab (rode_items.hpp): one wave per
// piece, slab after slab, so that the hub rows' nonzeros of one slab of rhs are worked on
// at the same time on one XCD and find its rows in that XCD's L2.
template <typename T, int KT, int NS, bool EDGE>
__global__ void __launch_bounds__(kWgThreads)
sddmm_hub_kernel(int k, int merge, const int* __restrict__ hub, const int* __restrict__ col, const float* __restrict__ val,
                 const T* __restrict__ lhs, const T* __restrict__ rhs, float* __restrict__ out)
{
    __shared__ __attribute__((aligned(16))) int lds[kWavesPerWg * kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const HubPlan hp = hub_plan_view(hub);
    const long long item = (long long)xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (item >= (long long)hp.n_hub * hub_groups(hp.slabs, merge)) return;
    const int slab = (int)(item / hp.n_hub) * merge, h = (int)(item % hp.n_hub);
    const int* piece = hp.pieces + (size_t)h * (hp.slabs + 1);
    const int base = piece[slab], cnt = piece[min(slab + merge, hp.slabs)] - base;
    if (cnt <= 0) return;
    sddmm_row_slots<T, KT, NS, EDGE>(hp.rows[h], base, 0, cnt, cnt, 0, k, lane, lds + wave * kWave, col, val, lhs, rhs, out);
}

// Up to this many workgroups, and when both kernels go to the same stream, the two lists
// are processed by one launch.
constexpr int kPairMaxWorkgroups = 16384;

inline int grid_for_waves(long long nwaves)
{
    long long wgs = (nwaves + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds; // xcd_logical_block needs a multiple of kXcds
    // a launch dimension holds fewer than 2^32 threads; more work items than that (over
    // 16 M workgroups) are refused instead of being launched wrongly
    return wgs * kWgThreads < (1ll << 32) ? (int)wgs : -1;
}

template <typename T, int KT, int NS, bool EDGE>
hipError_t launch(int m1, int m2, int k, const int* block_rows, const int* residue_rows, const int* st_off,
                  const int* row_ptr, const int* col, const float* val, const T* lhs, const T* rhs, float* out,
                  PlanRef plan, hipStream_t s1, hipStream_t s2)
{
    constexpr int RPW = kWave / SddmmShape<T, KT>::kLpr;
    const int chunk_hint = chunk_for_segments(plan.seg_length, m1); // (segments per wave; 0: the kernels find out)
    const int g1 = chunk_hint > 0 ? grid_for_waves((m1 + chunk_hint - 1) / chunk_hint) : grid_for_waves(min(m1, kBlockGridWaves));
    const int g2 = grid_for_waves(((long long)m2 + RPW - 1) / RPW);
    if (g1 < 0 || g2 < 0) return hipErrorInvalidConfiguration;
    // With a host copy of the plan's header, a kernel that would find every chunk taken by
    // the other one is not launched at all.
    bool standard_residue = true, window_residue = plan.dev != nullptr;
    if (plan.dev && plan.host_counts) {
        standard_residue = plan.host_counts[1] < plan.host_counts[0];
        window_residue = plan.host_counts[1] > 0;
    }
    const bool hub_plan = plan.hub != nullptr && plan.hub_counts != nullptr && plan.hub_counts[3] != 0 && plan.hub_counts[0] > 0;
    // (the group kernel keeps four lhs slices in registers: rows of one slab only)
    const bool group_plan = NS == 1 && plan.groups != nullptr && plan.group_counts != nullptr && plan.group_counts[1] > 0;
    RowOwners owners;
    owners.hub_min_len = hub_plan ? plan.hub_counts[2] : 0;
    if (group_plan) {
        owners.groups = reinterpret_cast<const RowGroup*>(plan.groups + kGroupHeaderInts);
        owners.n_groups = plan.group_counts[0];
    }
    const bool hubs = hub_plan && (plan.only == 0 || plan.only == kSpmmOnlyHub);
    const bool grouped = group_plan && (plan.only == 0 || plan.only == kSpmmOnlyHub); // (timed with the hub kernels)
    if (plan.only != 0) { // one kernel family of the call (timing each on its own)
        if (plan.only != kSpmmOnlyBlock) m1 = 0;
        if (plan.only != kSpmmOnlyResidue) m2 = 0;
    }
    if (group_plan && plan.group_counts[2] == 0) m1 = m2 = 0; // every row in a group with a run: nothing for the lists' kernels
    if (m1 > 0 && m2 > 0 && standard_residue && s1 == s2 && g1 + g2 <= kPairMaxWorkgroups) {
        sddmm_pair_kernel<T, KT, NS, EDGE><<<g1 + g2, kWgThreads, 0, s1>>>(
            g1, m1, m2, k, chunk_hint, owners, block_rows, residue_rows, st_off, row_ptr, col, val, lhs, rhs, out, plan.dev);
    } else {
        if (m1 > 0) {
            sddmm_block_kernel<T, KT, NS, EDGE><<<g1, kWgThreads, 0, s1>>>(
                m1, k, chunk_hint, owners, block_rows, st_off, row_ptr, col, val, lhs, rhs, out);
        }
        if (m2 > 0 && standard_residue) {
            sddmm_residue_kernel<T, KT, NS, EDGE><<<g2, kWgThreads, 0, s2>>>(
                m2, k, owners, residue_rows, row_ptr, col, val, lhs, rhs, out, plan.dev);
        }
    }
    hipError_t e = hipGetLastError();
    if (e == hipSuccess && hubs) {
        const int merge = hub_merge(k);
        const int gh = grid_for_waves((long long)plan.hub_counts[0] * hub_groups(plan.hub_counts[1], merge));
        if (gh < 0) return hipErrorInvalidConfiguration;
        sddmm_hub_kernel<T, KT, NS, EDGE><<<gh, kWgThreads, 0, s1>>>(k, merge, plan.hub, col, val, lhs, rhs, out);
        e = hipGetLastError();
    }
    if constexpr (NS == 1) {
        if (e == hipSuccess && grouped) {
            // one wave per group when there are groups enough to fill the GPU that way, else a workgroup
            // (two waves per group, 8192 waves on config 5: 0.052 ms instead of 0.038)
            if (plan.group_counts[1] >= kGroupWaveEach) {
                const int wgs = (owners.n_groups + kWavesPerWg - 1) / kWavesPerWg;
                sddmm_group_kernel<T, KT, EDGE, 1><<<(wgs + kXcds - 1) / kXcds * kXcds, kWgThreads, 0, s1>>>(
                    k, owners.n_groups, owners.groups, row_ptr, col, val, lhs, rhs, out);
            } else {
                sddmm_group_kernel<T, KT, EDGE, kWavesPerWg><<<(owners.n_groups + kXcds - 1) / kXcds * kXcds, kWgThreads, 0, s1>>>(
                    k, owners.n_groups, owners.groups, row_ptr, col, val, lhs, rhs, out);
            }
            e = hipGetLastError();
        }
    }
    if (e == hipSuccess && m2 > 0 && window_residue)
        e = sddmm_window_launch<T>(m2, k, col, val, lhs, rhs, out, plan.dev, plan.rows, s2);
    return e;
}

template <typename T, int KT, int NS>
hipError_t launch_edge(bool edge, int m1, int m2, int k, const int* block_rows, const int* residue_rows,
                       const int* st_off, const int* row_ptr, const int* col, const float* val, const T* lhs,
                       const T* rhs, float* out, PlanRef plan, hipStream_t s1, hipStream_t s2)
{
    return edge ? launch<T, KT, NS, true>(m1, m2, k, block_rows, residue_rows, st_off, row_ptr, col, val, lhs, rhs, out,
                                          plan, s1, s2)
                : launch<T, KT, NS, false>(m1, m2, k, block_rows, residue_rows, st_off, row_ptr, col, val, lhs, rhs,
                                           out, plan, s1, s2);
}

} // namespace

// k: any positive multiple of the 128-bit vector width (4 for fp32, 8 for fp16) up to 512.
// 32, 64 and 128 (the reference has 32 and 128) run without any bounds test.  Chunks of the
// residue list for which `plan` holds a window go to the window kernel when a dense row
// is wider than one 128-byte tile (with a single tile the window is not reused often
// enough to repay its staging).
template <typename T>
hipError_t sddmm_launch(int m1, int m2, int k, const int* block_rows, const int* residue_rows, const int* st_off,
                        const int* row_ptr, const int* col, const float* val, const T* lhs, const T* rhs,
                        float* out, PlanRef plan, hipStream_t s1, hipStream_t s2)
{
    if (k <= 0 || k % DenseVec<T>::kElems != 0 || k > 512) return hipErrorInvalidValue;
    // the window kernels are for rows of more than one 128-byte tile
    if ((size_t)k * sizeof(T) <= 128) {
        plan.dev = nullptr;
        plan.rows = nullptr;
        plan.host_counts = nullptr;
    }
#define RODE_SDDMM_CASE(KT, NS)                                                                                   \
    return launch_edge<T, KT, NS>(k != (KT) * (NS), m1, m2, k, block_rows, residue_rows, st_off, row_ptr, col, val, \
                                  lhs, rhs, out, plan, s1, s2)
    if (k <= 32) RODE_SDDMM_CASE(32, 1);
    if (k <= 64) RODE_SDDMM_CASE(64, 1);
    if (k <= 128) RODE_SDDMM_CASE(128, 1);
    if (k <= 256) RODE_SDDMM_CASE(128, 2);
    if (k <= 384) RODE_SDDMM_CASE(128, 3);
    RODE_SDDMM_CASE(128, 4);
#undef RODE_SDDMM_CASE
}

template hipError_t sddmm_launch<float>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                        const float*, const float*, const float*, float*, PlanRef, hipStream_t, hipStream_t);
template hipError_t sddmm_launch<__half>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                         const float*, const __half*, const __half*, float*, PlanRef, hipStream_t, hipStream_t);

} // namespace rode
