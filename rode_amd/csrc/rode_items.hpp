// Work items of the RoDe kernels: which nonzero slots a block-segment wave and a
// residue lane group process.  One statement of the index arithmetic, shared by the
// standard kernels and the window kernels, so that both always agree on who owns
// what (reference arithmetic: RoDe_SpMM/RoDeSpmm.cu:71-82, 210-234;
// RoDe_SDDMM/RoDeSddmm.cu:33-58, 237-243).
#pragma once
#include "rode_device.hpp"

namespace rode {

// Rows that the kernels of a plan have taken out of the two lists (see the hub plan and the
// group plan below): the standard kernels ask before they touch a row.
constexpr int kGroupRows = 4; // rows of one group of the group plan
// A kept group: every row has a run of consecutive columns, and the runs cover [lo, lo + len)
// between them - row r's own run is [lo + head(r), lo + len - tail(r)), with head and tail
// below 256 (the runs of a sliding window start and end a column apart from row to row).
// The group kernels walk the part of the range that all four runs hold (shared_run).
struct RowGroup {
    int lo, len;          // the columns [lo, lo + len) that the runs of the group's rows cover; len 0: no group
    int pos[kGroupRows];  // where its own run starts in each row (slots from the row's first nonzero)
    unsigned heads;       // byte r: columns of the range before row r's run
    unsigned tails;       // byte r: columns of the range after row r's run
    __host__ __device__ int head(int r) const { return (int)((heads >> (8 * r)) & 255u); }
    __host__ __device__ int tail(int r) const { return (int)((tails >> (8 * r)) & 255u); }
    __host__ __device__ int run(int r) const { return len - head(r) - tail(r); } // length of row r's own run
};
static_assert(sizeof(RowGroup) == 32, "the group plan holds 32 bytes per group");
// What the group kernels walk for all four rows at once: the columns that every row's own
// run holds, [lo + largest head, lo + len - largest tail).  A row's columns of the range
// before and after that part are left to the pass over its other nonzeros, so no row ever
// meets a dense row that it does not reference (a non-finite one would turn a zero value
// into NaN).  The plan keeps a group only if this part has at least 64 columns.
__host__ __device__ inline RowGroup shared_run(RowGroup d)
{
    int head = 0, tail = 0;
    for (int r = 0; r < kGroupRows; ++r) {
        head = d.head(r) > head ? d.head(r) : head;
        tail = d.tail(r) > tail ? d.tail(r) : tail;
    }
    for (int r = 0; r < kGroupRows; ++r) d.pos[r] += head - d.head(r);
    d.lo += head;
    d.len -= head + tail;
    d.heads = d.tails = 0u;
    return d;
}
struct RowOwners {
    int hub_min_len = 0;              // > 0: rows of that aligned length or more belong to the hub kernels
    const RowGroup* groups = nullptr; // the groups of a group plan, or null
    int n_groups = 0;
    bool overwrite = false;           // SpMM: a row with a single work item is stored, not added to C
};
__device__ __forceinline__ bool owned_elsewhere(const RowOwners& o, int row, int aligned_len)
{
    if (o.hub_min_len > 0 && aligned_len >= o.hub_min_len) return true;
    return o.groups != nullptr && row / kGroupRows < o.n_groups && o.groups[row / kGroupRows].len > 0;
}

// Several problems on one pattern in one launch (the heads of an attention layer): blockIdx.y
// picks the problem, whose operands start this many elements after those of problem 0.
struct HeadStrides {
    size_t rows = 0; // of an operand with a row of d elements per row of the pattern
    size_t cols = 0; // of an operand with a row of d elements per column of the pattern
    size_t nnz = 0;  // of an operand with an element per nonzero
};
template <typename P>
__device__ __forceinline__ P* of_head(P* first, size_t stride)
{
    return first ? first + (size_t)blockIdx.y * stride : first;
}

// Aligned slot range [base, base + cnt) of one block work item; the first `mask` slots
// belong to the previous row (unaligned start) and must not contribute.
struct BlockItem {
    int row, base, mask, cnt;
    bool whole = false; // the work item is its row's only one (SpMM: a row summed whole)
};

// Consecutive segments of one row whose starts fall into the same window of MERGE slots
// are handled by the wave of the first of them (the "leader"); with segments of MERGE
// slots or more every segment is its own leader.  Returns false for a follower.  All
// 64 lanes of the wave must call this together (they probe the next 64 segments, so a
// window may hold at most 64 followers: MERGE <= 64 x 32).  st_off[m1] must exist: the
// sentinel, or the next segment when the lists are a slice.
__device__ __forceinline__ bool merged_leader(int MERGE, int seg, int m1, int lane, int row, int row_start, int row_end,
                                              const int* __restrict__ block_rows, const int* __restrict__ st_off,
                                              BlockItem& it)
{
    const int start = st_off[seg];
    const int row_base = row_start - (row_start & (kVecLen - 1));
    const int window = (start - row_base) / MERGE;
    if (seg > 0 && block_rows[seg - 1] == row && (st_off[seg - 1] - row_base) / MERGE == window) return false;
    // the next leader: the first later segment of another row or another window
    const int probe = seg + 1 + lane;
    const bool follower = probe < m1 && block_rows[probe] == row && (st_off[probe] - row_base) / MERGE == window;
    const unsigned long long not_follower = ~__ballot(follower);
    const int next = seg + 1 + (not_follower ? __builtin_ctzll(not_follower) : kWave);
    // end of the row's block part, or the start of the next leader if that comes first
    // (another row's start, or the sentinel, lies past block_end)
    const int block_end = row_base + (row_end - row_base) / kBlockItems * kBlockItems;
    const int end = min(block_end, st_off[next]);
    it.row = row;
    it.mask = start & (kVecLen - 1);
    it.base = start - it.mask;
    it.cnt = end - it.base;
    it.whole = false;
    return true;
}

constexpr int kSddmmMergeSlots = 128;
constexpr int kSpmmMergeSlots = 512;

// SDDMM: merging needs no promise from the caller (an output computed twice at a slice
// boundary is harmless).
__device__ __forceinline__ bool sddmm_block_item(int seg, int m1, const RowOwners& owners, int lane,
                                                 const int* __restrict__ block_rows, const int* __restrict__ st_off,
                                                 const int* __restrict__ row_ptr, BlockItem& it)
{
    const int row = block_rows[seg];
    const int row_start = row_ptr[row], row_end = row_ptr[row + 1];
    if (owned_elsewhere(owners, row, row_end - row_start + (row_start & (kVecLen - 1)))) return false;
    return merged_leader(kSddmmMergeSlots, seg, m1, lane, row, row_start, row_end, block_rows, st_off, it);
}

// SpMM.  owned_slots > 0 means that the caller promised complete lists: a row of at
// most owned_slots aligned slots is then summed whole - all its segments and its tail -
// by the wave of its first segment (one update of C), longer rows are merged into
// leaders.  owned_slots < 0: no promise, but segments are merged into leaders all the
// same - a leader only ever takes segments of the list it was given (a slice of the lists
// merges within the slice), so every slot still contributes exactly once.
// owned_slots == 0: every segment on its own, rounded to whole 32-slot units as in
// RoDeSpmm.cu:210-234 (small launches: they need the waves more than they mind the
// atomics).
__device__ __forceinline__ bool spmm_block_item(int seg, int m1, int owned_slots, const RowOwners& owners, int lane,
                                                const int* __restrict__ block_rows, const int* __restrict__ st_off,
                                                const int* __restrict__ row_ptr, BlockItem& it)
{
    const int row = block_rows[seg];
    const int row_start = row_ptr[row], row_end = row_ptr[row + 1];
    if (owned_elsewhere(owners, row, row_end - row_start + (row_start & (kVecLen - 1)))) return false;
    if (row_end - row_start + (row_start & (kVecLen - 1)) <= owned_slots) {
        if (seg > 0 && block_rows[seg - 1] == row) return false;
        it.row = row;
        it.mask = row_start & (kVecLen - 1);
        it.base = row_start - it.mask;
        it.cnt = row_end - it.base;
        it.whole = true;
        return true;
    }
    if (owned_slots != 0)
        return merged_leader(kSpmmMergeSlots, seg, m1, lane, row, row_start, row_end, block_rows, st_off, it);
    const int start = st_off[seg];
    const int end = min(row_end, st_off[seg + 1]);
    it.row = row;
    it.mask = start & (kVecLen - 1);
    it.base = start - it.mask;
    it.cnt = (end - start + it.mask) / kBlockItems * kBlockItems;
    it.whole = false;
    return true;
}

// ---- lists with short segments ----------------------------------------------------------
// A decomposition with short segments (the reference's K = 128 parameter set has 32 slots)
// arrives as several hundred thousand segments of which most are followers.  One wave per
// segment then means mostly waves that load four indices to find out that they have
// nothing to do.  Instead a wave takes a chunk of consecutive segments - as many as make
// kWalkSlots slots at the decomposition's segment length - and walks it from leader to
// leader; the workgroups past the last chunk leave after a few scalar loads.  The segment length is read off the lists (the launch arguments do not
// carry it): two consecutive segments of one row start exactly one segment length apart,
// the row's first one up to three slots less.  Three evenly spaced pairs are looked at; if
// none lies within a row (rows of one segment each), or the segments are long, the chunk is
// one segment and nothing changes.  All waves of a launch compute the same answer.
constexpr int kWalkSlots = 512;
constexpr int kWalkMaxChunk = 16;
constexpr int kWalkMinSegments = 16384; // fewer segments: a small launch needs its waves more than it minds the followers
constexpr int kWalkMinWaves = 8192;     // a chunk is no longer than leaves this many waves (eight per SIMD)
// (a chunk of c segments needs at least c * kWalkMinWaves segments in the list)
__host__ __device__ inline int walk_chunk_limit(int m1) { return m1 / kWalkMinWaves > 1 ? m1 / kWalkMinWaves : 1; }

__device__ __forceinline__ int block_chunk(int m1, const int* __restrict__ block_rows, const int* __restrict__ st_off)
{
    // (every load is issued before any is used: one round trip of scalar loads for the waves
    // that only find out that they have no chunk)
    constexpr int kPairs = 3;
    int row[kPairs][2], start[kPairs][2];
#pragma unroll
    for (int i = 0; i < kPairs; ++i) {
        const int p = (int)((long long)m1 * (i + 1) / (kPairs + 1)); // (the same in every lane; m1 >= kWalkMinSegments, so p + 1 < m1)
        row[i][0] = block_rows[p];
        row[i][1] = block_rows[p + 1];
        start[i][0] = st_off[p];
        start[i][1] = st_off[p + 1];
    }
    int seg_len = 0;
#pragma unroll
    for (int i = 0; i < kPairs; ++i)
        if (row[i][0] == row[i][1]) seg_len = max(seg_len, start[i][1] - start[i][0]);
    if (seg_len <= 0) return 1;
    seg_len = (seg_len + kBlockItems - 1) / kBlockItems * kBlockItems;
    return min(min(max(kWalkSlots / seg_len, 1), kWalkMaxChunk), walk_chunk_limit(m1));
}

// The block part of a grid has at most kBlockGridWaves waves: a launch is sized before anybody
// knows how long the segments are, and workgroups that find nothing to do still cost their
// launch (a few hundred thousand of them cost more than the work of an attention mask).  A
// longer list is walked in chunks as well, of as many segments as it takes to cover it.
constexpr int kBlockGridWaves = 65536;
constexpr int kScanSegments = 32; // segments of a chunk looked at together (scan_chunk: a leader's followers end inside the 64 lanes)

// Segments per wave for a list of m1 segments on `nblocks` workgroups; 1: one wave per
// segment, in the order of xcd_logical_block.
__device__ __forceinline__ int block_chunk_for_grid(int estimate, int m1, int nblocks)
{
    const int waves = nblocks * kWavesPerWg;
    return max(estimate, (m1 + waves - 1) / waves);
}

// A caller that says how long the segments of its decomposition are (the plans struct of the
// planned entry points) spares the kernels the guess and the launch its spare workgroups:
// the grid then has exactly one wave per chunk.  0: not said.
__host__ __device__ inline int chunk_for_segments(int seg_length, int m1)
{
    if (seg_length <= 0) return 0;
    if (m1 < kWalkMinSegments) return 1;
    int c = kWalkSlots / ((seg_length + kBlockItems - 1) / kBlockItems * kBlockItems);
    c = c < 1 ? 1 : (c > kWalkMaxChunk ? kWalkMaxChunk : c);
    const int limit = walk_chunk_limit(m1);
    return c < limit ? c : limit;
}

// First segment of this wave's chunk, or -1 when it has none.  Consecutive chunks share an
// XCD: the workgroups with chunks are the first ceil(chunks / 4 / kXcds) of every XCD.
__device__ __forceinline__ long long chunk_first_segment(int bid, int wave, int m1, int chunk)
{
    const int chunks = (m1 + chunk - 1) / chunk;
    const int per_xcd = ((chunks + kWavesPerWg - 1) / kWavesPerWg + kXcds - 1) / kXcds;
    if (bid / kXcds >= per_xcd) return -1;
    const long long first = ((long long)((bid % kXcds) * per_xcd + bid / kXcds) * kWavesPerWg + wave) * chunk;
    return first < m1 ? first : -1;
}

// The 64 segments from `first` on, one per lane, looked at together: which of them start
// something - a work item (a leader), or a stretch that a plan has given to other kernels -
// and which follow the segment before them.  A row of at most owned_slots slots is one work
// item (SpMM under the whole-lists promise), else the segments of one window of MERGE slots
// are (merged_leader's rule).  Two rounds of loads for the whole chunk instead of three per
// segment.  All 64 lanes call this together.
struct ChunkScan {
    int row, row_start, row_end, start; // this lane's segment (start: st_off, also for the entry after the last segment)
    bool whole;                         // its row is one work item
    unsigned long long heads;           // bit i: segment first + i follows nothing (bits past the list are set)
    unsigned long long items;           // bit i: segment first + i starts a work item
};

__device__ __forceinline__ ChunkScan scan_chunk(int MERGE, int first, int m1, int owned_slots, const RowOwners& owners, int lane,
                                                const int* __restrict__ block_rows, const int* __restrict__ st_off,
                                                const int* __restrict__ row_ptr)
{
    ChunkScan c;
    const int s = first + lane;
    const bool valid = s < m1;
    c.row = valid ? block_rows[s] : -1;
    const int prev_row = valid && s > 0 ? block_rows[s - 1] : -1;
    c.start = s <= m1 ? st_off[s] : 0;
    const int prev_start = valid && s > 0 ? st_off[s - 1] : 0;
    c.row_start = valid ? row_ptr[c.row] : 0;
    c.row_end = valid ? row_ptr[c.row + 1] : 0;
    const int row_base = c.row_start - (c.row_start & (kVecLen - 1));
    const int aligned = c.row_end - row_base;
    const bool elsewhere = valid && owned_elsewhere(owners, c.row, aligned);
    c.whole = valid && !elsewhere && owned_slots > 0 && aligned <= owned_slots;
    const bool by_row = elsewhere || c.whole; // every segment of the row follows its first one
    const bool follower = valid && prev_row == c.row &&
                          (by_row || (prev_start - row_base) / MERGE == (c.start - row_base) / MERGE);
    c.heads = __ballot(!follower);
    c.items = __ballot(valid && !follower && !elsewhere);
    return c;
}

// Work item of the leader in lane `i` (the same i in all lanes) of a scanned chunk.  A leader
// among the first kScanSegments lanes has its last follower at most 31 segments further on
// (a window of 512 slots, or a row of at most 1024, in segments of 32 or more), so the
// segment after them is inside the scan as well.
__device__ __forceinline__ BlockItem chunk_item(const ChunkScan& c, int i)
{
    const unsigned long long later = c.heads & ~((2ull << i) - 1ull);
    const int next = later ? __builtin_ctzll(later) : -1;
    const int row_start = __builtin_amdgcn_readlane(c.row_start, i), row_end = __builtin_amdgcn_readlane(c.row_end, i);
    const int start = __builtin_amdgcn_readlane(c.start, i);
    const int next_start = next >= 0 ? __builtin_amdgcn_readlane(c.start, next) : 0x7fffffff;
    const int row_base = row_start - (row_start & (kVecLen - 1));
    BlockItem it;
    it.row = __builtin_amdgcn_readlane(c.row, i);
    if (__builtin_amdgcn_readlane((int)c.whole, i)) {
        it.mask = row_start & (kVecLen - 1);
        it.base = row_base;
        it.cnt = row_end - row_base;
        it.whole = true;
        return it;
    }
    // end of the row's block part, or the start of the next leader if that comes first
    const int block_end = row_base + (row_end - row_base) / kBlockItems * kBlockItems;
    it.mask = start & (kVecLen - 1);
    it.base = start - it.mask;
    it.cnt = min(block_end, next_start) - it.base;
    return it;
}

// The row of segment `seg` if spmm_block_item() gives it a work item, else -1 (a follower,
// or past the list).  The same rules, without the extent of the item: what the waves of a
// workgroup need to know about each other.
__device__ __forceinline__ int spmm_block_leader_row(int seg, int m1, int owned_slots, const RowOwners& owners,
                                                     const int* __restrict__ block_rows, const int* __restrict__ st_off,
                                                     const int* __restrict__ row_ptr)
{
    if (seg >= m1) return -1;
    const int row = block_rows[seg];
    const bool asks = owners.hub_min_len > 0 || owners.groups != nullptr;
    if (!asks && (seg == 0 || block_rows[seg - 1] != row || owned_slots == 0)) return row;
    const int row_start = row_ptr[row];
    const int row_base = row_start - (row_start & (kVecLen - 1));
    if (asks && owned_elsewhere(owners, row, row_ptr[row + 1] - row_base)) return -1; // another kernel's
    if (seg == 0 || block_rows[seg - 1] != row || owned_slots == 0) return row;
    if (row_ptr[row + 1] - row_base <= owned_slots) return -1; // summed whole by the wave of its first segment
    return (st_off[seg] - row_base) / kSpmmMergeSlots == (st_off[seg - 1] - row_base) / kSpmmMergeSlots ? -1 : row;
}

// Slots [first, first + cnt) of one residue row: with N = len + (start & 3), rows with
// N >= 32 keep only their last N % 32 slots, starting at (start & ~3) + floor(N / 32) * 32,
// and are accumulated into (the row also has block segments); shorter rows are taken
// whole and stored.
struct ResidueItem {
    int first, cnt, aligned; // aligned = N
    bool accumulate;
};

__device__ __forceinline__ ResidueItem residue_item(int row, const int* __restrict__ row_ptr)
{
    const int s = row_ptr[row], e = row_ptr[row + 1];
    const int pad = s & (kVecLen - 1);
    ResidueItem it;
    it.aligned = e - s + pad;
    it.accumulate = it.aligned >= kBlockItems;
    it.first = it.accumulate ? (s - pad) + it.aligned / kBlockItems * kBlockItems : s;
    it.cnt = it.accumulate ? it.aligned % kBlockItems : e - s;
    return it;
}

// ---- locality plan --------------------------------------------------------------
// A plan cuts the residue list into chunks of consecutive entries and says, for every
// chunk, whether the dense rows its nonzeros reference cluster in a window of at most
// kResidueWindowRowsMax consecutive rows (banded matrices).  A chunk with a window is
// processed by the window kernels (the window of the dense operand is staged in LDS once
// per column tile and every slot that falls into it reads LDS instead of gathering from
// L2); the standard residue kernels skip it.  Slots outside the window are still gathered
// from memory, so a plan never changes which nonzeros contribute - only where their dense
// rows are read from.  The plan has two device arrays:
//   descriptors, int[]:  [0] residue chunks  [1] residue chunks with a window  [2], [3] zero,
//                        then one WindowDesc per residue chunk;
//   rows, one PlannedChunk per chunk (filled for the chunks with a window): what the
//                        window kernels would otherwise work out per call for every
//                        residue row - its slots as positions in the window.
constexpr int kPlanHeaderInts = 4;
constexpr int kPlanDescInts = 4;
constexpr int kPlanResidueChunk = 128;     // residue-list entries per chunk
constexpr int kResidueWindowRowsMax = 512; // dense rows of one window (9 bits of a slot's 16-bit entry)

// Window of one chunk: dense rows [w0, w0 + wn); wn == 0: no window.  slots / misses: how
// many nonzero slots the chunk has / how many of them fall outside the window.
struct WindowDesc {
    int w0, wn, slots, misses;
};

// One residue row of a chunk with a window.  Its cnt slots are listed in an order chosen
// for the LDS banks (see below), entry i = (window row of the slot's column) | (slot << 9),
// slot counted from the row's first residue slot `first`; a slot whose column is outside
// the window (bit i of missmask) carries the window row of one that is inside; entries
// cnt..31 repeat such a window row and have no slot (their value is 0).
// Order: a ds_read_b128 of a wave serves lane groups (0, 3), (1, 2), (4, 7), (5, 6) in
// the same cycles, and two 128-byte window rows of equal parity collide in the banks.
// Rows that lane groups 0, 1, 4, 5 will take list their even window rows first, the rows
// of groups 2, 3, 6, 7 their odd ones: two groups that meet mostly read different parities.
struct PlannedRowMeta {
    int row;       // the residue row (-1: no such entry)
    int first;     // its first residue slot (index into column_indices / values)
    int packed;    // cnt | accumulate << 8 | min(aligned length, 0xffff) << 16
    unsigned missmask;
};
struct PlannedChunk {
    int w0, wn, reserved[2]; // the chunk's window again: the kernels need nothing else to start
    PlannedRowMeta meta[kPlanResidueChunk];
    unsigned short entry[kPlanResidueChunk][kBlockItems];
};
static_assert(sizeof(PlannedChunk) == 16 + kPlanResidueChunk * (16 + 2 * kBlockItems), "packed layout");

__host__ __device__ inline int plan_residue_chunks(int m2) { return (m2 + kPlanResidueChunk - 1) / kPlanResidueChunk; }
__host__ __device__ inline size_t plan_ints(int m2)
{
    return kPlanHeaderInts + (size_t)kPlanDescInts * plan_residue_chunks(m2);
}

__device__ __forceinline__ WindowDesc plan_residue_desc(const int* __restrict__ plan, int chunk)
{
    const int4 v = *reinterpret_cast<const int4*>(plan + kPlanHeaderInts + kPlanDescInts * chunk);
    return WindowDesc{v.x, v.y, v.z, v.w};
}

// ---- group plan -----------------------------------------------------------------
// Groups of kGroupRows adjacent rows that share a long run of consecutive columns (see
// rode_group.hip).  Layout, ints: header [0] groups (= rows / kGroupRows, whole groups
// only)  [1] groups with a run  [2] rows outside those groups  [3] zero; then one RowGroup per group; then three
// ints per row of scratch for the plan's own kernels.
constexpr int kGroupHeaderInts = 4;
// SpMM / SDDMM: from this many groups with a run on, a group is one wave's work, below it a
// workgroup's (measured on the attention-mask benchmark cut down to 128 .. 4096 groups: a wave
// per group is 20-30 % faster from 256 groups on and level at 128).
constexpr int kGroupWaveEach = 128;
// Attention kernels: from this many groups with a run on, the rows of groups go to the group
// kernels; below it every row gets a wave of its own.  Measured on the same benchmark cut
// down, forward + both gradient kernels, group kernels against a wave per row: 2048 groups
// 0.174 against 0.278 ms (fp16 operands 0.166 / 0.211); 1024 groups 0.133 / 0.148 (fp16: 0.128 /
// 0.110, the column pass alone 0.030 / 0.044); 512 groups 0.120 / 0.083.  Hence by operand
// size for the passes over the pattern, and one figure for the pass over its transpose.
template <typename T>
constexpr int attention_groups_min()
{
    return sizeof(T) == 2 ? 2048 : 1024;
}
constexpr int kAttentionColsGroupsMin = 1024;
static_assert(sizeof(RowGroup) == 32 && kGroupRows == kWavesPerWg, "one wave per row of a group");
__host__ __device__ inline int row_groups(int M) { return M / kGroupRows; }
__host__ __device__ inline size_t group_plan_ints(int M)
{
    return kGroupHeaderInts + (size_t)row_groups(M) * (sizeof(RowGroup) / sizeof(int)) + 3 * (size_t)M;
}

// ---- hub plan -------------------------------------------------------------------
// Rows with very many nonzeros (hubs of a power-law graph) reference dense rows all over
// the operand, and so does every other hub: the same dense rows, at other times, long
// evicted from L2.  A hub plan cuts every hub row into pieces by column slab (a slab is
// kHubSlabRows consecutive dense rows) and the hub kernels take the pieces slab by slab,
// a few neighbouring slabs at a time (hub_merge: about 4 MB of the dense operand, the size
// of an XCD's L2 - measured best on the power-law benchmark against half, twice and four
// times that; smaller pieces cost more than they save): all hub rows' nonzeros of those
// slabs at the same time on one XCD, so that a dense row is fetched from memory once and
// then found in L2 by the other hubs.
// Needs rows whose column indices ascend (the plan checks).  The standard kernels skip
// the rows of a usable plan (by their length), so every nonzero is still processed once.
// Layout, ints: header [0] hub rows  [1] slabs  [2] shortest hub row (aligned length)
// [3] usable (every hub row's columns ascend)  [4] room for hub rows  [5..7] zero;
// then the hub rows, ascending (room for [4] of them); then per hub row slabs + 1 piece
// starts (indices into column_indices / values; the last one is the row's end).
constexpr int kHubSlabRows = 2048;
constexpr int kHubHeaderInts = 8;

__host__ __device__ inline int hub_slabs(int dense_rows) { return (dense_rows + kHubSlabRows - 1) / kHubSlabRows; }
// (a hub row has at least min_len aligned slots, up to three of which belong to the row before it)
__host__ __device__ inline int hub_room(int nnz, int min_len) { return min_len > kVecLen ? nnz / (min_len - (kVecLen - 1)) + 1 : 0; }
// (after the piece table: one int per 2048 rows of the matrix, scratch of the selection)
constexpr int kHubSelectBlockRows = 2048;
__host__ __device__ inline size_t hub_table_ints(int dense_rows, int nnz, int min_len)
{
    const size_t room = hub_room(nnz, min_len);
    return kHubHeaderInts + room + room * (hub_slabs(dense_rows) + 1);
}
__host__ __device__ inline size_t hub_plan_ints(int M, int dense_rows, int nnz, int min_len)
{
    return hub_table_ints(dense_rows, nnz, min_len) + (M + kHubSelectBlockRows - 1) / kHubSelectBlockRows + 1;
}

// Slabs taken together by one work item of the hub kernels, for dense rows of `width`
// 4-byte elements (16-bit operands count as 4 bytes too: the pieces matter more than the bytes).
__host__ __device__ inline int hub_merge(int width)
{
    const int g = (4 << 20) / kHubSlabRows / (width > 0 ? width * 4 : 4);
    return g < 1 ? 1 : (g > 64 ? 64 : g);
}
__host__ __device__ inline int hub_groups(int slabs, int merge) { return (slabs + merge - 1) / merge; }

struct HubPlan {
    int n_hub, slabs, min_len;
    const int* rows;   // [n_hub]
    const int* pieces; // [n_hub][slabs + 1]
};
__device__ __forceinline__ HubPlan hub_plan_view(const int* __restrict__ plan)
{
    HubPlan v;
    v.n_hub = plan[0];
    v.slabs = plan[1];
    v.min_len = plan[2];
    v.rows = plan + kHubHeaderInts;
    v.pieces = plan + kHubHeaderInts + plan[4];
    return v;
}

} // namespace rode
