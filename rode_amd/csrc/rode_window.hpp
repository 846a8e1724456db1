// Pieces shared by the window kernels of SpMM and SDDMM (rode_spmm_window.hip,
// rode_sddmm_window.hip): the kernels for chunks of the residue list whose dense rows
// cluster in a window of consecutive rows (see the locality plan in rode_items.hpp).
//
// Shape of both kernels.  A workgroup of 512 threads takes 64 consecutive residue rows
// (half a chunk of the plan), one group of 8 lanes per row, and walks the dense operand in
// column tiles of 128 bytes (32 fp32 / 64 fp16 columns).  Per tile it copies the rows
// [w0, w0 + wn) of the operand - the chunk's window - into LDS with coalesced 128-bit
// loads, once (the loads of the next tile are issued before the current tile is worked
// on), and every nonzero slot whose column falls into the window reads its dense row from
// LDS (8 lanes x ds_read_b128, one contiguous 128-byte row per lane group) instead of
// gathering it from L2; a slot outside the window is gathered from memory as before.
// LDS (77 KB) and registers (128) are sized so that two workgroups share a CU: while one
// waits for memory the other computes.  The lanes of a group keep the LDS address of every
// slot's dense row in registers for all tiles, so a slot costs one ds_read_b128 plus its
// multiply-adds.  Which window row a slot reads is not worked out here: the plan holds it
// for every residue row of a chunk with a window (PlannedChunk), in an order that keeps
// lane groups that meet in the LDS banks on rows of different parity.
#pragma once
#include "rode_items.hpp"

#ifdef RODE_PHASE_TIMING
// Debug builds only: cycles spent per phase, summed over workgroups.
static __device__ unsigned long long rode_phase_clk[8];
#ifdef RODE_PHASE_READER
extern "C" void rode_phase_read(unsigned long long* out, int reset)
{
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(rode_phase_clk), sizeof(unsigned long long) * 8);
    if (reset) {
        unsigned long long z[8] = {0};
        (void)hipMemcpyToSymbol(HIP_SYMBOL(rode_phase_clk), z, sizeof(z));
    }
}
#endif
#define RODE_PHASE(i)                                                                    \
    do {                                                                                 \
        const unsigned now_ = (unsigned)__builtin_readcyclecounter();                    \
        phase_acc_[i] += now_ - phase_t_;                                                \
        phase_t_ = now_;                                                                 \
    } while (0)
#define RODE_PHASE_BEGIN                                                                 \
    unsigned phase_acc_[5] = {0, 0, 0, 0, 0};                                            \
    unsigned phase_t_ = (unsigned)__builtin_readcyclecounter()
#define RODE_PHASE_END                                                                   \
    do {                                                                                 \
        if (threadIdx.x == 0)                                                            \
            for (int i_ = 0; i_ < 5; ++i_) atomicAdd(&rode_phase_clk[i_], (unsigned long long)phase_acc_[i_]); \
    } while (0)
#else
#define RODE_PHASE(i)
#define RODE_PHASE_BEGIN
#define RODE_PHASE_END
#endif

namespace rode {

constexpr int kResThreads = 512;
constexpr int kResLanes = 8;                              // lanes per residue row: 8 x 16 bytes = one 128-byte tile row
constexpr int kResRows = kResThreads / kResLanes;         // residue rows per workgroup
constexpr int kResParts = kPlanResidueChunk / kResRows;   // workgroups per chunk of the plan
constexpr int kResWinVecs = kResidueWindowRowsMax * kResLanes;                 // 16-byte pieces of a window
constexpr int kResPrefetch = (kResWinVecs + kResThreads - 1) / kResThreads;    // pieces one thread moves per tile
// A group's 32 values in LDS are 36 floats apart: the eight groups of a wave read their
// float4 of the same quad from eight different sets of banks (32 apart, four groups would
// share each set).
constexpr int kResValStride = kBlockItems + 4;
static_assert(kPlanResidueChunk % kResRows == 0, "a workgroup takes a whole fraction of a chunk");
static_assert(kResWinVecs * 16 <= 65536, "an LDS address of the window fits 16 bits");
static_assert(kResidueWindowRowsMax == 512 && kBlockItems == 32, "a plan entry holds 9 bits of window row and 5 of slot");

inline int grid_for_residue_parts(int m2)
{
    const int parts = plan_residue_chunks(m2) * kResParts;
    return (parts + kXcds - 1) / kXcds * kXcds; // xcd_logical_block needs a multiple of kXcds
}

// Issues this thread's loads of one column tile of the window rows [0, wn): src_lane
// points at this lane's 16 bytes of the first row, rows are row_bytes apart.  Lanes with
// !ok (past the last column of an edge tile) get zeros.
__device__ __forceinline__ void res_prefetch(uint4 (&pf)[kResPrefetch], const char* src_lane, size_t row_bytes, int wn,
                                             bool ok)
{
    constexpr int RS = kResThreads / kResLanes;
    const int r0 = threadIdx.x / kResLanes;
#pragma unroll
    for (int u = 0; u < kResPrefetch; ++u) {
        pf[u] = make_uint4(0, 0, 0, 0);
        if (ok && r0 + u * RS < wn) pf[u] = *reinterpret_cast<const uint4*>(src_lane + (size_t)(r0 + u * RS) * row_bytes);
    }
}

__device__ __forceinline__ void res_commit(uint4* win, const uint4 (&pf)[kResPrefetch], int wn)
{
    constexpr int RS = kResThreads / kResLanes;
    const int r0 = threadIdx.x / kResLanes, ls = threadIdx.x % kResLanes;
#pragma unroll
    for (int u = 0; u < kResPrefetch; ++u)
        if (r0 + u * RS < wn) win[(r0 + u * RS) * kResLanes + ls] = pf[u];
}

// Copies one column tile of the window rows [0, wn) from memory into LDS without keeping
// it in registers meanwhile (for a kernel that has none to spare).
__device__ __forceinline__ void res_fill(uint4* win, const char* src_lane, size_t row_bytes, int wn, bool ok)
{
    constexpr int RS = kResThreads / kResLanes, U = 4;
    const int r0 = threadIdx.x / kResLanes, ls = threadIdx.x % kResLanes;
    for (int r = r0; r < wn; r += U * RS) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v[u] = make_uint4(0, 0, 0, 0);
            if (ok && r + u * RS < wn) v[u] = *reinterpret_cast<const uint4*>(src_lane + (size_t)(r + u * RS) * row_bytes);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (r + u * RS < wn) win[(r + u * RS) * kResLanes + ls] = v[u];
    }
}

// One residue row as its lane group keeps it: cnt slots at positions 0 .. cnt - 1 (the order
// of the plan), the rest of the 32 positions carry value 0.
// addr[i]: LDS byte address of this lane's 16 bytes of the dense row of position i; for a
// position whose dense row is outside the window (bit i of missmask) it is the address of
// one of the row's positions that is inside, and the data has to come from memory instead.
// PACKED: two addresses (each below 64 K) per register, position 2 i in the low half of
// addr[i] and 2 i + 1 in the high half - for a kernel that needs the 16 registers elsewhere
// and pays one extra instruction per read for it.
template <bool PACKED>
struct ResidueRow {
    int row;   // -1: nothing to do
    int first; // first residue slot of the row in column_indices / values
    int cnt, quads;
    unsigned missmask;
    bool accumulate; // the row also has block segments (SpMM adds instead of storing)
    unsigned addr[PACKED ? kBlockItems / 2 : kBlockItems];
};

// The slot (counted from rr.first) that the plan put at position i of row `local` of a chunk.
__device__ __forceinline__ int planned_slot(const PlannedChunk& pc, int local, int i)
{
    return (pc.entry[local][i] >> 9) & (kBlockItems - 1);
}

// Turns a row record of the plan and the row's 32 entries into the lane group's view of
// the row (everything but the values).  skip_owned_slots: rows with block segments and at
// most that many aligned slots are left to the block kernel (SpMM under the whole-lists
// promise); 0 for SDDMM.  usable = false: the chunk has no window (its records are not
// filled in), the row is skipped.
template <bool PACKED>
__device__ __forceinline__ void decode_planned_row(const int4& meta, const uint4 (&e4)[kBlockItems / 8], bool usable,
                                                   int skip_owned_slots, ResidueRow<PACKED>& rr)
{
    const int ls = threadIdx.x % kResLanes;
    rr.row = meta.x;
    rr.first = meta.y;
    rr.cnt = meta.z & 0xff;
    rr.accumulate = (meta.z >> 8) & 1;
    rr.missmask = (unsigned)meta.w;
    if (!usable || rr.row < 0 || (rr.accumulate && ((meta.z >> 16) & 0xffff) <= skip_owned_slots)) {
        rr.row = -1;
        rr.first = 0;
        rr.cnt = 0;
        rr.missmask = 0;
    }
    rr.quads = (rr.cnt + 3) / 4;
#pragma unroll
    for (int i = 0; i < kBlockItems / 8; ++i) {
        const unsigned w[4] = {e4[i].x, e4[i].y, e4[i].z, e4[i].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned even = (((w[j] & 0xffffu) & (kResidueWindowRowsMax - 1)) * kResLanes + ls) * 16;
            const unsigned odd = (((w[j] >> 16) & (kResidueWindowRowsMax - 1)) * kResLanes + ls) * 16;
            if (PACKED) {
                rr.addr[4 * i + j] = even | (odd << 16);
            } else {
                rr.addr[8 * i + 2 * j] = even;
                rr.addr[8 * i + 2 * j + 1] = odd;
            }
        }
    }
}

// Loads row `local` of a planned chunk for this lane group: the LDS addresses of its 32
// positions into registers, its values (in position order, 0 past the row) into `my_val`
// (32 floats of this group; the 8 lanes write 4 each).
template <bool PACKED>
__device__ __forceinline__ void load_planned_row(const PlannedChunk& pc, int local, int skip_owned_slots,
                                                 const float* __restrict__ val, float* my_val, ResidueRow<PACKED>& rr)
{
    const int ls = threadIdx.x % kResLanes;
    const int4 meta = *reinterpret_cast<const int4*>(&pc.meta[local]);
    const uint4* entries = reinterpret_cast<const uint4*>(pc.entry[local]);
    uint4 e4[kBlockItems / 8];
#pragma unroll
    for (int i = 0; i < kBlockItems / 8; ++i) e4[i] = entries[i];
    decode_planned_row(meta, e4, true, skip_owned_slots, rr);
    constexpr int OWN = kBlockItems / kResLanes;
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        const int pos = ls + i * kResLanes;
        my_val[pos] = pos < rr.cnt ? val[rr.first + planned_slot(pc, local, pos)] : 0.f;
    }
}

// Longest row (in slot quads) among the 8 lane groups of the wave, as a scalar: quads at
// or past it are skipped by the whole wave.
__device__ __forceinline__ int wave_max_quads(int quads)
{
#pragma unroll
    for (int m = kResLanes; m < kWave; m <<= 1) quads = max(quads, __shfl_xor(quads, m, kWave));
    return __builtin_amdgcn_readfirstlane(quads);
}

} // namespace rode
