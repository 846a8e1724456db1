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
// multiply-adds.
#pragma once
#include "rode_items.hpp"

#ifdef RODE_PHASE_TIMING
// Debug builds only: cycles spent per phase, summed over workgroups.
__device__ unsigned long long rode_phase_clk[8];
extern "C" void rode_phase_read(unsigned long long* out, int reset)
{
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(rode_phase_clk), sizeof(unsigned long long) * 8);
    if (reset) {
        unsigned long long z[8] = {0};
        (void)hipMemcpyToSymbol(HIP_SYMBOL(rode_phase_clk), z, sizeof(z));
    }
}
#define RODE_PHASE(i)                                                                    \
    do {                                                                                 \
        const unsigned long long now_ = __builtin_readcyclecounter();                    \
        phase_acc_[i] += now_ - phase_t_;                                                \
        phase_t_ = now_;                                                                 \
    } while (0)
#define RODE_PHASE_BEGIN                                                                 \
    unsigned long long phase_acc_[8] = {0, 0, 0, 0, 0, 0, 0, 0};                         \
    unsigned long long phase_t_ = __builtin_readcyclecounter()
#define RODE_PHASE_END                                                                   \
    do {                                                                                 \
        if (threadIdx.x == 0)                                                            \
            for (int i_ = 0; i_ < 8; ++i_) atomicAdd(&rode_phase_clk[i_], phase_acc_[i_]); \
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
constexpr unsigned kMiss = 0xffffu; // 16-bit window row of a slot whose dense row is outside the window
static_assert(kPlanResidueChunk % kResRows == 0, "a workgroup takes a whole fraction of a chunk");
static_assert(kResidueWindowRowsMax < (int)kMiss, "window rows must fit 16 bits");

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

__device__ __forceinline__ unsigned window_locator(int c, int w0, int wn)
{
    const unsigned d = (unsigned)(c - w0);
    return d < (unsigned)wn ? d : kMiss;
}

// One residue row as its lane group keeps it: its slots as whole quads from the 4-aligned
// slot `abase` at or before its first one; the row's own slots are [head, end) of the 32.
// addr[s]: LDS byte address of this lane's 16 bytes of slot s's dense row; for a slot
// whose dense row is outside the window (bit s of missmask) it is the address of one of
// the row's slots that is inside, and the data has to come from memory instead.
struct ResidueRow {
    int row; // -1: nothing to do
    int abase, head, end, quads;
    unsigned missmask;
    bool accumulate;      // the row also has block segments (SpMM adds instead of storing)
    int addr[kBlockItems];
};

// Prepares the residue row `listed` (-1: none) of this lane group: the 8 lanes classify 4
// slots each against the window, exchange the result through `stage_loc` (32 shorts of
// this group) and leave the row's values in `my_val` (32 floats of this group; 0 outside
// the row).  A slot outside the row gets value 0 and the column of the row's first slot.
// skip_owned_slots: rows with block segments and at most that many aligned slots are left
// to the block kernel (SpMM under the whole-lists promise); 0 for SDDMM.
__device__ __forceinline__ void prepare_residue_row(int listed, int skip_owned_slots, const WindowDesc& d,
                                                    const int* __restrict__ row_ptr, const int* __restrict__ col,
                                                    const float* __restrict__ val, unsigned short* stage_loc,
                                                    float* my_val, ResidueRow& rr)
{
    const int ls = threadIdx.x % kResLanes;
    rr.row = -1;
    rr.abase = rr.head = rr.end = 0;
    rr.accumulate = false;
    int fill = d.w0;
    if (listed >= 0) {
        const ResidueItem it = residue_item(listed, row_ptr);
        if (!(it.accumulate && it.aligned <= skip_owned_slots)) {
            rr.row = listed;
            rr.accumulate = it.accumulate;
            if (it.cnt > 0) {
                rr.abase = it.first & ~(kVecLen - 1);
                rr.head = it.first - rr.abase;
                rr.end = rr.head + it.cnt;
                fill = col[it.first];
            }
        }
    }
    rr.quads = (rr.end + 3) / 4;
    constexpr int OWN = kBlockItems / kResLanes;
    unsigned u[OWN];
    unsigned best = kMiss, missbits = 0;
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        const int s = ls + i * kResLanes;
        const bool in = s >= rr.head && s < rr.end;
        u[i] = window_locator(in ? col[rr.abase + s] : fill, d.w0, d.wn);
        my_val[s] = in ? val[rr.abase + s] : 0.f;
        best = min(best, u[i]);
        if (u[i] == kMiss) missbits |= 1u << s;
    }
#pragma unroll
    for (int m = 1; m < kResLanes; m <<= 1) {
        best = min(best, (unsigned)__shfl_xor((int)best, m, kWave));
        missbits |= (unsigned)__shfl_xor((int)missbits, m, kWave);
    }
    if (best == kMiss) best = 0; // no slot inside the window: every read is replaced anyway
    rr.missmask = missbits;
#pragma unroll
    for (int i = 0; i < OWN; ++i) stage_loc[ls + i * kResLanes] = (unsigned short)(u[i] == kMiss ? best : u[i]);
    wave_lds_sync(); // the 8 lanes of a group are lanes of one wave
    const uint4* src = reinterpret_cast<const uint4*>(stage_loc);
#pragma unroll
    for (int i = 0; i < kBlockItems / 8; ++i) {
        const uint4 w4 = src[i];
        const unsigned w[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            rr.addr[8 * i + 2 * j] = (int)(((w[j] & 0xffffu) * kResLanes + ls) * 16);
            rr.addr[8 * i + 2 * j + 1] = (int)(((w[j] >> 16) * kResLanes + ls) * 16);
        }
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
