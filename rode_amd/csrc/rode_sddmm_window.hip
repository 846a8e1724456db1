// SDDMM for the chunks of the residue list whose dense rows cluster in a window (banded
// matrices; see rode_window.hpp for the shape of the kernel and rode_plan.hip for how
// the chunks are chosen).  Same rows and slots as sddmm_residue_kernel in rode_sddmm.hip
// (reference: RoDe_SDDMM/RoDeSddmm.cu:206-494); what differs is where the rhs rows come
// from, and when the lane-slices of a dot product are combined (two variants, see the
// kernel): with a transpose-reduce over the 8 lanes of a row (DPP quad_perm for xor 1 / 2,
// ds_swizzle for xor 4) that leaves position 8i + l in lane l.
#include "rode_window.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

// Sum over the 8 lanes of a group of 8 per-lane values; lane l returns the total of p[l].
__device__ __forceinline__ float transpose_reduce8(const float (&p)[8], int ls)
{
    const bool b2 = ls & 4, b1 = ls & 2, b0 = ls & 1;
    float r4[4], r2[2];
#pragma unroll
    for (int k = 0; k < 4; ++k) r4[k] = (b2 ? p[k + 4] : p[k]) + lane_xor4(b2 ? p[k] : p[k + 4]);
#pragma unroll
    for (int k = 0; k < 2; ++k) r2[k] = (b1 ? r4[k + 2] : r4[k]) + lane_xor2(b1 ? r4[k] : r4[k + 2]);
    return (b0 ? r2[1] : r2[0]) + lane_xor1(b0 ? r2[0] : r2[1]);
}

// One slot quad of a tile: this lane's 16 bytes of the four dense rows, from the window or,
// for positions outside it, from memory.
template <typename T, bool EDGE, bool PACKED>
__device__ __forceinline__ void window_quad(const ResidueRow<PACKED>& rr, const PlannedChunk& pc, int local, int q,
                                            const char* win_bytes, bool wave_all_hit, unsigned miss_t, int first_t,
                                            const int* __restrict__ col, const T* rhs_lane, int k, bool col_ok,
                                            uint4 (&raw)[4])
{
    if (PACKED) {
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            unsigned pair = rr.addr[2 * q + j / 2];
            asm volatile("" : "+v"(pair)); // unpacked here, per tile, not once for all tiles
            raw[j] = *reinterpret_cast<const uint4*>(win_bytes + (pair & 0xffffu));
            raw[j + 1] = *reinterpret_cast<const uint4*>(win_bytes + (pair >> 16));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) raw[j] = *reinterpret_cast<const uint4*>(win_bytes + rr.addr[4 * q + j]);
    }
    if (!wave_all_hit) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if ((miss_t >> (4 * q + j)) & 1u) {
                // outside the window: the slot's column, then the rhs row from memory
                const int c = col[first_t + planned_slot(pc, local, 4 * q + j)];
                raw[j] = col_ok ? *reinterpret_cast<const uint4*>(rhs_lane + (size_t)c * k) : make_uint4(0, 0, 0, 0);
            }
        }
    }
}

// PER_TILE = false: each lane keeps, for every slot of its row, the partial dot product over
// its own 16 bytes of all column tiles; the 8 lanes of a row are summed once, after the
// last tile.  32 registers of partial sums leave none to carry the next tile of the window
// through the work on the current one: a tile is loaded, stored to LDS and waited for
// between two barriers (the CU's other workgroup computes meanwhile).
// PER_TILE = true: the 8 lanes are summed after every tile (position 8 i + l accumulates
// in lane l), the LDS addresses are kept two to a register, and the registers that frees
// prefetch the next tile.  More instructions per tile, no exposed load: faster for rows of
// up to two tiles (measured on the banded benchmark: fp32 K=64 0.40 -> 0.36 ms, K=128
// 0.54 -> 0.57 ms).
template <typename T, bool EDGE, bool PER_TILE>
__global__ void __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
sddmm_residue_window_kernel(int m2, int k, const int* __restrict__ col, const float* __restrict__ val,
                            const T* __restrict__ lhs, const T* __restrict__ rhs, float* __restrict__ out,
                            const PlannedChunk* __restrict__ rows)
{
    constexpr int VEC = DenseVec<T>::kElems;
    constexpr int TW = kResLanes * VEC; // elements of a dense row in one tile
    constexpr int QUADS = kBlockItems / 4;
    constexpr int OWN = kBlockItems / kResLanes;
    __shared__ uint4 win[kResWinVecs];
    __shared__ __attribute__((aligned(16))) float lds_val[kResRows * kResValStride];

    const int part = xcd_logical_block(blockIdx.x, gridDim.x);
    const int chunk = part / kResParts;
    if (chunk >= plan_residue_chunks(m2)) return;
    const int group = threadIdx.x / kResLanes, ls = threadIdx.x % kResLanes;
    const PlannedChunk& pc = rows[chunk];
    struct { int w0, wn; } d = {pc.w0, pc.wn};
    if (d.wn <= 0) return; // the standard kernel has this chunk
    const int local = (part % kResParts) * kResRows + group; // this lane group's row of the chunk
    const size_t row_bytes = (size_t)k * sizeof(T);
    const int tiles = (k + TW - 1) / TW;

    uint4 pf[PER_TILE ? kResPrefetch : 1];
    if constexpr (PER_TILE) { // first tile of the window on its way while the row is loaded
        const bool ok = !EDGE || ls * VEC < k;
        res_prefetch(pf, reinterpret_cast<const char*>(rhs + (size_t)d.w0 * k + (ok ? ls * VEC : 0)), row_bytes, d.wn, ok);
    }
    ResidueRow<PER_TILE> rr;
    float* my_v = lds_val + group * kResValStride;
    load_planned_row(pc, local, 0, val, my_v, rr);
    const int listed = rr.row;
    // first tile of the lhs row
    uint4 a_raw = make_uint4(0, 0, 0, 0);
    const T* lhs_row = lhs + (size_t)(listed >= 0 ? listed : 0) * k;
    if ((!EDGE || ls * VEC < k) && listed >= 0) a_raw = *reinterpret_cast<const uint4*>(lhs_row + ls * VEC);
    const int wave_quads = wave_max_quads(rr.quads);
    const bool wave_all_hit = __ballot(rr.missmask != 0) == 0ull;
    if constexpr (PER_TILE) {
        res_commit(win, pf, d.wn);
        __syncthreads();
    }

    // PER_TILE: acc[i] is the dot product of position 8 i + ls over the tiles done so far;
    // else acc[s] is this lane's share of position s
    constexpr int NACC = PER_TILE ? OWN : kBlockItems;
    float acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = 0.f;
    const char* win_bytes = reinterpret_cast<const char*>(win);
    for (int tile = 0; tile < tiles; ++tile) {
        const int col_off = tile * TW + ls * VEC;
        const bool col_ok = !EDGE || col_off < k;
        const T* rhs_lane = rhs + (col_ok ? col_off : 0);
        typename DotVec<T>::Reg a[DotVec<T>::kRegs]; // zeros past the last column: those lanes add nothing
        {
            const uint32_t w[4] = {a_raw.x, a_raw.y, a_raw.z, a_raw.w};
            DotVec<T>::load(reinterpret_cast<const T*>(w), a);
        }
        const bool more = tile + 1 < tiles;
        if constexpr (!PER_TILE) {
            if (tile > 0) __syncthreads(); // every wave is done with the previous tile's window
            res_fill(win, reinterpret_cast<const char*>(rhs_lane + (size_t)d.w0 * k), row_bytes, d.wn, col_ok);
        }
        if (more) {
            const int next_off = col_off + TW;
            const bool ok = !EDGE || next_off < k;
            if constexpr (PER_TILE)
                res_prefetch(pf, reinterpret_cast<const char*>(rhs + (size_t)d.w0 * k + (ok ? next_off : 0)), row_bytes,
                             d.wn, ok);
            a_raw = make_uint4(0, 0, 0, 0);
            if (ok && listed >= 0) a_raw = *reinterpret_cast<const uint4*>(lhs_row + next_off);
        }
        if constexpr (PER_TILE)
            __builtin_amdgcn_sched_barrier(0); // the loads above are issued before the work below, not after it
        else
            __syncthreads();
        // (the miss path's inputs are made opaque per tile: otherwise the compiler computes
        // every position's test and memory address once, outside the tile loop, and holds
        // them in registers of their own - more than there are)
        int first_t = rr.first;
        unsigned miss_t = rr.missmask;
        if (!wave_all_hit) asm volatile("" : "+v"(first_t), "+v"(miss_t));
        if constexpr (PER_TILE) {
#pragma unroll
            for (int i = 0; i < OWN; ++i) {
                if (2 * i < wave_quads) { // the same for every lane of the wave
                    float part8[kResLanes]; // this lane's share of the positions 8 i .. 8 i + 7
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        uint4 raw[4];
                        window_quad<T, EDGE, PER_TILE>(rr, pc, local, 2 * i + h, win_bytes, wave_all_hit, miss_t, first_t,
                                                       col, rhs_lane, k, col_ok, raw);
#pragma unroll
                        for (int j = 0; j < 4; ++j) part8[4 * h + j] = DotVec<T>::dot_raw(a, raw[j], 0.f);
                    }
                    acc[i] += transpose_reduce8(part8, ls);
                }
            }
        } else {
#pragma unroll
            for (int q = 0; q < QUADS; ++q) {
                if (q < wave_quads) { // the same for every lane of the wave
                    uint4 raw[4];
                    window_quad<T, EDGE, PER_TILE>(rr, pc, local, q, win_bytes, wave_all_hit, miss_t, first_t, col,
                                                   rhs_lane, k, col_ok, raw);
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[4 * q + j] = DotVec<T>::dot_raw(a, raw[j], acc[4 * q + j]);
                }
            }
        }
        if constexpr (PER_TILE) {
            if (more) {
                __syncthreads(); // every wave is done with this tile's window
                res_commit(win, pf, d.wn);
                __syncthreads();
            }
        }
    }

    // lane l of the group stores the positions l, 8 + l, 16 + l, 24 + l
#pragma unroll
    for (int i = 0; i < OWN; ++i) {
        float dot;
        if constexpr (PER_TILE) {
            dot = acc[i];
        } else {
            float part8[kResLanes];
#pragma unroll
            for (int j = 0; j < kResLanes; ++j) part8[j] = acc[i * kResLanes + j];
            dot = transpose_reduce8(part8, ls);
        }
        const int pos = i * kResLanes + ls;
        if (pos < rr.cnt) out[rr.first + planned_slot(pc, local, pos)] = my_v[pos] * dot;
    }
}

} // namespace

// The window kernel over the planned chunks of the residue list.  T = float or __half.
template <typename T>
hipError_t sddmm_window_launch(int m2, int k, const int* col, const float* val, const T* lhs, const T* rhs, float* out,
                               const int* plan, const void* plan_rows, hipStream_t stream)
{
    if (m2 <= 0) return hipSuccess;
    const int g = grid_for_residue_parts(m2);
    const PlannedChunk* rows = static_cast<const PlannedChunk*>(plan_rows);
    const bool edge = ((size_t)k * sizeof(T)) % (kResLanes * 16) != 0;
    const bool per_tile = (size_t)k * sizeof(T) <= 2 * kResLanes * 16; // at most two tiles per row
    if (edge && per_tile)
        sddmm_residue_window_kernel<T, true, true><<<g, kResThreads, 0, stream>>>(m2, k, col, val, lhs, rhs, out, rows);
    else if (edge)
        sddmm_residue_window_kernel<T, true, false><<<g, kResThreads, 0, stream>>>(m2, k, col, val, lhs, rhs, out, rows);
    else if (per_tile)
        sddmm_residue_window_kernel<T, false, true><<<g, kResThreads, 0, stream>>>(m2, k, col, val, lhs, rhs, out, rows);
    else
        sddmm_residue_window_kernel<T, false, false><<<g, kResThreads, 0, stream>>>(m2, k, col, val, lhs, rhs, out, rows);
    return hipGetLastError();
}

template hipError_t sddmm_window_launch<float>(int, int, const int*, const float*, const float*, const float*, float*,
                                               const int*, const void*, hipStream_t);
template hipError_t sddmm_window_launch<__half>(int, int, const int*, const float*, const __half*, const __half*, float*,
                                                const int*, const void*, hipStream_t);

} // namespace rode
