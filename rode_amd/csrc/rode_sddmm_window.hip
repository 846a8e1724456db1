// SDDMM for the chunks of the residue list whose dense rows cluster in a window (banded
// matrices; see rode_window.hpp for the shape of the kernel and rode_plan.hip for how
// the chunks are chosen).  Same rows and slots as sddmm_residue_kernel in rode_sddmm.hip
// (reference: RoDe_SDDMM/RoDeSddmm.cu:206-494); what differs is where the rhs rows come
// from, and when the lane-slices of a dot product are combined: each lane keeps, for every
// slot of its row, the partial dot product over its own 16 bytes of all column tiles, and
// the 8 lanes of a row are summed once, after the last tile, with a transpose-reduce (DPP
// quad_perm for xor 1 / 2, ds_swizzle for xor 4) that leaves slot 8i + l in lane l.
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

template <typename T, bool EDGE>
__global__ void __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
sddmm_residue_window_kernel(int m2, int k, const int* __restrict__ col, const float* __restrict__ val,
                            const T* __restrict__ lhs, const T* __restrict__ rhs, float* __restrict__ out,
                            const PlannedChunk* __restrict__ rows)
{
    constexpr int VEC = DenseVec<T>::kElems;
    constexpr int TW = kResLanes * VEC; // elements of a dense row in one tile
    constexpr int QUADS = kBlockItems / 4;
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

    ResidueRow rr;
    float* my_v = lds_val + group * kResValStride;
    load_planned_row(pc, local, 0, val, my_v, rr);
    const int listed = rr.row;
    // first tile of the lhs row
    uint4 a_raw = make_uint4(0, 0, 0, 0);
    const T* lhs_row = lhs + (size_t)(listed >= 0 ? listed : 0) * k;
    if ((!EDGE || ls * VEC < k) && listed >= 0) a_raw = *reinterpret_cast<const uint4*>(lhs_row + ls * VEC);
    const int wave_quads = wave_max_quads(rr.quads);
    const bool wave_all_hit = __ballot(rr.missmask != 0) == 0ull;

    float p[kBlockItems]; // this lane's share of every slot's dot product
#pragma unroll
    for (int s = 0; s < kBlockItems; ++s) p[s] = 0.f;
    const char* win_bytes = reinterpret_cast<const char*>(win);
    for (int tile = 0; tile < tiles; ++tile) {
        const int col_off = tile * TW + ls * VEC;
        const bool col_ok = !EDGE || col_off < k;
        const T* rhs_lane = rhs + (col_ok ? col_off : 0);
        float a[VEC];
        DenseVec<T>::unpack(a_raw, a); // zeros past the last column: those lanes add nothing
        // (no registers to spare for carrying the next tile through the work on this one:
        // the other workgroup of the CU computes while this one waits for its tile)
        if (tile > 0) __syncthreads(); // every wave is done with the previous tile's window
        res_fill(win, reinterpret_cast<const char*>(rhs_lane + (size_t)d.w0 * k), row_bytes, d.wn, col_ok);
        if (tile + 1 < tiles) {
            const int next_off = col_off + TW;
            a_raw = make_uint4(0, 0, 0, 0);
            if ((!EDGE || next_off < k) && listed >= 0) a_raw = *reinterpret_cast<const uint4*>(lhs_row + next_off);
        }
        __syncthreads();
        // (the miss path's inputs are made opaque per tile: otherwise the compiler computes
        // every position's test and memory address once, outside the tile loop, and holds
        // them in registers of their own - more than there are)
        int first_t = rr.first;
        unsigned miss_t = rr.missmask;
        if (!wave_all_hit) asm volatile("" : "+v"(first_t), "+v"(miss_t));
#pragma unroll
        for (int q = 0; q < QUADS; ++q) {
            if (q < wave_quads) { // the same for every lane of the wave
                uint4 raw[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) raw[j] = *reinterpret_cast<const uint4*>(win_bytes + rr.addr[4 * q + j]);
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
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float b[VEC];
                    DenseVec<T>::unpack(raw[j], b);
#pragma unroll
                    for (int x = 0; x < VEC; ++x) p[4 * q + j] = fmaf(a[x], b[x], p[4 * q + j]);
                }
            }
        }
    }

    // lane l of the group ends up with the dot products of the positions l, 8 + l, 16 + l, 24 + l
#pragma unroll
    for (int i = 0; i < kBlockItems / kResLanes; ++i) {
        float part8[kResLanes];
#pragma unroll
        for (int j = 0; j < kResLanes; ++j) part8[j] = p[i * kResLanes + j];
        const float dot = transpose_reduce8(part8, ls);
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
    if (((size_t)k * sizeof(T)) % (kResLanes * 16) != 0)
        sddmm_residue_window_kernel<T, true><<<g, kResThreads, 0, stream>>>(m2, k, col, val, lhs, rhs, out, rows);
    else
        sddmm_residue_window_kernel<T, false><<<g, kResThreads, 0, stream>>>(m2, k, col, val, lhs, rhs, out, rows);
    return hipGetLastError();
}

template hipError_t sddmm_window_launch<float>(int, int, const int*, const float*, const float*, const float*, float*,
                                               const int*, const void*, hipStream_t);
template hipError_t sddmm_window_launch<__half>(int, int, const int*, const float*, const __half*, const __half*, float*,
                                                const int*, const void*, hipStream_t);

} // namespace rode
