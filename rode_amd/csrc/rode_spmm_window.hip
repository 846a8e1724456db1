// SpMM for the chunks of the residue list whose dense rows cluster in a window (banded
// matrices; see rode_window.hpp for the shape of the kernel and rode_plan.hip for how
// the chunks are chosen).  Same rows, same slots and the same store/accumulate rule as
// spmm_residue_kernel in rode_spmm.hip (reference: RoDe_SpMM/RoDeSpmm.cu:41-195); what
// differs is where B comes from.
#define RODE_PHASE_READER // (debug builds with RODE_PHASE_TIMING: this file holds the counters that are read back)
#include "rode_window.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

template <typename T, bool EDGE>
__global__ void __launch_bounds__(kResThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
spmm_residue_window_kernel(int m2, int n, int owned_slots, const int* __restrict__ col, const float* __restrict__ val,
                           const T* __restrict__ B, float* __restrict__ C, const PlannedChunk* __restrict__ rows)
{
    constexpr int VEC = DenseVec<T>::kElems;
    constexpr int TW = kResLanes * VEC; // columns of one tile
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
    const size_t row_bytes = (size_t)n * sizeof(T);
    const int tiles = (n + TW - 1) / TW;
    RODE_PHASE_BEGIN;

    // first tile of the window on its way while the row is loaded
    uint4 pf[kResPrefetch];
    {
        const bool ok = !EDGE || ls * VEC < n;
        res_prefetch(pf, reinterpret_cast<const char*>(B + (size_t)d.w0 * n + (ok ? ls * VEC : 0)), row_bytes, d.wn, ok);
    }
    ResidueRow<false> rr;
    float* my_v = lds_val + group * kResValStride;
    load_planned_row(pc, local, owned_slots, val, my_v, rr);
    const int wave_quads = wave_max_quads(rr.quads);
    const bool wave_all_hit = __ballot(rr.missmask != 0) == 0ull;
    RODE_PHASE(0);
    res_commit(win, pf, d.wn);
    __syncthreads();
    RODE_PHASE(1);

    const char* win_bytes = reinterpret_cast<const char*>(win);
    for (int tile = 0; tile < tiles; ++tile) {
        const int col_off = tile * TW + ls * VEC;
        const bool col_ok = !EDGE || col_off < n;
        const T* b_lane = B + (col_ok ? col_off : 0);
        const bool more = tile + 1 < tiles;
        if (more) {
            const int next_off = col_off + TW;
            const bool ok = !EDGE || next_off < n;
            res_prefetch(pf, reinterpret_cast<const char*>(B + (size_t)d.w0 * n + (ok ? next_off : 0)), row_bytes, d.wn, ok);
        }
        __builtin_amdgcn_sched_barrier(0); // the loads above are issued before the work below, not after it
        float acc[VEC];
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[x] = 0.f;
        // (the miss path's inputs are made opaque per tile: otherwise the compiler computes
        // every position's test and memory address once, outside the tile loop, and holds
        // them in registers of their own - more than there are)
        int first_t = rr.first;
        unsigned miss_t = rr.missmask;
        if (!wave_all_hit) asm volatile("" : "+v"(first_t), "+v"(miss_t));
#pragma unroll
        for (int q = 0; q < QUADS; ++q) {
            if (q < wave_quads) { // the same for every lane of the wave
                const float4 v4 = *reinterpret_cast<const float4*>(my_v + 4 * q);
                const float v[4] = {v4.x, v4.y, v4.z, v4.w};
                uint4 raw[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) raw[j] = *reinterpret_cast<const uint4*>(win_bytes + rr.addr[4 * q + j]);
                if (!wave_all_hit) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if ((miss_t >> (4 * q + j)) & 1u) {
                            // outside the window: the slot's column, then the row of B from memory
                            const int c = col[first_t + planned_slot(pc, local, 4 * q + j)];
                            raw[j] = *reinterpret_cast<const uint4*>(b_lane + (size_t)c * n);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float b[VEC];
                    DenseVec<T>::unpack(raw[j], b);
#pragma unroll
                    for (int x = 0; x < VEC; ++x) acc[x] = fmaf(v[j], b[x], acc[x]);
                }
            }
        }
        if (rr.row >= 0 && col_ok) {
            float* c_lane = C + (size_t)rr.row * n + col_off;
            if (rr.accumulate) {
                if (rr.quads > 0) {
#pragma unroll
                    for (int x = 0; x < VEC; ++x) atomicAdd(c_lane + x, acc[x]);
                }
            } else {
                // a listed row without slots of its own (empty, unaligned start) is stored as zeros
                const bool any = rr.quads > 0;
#pragma unroll
                for (int x = 0; x < VEC; x += 4)
                    *reinterpret_cast<float4*>(c_lane + x) = make_float4(any ? acc[x] : 0.f, any ? acc[x + 1] : 0.f,
                                                                         any ? acc[x + 2] : 0.f, any ? acc[x + 3] : 0.f);
            }
        }
        RODE_PHASE(2);
        if (more) {
            __syncthreads(); // every wave is done with this tile's window
            RODE_PHASE(3);
            res_commit(win, pf, d.wn);
            __syncthreads();
            RODE_PHASE(4);
        }
    }
    RODE_PHASE_END;
}

} // namespace

// The window kernel over the planned chunks of the residue list.  T = float or __half.
template <typename T>
hipError_t spmm_window_launch(int m2, int n, int owned_slots, const int* col, const float* val, const T* B, float* C,
                              const int* plan, const void* plan_rows, hipStream_t stream)
{
    if (m2 <= 0) return hipSuccess;
    const int g = grid_for_residue_parts(m2);
    const PlannedChunk* rows = static_cast<const PlannedChunk*>(plan_rows);
    if (((size_t)n * sizeof(T)) % (kResLanes * 16) != 0)
        spmm_residue_window_kernel<T, true><<<g, kResThreads, 0, stream>>>(m2, n, owned_slots, col, val, B, C, rows);
    else
        spmm_residue_window_kernel<T, false><<<g, kResThreads, 0, stream>>>(m2, n, owned_slots, col, val, B, C, rows);
    return hipGetLastError();
}

template hipError_t spmm_window_launch<float>(int, int, int, const int*, const float*, const float*, float*, const int*,
                                              const void*, hipStream_t);
template hipError_t spmm_window_launch<__half>(int, int, int, const int*, const float*, const __half*, float*,
                                               const int*, const void*, hipStream_t);

} // namespace rode
