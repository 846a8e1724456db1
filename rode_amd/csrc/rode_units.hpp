// Inner loops shared by the SDDMM, SpMM and fused attention kernels: the dot products of
// one 32-slot unit (SDDMM) and the gather-accumulate over staged slot quads (SpMM).
#pragma once
#include "rode_device.hpp"

namespace rode {

// ---- SDDMM ------------------------------------------------------------------
// KT = width of the lane tile (32, 64 or 128 elements): LPR = KT / VEC lanes read KT
// consecutive elements of a dense row per load instruction.  A row of K elements is
// covered by NS such slabs (KT * NS >= K); EDGE says that the last slab is partial, in
// which case the lanes past K read nothing and contribute zero.
template <typename T, int KT>
struct SddmmShape {
    static constexpr int kVec = DenseVec<T>::kElems;
    static constexpr int kRegs = DotVec<T>::kRegs; // registers of a lane's part of the lhs row
    using Reg = typename DotVec<T>::Reg;
    static constexpr int kLpr = KT / kVec;     // lanes that cover one slab of a dense row
    static constexpr int kQuads = kLpr / 4;    // slot quads per lane group per unit
    static_assert(KT % kVec == 0 && kLpr >= 4 && kLpr <= 32 && (kLpr & (kLpr - 1)) == 0,
                  "unsupported tile width for this dense type");
};

// <lhs row, rhs row> restricted to this lane's elements.
template <typename T, int KT, int NS, bool EDGE>
__device__ __forceinline__ float lane_dot(const typename DotVec<T>::Reg (&a)[NS][DotVec<T>::kRegs],
                                          const T* __restrict__ row_lane, int k, int lane_elem)
{
    float d = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s)
        if (!EDGE || lane_elem + s * KT < k) d = DotVec<T>::dot(a[s], row_lane + s * KT, d);
    return d;
}

// Dot products of the 32-slot units of one step, the slots' columns already in lds_cols
// (lds_cols[e] = column of lane e's slot).  Returns the dot product for this lane's slot.
template <typename T, int KT, int NS, bool EDGE>
__device__ __forceinline__ float sddmm_unit_staged(const T* __restrict__ rhs_lane,
                                                   const typename DotVec<T>::Reg (&a)[NS][DotVec<T>::kRegs], int k,
                                                   const int* lds_cols, int lane)
{
    using S = SddmmShape<T, KT>;
    constexpr int LPR = S::kLpr;
    const int ls = lane % LPR;                    // lane inside its group
    const int group_first = (lane & 31) - ls;     // first slot (within the half) of this group
    const int* group_cols = lds_cols + (lane & 32) + group_first;
    float result = 0.f;

#pragma unroll
    for (int q = 0; q < S::kQuads; ++q) {
        const int4 c4 = *reinterpret_cast<const int4*>(group_cols + 4 * q);
        const int c[4] = {c4.x, c4.y, c4.z, c4.w};
        float p[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            p[j] = lane_dot<T, KT, NS, EDGE>(a, rhs_lane + (size_t)c[j] * k, k, ls * S::kVec);
        // transpose-reduce: afterwards lane (ls & 3) == j holds slot j of the quad
        const bool hi2 = ls & 2, hi1 = ls & 1;
        const float k0 = hi2 ? p[2] : p[0], s0 = hi2 ? p[0] : p[2];
        const float k1 = hi2 ? p[3] : p[1], s1 = hi2 ? p[1] : p[3];
        const float q0 = k0 + lane_xor2(s0);
        const float q1 = k1 + lane_xor2(s1);
        float r = (hi1 ? q1 : q0) + lane_xor1(hi1 ? q0 : q1);
        r = butterfly_sum<4, LPR>(r);
        if ((ls >> 2) == q) result = r;
    }
    return result;
}

// Dot products of one 32-slot unit of a block segment.  `my_col` is the column of this
// lane's slot.  Returns the dot product for this lane's slot.
template <typename T, int KT, int NS, bool EDGE>
__device__ __forceinline__ float sddmm_unit(const T* __restrict__ rhs_lane,
                                            const typename DotVec<T>::Reg (&a)[NS][DotVec<T>::kRegs], int my_col, int k,
                                            int* lds_cols, int lane)
{
    lds_cols[lane] = my_col;
    wave_lds_sync();
    return sddmm_unit_staged<T, KT, NS, EDGE>(rhs_lane, a, k, lds_cols, lane);
}

// ONCE: the row is used by this work item only (a residue row): loaded with the non-temporal
// hint, so that the stream of lhs rows does not displace gathered rhs rows (config 4: residue
// kernel 1.375 -> 1.334 ms at K=128, 0.656 -> 0.626 at K=64; for the group kernels, which
// read their lhs rows twice, the hint costs 8 %).
template <typename T, int KT, int NS, bool EDGE, bool ONCE = false>
__device__ __forceinline__ void load_lhs_slice(const T* __restrict__ lhs, int row, int k, int lane,
                                               typename DotVec<T>::Reg (&a)[NS][DotVec<T>::kRegs])
{
    using S = SddmmShape<T, KT>;
    const int e0 = (lane % S::kLpr) * S::kVec;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        DotVec<T>::zero(a[s]);
        if (!EDGE || e0 + s * KT < k) {
            if constexpr (ONCE)
                DotVec<T>::load_once(lhs + (size_t)row * k + e0 + s * KT, a[s]);
            else
                DotVec<T>::load(lhs + (size_t)row * k + e0 + s * KT, a[s]);
        }
    }
}

// ---- SpMM -------------------------------------------------------------------
template <typename T, int TN>
struct SpmmShape {
    using Acc = typename DenseVec<T>::Acc;          // type of values, accumulators and C
    static constexpr int kVec = DenseVec<T>::kElems;
    static constexpr int kLpr = TN / kVec;          // lanes that cover one B-row tile
    static constexpr int kGroupsWave = kWave / kLpr; // lane groups per wave
    static_assert(TN % kVec == 0 && kLpr >= 4 && kLpr <= 32 && (kLpr & (kLpr - 1)) == 0,
                  "unsupported tile width for this dense type");
};

__device__ __forceinline__ void load_quad(const float* p, float (&v)[4])
{
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load_quad(const double* p, double (&v)[4])
{
    const double2 t0 = *reinterpret_cast<const double2*>(p), t1 = *reinterpret_cast<const double2*>(p + 2);
    v[0] = t0.x; v[1] = t0.y; v[2] = t1.x; v[3] = t1.y;
}

// acc += sum over the slot quads {first_quad, first_quad + stride, ...} < nquads of
// value * B[col, tile].  QUADS_MAX bounds the trip count at compile time.
template <typename T, int TN, int QUADS_MAX, bool FULL>
__device__ __forceinline__ void spmm_gather(const T* __restrict__ b_lane, size_t ldb,
                                            typename DenseVec<T>::Acc (&acc)[SpmmShape<T, TN>::kVec],
                                            const int* lds_col, const typename DenseVec<T>::Acc* lds_val,
                                            int first_quad, int stride, int nquads)
{
    using A = typename DenseVec<T>::Acc;
    constexpr int VEC = SpmmShape<T, TN>::kVec;
#pragma unroll
    for (int i = 0; i < QUADS_MAX; ++i) {
        const int q = first_quad + i * stride;
        if (FULL || q < nquads) {
            const int4 c4 = *reinterpret_cast<const int4*>(lds_col + 4 * q);
            const int c[4] = {c4.x, c4.y, c4.z, c4.w};
            A v[4];
            load_quad(lds_val + 4 * q, v);
            A b[4][VEC];
#pragma unroll
            for (int j = 0; j < 4; ++j) DenseVec<T>::load(b_lane + (size_t)c[j] * ldb, b[j]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int x = 0; x < VEC; ++x) acc[x] = fma(v[j], b[j][x], acc[x]);
        }
    }
}

// The same sum over the quads 0 .. nquads - 1, two quads per step: the loads of both are
// issued before either is used (eight dense rows in flight per lane instead of four), and a
// quad that does not exist loads nothing and adds zeros.  For work items of a few quads
// whose kernels are bound by memory latency (residue rows).
template <typename T, int TN, int QUADS_MAX>
__device__ __forceinline__ void spmm_gather_pairs(const T* __restrict__ b_lane, size_t ldb,
                                                  typename DenseVec<T>::Acc (&acc)[SpmmShape<T, TN>::kVec],
                                                  const int* lds_col, const typename DenseVec<T>::Acc* lds_val, int nquads)
{
    using A = typename DenseVec<T>::Acc;
    constexpr int VEC = SpmmShape<T, TN>::kVec;
    static_assert(QUADS_MAX % 2 == 0, "two quads per step");
#pragma unroll
    for (int q = 0; q < QUADS_MAX; q += 2) {
        if (q < nquads) {
            A v[2][4], b[2][4][VEC];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v[h][j] = A(0);
#pragma unroll
                    for (int x = 0; x < VEC; ++x) b[h][j][x] = A(0);
                }
                if (q + h < nquads) {
                    const int4 c4 = *reinterpret_cast<const int4*>(lds_col + 4 * (q + h));
                    const int c[4] = {c4.x, c4.y, c4.z, c4.w};
                    load_quad(lds_val + 4 * (q + h), v[h]);
#pragma unroll
                    for (int j = 0; j < 4; ++j) DenseVec<T>::load(b_lane + (size_t)c[j] * ldb, b[h][j]);
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int x = 0; x < VEC; ++x) acc[x] = fma(v[h][j], b[h][j][x], acc[x]);
        }
    }
}

} // namespace rode
