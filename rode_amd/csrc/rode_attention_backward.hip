// Gradient of sparse attention on a CSR pattern in two kernels.  With
//     s[idx] = scale * values[idx] * <q[r, :], k[col(idx), :]>,  p = softmax over the row of s,
//     out[r, :] = sum_idx p[idx] * v[col(idx), :]
// and g = d(loss)/d(out), the gradients are
//     dp[idx] = <g[r, :], v[col(idx), :]>
//     dz[idx] = scale * values[idx] * p[idx] * (dp[idx] - <g[r, :], out[r, :]>)     (= d(loss)/d<q, k>)
//     dq[r, :] = sum_idx dz[idx] * k[col(idx), :]
//     dk[c, :] = sum over the nonzeros of column c of dz * q[row, :]
//     dv[c, :] = sum over the nonzeros of column c of p  * g[row, :]
// (the row sum of p * dp in the softmax gradient equals <g[r, :], out[r, :]>, so a row needs
// one pass).  The reference's op is the forward SDDMM alone (RoDe_SDDMM/rode_sddmm.py:194-248);
// chained from the separate kernels this gradient takes an SDDMM, a softmax gradient, three
// SpMMs and two permutations of nonzero-sized arrays into the transposed order.
//
//   * row pass (attention_backward_rows_kernel, attention_backward_group_kernel): the shape of
//     the forward kernels with k and v in each other's place - dp is the SDDMM unit on rows of
//     v, dq the SpMM gather of rows of k - and no running softmax.  Writes dq and, per nonzero,
//     the pair (p, dz) to the nonzero's slot in the transposed pattern (8-byte stores that
//     nobody waits for; the four rows of a group write 32 consecutive bytes per column).
//   * column pass (attention_backward_cols_kernel, attention_backward_cols_group_kernel) over
//     the transposed pattern: dv and dk in one walk, every row of g and of q loaded once for
//     both, the pairs read in order (the separate kernels make two permuted copies of
//     nonzero-sized arrays instead).
// fp16 operands: the rows of v meet g in packed fp16 dot products like the scores of the
// forward pass; g (always fp32) is scaled by the largest magnitude of its row before it is
// rounded to fp16 for that purpose, so that small gradients keep eleven bits whatever their
// size.  Everything else accumulates g, p and dz in fp32.
#include "rode_items.hpp"
#include "rode_units.hpp"
#include "rode_internal.hpp"

#include <type_traits>

namespace rode {

namespace {

template <int LO, int HI>
__device__ __forceinline__ float butterfly_max(float v)
{
    if (LO <= 1 && 1 < HI) v = fmaxf(v, lane_xor1(v));
    if (LO <= 2 && 2 < HI) v = fmaxf(v, lane_xor2(v));
    if (LO <= 4 && 4 < HI) v = fmaxf(v, lane_xor4(v));
    if (LO <= 8 && 8 < HI) v = fmaxf(v, lane_xor8(v));
    if (LO <= 16 && 16 < HI) v = fmaxf(v, lane_xor16(v));
    if (LO <= 32 && 32 < HI) v = fmaxf(v, lane_xor32(v));
    return v;
}

template <int N>
__device__ __forceinline__ void load_floats(const float* p, float (&out)[N])
{
    static_assert(N % 4 == 0, "whole 128-bit loads");
#pragma unroll
    for (int x = 0; x < N; x += 4) {
        const float4 t = *reinterpret_cast<const float4*>(p + x);
        out[x] = t.x; out[x + 1] = t.y; out[x + 2] = t.z; out[x + 3] = t.w;
    }
}

// A lane's DenseVec<T>::kElems consecutive fp32 elements of a row of g as the left operand of
// DotVec<T>: as they are (fp32), or times inv_scale and rounded to fp16 pairs.
template <typename T>
__device__ __forceinline__ void grad_regs(const float (&raw)[DenseVec<T>::kElems], float inv_scale,
                                          typename DotVec<T>::Reg (&a)[DotVec<T>::kRegs])
{
    if constexpr (std::is_same<T, __half>::value) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const __half2 h = __floats2half2_rn(raw[2 * x] * inv_scale, raw[2 * x + 1] * inv_scale);
            a[x] = *reinterpret_cast<const uint32_t*>(&h);
        }
    } else {
#pragma unroll
        for (int x = 0; x < 4; ++x) a[x] = raw[x];
    }
}

template <int VEC>
__device__ __forceinline__ float abs_max(const float (&raw)[VEC])
{
    float m = 0.f;
#pragma unroll
    for (int x = 0; x < VEC; ++x) m = fmaxf(m, fabsf(raw[x]));
    return m;
}

template <int VEC>
__device__ __forceinline__ void store_floats(float* p, const float (&v)[VEC])
{
#pragma unroll
    for (int x = 0; x < VEC; x += 4) *reinterpret_cast<float4*>(p + x) = make_float4(v[x], v[x + 1], v[x + 2], v[x + 3]);
}

// What the forward kernel left per nonzero is the probability itself (stats == NULL) or the
// scaled score, with the row's (maximum, 1 / sum) in stats: p = exp(score - maximum) / sum.
struct RowStat {
    float max = 0.f, inv = 1.f;
    bool scores = false;
    __device__ __forceinline__ float prob(float kept) const { return scores ? __expf(kept - max) * inv : kept; }
};
__device__ __forceinline__ RowStat row_stat(const float2* stats, int row)
{
    RowStat r;
    if (stats != nullptr) {
        const float2 s = stats[row];
        r.max = s.x, r.inv = s.y, r.scores = true;
    }
    return r;
}

// ---- row pass -------------------------------------------------------------------------------
// One wave per row of the pattern, 64 slots per step (attention_rows_kernel's walk).
template <typename T, int D>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
attention_backward_rows_kernel(int M, const int* __restrict__ row_ptr, const int* __restrict__ col,
                               const float* __restrict__ val, const float* __restrict__ probs,
                               const float2* __restrict__ stats, const float* __restrict__ g, const float* __restrict__ out,
                               const T* __restrict__ k, const T* __restrict__ v, float scale, const int* __restrict__ t_slot,
                               float* __restrict__ dq, float2* __restrict__ pz, RowOwners owners, HeadStrides heads)
{
    probs = of_head(probs, heads.nnz), g = of_head(g, heads.rows), out = of_head(out, heads.rows);
    stats = of_head(stats, heads.rows / D);
    k = of_head(k, heads.cols), v = of_head(v, heads.cols), dq = of_head(dq, heads.rows), pz = of_head(pz, heads.nnz);
    using S = SpmmShape<T, D>;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    constexpr bool kScaled = std::is_same<T, __half>::value;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg * kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int row = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (row >= M) return;
    if (owned_elsewhere(owners, row, 0)) return; // a row of a group: attention_backward_group_kernel has it
    const int s = row_ptr[row], e = row_ptr[row + 1];
    const int ls = lane % LPR, group = lane / LPR;
    float acc[VEC];
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = 0.f;
    float* dq_lane = dq + (size_t)row * D + ls * VEC;
    if (e <= s) { // a row without nonzeros: nothing depends on its q
        if (group == 0) store_floats<VEC>(dq_lane, acc);
        return;
    }
    const RowStat stat = row_stat(stats, row);
    float g_raw[VEC], o_raw[VEC];
    load_floats<VEC>(g + (size_t)row * D + ls * VEC, g_raw);
    load_floats<VEC>(out + (size_t)row * D + ls * VEC, o_raw);
    float part = 0.f;
#pragma unroll
    for (int x = 0; x < VEC; ++x) part = fmaf(g_raw[x], o_raw[x], part);
    const float delta = butterfly_sum<1, LPR>(part);
    float g_scale = 1.f, g_inv = 1.f;
    if constexpr (kScaled) {
        g_scale = butterfly_max<1, LPR>(abs_max<VEC>(g_raw));
        g_inv = g_scale > 0.f ? 1.0f / g_scale : 0.f;
    }
    typename DotVec<T>::Reg a[1][DotVec<T>::kRegs];
    grad_regs<T>(g_raw, g_inv, a[0]);

    const T* v_lane = v + ls * VEC;
    const T* k_lane = k + ls * VEC;
    int* my_c = lds_c + wave * kWave;
    float* my_p = lds_p + wave * kWave;
    for (int off = s; off < e; off += kWave) {
        const int slot = off + lane;
        const bool live = slot < e;
        const int idx = live ? slot : e - 1; // lanes past the row repeat its last slot with weight 0
        const int c = col[idx];
        const float w = val[idx], p = stat.prob(probs[idx]);
        float dz = 0.f;
        if (off + (lane & 32) < e) { // the upper half sits out a step that has nothing for it
            const float dp = sddmm_unit<T, D, 1, false>(v_lane, a, c, D, my_c, lane) * g_scale;
            if (live) dz = scale * w * p * (dp - delta);
        }
        if (live) pz[t_slot[idx]] = make_float2(p, dz);
        my_p[lane] = dz;
        wave_lds_sync();
        const int nlive = min(e - off, kWave);
        if (nlive == kWave)
            spmm_gather<T, D, 16 / G, true>(k_lane, (size_t)D, acc, my_c, my_p, group, G, 16);
        else
            spmm_gather<T, D, 16 / G, false>(k_lane, (size_t)D, acc, my_c, my_p, group, G, (nlive + 3) / 4);
        wave_lds_sync();
    }
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = butterfly_sum<LPR, kWave>(acc[x]);
    if (group == 0) store_floats<VEC>(dq_lane, acc);
}

// The groups of a group plan: one wave per group of four adjacent rows, along their shared
// run every v row and every k row loaded once for the four rows (attention_group_kernel's
// walk), then each row's other nonzeros the way attention_backward_rows_kernel takes them.
template <typename T, int D>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
attention_backward_group_kernel(int n_groups, const RowGroup* __restrict__ groups, const int* __restrict__ row_ptr,
                                const int* __restrict__ col, const float* __restrict__ val,
                                const float* __restrict__ probs, const float2* __restrict__ stats,
                                const float* __restrict__ g, const float* __restrict__ out, const T* __restrict__ k,
                                const T* __restrict__ v, float scale, const int* __restrict__ t_slot,
                                float* __restrict__ dq, float2* __restrict__ pz, HeadStrides heads)
{
    probs = of_head(probs, heads.nnz), g = of_head(g, heads.rows), out = of_head(out, heads.rows);
    stats = of_head(stats, heads.rows / D);
    k = of_head(k, heads.cols), v = of_head(v, heads.cols), dq = of_head(dq, heads.rows), pz = of_head(pz, heads.nnz);
    using S = SpmmShape<T, D>;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave, R = kGroupRows;
    constexpr bool kScaled = std::is_same<T, __half>::value;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg][R][kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int grp = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (grp >= n_groups) return;
    if (groups[grp].len <= 0) return; // not a group: attention_backward_rows_kernel has its rows
    const RowGroup d = shared_run(groups[grp]); // the columns [lo, lo + len) that all four runs hold
    const int ls = lane % LPR, group = lane / LPR;
    const int row0 = grp * R;
    // dp along the run: LP lanes per v row, each with E of its 16-byte vectors (LP lanes apart), as in
    // attention_group_kernel: a dot product crosses half as many lanes
    constexpr int LP = LPR >= 8 ? LPR / 2 : LPR, E = LPR / LP;
    const int lp = lane % LP;
    typename DotVec<T>::Reg a[R][E][DotVec<T>::kRegs];
    int first[R]; // per row: the slot of column j of the shared run is first[r] + j
    float delta[R], g_scale[R], g_inv[R];
    RowStat stat[R];
#pragma unroll
    for (int r = 0; r < R; ++r) stat[r] = row_stat(stats, row0 + r);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float g_raw[E][VEC], part = 0.f, big = 0.f;
#pragma unroll
        for (int i = 0; i < E; ++i) {
            float o_raw[VEC];
            load_floats<VEC>(g + (size_t)(row0 + r) * D + (lp + LP * i) * VEC, g_raw[i]);
            load_floats<VEC>(out + (size_t)(row0 + r) * D + (lp + LP * i) * VEC, o_raw);
#pragma unroll
            for (int x = 0; x < VEC; ++x) part = fmaf(g_raw[i][x], o_raw[x], part);
            big = fmaxf(big, abs_max<VEC>(g_raw[i]));
        }
        delta[r] = butterfly_sum<1, LP>(part);
        g_scale[r] = g_inv[r] = 1.f;
        if constexpr (kScaled) {
            g_scale[r] = butterfly_max<1, LP>(big);
            g_inv[r] = g_scale[r] > 0.f ? 1.0f / g_scale[r] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < E; ++i) grad_regs<T>(g_raw[i], g_inv[r], a[r][i]);
        first[r] = row_ptr[row0 + r] + d.pos[r];
    }
    const T* k_lane = k + ls * VEC;
    const T* v_lane = v + ls * VEC;
    int* my_c = lds_c + wave * kWave;
    float acc[R][VEC];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[r][x] = 0.f;

    // the run: lane e of a step has column j0 + e
    const int group_first = lane - lp; // first column (within the step) of this lane group
    for (int j0 = 0; j0 < d.len; j0 += kWave) {
        const int j = j0 + lane;
        float dot[R];
#pragma unroll
        for (int r = 0; r < R; ++r) dot[r] = 0.f;
        if (j0 + (lane & 32) < d.len) { // the upper half sits out a step that has nothing for it
#pragma unroll
            for (int qd = 0; qd < LP / 4; ++qd) {
                float p4[R][4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    // (rows past the run repeat its last row)
                    const T* v_row = v + (size_t)(d.lo + min(j0 + group_first + 4 * qd + t, d.len - 1)) * D + lp * VEC;
#pragma unroll
                    for (int r = 0; r < R; ++r) p4[r][t] = 0.f;
#pragma unroll
                    for (int i = 0; i < E; ++i) {
                        const uint4 b = *reinterpret_cast<const uint4*>(v_row + LP * i * VEC);
#pragma unroll
                        for (int r = 0; r < R; ++r) p4[r][t] = DotVec<T>::dot_raw(a[r][i], b, p4[r][t]);
                    }
                }
                const bool hi2 = lp & 2, hi1 = lp & 1;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float q0 = (hi2 ? p4[r][2] : p4[r][0]) + lane_xor2(hi2 ? p4[r][0] : p4[r][2]);
                    const float q1 = (hi2 ? p4[r][3] : p4[r][1]) + lane_xor2(hi2 ? p4[r][1] : p4[r][3]);
                    float sum = (hi1 ? q1 : q0) + lane_xor1(hi1 ? q0 : q1);
                    sum = butterfly_sum<4, LP>(sum);
                    if ((lp >> 2) == qd) dot[r] = sum;
                }
            }
        }
        const bool live = j < d.len;
        float p[R], dz[R];
        int to[R]; // where the pairs of this column go: the four rows' slots in its row of the transposed pattern
#pragma unroll
        for (int r = 0; r < R; ++r) {
            p[r] = dz[r] = 0.f;
            to[r] = 0;
            if (live) {
                p[r] = stat[r].prob(probs[first[r] + j]);
                to[r] = t_slot[first[r] + j];
                dz[r] = scale * val[first[r] + j] * p[r] * (dot[r] * g_scale[r] - delta[r]);
            }
            lds_p[wave][r][lane] = dz[r];
        }
        if (live) {
            // four adjacent rows that hold one column are neighbours in that column's row of
            // the transposed pattern: their pairs leave as 32 consecutive bytes
            static_assert(R == 4, "the pairs of a group's four rows are stored together");
            if (to[1] == to[0] + 1 && to[2] == to[0] + 2 && to[3] == to[0] + 3) {
                typedef float Quad8 __attribute__((ext_vector_type(4), aligned(8)));
                Quad8* dst = reinterpret_cast<Quad8*>(pz + to[0]);
                dst[0] = Quad8{p[0], dz[0], p[1], dz[1]};
                dst[1] = Quad8{p[2], dz[2], p[3], dz[3]};
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r) pz[to[r]] = make_float2(p[r], dz[r]);
            }
        }
        wave_lds_sync();
        const int nq = min(kWave / 4, (d.len - j0 + 3) / 4);
#pragma unroll
        for (int i = 0; i < kWave / 4 / G; ++i) {
            const int qd = group + i * G;
            if (qd < nq) {
                const T* k_quad = k_lane + (size_t)(d.lo + j0 + 4 * qd) * D;
                const int room = d.len - 1 - (j0 + 4 * qd);
                float b[4][VEC];
#pragma unroll
                for (int t = 0; t < 4; ++t) DenseVec<T>::load(k_quad + (ptrdiff_t)min(t, room) * D, b[t]);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float4 z4 = *reinterpret_cast<const float4*>(&lds_p[wave][r][4 * qd]);
                    const float zv[4] = {z4.x, z4.y, z4.z, z4.w};
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int x = 0; x < VEC; ++x) acc[r][x] = fmaf(zv[t], b[t][x], acc[r][x]);
                }
            }
        }
        wave_lds_sync();
    }

    // the nonzeros outside the run, row by row: the slots before it and, in the same pass, those after it
    float* my_p = lds_p[wave][0];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int s = row_ptr[row0 + r], e = row_ptr[row0 + r + 1];
        const int split = d.pos[r], jump = d.len, cnt = e - s - jump;
        if (cnt <= 0) continue;
        float g_raw[VEC]; // this row of g as the lanes of sddmm_unit hold it
        load_floats<VEC>(g + (size_t)(row0 + r) * D + ls * VEC, g_raw);
        typename DotVec<T>::Reg a_row[1][DotVec<T>::kRegs];
        grad_regs<T>(g_raw, g_inv[r], a_row[0]);
        for (int off = 0; off < cnt; off += kWave) {
            const int slot = off + lane;
            const bool live_slot = slot < cnt;
            const int at = live_slot ? slot : cnt - 1;
            const int idx = s + at + (at >= split ? jump : 0);
            const int c = col[idx];
            const float w = val[idx], p = stat[r].prob(probs[idx]);
            float dz = 0.f;
            if (off + (lane & 32) < cnt) {
                const float dp = sddmm_unit<T, D, 1, false>(v_lane, a_row, c, D, my_c, lane) * g_scale[r];
                if (live_slot) dz = scale * w * p * (dp - delta[r]);
            }
            if (live_slot) pz[t_slot[idx]] = make_float2(p, dz);
            my_p[lane] = dz;
            wave_lds_sync();
            const int nlive = min(cnt - off, kWave);
            if (nlive == kWave)
                spmm_gather<T, D, 16 / G, true>(k_lane, (size_t)D, acc[r], my_c, my_p, group, G, 16);
            else
                spmm_gather<T, D, 16 / G, false>(k_lane, (size_t)D, acc[r], my_c, my_p, group, G, (nlive + 3) / 4);
            wave_lds_sync();
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[r][x] = butterfly_sum<LPR, kWave>(acc[r][x]);
        if (group == 0) store_floats<VEC>(dq + (size_t)(row0 + r) * D + ls * VEC, acc[r]);
    }
}

// ---- column pass ----------------------------------------------------------------------------
// Lane layout of the column pass for every operand type: D / 4 lanes per dense row, four
// elements each (g is fp32 whatever q is, and both feed accumulators of the same shape).
__device__ __forceinline__ void load4(const float* p, float (&out)[4]) { load_floats<4>(p, out); }
__device__ __forceinline__ void load4(const __half* p, float (&out)[4])
{
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    const float2 lo = __half22float2(*reinterpret_cast<const __half2*>(&raw.x));
    const float2 hi = __half22float2(*reinterpret_cast<const __half2*>(&raw.y));
    out[0] = lo.x; out[1] = lo.y; out[2] = hi.x; out[3] = hi.y;
}

// dv += p * g[row], dk += dz * q[row] over the slot quads {first_quad, first_quad + stride, ...}
// < nquads of a staged step (rows, p and dz of the slots in LDS).
template <typename T, int D, int QUADS_MAX, bool FULL>
__device__ __forceinline__ void cols_gather(const float* __restrict__ g_lane, const T* __restrict__ q_lane,
                                            float (&acc_v)[4], float (&acc_k)[4], const int* lds_row,
                                            const float* lds_p, const float* lds_z, int first_quad, int stride, int nquads)
{
#pragma unroll
    for (int i = 0; i < QUADS_MAX; ++i) {
        const int qd = first_quad + i * stride;
        if (FULL || qd < nquads) {
            const int4 r4 = *reinterpret_cast<const int4*>(lds_row + 4 * qd);
            const int r[4] = {r4.x, r4.y, r4.z, r4.w};
            float pv[4], zv[4], bg[4][4], bq[4][4];
            load_quad(lds_p + 4 * qd, pv);
            load_quad(lds_z + 4 * qd, zv);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                load4(g_lane + (size_t)r[t] * D, bg[t]);
                load4(q_lane + (size_t)r[t] * D, bq[t]);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    acc_v[x] = fmaf(pv[t], bg[t][x], acc_v[x]);
                    acc_k[x] = fmaf(zv[t], bq[t][x], acc_k[x]);
                }
        }
    }
}

// One wave per row of the transposed pattern (a column of the mask), 64 slots per step.
template <typename T, int D>
__global__ void __launch_bounds__(kWgThreads)
attention_backward_cols_kernel(int N, const int* __restrict__ t_row_ptr, const int* __restrict__ t_col,
                               const float2* __restrict__ pz, const float* __restrict__ g,
                               const T* __restrict__ q, float* __restrict__ dk, float* __restrict__ dv, RowOwners owners,
                               HeadStrides heads)
{
    // (rows / cols of the pattern itself: g and q have a row per row of it, dk and dv one per column)
    pz = of_head(pz, heads.nnz), g = of_head(g, heads.rows), q = of_head(q, heads.rows);
    dk = of_head(dk, heads.cols), dv = of_head(dv, heads.cols);
    constexpr int LPR = D / 4, G = kWave / LPR;
    __shared__ __attribute__((aligned(16))) int lds_r[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_z[kWavesPerWg * kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int c = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (c >= N) return;
    if (owned_elsewhere(owners, c, 0)) return; // a row of a group: attention_backward_cols_group_kernel has it
    const int s = t_row_ptr[c], e = t_row_ptr[c + 1];
    const int ls = lane % LPR, group = lane / LPR;
    float acc_v[4] = {0.f, 0.f, 0.f, 0.f}, acc_k[4] = {0.f, 0.f, 0.f, 0.f};
    int* my_r = lds_r + wave * kWave;
    float* my_p = lds_p + wave * kWave;
    float* my_z = lds_z + wave * kWave;
    const float* g_lane = g + ls * 4;
    const T* q_lane = q + ls * 4;
    for (int off = s; off < e; off += kWave) {
        const int slot = off + lane;
        const bool live = slot < e;
        const int idx = live ? slot : e - 1; // lanes past the end repeat the last slot with weights 0
        my_r[lane] = t_col[idx];
        const float2 x = live ? pz[idx] : make_float2(0.f, 0.f);
        my_p[lane] = x.x;
        my_z[lane] = x.y;
        wave_lds_sync();
        const int nlive = min(e - off, kWave);
        if (nlive == kWave)
            cols_gather<T, D, 16 / G, true>(g_lane, q_lane, acc_v, acc_k, my_r, my_p, my_z, group, G, 16);
        else
            cols_gather<T, D, 16 / G, false>(g_lane, q_lane, acc_v, acc_k, my_r, my_p, my_z, group, G, (nlive + 3) / 4);
        wave_lds_sync();
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        acc_v[x] = butterfly_sum<LPR, kWave>(acc_v[x]);
        acc_k[x] = butterfly_sum<LPR, kWave>(acc_k[x]);
    }
    if (group == 0) { // (a column without nonzeros gets zeros)
        store_floats<4>(dv + (size_t)c * D + ls * 4, acc_v);
        store_floats<4>(dk + (size_t)c * D + ls * 4, acc_k);
    }
}

// The groups of a group plan of the transposed pattern: four adjacent columns of the mask
// whose rows share a run [lo, lo + len).  One wave per group: along the run every row of g
// and of q is loaded once for the four columns; then the columns' other nonzeros, of the four
// together (spmm_group_kernel's walk, with two dense operands and two weights per slot).
template <typename T, int D>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
attention_backward_cols_group_kernel(int n_groups, const RowGroup* __restrict__ groups, const int* __restrict__ t_row_ptr,
                                     const int* __restrict__ t_col, const float2* __restrict__ pz, const float* __restrict__ g,
                                     const T* __restrict__ q, float* __restrict__ dk, float* __restrict__ dv, HeadStrides heads)
{
    pz = of_head(pz, heads.nnz), g = of_head(g, heads.rows), q = of_head(q, heads.rows);
    dk = of_head(dk, heads.cols), dv = of_head(dv, heads.cols);
    constexpr int LPR = D / 4, G = kWave / LPR, R = kGroupRows;
    __shared__ __attribute__((aligned(16))) int lds_r[kWavesPerWg][R][kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg][R][kWave];
    __shared__ __attribute__((aligned(16))) float lds_z[kWavesPerWg][R][kWave];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int grp = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (grp >= n_groups) return;
    if (groups[grp].len <= 0) return; // not a group: attention_backward_cols_kernel has its rows
    const RowGroup d = shared_run(groups[grp]);
    const int ls = lane % LPR, group = lane / LPR;
    const int c0 = grp * R;
    int at[R]; // per column: the slot of row lo + j of the shared run is at[i] + j
#pragma unroll
    for (int i = 0; i < R; ++i) at[i] = t_row_ptr[c0 + i] + d.pos[i];
    float acc_v[R][4], acc_k[R][4];
#pragma unroll
    for (int i = 0; i < R; ++i)
#pragma unroll
        for (int x = 0; x < 4; ++x) acc_v[i][x] = acc_k[i][x] = 0.f;
    const float* g_lane = g + ls * 4;
    const T* q_lane = q + ls * 4;

    float2 next[R]; // the weights of the next step are fetched while this one is computed
#pragma unroll
    for (int i = 0; i < R; ++i) next[i] = lane < d.len ? pz[at[i] + lane] : make_float2(0.f, 0.f);
    for (int j0 = 0; j0 < d.len; j0 += kWave) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            lds_p[wave][i][lane] = next[i].x;
            lds_z[wave][i][lane] = next[i].y;
        }
        wave_lds_sync();
        {
            const int j = j0 + kWave + lane;
#pragma unroll
            for (int i = 0; i < R; ++i) next[i] = j < d.len ? pz[at[i] + j] : make_float2(0.f, 0.f);
        }
        const int nq = min(kWave / 4, (d.len - j0 + 3) / 4);
#pragma unroll
        for (int u = 0; u < kWave / 4 / G; ++u) {
            const int qd = group + u * G;
            if (qd < nq) {
                // four consecutive rows of g and of q (the last quad of a run may be cut short: its
                // rows past the run repeat the run's last row, which all four columns reference;
                // their weights are zero)
                const size_t row = (size_t)(d.lo + j0 + 4 * qd);
                const int room = d.len - 1 - (j0 + 4 * qd);
                float bg[4][4], bq[4][4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    load4(g_lane + (row + min(t, room)) * D, bg[t]);
                    load4(q_lane + (row + min(t, room)) * D, bq[t]);
                }
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    float pv[4], zv[4];
                    load_quad(&lds_p[wave][i][4 * qd], pv);
                    load_quad(&lds_z[wave][i][4 * qd], zv);
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            acc_v[i][x] = fmaf(pv[t], bg[t][x], acc_v[i][x]);
                            acc_k[i][x] = fmaf(zv[t], bq[t][x], acc_k[i][x]);
                        }
                }
            }
        }
        wave_lds_sync();
    }

    // the nonzeros outside the run, of the four columns at once
    int row_first[R], split[R], cnt[R], max_cnt = 0;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        row_first[i] = t_row_ptr[c0 + i];
        split[i] = d.pos[i];
        cnt[i] = t_row_ptr[c0 + i + 1] - row_first[i] - d.len; // the slots before the run + those after it
        max_cnt = max(max_cnt, cnt[i]);
    }
    for (int off = 0; off < max_cnt; off += kWave) {
        const int slot = off + lane;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int live = min(cnt[i] - off, kWave); // this column's slots in this step (may be <= 0)
            int r = 0;
            float2 x = make_float2(0.f, 0.f);
            if (lane < ((live + 3) & ~3)) { // (slots past the end of the last quad: weights 0, row of a real slot)
                const bool past = slot >= cnt[i];
                const int slot_at = past ? cnt[i] - 1 : slot;
                const int idx = row_first[i] + slot_at + (slot_at >= split[i] ? d.len : 0);
                r = t_col[idx];
                if (!past) x = pz[idx];
            }
            lds_r[wave][i][lane] = r;
            lds_p[wave][i][lane] = x.x;
            lds_z[wave][i][lane] = x.y;
        }
        wave_lds_sync();
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int live = min(cnt[i] - off, kWave);
            if (live >= kWave)
                cols_gather<T, D, 16 / G, true>(g_lane, q_lane, acc_v[i], acc_k[i], lds_r[wave][i], lds_p[wave][i],
                                                lds_z[wave][i], group, G, 16);
            else if (live > 0)
                cols_gather<T, D, 16 / G, false>(g_lane, q_lane, acc_v[i], acc_k[i], lds_r[wave][i], lds_p[wave][i],
                                                 lds_z[wave][i], group, G, (live + 3) / 4);
        }
        wave_lds_sync();
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            acc_v[i][x] = butterfly_sum<LPR, kWave>(acc_v[i][x]);
            acc_k[i][x] = butterfly_sum<LPR, kWave>(acc_k[i][x]);
        }
        if (group == 0) {
            store_floats<4>(dv + (size_t)(c0 + i) * D + ls * 4, acc_v[i]);
            store_floats<4>(dk + (size_t)(c0 + i) * D + ls * 4, acc_k[i]);
        }
    }
}

// grid of one wave per item, a multiple of kXcds workgroups; -1: more than a launch holds
inline int wave_grid(long long items)
{
    long long wgs = (items + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds;
    return wgs * kWgThreads < (1ll << 32) ? (int)wgs : -1;
}

// (a group plan is used when a wave per group fills the GPU, as in the forward pass)
inline bool use_groups(const PlanRef& plan, int groups_min, RowOwners& owners)
{
    const bool grouped = plan.groups != nullptr && plan.group_counts != nullptr && plan.group_counts[1] >= groups_min;
    if (grouped) {
        owners.groups = reinterpret_cast<const RowGroup*>(plan.groups + kGroupHeaderInts);
        owners.n_groups = plan.group_counts[0];
    }
    return grouped;
}

template <typename T, int D>
hipError_t launch_rows(HeadStrides heads, int nheads, int M, const int* row_ptr, const int* col, const float* val,
                       const float* probs, const float2* stats, const float* g, const float* out, const T* k, const T* v,
                       float scale, const int* t_slot, float* dq, float* pz, PlanRef plan, hipStream_t stream)
{
    const int wgs = wave_grid(M);
    if (wgs < 0 || nheads > 65535) return hipErrorInvalidConfiguration;
    RowOwners owners;
    const bool grouped = use_groups(plan, attention_groups_min<T>(), owners);
    float2* pairs = reinterpret_cast<float2*>(pz);
    if (!(grouped && plan.group_counts[2] == 0)) // (else every row is in a group)
        attention_backward_rows_kernel<T, D><<<dim3(wgs, nheads), kWgThreads, 0, stream>>>(
            M, row_ptr, col, val, probs, stats, g, out, k, v, scale, t_slot, dq, pairs, owners, heads);
    if (grouped)
        attention_backward_group_kernel<T, D><<<dim3(wave_grid(owners.n_groups), nheads), kWgThreads, 0, stream>>>(
            owners.n_groups, owners.groups, row_ptr, col, val, probs, stats, g, out, k, v, scale, t_slot, dq, pairs, heads);
    return hipGetLastError();
}

template <typename T, int D>
hipError_t launch_cols(HeadStrides heads, int nheads, int N, const int* t_row_ptr, const int* t_col, const float* pz,
                       const float* g, const T* q, float* dk, float* dv, PlanRef plan, hipStream_t stream)
{
    const int wgs = wave_grid(N);
    if (wgs < 0 || nheads > 65535) return hipErrorInvalidConfiguration;
    RowOwners owners;
    const bool grouped = use_groups(plan, kAttentionColsGroupsMin, owners);
    const float2* pairs = reinterpret_cast<const float2*>(pz);
    if (!(grouped && plan.group_counts[2] == 0))
        attention_backward_cols_kernel<T, D><<<dim3(wgs, nheads), kWgThreads, 0, stream>>>(N, t_row_ptr, t_col, pairs, g, q, dk, dv,
                                                                                            owners, heads);
    if (grouped)
        attention_backward_cols_group_kernel<T, D><<<dim3(wave_grid(owners.n_groups), nheads), kWgThreads, 0, stream>>>(
            owners.n_groups, owners.groups, t_row_ptr, t_col, pairs, g, q, dk, dv, heads);
    return hipGetLastError();
}

} // namespace

// nheads problems on one pattern of M rows, N columns and nnz nonzeros (operands head after
// head); d: width of q, k, v, g and out (32, 64 or 128).  pz: nheads x 2 * nnz floats, the pairs
// (p, dz) in the order of the transposed pattern; t_slot: for every nonzero, its slot there.
template <typename T>
hipError_t attention_backward_rows_launch(int nheads, int M, int N, int nnz, int d, const int* row_ptr, const int* col,
                                          const float* val, const float* probs, const float* row_stats, const float* g,
                                          const float* out, const T* k, const T* v, float scale, const int* t_slot, float* dq,
                                          float* pz, PlanRef plan, hipStream_t stream)
{
    if (M <= 0 || nheads <= 0) return hipSuccess;
    const float2* stats = reinterpret_cast<const float2*>(row_stats);
    HeadStrides heads;
    heads.rows = (size_t)M * d, heads.cols = (size_t)N * d, heads.nnz = (size_t)nnz;
    switch (d) {
    case 32: return launch_rows<T, 32>(heads, nheads, M, row_ptr, col, val, probs, stats, g, out, k, v, scale, t_slot, dq, pz, plan, stream);
    case 64: return launch_rows<T, 64>(heads, nheads, M, row_ptr, col, val, probs, stats, g, out, k, v, scale, t_slot, dq, pz, plan, stream);
    case 128: return launch_rows<T, 128>(heads, nheads, M, row_ptr, col, val, probs, stats, g, out, k, v, scale, t_slot, dq, pz, plan, stream);
    default: return hipErrorInvalidValue;
    }
}

template <typename T>
hipError_t attention_backward_cols_launch(int nheads, int M, int N, int nnz, int d, const int* t_row_ptr, const int* t_col,
                                          const float* pz, const float* g, const T* q, float* dk, float* dv, PlanRef plan,
                                          hipStream_t stream)
{
    if (N <= 0 || nheads <= 0) return hipSuccess;
    HeadStrides heads;
    heads.rows = (size_t)M * d, heads.cols = (size_t)N * d, heads.nnz = (size_t)nnz;
    switch (d) {
    case 32: return launch_cols<T, 32>(heads, nheads, N, t_row_ptr, t_col, pz, g, q, dk, dv, plan, stream);
    case 64: return launch_cols<T, 64>(heads, nheads, N, t_row_ptr, t_col, pz, g, q, dk, dv, plan, stream);
    case 128: return launch_cols<T, 128>(heads, nheads, N, t_row_ptr, t_col, pz, g, q, dk, dv, plan, stream);
    default: return hipErrorInvalidValue;
    }
}

template hipError_t attention_backward_rows_launch<float>(int, int, int, int, int, const int*, const int*, const float*,
                                                          const float*, const float*, const float*, const float*, const float*,
                                                          const float*, float, const int*, float*, float*, PlanRef, hipStream_t);
template hipError_t attention_backward_rows_launch<__half>(int, int, int, int, int, const int*, const int*, const float*,
                                                           const float*, const float*, const float*, const float*, const __half*,
                                                           const __half*, float, const int*, float*, float*, PlanRef, hipStream_t);
template hipError_t attention_backward_cols_launch<float>(int, int, int, int, int, const int*, const int*, const float*,
                                                          const float*, const float*, float*, float*, PlanRef, hipStream_t);
template hipError_t attention_backward_cols_launch<__half>(int, int, int, int, int, const int*, const int*, const float*,
                                                           const float*, const __half*, float*, float*, PlanRef, hipStream_t);

} // namespace rode
