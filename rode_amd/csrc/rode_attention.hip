// Sparse attention on a CSR pattern in one kernel:
//     out[r, :] = sum_idx p[idx] * v[col(idx), :],
//     p = softmax over the row of  scale * values[idx] * < q[r, :], k[col(idx), :] >
// i.e. SDDMM -> row softmax -> SpMM without the two nonzero-sized round trips through
// memory that the three separate kernels make (scores written and read, probabilities
// written and read, column indices read twice).  The reference has no such kernel: its op
// is the forward SDDMM alone (RoDe_SDDMM/rode_sddmm.py:194-248); this is the pipeline its
// attention benchmark configuration describes.
//
// One wave per row of the pattern, 64 slots per step:
//   * scores: the 32-slot unit of the SDDMM block kernel in both halves of the wave
//     (lane e ends up with the dot product of slot e);
//   * softmax: running maximum and running sum over the steps; when the maximum grows the
//     sum and the accumulated output row are rescaled by exp(old max - new max);
//   * output: (column, probability) of the step staged in LDS, then the gather-accumulate
//     of the SpMM block kernel over the lane groups, combined by a butterfly at the end.
// A softmax needs its whole row, so the row decomposition is not used here: rows are not
// split across waves, and a matrix with very long rows is better served by the three
// separate kernels (the Python layer chooses).  What the gradient needs is written out on
// request, in one of two forms.  Probabilities: the raw scores of a row's first 1024 slots
// wait in LDS (those of longer rows in the output array itself) until maximum and sum are
// known, then the lanes that produced them normalise and store them.  Scores: every score is
// stored as it is computed, and the row's (maximum, 1 / sum) pair at the end, so that a
// reader gets p = exp(score - maximum) * (1 / sum) without this kernel's second pass.
#include "rode_items.hpp"
#include "rode_units.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

__device__ __forceinline__ float wave_max_f(float v)
{
    v = fmaxf(v, lane_xor1(v));
    v = fmaxf(v, lane_xor2(v));
    v = fmaxf(v, lane_xor4(v));
    v = fmaxf(v, lane_xor8(v));
    v = fmaxf(v, lane_xor16(v));
    return fmaxf(v, lane_xor32(v));
}

// (four waves per SIMD: measured best on the attention-mask benchmark, 16384 rows of 570
// nonzeros, against 3, 5, 6 and 8; the registers that frees go to gathers in flight)
// Raw scores of a row that wait in LDS for the row's maximum and sum (per wave).
constexpr int kScoresKept = 1024;

// What a kernel leaves behind for the gradient.
enum Keep : int {
    kKeepNothing = 0,
    kKeepProbs = 1,  // probs[idx] = the probability
    kKeepScores = 2, // probs[idx] = the scaled score, stats[row] = (row maximum, 1 / row sum)
};

template <typename T, int D, int KEEP>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
attention_rows_kernel(int M, const int* __restrict__ row_ptr, const int* __restrict__ col, const float* __restrict__ val,
                      const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, float scale,
                      float* __restrict__ out, float* probs, float2* __restrict__ stats, RowOwners owners, HeadStrides heads)
{
    constexpr bool WRITE_P = KEEP == kKeepProbs;
    q = of_head(q, heads.rows), k = of_head(k, heads.cols), v = of_head(v, heads.cols);
    out = of_head(out, heads.rows), probs = of_head(probs, heads.nnz), stats = of_head(stats, heads.rows / D);
    using S = SpmmShape<T, D>;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg * kWave];
    __shared__ float lds_s[WRITE_P ? kWavesPerWg * kScoresKept : 1];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    const int row = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (row >= M) return;
    if (owned_elsewhere(owners, row, 0)) return; // a row of a group: attention_group_kernel has it
    const int s = row_ptr[row], e = row_ptr[row + 1];
    const int ls = lane % LPR, group = lane / LPR;
    float* out_lane = out + (size_t)row * D + ls * VEC;

    float acc[VEC];
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = 0.f;
    if (e <= s) { // a row without nonzeros attends to nothing
        if (group == 0) {
#pragma unroll
            for (int x = 0; x < VEC; x += 4) *reinterpret_cast<float4*>(out_lane + x) = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        if (KEEP == kKeepScores && lane == 0) stats[row] = make_float2(0.f, 0.f);
        return;
    }

    typename DotVec<T>::Reg a[1][DotVec<T>::kRegs];
    load_lhs_slice<T, D, 1, false>(q, row, D, lane, a);
    const T* k_lane = k + ls * VEC;
    const T* v_lane = v + ls * VEC;
    int* my_c = lds_c + wave * kWave;
    float* my_p = lds_p + wave * kWave;
    float* my_s = lds_s + (WRITE_P ? wave * kScoresKept : 0);

    float m_run = -INFINITY, l_lane = 0.f;
    for (int off = s; off < e; off += kWave) {
        const int slot = off + lane;
        const bool live = slot < e;
        const int idx = live ? slot : e - 1; // lanes past the row repeat its last slot with probability 0
        const int c = col[idx];
        const float w = val[idx];
        float sc = -INFINITY;
        if (off + (lane & 32) < e) { // the upper half sits out a step that has nothing for it
            const float d = sddmm_unit<T, D, 1, false>(k_lane, a, c, D, my_c, lane);
            if (live) sc = scale * (w * d);
        }
        const float m_new = fmaxf(m_run, wave_max_f(sc));
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float corr = __expf(m_run - m_safe);
        const float p = live ? __expf(sc - m_safe) : 0.f;
        l_lane = fmaf(l_lane, corr, p);
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[x] *= corr;
        m_run = m_new;
        if (WRITE_P && live) {
            if (slot - s < kScoresKept) my_s[slot - s] = sc; else probs[slot] = sc;
        }
        if (KEEP == kKeepScores && live) probs[slot] = sc;
        my_p[lane] = p;
        wave_lds_sync();
        const int nlive = min(e - off, kWave);
        if (nlive == kWave)
            spmm_gather<T, D, 16 / G, true>(v_lane, (size_t)D, acc, my_c, my_p, group, G, 16);
        else
            spmm_gather<T, D, 16 / G, false>(v_lane, (size_t)D, acc, my_c, my_p, group, G, (nlive + 3) / 4);
        wave_lds_sync();
    }

    const float inv = 1.0f / butterfly_sum<1, kWave>(l_lane);
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = butterfly_sum<LPR, kWave>(acc[x]) * inv;
    if (group == 0) {
#pragma unroll
        for (int x = 0; x < VEC; x += 4)
            *reinterpret_cast<float4*>(out_lane + x) = make_float4(acc[x], acc[x + 1], acc[x + 2], acc[x + 3]);
    }
    if (KEEP == kKeepScores && lane == 0) stats[row] = make_float2(m_run == -INFINITY ? 0.f : m_run, inv);
    if (WRITE_P) {
        // every lane normalises the scores it wrote itself
        const float m_safe = m_run == -INFINITY ? 0.f : m_run;
        for (int slot = s + lane; slot < e; slot += kWave) {
            const float sc = slot - s < kScoresKept ? my_s[slot - s] : probs[slot];
            probs[slot] = __expf(sc - m_safe) * inv;
        }
    }
}

// One step of the running softmax of a row: the scores of up to 64 slots (sc, -inf for a
// lane without a slot) move the maximum; the row's sum and accumulated output are rescaled.
// Returns this lane's probability relative to the new maximum.
template <int VEC>
__device__ __forceinline__ float softmax_step(float sc, bool live, float& m_run, float& l_lane, float (&acc)[VEC])
{
    const float m_new = fmaxf(m_run, wave_max_f(sc));
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __expf(m_run - m_safe);
    const float p = live ? __expf(sc - m_safe) : 0.f;
    l_lane = fmaf(l_lane, corr, p);
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] *= corr;
    m_run = m_new;
    return p;
}

// The groups of a group plan (rode_group.hip): one wave per group of four adjacent rows
// whose runs of consecutive columns overlap in a long shared run (shared_run).  Along it every
// k row and every v row is loaded once for the four rows (the score part is the SDDMM group kernel's, the output
// part the SpMM group kernel's, with a running softmax per row in between); then the wave
// takes the nonzeros outside the run, row by row, the way attention_rows_kernel does.
// Keeping probabilities, the raw scores of the first kGroupScoresKept columns of the run wait in
// LDS, the others in the probs array itself; the lanes that wrote them normalise them.
constexpr int kGroupScoresKept = 512;

template <typename T, int D, int KEEP>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
attention_group_kernel(int n_groups, const RowGroup* __restrict__ groups, const int* __restrict__ row_ptr,
                       const int* __restrict__ col, const float* __restrict__ val, const T* __restrict__ q,
                       const T* __restrict__ k, const T* __restrict__ v, float scale, float* __restrict__ out,
                       float* probs, float2* __restrict__ stats, HeadStrides heads)
{
    constexpr bool WRITE_P = KEEP == kKeepProbs;
    q = of_head(q, heads.rows), k = of_head(k, heads.cols), v = of_head(v, heads.cols);
    out = of_head(out, heads.rows), probs = of_head(probs, heads.nnz), stats = of_head(stats, heads.rows / D);
    using S = SpmmShape<T, D>;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave, R = kGroupRows;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg][R][kWave];
    __shared__ float lds_s[WRITE_P ? kWavesPerWg * R * kGroupScoresKept : 1];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave; // (uniform: scalar registers)
    float* my_s = lds_s + (WRITE_P ? wave * R * kGroupScoresKept : 0);
    const int g = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (g >= n_groups) return;
    if (groups[g].len <= 0) return; // not a group: attention_rows_kernel has its rows
    const RowGroup d = shared_run(groups[g]); // the columns [lo, lo + len) that all four runs hold
    const int ls = lane % LPR, group = lane / LPR;
    const int row0 = g * R;
    // the scores of the run: LP lanes per k row, each with E of its 16-byte vectors (LP lanes apart), as in
    // sddmm_group_kernel: a dot product crosses half as many lanes
    constexpr int LP = LPR >= 8 ? LPR / 2 : LPR, E = LPR / LP;
    const int lp = lane % LP;
    typename DotVec<T>::Reg a[R][E][DotVec<T>::kRegs];
    // per row: the slot of column j of the shared run is first[r] + j
    int first[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int i = 0; i < E; ++i) DotVec<T>::load(q + (size_t)(row0 + r) * D + (lp + LP * i) * VEC, a[r][i]);
        first[r] = row_ptr[row0 + r] + d.pos[r];
    }
    const T* k_lane = k + ls * VEC;
    const T* v_lane = v + ls * VEC;
    int* my_c = lds_c + wave * kWave;
    float m_run[R], l_lane[R], acc[R][VEC];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        m_run[r] = -INFINITY;
        l_lane[r] = 0.f;
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[r][x] = 0.f;
    }

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
                    // (rows past the range repeat its last row)
                    const T* k_row = k + (size_t)(d.lo + min(j0 + group_first + 4 * qd + t, d.len - 1)) * D + lp * VEC;
#pragma unroll
                    for (int r = 0; r < R; ++r) p4[r][t] = 0.f;
#pragma unroll
                    for (int i = 0; i < E; ++i) {
                        const uint4 b = *reinterpret_cast<const uint4*>(k_row + LP * i * VEC);
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
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const bool live = j < d.len;
            const float sc = live ? scale * (val[first[r] + j] * dot[r]) : -INFINITY;
            lds_p[wave][r][lane] = softmax_step<VEC>(sc, live, m_run[r], l_lane[r], acc[r]);
            if (WRITE_P && live) {
                if (j < kGroupScoresKept) my_s[r * kGroupScoresKept + j] = sc; else probs[first[r] + j] = sc;
            }
            if (KEEP == kKeepScores && live) probs[first[r] + j] = sc;
        }
        wave_lds_sync();
        const int nq = min(kWave / 4, (d.len - j0 + 3) / 4);
#pragma unroll
        for (int i = 0; i < kWave / 4 / G; ++i) {
            const int qd = group + i * G;
            if (qd < nq) {
                const T* v_quad = v_lane + (size_t)(d.lo + j0 + 4 * qd) * D;
                const int room = d.len - 1 - (j0 + 4 * qd);
                float b[4][VEC];
#pragma unroll
                for (int t = 0; t < 4; ++t) DenseVec<T>::load(v_quad + (ptrdiff_t)min(t, room) * D, b[t]);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float4 p4 = *reinterpret_cast<const float4*>(&lds_p[wave][r][4 * qd]);
                    const float pv[4] = {p4.x, p4.y, p4.z, p4.w};
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int x = 0; x < VEC; ++x) acc[r][x] = fmaf(pv[t], b[t][x], acc[r][x]);
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
        typename DotVec<T>::Reg a_row[1][DotVec<T>::kRegs]; // this row of q as the lanes of sddmm_unit hold it
        load_lhs_slice<T, D, 1, false>(q, row0 + r, D, lane, a_row);
        for (int off = 0; off < cnt; off += kWave) {
            const int slot = off + lane;
            const bool live = slot < cnt;
            const int at = live ? slot : cnt - 1;
            const int idx = s + at + (at >= split ? jump : 0);
            const int c = col[idx];
            const float w = val[idx];
            float sc = -INFINITY;
            if (off + (lane & 32) < cnt) {
                const float dd = sddmm_unit<T, D, 1, false>(k_lane, a_row, c, D, my_c, lane);
                if (live) sc = scale * (w * dd);
            }
            my_p[lane] = softmax_step<VEC>(sc, live, m_run[r], l_lane[r], acc[r]);
            if (KEEP != kKeepNothing && live) probs[idx] = sc;
            wave_lds_sync();
            const int nlive = min(cnt - off, kWave);
            if (nlive == kWave)
                spmm_gather<T, D, 16 / G, true>(v_lane, (size_t)D, acc[r], my_c, my_p, group, G, 16);
            else
                spmm_gather<T, D, 16 / G, false>(v_lane, (size_t)D, acc[r], my_c, my_p, group, G, (nlive + 3) / 4);
            wave_lds_sync();
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float inv = 1.0f / butterfly_sum<1, kWave>(l_lane[r]);
#pragma unroll
        for (int x = 0; x < VEC; ++x) acc[r][x] = butterfly_sum<LPR, kWave>(acc[r][x]) * inv;
        if (group == 0) {
            float* out_lane = out + (size_t)(row0 + r) * D + ls * VEC;
#pragma unroll
            for (int x = 0; x < VEC; x += 4)
                *reinterpret_cast<float4*>(out_lane + x) = make_float4(acc[r][x], acc[r][x + 1], acc[r][x + 2], acc[r][x + 3]);
        }
        if (KEEP == kKeepScores && lane == 0) stats[row0 + r] = make_float2(m_run[r] == -INFINITY ? 0.f : m_run[r], inv);
        if (WRITE_P) {
            // every lane normalises the scores it wrote itself: same walk over the run and over the rest
            const float m_safe = m_run[r] == -INFINITY ? 0.f : m_run[r];
            for (int j = lane; j < d.len; j += kWave) {
                const float sc = j < kGroupScoresKept ? my_s[r * kGroupScoresKept + j] : probs[first[r] + j];
                probs[first[r] + j] = __expf(sc - m_safe) * inv;
            }
            const int s = row_ptr[row0 + r], e = row_ptr[row0 + r + 1];
            const int split = d.pos[r], jump = d.len, cnt = e - s - jump;
            for (int slot = lane; slot < cnt; slot += kWave) {
                const int idx = s + slot + (slot >= split ? jump : 0);
                probs[idx] = __expf(probs[idx] - m_safe) * inv;
            }
        }
    }
}

template <typename T, int D>
hipError_t launch_rows(int nheads, int M, int N, int nnz, const int* row_ptr, const int* col, const float* val, const T* q,
                       const T* k, const T* v, float scale, float* out, float* probs, float2* stats, PlanRef plan,
                       hipStream_t stream)
{
    long long wgs = ((long long)M + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds;
    if (wgs * kWgThreads >= (1ll << 32) || nheads > 65535) return hipErrorInvalidConfiguration;
    HeadStrides heads;
    heads.rows = (size_t)M * D, heads.cols = (size_t)N * D, heads.nnz = (size_t)nnz;
    const Keep keep = probs == nullptr ? kKeepNothing : stats != nullptr ? kKeepScores : kKeepProbs;
    // a group plan is used when a wave per group fills the GPU
    RowOwners owners;
    const bool grouped = plan.groups != nullptr && plan.group_counts != nullptr && plan.group_counts[1] >= attention_groups_min<T>();
    if (grouped) {
        owners.groups = reinterpret_cast<const RowGroup*>(plan.groups + kGroupHeaderInts);
        owners.n_groups = plan.group_counts[0];
    }
    if (!(grouped && plan.group_counts[2] == 0)) { // (else every row is in a group)
        const dim3 grid((unsigned)wgs, (unsigned)nheads);
        if (keep == kKeepScores)
            attention_rows_kernel<T, D, kKeepScores><<<grid, kWgThreads, 0, stream>>>(M, row_ptr, col, val, q, k, v, scale, out,
                                                                                      probs, stats, owners, heads);
        else if (keep == kKeepProbs)
            attention_rows_kernel<T, D, kKeepProbs><<<grid, kWgThreads, 0, stream>>>(M, row_ptr, col, val, q, k, v, scale, out,
                                                                                     probs, stats, owners, heads);
        else
            attention_rows_kernel<T, D, kKeepNothing><<<grid, kWgThreads, 0, stream>>>(M, row_ptr, col, val, q, k, v, scale, out,
                                                                                       probs, stats, owners, heads);
    }
    if (grouped) {
        int gw = (owners.n_groups + kWavesPerWg - 1) / kWavesPerWg;
        gw = (gw + kXcds - 1) / kXcds * kXcds;
        const dim3 grid((unsigned)gw, (unsigned)nheads);
        if (keep == kKeepScores)
            attention_group_kernel<T, D, kKeepScores><<<grid, kWgThreads, 0, stream>>>(
                owners.n_groups, owners.groups, row_ptr, col, val, q, k, v, scale, out, probs, stats, heads);
        else if (keep == kKeepProbs)
            attention_group_kernel<T, D, kKeepProbs><<<grid, kWgThreads, 0, stream>>>(
                owners.n_groups, owners.groups, row_ptr, col, val, q, k, v, scale, out, probs, stats, heads);
        else
            attention_group_kernel<T, D, kKeepNothing><<<grid, kWgThreads, 0, stream>>>(
                owners.n_groups, owners.groups, row_ptr, col, val, q, k, v, scale, out, probs, stats, heads);
    }
    return hipGetLastError();
}

} // namespace

// nheads problems on one pattern (q, out: [nheads][M][d]; k, v: [nheads][N][d]; probs: NULL or
// [nheads][nnz]; row_stats: NULL or [nheads][M][2], and then probs receives the scaled scores
// and row_stats the (maximum, 1 / sum) of every row); d: width of q, k and v rows (32, 64 or 128).
template <typename T>
hipError_t attention_launch(int nheads, int M, int N, int nnz, int d, const int* row_ptr, const int* col, const float* val,
                            const T* q, const T* k, const T* v, float scale, float* out, float* probs, float* row_stats,
                            PlanRef plan, hipStream_t stream)
{
    if (M <= 0 || nheads <= 0) return hipSuccess;
    if (row_stats != nullptr && probs == nullptr) return hipErrorInvalidValue;
    float2* stats = reinterpret_cast<float2*>(row_stats);
    switch (d) {
    case 32: return launch_rows<T, 32>(nheads, M, N, nnz, row_ptr, col, val, q, k, v, scale, out, probs, stats, plan, stream);
    case 64: return launch_rows<T, 64>(nheads, M, N, nnz, row_ptr, col, val, q, k, v, scale, out, probs, stats, plan, stream);
    case 128: return launch_rows<T, 128>(nheads, M, N, nnz, row_ptr, col, val, q, k, v, scale, out, probs, stats, plan, stream);
    default: return hipErrorInvalidValue;
    }
}

template hipError_t attention_launch<float>(int, int, int, int, int, const int*, const int*, const float*, const float*,
                                            const float*, const float*, float, float*, float*, float*, PlanRef, hipStream_t);
template hipError_t attention_launch<__half>(int, int, int, int, int, const int*, const int*, const float*, const __half*,
                                             const __half*, const __half*, float, float*, float*, float*, PlanRef, hipStream_t);

} // namespace rode
