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
// separate kernels (the Python layer chooses).  The probabilities are written out on
// request (the gradient needs them): the raw scores of a row's first 1024 slots wait in
// LDS (those of longer rows in the output array itself) until maximum and sum are known,
// then the lanes that produced them normalise and store them.
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

template <typename T, int D, bool WRITE_P>
__global__ void __launch_bounds__(kWgThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
attention_rows_kernel(int M, const int* __restrict__ row_ptr, const int* __restrict__ col, const float* __restrict__ val,
                      const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, float scale,
                      float* __restrict__ out, float* probs)
{
    using S = SpmmShape<T, D>;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_p[kWavesPerWg * kWave];
    __shared__ float lds_s[WRITE_P ? kWavesPerWg * kScoresKept : 1];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int row = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (row >= M) return;
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
        return;
    }

    float a[1][VEC];
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
    if (WRITE_P) {
        // every lane normalises the scores it wrote itself
        const float m_safe = m_run == -INFINITY ? 0.f : m_run;
        for (int slot = s + lane; slot < e; slot += kWave) {
            const float sc = slot - s < kScoresKept ? my_s[slot - s] : probs[slot];
            probs[slot] = __expf(sc - m_safe) * inv;
        }
    }
}

template <typename T, int D>
hipError_t launch_rows(int M, const int* row_ptr, const int* col, const float* val, const T* q, const T* k, const T* v,
                       float scale, float* out, float* probs, hipStream_t stream)
{
    long long wgs = ((long long)M + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds;
    if (wgs * kWgThreads >= (1ll << 32)) return hipErrorInvalidConfiguration;
    if (probs)
        attention_rows_kernel<T, D, true><<<(int)wgs, kWgThreads, 0, stream>>>(M, row_ptr, col, val, q, k, v, scale, out, probs);
    else
        attention_rows_kernel<T, D, false><<<(int)wgs, kWgThreads, 0, stream>>>(M, row_ptr, col, val, q, k, v, scale, out, probs);
    return hipGetLastError();
}

} // namespace

// d: width of q, k and v rows (32, 64 or 128).  probs: NULL or nnz floats.
template <typename T>
hipError_t attention_launch(int M, int d, const int* row_ptr, const int* col, const float* val, const T* q, const T* k,
                            const T* v, float scale, float* out, float* probs, hipStream_t stream)
{
    if (M <= 0) return hipSuccess;
    switch (d) {
    case 32: return launch_rows<T, 32>(M, row_ptr, col, val, q, k, v, scale, out, probs, stream);
    case 64: return launch_rows<T, 64>(M, row_ptr, col, val, q, k, v, scale, out, probs, stream);
    case 128: return launch_rows<T, 128>(M, row_ptr, col, val, q, k, v, scale, out, probs, stream);
    default: return hipErrorInvalidValue;
    }
}

template hipError_t attention_launch<float>(int, int, const int*, const int*, const float*, const float*, const float*,
                                            const float*, float, float*, float*, hipStream_t);
template hipError_t attention_launch<__half>(int, int, const int*, const int*, const float*, const __half*, const __half*,
                                             const __half*, float, float*, float*, hipStream_t);

} // namespace rode
