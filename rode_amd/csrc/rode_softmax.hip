// Row softmax over the values of a CSR pattern (forward and backward), the step
// between SDDMM and SpMM in a sparse-attention pipeline:
//     p[idx] = exp(scale * s[idx] - max_row) / sum_row exp(scale * s - max_row)
//     ds[idx] = scale * p[idx] * (dp[idx] - sum_row(dp * p))
// The reference has no such kernel (its op is forward-only SDDMM,
// RoDe_SDDMM/rode_sddmm.py:194-248); this serves the pipeline its benchmark
// configuration describes.  One wave per row, lanes strided over the row's
// values, wave-wide max / sum by butterfly; HBM-bound (4 B read + 4 B written
// per nonzero, re-reads of a row come from L2).
#include "rode_device.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) v = fmaxf(v, __shfl_xor(v, m, kWave));
    return v;
}

__global__ void __launch_bounds__(kWgThreads)
csr_softmax_kernel(int M, const int* __restrict__ row_ptr, const float* in, float* out, float scale)
// in / out (and dp / ds below) may be the same array: no __restrict__ on them; every index
// is read and then written by the same lane
{
    const int lane = threadIdx.x % kWave;
    const int row = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + threadIdx.x / kWave;
    if (row >= M) return;
    const int s = row_ptr[row], e = row_ptr[row + 1];
    if (e <= s) return;
    float mx = -INFINITY;
    for (int i = s + lane; i < e; i += kWave) mx = fmaxf(mx, scale * in[i]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int i = s + lane; i < e; i += kWave) sum += __expf(scale * in[i] - mx);
    sum = butterfly_sum<1, kWave>(sum);
    const float inv = 1.0f / sum;
    for (int i = s + lane; i < e; i += kWave) out[i] = __expf(scale * in[i] - mx) * inv;
}

__global__ void __launch_bounds__(kWgThreads)
csr_softmax_backward_kernel(int M, const int* __restrict__ row_ptr, const float* __restrict__ p, const float* dp,
                            float* ds, float scale)
{
    const int lane = threadIdx.x % kWave;
    const int row = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + threadIdx.x / kWave;
    if (row >= M) return;
    const int s = row_ptr[row], e = row_ptr[row + 1];
    if (e <= s) return;
    float dot = 0.f;
    for (int i = s + lane; i < e; i += kWave) dot = fmaf(dp[i], p[i], dot);
    dot = butterfly_sum<1, kWave>(dot);
    for (int i = s + lane; i < e; i += kWave) ds[i] = scale * p[i] * (dp[i] - dot);
}

inline int grid_for_rows(int M)
{
    long long wgs = ((long long)M + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds;
    return wgs * kWgThreads < (1ll << 32) ? (int)wgs : -1; // a launch dimension holds fewer than 2^32 threads
}

} // namespace

hipError_t csr_softmax_launch(int M, const int* row_ptr, const float* in, float* out, float scale, hipStream_t stream)
{
    if (grid_for_rows(M) < 0) return hipErrorInvalidConfiguration;
    if (M > 0) csr_softmax_kernel<<<grid_for_rows(M), kWgThreads, 0, stream>>>(M, row_ptr, in, out, scale);
    return hipGetLastError();
}

hipError_t csr_softmax_backward_launch(int M, const int* row_ptr, const float* p, const float* dp, float* ds,
                                       float scale, hipStream_t stream)
{
    if (grid_for_rows(M) < 0) return hipErrorInvalidConfiguration;
    if (M > 0) csr_softmax_backward_kernel<<<grid_for_rows(M), kWgThreads, 0, stream>>>(M, row_ptr, p, dp, ds, scale);
    return hipGetLastError();
}

} // namespace rode
