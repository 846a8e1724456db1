// SpMM over a row-decomposed CSR matrix:  C[row, :] += sum_idx values[idx] * B[col(idx), :]
// Same work split, index arithmetic and store/accumulate rules as the
// reference's SparseKernel::Kernel4Block (RoDe_SpMM/RoDeSpmm.cu:197-476) and
// Kernel4Residue (:41-195); the execution shape is written for 64-lane
// wavefronts:
//
//   * the dense tile is TN columns wide; LPR = TN / (elements per 128-bit load)
//     lanes cover one B row, so one load instruction of a wave gathers 64 / LPR
//     different B rows, each as full 128-bit coalesced reads;
//   * (col, value) pairs of up to 64 nonzero slots are staged in LDS with one
//     coalesced load per lane and read back four at a time as broadcasts;
//   * block kernel: one wave per block segment; its lane groups take
//     interleaved slot quads, the partial rows are combined with a butterfly
//     over the groups and added to C with hardware fp32 atomics (always, as in
//     RoDeSpmm.cu:464-474: a long row has several segments and usually a residue);
//   * residue kernel: one group of LPR lanes per residue row, 64 / LPR rows per
//     wave (short rows are latency-bound and need many rows in flight); rows
//     shorter than 32 slots are stored with plain 128-bit stores, tails of
//     longer rows are added atomically (RoDeSpmm.cu:76-82, 173-194).
//
// Slots that belong to the previous row (the `start & 3` head of an unaligned
// segment) are neutralised with value 0 *and* the column of the first real slot,
// so a non-finite B row can never leak into a row that does not reference it
// (the reference multiplies B[0, :] by zero there, RoDeSpmm.cu:271-274).
#include "rode_device.hpp"
#include "rode_internal.hpp"

namespace rode {

namespace {

template <typename T, int TN>
struct SpmmShape {
    static constexpr int kVec = DenseVec<T>::kElems;
    static constexpr int kLpr = TN / kVec;          // lanes that cover one B-row tile
    static constexpr int kGroupsWave = kWave / kLpr; // lane groups per wave
    static_assert(TN % kVec == 0 && kLpr >= 4 && kLpr <= 32 && (kLpr & (kLpr - 1)) == 0,
                  "unsupported tile width for this dense type");
};

// acc += sum over the slot quads {first_quad, first_quad + stride, ...} < nquads of
// value * B[col, tile].  QUADS_MAX bounds the trip count at compile time.
template <typename T, int TN, int QUADS_MAX, bool FULL>
__device__ __forceinline__ void spmm_gather(const T* __restrict__ b_lane, size_t ldb,
                                            float (&acc)[SpmmShape<T, TN>::kVec], const int* lds_col,
                                            const float* lds_val, int first_quad, int stride, int nquads)
{
    constexpr int VEC = SpmmShape<T, TN>::kVec;
#pragma unroll
    for (int i = 0; i < QUADS_MAX; ++i) {
        const int q = first_quad + i * stride;
        if (FULL || q < nquads) {
            const int4 c4 = *reinterpret_cast<const int4*>(lds_col + 4 * q);
            const float4 v4 = *reinterpret_cast<const float4*>(lds_val + 4 * q);
            const int c[4] = {c4.x, c4.y, c4.z, c4.w};
            const float v[4] = {v4.x, v4.y, v4.z, v4.w};
            float b[4][VEC];
#pragma unroll
            for (int j = 0; j < 4; ++j) DenseVec<T>::load(b_lane + (size_t)c[j] * ldb, b[j]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int x = 0; x < VEC; ++x) acc[x] = fmaf(v[j], b[j][x], acc[x]);
        }
    }
}

template <int VEC>
__device__ __forceinline__ void store_row(float* dst, const float (&acc)[VEC])
{
#pragma unroll
    for (int x = 0; x < VEC; x += 4)
        *reinterpret_cast<float4*>(dst + x) = make_float4(acc[x], acc[x + 1], acc[x + 2], acc[x + 3]);
}

// One wave per block segment (see sddmm_block_kernel for the slot arithmetic,
// identical at RoDeSpmm.cu:210-234).
template <typename T, int TN>
__global__ void __launch_bounds__(kWgThreads)
spmm_block_kernel(int m1, int n, const int* __restrict__ block_rows, const int* __restrict__ st_off,
                  const int* __restrict__ row_ptr, const int* __restrict__ col, const float* __restrict__ val,
                  const T* __restrict__ B, float* __restrict__ C)
{
    using S = SpmmShape<T, TN>;
    constexpr int VEC = S::kVec, LPR = S::kLpr, G = S::kGroupsWave;
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * kWave];
    __shared__ __attribute__((aligned(16))) float lds_v[kWavesPerWg * kWave];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int seg = xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave;
    if (seg >= m1) return;

    const int row = block_rows[seg];
    const int start = st_off[seg];
    const int end = min(row_ptr[row + 1], st_off[seg + 1]);
    const int mask = start & (kVecLen - 1);
    const int base = start - mask;
    const int cnt = (end - start + mask) / kBlockItems * kBlockItems;

    const int ls = lane % LPR, group = lane / LPR;
    const int tile = blockIdx.y * TN;
    const T* b_lane = B + tile + ls * VEC;
    int* my_c = lds_c + wave * kWave;
    float* my_v = lds_v + wave * kWave;

    float acc[VEC];
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = 0.f;

    for (int off = 0; off < cnt; off += kWave) {
        const int slot = off + lane;
        const int live = min(cnt - off, kWave); // 64, or 32 on a trailing half step
        int c = 0;
        float v = 0.f;
        if (lane < live) {
            const bool head = slot < mask; // previous row's slots
            c = col[base + (head ? mask : slot)];
            v = head ? 0.f : val[base + slot];
        }
        my_c[lane] = c;
        my_v[lane] = v;
        wave_lds_sync();
        if (live == kWave)
            spmm_gather<T, TN, 16 / G, true>(b_lane, (size_t)n, acc, my_c, my_v, group, G, 16);
        else
            spmm_gather<T, TN, 16 / G, false>(b_lane, (size_t)n, acc, my_c, my_v, group, G, live / 4);
        wave_lds_sync();
    }

    // combine the lane groups, then spread the atomics over them
    constexpr int EPG = VEC / G > 0 ? VEC / G : 1; // elements each group adds
    float* c_lane = C + (size_t)row * n + tile + ls * VEC;
#pragma unroll
    for (int x = 0; x < VEC; ++x) {
        const float total = butterfly_sum<LPR, kWave>(acc[x]);
        if (group == x / EPG) atomicAdd(c_lane + x, total);
    }
}

// One group of LPR lanes per residue row (tail selection: RoDeSpmm.cu:71-82); the
// group walks its row's slot quads one after the other, no cross-lane reduction.
template <typename T, int TN>
__global__ void __launch_bounds__(kWgThreads)
spmm_residue_kernel(int m2, int n, const int* __restrict__ residue_rows, const int* __restrict__ row_ptr,
                    const int* __restrict__ col, const float* __restrict__ val, const T* __restrict__ B,
                    float* __restrict__ C)
{
    using S = SpmmShape<T, TN>;
    constexpr int VEC = S::kVec, LPR = S::kLpr;
    constexpr int RPW = kWave / LPR;        // rows per wave
    constexpr int OWN = kBlockItems / LPR;  // slots staged by one lane
    __shared__ __attribute__((aligned(16))) int lds_c[kWavesPerWg * RPW * kBlockItems];
    __shared__ __attribute__((aligned(16))) float lds_v[kWavesPerWg * RPW * kBlockItems];
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int group = lane / LPR, ls = lane % LPR;
    const int item = (xcd_logical_block(blockIdx.x, gridDim.x) * kWavesPerWg + wave) * RPW + group;
    if (item >= m2) return;

    const int row = residue_rows[item];
    const int s = row_ptr[row], e = row_ptr[row + 1];
    const int pad = s & (kVecLen - 1);
    const int N = e - s + pad;
    int first = s, cnt = e - s;
    const bool accumulate = N >= kBlockItems; // the row also has block segments
    if (accumulate) {
        first = (s - pad) + N / kBlockItems * kBlockItems;
        cnt = N % kBlockItems;
    }

    const int tile = blockIdx.y * TN;
    int* my_c = lds_c + (wave * RPW + group) * kBlockItems;
    float* my_v = lds_v + (wave * RPW + group) * kBlockItems;

    float acc[VEC];
#pragma unroll
    for (int x = 0; x < VEC; ++x) acc[x] = 0.f;

    if (cnt > 0) {
        const int padded = (cnt + 3) & ~3; // slots past the tail repeat its last column with value 0
#pragma unroll
        for (int i = 0; i < OWN; ++i) {
            const int slot = ls + i * LPR;
            if (slot < padded) {
                my_c[slot] = col[first + min(slot, cnt - 1)];
                my_v[slot] = slot < cnt ? val[first + slot] : 0.f;
            }
        }
        wave_lds_sync();
        spmm_gather<T, TN, kBlockItems / 4, false>(B + tile + ls * VEC, (size_t)n, acc, my_c, my_v, 0, 1, padded / 4);
    }

    float* c_lane = C + (size_t)row * n + tile + ls * VEC;
    if (accumulate) {
#pragma unroll
        for (int x = 0; x < VEC; ++x) atomicAdd(c_lane + x, acc[x]);
    } else {
        store_row<VEC>(c_lane, acc);
    }
}

inline int grid_for_waves(long long nwaves)
{
    long long wgs = (nwaves + kWavesPerWg - 1) / kWavesPerWg;
    wgs = (wgs + kXcds - 1) / kXcds * kXcds; // xcd_logical_block needs a multiple of kXcds
    return (int)wgs;
}

template <typename T, int TN>
hipError_t launch(int m1, int m2, int n, const int* block_rows, const int* residue_rows, const int* st_off,
                  const int* row_ptr, const int* col, const float* val, const T* B, float* C, hipStream_t s1,
                  hipStream_t s2)
{
    const int tiles = n / TN;
    if (m1 > 0) {
        dim3 grid(grid_for_waves(m1), tiles);
        spmm_block_kernel<T, TN><<<grid, kWgThreads, 0, s1>>>(m1, n, block_rows, st_off, row_ptr, col, val, B, C);
    }
    if (m2 > 0) {
        constexpr int RPW = kWave / SpmmShape<T, TN>::kLpr;
        dim3 grid(grid_for_waves(((long long)m2 + RPW - 1) / RPW), tiles);
        spmm_residue_kernel<T, TN><<<grid, kWgThreads, 0, s2>>>(m2, n, residue_rows, row_ptr, col, val, B, C);
    }
    return hipGetLastError();
}

} // namespace

template <typename T>
hipError_t spmm_launch(int m1, int m2, int n, const int* block_rows, const int* residue_rows, const int* st_off,
                       const int* row_ptr, const int* col, const float* val, const T* B, float* C, hipStream_t s1,
                       hipStream_t s2)
{
    if (n <= 0 || n % 32 != 0) return hipErrorInvalidValue;
    if (n % 128 == 0) return launch<T, 128>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C, s1, s2);
    if (n % 64 == 0) return launch<T, 64>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C, s1, s2);
    return launch<T, 32>(m1, m2, n, block_rows, residue_rows, st_off, row_ptr, col, val, B, C, s1, s2);
}

template hipError_t spmm_launch<float>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                       const float*, const float*, float*, hipStream_t, hipStream_t);
template hipError_t spmm_launch<__half>(int, int, int, const int*, const int*, const int*, const int*, const int*,
                                        const float*, const __half*, float*, hipStream_t, hipStream_t);

} // namespace rode
