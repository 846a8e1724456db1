// Device-side helpers shared by the RoDe kernels (gfx950 / CDNA4, wave64 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace rode {

constexpr int kWave = 64;         // lanes per wavefront
constexpr int kWavesPerWg = 4;    // every kernel here launches 256-thread workgroups
constexpr int kWgThreads = kWave * kWavesPerWg;
constexpr int kXcds = 8;          // MI355X: 8 XCDs, each with its own L2
constexpr int kBlockItems = 32;   // k_block the kernels are written for (RoDeSpmm.cu:513, RoDeSddmm.cu:517)
constexpr int kVecLen = 4;        // vec_len the kernels are written for (128-bit sparse loads)

// Workgroups are dealt round-robin to the XCDs, so neighbouring blockIdx values
// land on different L2s.  Remap so that a contiguous range of logical ids shares
// one XCD (neighbouring sparse rows touch neighbouring dense rows).  The grid
// must be a multiple of kXcds; ids past the item count are discarded by the
// caller's bounds check.
__device__ __forceinline__ int xcd_logical_block(int bid, int nblocks)
{
    const int per_xcd = nblocks / kXcds;
    return (bid % kXcds) * per_xcd + bid / kXcds;
}

// ---- cross-lane exchanges ------------------------------------------------
// xor 1 / xor 2 inside a quad: DPP quad_perm, full rate on the VALU.
__device__ __forceinline__ float lane_xor1(float v)
{
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1 /*[1,0,3,2]*/, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_xor2(float v)
{
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E /*[2,3,0,1]*/, 0xF, 0xF, true));
}
// xor 4 / 8 / 16: ds_swizzle in bit-mask mode (and=0x1f, or=0, xor=mask); no LDS memory is touched.
__device__ __forceinline__ float lane_xor4(float v)
{
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (4 << 10) | 0x1F));
}
__device__ __forceinline__ float lane_xor8(float v)
{
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (8 << 10) | 0x1F));
}
__device__ __forceinline__ float lane_xor16(float v)
{
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), (16 << 10) | 0x1F));
}
// xor 32: swap the two 32-lane halves of the wave.
__device__ __forceinline__ float lane_xor32(float v)
{
    return __shfl_xor(v, 32, kWave);
}

// Sum over the lanes l ^ m for every power of two m with LO <= m < HI.
// Every lane ends up with the total of its group.
template <int LO, int HI>
__device__ __forceinline__ float butterfly_sum(float v)
{
    if (LO <= 1 && 1 < HI) v += lane_xor1(v);
    if (LO <= 2 && 2 < HI) v += lane_xor2(v);
    if (LO <= 4 && 4 < HI) v += lane_xor4(v);
    if (LO <= 8 && 8 < HI) v += lane_xor8(v);
    if (LO <= 16 && 16 < HI) v += lane_xor16(v);
    if (LO <= 32 && 32 < HI) v += lane_xor32(v);
    return v;
}

__device__ __forceinline__ double lane_xor_any(double v, int m) { return __shfl_xor(v, m, kWave); }

template <int LO, int HI>
__device__ __forceinline__ double butterfly_sum(double v)
{
#pragma unroll
    for (int m = LO; m < HI; m <<= 1) v += lane_xor_any(v, m);
    return v;
}

// ---- dense operand access --------------------------------------------------
// One lane reads DenseVec<T>::kElems consecutive dense elements with a single
// 128-bit load and widens them to the accumulation type (fp32 for fp32 / fp16
// operands, fp64 for fp64 operands).
template <typename T>
struct DenseVec;

template <>
struct DenseVec<float> {
    using Acc = float;
    static constexpr int kElems = 4;
    __device__ __forceinline__ static void load(const float* p, float (&out)[4])
    {
        const float4 v = *reinterpret_cast<const float4*>(p);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    }
    // the same 16 bytes, already in registers (e.g. read back from an LDS copy of the row)
    __device__ __forceinline__ static void unpack(const uint4& raw, float (&out)[4])
    {
        out[0] = __uint_as_float(raw.x); out[1] = __uint_as_float(raw.y);
        out[2] = __uint_as_float(raw.z); out[3] = __uint_as_float(raw.w);
    }
};

template <>
struct DenseVec<double> {
    using Acc = double;
    static constexpr int kElems = 2;
    __device__ __forceinline__ static void load(const double* p, double (&out)[2])
    {
        const double2 v = *reinterpret_cast<const double2*>(p);
        out[0] = v.x; out[1] = v.y;
    }
};

template <>
struct DenseVec<__half> {
    using Acc = float;
    static constexpr int kElems = 8;
    __device__ __forceinline__ static void load(const __half* p, float (&out)[8])
    {
        unpack(*reinterpret_cast<const uint4*>(p), out);
    }
    __device__ __forceinline__ static void unpack(const uint4& raw, float (&out)[8])
    {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const __half2 h = *reinterpret_cast<const __half2*>(&w[i]);
            const float2 f = __half22float2(h);
            out[2 * i] = f.x;
            out[2 * i + 1] = f.y;
        }
    }
};

// The left operand of a dot product as a lane keeps it (DenseVec<T>::kElems elements), and
// its dot product with as many consecutive elements of the right operand, accumulated in
// fp32.  fp32: one fused multiply-add per element.  fp16: the pairs stay packed as loaded
// and go through v_dot2c_f32_f16 (two products, exact in fp32, and the sum per
// instruction; no conversion instructions).
template <typename T>
struct DotVec {
    using Reg = float;
    static constexpr int kRegs = DenseVec<T>::kElems;
    __device__ __forceinline__ static void zero(Reg (&a)[kRegs])
    {
#pragma unroll
        for (int x = 0; x < kRegs; ++x) a[x] = 0.f;
    }
    __device__ __forceinline__ static void load(const T* p, Reg (&a)[kRegs]) { DenseVec<T>::load(p, a); }
    // the same for a row that nobody reads again soon: loaded with the non-temporal hint
    __device__ __forceinline__ static void load_once(const T* p, Reg (&a)[kRegs])
    {
        typedef unsigned Quad __attribute__((ext_vector_type(4)));
        const Quad v = __builtin_nontemporal_load(reinterpret_cast<const Quad*>(p));
        DenseVec<T>::unpack(make_uint4(v[0], v[1], v[2], v[3]), a);
    }
    __device__ __forceinline__ static float dot_raw(const Reg (&a)[kRegs], const uint4& raw, float acc)
    {
        float b[kRegs];
        DenseVec<T>::unpack(raw, b);
#pragma unroll
        for (int x = 0; x < kRegs; ++x) acc = fmaf(a[x], b[x], acc);
        return acc;
    }
    __device__ __forceinline__ static float dot(const Reg (&a)[kRegs], const T* p, float acc)
    {
        return dot_raw(a, *reinterpret_cast<const uint4*>(p), acc);
    }
};

template <>
struct DotVec<__half> {
    using Reg = uint32_t; // two fp16 elements
    static constexpr int kRegs = 4;
    typedef _Float16 Pair __attribute__((ext_vector_type(2)));
    __device__ __forceinline__ static void zero(Reg (&a)[kRegs])
    {
#pragma unroll
        for (int x = 0; x < kRegs; ++x) a[x] = 0u;
    }
    __device__ __forceinline__ static void load(const __half* p, Reg (&a)[kRegs])
    {
        const uint4 raw = *reinterpret_cast<const uint4*>(p);
        a[0] = raw.x; a[1] = raw.y; a[2] = raw.z; a[3] = raw.w;
    }
    __device__ __forceinline__ static void load_once(const __half* p, Reg (&a)[kRegs])
    {
        typedef unsigned Quad __attribute__((ext_vector_type(4)));
        const Quad v = __builtin_nontemporal_load(reinterpret_cast<const Quad*>(p));
        a[0] = v[0]; a[1] = v[1]; a[2] = v[2]; a[3] = v[3];
    }
    __device__ __forceinline__ static float dot_raw(const Reg (&a)[kRegs], const uint4& raw, float acc)
    {
        const uint32_t b[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int x = 0; x < kRegs; ++x)
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(Pair, a[x]), __builtin_bit_cast(Pair, b[x]), acc, false);
        return acc;
    }
    __device__ __forceinline__ static float dot(const Reg (&a)[kRegs], const __half* p, float acc)
    {
        return dot_raw(a, *reinterpret_cast<const uint4*>(p), acc);
    }
};

// Make LDS writes of this wave visible to its other lanes.  A wave executes its
// LDS instructions in order, so only the compiler has to be kept from moving
// accesses across this point.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

} // namespace rode
