// C++ host API with the reference's signatures (RoDe_SDDMM/RoDeSddmm.h:4-9;
// cudaStream_t becomes hipStream_t).  Thin forwards to the C ABI in rode_hip.h.
#ifndef RODE_SDDMM_H_
#define RODE_SDDMM_H_

#include <hip/hip_runtime_api.h>

// k == 32; decomposition made with (seg 512, k_block 32, vec_len 4) in the reference.
void RoDeSDDMM_n32(int m1, int m2, int n, int k, const int* row_indices_block, const int* row_indices_residue,
                   const int* st_offsets, const int* row_offsets, const int* column_indices, const float* values,
                   const float* lhs_matrix, const float* rhs_matrix, float* out, hipStream_t stream1,
                   hipStream_t stream2);

// k == 128; decomposition made with (seg 32, k_block 32, vec_len 4) in the reference.
void RoDeSDDMM_n128(int m1, int m2, int n, int k, const int* row_indices_block, const int* row_indices_residue,
                    const int* st_offsets, const int* row_offsets, const int* column_indices, const float* values,
                    const float* lhs_matrix, const float* rhs_matrix, float* out, hipStream_t stream1,
                    hipStream_t stream2);

#endif
