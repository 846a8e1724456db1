// C++ host API with the reference's signatures (RoDe_SpMM/RoDeSpmm.h:4-8;
// cudaStream_t becomes hipStream_t).  Thin forwards to the C ABI in rode_hip.h.
#ifndef RODE_SPMM_H_
#define RODE_SPMM_H_

#include <hip/hip_runtime_api.h>

// C[M x n] += A * B with 32-wide dense tiles in the reference (n % 32 == 0).
void RoDeSpmm_n32(int m1, int m2, int k, int n, const float* values, const int* column_indices,
                  const int* row_offsets, const int* row_indices1, const int* row_indices2,
                  const int* row_seg_st_offsets, const float* B, float* C, hipStream_t stream1,
                  hipStream_t stream2);

// Same with 64-wide dense tiles in the reference (n % 64 == 0).
void RoDeSpmm_n128(int m1, int m2, int k, int n, const float* values, const int* column_indices,
                   const int* row_offsets, const int* row_indices1, const int* row_indices2,
                   const int* row_seg_st_offsets, const float* B, float* C, hipStream_t stream1,
                   hipStream_t stream2);

// fp64 overloads (RoDe_SpMM/RoDeSpmm.h:10-14).
void RoDeSpmm_n32(int m1, int m2, int k, int n, const double* values, const int* column_indices,
                  const int* row_offsets, const int* row_indices1, const int* row_indices2,
                  const int* row_seg_st_offsets, const double* B, double* C, hipStream_t stream1,
                  hipStream_t stream2);

void RoDeSpmm_n128(int m1, int m2, int k, int n, const double* values, const int* column_indices,
                   const int* row_offsets, const int* row_indices1, const int* row_indices2,
                   const int* row_seg_st_offsets, const double* B, double* C, hipStream_t stream1,
                   hipStream_t stream2);

#endif
