// C++ host API with the reference's signatures for the row decomposition
// (Preprocess_opt/_preprocess.cu:323 GPU, :340 CPU twin; RoDe_SDDMM/main.cu:114-123).
#ifndef RODE_PREPROCESS_H_
#define RODE_PREPROCESS_H_

// GPU: every pointer is device memory.  block_r_ind needs room for
// (nnz + 3*M)/N_SEG + M entries, st_off one more (the sentinel st_off[n_blk] =
// row_ptr[M] is written, as main.cu:161-162 does), residue_r_ind M entries.
// Like the reference (_preprocess.cu:331,335) the call allocates and frees its
// own scratch; it runs on the default stream and returns without a host sync
// apart from that of the free.
void RoDe_preprocess(int N_SEG, int blockX, int vecLen, int M, const int* row_ptr, int* block_r_ind,
                     int* st_off, int* residue_r_ind, int* n_blk, int* n_res);

// Host-pointer twins: every pointer is HOST memory, the counts come back by reference, the
// call returns when the arrays are filled.  Same results as the reference's sequential
// loops, sentinel st_off[n_blk] = row_ptr[M] included (so st_off needs n_blk + 1 entries;
// _preprocess.cu:340-373 itself leaves it out, main.cu:161-162 writes it).  The
// decomposition runs on the current GPU (copy in, the kernels of the device routine, copy
// out): there is one implementation, not a second CPU one.
//
// Argument order of Preprocess_opt/_preprocess.cu:340: (segment length, k_block, vec_len).
void RoDe_preprocess_cpu(int N_SEG, int blockX, int vecLen, int M, const int* row_ptr, int* block_r_ind,
                         int* st_off, int* residue_r_ind, int& n_blk, int& n_res);
// Argument order of RoDe_SDDMM/main.cu:114-123 (and test.cu:73-82): (segment length,
// vec_len, k_block) -- note the swap.  Overloads the device routine above: the last two
// parameters are references here and device pointers there.
void RoDe_preprocess(int SegmentLength, int vectorLen, int KBLOCK, int M, const int* row_ptr, int* block_r_ind,
                     int* st_off, int* residue_r_ind, int& n_blk, int& n_res);

#endif
