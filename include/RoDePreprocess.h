// C++ host API with the reference's signatures for the row decomposition
// (Preprocess_opt/_preprocess.cu:323 GPU, :340 CPU twin).
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

#endif
