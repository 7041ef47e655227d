// NM-SpMM.h — C++ drop-in surface of the MI355X N:M sparse x dense fp32 library.
//
// Same free functions, argument order and argument meaning as the reference project's
// include/NM-SpMM.h:10-24, so a caller written against that header recompiles against this one
// and links libnmspmm.so instead of the CUDA objects.  Every function is a thin wrapper over
// the C-ABI in nmspmm.h (which returns status codes and takes a stream); use that layer directly
// when you need either.
//
// Conventions kept from the reference:
//   * the three preprocessing calls take HOST pointers and work in place;
//   * the eight launchers take DEVICE pointers, enqueue on the default stream and return at once;
//   * a launcher given a sparsity of the other family prints "Not support! ..." and does nothing;
//     a sparsity outside {0, 0.5, 0.625, 0.75, 0.875} does nothing;
//   * SPLIT_K == 1 overwrites C, SPLIT_K > 1 adds the product to what C holds (the reference
//     kernels' atomicAdd epilogue, src/kernel_64x128_8x8.cu:235-251): zero C before a split call.
//     Here the slices are summed in a fixed order through a workspace, so the result is
//     reproducible bit for bit.
#ifndef NM_SPMM_DROP_IN_H
#define NM_SPMM_DROP_IN_H

// The reference header brings the GPU runtime API to its includers (include/NM-SpMM.h:4-5 include
// <cuda.h> and <cuda_runtime.h>); this one brings HIP's, so a driver needs no include of its own.
#include <hip/hip_runtime.h>
#include <iostream>

// Adjacent columns of B that share one index pattern (reference include/NM-SpMM.h:8).
#define VEC_LEN (32)

// ---- index preprocessing (host pointers, in place) ---------------------------------------------

// Re-blocks the window-local index matrix index_rowmajor[W][Q] for column blocks of width Ns.
// Reference: include/NM-SpMM.h:10.
void PreProcessing_low_sparsity(int* index_rowmajor, int W, int Q, int Ns);

// Writes the per-(column block, window) lists of used rows to column_info, renumbers the
// indices to ranks and re-blocks them.  Reference: include/NM-SpMM.h:11.
void PreProcessing_high_sparsity(int* column_info, int pruning_M, int pruning_N, int* index_rowmajor,
                                 int W, int Q, int N, int Ns);

// Merges adjacent index windows pairwise and doubles both pattern counters.
// Reference: include/NM-SpMM.h:12.
void transIndex(int* index_rowmajor, int W, int N, int Q, int& pruning_N, int& pruning_M);

// ---- launchers (device pointers, default stream) -------------------------------------------------
// A: column-major M x K, B: row-major W x N compressed values, D: preprocessed indices,
// C: row-major M x N.  The name selects the column-block width the indices were preprocessed
// for: huge 128, large 64, medium 64, small 32.  Reference: include/NM-SpMM.h:14-24.

void nmGEMM_huge_matrices_low_sparsity(float* A, float* B, int* D, float* C,
                                       int M, int N, int K, int W, float sparsity, int SPLIT_K);
void nmGEMM_huge_matrices_high_sparsity(float* A, float* B, int* D, int* column_info, float* C,
                                        int M, int N, int K, int W, float sparsity, int SPLIT_K);

void nmGEMM_large_matrices_low_sparsity(float* A, float* B, int* D, float* C,
                                        int M, int N, int K, int W, float sparsity, int SPLIT_K);
void nmGEMM_large_matrices_high_sparsity(float* A, float* B, int* D, int* column_info, float* C,
                                         int M, int N, int K, int W, float sparsity, int SPLIT_K);

void nmGEMM_medium_matrices_low_sparsity(float* A, float* B, int* D, float* C,
                                         int M, int N, int K, int W, float sparsity, int SPLIT_K);
void nmGEMM_medium_matrices_high_sparsity(float* A, float* B, int* D, int* column_info, float* C,
                                          int M, int N, int K, int W, float sparsity, int SPLIT_K);

void nmGEMM_small_matrices_low_sparsity(float* A, float* B, int* D, float* C,
                                        int M, int N, int K, int W, float sparsity, int SPLIT_K);
void nmGEMM_small_matrices_high_sparsity(float* A, float* B, int* D, int* column_info, float* C,
                                         int M, int N, int K, int W, float sparsity, int SPLIT_K);

// ---- one launcher that chooses for the caller ----------------------------------------------------
// No counterpart in the reference, whose callers pick the tile and SPLIT_K by timing all of them
// (benchmark/kernel_performance/run_test/nmspmm/run_nmspmm.sh:19-36).  Indices must have been
// preprocessed for Ns = 128; the sparsity selects the low- or high-sparsity layout (column_info
// may be null for the former); the split of the reduction is chosen from the shape.
void nmGEMM(float* A, float* B, int* D, int* column_info, float* C,
            int M, int N, int K, int W, float sparsity);

#endif // NM_SPMM_DROP_IN_H
