// TEST INFRASTRUCTURE — C-linkage doorway onto the reference project's own host code.
//
// This translation unit contains no algorithm.  It includes the reference's headers where they
// lie (the include path is given by oracle/Makefile) and is linked with the reference's
// src/preprocessing.cu compiled as plain C++, so that tests can call the reference's
// transIndex / PreProcessing_* / nmGEMM_on_cpu through ctypes.  The CUDA headers that
// NM-SpMM.h asks for are the genuine ones this image ships with its Triton wheel; nothing is
// stubbed.  Output goes to oracle/_ref/ only.
#include "NM-SpMM.h"
#include <cmath>
#include <cstdio>
#include <ctime>
#include "utils.h"

extern "C" {

int nmref_vec_len(void) { return VEC_LEN; }

void nmref_trans_index(int* DT, int W, int N, int Q, int* pruning_N, int* pruning_M)
{
    transIndex(DT, W, N, Q, *pruning_N, *pruning_M);
}

void nmref_preprocess_low(int* DT, int W, int Q, int Ns) { PreProcessing_low_sparsity(DT, W, Q, Ns); }

void nmref_preprocess_high(int* column_info, int pruning_M, int pruning_N, int* DT, int W, int Q,
                           int N, int Ns)
{
    PreProcessing_high_sparsity(column_info, pruning_M, pruning_N, DT, W, Q, N, Ns);
}

void nmref_gemm_cpu(float* A, float* B, int* D, float* C, int M, int N, int K, int W)
{
    nmGEMM_on_cpu(A, B, D, C, M, N, K, W);
}

int nmref_allclose(float* A, float* B, int n) { return allclose(A, B, n) ? 1 : 0; }

} // extern "C"
