// C++ drop-in functions of include/NM-SpMM.h, implemented on the C-ABI of include/nmspmm.h.
#include "../../include/NM-SpMM.h"
#include "../../include/nmspmm.h"

#include <cstdio>

namespace {

void report(const char* fn, int status)
{
    if (status != NMSPMM_OK)
        std::fprintf(stderr, "%s: %s\n", fn, nmspmm_status_string(status));
}

void low(const char* fn, int tile, float* A, float* B, int* D, float* C, int M, int N, int K, int W,
         float sparsity, int split_k)
{
    const int st = nmspmm_gemm_low_sparsity(tile, A, B, D, C, M, N, K, W, sparsity, split_k, nullptr);
    if (st == NMSPMM_ERR_WRONG_PATH)
        std::printf("Not support! Please use high sparsity version for sparsity %.3f\n", sparsity);
    else if (st != NMSPMM_ERR_BAD_PATTERN)  // an unknown sparsity is a silent no-op in the reference
        report(fn, st);
}

void high(const char* fn, int tile, float* A, float* B, int* D, int* column_info, float* C, int M, int N,
          int K, int W, float sparsity, int split_k)
{
    const int st =
        nmspmm_gemm_high_sparsity(tile, A, B, D, column_info, C, M, N, K, W, sparsity, split_k, nullptr);
    if (st == NMSPMM_ERR_WRONG_PATH)
        std::printf("Not support! Please use low sparsity version for sparsity %.2f\n", sparsity);
    else if (st != NMSPMM_ERR_BAD_PATTERN)
        report(fn, st);
}

} // namespace

void PreProcessing_low_sparsity(int* index_rowmajor, int W, int Q, int Ns)
{
    report("PreProcessing_low_sparsity", nmspmm_preprocess_low_host(index_rowmajor, W, Q, Ns, VEC_LEN));
}

void PreProcessing_high_sparsity(int* column_info, int pruning_M, int pruning_N, int* index_rowmajor, int W,
                                 int Q, int N, int Ns)
{
    report("PreProcessing_high_sparsity",
           nmspmm_preprocess_high_host(column_info, pruning_M, pruning_N, index_rowmajor, W, Q, N, Ns, VEC_LEN));
}

void transIndex(int* index_rowmajor, int W, int N, int Q, int& pruning_N, int& pruning_M)
{
    report("transIndex", nmspmm_trans_index_host(index_rowmajor, W, N, Q, &pruning_N, &pruning_M));
}

#define NMSPMM_DEFINE_PAIR(NAME, TILE)                                                                          \
    void nmGEMM_##NAME##_matrices_low_sparsity(float* A, float* B, int* D, float* C, int M, int N, int K,      \
                                               int W, float sparsity, int SPLIT_K)                             \
    {                                                                                                           \
        low("nmGEMM_" #NAME "_matrices_low_sparsity", TILE, A, B, D, C, M, N, K, W, sparsity, SPLIT_K);        \
    }                                                                                                           \
    void nmGEMM_##NAME##_matrices_high_sparsity(float* A, float* B, int* D, int* column_info, float* C, int M, \
                                                int N, int K, int W, float sparsity, int SPLIT_K)              \
    {                                                                                                           \
        high("nmGEMM_" #NAME "_matrices_high_sparsity", TILE, A, B, D, column_info, C, M, N, K, W, sparsity,   \
             SPLIT_K);                                                                                          \
    }

NMSPMM_DEFINE_PAIR(huge, NMSPMM_TILE_HUGE)
NMSPMM_DEFINE_PAIR(large, NMSPMM_TILE_LARGE)
NMSPMM_DEFINE_PAIR(medium, NMSPMM_TILE_MEDIUM)
NMSPMM_DEFINE_PAIR(small, NMSPMM_TILE_SMALL)

void nmGEMM(float* A, float* B, int* D, int* column_info, float* C, int M, int N, int K, int W, float sparsity)
{
    const int st = nmspmm_gemm_auto(A, B, D, column_info, C, M, N, K, W, sparsity, nullptr);
    if (st != NMSPMM_ERR_BAD_PATTERN)
        report("nmGEMM", st);
}
