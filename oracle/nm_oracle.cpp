// TEST INFRASTRUCTURE — not part of the shipped library.
//
// CPU restatement of the N:M sparse-times-dense path of M-H482/NM-SpMM, written from the
// algorithm (closed forms) rather than from the reference's loops, so that it can serve as an
// independent checker for the HIP library.  Only the test-suite, the smoke check and the
// cpu_baseline leg of the benchmark may load this file; the library never does.
//
// Every function names the reference lines whose behaviour it restates.  What pins each one
// (see tests/test_oracle_*.py):
//   nm_oracle_trans_index      closed form + decode invariant + oracle/_ref (compiled reference)
//   nm_oracle_preprocess_low   numpy transpose identity + oracle/_ref
//   nm_oracle_preprocess_high  sorted(set()) brute force, gather round trip + oracle/_ref
//   nm_oracle_gemm_cpu         dense fp64 GEMM of the decompressed operand + oracle/_ref (bit-exact)
//   nm_oracle_decompress       scatter/gather round trip
//   nm_oracle_compress         recovers generated (BT, DT) from their dense expansion, fp64 score
//                              dominance of kept over dropped rows, constructed ties, sign symmetry
//   nm_oracle_row_index        equals the generator's global rows (the D the reference's own CPU
//                              path multiplies with, include/utils.h:60) entry by entry, on every
//                              geometry and column-block width; padding entries are 0
// No function here is "parity unpinned".
//
// Vocabulary (reference include/utils.h:10-66, include/NM-SpMM.h:8):
//   W  compressed reduction length, Q = N / vec_len column vectors, pN kept rows per window of
//   pM rows.  DT is row-major int32[W][Q] with window-local indices; D is column-major
//   int32[W][Q] (element (k,a) at k + a*W) with global K indices; B is column-major
//   float[W][N] (element (k,j) at k + j*W); BT is row-major float[W][N]; A is column-major
//   float[M][K] (element (i,k) at i + k*M); C is row-major float[M][N].

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

extern "C" {

int nm_oracle_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

// Restates transIndex, reference src/preprocessing.cu:3-15.
// Every odd window of pN rows gets pM added to its indices, so two adjacent pN:pM windows
// become one 2pN:2pM window; both counters are doubled on return.
void nm_oracle_trans_index(int32_t* DT, int W, int Q, int* pruning_N, int* pruning_M)
{
    const int pN = *pruning_N, pM = *pruning_M;
    for (int64_t r = 0; r < W; ++r) {
        if (((r / pN) & 1) == 0)
            continue;
        int32_t* row = DT + r * Q;
        for (int a = 0; a < Q; ++a)
            row[a] += pM;
    }
    *pruning_N = 2 * pN;
    *pruning_M = 2 * pM;
}

// The re-blocking both preprocessing entry points end with, reference
// src/preprocessing.cu:61-77 and :80-100: [W][Q] -> [Q/Qs][W][Qs], Qs = Ns / vec_len.
static void reblock(int32_t* DT, int W, int Q, int Qs)
{
    std::vector<int32_t> out((size_t)W * Q);
    for (int jb = 0; jb < Q / Qs; ++jb)
        for (int64_t r = 0; r < W; ++r)
            for (int c = 0; c < Qs; ++c)
                out[((size_t)jb * W + r) * Qs + c] = DT[r * Q + (int64_t)jb * Qs + c];
    std::memcpy(DT, out.data(), out.size() * sizeof(int32_t));
}

// Restates PreProcessing_low_sparsity, reference src/preprocessing.cu:80-100.
void nm_oracle_preprocess_low(int32_t* DT, int W, int Q, int Ns, int vec_len)
{
    reblock(DT, W, Q, Ns / vec_len);
}

// Restates PreProcessing_high_sparsity, reference src/preprocessing.cu:17-78.
// Per (column block jb, window w): column_info[jb][w][0..pM) = ascending distinct window-local
// rows referenced by the block's pN x Qs indices, then -1; each index is replaced by its rank
// in that list; finally the same re-blocking as the low-sparsity entry.
void nm_oracle_preprocess_high(int32_t* column_info, int pM, int pN, int32_t* DT, int W, int Q,
                               int Ns, int vec_len)
{
    const int Qs = Ns / vec_len;
    const int nwin = W / pN;
    std::vector<int32_t> rank(pM);
    std::vector<char> used(pM);
    for (int jb = 0; jb < Q / Qs; ++jb) {
        for (int w = 0; w < nwin; ++w) {
            int32_t* ci = column_info + ((int64_t)jb * nwin + w) * pM;
            std::fill(used.begin(), used.end(), 0);
            for (int p = 0; p < pN; ++p)
                for (int c = 0; c < Qs; ++c)
                    used[DT[((int64_t)w * pN + p) * Q + jb * Qs + c]] = 1;
            int n = 0;
            for (int x = 0; x < pM; ++x) {
                if (used[x]) {
                    rank[x] = n;
                    ci[n++] = x;
                }
            }
            for (int x = n; x < pM; ++x)
                ci[x] = -1;
            for (int p = 0; p < pN; ++p)
                for (int c = 0; c < Qs; ++c) {
                    int32_t& v = DT[((int64_t)w * pN + p) * Q + jb * Qs + c];
                    v = rank[v];
                }
        }
    }
    reblock(DT, W, Q, Qs);
}

// Restates nmGEMM_on_cpu, reference include/utils.h:82-95, for rows [row_begin, row_end):
//   C[i][j] += A[i + D[k + (j/vec_len)*W]*M] * B[k + j*W], k ascending, one rounded multiply and
//   one rounded add per term (no fused multiply-add), accumulating into the caller's C.
// The per-element operation order is the reference's, so the result is bit-identical to it;
// only the memory walk differs (B is transposed once into row-major and rows of C are
// processed in blocks so that the operand streams stay in cache).
void nm_oracle_gemm_cpu(const float* A, const float* B, const int32_t* D, float* C, int M, int N,
                        int W, int vec_len, int row_begin, int row_end)
{
    const int Q = N / vec_len;
    std::vector<float> BT((size_t)W * N);
#pragma omp parallel for schedule(static)
    for (int k = 0; k < W; ++k)
        for (int j = 0; j < N; ++j)
            BT[(size_t)k * N + j] = B[(size_t)k + (size_t)j * W];

    const int RB = 8;
    const int nblk = (row_end - row_begin + RB - 1) / RB;
#pragma omp parallel for schedule(dynamic, 1)
    for (int blk = 0; blk < nblk; ++blk) {
        const int i0 = row_begin + blk * RB;
        const int i1 = std::min(i0 + RB, row_end);
        for (int k = 0; k < W; ++k) {
            const float* brow = BT.data() + (size_t)k * N;
            for (int a = 0; a < Q; ++a) {
                const float* acol = A + (size_t)D[(size_t)k + (size_t)a * W] * M;
                const float* bv = brow + (size_t)a * vec_len;
                for (int i = i0; i < i1; ++i) {
                    const float av = acol[i];
                    float* cv = C + (size_t)i * N + (size_t)a * vec_len;
                    for (int j = 0; j < vec_len; ++j) {
                        const float prod = av * bv[j];
                        cv[j] = cv[j] + prod;
                    }
                }
            }
        }
    }
}

// Expands the compressed operand to a dense row-major float[K][N]: row D[k + a*W] of column
// vector a receives B's compressed row k (the meaning of D and B in include/utils.h:56-61).
void nm_oracle_decompress(const float* B, const int32_t* D, float* dense, int K, int N, int W,
                          int vec_len)
{
    std::memset(dense, 0, sizeof(float) * (size_t)K * N);
    for (int j = 0; j < N; ++j) {
        const int a = j / vec_len;
        for (int k = 0; k < W; ++k)
            dense[(size_t)D[(size_t)k + (size_t)a * W] * N + j] = B[(size_t)k + (size_t)j * W];
    }
}

// Compresses a dense row-major float[K][N] operand to the format of include/utils.h:40-64 (BT
// row-major float[W][N], DT row-major int32[W][Q] window-local, ascending inside a window).  The
// reference has no such function; the rule restated here is the library's: per window of m rows
// and vector of vec_len columns, score(row) = sum of |b| over the vector, added pairwise in fp32
// (distance 1, 2, 4, ...), keep the n largest, ties to the lower row, scores ordered by bit
// pattern.
void nm_oracle_compress(const float* dense, int K, int N, int n, int m, int vec_len, float* BT, int32_t* DT)
{
    const int Q = N / vec_len;
    const int nwin = K / m;
#pragma omp parallel for schedule(static)
    for (int w = 0; w < nwin; ++w) {
        std::vector<float> part(vec_len);
        std::vector<uint32_t> key(m);
        std::vector<int> order(m);
        for (int a = 0; a < Q; ++a) {
            for (int r = 0; r < m; ++r) {
                const float* src = dense + ((size_t)w * m + r) * N + (size_t)a * vec_len;
                for (int c = 0; c < vec_len; ++c)
                    part[c] = src[c] < 0 ? -src[c] : src[c];
                for (int width = vec_len; width > 1; width /= 2)  // pairwise: (0,1) (2,3) ... then pairs of pairs
                    for (int c = 0; c < width / 2; ++c) {
                        volatile float t = part[2 * c] + part[2 * c + 1];
                        part[c] = t;
                    }
                std::memcpy(&key[r], &part[0], sizeof(uint32_t));
                order[r] = r;
            }
            std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return key[x] > key[y]; });
            std::sort(order.begin(), order.begin() + n);
            for (int p = 0; p < n; ++p) {
                const size_t row = (size_t)w * n + p;
                DT[row * Q + a] = order[p];
                const float* src = dense + ((size_t)w * m + order[p]) * N + (size_t)a * vec_len;
                std::memcpy(BT + row * N + (size_t)a * vec_len, src, sizeof(float) * vec_len);
            }
        }
    }
}

// The row list of the decode kernel (no reference counterpart; it restates how the reference
// kernels address a row of A: src/kernel_64x128_8x8.cu:75-77 for the low-sparsity layout,
// dense row = window * Ks + D[...]; :371 for the high-sparsity one, through column_info).
// D is the preprocessed blocked buffer [N/Ns][W][Ns/32], column_info [N/Ns][W/kept][window] or
// NULL.  R[(v * G + g) * 16 + kq * 4 + t] = 1 + dense row of kept row 16 g + 4 t + kq of vector v,
// 0 beyond W; G = ceil(W / 16).
void nm_oracle_row_index(const int32_t* D, const int32_t* column_info, int W, int N, int window, int kept, int Ns,
                         int32_t* R)
{
    const int Q = N / 32, Qs = Ns / 32, G = (W + 15) / 16, nwin = W / kept;
    for (int v = 0; v < Q; ++v) {
        const int jb = v / Qs, c = v % Qs;
        for (int g = 0; g < G; ++g)
            for (int kq = 0; kq < 4; ++kq)
                for (int t = 0; t < 4; ++t) {
                    const int r = 16 * g + 4 * t + kq;
                    int32_t out = 0;
                    if (r < W) {
                        const int w = r / kept;
                        int32_t local = D[((int64_t)jb * W + r) * Qs + c];
                        if (column_info)
                            local = column_info[((int64_t)jb * nwin + w) * window + local];
                        out = 1 + w * window + local;
                    }
                    R[((int64_t)v * G + g) * 16 + kq * 4 + t] = out;
                }
    }
}

} // extern "C"
