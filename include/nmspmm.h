/*
 * nmspmm.h — C-ABI of the MI355X (gfx950) N:M sparse x dense fp32 matrix-multiply library.
 *
 * Plain pointers and sizes only; every function returns an nmspmm_status and never prints.
 * The C++ drop-in header NM-SpMM.h (same directory) is a thin layer over these entry points.
 *
 * Operands (the reference project's device layouts, src/kernel_64x128_8x8.cu:14-16):
 *   A            fp32, column-major M x K: element (i,k) at A[i + k*M]
 *   B            fp32, row-major   W x N: compressed values, W = K * kept / window
 *   D            int32, preprocessed indices, blocked [N/Ns][W][Ns/vec_len]
 *   column_info  int32, [N/Ns][W/kept][window], -1 padded (high-sparsity path only)
 *   C            fp32, row-major M x N
 * "window" is the number of dense K rows one index window spans (the M of N:M after any
 * widening), "kept" the number of rows kept in it, "vec_len" the number of adjacent columns of
 * B that share one index pattern, "Ns" the column-block width the indices were preprocessed for.
 *
 * Device pointers are HIP device pointers on the current device; `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  Launches are asynchronous.
 */
#ifndef NMSPMM_C_API_H
#define NMSPMM_C_API_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum nmspmm_status {
    NMSPMM_OK = 0,
    NMSPMM_ERR_NULL_POINTER = 1, /* a required pointer is NULL */
    NMSPMM_ERR_BAD_SHAPE = 2,    /* sizes are non-positive or violate a divisibility rule */
    NMSPMM_ERR_BAD_PATTERN = 3,  /* window / kept / vec_len / sparsity not representable */
    NMSPMM_ERR_WRONG_PATH = 4,   /* sparsity belongs to the other (low/high) entry point */
    NMSPMM_ERR_BAD_SPLIT = 5,    /* split_k < 1 or larger than the number of windows */
    NMSPMM_ERR_WORKSPACE = 6,    /* split_k > 1 and the workspace is missing or too small */
    NMSPMM_ERR_HIP = 7,          /* a HIP runtime call failed (no device, out of memory, ...) */
    NMSPMM_ERR_ALIGNMENT = 8     /* a pointer is not aligned as the kernels require (16 bytes) */
} nmspmm_status;

/* Column-block widths of the four named entry points of the reference API
 * (reference tests/test_nmspmm.cu:207-237: small 32, medium 64, large 64, huge 128). */
typedef enum nmspmm_tile {
    NMSPMM_TILE_SMALL = 32,
    NMSPMM_TILE_MEDIUM = 64,
    NMSPMM_TILE_LARGE = 64,
    NMSPMM_TILE_HUGE = 128
} nmspmm_tile;

int nmspmm_version(void);
const char* nmspmm_status_string(int status);

/* Maps a sparsity in {0, 0.5, 0.625, 0.75, 0.875} (matched within 1e-6, as the reference
 * launchers do, src/kernel_64x128_8x8.cu:264-289,584-602) to the window geometry the kernels
 * use: 0 -> 32/32, 0.5 -> 32/16, 0.625 -> 32/12 (low path), 0.75 -> 64/16, 0.875 -> 64/8
 * (high path).  *is_high is set to 1 for the high path.  Any other value:
 * NMSPMM_ERR_BAD_PATTERN. */
int nmspmm_pattern_from_sparsity(float sparsity, int* window, int* kept, int* is_high);

/* ---- index preprocessing ------------------------------------------------------------------ */

/* Replaces transIndex (reference include/NM-SpMM.h:12, src/preprocessing.cu:3-15): merges each
 * pair of adjacent windows of the row-major int32 DT[W][Q] by adding *pruning_M to the indices
 * of every odd window, then doubles *pruning_N and *pruning_M.  N is accepted for signature
 * parity and only checked against Q * vec_len.  Host-pointer form: DT is host memory, updated
 * in place (staged through the device, the work is done by the HIP kernel).  The three
 * host-pointer forms are synchronous and share one staging buffer per device, grown on demand and
 * kept until nmspmm_release(): concurrent calls from several threads are safe and take turns. */
int nmspmm_trans_index_host(int32_t* DT, int W, int N, int Q, int* pruning_N, int* pruning_M);
/* Device-pointer form of the same operation, in place on device memory, asynchronous. */
int nmspmm_trans_index_device(int32_t* dDT, int W, int N, int Q, int* pruning_N, int* pruning_M,
                              void* stream);

/* Replaces PreProcessing_low_sparsity (reference include/NM-SpMM.h:10,
 * src/preprocessing.cu:80-100): re-blocks DT[W][Q] to [Q/Qs][W][Qs], Qs = Ns / vec_len.
 * Host form works in place on host memory. */
int nmspmm_preprocess_low_host(int32_t* DT, int W, int Q, int Ns, int vec_len);
/* Device form: reads dDT_in, writes dDT_out (distinct buffers of W*Q int32). */
int nmspmm_preprocess_low_device(const int32_t* dDT_in, int32_t* dDT_out, int W, int Q, int Ns,
                                 int vec_len, void* stream);

/* Replaces PreProcessing_high_sparsity (reference include/NM-SpMM.h:11,
 * src/preprocessing.cu:17-78): per (column block, window) writes the ascending list of used
 * window-local rows to column_info (-1 padded to pruning_M), renumbers the indices to ranks in
 * that list, then re-blocks like the low form.  column_info must hold at least
 * nmspmm_column_info_ints() int32; only that many are written.  pruning_M <= 1024. */
int nmspmm_preprocess_high_host(int32_t* column_info, int pruning_M, int pruning_N, int32_t* DT,
                                int W, int Q, int N, int Ns, int vec_len);
int nmspmm_preprocess_high_device(int32_t* d_column_info, int pruning_M, int pruning_N,
                                  const int32_t* dDT_in, int32_t* dDT_out, int W, int Q, int N,
                                  int Ns, int vec_len, void* stream);

/* The whole preprocessing of a 32-column-vector pattern in one kernel: dDT_in holds the indices as
 * generated (n kept rows in every window of m, row-major int32[W][Q]); the transIndex doublings
 * that take the pattern to the kernels' window (reference tests/test_nmspmm.cu:72-79 calls them one
 * after the other) are folded into the re-blocking / ranking pass.  dD_out and, for the
 * high-sparsity geometries, d_column_info receive exactly what the separate calls produce;
 * *window and *kept are what nmspmm_spmm then takes.  dDT_in is not modified.  n/m must reduce to
 * 1/1, 1/2, 3/8, 1/4 or 1/8 with m a power-of-two fraction of the kernel window.  With vectors
 * of 4, 8 or 16 columns (N / Q below 32) the kernels take the window as generated: the call
 * re-blocks, *window = m, *kept = n, d_column_info is not used. */
int nmspmm_preprocess_device(const int32_t* dDT_in, int n, int m, int W, int Q, int N, int Ns,
                             int32_t* dD_out, int32_t* d_column_info, int* window, int* kept,
                             void* stream);

/* Number of int32 the high-sparsity preprocessing writes: (N/Ns) * (W/pruning_N) * pruning_M.
 * (The reference driver allocates one extra window of slack, tests/test_nmspmm.cu:23; this
 * library neither needs nor touches it.)  Returns 0 for invalid arguments. */
size_t nmspmm_column_info_ints(int W, int pruning_N, int pruning_M, int N, int Ns);

/* ---- dense <-> compressed operand ---------------------------------------------------------- */

/* No counterpart in the reference, which only synthesises operands that are already compressed
 * (reference include/utils.h:40-64); these produce and expand exactly that format.
 * nmspmm_compress_device: dB is the dense row-major float[K][N] operand.  In every window of m rows
 * and every vector of vec_len columns the n rows with the largest sum of |b| (added pairwise in
 * fp32: neighbours at distance 1, then 2, 4, ...; equal sums prefer the lower row) are kept:
 * dBT[W][N] receives their values, dDT[W][N/vec_len] their window-local row numbers, ascending,
 * W = K*n/m.  The output is what the preprocessing entry points above take.
 * nmspmm_decompress_device is the inverse: compressed row p of a window goes to the row its index
 * names (the indices of a window need not ascend; they are expected to be distinct), every other
 * row of the window becomes zero, and an index outside 0 .. m-1 stores nothing.
 * Requirements: m in {4, 8, 16, 32}, 0 < n < m, vec_len in {4, 8, 16, 32}, K % m == 0,
 * N % vec_len == 0, m * N * 4 bytes below 4 GiB, 16-byte aligned dB and dBT.  Asynchronous on
 * `stream`. */
int nmspmm_compress_device(const float* dB, int K, int N, int n, int m, int vec_len, float* dBT,
                           int32_t* dDT, void* stream);
int nmspmm_decompress_device(const float* dBT, const int32_t* dDT, int K, int N, int n, int m,
                             int vec_len, float* dB, void* stream);

/* ---- multiplication ----------------------------------------------------------------------- */

/* Bytes of device workspace nmspmm_spmm needs for a given split_k (0 when split_k <= 1):
 * split_k partial M x N fp32 results that a second pass sums in a fixed order. */
size_t nmspmm_workspace_bytes(int M, int N, int split_k);

/* General entry point: C = A . B for one (window, kept, vec_len, Ns) geometry.
 * column_info == NULL selects the low-sparsity layout (all window rows staged), non-NULL the
 * high-sparsity layout (only the rows column_info lists are staged, D holds ranks).
 * split_k > 1 requires `workspace` of at least nmspmm_workspace_bytes(); C is overwritten
 * whatever the split (the reference's atomicAdd reduction, include/ptx.h:34-40, adds to C when
 * SPLIT_K > 1: nmspmm_spmm_ex with NMSPMM_ACCUMULATE does that).  With
 * split_k == 1 the workspace is not used and may be NULL.
 * Requirements: N % Ns == 0, Ns % vec_len == 0, W % kept == 0, 1 <= split_k <= W / kept,
 * K * kept == W * window, 16-byte aligned A, B and C. */
int nmspmm_spmm(const float* A, const float* B, const int32_t* D, const int32_t* column_info,
                float* C, int M, int N, int K, int W, int window, int kept, int vec_len, int Ns,
                int split_k, void* workspace, size_t workspace_bytes, void* stream);

/* nmspmm_spmm with flags and the optional row list.
 * NMSPMM_ACCUMULATE: with split_k > 1 the sum of the reduction slices is added to what C holds,
 * C += A . B, exactly what the reference kernels do with their atomicAdd epilogue
 * (src/kernel_64x128_8x8.cu:235-242; deterministic here: C, then the slices in order); with
 * split_k == 1 C is overwritten, as in the reference (:243-251).
 * NMSPMM_STREAM_B: B is loaded with the non-temporal hint, for weights that will not be read again
 * before they would have left the caches anyway (a decode step walks through every layer of a
 * model: gigabytes between two uses of one B).  Only the decode kernel on the row list honours
 * it; measured there: faster when B comes from HBM, slower when a loop re-reads one B that fits
 * the 256 MB Infinity Cache.
 * NMSPMM_DECODE_SPLIT: with fewer 32-column vectors than the GPU has compute units (Ncols below
 * 8192 on an MI355X) the decode kernel on the row list leaves compute units idle; this flag lets it
 * cut each vector's reduction across several workgroups, the last of which to finish adds the
 * partial sums up in slice order (one launch, no workgroup waits for another, reproducible bit for
 * bit, safe to capture in a HIP graph and replay).  The partial sums and the arrival words live in
 * a device-resident array of the library (the one nmspmm_spmm_noalloc uses), one copy per GPU:
 * calls with this flag, and nmspmm_spmm_noalloc calls, that overlap on one GPU (two streams, two
 * threads) race on it, so the flag is for callers that issue their multiplications on one stream.
 * Nothing has to be cleared between calls, also not after a launch that was cut short: every
 * launch tags its arrivals with a number that is larger than any earlier launch's.  Measured:
 * K = 11008, Ncols = 4096 at 2:8, 1 / 16 / 32 rows 12.1 / 13.0 / 15.9 -> 11.0 / 12.3 / 13.2 us
 * re-reading one B, 16.6 / 20.7 / 20.4 -> 12.7 / 14.7 / 15.8 us with B from HBM; the library splits
 * only where the model expects a gain (long reductions, at most half as many vectors as compute
 * units).
 * Any other flag bit: NMSPMM_ERR_BAD_SHAPE.
 * row_index: NULL, or the row list nmspmm_row_index_device() made from these same D / column_info
 * (16-byte aligned).  With it, M <= 32 runs on the decode kernel that reads the list instead of
 * D and column_info, and so does M of 33 to 64 with column-major A wherever the library expects
 * one workgroup per vector to beat the tile kernel (short reductions, or few columns: K = Ncols =
 * 4096 at 64 rows 8.4 us on the list against 8.8 us on D / column_info at 2:8, 5.4 against 6.1 us
 * at 1:8), and M up to 128 on so few columns that its 32-row
 * parts get a workgroup each (one per 32 columns and part, at most as many as compute units:
 * Ncols <= 2048 on an MI355X); larger M ignore it. */
#define NMSPMM_ACCUMULATE 1u
#define NMSPMM_STREAM_B 2u
#define NMSPMM_DECODE_SPLIT 4u
int nmspmm_spmm_ex(const float* A, const float* B, const int32_t* D, const int32_t* column_info,
                   const int32_t* row_index, float* C, int M, int N, int K, int W, int window,
                   int kept, int vec_len, int Ns, int split_k, void* workspace,
                   size_t workspace_bytes, unsigned flags, void* stream);

/* No counterpart in the reference: a second, kernel-friendly form of the index metadata for the
 * memory-bound decode sizes, derived from the reference-layout buffers, which stay bit-exact and
 * remain what every other kernel reads.  The reference kernels find a row of A through two
 * dependent loads (the rank in D, then the window's column_info list, src/kernel_64x128_8x8.cu:371);
 * the row list holds the absolute dense row per (32-column vector, kept row):
 *   row_index[(v * G + g) * 16 + kq * 4 + t] = 1 + k(16 g + 4 t + kq, v),  0 where 16 g + 4 t + kq >= W
 * G = ceil(W / 16), v = column / 32, k(r, v) = (r / kept) * window + the window-local row that
 * D (through column_info on the high-sparsity layout) gives for kept row r of vector v.
 * nmspmm_row_index_ints: int32 the list holds, (N / 32) * G * 16 (0 for invalid arguments).
 * nmspmm_row_index_device: builds it on the GPU from D [N/Ns][W][Ns/32] and, when non-NULL,
 * column_info [N/Ns][W/kept][window]; vec_len is 32; asynchronous on `stream`. */
size_t nmspmm_row_index_ints(int W, int N);
int nmspmm_row_index_device(const int32_t* dD, const int32_t* d_column_info, int W, int N, int window,
                            int kept, int Ns, int32_t* d_row_index, void* stream);

/* No counterpart in the reference: the named launchers (nmGEMM_*_matrices_*_sparsity, nmGEMM,
 * nmspmm_gemm_low_sparsity / _high_sparsity / _auto) keep the reference's signatures, which have
 * no argument for the row list, so their decode-sized calls (M <= 128) run on D / column_info.
 * nmspmm_row_index_attach tells the library that `row_index` (device memory, made by
 * nmspmm_row_index_device from this D and its column_info) belongs to the index buffer that
 * starts at device address dD; from then on a named launcher that is handed this dD on this device
 * passes the list on, exactly as if the caller had called nmspmm_spmm_ex with it.  The caller keeps
 * both buffers alive and unchanged while attached; attaching again replaces the list; a NULL
 * row_index, nmspmm_row_index_detach, or nmspmm_release end it.  Thread-safe.  Returns
 * NMSPMM_ERR_NULL_POINTER for a NULL dD. */
int nmspmm_row_index_attach(const int32_t* dD, const int32_t* row_index);
int nmspmm_row_index_detach(const int32_t* dD);

/* No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  nmspmm_spmm with the
 * split-K slices in a fixed device-resident array of NMSPMM_NOALLOC_MAX_BYTES that belongs to the
 * library (each GPU the library runs on holds one such array from the first use of the library on
 * it until the process ends): no workspace argument, and no hipMalloc, hipFree or other
 * allocating call on any path.  nmspmm_workspace_bytes(M, N, split_k) beyond that size:
 * NMSPMM_ERR_WORKSPACE, nothing launched.  split_k == 1 uses no scratch at all.  C is
 * overwritten; results are bit-identical to nmspmm_spmm with a caller-owned workspace.  All calls
 * on a GPU share that GPU's array (the kernels overwrite every slice element they later read, so
 * nothing needs clearing between calls): split calls that overlap in time on one GPU, from
 * different streams or threads, race on it and must be serialised by the caller (so must they and
 * nmspmm_spmm_ex calls with NMSPMM_DECODE_SPLIT, which keep their partial sums in the same array). */
#define NMSPMM_NOALLOC_MAX_BYTES (32u << 20)
int nmspmm_spmm_noalloc(const float* A, const float* B, const int32_t* D, const int32_t* column_info,
                        float* C, int M, int N, int K, int W, int window, int kept, int vec_len,
                        int Ns, int split_k, void* stream);

/* Row-major A (M x K, K contiguous per row: activations as a model produces them).  No
 * counterpart: the reference kernels demand column-major A (reference
 * src/kernel_64x128_8x8.cu:15), i.e. a transpose before every layer.  nmspmm_transpose_device
 * writes dst[c][r] = src[r][c] for a rows x cols row-major src (so rows = M, cols = K turns a
 * row-major A into the layout nmspmm_spmm takes; one such copy serves every weight matrix that
 * multiplies the same activations).  nmspmm_spmm_rowmajor does both steps: the workspace holds the
 * column-major copy followed by the split-K slices, nmspmm_workspace_bytes_rowmajor() bytes, never
 * optional.  The copy's row pitch is M rounded up to 4 floats (the matrix-core kernels take any
 * pitch; this one keeps their 128-bit loads on 16-byte boundaries).  Up to 8 rows (decoding) the
 * kernel reads the row-major A in place and nothing is copied; the workspace is still required,
 * so that a caller sizes it once for every M.  Other arguments and requirements as nmspmm_spmm. */
int nmspmm_transpose_device(const float* src, int rows, int cols, float* dst, void* stream);
size_t nmspmm_workspace_bytes_rowmajor(int M, int N, int K, int split_k);
int nmspmm_spmm_rowmajor(const float* A_rowmajor, const float* B, const int32_t* D,
                         const int32_t* column_info, float* C, int M, int N, int K, int W, int window,
                         int kept, int vec_len, int Ns, int split_k, void* workspace,
                         size_t workspace_bytes, void* stream);
/* The same with the optional row list and the flags of nmspmm_spmm_ex (up to 8 rows the decode
 * kernel on the row list reads the row-major A in place, like the kernel it replaces). */
int nmspmm_spmm_rowmajor_ex(const float* A_rowmajor, const float* B, const int32_t* D,
                            const int32_t* column_info, const int32_t* row_index, float* C, int M,
                            int N, int K, int W, int window, int kept, int vec_len, int Ns,
                            int split_k, void* workspace, size_t workspace_bytes, unsigned flags,
                            void* stream);

/* Replace the reference launchers nmGEMM_{small,medium,large,huge}_matrices_low_sparsity
 * (reference include/NM-SpMM.h:14,17,20,23) and ..._high_sparsity (:15,18,21,24): `tile` is the
 * nmspmm_tile of the named entry point, `sparsity` selects the geometry as
 * nmspmm_pattern_from_sparsity does, vec_len is 32.  A sparsity that belongs to the other path
 * returns NMSPMM_ERR_WRONG_PATH (the reference prints "Not support!" there).  As in the reference,
 * split_k == 1 overwrites C and split_k > 1 adds the product to what C holds (NMSPMM_ACCUMULATE),
 * so a caller zeroes C before a split call.
 * Shared state: none when split_k == 1 (any number of streams and threads, and the call can be
 * recorded into a HIP graph).  When split_k > 1 the slices go to a per-device workspace that the
 * library grows on demand (hipMalloc, so not under graph capture unless an earlier call has
 * already grown it to the size) and keeps until nmspmm_release(); split calls that share a device
 * must be issued on one stream at a time, or they overwrite each other's slices. */
int nmspmm_gemm_low_sparsity(int tile, const float* A, const float* B, const int32_t* D, float* C,
                             int M, int N, int K, int W, float sparsity, int split_k, void* stream);
int nmspmm_gemm_high_sparsity(int tile, const float* A, const float* B, const int32_t* D,
                              const int32_t* column_info, float* C, int M, int N, int K, int W,
                              float sparsity, int split_k, void* stream);

/* No counterpart in the reference, which leaves tile and SPLIT_K to the caller and finds them by
 * exhaustive timing (benchmark/kernel_performance/run_test/nmspmm/run_nmspmm.sh:19-36,
 * benchmark/different_kernel/search_shape/search_shape.sh:16-43).  On this hardware the
 * column-block width does not change the speed (waves are independent), so only the split is
 * chosen: nmspmm_suggest_split_k returns the split_k the library would use for a shape (1..16;
 * 0 for invalid arguments); nmspmm_gemm_auto multiplies with that choice and the per-device
 * workspace, for indices preprocessed with Ns = 128 (NMSPMM_TILE_HUGE); `sparsity` selects the
 * geometry and the layout as nmspmm_pattern_from_sparsity does, column_info is required for the
 * high-sparsity layout and ignored otherwise. */
int nmspmm_suggest_split_k(int M, int N, int W, int kept);
/* No counterpart in the reference.  Rows per workgroup (128 or 64) when an unsplit multiplication
 * (split_k == 1) of this shape on the matrix-core kernel is computed with the reduction shared
 * between the four waves of each workgroup and added up in LDS (problems of few tiles; no
 * workspace, one launch), 0 when it is computed tile by tile or the arguments are invalid.
 * Informational: the choice is the library's. */
int nmspmm_waves_along_k_rows(int M, int N, int W, int kept);
/* No counterpart in the reference.  Waves of each workgroup of that launch (4 or 8: with eight, a
 * compute unit holds half as many workgroups, each with twice the waves), 0 where
 * nmspmm_waves_along_k_rows returns 0.  Informational. */
int nmspmm_waves_along_k_count(int M, int N, int W, int kept);
/* No counterpart in the reference.  Rows that an unsplit multiplication of this shape on the
 * matrix-core kernel hands to the decode-sized kernels: the last 1 to 32 rows of a row count a
 * little above a multiple of 128, where the library expects the tile kernel's extra layer of
 * 128-row workgroups to cost more than reading B once more; 0 otherwise.  Informational. */
int nmspmm_rows_apart(int M, int N, int W, int kept);
/* No counterpart in the reference.  What the library's planning (split choice, wave height, tile
 * walk) assumes about the current device: compute units, accelerator dies (each with its own L2)
 * and shader clock, read from the HIP runtime once per device; the figures of an MI355X
 * (256, 8, 2.4e9) when there is no device.  Any pointer may be NULL. */
int nmspmm_device_figures(int* compute_units, int* dies, double* clock_hz);

/* No counterpart in the reference.  Rows of C one wave of the matrix-core tile kernel covers for
 * this shape, column-block width and split (256, 128 or 64; a workgroup is four waves: 1 x 4,
 * 2 x 2 or 4 x 1 rows x column vectors for Ns = 128, 64, 32), 0 when the call takes the launch
 * with waves along K (nmspmm_waves_along_k_rows) or the arguments are invalid.  Informational,
 * for profiles and benchmarks that want to name the kernel instance that ran. */
int nmspmm_tile_wave_rows(int M, int N, int W, int kept, int Ns, int split_k);
/* No counterpart in the reference.  Sets of four waves per workgroup of the matrix-core tile
 * kernel for this shape: 2 when a whole unsplit problem is at most one workgroup of 256-row waves
 * per compute unit and long enough along K (each set then takes half of the windows and the halves
 * are added up in LDS), 1 otherwise, 0 where nmspmm_tile_wave_rows returns 0.  Informational. */
int nmspmm_tile_wave_sets(int M, int N, int W, int kept, int Ns, int split_k);
int nmspmm_gemm_auto(const float* A, const float* B, const int32_t* D, const int32_t* column_info,
                     float* C, int M, int N, int K, int W, float sparsity, void* stream);

/* Frees what the library keeps per device: the cached split-K workspaces and the staging buffer
 * of the host-pointer preprocessing forms; forgets every attached row list. */
int nmspmm_release(void);

/* Name of the kernel family the last successful nmspmm_spmm call on this thread dispatched to
 * ("mfma", "short", "gather", "skinny", "decode", "simt"), for tests and profiles; where a call
 * hands its last 1 to 32 rows to another family than the rest, the family of the rest.  Never NULL. */
const char* nmspmm_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* NMSPMM_C_API_H */
