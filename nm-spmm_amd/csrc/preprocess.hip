// Index preprocessing on the GPU (replaces the host loops of reference src/preprocessing.cu).
// All three kernels are pure int32 data movement and are HBM-bound; the outputs are bit-identical
// to the reference's.
#include "internal.h"

namespace nmspmm {

// transIndex (reference src/preprocessing.cu:3-15): rows of odd windows get +pM.
__global__ void __launch_bounds__(256)
trans_index_kernel(int32_t* __restrict__ DT, size_t total, int Q, int pN, int pM)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
        const size_t r = e / Q;
        if ((r / pN) & 1)
            DT[e] += pM;
    }
}

// The indices may still be the narrow n0:m0 windows they were generated with: `times` doublings of
// transIndex (reference src/preprocessing.cu:3-15) add m0 * ((r / n0) mod 2^times) to the index in
// compressed row r, which these kernels fold into their read instead of a pass of its own
// (times == 0: the indices are used as they are).
__device__ inline int widened(int v, size_t r, int n0, int m0, int times)
{
    return v + m0 * (int)((r / n0) & ((1u << times) - 1u));
}

// [W][Q] -> [Q/Qs][W][Qs] (reference src/preprocessing.cu:61-77,80-100).  Threads run along the
// output, which is written fully coalesced; reads come in runs of Qs int32.
__global__ void __launch_bounds__(256)
reblock_kernel(const int32_t* __restrict__ in, int32_t* __restrict__ out, int W, int Q, int Qs, int n0, int m0,
               int times)
{
    const size_t total = (size_t)W * Q;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const size_t per_block = (size_t)W * Qs;
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += stride) {
        const size_t jb = o / per_block;
        const size_t rem = o - jb * per_block;
        const size_t r = rem / Qs;
        const size_t c = rem - r * Qs;
        out[o] = widened(in[r * Q + jb * Qs + c], r, n0, m0, times);
    }
}

// PreProcessing_high_sparsity (reference src/preprocessing.cu:17-78).  One wave per
// (column block, window): the window's pN x Qs indices are marked in an LDS presence table, a
// ballot over the table gives each used row its rank (number of used rows below it), the wave
// writes the ascending row list padded with -1 to column_info and the ranks to the re-blocked
// index buffer.  pM <= 1024.
constexpr int kMaxWindow = 1024;

__global__ void __launch_bounds__(64)
preprocess_high_kernel(int32_t* __restrict__ cinfo, const int32_t* __restrict__ in,
                       int32_t* __restrict__ out, int W, int Q, int Qs, int pN, int pM, int nwin, int n0, int m0,
                       int times)
{
    __shared__ int present[kMaxWindow];
    __shared__ int rank[kMaxWindow];
    const int lane = threadIdx.x;
    const int w = blockIdx.x;
    const int jb = blockIdx.y;
    const int cells = pN * Qs;

    for (int x = lane; x < pM; x += 64)
        present[x] = 0;
    __syncthreads();
    for (int e = lane; e < cells; e += 64) {
        const int p = e / Qs, c = e - p * Qs;
        const size_t r = (size_t)w * pN + p;
        const int v = widened(in[r * Q + (size_t)jb * Qs + c], r, n0, m0, times);
        if ((unsigned)v < (unsigned)pM)  // malformed indices must not leave the table
            present[v] = 1;
    }
    __syncthreads();

    int32_t* ci = cinfo + ((size_t)jb * nwin + w) * pM;
    int base = 0;
    for (int x0 = 0; x0 < pM; x0 += 64) {
        const int x = x0 + lane;
        const bool used = x < pM && present[x] != 0;
        const unsigned long long mask = __ballot(used);
        const int below = __popcll(mask & ((1ull << lane) - 1ull));
        if (used) {
            rank[x] = base + below;
            ci[base + below] = x;
        }
        base += __popcll(mask);
    }
    for (int x = base + lane; x < pM; x += 64)
        ci[x] = -1;
    __syncthreads();

    for (int e = lane; e < cells; e += 64) {
        const int p = e / Qs, c = e - p * Qs;
        const size_t r = (size_t)w * pN + p;
        const int v = widened(in[r * Q + (size_t)jb * Qs + c], r, n0, m0, times);
        out[((size_t)jb * W + r) * Qs + c] = (unsigned)v < (unsigned)pM ? rank[v] : -1;
    }
}

static unsigned grid_for(size_t total)
{
    size_t blocks = (total + 255) / 256;
    if (blocks < 1)
        blocks = 1;
    if (blocks > 256 * 32)
        blocks = 256 * 32;
    return (unsigned)blocks;
}

hipError_t launch_trans_index(int32_t* dDT, int W, int Q, int pN, int pM, hipStream_t stream)
{
    const size_t total = (size_t)W * Q;
    hipLaunchKernelGGL(trans_index_kernel, dim3(grid_for(total)), dim3(256), 0, stream, dDT, total, Q, pN, pM);
    return hipGetLastError();
}

hipError_t launch_reblock(const int32_t* in, int32_t* out, int W, int Q, int Qs, int n0, int m0, int times,
                          hipStream_t stream)
{
    hipLaunchKernelGGL(reblock_kernel, dim3(grid_for((size_t)W * Q)), dim3(256), 0, stream, in, out, W, Q, Qs, n0,
                       m0, times);
    return hipGetLastError();
}

hipError_t launch_preprocess_high(int32_t* cinfo, int pM, int pN, const int32_t* in, int32_t* out,
                                  int W, int Q, int Qs, int n0, int m0, int times, hipStream_t stream)
{
    const int nwin = W / pN;
    hipLaunchKernelGGL(preprocess_high_kernel, dim3(nwin, Q / Qs), dim3(64), 0, stream, cinfo, in, out, W, Q,
                       Qs, pN, pM, nwin, n0, m0, times);
    return hipGetLastError();
}

} // namespace nmspmm
