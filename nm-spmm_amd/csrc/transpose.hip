// Row-major -> column-major copy of the dense operand.  The multiplication kernels read A
// column-major (reference src/kernel_64x128_8x8.cu:15: M contiguous per k), while a model produces
// activations row-major (K contiguous per token); this HBM-bound tile transpose bridges the two.
// 64 x 64 tiles through LDS, 128-bit global accesses on both sides when the shape allows it.
#include "internal.h"

namespace nmspmm {

constexpr int kTile = 64;

// dst[c * dst_ld + r] = src[r * cols + c]; src is rows x cols.  VEC: cols and dst_ld are multiples
// of 4, dst_ld covers rows rounded up to 4 (the excess is written with zeros) and both pointers are
// 16-byte aligned.
template <bool VEC>
__global__ void __launch_bounds__(256)
transpose_kernel(const float* __restrict__ src, float* __restrict__ dst, int rows, int cols, int dst_ld)
{
    __shared__ float tile[kTile][kTile + 1];
    const int r0 = blockIdx.y * kTile, c0 = blockIdx.x * kTile;
    const int t = threadIdx.x;
    if (VEC) {
        const int q = (t & 15) * 4;  // 16 threads cover one 64-float row segment
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int r = pass * 16 + (t >> 4);
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (r0 + r < rows && c0 + q < cols)
                v = *reinterpret_cast<const float4*>(src + (size_t)(r0 + r) * cols + c0 + q);
            tile[r][q] = v.x;
            tile[r][q + 1] = v.y;
            tile[r][q + 2] = v.z;
            tile[r][q + 3] = v.w;
        }
        __syncthreads();
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int c = pass * 16 + (t >> 4);
            if (c0 + c < cols && r0 + q < rows) {
                const float4 v = make_float4(tile[q][c], tile[q + 1][c], tile[q + 2][c], tile[q + 3][c]);
                *reinterpret_cast<float4*>(dst + (size_t)(c0 + c) * dst_ld + r0 + q) = v;
            }
        }
    } else {
        const int x = t & 63;
        for (int r = t >> 6; r < kTile; r += 4)
            tile[r][x] = (r0 + r < rows && c0 + x < cols) ? src[(size_t)(r0 + r) * cols + c0 + x] : 0.0f;
        __syncthreads();
        for (int c = t >> 6; c < kTile; c += 4)
            if (c0 + c < cols && r0 + x < rows)
                dst[(size_t)(c0 + c) * dst_ld + r0 + x] = tile[x][c];
    }
}

hipError_t launch_transpose(const float* src, float* dst, int rows, int cols, int dst_ld, hipStream_t stream)
{
    const dim3 grid((cols + kTile - 1) / kTile, (rows + kTile - 1) / kTile), block(256);
    // a partial run of four rows at the bottom edge is stored whole: it lands in dst's padding
    const bool vec = cols % 4 == 0 && dst_ld % 4 == 0 && dst_ld >= (rows + 3) / 4 * 4 &&
                     ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
    if (vec)
        transpose_kernel<true><<<grid, block, 0, stream>>>(src, dst, rows, cols, dst_ld);
    else
        transpose_kernel<false><<<grid, block, 0, stream>>>(src, dst, rows, cols, dst_ld);
    return hipGetLastError();
}

} // namespace nmspmm
