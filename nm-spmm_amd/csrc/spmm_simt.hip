// Generic SIMT kernel and the split-K reduction pass.
//
// The SIMT kernel accepts every geometry the C-ABI admits (any window / kept, vec_len 4..32, any
// M including M not divisible by 4), so that shapes the matrix-core tiles do not cover still run
// on the GPU.  One wave handles 64 rows of C for one column vector: lanes run along M, so the
// gathered reads A[i + k*M] are coalesced 256-byte rows and the B / index reads are
// wave-uniform.  Semantics are those of the reference's nmGEMM_on_cpu (include/utils.h:82-95)
// expressed on the device layouts (row-major B, blocked window-local D, optional column_info).
#include "internal.h"

namespace nmspmm {

struct SimtParams {
    const float* A;
    const float* B;
    const int32_t* D;
    const int32_t* cinfo;
    float* out;
    size_t slice_elems;
    int M, N, W;
    int window, kept, Qs, nwin, split_k;
};

template <int VL>
__global__ void __launch_bounds__(64) spmm_simt_kernel(const SimtParams p)
{
    const int a = blockIdx.x;             // column vector
    const int i = blockIdx.y * 64 + threadIdx.x;
    const int jb = a / p.Qs, c = a % p.Qs;  // column block and vector inside it
    int w_begin, w_count;
    split_windows(p.nwin, p.split_k, blockIdx.z, &w_begin, &w_count);

    float acc[VL];
#pragma unroll
    for (int x = 0; x < VL; ++x)
        acc[x] = 0.0f;

    const bool live = i < p.M;
    const float* Arow = p.A + (live ? i : 0);
    const float* Bcol = p.B + (size_t)a * VL;
    const int32_t* Dblk = p.D + (size_t)jb * p.W * p.Qs + c;

    for (int w = w_begin; w < w_begin + w_count; ++w) {
        const int32_t* ci = p.cinfo ? p.cinfo + ((size_t)jb * p.nwin + w) * p.window : nullptr;
        for (int u = 0; u < p.kept; ++u) {
            const int k = w * p.kept + u;
            int local = Dblk[(size_t)k * p.Qs];
            if (ci)
                local = ci[local];
            const float av = Arow[(size_t)(w * p.window + local) * p.M];
            const float* brow = Bcol + (size_t)k * p.N;
#pragma unroll
            for (int x = 0; x < VL; ++x)
                acc[x] = fmaf(av, brow[x], acc[x]);
        }
    }
    if (live) {
        float* o = p.out + (size_t)blockIdx.z * p.slice_elems + (size_t)i * p.N + (size_t)a * VL;
#pragma unroll
        for (int x = 0; x < VL; ++x)
            o[x] = acc[x];
    }
}

bool simt_supported(const SpmmArgs& a)
{
    if (a.a_rowmajor)
        return false;
    return a.vec_len == 4 || a.vec_len == 8 || a.vec_len == 16 || a.vec_len == 32;
}

hipError_t launch_simt(const SpmmArgs& a)
{
    SimtParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.window = a.window;
    p.kept = a.kept;
    p.Qs = a.Ns / a.vec_len;
    p.nwin = a.W / a.kept;
    p.split_k = a.split_k;
    dim3 grid(a.N / a.vec_len, (a.M + 63) / 64, a.split_k);
    switch (a.vec_len) {
    case 32: hipLaunchKernelGGL(spmm_simt_kernel<32>, grid, dim3(64), 0, a.stream, p); break;
    case 16: hipLaunchKernelGGL(spmm_simt_kernel<16>, grid, dim3(64), 0, a.stream, p); break;
    case 8: hipLaunchKernelGGL(spmm_simt_kernel<8>, grid, dim3(64), 0, a.stream, p); break;
    case 4: hipLaunchKernelGGL(spmm_simt_kernel<4>, grid, dim3(64), 0, a.stream, p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// C[e] = partial[0][e] + partial[1][e] + ... in slice order (deterministic, unlike atomics); with
// ACC the chain starts from what C[e] holds, as the reference's atomicAdd reduction into the
// caller's C does (include/ptx.h:34-40, src/kernel_64x128_8x8.cu:235-242).
template <bool ACC>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float* __restrict__ partial, float* __restrict__ C, size_t elems,
                     size_t slice_stride, int split_k)
{
    const size_t n4 = elems / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n4; e += stride) {
        float4 s = reinterpret_cast<const float4*>(partial)[e];
        if (ACC) {
            const float4 c = reinterpret_cast<const float4*>(C)[e];
            s.x = c.x + s.x;
            s.y = c.y + s.y;
            s.z = c.z + s.z;
            s.w = c.w + s.w;
        }
        for (int z = 1; z < split_k; ++z) {
            const float4 v = reinterpret_cast<const float4*>(partial + (size_t)z * slice_stride)[e];
            s.x += v.x;
            s.y += v.y;
            s.z += v.z;
            s.w += v.w;
        }
        reinterpret_cast<float4*>(C)[e] = s;
    }
    // tail (elems not a multiple of 4)
    if (blockIdx.x == 0 && threadIdx.x < (elems & 3)) {
        const size_t e = n4 * 4 + threadIdx.x;
        float s = ACC ? C[e] + partial[e] : partial[e];
        for (int z = 1; z < split_k; ++z)
            s += partial[(size_t)z * slice_stride + e];
        C[e] = s;
    }
}

hipError_t launch_splitk_reduce(const float* partial, float* C, size_t elems, size_t slice_stride,
                                int split_k, bool accumulate, hipStream_t stream)
{
    const size_t n4 = elems / 4;
    size_t blocks = (n4 + 255) / 256;
    if (blocks < 1)
        blocks = 1;
    if (blocks > 256 * 16)
        blocks = 256 * 16;
    if (accumulate)
        hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, stream, partial, C,
                           elems, slice_stride, split_k);
    else
        hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, stream, partial, C,
                           elems, slice_stride, split_k);
    return hipGetLastError();
}

} // namespace nmspmm
