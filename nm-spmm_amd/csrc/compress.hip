// Compression of a dense operand to the N:M vector-sparse format and back.  The reference only
// synthesises operands that are already compressed (include/utils.h:40-64); these kernels produce
// and expand exactly that format: BT row-major float[W][N] (W = K*n/m kept rows), DT row-major
// int32[W][Q] of window-local row numbers, one per kept row and L-column vector.
//
// Selection rule: in every window of m rows and every vector of L columns, the score of a row is
// the sum of |b| over the vector's L columns, added pairwise in fp32 (neighbours at distance 1,
// then 2, 4, ... L/2); the n rows with the largest scores are kept, equal scores prefer the lower
// row; scores are ordered by their bit patterns, so NaNs rank above everything instead of
// breaking the order.  Both kernels are HBM-bound: every global access is a coalesced run of
// 16-byte segments of one row.
#include "internal.h"

namespace nmspmm {

// One thread owns four adjacent columns (a 16-byte segment of every row), so a vector of L columns
// is a group of L/4 lanes: the first two levels of the pairwise sum happen inside the thread, the
// remaining ones by lane exchange.
constexpr int kColsPerBlock = 1024;

typedef unsigned int cuintx4 __attribute__((ext_vector_type(4)));
typedef float cfloatx4 __attribute__((ext_vector_type(4)));

// The dense operand (compressing) and the compressed one (expanding) are read once, the compressed
// values are written once: non-temporal 16-byte accesses.  With B from HBM the compression runs 3 to
// 20 % faster with the loads (4096 x 4096 at 2:8: 0.52 -> 0.62 of 8 TB/s) and the 2:4 cases another
// 10 % with the stores.
__device__ inline float4 load_streaming(const float* p)
{
    const cfloatx4 x = __builtin_nontemporal_load(reinterpret_cast<const cfloatx4*>(p));
    return make_float4(x[0], x[1], x[2], x[3]);
}
__device__ inline void store_streaming(float* p, float4 v)
{
    const cfloatx4 x = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(x, reinterpret_cast<cfloatx4*>(p));
}

// The expanded operand is stored system-coherent (sc1, bit 4 of the cache-policy operand): written
// through, the stores leave no dirty lines in L2 for the end of the launch to flush, which makes
// the expansion 4 to 20 % shorter (4096 x 4096 at 2:8: 12.4 -> 10.0 us); the compression, which
// writes less than it reads, gains nothing from it.  (The non-temporal bit on top of it: 1 to 8 %
// faster into HBM, 10 to 30 % slower while the expanded operand stays in the Infinity Cache for its
// consumer: not set.)  `base` is the same for
// the whole workgroup: the rows of one window, `bytes` long.
__device__ inline void store_segment(float* base, uint32_t bytes, uint32_t offset_bytes, float4 v)
{
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)bytes, 0x00020000);
    const cuintx4 x = {__float_as_uint(v.x), __float_as_uint(v.y), __float_as_uint(v.z), __float_as_uint(v.w)};
    __builtin_amdgcn_raw_buffer_store_b128(x, rs, (int)offset_bytes, 0, 16);
}

template <int MW>
__global__ void __launch_bounds__(256)
compress_kernel(const float* __restrict__ B, float* __restrict__ BT, int32_t* __restrict__ DT, int N, int Q,
                int n, int L, int col_blocks)
{
    // consecutive workgroups take neighbouring column blocks of one window: what runs at the same
    // time reads and writes whole rows
    const int w = blockIdx.x / col_blocks;
    const int col = (blockIdx.x % col_blocks) * kColsPerBlock + threadIdx.x * 4;
    const bool active = col < N;  // whole vectors are active or not: N and 1024 are multiples of L
    const int lane = threadIdx.x & 63;
    const int G = L / 4;                // lanes per vector
    const int c = lane & (G - 1);       // position inside the group
    const int group = lane & ~(G - 1);  // first lane of the group

    float4 v[MW];
    uint32_t key[MW];
#pragma unroll
    for (int r = 0; r < MW; ++r)
        v[r] = active ? load_streaming(B + ((size_t)w * MW + r) * N + col)
                      : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
    for (int r = 0; r < MW; ++r) {
        float s = (fabsf(v[r].x) + fabsf(v[r].y)) + (fabsf(v[r].z) + fabsf(v[r].w));
        for (int mask = 1; mask < G; mask <<= 1)
            s += __shfl_xor(s, mask, 64);
        key[r] = __float_as_uint(s);
    }

    // Lane c of the group ranks rows c, c + G, ...; a ballot hands the outcome to the whole group.
    uint32_t keep = 0;
    for (int t = 0; t * G < MW; ++t) {
        const int mine = c + t * G;
        uint32_t key_mine = 0;
#pragma unroll
        for (int r = 0; r < MW; ++r)
            key_mine = r == mine ? key[r] : key_mine;
        int rank = 0;
#pragma unroll
        for (int r = 0; r < MW; ++r)
            rank += (key[r] > key_mine || (key[r] == key_mine && r < mine)) ? 1 : 0;
        const unsigned long long votes = __ballot(mine < MW && rank < n);
        const uint32_t bits = (uint32_t)(votes >> group) & ((1u << G) - 1u);
        keep |= bits << (t * G);
    }

    if (!active)
        return;
    const int a = col / L;
#pragma unroll
    for (int r = 0; r < MW; ++r) {
        if ((keep >> r) & 1u) {
            const int p = __popc(keep & ((1u << r) - 1u));
            const size_t row = (size_t)w * n + p;
            store_streaming(BT + row * N + col, v[r]);
            if (c == (r & (G - 1)))
                DT[row * Q + a] = r;
        }
    }
}

// Expansion.  What a thread loads depends on nothing it has loaded: its window's n index entries and
// its 16-byte segments of the window's n compressed rows, all requested at once through
// descriptors that end with the window (entries and rows from n on read as zero without a memory
// access, so the instruction count is fixed).  The rows the indices leave out are zero-filled as
// soon as the indices are there, while the values are still on their way; then every compressed row
// goes to the row its index names (the checker's scatter: the indices need not ascend; a malformed
// index stores nothing).
template <int MW>
__global__ void __launch_bounds__(256)
decompress_kernel(const float* __restrict__ BT, const int32_t* __restrict__ DT, float* __restrict__ B, int N,
                  int Q, int n, int L, int col_blocks)
{
    const int w = blockIdx.x / col_blocks;
    const int col = (blockIdx.x % col_blocks) * kColsPerBlock + threadIdx.x * 4;
    if (col >= N)
        return;
    const int a = col / L;
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(DT) + (size_t)w * n * Q, 0,
                                                                         (int)((size_t)n * Q * sizeof(int32_t)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(BT) + (size_t)w * n * N, 0,
                                                                         (int)((size_t)n * N * sizeof(float)), 0x00020000);
    uint32_t rp[MW];
    cuintx4 x[MW];
#pragma unroll
    for (int p = 0; p < MW; ++p)
        rp[p] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rd, (int)(((uint32_t)p * Q + a) * 4u), 0, 0);
#pragma unroll
    for (int p = 0; p < MW; ++p)
        x[p] = __builtin_amdgcn_raw_buffer_load_b128(rv, (int)(((uint32_t)p * N + col) * 4u), 0, 2);  // read once: non-temporal
    uint32_t keep = 0;
#pragma unroll
    for (int p = 0; p < MW; ++p) {
        if (p >= n)
            rp[p] = 0xffffffffu;
        keep |= rp[p] < (uint32_t)MW ? 1u << rp[p] : 0u;
    }
    float* const base = B + (size_t)w * MW * N;
    const uint32_t bytes = (uint32_t)MW * N * 4u;
#pragma unroll
    for (int r = 0; r < MW; ++r)
        if (!((keep >> r) & 1u))
            store_segment(base, bytes, ((uint32_t)r * N + col) * 4u, make_float4(0.0f, 0.0f, 0.0f, 0.0f));
#pragma unroll
    for (int p = 0; p < MW; ++p)
        if (rp[p] < (uint32_t)MW)
            store_segment(base, bytes, (rp[p] * (uint32_t)N + col) * 4u,
                          make_float4(__uint_as_float(x[p][0]), __uint_as_float(x[p][1]), __uint_as_float(x[p][2]),
                                      __uint_as_float(x[p][3])));
}


// ---- windows of 32 rows with 32-column vectors (the reference's n:32 patterns) ------------------
// One thread of the kernels above would hold all 32 rows of its four columns (128 registers of
// values alone): two waves per SIMD, and every wave loads, ranks and stores in turn with nothing
// to cover it.  Here the window is cut into four quarters of eight rows, one per wave of the
// workgroup: lane (vector j, position c) of wave q holds rows 8 q .. 8 q + 7 of columns
// 4 c .. 4 c + 3 of vector j, so a wave instruction still moves 1 KB of one row (eight vectors,
// 256 columns).  The row scores are summed in the same order as above (inside the thread, then over
// the eight lanes of the vector by lane exchange); the four waves swap their eight scores per
// vector through LDS, lane (j, c) of wave q ranks row 8 q + c, and the waves' ballots are put
// together through LDS to the mask of kept rows of all 32.  About 70 registers: six waves per SIMD.

__device__ inline float dpp_quad_1032(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, false));
}
__device__ inline float dpp_quad_2301(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, false));
}
__device__ inline float dpp_half_mirror(float x)  // lane i of each 8 <- lane 7 - i: the other quad
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x141, 0xF, 0xF, false));
}

constexpr int kVectorsPerBlock32 = 8;

__global__ void __launch_bounds__(256)
compress32_kernel(const float* __restrict__ B, float* __restrict__ BT, int32_t* __restrict__ DT, int N, int Q, int n,
                  int col_blocks)
{
    __shared__ __attribute__((aligned(16))) uint32_t scores[kVectorsPerBlock32][32];
    __shared__ unsigned char kept_bits[kVectorsPerBlock32][4];  // byte q: rows 8 q .. 8 q + 7
    const int w = blockIdx.x / col_blocks;
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int c = lane & 7, j = lane >> 3;
    const int vec = (blockIdx.x % col_blocks) * kVectorsPerBlock32 + j;
    const bool active = vec < Q;                          // whole vectors are active or not
    const int col = vec * 32 + c * 4;

    float4 v[8];
#pragma unroll
    for (int r = 0; r < 8; ++r)
        v[r] = active ? load_streaming(B + ((size_t)w * 32 + q * 8 + r) * N + col)
                      : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    uint32_t mine8[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        // neighbours at distance 1 and 2 inside the thread, then 4, 8, 16 by lane exchange: in each
        // exchange both partners add the same two numbers, so all eight lanes end with the same bits
        float s = (fabsf(v[r].x) + fabsf(v[r].y)) + (fabsf(v[r].z) + fabsf(v[r].w));
        s += dpp_quad_1032(s);
        s += dpp_quad_2301(s);
        s += dpp_half_mirror(s);
        mine8[r] = __float_as_uint(s);
    }
    if (c == 0) {
        *reinterpret_cast<uint4*>(&scores[j][q * 8]) = make_uint4(mine8[0], mine8[1], mine8[2], mine8[3]);
        *reinterpret_cast<uint4*>(&scores[j][q * 8 + 4]) = make_uint4(mine8[4], mine8[5], mine8[6], mine8[7]);
    }
    __syncthreads();
    // lane (j, c) of wave q ranks row 8 q + c among the window's 32: larger scores first, equal
    // scores prefer the lower row; scores are compared as bit patterns (they are sums of
    // magnitudes, so NaNs rank above everything instead of breaking the order)
    const int my_row = q * 8 + c;
    uint32_t key_mine = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r)
        key_mine = r == c ? mine8[r] : key_mine;
    int rank = 0;
#pragma unroll
    for (int r4 = 0; r4 < 8; ++r4) {
        const uint4 k = *reinterpret_cast<const uint4*>(&scores[j][r4 * 4]);
        const uint32_t ks[4] = {k.x, k.y, k.z, k.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int r = r4 * 4 + e;
            rank += (ks[e] > key_mine || (ks[e] == key_mine && r < my_row)) ? 1 : 0;
        }
    }
    const unsigned long long votes = __ballot(rank < n);   // bit 8 j + c: row 8 q + c of vector j
    if (c == 0)
        kept_bits[j][q] = (unsigned char)(votes >> (8 * j));
    __syncthreads();
    const uint32_t keep = *reinterpret_cast<const uint32_t*>(kept_bits[j]);   // bit r: row r of the vector is kept
    if (!active)
        return;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const int row = q * 8 + r;
        if ((keep >> row) & 1u) {
            const int p = __popc(keep & ((1u << row) - 1u));
            const size_t out = (size_t)w * n + p;
            store_streaming(BT + out * N + col, v[r]);
            if (c == r)
                DT[out * Q + vec] = row;
        }
    }
}

// Expansion of n:32 windows, in the manner of decompress_kernel: nothing a thread loads depends on
// what it has loaded.  Lane (j, c) of wave q reads the index entries c, c + 8, c + 16, c + 24 of its
// vector (the eight lanes of the vector OR their four bits each into the mask of kept rows), the
// entries q, q + 4, ... and its 16-byte segments of those compressed rows; wave q zero-fills what
// the mask leaves out of rows 8 q .. 8 q + 7 and sends its compressed rows where their indices say.
__device__ inline uint32_t dpp_or_over_eight_lanes(uint32_t x)
{
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, false);
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, false);
    x |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, false);
    return x;
}

__global__ void __launch_bounds__(256)
decompress32_kernel(const float* __restrict__ BT, const int32_t* __restrict__ DT, float* __restrict__ B, int N, int Q,
                    int n, int col_blocks)
{
    const int w = blockIdx.x / col_blocks;
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
    const int c = lane & 7, j = lane >> 3;
    // a vector beyond the last one reads the last one's entries (the lanes of a wave exchange their
    // bits, so all of them stay) and stores nothing
    const int vec_raw = (blockIdx.x % col_blocks) * kVectorsPerBlock32 + j;
    const bool active = vec_raw < Q;
    const int vec = active ? vec_raw : Q - 1;
    const int col = vec * 32 + c * 4;
    const __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(DT) + (size_t)w * n * Q, 0,
                                                                         (int)((size_t)n * Q * sizeof(int32_t)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(BT) + (size_t)w * n * N, 0,
                                                                         (int)((size_t)n * N * sizeof(float)), 0x00020000);
    uint32_t part[4], rp[8];
    cuintx4 x[8];
#pragma unroll
    for (int u = 0; u < 4; ++u)
        part[u] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rd, (int)(((uint32_t)(c + 8 * u) * Q + vec) * 4u), 0, 0);
#pragma unroll
    for (int t = 0; t < 8; ++t)
        rp[t] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rd, (int)(((uint32_t)(q + 4 * t) * Q + vec) * 4u), 0, 0);
#pragma unroll
    for (int t = 0; t < 8; ++t)
        x[t] = __builtin_amdgcn_raw_buffer_load_b128(rv, (int)(((uint32_t)(q + 4 * t) * N + col) * 4u), 0, 2);  // read once
    uint32_t keep = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u)
        keep |= (c + 8 * u < n && part[u] < 32u) ? 1u << part[u] : 0u;
    keep = dpp_or_over_eight_lanes(keep);
    if (!active)
        return;
    float* const base = B + (size_t)w * 32 * N;
    const uint32_t bytes = 32u * (uint32_t)N * 4u;
#pragma unroll
    for (int r = 0; r < 8; ++r)
        if (!((keep >> (q * 8 + r)) & 1u))
            store_segment(base, bytes, ((uint32_t)(q * 8 + r) * N + col) * 4u, make_float4(0.0f, 0.0f, 0.0f, 0.0f));
#pragma unroll
    for (int t = 0; t < 8; ++t)
        if (q + 4 * t < n && rp[t] < 32u)
            store_segment(base, bytes, (rp[t] * (uint32_t)N + col) * 4u,
                          make_float4(__uint_as_float(x[t][0]), __uint_as_float(x[t][1]), __uint_as_float(x[t][2]),
                                      __uint_as_float(x[t][3])));
}

bool compress_supported(int m, int vec_len)
{
    return (m == 4 || m == 8 || m == 16 || m == 32) && (vec_len == 4 || vec_len == 8 || vec_len == 16 || vec_len == 32);
}

hipError_t launch_compress(const float* B, float* BT, int32_t* DT, int K, int N, int n, int m, int vec_len,
                           hipStream_t stream)
{
    const int col_blocks = (N + kColsPerBlock - 1) / kColsPerBlock;
    if ((size_t)(K / m) * col_blocks > 0x7fffffffull)
        return hipErrorInvalidValue;
    const dim3 grid((unsigned)((K / m) * col_blocks)), block(256);
    const int Q = N / vec_len;
    const int col_blocks32 = (Q + kVectorsPerBlock32 - 1) / kVectorsPerBlock32;
    if (m == 32 && vec_len == 32 && (size_t)(K / 32) * col_blocks32 <= 0x7fffffffull) {
        const dim3 grid32((unsigned)((K / 32) * col_blocks32));
        compress32_kernel<<<grid32, block, 0, stream>>>(B, BT, DT, N, Q, n, col_blocks32);
        return hipGetLastError();
    }
    switch (m) {
    case 4: compress_kernel<4><<<grid, block, 0, stream>>>(B, BT, DT, N, Q, n, vec_len, col_blocks); break;
    case 8: compress_kernel<8><<<grid, block, 0, stream>>>(B, BT, DT, N, Q, n, vec_len, col_blocks); break;
    case 16: compress_kernel<16><<<grid, block, 0, stream>>>(B, BT, DT, N, Q, n, vec_len, col_blocks); break;
    case 32: compress_kernel<32><<<grid, block, 0, stream>>>(B, BT, DT, N, Q, n, vec_len, col_blocks); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_decompress(const float* BT, const int32_t* DT, float* B, int K, int N, int n, int m, int vec_len,
                             hipStream_t stream)
{
    const int col_blocks = (N + kColsPerBlock - 1) / kColsPerBlock;
    if ((size_t)(K / m) * col_blocks > 0x7fffffffull)
        return hipErrorInvalidValue;
    const dim3 grid((unsigned)((K / m) * col_blocks)), block(256);
    const int Q = N / vec_len;
    const int col_blocks32 = (Q + kVectorsPerBlock32 - 1) / kVectorsPerBlock32;
    if (m == 32 && vec_len == 32 && (size_t)(K / 32) * col_blocks32 <= 0x7fffffffull) {
        const dim3 grid32((unsigned)((K / 32) * col_blocks32));
        decompress32_kernel<<<grid32, block, 0, stream>>>(BT, DT, B, N, Q, n, col_blocks32);
        return hipGetLastError();
    }
    switch (m) {
    case 4: decompress_kernel<4><<<grid, block, 0, stream>>>(BT, DT, B, N, Q, n, vec_len, col_blocks); break;
    case 8: decompress_kernel<8><<<grid, block, 0, stream>>>(BT, DT, B, N, Q, n, vec_len, col_blocks); break;
    case 16: decompress_kernel<16><<<grid, block, 0, stream>>>(BT, DT, B, N, Q, n, vec_len, col_blocks); break;
    case 32: decompress_kernel<32><<<grid, block, 0, stream>>>(BT, DT, B, N, Q, n, vec_len, col_blocks); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace nmspmm
