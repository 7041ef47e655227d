// Matrix-core kernel for index vectors shorter than 32 columns (4, 8 or 16 columns share one
// pattern; the reference fixes the vector length at compile time, include/NM-SpMM.h:8).
//
// A 32-column MFMA tile then spans several vectors with different patterns, so the gather of the
// long-vector kernel (one row offset per half wave) does not apply.  Instead the sparse operand is
// expanded on the fly: for a chunk of 16 dense K rows every lane rebuilds its B operands - row
// 2s+h of the chunk, column j - from the kept values and indices of its own column (a compare and a
// select per kept row), zeros included, and A is read ungathered.  The matrix pipes therefore also
// multiply the zeros: the useful rate is bounded by kept/window of the peak, which is still an
// order of magnitude above a SIMT formulation.
//
// Everything else follows the long-vector kernel: one wave = 32 columns x RM 32-row blocks with
// interleaved rows, 128-bit A loads straight into MFMA operand registers through a rolling
// register pipeline, buffer descriptors instead of branches, no LDS, no barrier.
#include "internal.h"

namespace nmspmm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct ShortParams {
    const float* A;
    const float* B;
    const int32_t* D;
    float* out;
    size_t slice_elems;
    int M, N, W, lda;
    int L, Qs;           // columns per vector, vectors per preprocessed column block
    int nchunk;          // chunks of 16 dense rows in the whole reduction
    int split_k;
    int tiles_m, tiles_n;
    int tile_offset;     // first tile of this launch (tiles are numbered column block by column block)
    int sub_tiles;       // > 1: every workgroup of this launch is one of sub_tiles pieces, along M, of a
                         // tile of sub_tiles * 32 * RM rows (tiles_m counts those taller tiles)
};

struct sfloat8 { float4 lo, hi; };
template <int RM> struct SFrag;
template <> struct SFrag<8> { typedef sfloat8 type; };
template <> struct SFrag<4> { typedef float4 type; };
__device__ inline float sfrag_get(const float4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
__device__ inline float sfrag_get(const sfloat8& v, int i) { return i < 4 ? sfrag_get(v.lo, i) : sfrag_get(v.hi, i - 4); }

__device__ inline __amdgpu_buffer_rsrc_t short_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ inline float4 short_load_f4(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    auto v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    return *reinterpret_cast<float4*>(&v);
}

constexpr int kChunk = 16;  // dense K rows per pipeline step: eight MFMA k-steps

// MWIN: rows per window (4, 8, 16), NK: kept rows per window, RM: 32-row blocks per wave.
template <int MWIN, int NK, int RM>
__global__ void __launch_bounds__(256, RM == 8 ? 2 : 3)
spmm_short_kernel(const ShortParams p)
{
    typedef typename SFrag<RM>::type afrag_t;
    constexpr int MW = RM * 32;
    constexpr int WPC = kChunk / MWIN;  // windows per chunk
    constexpr int KSTEPS = kChunk / 2;
    constexpr int RAW = WPC * NK;       // kept rows per chunk

    const int tile = p.tile_offset + blockIdx.x / p.sub_tiles;
    const int tile_m = (tile % p.tiles_m) * p.sub_tiles + blockIdx.x % p.sub_tiles;
    const int tile_n = tile / p.tiles_m;
    int c_begin, c_count;
    split_windows(p.nchunk, p.split_k, blockIdx.y, &c_begin, &c_count);
    const int c_last = c_begin + c_count - 1;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5;
    const int j = lane & 31;
    const int M = p.M, N = p.N, lda = p.lda;
    const int bi = tile_m * MW;
    const int bj = tile_n * 128 + wave * 32;
    const int col = bj + j;
    // the wave's 32 columns lie inside one preprocessed column block; c is this lane's vector in it
    const int Ns = p.Qs * p.L;
    const int32_t* const Dblk = p.D + (size_t)(bj / Ns) * p.W * p.Qs;
    const uint32_t d_lane = (uint32_t)(((col % Ns) / p.L) * sizeof(int32_t));
    const float* const Bvec = p.B + bj;
    const float* const Ablk = p.A + min(bi, lda);

    const uint32_t a_bytes = bi < M ? (uint32_t)(((size_t)(kChunk - 1) * lda + (size_t)(lda - bi)) * sizeof(float)) : 0u;
    const uint32_t b_bytes = (uint32_t)(((size_t)(RAW - 1) * N + 32) * sizeof(float));
    const uint32_t d_bytes = (uint32_t)((size_t)RAW * p.Qs * sizeof(int32_t));
    const uint32_t b_row = (uint32_t)((size_t)N * sizeof(float));
    const uint32_t d_row = (uint32_t)(p.Qs * sizeof(int32_t));
    uint32_t a_off[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
        a_off[s] = (uint32_t)(((size_t)(2 * s + h) * lda + j * 4) * sizeof(float));

    // kept values and indices of this lane's column for one chunk (RAW consecutive kept rows)
    float val[RAW];
    int idx[RAW];
    auto load_raw = [&](int chunk) {
        const size_t krow0 = (size_t)chunk * RAW;
        const __amdgpu_buffer_rsrc_t rb = short_rsrc(Bvec + krow0 * N, b_bytes);
        const __amdgpu_buffer_rsrc_t rd = short_rsrc(Dblk + krow0 * p.Qs, d_bytes);
#pragma unroll
        for (int q = 0; q < RAW; ++q) {
            val[q] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rb, q * b_row + j * 4, 0, 0));
            idx[q] = __builtin_amdgcn_raw_buffer_load_b32(rd, q * d_row + d_lane, 0, 0);
        }
    };
    afrag_t a_op[KSTEPS];
    float b_op[KSTEPS];
    auto load_a_step = [&](int s, __amdgpu_buffer_rsrc_t ra) {
        if constexpr (RM == 8) {
            a_op[s].lo = short_load_f4(ra, a_off[s]);
            a_op[s].hi = short_load_f4(ra, a_off[s] + 512);
        } else {
            a_op[s] = short_load_f4(ra, a_off[s]);
        }
    };
    // dense B operands of the chunk whose kept rows are in val / idx: row 2s + h of the chunk lies
    // in window (2s) / MWIN at local row (2s) % MWIN + h
    auto expand = [&]() {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const int wi = (2 * s) / MWIN;
            const int local = (2 * s) % MWIN;
            float b = 0.0f;
#pragma unroll
            for (int q = 0; q < NK; ++q)
                b = idx[wi * NK + q] - h == local ? val[wi * NK + q] : b;
            b_op[s] = b;
        }
    };

    floatx16 acc[RM];
#pragma unroll
    for (int b = 0; b < RM; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[b][v] = 0.0f;

    if (c_count > 0) {
        load_raw(c_begin);
        const __amdgpu_buffer_rsrc_t ra = short_rsrc(Ablk + (size_t)c_begin * kChunk * lda, a_bytes);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            load_a_step(s, ra);
    }
    for (int t = 0; t < c_count; ++t) {
        const int chunk = c_begin + t;
        const int next = min(chunk + 1, c_last);  // the last chunk reloads itself; nothing consumes it
        expand();
        __builtin_amdgcn_sched_barrier(0);
        load_raw(next);
        const __amdgpu_buffer_rsrc_t ra = short_rsrc(Ablk + (size_t)next * kChunk * lda, a_bytes);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < RM; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(sfrag_get(a_op[s], b), b_op[s], acc[b], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            load_a_step(s, ra);
        }
    }

    // epilogue as in the long-vector kernel: register v of lane (h, j) is row 8*(v/4) + 4*h + v%4 of
    // its block, block b holds rows (b/4)*128 + 4*r + b%4; rows beyond M are dropped by the descriptor
    float* const out = p.out + (size_t)blockIdx.y * p.slice_elems;
    const int rows_here = min(M - bi, MW);
    const uint32_t c_bytes = rows_here > 0 ? (uint32_t)(((size_t)(rows_here - 1) * N + 32) * sizeof(float)) : 0u;
    const __amdgpu_buffer_rsrc_t rc = short_rsrc(out + (size_t)min(bi, M) * N + bj, c_bytes);
    const uint32_t c_lane = (uint32_t)(((size_t)16 * h * N + j) * sizeof(float));
    const uint32_t n_bytes = (uint32_t)((size_t)N * sizeof(float));
#pragma unroll
    for (int v = 0; v < 16; ++v) {
#pragma unroll
        for (int b = 0; b < RM; ++b) {
            const uint32_t row = (b / 4) * 128 + 32 * (v / 4) + 4 * (v % 4) + (b % 4);
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(acc[b][v]), rc, c_lane + row * n_bytes, 0, 0);
        }
    }
}

template <int MWIN, int NK>
static hipError_t launch_short_cfg(const SpmmArgs& a)
{
    ShortParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.lda = a.lda;
    p.L = a.vec_len;
    p.Qs = a.Ns / a.vec_len;
    p.nchunk = a.K / kChunk;
    p.split_k = a.split_k;
    p.tiles_n = a.N / 128;
    p.tile_offset = 0;
    p.sub_tiles = 1;
    // wave height and leftover tiles as in the long-vector kernel: a chunk of 16 dense rows costs
    // what a window of 16 kept rows costs there
    TailPlan plan = plan_tail(a.M, a.N, p.nchunk, kChunk, 1, 2);
    if (a.split_k != 1) {
        plan.blocks = choose_wave_blocks(a.M, a.N, p.nchunk, kChunk, a.split_k);
        plan.separate = false;
    }
    const bool tall = plan.blocks == 8;
    p.tiles_m = (a.M + (tall ? 255 : 127)) / (tall ? 256 : 128);
    const dim3 block(256);
    dim3 grid(p.tiles_m * p.tiles_n, a.split_k);
    if (plan.separate && plan.head + plan.tail == (long long)p.tiles_m * p.tiles_n)
        grid.x = (unsigned)plan.head;
    else
        plan.separate = false;
    if (tall)
        spmm_short_kernel<MWIN, NK, 8><<<grid, block, 0, a.stream>>>(p);
    else
        spmm_short_kernel<MWIN, NK, 4><<<grid, block, 0, a.stream>>>(p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !plan.separate)
        return e;
    // the leftover tiles of a ragged last round in a launch of their own, whole or as two
    // 128-row pieces each (internal.h: plan_tail)
    p.tile_offset = (int)plan.head;
    p.sub_tiles = tall ? plan.sub : 1;
    grid.x = (unsigned)(plan.tail * p.sub_tiles);
    if (tall && p.sub_tiles == 1)
        spmm_short_kernel<MWIN, NK, 8><<<grid, block, 0, a.stream>>>(p);
    else
        spmm_short_kernel<MWIN, NK, 4><<<grid, block, 0, a.stream>>>(p);
    return hipGetLastError();
}

// Instantiated patterns (window, kept); anything else stays on the generic kernel.
#define NMSPMM_SHORT_PATTERNS(X) X(4, 1) X(4, 2) X(4, 3) X(8, 1) X(8, 2) X(8, 3) X(8, 4) X(16, 2) X(16, 4) X(16, 8)

bool short_supported(const SpmmArgs& a)
{
    if (a.a_rowmajor)
        return false;
    if (a.cinfo != nullptr || a.vec_len >= 32 || (a.vec_len != 4 && a.vec_len != 8 && a.vec_len != 16))
        return false;
    if (a.N % 128 != 0 || a.Ns % 32 != 0 || a.K % kChunk != 0 || a.M <= 32 || a.lda < a.M)
        return false;
    if (a.split_k > a.K / kChunk)
        return false;
    if ((size_t)kChunk * a.lda * sizeof(float) >= 0x80000000ull || (size_t)256 * a.N * sizeof(float) >= 0x80000000ull)
        return false;
#define X(MW_, NK_) if (a.window == MW_ && a.kept == NK_) return true;
    NMSPMM_SHORT_PATTERNS(X)
#undef X
    return false;
}

hipError_t launch_short(const SpmmArgs& a)
{
#define X(MW_, NK_) if (a.window == MW_ && a.kept == NK_) return launch_short_cfg<MW_, NK_>(a);
    NMSPMM_SHORT_PATTERNS(X)
#undef X
    return hipErrorInvalidValue;
}

} // namespace nmspmm
