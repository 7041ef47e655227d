// Decode-sized multiplication (M <= 128): the product is bound by streaming B from HBM once (and,
// towards 128 rows, by the matrix pipes), so the design goal is bytes in flight and a single launch.
//
//  * One workgroup per 32-column index vector; its waves split the reduction (the windows of the
//    compressed K dimension) between them and sum their partial results through LDS in wave
//    order, so the result is deterministic and needs no workspace or second launch.
//  * A wave covers 32 * RB rows (RB = 1, 2 or 4 for M <= 32, 64, 128) with the rows interleaved
//    (block b holds rows RB*r + b), so the A operands of all RB blocks of a k-step are one load of
//    RB adjacent floats per lane and the B operand is reused RB times.
//  * No LDS staging and no barrier in the streaming loop: each lane loads its own MFMA operands,
//    B[2s+h][j] (two 128-byte row segments per wave and instruction, read exactly once from HBM)
//    and A[i][k(2s+h)] (L2 resident), a whole chunk of windows ahead of the
//    v_mfma_f32_32x32x2_f32 that consumes them; rows i >= M are out-of-range loads that return
//    zero, or neighbouring values that land in accumulators that are never stored.
//  * Index metadata comes as one wave-wide load per window ([kept][Ns/32] ints, plus the 64-entry
//    column_info list on the high-sparsity layout) and is handed to the lanes with ds_bpermute.
//  * Up to 16 rows a second kernel does the same on v_mfma_f32_16x16x4_f32 (further down).
//  * A itself may be row-major for the one-block forms: a lane loads one float of A per k-step,
//    so the storage order is two strides.  The C-ABI uses that up to 8 rows.
#include "internal.h"

namespace nmspmm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct SkinnyParams {
    const float* A;
    const float* B;
    const int32_t* D;
    const int32_t* cinfo;
    float* C;
    int M, N, W, K, lda;
    int nwin;
    // element (i, k) of A lies i * a_row_stride + k * a_k_stride bytes into its a_bytes bytes:
    // (4, 4 * lda) for the column-major operand, (4 * lda, 4) for a row-major one (up to 32 rows)
    uint32_t a_row_stride, a_k_stride, a_bytes;
    int accumulate;  // the result is added to what C holds instead of replacing it
    int part_rows;   // workgroup (x, y) computes rows [y * part_rows, min(M, (y + 1) * part_rows)) of vector x
};

static int skinny_part_rows(const SpmmArgs& a);

__device__ inline __amdgpu_buffer_rsrc_t sk_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ inline float sk_load(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}

// the A operands of one k-step: RB adjacent floats
template <int RB> struct SkFrag { float v[RB]; };
template <int RB> __device__ inline SkFrag<RB> sk_load_frag(__amdgpu_buffer_rsrc_t r, uint32_t off);
template <> __device__ inline SkFrag<1> sk_load_frag<1>(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    SkFrag<1> f;
    f.v[0] = sk_load(r, off);
    return f;
}
template <> __device__ inline SkFrag<2> sk_load_frag<2>(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    auto x = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    SkFrag<2> f;
    f.v[0] = __int_as_float(x[0]);
    f.v[1] = __int_as_float(x[1]);
    return f;
}
template <> __device__ inline SkFrag<4> sk_load_frag<4>(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    auto x = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
    SkFrag<4> f;
    f.v[0] = __int_as_float(x[0]);
    f.v[1] = __int_as_float(x[1]);
    f.v[2] = __int_as_float(x[2]);
    f.v[3] = __int_as_float(x[3]);
    return f;
}

constexpr int kSkinnyMaxRows = 128;
constexpr int kSkinnyWaves = 8;

// KS: dense rows per window, WS: kept rows per window, QS: column vectors per preprocessed column
// block, HIGH: high-sparsity layout, RB: 32-row blocks per wave, U: windows per chunk (all loads
// of a chunk are in flight at once).
template <int KS, int WS, int QS, bool HIGH, int RB, int U>
__global__ void __launch_bounds__(64 * kSkinnyWaves)
spmm_skinny_kernel(const SkinnyParams p)
{
    constexpr int KSTEPS = WS / 2;
    constexpr int STEPS = U * KSTEPS;          // k-steps per chunk
    constexpr int ND = (WS * QS + 63) / 64;    // wave-wide loads per window of indices
    typedef SkFrag<RB> afrag_t;
    __shared__ float red[kSkinnyWaves][16][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5;
    const int j = lane & 31;
    const int vec_g = blockIdx.x;     // global column vector
    const int jb = vec_g / QS;        // preprocessed column block
    const int vec = vec_g % QS;       // vector inside it
    const int m0 = blockIdx.y * p.part_rows;
    const int M = min(p.M - m0, p.part_rows), N = p.N;

    // windows of this wave: the same partition rule the large-tile kernels use for split-K
    int w_begin, w_count;
    split_windows(p.nwin, kSkinnyWaves, wave, &w_begin, &w_count);
    const int w_end = w_begin + w_count;

    const float* const Bvec = p.B + (size_t)vec_g * 32;
    const int32_t* const Dblk = p.D + (size_t)jb * p.W * QS;
    const int32_t* const Cinfo = HIGH ? p.cinfo + (size_t)jb * p.nwin * KS : nullptr;
    const uint32_t a_bytes = p.a_bytes;
    // lanes beyond the last row read the last fragment that exists (their tile rows are never stored):
    // loads with most lanes out of range are slow
    const uint32_t a_lane = (uint32_t)(m0 + min(RB * j, (M - 1) / RB * RB)) * p.a_row_stride;
    const uint32_t row_bytes = p.a_k_stride;
    const uint32_t b_lane = (uint32_t)(((size_t)h * N + j) * sizeof(float));
    const uint32_t b_step = (uint32_t)(2 * (size_t)N * sizeof(float));
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));
    const int perm_addr = (h * QS + vec) * (int)sizeof(int32_t);

    floatx16 acc[RB];
#pragma unroll
    for (int b = 0; b < RB; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[b][v] = 0.0f;

    int dvec[U][ND];
    int civec[U];
    // two operand sets: one is multiplied while the other is in flight
    afrag_t a0[STEPS], a1[STEPS];
    float b0[STEPS], b1[STEPS];

    // metadata of the U windows starting at w (windows past the end are clamped; their operand
    // loads are suppressed below, so whatever they index contributes nothing)
    auto load_meta = [&](int w) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = min(w + u, p.nwin - 1);
            const __amdgpu_buffer_rsrc_t rd = sk_rsrc(Dblk + (size_t)wu * WS * QS, WS * QS * sizeof(int32_t));
#pragma unroll
            for (int q = 0; q < ND; ++q)
                dvec[u][q] = __builtin_amdgcn_raw_buffer_load_b32(rd, (lane + 64 * q) * (int)sizeof(int32_t), 0, 0);
            if (HIGH) {
                const __amdgpu_buffer_rsrc_t rc = sk_rsrc(Cinfo + (size_t)wu * KS, KS * sizeof(int32_t));
                civec[u] = __builtin_amdgcn_raw_buffer_load_b32(rc, lane * (int)sizeof(int32_t), 0, 0);
            }
        }
    };
    // B operands of the U windows starting at w: addresses depend on nothing, so these go out first
    // and the HBM stream starts with the kernel.  A window past this wave's share loads nothing
    // (zero-sized descriptor) and so adds exact zeros.
    auto load_b = [&](int w, float (&b_dst)[STEPS]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = w + u;
            const __amdgpu_buffer_rsrc_t rb =
                sk_rsrc(Bvec + (size_t)min(wu, p.nwin - 1) * WS * N, wu < w_end ? b_bytes : 0u);
            uint32_t boff = b_lane;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s, boff += b_step)
                b_dst[u * KSTEPS + s] = sk_load(rb, boff);
        }
    };
    // A operands of the same windows, from the metadata currently in dvec / civec.  Lane half h of
    // k-step s needs the dense row that index entry (2s + h) * QS + vec selects: ds_bpermute
    // fetches it from the lane that holds it (no LDS memory involved); on the high-sparsity layout
    // one more permute per window first turns all ranks into rows.
    auto load_a = [&](int w, afrag_t (&a_dst)[STEPS]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = w + u;
            const __amdgpu_buffer_rsrc_t ra_u = sk_rsrc(p.A, wu < w_end ? a_bytes : 0u);
            const uint32_t win_row = (uint32_t)(min(wu, p.nwin - 1) * KS);
            if (HIGH) {
                static_assert(!HIGH || ND == 1, "one register of ranks per window");
                dvec[u][0] = __builtin_amdgcn_ds_bpermute(dvec[u][0] << 2, civec[u]);
            }
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) {
                const int e = 2 * s * QS;
                const int row = __builtin_amdgcn_ds_bpermute(perm_addr + (e % 64) * (int)sizeof(int32_t), dvec[u][e / 64]);
                a_dst[u * KSTEPS + s] = sk_load_frag<RB>(ra_u, a_lane + (win_row + (uint32_t)row) * row_bytes);
            }
        }
    };
    // one chunk: the next chunk's loads go out, then this chunk's operands are multiplied
    auto chunk = [&](int w, afrag_t (&a_cur)[STEPS], float (&b_cur)[STEPS], afrag_t (&a_nxt)[STEPS],
                     float (&b_nxt)[STEPS]) {
        if (w + U < w_end) {
            load_b(w + U, b_nxt);
            load_a(w + U, a_nxt);
            if (w + 2 * U < w_end)
                load_meta(w + 2 * U);
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
#pragma unroll
            for (int b = 0; b < RB; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[s].v[b], b_cur[s], acc[b], 0, 0, 0);
    };

    // Load order per chunk: metadata, B, then (once the metadata has landed) A.  Loads return in
    // order, so waiting for the metadata never waits for the B stream issued after it.
    if (w_count > 0) {
        load_meta(w_begin);
        load_b(w_begin, b0);
        load_a(w_begin, a0);
        if (U < w_count)
            load_meta(w_begin + U);
    }
    for (int w = w_begin; w < w_end; w += 2 * U) {
        chunk(w, a0, b0, a1, b1);
        if (w + U < w_end)
            chunk(w + U, a1, b1, a0, b0);
    }

    // ---- sum the waves' partial tiles in wave order, one 32-row block at a time, and store the
    // live rows.  Result register v of lane (h, j) is row 8*(v/4) + 4*h + v%4 of its block, column
    // j; block b holds rows RB*r + b.
#pragma unroll
    for (int b = 0; b < RB; ++b) {
        if (b > 0)
            __syncthreads();
#pragma unroll
        for (int v = 0; v < 16; ++v)
            red[wave][v][lane] = acc[b][v];
        __syncthreads();
        for (int v = wave; v < 16; v += kSkinnyWaves) {
            float s = red[0][v][lane];
#pragma unroll
            for (int x = 1; x < kSkinnyWaves; ++x)
                s += red[x][v][lane];
            const int row = RB * (8 * (v / 4) + 4 * h + (v % 4)) + b;
            if (row < M) {
                float* const dst = p.C + (size_t)(m0 + row) * N + (size_t)vec_g * 32 + j;
                *dst = p.accumulate ? *dst + s : s;
            }
        }
    }
}

// Up to 16 rows: the same design on v_mfma_f32_16x16x4_f32.  A k-step is four kept rows, so the
// streaming loop issues half as many loads and spends half as many matrix-pipe cycles per kept
// row as the 32-row form.  Lane l = (kq, jl) = (l / 16, l % 16) supplies A[jl][row of kept row
// 4s + kq] and, with one 64-bit load, B[4s + kq][2 jl] and B[4s + kq][2 jl + 1] (four 128-byte row
// segments per wave and instruction): the even columns of the vector accumulate in one MFMA
// tile, the odd ones in a second.  Result register v of lane (kq, jl) is row 4 kq + v.
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int KS, int WS, int QS, bool HIGH, int U>
__global__ void __launch_bounds__(64 * kSkinnyWaves)
spmm_skinny16_kernel(const SkinnyParams p)
{
    constexpr int KSTEPS = WS / 4;
    constexpr int STEPS = U * KSTEPS;
    constexpr int ND = (WS * QS + 63) / 64;
    static_assert(WS % 4 == 0, "k-steps of four kept rows");
    __shared__ float red[kSkinnyWaves][8][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4;
    const int jl = lane & 15;
    const int vec_g = blockIdx.x;
    const int jb = vec_g / QS;
    const int vec = vec_g % QS;
    const int m0 = blockIdx.y * p.part_rows;
    const int M = min(p.M - m0, p.part_rows), N = p.N;

    int w_begin, w_count;
    split_windows(p.nwin, kSkinnyWaves, wave, &w_begin, &w_count);
    const int w_end = w_begin + w_count;

    const float* const Bvec = p.B + (size_t)vec_g * 32;
    const int32_t* const Dblk = p.D + (size_t)jb * p.W * QS;
    const int32_t* const Cinfo = HIGH ? p.cinfo + (size_t)jb * p.nwin * KS : nullptr;
    const uint32_t a_bytes = p.a_bytes;
    // lanes beyond the last row read the last row (their tile rows are never stored): loads with most
    // lanes out of range are slow
    const uint32_t a_lane = (uint32_t)(m0 + min(jl, M - 1)) * p.a_row_stride;
    const uint32_t row_bytes = p.a_k_stride;
    const uint32_t b_lane = (uint32_t)(((size_t)kq * N + 2 * jl) * sizeof(float));
    const uint32_t b_step = (uint32_t)(4 * (size_t)N * sizeof(float));
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));
    const int perm_addr = (kq * QS + vec) * (int)sizeof(int32_t);

    floatx4 acc_even = {0.0f, 0.0f, 0.0f, 0.0f}, acc_odd = {0.0f, 0.0f, 0.0f, 0.0f};

    int dvec[U][ND];
    int civec[U];
    // two operand sets: one is multiplied while the other is in flight
    float a0[STEPS], a1[STEPS];
    float2 b0[STEPS], b1[STEPS];

    auto load_meta = [&](int w) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = min(w + u, p.nwin - 1);
            const __amdgpu_buffer_rsrc_t rd = sk_rsrc(Dblk + (size_t)wu * WS * QS, WS * QS * sizeof(int32_t));
#pragma unroll
            for (int q = 0; q < ND; ++q)
                dvec[u][q] = __builtin_amdgcn_raw_buffer_load_b32(rd, (lane + 64 * q) * (int)sizeof(int32_t), 0, 0);
            if (HIGH) {
                const __amdgpu_buffer_rsrc_t rc = sk_rsrc(Cinfo + (size_t)wu * KS, KS * sizeof(int32_t));
                civec[u] = __builtin_amdgcn_raw_buffer_load_b32(rc, lane * (int)sizeof(int32_t), 0, 0);
            }
        }
    };
    auto load_b = [&](int w, float2 (&b_dst)[STEPS]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = w + u;
            const __amdgpu_buffer_rsrc_t rb =
                sk_rsrc(Bvec + (size_t)min(wu, p.nwin - 1) * WS * N, wu < w_end ? b_bytes : 0u);
            uint32_t boff = b_lane;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s, boff += b_step) {
                const auto x = __builtin_amdgcn_raw_buffer_load_b64(rb, boff, 0, 0);
                b_dst[u * KSTEPS + s] = make_float2(__int_as_float(x[0]), __int_as_float(x[1]));
            }
        }
    };
    // lane quarter kq of k-step s needs the dense row that index entry (4s + kq) * QS + vec selects
    auto load_a = [&](int w, float (&a_dst)[STEPS]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = w + u;
            const __amdgpu_buffer_rsrc_t ra_u = sk_rsrc(p.A, wu < w_end ? a_bytes : 0u);
            const uint32_t win_row = (uint32_t)(min(wu, p.nwin - 1) * KS);
            if (HIGH) {
                static_assert(!HIGH || ND == 1, "one register of ranks per window");
                dvec[u][0] = __builtin_amdgcn_ds_bpermute(dvec[u][0] << 2, civec[u]);
            }
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) {
                const int e = 4 * s * QS;
                const int row = __builtin_amdgcn_ds_bpermute(perm_addr + (e % 64) * (int)sizeof(int32_t), dvec[u][e / 64]);
                a_dst[u * KSTEPS + s] = sk_load(ra_u, a_lane + (win_row + (uint32_t)row) * row_bytes);
            }
        }
    };
    auto chunk = [&](int w, float (&a_cur)[STEPS], float2 (&b_cur)[STEPS], float (&a_nxt)[STEPS], float2 (&b_nxt)[STEPS]) {
        if (w + U < w_end) {
            load_b(w + U, b_nxt);
            load_a(w + U, a_nxt);
            if (w + 2 * U < w_end)
                load_meta(w + 2 * U);
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            acc_even = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[s], b_cur[s].x, acc_even, 0, 0, 0);
            acc_odd = __builtin_amdgcn_mfma_f32_16x16x4f32(a_cur[s], b_cur[s].y, acc_odd, 0, 0, 0);
        }
    };

    if (w_count > 0) {
        load_meta(w_begin);
        load_b(w_begin, b0);
        load_a(w_begin, a0);
        if (U < w_count)
            load_meta(w_begin + U);
    }
    for (int w = w_begin; w < w_end; w += 2 * U) {
        chunk(w, a0, b0, a1, b1);
        if (w + U < w_end)
            chunk(w + U, a1, b1, a0, b0);
    }

    // sum the waves' partial tiles in wave order: value x of a lane is register x % 4 (row
    // 4 kq + x % 4) of the even (x < 4) or odd columns
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        red[wave][v][lane] = acc_even[v];
        red[wave][4 + v][lane] = acc_odd[v];
    }
    __syncthreads();
    for (int x = wave; x < 8; x += kSkinnyWaves) {
        float s = red[0][x][lane];
#pragma unroll
        for (int y = 1; y < kSkinnyWaves; ++y)
            s += red[y][x][lane];
        const int row = 4 * kq + (x % 4);
        if (row < M) {
            float* const dst = p.C + (size_t)(m0 + row) * N + (size_t)vec_g * 32 + 2 * jl + x / 4;
            *dst = p.accumulate ? *dst + s : s;
        }
    }
}

template <int KS, int WS, bool HIGH, int RB, int U>
static hipError_t launch_qs(const SpmmArgs& a)
{
    SkinnyParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.C = a.C;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.K = a.K;
    p.lda = a.lda;
    p.nwin = a.W / WS;
    p.a_row_stride = (uint32_t)(a.a_rowmajor ? a.lda * sizeof(float) : sizeof(float));
    p.a_k_stride = (uint32_t)(a.a_rowmajor ? sizeof(float) : a.lda * sizeof(float));
    p.a_bytes = (uint32_t)((size_t)(a.a_rowmajor ? a.M : a.K) * a.lda * sizeof(float));
    p.accumulate = (a.accumulate && a.split_k > 1) ? 1 : 0;
    p.part_rows = skinny_part_rows(a);
    const dim3 grid(a.N / 32, (a.M + p.part_rows - 1) / p.part_rows), block(64 * kSkinnyWaves);
    switch (a.Ns) {
    case 128: spmm_skinny_kernel<KS, WS, 4, HIGH, RB, U><<<grid, block, 0, a.stream>>>(p); break;
    case 64: spmm_skinny_kernel<KS, WS, 2, HIGH, RB, U><<<grid, block, 0, a.stream>>>(p); break;
    case 32: spmm_skinny_kernel<KS, WS, 1, HIGH, RB, U><<<grid, block, 0, a.stream>>>(p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

template <int KS, int WS, bool HIGH, int U>
static hipError_t launch_qs16(const SpmmArgs& a)
{
    SkinnyParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.C = a.C;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.K = a.K;
    p.lda = a.lda;
    p.nwin = a.W / WS;
    p.a_row_stride = (uint32_t)(a.a_rowmajor ? a.lda * sizeof(float) : sizeof(float));
    p.a_k_stride = (uint32_t)(a.a_rowmajor ? sizeof(float) : a.lda * sizeof(float));
    p.a_bytes = (uint32_t)((size_t)(a.a_rowmajor ? a.M : a.K) * a.lda * sizeof(float));
    p.accumulate = (a.accumulate && a.split_k > 1) ? 1 : 0;
    p.part_rows = skinny_part_rows(a);
    const dim3 grid(a.N / 32, (a.M + p.part_rows - 1) / p.part_rows), block(64 * kSkinnyWaves);
    switch (a.Ns) {
    case 128: spmm_skinny16_kernel<KS, WS, 4, HIGH, U><<<grid, block, 0, a.stream>>>(p); break;
    case 64: spmm_skinny16_kernel<KS, WS, 2, HIGH, U><<<grid, block, 0, a.stream>>>(p); break;
    case 32: spmm_skinny16_kernel<KS, WS, 1, HIGH, U><<<grid, block, 0, a.stream>>>(p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
// 32-row blocks per wave for a row count
static int skinny_blocks(int M) { return M <= 32 ? 1 : M <= 64 ? 2 : 4; }

// Rows per workgroup (decode_part_rows): a row-major A only has the one-block forms, and a
// column-major one needs a pitch that the part's blocks divide.
static int skinny_part_rows(const SpmmArgs& a)
{
    const int rows = decode_part_rows(a.M, a.N / 32);
    if (!a.a_rowmajor && a.lda % skinny_blocks(rows) != 0)
        return a.M;
    return rows;
}

// the 16-row form reads B with 64-bit loads; the C-ABI layer has checked that B is 16-byte aligned
static bool skinny16_applies(const SpmmArgs& a) { return skinny_part_rows(a) <= 16; }

bool skinny_supported(const SpmmArgs& a)
{
    if (a.M > kSkinnyMaxRows || a.vec_len != 32 || (a.Ns != 32 && a.Ns != 64 && a.Ns != 128))
        return false;
    if (a.a_rowmajor) {
        // a lane then loads one float of A per k-step, whatever the pitch: the one-block forms only
        if (a.M > 32 || a.lda < a.K || (size_t)a.M * a.lda * sizeof(float) >= 0x80000000ull)
            return false;
    } else {
        if (a.lda < a.M || a.lda % skinny_blocks(a.M) != 0)  // a lane's run of rows must not straddle the pitch
            return false;
        if ((size_t)a.K * a.lda * sizeof(float) >= 0x80000000ull)
            return false;
    }
    const bool high = a.cinfo != nullptr;
    if (!high)
        return a.window == 32 && ((a.kept == 32 && a.M <= 32) || a.kept == 16 || a.kept == 12);
    return a.window == 64 && (a.kept == 16 || a.kept == 8);
}

// Windows per chunk: sixteen kept rows for the 32-row form, thirty-two for the 16-row form (eight
// k-steps either way; U1 is the count for sixteen k-steps).  Measured against chunks two and three
// times as long: shorter chunks win by 5 to 15 %, most where there are more workgroups than CUs
// and the smaller register footprint lets two of them share a CU.
template <int KS, int WS, bool HIGH, int U1>
static hipError_t launch_rb(const SpmmArgs& a)
{
    constexpr int UN = U1 >= 2 ? U1 / 2 : 1;
    constexpr int U16 = 32 / WS > 0 ? 32 / WS : 1;
    if (skinny16_applies(a))
        return launch_qs16<KS, WS, HIGH, U16>(a);
    switch (skinny_blocks(skinny_part_rows(a))) {
    case 1: return launch_qs<KS, WS, HIGH, 1, UN>(a);
    case 2: return launch_qs<KS, WS, HIGH, 2, UN>(a);
    default: return launch_qs<KS, WS, HIGH, 4, UN>(a);
    }
}

hipError_t launch_skinny(const SpmmArgs& a)
{
    const bool high = a.cinfo != nullptr;
    if (!high) {
        if (a.kept == 32) return skinny16_applies(a) ? launch_qs16<32, 32, false, 1>(a) : launch_qs<32, 32, false, 1, 1>(a);
        if (a.kept == 16) return launch_rb<32, 16, false, 2>(a);
        if (a.kept == 12) return launch_rb<32, 12, false, 2>(a);
    } else {
        if (a.kept == 16) return launch_rb<64, 16, true, 2>(a);
        if (a.kept == 8) return launch_rb<64, 8, true, 4>(a);
    }
    return hipErrorInvalidValue;
}

} // namespace nmspmm
