// Decode-sized multiplication (M <= 32): the product is bound by streaming B from HBM once, so
// the design goal is bytes in flight, not arithmetic.
//
//  * One workgroup per 32-column index vector; its waves split the reduction (the windows of
//    the compressed K dimension) between them and sum their partial 32 x 32 results through LDS
//    in wave order, so the result is deterministic and needs no workspace or second launch.
//  * No LDS staging and no barrier in the streaming loop: each lane loads its own MFMA operands,
//    B[2s+h][j] (two 128-byte row segments per wave and instruction, read exactly once from HBM)
//    and A[i][k(2s+h)] (M contiguous floats per half wave, L2 resident), a whole chunk of
//    windows ahead of the v_mfma_f32_32x32x2_f32 that consumes them; rows i >= M are
//    out-of-range loads that return zero.
//  * Index metadata comes as one wave-wide load per window ([kept][Ns/32] ints, plus the 64-entry
//    column_info list on the high-sparsity layout) and is handed to the lanes with ds_bpermute.
#include "internal.h"

namespace nmspmm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct SkinnyParams {
    const float* A;
    const float* B;
    const int32_t* D;
    const int32_t* cinfo;
    float* C;
    int M, N, W, K;
    int nwin;
};

__device__ inline __amdgpu_buffer_rsrc_t sk_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ inline float sk_load(__amdgpu_buffer_rsrc_t r, uint32_t off)
{
    return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}

#ifndef NMSPMM_SK_WAVES
#define NMSPMM_SK_WAVES 8
#endif
#ifndef NMSPMM_SK_UMUL
#define NMSPMM_SK_UMUL 1
#endif
#define NMSPMM_SK_U(u) ((u) * NMSPMM_SK_UMUL)
constexpr int kSkinnyWaves = NMSPMM_SK_WAVES;
constexpr uint32_t kSkNoLoad = 0x80000000u;

// KS: dense rows per window, WS: kept rows per window, QS: column vectors per preprocessed column
// block, HIGH: high-sparsity layout, U: windows per chunk (all loads of a chunk are in flight at once).
template <int KS, int WS, int QS, bool HIGH, int U>
__global__ void __launch_bounds__(64 * kSkinnyWaves)
spmm_skinny_kernel(const SkinnyParams p)
{
    constexpr int KSTEPS = WS / 2;
    constexpr int STEPS = U * KSTEPS;          // MFMAs per chunk
    constexpr int ND = (WS * QS + 63) / 64;    // wave-wide loads per window of indices
    __shared__ float red[kSkinnyWaves][16][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5;
    const int j = lane & 31;
    const int vec_g = blockIdx.x;     // global column vector
    const int jb = vec_g / QS;        // preprocessed column block
    const int vec = vec_g % QS;       // vector inside it
    const int M = p.M, N = p.N;

    // windows of this wave: the same partition rule the large-tile kernels use for split-K
    int w_begin, w_count;
    split_windows(p.nwin, kSkinnyWaves, wave, &w_begin, &w_count);
    const int w_end = w_begin + w_count;

    const float* const Bvec = p.B + (size_t)vec_g * 32;
    const int32_t* const Dblk = p.D + (size_t)jb * p.W * QS;
    const int32_t* const Cinfo = HIGH ? p.cinfo + (size_t)jb * p.nwin * KS : nullptr;
    const uint32_t a_bytes = (uint32_t)((size_t)p.K * M * sizeof(float));
    const uint32_t a_lane = j < M ? (uint32_t)(j * sizeof(float)) : kSkNoLoad;
    const uint32_t b_lane = (uint32_t)(((size_t)h * N + j) * sizeof(float));
    const uint32_t b_step = (uint32_t)(2 * (size_t)N * sizeof(float));
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));

    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v)
        acc[v] = 0.0f;

    int dvec[U][ND];
    int civec[U];
    float a_nxt[STEPS], b_nxt[STEPS];

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
    auto load_b = [&](int w) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int wu = w + u;
            const __amdgpu_buffer_rsrc_t rb =
                sk_rsrc(Bvec + (size_t)min(wu, p.nwin - 1) * WS * N, wu < w_end ? b_bytes : 0u);
            uint32_t boff = b_lane;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s, boff += b_step)
                b_nxt[u * KSTEPS + s] = sk_load(rb, boff);
        }
    };
    // A operands of the same windows, from the metadata currently in dvec / civec.  Lane half h of
    // k-step s needs the dense row that index entry (2s + h) * QS + vec selects: ds_bpermute
    // fetches it from the lane that holds it (no LDS memory involved); on the high-sparsity layout
    // one more permute per window first turns all ranks into rows.
    const int perm_addr = (h * QS + vec) * (int)sizeof(int32_t);
    const uint32_t row_bytes = (uint32_t)((size_t)M * sizeof(float));
    auto load_a = [&](int w) {
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
                a_nxt[u * KSTEPS + s] = sk_load(ra_u, a_lane + (win_row + (uint32_t)row) * row_bytes);
            }
        }
    };

    // Load order per chunk: metadata, B, then (once the metadata has landed) A.  Loads return in
    // order, so waiting for the metadata never waits for the B stream issued after it.
    if (w_count > 0) {
        load_meta(w_begin);
        load_b(w_begin);
        load_a(w_begin);
        if (U < w_count)
            load_meta(w_begin + U);
    }
    for (int w = w_begin; w < w_end; w += U) {
        float a_cur[STEPS], b_cur[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            a_cur[s] = a_nxt[s];
            b_cur[s] = b_nxt[s];
        }
        if (w + U < w_end) {
            load_b(w + U);
            load_a(w + U);
            if (w + 2 * U < w_end)
                load_meta(w + 2 * U);
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_cur[s], b_cur[s], acc, 0, 0, 0);
    }

    // ---- sum the waves' partial tiles in wave order and store the M live rows ---------------------
#pragma unroll
    for (int v = 0; v < 16; ++v)
        red[wave][v][lane] = acc[v];
    __syncthreads();
    // wave v finishes result register v: rows 8*(v/4) + 4*h + v%4 (h = lane half), column j
    for (int v = wave; v < 16; v += kSkinnyWaves) {
        float s = red[0][v][lane];
#pragma unroll
        for (int x = 1; x < kSkinnyWaves; ++x)
            s += red[x][v][lane];
        const int row = 8 * (v / 4) + 4 * h + (v % 4);
        if (row < M)
            p.C[(size_t)row * N + (size_t)vec_g * 32 + j] = s;
    }
}

template <int KS, int WS, bool HIGH, int U>
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
    p.nwin = a.W / WS;
    const dim3 grid(a.N / 32), block(64 * kSkinnyWaves);
    switch (a.Ns) {
    case 128: spmm_skinny_kernel<KS, WS, 4, HIGH, U><<<grid, block, 0, a.stream>>>(p); break;
    case 64: spmm_skinny_kernel<KS, WS, 2, HIGH, U><<<grid, block, 0, a.stream>>>(p); break;
    case 32: spmm_skinny_kernel<KS, WS, 1, HIGH, U><<<grid, block, 0, a.stream>>>(p); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

bool skinny_supported(const SpmmArgs& a)
{
    if (a.M > 32 || a.vec_len != 32 || (a.Ns != 32 && a.Ns != 64 && a.Ns != 128))
        return false;
    if ((size_t)a.K * a.M * sizeof(float) >= 0x80000000ull)
        return false;
    const bool high = a.cinfo != nullptr;
    if (!high)
        return a.window == 32 && (a.kept == 32 || a.kept == 16 || a.kept == 12);
    return a.window == 64 && (a.kept == 16 || a.kept == 8);
}

hipError_t launch_skinny(const SpmmArgs& a)
{
    const bool high = a.cinfo != nullptr;
    if (!high) {
        if (a.kept == 32) return launch_qs<32, 32, false, NMSPMM_SK_U(1)>(a);
        if (a.kept == 16) return launch_qs<32, 16, false, NMSPMM_SK_U(2)>(a);
        if (a.kept == 12) return launch_qs<32, 12, false, NMSPMM_SK_U(2)>(a);
    } else {
        if (a.kept == 16) return launch_qs<64, 16, true, NMSPMM_SK_U(2)>(a);
        if (a.kept == 8) return launch_qs<64, 8, true, NMSPMM_SK_U(4)>(a);
    }
    return hipErrorInvalidValue;
}

} // namespace nmspmm
