// Gathering matrix-core kernel for index vectors shorter than 32 columns (4, 8 or 16 columns share
// one pattern; the reference fixes the vector length at compile time, include/NM-SpMM.h:8) at
// densities of at most one half.
//
// The expanding kernel (spmm_short.hip) multiplies the zeros of B too, so its useful rate is capped
// at kept/window of the matrix-core peak.  This kernel multiplies only kept rows.  The one MFMA
// whose blocks are as narrow as a 4-column vector is v_mfma_f32_4x4x1_16b_f32: sixteen independent
// 4 x 4 x 1 outer products, block b in lanes 4b .. 4b+3 (lane 4b+i supplies A row i, lane 4b+j
// supplies B column j, register i of lane 4b+j receives C[i][j]).  A wave takes 64 columns: block b
// is its 4-column group b, and each block multiplies with the dense row of A that ITS vector keeps.
//
// Every MFMA needs 64 fresh values of A (4 rows for each of 16 blocks), so the kernel is bound by
// how fast those are delivered, not by the matrix pipes: gathered straight from global memory the
// vector L1 caps it at 42 useful TFLOP/s.  Here the four waves of a workgroup share 64 rows of C and
// stage a chunk of 64 (32) dense rows of A in LDS, k-major with a 32-byte skew per dense row; lane
// (b, i) reads rows 16q + 4i .. 4i+3 of its block's dense row with one ds_read_b128, which feeds four
// MFMAs, and the value of B it needs (one 32-bit load per kept row) is reused by all sixteen MFMAs of
// the step.  Index and B value are loaded eight steps ahead, the next chunk of A is fetched into
// registers while the current one is multiplied.  Measured at 4096 cubed with vectors of 4 columns:
// 1:8 85, 2:8 93, 2:4 93 useful TFLOP/s, where the expanding kernel reaches 18, 36 and 71.
#include "internal.h"

namespace nmspmm {

typedef float gfloatx4 __attribute__((ext_vector_type(4)));

struct GatherParams {
    const float* A;
    const float* B;
    const int32_t* D;
    float* out;
    size_t slice_elems;
    int M, N, W, lda;
    int lshift;   // log2(vector length / 4): 4-column groups per vector
    int Qs;       // vectors per preprocessed column block
    int tiles_m;
    int nchunk;   // chunks of kGatherChunk dense rows in the whole reduction
    int split_k;
};

__device__ inline __amdgpu_buffer_rsrc_t gather_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

constexpr int kGatherRows = 64;     // rows of C per workgroup
constexpr int kGatherCols = 256;    // columns of C per workgroup: four waves of 64
constexpr int kGatherAhead = 8;     // steps by which index and B value are loaded ahead
constexpr uint32_t kGatherNoLoad = 0x80000000u;  // beyond every descriptor here: loads 0

template <int MWIN>
struct GatherChunk { static constexpr int value = MWIN == 4 ? 32 : 64; };

// MWIN: rows per window (4, 8, 16), NK: kept rows per window.
template <int MWIN, int NK>
__global__ void __launch_bounds__(256) spmm_gather_kernel(const GatherParams p)
{
    constexpr int R = kGatherRows;
    constexpr int RB = R / 16;                       // 128-bit LDS reads per lane and step
    constexpr int KC = GatherChunk<MWIN>::value;     // dense rows per chunk
    constexpr int STRIDE = R * 4 + 32;               // bytes per dense row in LDS
    constexpr int SEGS = KC * 4 * RB;                // 16-byte segments per chunk
    constexpr int SPT = SEGS / 256;                  // per thread
    constexpr int STEPS = KC / MWIN * NK;            // kept rows per chunk: one step each
    constexpr int PF = kGatherAhead;
    static_assert(SEGS % 256 == 0 && STEPS % PF == 0, "chunk geometry");
    __shared__ __attribute__((aligned(16))) unsigned char lds[KC * STRIDE];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = lane >> 2, i = lane & 3;
    const int tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
    const int row0 = tile_m * R;
    const int M = p.M, N = p.N, W = p.W, lda = p.lda;
    // a wave beyond the last column repeats the last 64 columns (it has to reach the barriers)
    const int col0 = min(tile_n * kGatherCols + wave * 64, N - 64);
    // this slice's chunks: everything below counts chunks and steps from the slice's first one
    int c_begin, c_count;
    split_windows(p.nchunk, p.split_k, blockIdx.y, &c_begin, &c_count);
    const int s_begin = c_begin * STEPS, s_count = c_count * STEPS;

    const size_t K = (size_t)p.nchunk * KC;
    const __amdgpu_buffer_rsrc_t ra = gather_rsrc(p.A, (uint32_t)(K * lda * sizeof(float)));
    const __amdgpu_buffer_rsrc_t rb = gather_rsrc(p.B + (size_t)s_begin * N + col0,
                                                  (uint32_t)(((size_t)(W - 1 - s_begin) * N + 64) * sizeof(float)));
    const __amdgpu_buffer_rsrc_t rd = gather_rsrc(p.D, (uint32_t)((size_t)W * (N >> (2 + p.lshift)) * sizeof(int32_t)));
    const uint32_t b_row = (uint32_t)N * 4u, d_row = (uint32_t)p.Qs * 4u;
    // D is blocked [N / Ns][W][Qs]: this block's vector is (col0 + 4b) / L
    const int Ns = p.Qs << (2 + p.lshift);
    const int col = col0 + 4 * b;
    const uint32_t d_lane = (uint32_t)(((size_t)(col / Ns) * W * p.Qs + (size_t)s_begin * p.Qs + ((col % Ns) >> (2 + p.lshift))) *
                                       sizeof(int32_t));
    const uint32_t b_lane = (uint32_t)lane * 4u;

    // chunk copy: segment tid + 256 j is 16 bytes (4 rows) of dense row seg / 16 of the chunk
    uint32_t cp_src[SPT], cp_dst[SPT];
#pragma unroll
    for (int j = 0; j < SPT; ++j) {
        const int seg = tid + 256 * j, kk = seg / (4 * RB), part = seg % (4 * RB);
        cp_src[j] = (uint32_t)((((size_t)c_begin * KC + kk) * lda + row0 + part * 4) * sizeof(float));
        cp_dst[j] = (uint32_t)(kk * STRIDE + part * 16);
    }
    const uint32_t chunk_bytes = (uint32_t)((size_t)KC * lda * sizeof(float));
    gfloatx4 stage[SPT];
    // rows beyond M are read as whatever follows them in A (or 0 beyond its end): never stored
    auto fetch_chunk = [&](int c) {
#pragma unroll
        for (int j = 0; j < SPT; ++j) {
            const auto x = __builtin_amdgcn_raw_buffer_load_b128(
                ra, c < c_count ? cp_src[j] + (uint32_t)c * chunk_bytes : kGatherNoLoad, 0, 0);
            stage[j] = gfloatx4{__int_as_float(x[0]), __int_as_float(x[1]), __int_as_float(x[2]), __int_as_float(x[3])};
        }
    };
    auto store_chunk = [&]() {
#pragma unroll
        for (int j = 0; j < SPT; ++j)
            *(gfloatx4*)(lds + cp_dst[j]) = stage[j];
    };

    gfloatx4 acc[4 * RB];
#pragma unroll
    for (int r = 0; r < 4 * RB; ++r)
        acc[r] = {0.0f, 0.0f, 0.0f, 0.0f};

    // step s = kept row s of the slice.  The uniform part of both addresses is a scalar offset
    // (not covered by the descriptor's range check: steps outside the slice take the vector offset
    // that is out of range instead).
    int idx[PF];
    float bv[PF];
    auto load_meta = [&](int s, int slot) {
        const bool ok = s < s_count;
        idx[slot] = __builtin_amdgcn_raw_buffer_load_b32(rd, ok ? d_lane : kGatherNoLoad, ok ? (uint32_t)s * d_row : 0u, 0);
        bv[slot] = __int_as_float(
            __builtin_amdgcn_raw_buffer_load_b32(rb, ok ? b_lane : kGatherNoLoad, ok ? (uint32_t)s * b_row : 0u, 0));
    };
    float a[2][4 * RB];
    const uint32_t l_lane = (uint32_t)(i * 16);
    // step t of the chunk lies in window t / NK of it; lane (b, i), read q: rows 16 q + 4 i .. 4 i + 3
    auto read_a = [&](int t, int k_local, float (&dst)[4 * RB]) {
        const uint32_t off = (uint32_t)((t / NK) * MWIN + k_local) * STRIDE + l_lane;
#pragma unroll
        for (int q = 0; q < RB; ++q) {
            const gfloatx4 x = *(const gfloatx4*)(lds + off + q * 64);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                dst[4 * q + e] = x[e];
        }
    };

#pragma unroll
    for (int t = 0; t < PF; ++t)
        load_meta(t, t);
    fetch_chunk(0);
    store_chunk();
    __syncthreads();
    for (int c = 0; c < c_count; ++c) {
        fetch_chunk(c + 1);
        const int s_base = c * STEPS;
        read_a(0, idx[0], a[0]);
#pragma unroll
        for (int t0 = 0; t0 < STEPS; t0 += PF) {
#pragma unroll
            for (int t = 0; t < PF; ++t) {
                const int tt = t0 + t;
                if (tt + 1 < STEPS)
                    read_a(tt + 1, idx[(t + 1) % PF], a[(t + 1) & 1]);
                const float bval = bv[t];
#pragma unroll
                for (int r = 0; r < 4 * RB; ++r)
                    acc[r] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[t & 1][r], bval, acc[r], 0, 0, 0);
                load_meta(s_base + tt + PF, t);
            }
        }
        __syncthreads();
        store_chunk();
        __syncthreads();
    }

    // register i' of lane (b, j), accumulator r: row 16 (r / 4) + 4 i' + r % 4, column col0 + lane
    float* const out = p.out + (size_t)blockIdx.y * p.slice_elems;
#pragma unroll
    for (int r = 0; r < 4 * RB; ++r)
#pragma unroll
        for (int ii = 0; ii < 4; ++ii) {
            const int row = row0 + (r / 4) * 16 + ii * 4 + r % 4;
            if (row < M)
                out[(size_t)row * N + col0 + lane] = acc[r][ii];
        }
}

// Instantiated patterns (window, kept): densities up to one half.
#define NMSPMM_GATHER_PATTERNS(X) X(4, 1) X(4, 2) X(8, 1) X(8, 2) X(8, 3) X(8, 4) X(16, 2) X(16, 4) X(16, 8)

bool gather_supported(const SpmmArgs& a)
{
    if (a.a_rowmajor || a.cinfo != nullptr)
        return false;
    if (a.vec_len != 4 && a.vec_len != 8 && a.vec_len != 16)
        return false;
    const int chunk = a.window == 4 ? 32 : 64;
    if (a.N % 64 != 0 || a.Ns % a.vec_len != 0 || a.N % a.Ns != 0 || a.K % chunk != 0 || a.M < 1 || a.lda < a.M)
        return false;
    if (a.split_k < 1 || a.split_k > a.K / chunk)
        return false;
    if ((size_t)a.K * a.lda * sizeof(float) >= 0x80000000ull || (size_t)a.W * a.N * sizeof(float) >= 0x80000000ull)
        return false;
#define X(MW_, NK_) if (a.window == MW_ && a.kept == NK_) return true;
    NMSPMM_GATHER_PATTERNS(X)
#undef X
    return false;
}

template <int MWIN, int NK>
static hipError_t launch_gather_cfg(const SpmmArgs& a)
{
    GatherParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.lda = a.lda;
    p.lshift = a.vec_len == 4 ? 0 : a.vec_len == 8 ? 1 : 2;
    p.Qs = a.Ns / a.vec_len;
    p.tiles_m = (a.M + kGatherRows - 1) / kGatherRows;
    p.nchunk = a.K / GatherChunk<MWIN>::value;
    p.split_k = a.split_k;
    const int tiles_n = (a.N + kGatherCols - 1) / kGatherCols;
    const dim3 grid((unsigned)(p.tiles_m * tiles_n), (unsigned)a.split_k);
    spmm_gather_kernel<MWIN, NK><<<grid, dim3(256), 0, a.stream>>>(p);
    return hipGetLastError();
}

hipError_t launch_gather(const SpmmArgs& a)
{
#define X(MW_, NK_) if (a.window == MW_ && a.kept == NK_) return launch_gather_cfg<MW_, NK_>(a);
    NMSPMM_GATHER_PATTERNS(X)
#undef X
    return hipErrorInvalidValue;
}

} // namespace nmspmm
