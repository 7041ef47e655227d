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
// stage a chunk of dense rows of A in LDS, k-major with a 64-byte skew per dense row (no bank
// conflict in 4-row windows, few in larger ones); lane (b, i) reads rows
// 16q + 4i .. 4i+3 of its block's dense row with one ds_read_b128, which feeds four MFMAs, through
// a ring of four such reads that is kept three reads ahead of the MFMAs.
//
// A chunk (32 dense rows for 4-row windows, 64 otherwise) is one to four "phases" of eight kept
// rows.  A phase's indices and values of B do not come through registers: two global loads per step cost the matrix
// pipes 14 % of their time however far ahead they are issued (measured in isolation), an LDS read
// about a cycle.  Each wave copies two of the phase's eight rows of B (the workgroup's 256 columns,
// one 128-bit LDS-direct load per row) and their indices straight into one half of a small
// double-buffered LDS area a phase ahead, and every lane reads its index and value from there; the
// next chunk of A is fetched into registers while the current one is multiplied and stored between
// the two barriers that end the chunk.  The GPU does not hold its 2.4 GHz under this kernel (LDS and
// matrix pipes both busy: about 2.1 GHz at 2:4), so fewer instructions and fewer LDS cycles also
// mean a higher clock.  Measured at 4096 cubed with vectors of 4 columns: 2:4 108, 2:8 100, 1:8 90
// useful TFLOP/s, where the expanding kernel reaches 71, 36 and 18.
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
    int nchunk;   // chunks of gather_chunk(window, kept) dense rows in the whole reduction
    int split_k;
};

__device__ inline __amdgpu_buffer_rsrc_t gather_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

constexpr int kGatherRows = 64;     // rows of C per workgroup
constexpr int kGatherCols = 256;    // columns of C per workgroup: four waves of 64
constexpr int kGatherPhase = 8;     // steps (kept rows) whose index and B value sit in one half of the meta buffers
constexpr uint32_t kGatherNoLoad = 0x80000000u;  // beyond every descriptor here: loads 0

// Dense rows of A per chunk: 32 for 4-row windows, 64 otherwise: one to four phases of eight kept rows.
constexpr int gather_chunk(int window, int kept) { return window == 4 ? 32 : 64; }

typedef __attribute__((address_space(3))) float gather_lds_f32;
typedef __attribute__((address_space(3))) int32_t gather_lds_i32;

// Global -> LDS loads without a register stop-over: lane l's 16 (4) bytes land at dst + 16 l
// (dst + 4 l); dst is wave-uniform; completion is counted in vmcnt.  Kept out of the kernel
// template: the host pass drops a kernel template that names the builtin directly.
__device__ inline void gather_row_to_lds(__amdgpu_buffer_rsrc_t r, gather_lds_f32* dst, uint32_t v_off, uint32_t s_off)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst, 16, v_off, s_off, 0, 0);
}
__device__ inline void gather_word_to_lds(__amdgpu_buffer_rsrc_t r, gather_lds_i32* dst, uint32_t v_off, uint32_t s_off)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst, 4, v_off, s_off, 0, 0);
}

// MWIN: rows per window (4, 8, 16), NK: kept rows per window.
template <int MWIN, int NK>
__global__ void __launch_bounds__(256) spmm_gather_kernel(const GatherParams p)
{
    constexpr int R = kGatherRows;
    constexpr int RB = R / 16;                       // 128-bit LDS reads per lane and step
    constexpr int KC = gather_chunk(MWIN, NK);       // dense rows per chunk
    // bytes per dense row in LDS.  A pass of a 128-bit LDS read serves 16 lanes, i.e. four blocks of
    // 64 bytes, out of 64 banks: with a 64-byte skew the rows k, k + 1, k + 2, k + 3 fall into the four
    // quarters of the banks, so a 4-row window never conflicts and in larger windows only rows 4, 8
    // or 12 apart do (with 32 bytes neighbours overlap by half: 1:8 ran 4 % slower)
    constexpr int STRIDE = R * 4 + 64;
    constexpr int SEGS = KC * 4 * RB;                // 16-byte segments per chunk
    constexpr int SPT = SEGS / 256;                  // per thread
    constexpr int STEPS = KC / MWIN * NK;            // kept rows per chunk: one step each
    constexpr int PH = kGatherPhase;
    constexpr int P = STEPS / PH;                    // phases per chunk
    static_assert(SEGS % 256 == 0 && STEPS % PH == 0, "chunk geometry");
    // A's chunk; and, twice (the phase being multiplied and the next one), a phase's values of B (a
    // row of the workgroup's 256 columns per step) and its indices (one per step and vector)
    __shared__ __attribute__((aligned(16))) unsigned char lds[KC * STRIDE];
    __shared__ __attribute__((aligned(16))) float lds_b[2 * PH * kGatherCols];
    __shared__ __attribute__((aligned(16))) int32_t lds_i[2 * PH * 64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = lane >> 2, i = lane & 3;
    const int tile_m = blockIdx.x % p.tiles_m, tile_n = blockIdx.x / p.tiles_m;
    const int row0 = tile_m * R;
    const int M = p.M, N = p.N, W = p.W, lda = p.lda;
    // a wave beyond the last column repeats the last 64 columns (it has to reach the barriers)
    const int colwg = tile_n * kGatherCols;
    const int col0 = min(colwg + wave * 64, N - 64);
    // this slice's chunks: everything below counts chunks, phases and steps from the slice's first one
    int c_begin, c_count;
    split_windows(p.nchunk, p.split_k, blockIdx.y, &c_begin, &c_count);
    const int s_begin = c_begin * STEPS;
    const int phases = c_count * P;

    const size_t K = (size_t)p.nchunk * KC;
    const __amdgpu_buffer_rsrc_t ra = gather_rsrc(p.A, (uint32_t)(K * lda * sizeof(float)));
    // B from this slice's first kept row and this workgroup's first column on
    const __amdgpu_buffer_rsrc_t rb = gather_rsrc(p.B + (size_t)s_begin * N + colwg,
                                                  (uint32_t)(((size_t)(W - 1 - s_begin) * N + (N - colwg)) * sizeof(float)));
    const __amdgpu_buffer_rsrc_t rd = gather_rsrc(p.D, (uint32_t)((size_t)W * (N >> (2 + p.lshift)) * sizeof(int32_t)));
    const uint32_t b_row = (uint32_t)N * 4u, d_row = (uint32_t)p.Qs * 4u;
    // D is blocked [N / Ns][W][Qs].  The workgroup's 256 columns hold nv = 256 / L vectors; lane l
    // fetches the index of vector l % nv (a vector beyond the last column: the last one)
    const int Ns = p.Qs << (2 + p.lshift);
    const int nv = 64 >> p.lshift;
    const int vcol = min(colwg + ((lane & (nv - 1)) << (2 + p.lshift)), N - (4 << p.lshift));
    const uint32_t d_lane = (uint32_t)(((size_t)(vcol / Ns) * W * p.Qs + (size_t)s_begin * p.Qs + ((vcol % Ns) >> (2 + p.lshift))) *
                                       sizeof(int32_t));
    // Phase g (eight steps of the slice) into half g & 1 of the meta buffers: step s's row of B to
    // lds_b[half][s][0 .. 255] (one instruction of one wave; columns beyond the matrix read the next
    // row or, behind the last one, zeros: no wave uses them) and its indices to lds_i[half][s][0 .. 63]
    // (entry l: vector l % nv).  The uniform part of both addresses is a scalar offset.
    auto fetch_meta = [&](int g) {
        const int half = g & 1;
#pragma unroll
        for (int s0 = 0; s0 < PH; s0 += 4) {
            const int s = s0 + wave;
            const uint32_t step = (uint32_t)(g * PH + s);
            gather_row_to_lds(rb, (gather_lds_f32*)lds_b + (half * PH + s) * kGatherCols, (uint32_t)lane * 16u, step * b_row);
            gather_word_to_lds(rd, (gather_lds_i32*)lds_i + (half * PH + s) * 64, d_lane, step * d_row);
        }
    };

    // chunk copy: segment tid + 256 j is 16 bytes (4 rows) of dense row seg / 16 of the chunk, i.e.
    // thread tid's segments lie 16 dense rows apart: one vector offset each for source and
    // destination, the rest is uniform (scalar offset of the load, immediate of the LDS write)
    static_assert(RB == 4, "a dense row is sixteen 16-byte segments");
    const uint32_t cp_src = (uint32_t)((((size_t)c_begin * KC + (tid >> 4)) * lda + row0 + (tid & 15) * 4) * sizeof(float));
    const uint32_t cp_dst = (uint32_t)((tid >> 4) * STRIDE + (tid & 15) * 16);
    const uint32_t chunk_bytes = (uint32_t)((size_t)KC * lda * sizeof(float));
    const uint32_t seg_bytes = (uint32_t)((size_t)16 * lda * sizeof(float));
    gfloatx4 stage[SPT];
    // rows beyond M are read as whatever follows them in A (or 0 beyond its end): never stored
    auto fetch_chunk = [&](int c) {
#pragma unroll
        for (int j = 0; j < SPT; ++j) {
            const auto x = __builtin_amdgcn_raw_buffer_load_b128(ra, cp_src, (uint32_t)c * chunk_bytes + (uint32_t)j * seg_bytes, 0);
            stage[j] = gfloatx4{__int_as_float(x[0]), __int_as_float(x[1]), __int_as_float(x[2]), __int_as_float(x[3])};
        }
    };
    auto store_chunk = [&]() {
#pragma unroll
        for (int j = 0; j < SPT; ++j)
            *(gfloatx4*)(lds + cp_dst + j * 16 * STRIDE) = stage[j];
    };

    gfloatx4 acc[4 * RB];
#pragma unroll
    for (int r = 0; r < 4 * RB; ++r)
        acc[r] = {0.0f, 0.0f, 0.0f, 0.0f};

    // this lane's column and its block's vector within the workgroup's meta rows
    const int rel = col0 - colwg;
    const int my_b = rel + lane, my_v = ((rel >> 2) + b) >> p.lshift;
    uint32_t l_lane = (uint32_t)(i * 16);
    // opaque, so that a step's row offset stays one multiply-add: knowing the low bits, the compiler
    // splits it into a multiply and an OR, and every vector instruction between the MFMAs costs
    // about four of their cycles
    asm volatile("" : "+v"(l_lane));
    // The A operands travel through a ring of kRing quarter-steps (one 128-bit read = the operands
    // of four MFMAs): the read for quarter j + kRing - 1 is issued right before the MFMAs of quarter
    // j, i.e. kRing - 1 groups of four 8-cycle MFMAs ahead of its use, with 4 kRing registers.
    constexpr int kRing = 4;
    gfloatx4 ring[kRing];
    // step t of the chunk lies in window t / NK of it; lane (b, i), quarter q: rows 16 q + 4 i .. 4 i + 3.
    // One full-rate multiply-add per step; the window's offset is an immediate of the read.
    auto row_offset = [&](int k_local, uint32_t base) { return __umul24((uint32_t)k_local, (uint32_t)STRIDE) + base; };
    auto read_quarter = [&](int t, int q, uint32_t off) {
        return *(const gfloatx4*)(lds + off + (t / NK) * MWIN * STRIDE + q * 64);
    };

    // No vector-memory instruction between the MFMAs of a phase except the fetches for the next
    // phase and chunk, which nothing in the phase waits for: index and B value come from LDS.
    // (Measured: two 32-bit global loads per step cost the matrix pipes 14 % of their time however
    // far ahead they are issued; an LDS read costs about one cycle.)
    fetch_meta(0);
    fetch_chunk(0);
    store_chunk();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows of B and indices have landed in LDS
    __syncthreads();
    for (int c = 0; c < c_count; ++c) {
        if (c + 1 < c_count)
            fetch_chunk(c + 1);   // into registers: A has one buffer, stored after the chunk's last barrier
        // The phases of a chunk run as a loop (its body is the eight steps, unrolled): a phase starts
        // on a window boundary whenever eight is a multiple of the kept rows per window, and then only
        // the base of its LDS offsets changes.  (3:8: windows straddle phases, the loop is unrolled.)
        constexpr bool kRolled = PH % NK == 0;
#pragma unroll(kRolled ? 1 : P)
        for (int h = 0; h < P; ++h) {
            const int g = c * P + h, half = g & 1;
            const int hs = kRolled ? 0 : h;   // compile-time step base of the phase (rolled: in l_phase)
            uint32_t l_phase = l_lane + (kRolled ? (uint32_t)(h * (PH / NK) * MWIN * STRIDE) : 0u);
            asm volatile("" : "+v"(l_phase));   // one register, for the same reason
            if (g + 1 < phases)
                fetch_meta(g + 1);   // the other half: free since the barrier that ended the phase before
            const float* const mb = lds_b + half * PH * kGatherCols + my_b;
            const int32_t* const mi = lds_i + half * PH * 64 + my_v;
            // quarter j of the phase = step j / 4, rows 16 (j % 4) ..; off[] holds the row offsets of
            // the steps whose quarters are in flight (at most two steps at a time)
            constexpr int Q = PH * 4;
            static_assert(kRing <= 9, "reads reach at most two steps ahead");
            // row offsets of this step and the two after it
            uint32_t off0 = row_offset(mi[0], l_phase), off1 = PH > 1 ? row_offset(mi[64], l_phase) : 0u,
                     off2 = PH > 2 ? row_offset(mi[128], l_phase) : 0u;
            float bv_cur = mb[0], bv_next = 0.0f;
#pragma unroll
            for (int j = 0; j < kRing - 1; ++j)
                ring[j] = read_quarter(hs * PH + j / 4, j % 4, j / 4 == 0 ? off0 : j / 4 == 1 ? off1 : off2);
#pragma unroll
            for (int j = 0; j < Q; ++j) {
                const int t = j / 4, q = j % 4;
                const int ahead = j + kRing - 1;       // the quarter whose read is issued now
                if (ahead < Q)
                    ring[ahead % kRing] = read_quarter(hs * PH + ahead / 4, ahead % 4,
                                                       ahead / 4 == t ? off0 : ahead / 4 == t + 1 ? off1 : off2);
                if (q == 0 && t + 1 < PH)
                    bv_next = mb[(t + 1) * kGatherCols];
                __builtin_amdgcn_sched_barrier(0);  // reads are issued where they are written, ahead of these MFMAs
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc[4 * q + e] = __builtin_amdgcn_mfma_f32_4x4x1f32(ring[j % kRing][e], bv_cur, acc[4 * q + e], 0, 0, 0);
                if (q == 3) {          // the step is over: shift the per-step values
                    bv_cur = bv_next;
                    off0 = off1;
                    off1 = off2;
                    if (t + 3 < PH)
                        off2 = row_offset(mi[(t + 3) * 64], l_phase);
                }
            }
            if (h + 1 < P) {
                // the next phase's meta rows have landed (this wave's part) and every wave is done
                // with this phase's half, which the phase after next overwrites
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
            }
        }
        __syncthreads();  // every wave is done with A's chunk and with the last phase's half
        store_chunk();
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
    const int chunk = gather_chunk(a.window, a.kept);
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
    p.nchunk = a.K / gather_chunk(MWIN, NK);
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
