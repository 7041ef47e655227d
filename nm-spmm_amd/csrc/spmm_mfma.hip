// Matrix-core kernels for C = A . B with an N:M-sparse B whose index pattern is shared by 32
// adjacent columns (reference kernels: src/kernel_{64x128_8x8,64x64_8x8,32x64_8x4,32x32_4x4}.cu;
// this file replaces their role, not their design).
//
// Design for gfx950 (64-lane waves, v_mfma_f32_32x32x2_f32):
//  * A 32-column index vector is exactly the N extent of one 32x32x2 MFMA, so one wave owns one
//    column vector and RM row blocks of 32 rows.  Its A operand for one MFMA is A[row][k] with
//    lane = (row % 32, k half): lanes 0-31 take compressed row 2s, lanes 32-63 row 2s+1, and each
//    half reads the LDS row of A that *its* index selects.  The gather is therefore just a
//    per-lane LDS row offset; no data is moved to perform it.
//  * The wave's RM row blocks interleave rows (block b holds rows 4*r + b, a 256-row wave two
//    such groups), so one 128-bit LDS read yields the A operands of four blocks and the B
//    operand is reused RM times.
//  * The A tile (window rows x Ms, k-major as in global memory) is shared by the tile's column
//    vectors, so it is staged global -> registers -> LDS with 128-bit accesses, double
//    buffered: the loads of window t+1 are in flight while window t is multiplied, one barrier
//    per window.  A B element is consumed by exactly one wave, so B never touches LDS: each
//    lane loads its MFMA operands (two 128-byte row segments per wave and k-step) straight
//    from global memory one window ahead.
//  * High-sparsity layout: only the rows listed in column_info are staged (the indices are
//    already ranks into that list); column_info is fetched two windows ahead.
//  * Workgroup ids are remapped so that the tiles resident on one XCD form a compact patch of
//    C and share A / B panels in that XCD's L2.
#include "internal.h"

namespace nmspmm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kXcds = 8;

struct MfmaParams {
    const float* A;
    const float* B;
    const int32_t* D;
    const int32_t* cinfo;
    float* out;          // C, or the first partial slice when split_k > 1
    size_t slice_elems;  // M * N
    int M, N, W;
    int nwin;            // windows in the whole reduction
    int split_k;
    int tiles_m, tiles_n;
};

struct float8 { float4 lo, hi; };
template <int RM> struct AFrag;
template <> struct AFrag<8> { typedef float8 type; };
template <> struct AFrag<4> { typedef float4 type; };
template <> struct AFrag<2> { typedef float2 type; };
template <> struct AFrag<1> { typedef float type; };

template <typename F> __device__ inline F load_frag(const float* p) { return *reinterpret_cast<const F*>(p); }
template <> __device__ inline float8 load_frag<float8>(const float* p)
{
    float8 f;
    f.lo = *reinterpret_cast<const float4*>(p);
    f.hi = *reinterpret_cast<const float4*>(p + 128);
    return f;
}
__device__ inline float frag_get(const float4& v, int i);
__device__ inline float frag_get(const float8& v, int i) { return i < 4 ? frag_get(v.lo, i) : frag_get(v.hi, i - 4); }
__device__ inline float frag_get(const float4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
__device__ inline float frag_get(const float2& v, int i) { return i == 0 ? v.x : v.y; }
__device__ inline float frag_get(const float& v, int) { return v; }

// KS: dense rows per window, WS: kept rows per window, QS: column vectors per workgroup tile
// (Ns = 32*QS, the width the indices were preprocessed for), WR: waves along M, RM: 32-row
// blocks per wave, HIGH: high-sparsity layout.
template <int KS, int WS, int QS, int WR, int RM, bool HIGH>
struct TileCfg {
    static constexpr int MS = WR * RM * 32;
    static constexpr int NS = QS * 32;
    static constexpr int NT = 64 * QS * WR;
    static constexpr int AROWS = HIGH ? (KS < WS * QS ? KS : WS * QS) : KS;
    static constexpr int ASTR = MS;       // floats per staged A row
    static constexpr int A_F4_ROW = MS / 4;
    static constexpr int A_F4 = AROWS * A_F4_ROW;
    static constexpr int A_SLOTS = (A_F4 + NT - 1) / NT;
    static constexpr int KSTEPS = WS / 2;
    static constexpr size_t LDS_BYTES = sizeof(float) * 2 * (size_t)(AROWS * ASTR);
    static_assert(WS % 2 == 0, "two compressed rows per MFMA");
};

// The buffers of the multi-buffered A tile are separate LDS objects (not one array indexed by
// t % NBUF): the compiler can then prove that the fragment reads of one buffer do not alias the
// asynchronous global->LDS writes into another and does not serialise them with a vmcnt(0)
// wait.  They live at namespace scope, one set per tile size in floats; a kernel is charged
// only for the buffers it references.
#define NMSPMM_LDS_SET(FLOATS)                                                  \
    __shared__ __align__(16) float g_lds_a0_##FLOATS[FLOATS];                  \
    __shared__ __align__(16) float g_lds_a1_##FLOATS[FLOATS];                  \
    __shared__ __align__(16) float g_lds_a2_##FLOATS[FLOATS];                  \
    template <> struct LdsSet<FLOATS> {                                         \
        __device__ static float* buf0() { return g_lds_a0_##FLOATS; }          \
        __device__ static float* buf1() { return g_lds_a1_##FLOATS; }          \
        __device__ static float* buf2() { return g_lds_a2_##FLOATS; }          \
    };
template <int FLOATS> struct LdsSet;
NMSPMM_LDS_SET(1024)
NMSPMM_LDS_SET(2048)
NMSPMM_LDS_SET(4096)
NMSPMM_LDS_SET(8192)
NMSPMM_LDS_SET(16384)
NMSPMM_LDS_SET(32768)

// Buffer descriptors give branch-free guarded loads: an offset at or beyond num_records reads 0
// without touching memory, so "this slot has nothing to load" is just an out-of-range offset.
__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ inline float4 buffer_load_f4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off)
{
    auto v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0);
    return *reinterpret_cast<float4*>(&v);
}
typedef __attribute__((address_space(3))) float lds_f32;
__device__ inline float buffer_load_f1(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, uint32_t s_off)
{
    return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, byte_off, s_off, 0));
}
// 128-bit global -> LDS load without a register stop-over: lane l's 16 bytes land at
// dst + 16*l (dst is wave-uniform).  Completion is tracked by vmcnt.  Kept out of the kernel
// template: the host pass drops a kernel template that names this builtin directly.
__device__ inline void buffer_load_f4_to_lds(__amdgpu_buffer_rsrc_t r, lds_f32* dst, uint32_t byte_off)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst, 16, byte_off, 0, 0, 0);
}
constexpr uint32_t kNoLoad = 0x80000000u;  // beyond any window's num_records
constexpr int kWaitVm0 = 0x0F70;           // s_waitcnt vmcnt(0), other counters untouched

// Tuning knobs (compile-time): minimum waves per SIMD the register allocation must allow, the
// tile-walk band height, and the (waves along M, 32-row blocks per wave) of each tile width.
#ifndef NMSPMM_OCC
#define NMSPMM_OCC 3
#endif
#ifndef NMSPMM_LDS_MIN
#define NMSPMM_LDS_MIN 0  // extra dynamic LDS bytes to claim (caps workgroups per CU)
#endif
#ifndef NMSPMM_NBUF
#define NMSPMM_NBUF 2       // LDS buffers of the A tile, 128-row waves
#endif
#ifndef NMSPMM_NBUF_TALL
#define NMSPMM_NBUF_TALL 2  // same for 256-row waves
#endif
#ifndef NMSPMM_TALL
#define NMSPMM_TALL 1  // allow 256-row waves
#endif
#ifndef NMSPMM_GATHER
#define NMSPMM_GATHER 1          // high-sparsity layout: wave-private gather kernel
#endif
#ifndef NMSPMM_DIRECT_LOW
#define NMSPMM_DIRECT_LOW 0
#endif
#ifndef NMSPMM_GATHER_RM_TALL
#define NMSPMM_GATHER_RM_TALL 8  // its wave height (32-row blocks) for large problems
#endif
#ifndef NMSPMM_GROUP
#define NMSPMM_GROUP 8
#endif
#ifndef NMSPMM_CFG128
#define NMSPMM_CFG128 1, 4
#endif
#ifndef NMSPMM_CFG64
#define NMSPMM_CFG64 2, 2
#endif
#ifndef NMSPMM_CFG32
#define NMSPMM_CFG32 4, 1
#endif

// NBUF: LDS buffers of the A tile.  2: the tile of window t+1 is loaded while window t is
// multiplied and must have landed when the iteration ends.  3: the tile of window t+2 is loaded
// during window t, its loads are spread between the MFMAs and have a whole further iteration to
// land, so memory issue and the matrix pipe overlap inside one wave.
template <int KS, int WS, int QS, int WR, int RM, bool HIGH, int NBUF>
__global__ void __launch_bounds__(64 * QS * WR, NMSPMM_OCC)
spmm_mfma_kernel(const MfmaParams p)
{
    typedef TileCfg<KS, WS, QS, WR, RM, HIGH> T;
    static_assert(NBUF == 2 || NBUF == 3, "double or triple buffering");
    static_assert(T::A_F4 % T::NT == 0, "every wave issues the same number of A loads");
    typedef typename AFrag<RM>::type afrag_t;
    float* const As0 = LdsSet<T::AROWS * T::ASTR>::buf0();
    float* const As1 = LdsSet<T::AROWS * T::ASTR>::buf1();
    float* const As2 = NBUF == 3 ? LdsSet<T::AROWS * T::ASTR>::buf2() : nullptr;

    // ---- which tile -------------------------------------------------------------------------
    // Consecutive workgroup ids go to consecutive XCDs; give every XCD a contiguous run of
    // logical tile ids, then walk the tiles in bands of GROUP tile-rows.
    const int total = p.tiles_m * p.tiles_n;
    int logical;
    {
        const int id = blockIdx.x;
        const int q = total / kXcds, r = total % kXcds;
        const int xcd = id % kXcds, loc = id / kXcds;
        logical = xcd < r ? xcd * (q + 1) + loc : r * (q + 1) + (xcd - r) * q + loc;
    }
    constexpr int GROUP = NMSPMM_GROUP;
    int tile_m, tile_n;
    {
        const int band = logical / (GROUP * p.tiles_n);
        const int first_m = band * GROUP;
        const int rows = min(GROUP, p.tiles_m - first_m);
        const int in_band = logical - band * GROUP * p.tiles_n;
        tile_m = first_m + in_band % rows;
        tile_n = in_band / rows;
    }
    const int bi = tile_m * T::MS;
    const int bj = tile_n * T::NS;

    int w_begin, w_count;
    split_windows(p.nwin, p.split_k, blockIdx.y, &w_begin, &w_count);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int vec = wave % QS;   // column vector inside the tile
    const int grp = wave / QS;   // row group inside the tile
    const int h = lane >> 5;     // which of the two compressed rows of a k-step
    const int j = lane & 31;

    const int M = p.M, N = p.N;
    const float* const Ablk = p.A + bi;
    const float* const Bvec = p.B + bj + vec * 32;
    const int32_t* const Cinfo = HIGH ? p.cinfo + (size_t)tile_n * p.nwin * KS : nullptr;
    // Bytes addressable from the first element of a window's A tile / B vector.  Columns past
    // M in an A row that is not the last one alias the next row (finite garbage that only
    // reaches C rows >= M, which are never stored); the descriptor bound keeps the last row
    // inside the matrix.
    const uint32_t a_bytes = (uint32_t)(((size_t)(KS - 1) * M + (M - bi)) * sizeof(float));
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));

    // ---- A staging: global -> LDS without passing through registers -------------------------------
    // Slot s of wave `wave` is the 1 KiB chunk number wave + s*NW of the [AROWS][MS] tile: float4
    // number 64*chunk + lane, which is also where an LDS-direct 128-bit load puts lane's data.
    // HIGH: staged row r of window w is A row column_info[w][r]; -1 means "no such row".  One
    // wave-wide load brings the whole list (KS = 64 entries, lane l holds entry l) two windows
    // ahead; readlane hands every lane the entry of the row its load slot covers.  Load offsets
    // are formed right before use so that nothing per slot stays live across the multiplication.
    constexpr int NW = T::NT / 64;
    constexpr int RPC = T::A_F4_ROW < 64 ? 64 / T::A_F4_ROW : 1;  // tile rows per 1 KiB chunk
    int ci_vec = -1;  // HIGH: column_info of the window whose A tile is loaded next
    int ci_nxt = -1;  //       and of the one after it (in flight)
    auto load_cinfo = [&](int w) {
        const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cinfo + (size_t)w * KS, KS * sizeof(int32_t));
        ci_nxt = __builtin_amdgcn_raw_buffer_load_b32(rc, lane * (int)sizeof(int32_t), 0, 0);
    };
    // Byte offset of every load slot inside its window.  LOW: fixed.  HIGH: formed from ci_vec;
    // with few slots at the end of an iteration, where the readlanes and integer ops run under
    // the tail of the MFMA phase instead of in front of the next iteration's loads (EARLY); with
    // many slots right before each load, so that they do not all stay live across the MFMAs.
    constexpr bool EARLY = !HIGH || T::A_SLOTS <= 8;
    uint32_t a_off[EARLY ? T::A_SLOTS : 1];
    auto slot_offset = [&](int s) -> uint32_t {
        const int chunk = wave + s * NW;
        const int r0 = chunk * 64 / T::A_F4_ROW;  // first tile row of the chunk (wave-uniform)
        const int f4 = lane % T::A_F4_ROW + (T::A_F4_ROW > 64 ? (chunk * 64) % T::A_F4_ROW : 0);
        int src = r0 + lane / T::A_F4_ROW;
        if (HIGH) {
            src = __builtin_amdgcn_readlane(ci_vec, r0 & 63);
#pragma unroll
            for (int g = 1; g < RPC; ++g) {
                const int v = __builtin_amdgcn_readlane(ci_vec, (r0 + g) & 63);
                src = (lane / T::A_F4_ROW == g) ? v : src;
            }
        }
        return src >= 0 ? (uint32_t)(((size_t)src * M + f4 * 4) * sizeof(float)) : kNoLoad;
    };
    auto form_a_offsets = [&]() {
        if (EARLY) {
#pragma unroll
            for (int s = 0; s < T::A_SLOTS; ++s)
                a_off[s] = slot_offset(s);
        }
    };
    auto load_a = [&](int w, float* dst) {
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ablk + (size_t)w * KS * M, a_bytes);
        lds_f32* Ab = (lds_f32*)dst + wave * 256;
#pragma unroll
        for (int s = 0; s < T::A_SLOTS; ++s)
            buffer_load_f4_to_lds(ra, Ab + s * NW * 256, EARLY ? a_off[s] : slot_offset(s));
    };

    // ---- per-wave operands that bypass LDS ---------------------------------------------------------
    // B values of compressed rows 2s + h come one dword per lane.  The window's index block
    // ([WS][QS] ints, contiguous) comes as one wave-wide load per 64 entries; readlane then
    // gives lane (h, j) the index of row 2s + h of this wave's column vector.
    constexpr int ND = (WS * QS + 63) / 64;
    float b_next[T::KSTEPS];
    int d_next[ND];
    const uint32_t b_lane = (uint32_t)(((size_t)h * N + j) * sizeof(float));
    const uint32_t b_step = (uint32_t)(2 * (size_t)N * sizeof(float));
    const int32_t* const Dblk = p.D + (size_t)tile_n * p.W * QS;
    auto load_b_idx = [&](int w) {
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bvec + (size_t)w * WS * N, b_bytes);
        const __amdgpu_buffer_rsrc_t rd = make_rsrc(Dblk + (size_t)w * WS * QS, WS * QS * sizeof(int32_t));
        uint32_t off = b_lane;
#pragma unroll
        for (int s = 0; s < T::KSTEPS; ++s, off += b_step)
            b_next[s] = buffer_load_f1(rb, off, 0);
#pragma unroll
        for (int q = 0; q < ND; ++q)
            d_next[q] = __builtin_amdgcn_raw_buffer_load_b32(rd, (lane + 64 * q) * (int)sizeof(int32_t), 0, 0);
    };

    int aoff[T::KSTEPS];
    float bv[T::KSTEPS];
    // A lane owns runs of up to four adjacent rows, so that the 64 lanes of one 128-bit read cover
    // contiguous LDS; a 256-row wave tile (RM = 8) is two such runs 128 rows apart.
    constexpr int RUN = RM < 4 ? RM : 4;
    const int a_lane = grp * (RM * 32) + j * RUN;
    auto take_b_idx = [&]() {
#pragma unroll
        for (int s = 0; s < T::KSTEPS; ++s) {
            const int e0 = 2 * s * QS, e1 = (2 * s + 1) * QS;  // entries of rows 2s, 2s+1, vector 0
            const int lo = __builtin_amdgcn_readlane(d_next[e0 / 64], e0 % 64 + vec);
            const int hi = __builtin_amdgcn_readlane(d_next[e1 / 64], e1 % 64 + vec);
            aoff[s] = (h ? hi : lo) * T::ASTR + a_lane;
            bv[s] = b_next[s];
        }
    };

    floatx16 acc[RM];
#pragma unroll
    for (int b = 0; b < RM; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[b][v] = 0.0f;

    // ---- prologue: windows 0 .. DA-1 of the slice into their buffers ---------------------------------
    constexpr int DA = NBUF - 1;  // how many windows ahead of the multiplication the A tile is loaded
    const int w_last = w_begin + w_count - 1;
    if (w_count > 0) {
        if (HIGH) {
            load_cinfo(w_begin);
            ci_vec = ci_nxt;
        }
        form_a_offsets();
        load_a(w_begin, As0);
        if (NBUF == 3) {
            if (HIGH) {
                load_cinfo(min(w_begin + 1, w_last));
                ci_vec = ci_nxt;
                form_a_offsets();
            }
            load_a(min(w_begin + 1, w_last), As1);
        }
        load_b_idx(w_begin);
        if (HIGH) {
            load_cinfo(min(w_begin + DA, w_last));
            ci_vec = ci_nxt;
            form_a_offsets();
        }
        take_b_idx();
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm0);
    __syncthreads();

    // ---- main loop: one window per iteration --------------------------------------------------
    // The body is one basic block: loads for later windows are always issued (past the end of the
    // slice they re-read its last window into an idle buffer, which is harmless).  Per iteration:
    // B, index and column_info loads for the next window first (few bytes, they have the whole
    // iteration to land), then the MFMAs of this window with the LDS-direct loads of the A tile DA
    // windows ahead; the wave waits for what the next iteration needs, then the barrier publishes
    // it to the other waves.
    constexpr int kWaitTile = NBUF == 2 ? 0 : T::A_SLOTS;  // NBUF 3: this iteration's A loads may stay in flight
    // s_waitcnt vmcnt(kWaitTile) lgkmcnt(0): the loads the next iteration depends on have landed and
    // every LDS read of this wave has executed, so after the barrier the buffer it read may be
    // overwritten.  The barrier is the bare instruction: __syncthreads() carries a release fence
    // that waits for ALL outstanding loads, including the tile loads meant to stay in flight.
    constexpr int kWaitImm = (kWaitTile & 15) | (7 << 4) | (0 << 8) | ((kWaitTile >> 4) << 14);
    auto window = [&](int t, const float* cur, float* dst) {
        const int w = w_begin + t;
        if (NBUF == 2)
            load_a(min(w + 1, w_last), dst);
        load_b_idx(min(w + 1, w_last));
        if (HIGH)
            load_cinfo(min(w + DA + 1, w_last));
        if (NBUF == 2) {
            // Keep the loads ahead of the multiplication: they need the whole MFMA phase to land.
            __builtin_amdgcn_sched_barrier(0);
        }

        afrag_t av[T::KSTEPS];
#pragma unroll
        for (int s = 0; s < T::KSTEPS; ++s)
            av[s] = load_frag<afrag_t>(cur + aoff[s]);
        if (NBUF == 3)
            load_a(min(w + DA, w_last), dst);
#pragma unroll
        for (int s = 0; s < T::KSTEPS; ++s) {
#pragma unroll
            for (int b = 0; b < RM; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_get(av[s], b), bv[s], acc[b], 0, 0, 0);
        }
        if (NBUF == 3) {
            // Issue order: the small loads, two fragment reads, then per k-step its MFMAs, a share
            // of the A-tile loads and the fragment reads of a later k-step.
            constexpr int FR = RM == 8 ? 2 : 1;  // LDS reads per fragment
            constexpr int DPS = (T::A_SLOTS + T::KSTEPS - 1) / T::KSTEPS;
            __builtin_amdgcn_sched_group_barrier(0x020, T::KSTEPS + ND + (HIGH ? 1 : 0), 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2 * FR, 0);
#pragma unroll
            for (int s = 0; s < T::KSTEPS; ++s) {
                __builtin_amdgcn_sched_group_barrier(0x008, RM, 0);
                if (s * DPS < T::A_SLOTS)
                    __builtin_amdgcn_sched_group_barrier(0x020, DPS, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, FR, 0);
            }
        }

        // Nothing below may drift up: it consumes what was loaded at the top of this iteration.
        __builtin_amdgcn_sched_barrier(0);
        take_b_idx();
        if (HIGH) {
            ci_vec = ci_nxt;
            form_a_offsets();
        }
        __builtin_amdgcn_s_waitcnt(kWaitImm);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    if (NBUF == 2) {
        for (int t = 0; t < w_count; t += 2) {
            window(t, As0, As1);
            if (t + 1 < w_count)
                window(t + 1, As1, As0);
        }
    } else {
        for (int t = 0; t < w_count; t += 3) {
            window(t, As0, As2);
            if (t + 1 < w_count)
                window(t + 1, As1, As0);
            if (t + 2 < w_count)
                window(t + 2, As2, As1);
        }
    }

    // ---- epilogue -----------------------------------------------------------------------------
    // MFMA result register v of lane (h, j) is row 8*(v/4) + 4*h + v%4, column j of the 32x32
    // block; block b holds tile rows 128*(b/4) + RUN*row + b%4 of this wave's row group.
    float* out = p.out + (size_t)blockIdx.y * p.slice_elems;
    const int col = bj + vec * 32 + j;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int r32 = 8 * (v / 4) + 4 * h + (v % 4);
#pragma unroll
        for (int b = 0; b < RM; ++b) {
            const int row = bi + grp * (RM * 32) + (b / 4) * 128 + r32 * RUN + (b % 4);
            if (row < M)
                out[(size_t)row * N + col] = acc[b][v];
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Wave-private gather kernel for the high-sparsity layout.
//
// At 75 % sparsity and above a column vector touches only WS of a window's 64 rows, so the rows one
// wave needs (WS per window) are about as many bytes as its quarter share of the workgroup's
// compacted tile.  Each wave therefore stages ITS OWN rows: the gather happens in the global
// address of the LDS-direct load (row = column_info[rank]), the rows land in kept order in a
// region of LDS that only this wave reads, the MFMA operand reads use fixed addresses, and the
// window loop needs no barrier and no cross-wave wait at all: waves drift apart and their memory
// and matrix phases overlap on the CU.
//
// One workgroup = QS waves = one 32-column vector each, RM*32 rows tall.  Two LDS objects (window
// parity) so that the compiler can tell the reads of one from the asynchronous writes into the other.
template <int FLOATS> struct LdsPairG;
#define NMSPMM_LDS_PAIRG(FLOATS)                                                \
    __shared__ __align__(16) float g_lds_g0_##FLOATS[FLOATS];                  \
    __shared__ __align__(16) float g_lds_g1_##FLOATS[FLOATS];                  \
    template <> struct LdsPairG<FLOATS> {                                       \
        __device__ static float* even() { return g_lds_g0_##FLOATS; }          \
        __device__ static float* odd() { return g_lds_g1_##FLOATS; }           \
    };
NMSPMM_LDS_PAIRG(1024)
NMSPMM_LDS_PAIRG(2048)
NMSPMM_LDS_PAIRG(4096)
NMSPMM_LDS_PAIRG(8192)
NMSPMM_LDS_PAIRG(16384)

__device__ inline void buffer_load_f4_to_lds_s(__amdgpu_buffer_rsrc_t r, lds_f32* dst, uint32_t v_off, uint32_t s_off)
{
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, dst, 16, v_off, s_off, 0, 0);
}

template <int KS, int WS, int QS, int RM>
__global__ void __launch_bounds__(64 * QS, NMSPMM_OCC)
spmm_gather_kernel(const MfmaParams p)
{
    static_assert(RM == 4 || RM == 8, "128- or 256-row waves");
    typedef typename AFrag<RM>::type afrag_t;
    constexpr int MS = RM * 32;
    constexpr int NS = QS * 32;
    constexpr int KSTEPS = WS / 2;
    constexpr int RPI = 256 / MS;            // rows per 1 KiB load: 1 (256-row waves) or 2
    constexpr int A_SLOTS = WS / RPI;
    constexpr int ND = (WS * QS + 63) / 64;
    constexpr int WAVE_FLOATS = WS * MS;     // one window of one wave
    float* const L0 = LdsPairG<QS * WAVE_FLOATS>::even();
    float* const L1 = LdsPairG<QS * WAVE_FLOATS>::odd();

    // ---- which tile (same walk as the shared-tile kernel) ---------------------------------------
    const int total = p.tiles_m * p.tiles_n;
    int logical;
    {
        const int id = blockIdx.x;
        const int q = total / kXcds, r = total % kXcds;
        const int xcd = id % kXcds, loc = id / kXcds;
        logical = xcd < r ? xcd * (q + 1) + loc : r * (q + 1) + (xcd - r) * q + loc;
    }
    constexpr int GROUP = NMSPMM_GROUP;
    int tile_m, tile_n;
    {
        const int band = logical / (GROUP * p.tiles_n);
        const int first_m = band * GROUP;
        const int rows = min(GROUP, p.tiles_m - first_m);
        const int in_band = logical - band * GROUP * p.tiles_n;
        tile_m = first_m + in_band % rows;
        tile_n = in_band / rows;
    }
    const int bi = tile_m * MS;
    const int bj = tile_n * NS;
    int w_begin, w_count;
    split_windows(p.nwin, p.split_k, blockIdx.y, &w_begin, &w_count);
    const int w_last = w_begin + w_count - 1;

    const int lane = threadIdx.x & 63;
    const int vec = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave = column vector
    const int h = lane >> 5;
    const int j = lane & 31;
    const int M = p.M, N = p.N;
    const float* const Ablk = p.A + bi;
    const float* const Bvec = p.B + bj + vec * 32;
    const int32_t* const Dblk = p.D + (size_t)tile_n * p.W * QS;
    const int32_t* const Cinfo = p.cinfo + (size_t)tile_n * p.nwin * KS;
    const uint32_t a_bytes = (uint32_t)(((size_t)(KS - 1) * M + (M - bi)) * sizeof(float));
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));
    const uint32_t b_lane = (uint32_t)(((size_t)h * N + j) * sizeof(float));
    const uint32_t b_step = (uint32_t)(2 * (size_t)N * sizeof(float));
    const uint32_t row_bytes = (uint32_t)((size_t)M * sizeof(float));
    const uint32_t a_vlane = (uint32_t)((lane % (MS / 4)) * 16);  // this lane's 16 bytes inside a row

    // metadata one window ahead of the loads that use it: ranks of this block's vectors and the
    // block's row list, one wave-wide load each
    int d_vec[ND], d_nxt[ND], ci_vec = -1, ci_nxt = -1;
    auto load_meta = [&](int w) {
        const __amdgpu_buffer_rsrc_t rd = make_rsrc(Dblk + (size_t)w * WS * QS, WS * QS * sizeof(int32_t));
#pragma unroll
        for (int q = 0; q < ND; ++q)
            d_nxt[q] = __builtin_amdgcn_raw_buffer_load_b32(rd, (lane + 64 * q) * (int)sizeof(int32_t), 0, 0);
        const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cinfo + (size_t)w * KS, KS * sizeof(int32_t));
        ci_nxt = __builtin_amdgcn_raw_buffer_load_b32(rc, lane * (int)sizeof(int32_t), 0, 0);
    };
    auto take_meta = [&]() {
#pragma unroll
        for (int q = 0; q < ND; ++q)
            d_vec[q] = d_nxt[q];
        ci_vec = ci_nxt;
    };
    // window-local A row of kept row p of this wave's vector (wave-uniform)
    auto row_of = [&](int pp) -> int {
        const int e = pp * QS;
        const int rank = __builtin_amdgcn_readlane(d_vec[e / 64], e % 64 + vec);
        return __builtin_amdgcn_readlane(ci_vec, rank & 63);
    };
    // the wave's WS rows of window w -> dst (kept order), gathered by the load addresses
    auto load_rows = [&](int w, float* dst) {
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ablk + (size_t)w * KS * M, a_bytes);
        lds_f32* Ab = (lds_f32*)dst + vec * WAVE_FLOATS;
#pragma unroll
        for (int s = 0; s < A_SLOTS; ++s) {
            if (RPI == 1) {
                buffer_load_f4_to_lds_s(ra, Ab + s * 256, a_vlane, (uint32_t)row_of(s) * row_bytes);
            } else {
                const int r0 = row_of(2 * s), r1 = row_of(2 * s + 1);
                buffer_load_f4_to_lds(ra, Ab + s * 256, (uint32_t)(h ? r1 : r0) * row_bytes + a_vlane);
            }
        }
    };
    float b_next[KSTEPS], bv[KSTEPS];
    auto load_b = [&](int w) {
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bvec + (size_t)w * WS * N, b_bytes);
        uint32_t off = b_lane;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s, off += b_step)
            b_next[s] = buffer_load_f1(rb, off, 0);
    };

    floatx16 acc[RM];
#pragma unroll
    for (int b = 0; b < RM; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[b][v] = 0.0f;

    // fixed operand address: kept row 2s + h, this lane's runs of four rows
    const int a_lane = vec * WAVE_FLOATS + h * MS + j * 4;

    if (w_count > 0) {
        load_meta(w_begin);
        take_meta();
        load_rows(w_begin, L0);
        load_b(w_begin);
        load_meta(min(w_begin + 1, w_last));
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            bv[s] = b_next[s];
        take_meta();
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm0);

    auto window = [&](int t, const float* cur, float* nxt) {
        const int w = w_begin + t;
        load_rows(min(w + 1, w_last), nxt);
        load_b(min(w + 1, w_last));
        load_meta(min(w + 2, w_last));
        __builtin_amdgcn_sched_barrier(0);

        afrag_t av[KSTEPS];
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            av[s] = load_frag<afrag_t>(cur + a_lane + 2 * s * MS);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
#pragma unroll
            for (int b = 0; b < RM; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_get(av[s], b), bv[s], acc[b], 0, 0, 0);
        }

        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            bv[s] = b_next[s];
        take_meta();
        // own loads landed, own LDS reads executed: the other buffer may be read, this one refilled
        __builtin_amdgcn_s_waitcnt(0x0070);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int t = 0; t < w_count; t += 2) {
        window(t, L0, L1);
        if (t + 1 < w_count)
            window(t + 1, L1, L0);
    }

    float* out = p.out + (size_t)blockIdx.y * p.slice_elems;
    const int col = bj + vec * 32 + j;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int r32 = 8 * (v / 4) + 4 * h + (v % 4);
#pragma unroll
        for (int b = 0; b < RM; ++b) {
            const int row = bi + (b / 4) * 128 + r32 * 4 + (b % 4);
            if (row < M)
                out[(size_t)row * N + col] = acc[b][v];
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Direct gather kernel for the high-sparsity layout: the same wave-private idea without LDS.  A
// lane's MFMA operand for k-step s is 16 contiguous bytes of A row column_info[rank(2s+h)], so it
// is loaded straight into the operand registers (128-bit loads, two 512-byte row segments per wave
// and instruction), one window ahead.  No LDS, no barrier, and the only memory instructions left
// are the operand loads themselves.
template <int KS, int WS, int QS, int RM, bool HIGH>
__global__ void __launch_bounds__(64 * QS, RM == 8 ? 2 : NMSPMM_OCC)
spmm_direct_kernel(const MfmaParams p)
{
    static_assert(RM == 4 || RM == 8, "128- or 256-row waves");
    typedef typename AFrag<RM>::type afrag_t;
    constexpr int MS = RM * 32;
    constexpr int NS = QS * 32;
    constexpr int KSTEPS = WS / 2;
    constexpr int ND = (WS * QS + 63) / 64;

    const int total = p.tiles_m * p.tiles_n;
    int logical;
    {
        const int id = blockIdx.x;
        const int q = total / kXcds, r = total % kXcds;
        const int xcd = id % kXcds, loc = id / kXcds;
        logical = xcd < r ? xcd * (q + 1) + loc : r * (q + 1) + (xcd - r) * q + loc;
    }
    constexpr int GROUP = NMSPMM_GROUP;
    int tile_m, tile_n;
    {
        const int band = logical / (GROUP * p.tiles_n);
        const int first_m = band * GROUP;
        const int rows = min(GROUP, p.tiles_m - first_m);
        const int in_band = logical - band * GROUP * p.tiles_n;
        tile_m = first_m + in_band % rows;
        tile_n = in_band / rows;
    }
    const int bi = tile_m * MS;
    const int bj = tile_n * NS;
    int w_begin, w_count;
    split_windows(p.nwin, p.split_k, blockIdx.y, &w_begin, &w_count);
    const int w_last = w_begin + w_count - 1;

    const int lane = threadIdx.x & 63;
    const int vec = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int h = lane >> 5;
    const int j = lane & 31;
    const int M = p.M, N = p.N;
    const float* const Ablk = p.A + bi;
    const float* const Bvec = p.B + bj + vec * 32;
    const int32_t* const Dblk = p.D + (size_t)tile_n * p.W * QS;
    const int32_t* const Cinfo = HIGH ? p.cinfo + (size_t)tile_n * p.nwin * KS : nullptr;
    const uint32_t a_bytes = (uint32_t)(((size_t)(KS - 1) * M + (M - bi)) * sizeof(float));
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));
    const uint32_t b_lane = (uint32_t)(((size_t)h * N + j) * sizeof(float));
    const uint32_t b_step = (uint32_t)(2 * (size_t)N * sizeof(float));
    const uint32_t row_bytes = (uint32_t)((size_t)M * sizeof(float));
    const uint32_t a_vlane = (uint32_t)(j * 16);  // this lane's run of four rows inside the tile

    int d_vec[ND], d_nxt[ND], ci_vec = -1, ci_nxt = -1;
    auto load_meta = [&](int w) {
        const __amdgpu_buffer_rsrc_t rd = make_rsrc(Dblk + (size_t)w * WS * QS, WS * QS * sizeof(int32_t));
#pragma unroll
        for (int q = 0; q < ND; ++q)
            d_nxt[q] = __builtin_amdgcn_raw_buffer_load_b32(rd, (lane + 64 * q) * (int)sizeof(int32_t), 0, 0);
        if constexpr (HIGH) {
            const __amdgpu_buffer_rsrc_t rc = make_rsrc(Cinfo + (size_t)w * KS, KS * sizeof(int32_t));
            ci_nxt = __builtin_amdgcn_raw_buffer_load_b32(rc, lane * (int)sizeof(int32_t), 0, 0);
        }
    };
    auto take_meta = [&]() {
#pragma unroll
        for (int q = 0; q < ND; ++q)
            d_vec[q] = d_nxt[q];
        ci_vec = ci_nxt;
    };
    auto row_of = [&](int pp) -> int {
        const int e = pp * QS;
        const int rank = __builtin_amdgcn_readlane(d_vec[e / 64], e % 64 + vec);
        if constexpr (!HIGH)
            return rank;  // low-sparsity layout: the index is the window-local row itself
        return __builtin_amdgcn_readlane(ci_vec, rank & 63);
    };
    floatx16 acc[RM];
#pragma unroll
    for (int b = 0; b < RM; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[b][v] = 0.0f;

    // Rolling register pipeline: the operands of k-step s are reloaded for the next window right
    // after the MFMAs of k-step s have been issued, so every load has one whole window of MFMA work
    // to land and the operands need a single set of registers.
    afrag_t a_op[KSTEPS];
    float b_op[KSTEPS];
    uint32_t b_off[KSTEPS];
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s)
        b_off[s] = b_lane + s * b_step;
    auto load_step = [&](int s, __amdgpu_buffer_rsrc_t ra, __amdgpu_buffer_rsrc_t rb) {
        const int r0 = row_of(2 * s), r1 = row_of(2 * s + 1);
        const uint32_t off = (uint32_t)(h ? r1 : r0) * row_bytes + a_vlane;
        if constexpr (RM == 8) {
            a_op[s].lo = buffer_load_f4(ra, off);
            a_op[s].hi = buffer_load_f4(ra, off + 512);
        } else {
            a_op[s] = buffer_load_f4(ra, off);
        }
        b_op[s] = buffer_load_f1(rb, b_off[s], 0);
    };
    if (w_count > 0) {
        load_meta(w_begin);
        take_meta();
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ablk + (size_t)w_begin * KS * M, a_bytes);
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bvec + (size_t)w_begin * WS * N, b_bytes);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
            load_step(s, ra, rb);
        load_meta(min(w_begin + 1, w_last));
        take_meta();
    }
    for (int t = 0; t < w_count; ++t) {
        const int w = w_begin + t;
        const int wn = min(w + 1, w_last);
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ablk + (size_t)wn * KS * M, a_bytes);
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bvec + (size_t)wn * WS * N, b_bytes);
        load_meta(min(w + 2, w_last));
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < RM; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_get(a_op[s], b), b_op[s], acc[b], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            load_step(s, ra, rb);
        }
        __builtin_amdgcn_sched_barrier(0);
        take_meta();
    }

    float* out = p.out + (size_t)blockIdx.y * p.slice_elems;
    const int col = bj + vec * 32 + j;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int r32 = 8 * (v / 4) + 4 * h + (v % 4);
#pragma unroll
        for (int b = 0; b < RM; ++b) {
            const int row = bi + (b / 4) * 128 + r32 * 4 + (b % 4);
            if (row < M)
                out[(size_t)row * N + col] = acc[b][v];
        }
    }
}

template <int KS, int WS, int QS, int RM>
static hipError_t launch_gather(const SpmmArgs& a)
{
    MfmaParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.nwin = a.W / WS;
    p.split_k = a.split_k;
    p.tiles_m = (a.M + RM * 32 - 1) / (RM * 32);
    p.tiles_n = a.N / (QS * 32);
    dim3 grid(p.tiles_m * p.tiles_n, a.split_k, 1);
#if NMSPMM_GATHER == 2
    spmm_direct_kernel<KS, WS, QS, RM, true><<<grid, dim3(64 * QS), 0, a.stream>>>(p);
#else
    spmm_gather_kernel<KS, WS, QS, RM><<<grid, dim3(64 * QS), 0, a.stream>>>(p);
#endif
    return hipGetLastError();
}

template <int KS, int WS, int QS, int RM>
static hipError_t launch_direct_low(const SpmmArgs& a)
{
    constexpr int MS = RM * 32;
    MfmaParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = nullptr;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.nwin = a.W / WS;
    p.split_k = a.split_k;
    p.tiles_m = (a.M + MS - 1) / MS;
    p.tiles_n = a.N / (QS * 32);
    dim3 grid(p.tiles_m * p.tiles_n, a.split_k, 1);
    spmm_direct_kernel<KS, WS, QS, RM, false><<<grid, dim3(64 * QS), 0, a.stream>>>(p);
    return hipGetLastError();
}

template <int KS, int WS, int QS, int WR, int RM, bool HIGH, int NBUF>
static hipError_t launch_cfg(const SpmmArgs& a)
{
    typedef TileCfg<KS, WS, QS, WR, RM, HIGH> T;
    MfmaParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.nwin = a.W / WS;
    p.split_k = a.split_k;
    p.tiles_m = (a.M + T::MS - 1) / T::MS;
    p.tiles_n = a.N / T::NS;
    dim3 grid(p.tiles_m * p.tiles_n, a.split_k, 1);
    spmm_mfma_kernel<KS, WS, QS, WR, RM, HIGH, NBUF><<<grid, dim3(T::NT), (size_t)NMSPMM_LDS_MIN, a.stream>>>(p);
    return hipGetLastError();
}

// Row extent of the workgroup tile.  Every tile has four waves: 1 x 4, 2 x 2 or 4 x 1 (rows x
// column vectors).  For 128-wide column blocks a wave is 128 rows tall, or 256 rows when the
// matrix is large enough that 256-row tiles still give every CU at least two workgroups: the
// taller wave amortises its per-window loads and barrier over twice the MFMAs.
constexpr int kCus = 256;

template <int KS, int WS, bool HIGH>
static hipError_t launch_ns(const SpmmArgs& a)
{
#if NMSPMM_GATHER
    if constexpr (HIGH) {
        const bool tall = (long long)((a.M + 255) / 256) * (a.N / a.Ns) * a.split_k >= 2 * kCus;
        switch (a.Ns) {
        case 128: {
            // 256-row waves only while two workgroups still fit a CU (64 KiB of LDS each)
#if NMSPMM_GATHER == 2
            constexpr int tall_rm = NMSPMM_GATHER_RM_TALL;
#else
            constexpr int tall_rm = 2 * 4 * WS * 256 * (int)sizeof(float) <= 64 * 1024 ? NMSPMM_GATHER_RM_TALL : 4;
#endif
            return tall ? launch_gather<KS, WS, 4, tall_rm>(a) : launch_gather<KS, WS, 4, 4>(a);
        }
        case 64: return launch_gather<KS, WS, 2, 4>(a);
        case 32: return launch_gather<KS, WS, 1, 4>(a);
        }
    }
#endif
#if NMSPMM_DIRECT_LOW
    if constexpr (!HIGH && WS <= 16) {
        if (a.Ns == 128) {
            const bool tall = (long long)((a.M + 255) / 256) * (a.N / a.Ns) * a.split_k >= 2 * kCus;
            return tall ? launch_direct_low<KS, WS, 4, NMSPMM_GATHER_RM_TALL>(a) : launch_direct_low<KS, WS, 4, 4>(a);
        }
    }
#endif
    switch (a.Ns) {
    case 128:
        if (NMSPMM_TALL && (long long)((a.M + 255) / 256) * (a.N / 128) * a.split_k >= 2 * kCus) {
            // three buffers only where they fit the 160 KiB of LDS
            constexpr int nbuf = TileCfg<KS, WS, 4, 1, 8, HIGH>::LDS_BYTES / 2 * NMSPMM_NBUF_TALL <= 160 * 1024
                                     ? NMSPMM_NBUF_TALL : 2;
            return launch_cfg<KS, WS, 4, 1, 8, HIGH, nbuf>(a);
        }
        return launch_cfg<KS, WS, 4, NMSPMM_CFG128, HIGH, NMSPMM_NBUF>(a);
    case 64: return launch_cfg<KS, WS, 2, NMSPMM_CFG64, HIGH, NMSPMM_NBUF>(a);
    case 32: return launch_cfg<KS, WS, 1, NMSPMM_CFG32, HIGH, NMSPMM_NBUF>(a);
    }
    return hipErrorInvalidValue;
}

bool mfma_supported(const SpmmArgs& a)
{
    if (a.vec_len != 32 || (a.Ns != 32 && a.Ns != 64 && a.Ns != 128))
        return false;
    if (a.M % 4 != 0 || a.M < 32)
        return false;
    const bool high = a.cinfo != nullptr;
    if (!high)
        return a.window == 32 && (a.kept == 32 || a.kept == 16 || a.kept == 12);
    return a.window == 64 && (a.kept == 16 || a.kept == 8);
}

hipError_t launch_mfma(const SpmmArgs& a)
{
    const bool high = a.cinfo != nullptr;
    if (!high) {
        if (a.kept == 32) return launch_ns<32, 32, false>(a);
        if (a.kept == 16) return launch_ns<32, 16, false>(a);
        if (a.kept == 12) return launch_ns<32, 12, false>(a);
    } else {
        if (a.kept == 16) return launch_ns<64, 16, true>(a);
        if (a.kept == 8) return launch_ns<64, 8, true>(a);
    }
    return hipErrorInvalidValue;
}

} // namespace nmspmm
