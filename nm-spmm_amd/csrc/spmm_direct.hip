// Matrix-core kernel for C = A . B with an N:M-sparse B whose index pattern is shared by 32
// adjacent columns (reference kernels: src/kernel_{64x128_8x8,64x64_8x8,32x64_8x4,32x32_4x4}.cu;
// this file replaces their role, not their design).
//
// Design for gfx950 (64-lane waves, v_mfma_f32_32x32x2_f32):
//  * A 32-column index vector is exactly the N extent of one 32x32x2 MFMA, so one wave owns one
//    column vector and RM row blocks of 32 rows, and is independent of every other wave: no LDS,
//    no barrier (the one exception: problems of few tiles, where the four waves of a workgroup
//    share the reduction of one vector and add their sums up in LDS at the end).
//  * The A operand of one MFMA is A[row][k] with lane = (row % 32, k half): lanes 0-31 take kept
//    row 2s of the window, lanes 32-63 kept row 2s+1, and each half reads the dense row of A that
//    *its* index selects.  A is column-major, so that is M contiguous floats: the gather is a
//    per-lane row offset of an ordinary load and moves no data.
//  * The wave's RM row blocks interleave rows (block b holds rows 4*r + b; a 256-row wave has two
//    such groups 128 rows apart), so one 128-bit load per lane is the A operand of four MFMAs -
//    two 512-byte row segments per wave and instruction - and the B operand is reused RM times.
//  * Rolling register pipeline: right after the MFMAs of k-step s have been issued, the operands
//    of k-step s of the next chunk of kept rows are loaded into the same registers, so every load
//    has a whole chunk of MFMA work (thousands of cycles) to land, memory instructions are spread
//    evenly between the MFMAs, and one set of operand registers suffices.  The reuse of A between
//    the column vectors of a workgroup and between neighbouring workgroups is left to the vector
//    L1 and the L2: the tile walk keeps the workgroups resident on one XCD in a compact patch of C.
//  * Index metadata arrives as one wave-wide load per window ([kept][Ns/32] ints, plus the
//    column_info list of the window on the high-sparsity layout), two windows ahead, and is
//    handed to the lanes that need it with ds_bpermute (the LDS crossbar, no LDS memory): one
//    permute and one multiply-add per k-step form the per-lane row offset.  Vector ALU work in
//    the loop is not free next to back-to-back MFMAs, so it is kept to that.
//  * All loads go through buffer descriptors whose extent ends with the window's last row, so no
//    lane reads outside A or B without a branch; lanes whose rows lie beyond M read zeros or
//    other rows' values into accumulators that are never stored.
#include "internal.h"
#include <type_traits>

namespace nmspmm {

typedef float floatx16 __attribute__((ext_vector_type(16)));

struct DirectParams {
    const float* A;
    const float* B;
    const int32_t* D;
    const int32_t* cinfo;
    float* out;          // C, or the first partial slice when split_k > 1
    size_t slice_elems;  // floats between partial slices
    int M, N, W;
    int lda;             // floats between consecutive dense rows of A (>= M, a multiple of 4)
    int nwin;            // windows in the whole reduction
    int split_k;
    int tiles_m, tiles_n;
    int tile_offset;     // first logical tile of this launch (the tail tiles may get a launch of their own)
    int head_units;      // workgroups of this launch that compute whole tiles (the first ones)
    int tail_offset;     // first logical tile computed in pieces along M by the workgroups after them
    int sub_tiles;       // > 1: every workgroup of this launch is one of sub_tiles pieces, along M, of a
                         // tile of sub_tiles * MS rows (the tile walk and tiles_m are those taller tiles')
    int xcds;            // accelerator dies of the GPU: consecutive workgroup ids go to consecutive dies
};

struct float8 { float4 lo, hi; };
template <int RM> struct AFrag;
template <> struct AFrag<8> { typedef float8 type; };
template <> struct AFrag<4> { typedef float4 type; };
template <> struct AFrag<2> { typedef float2 type; };

__device__ inline float frag_get(const float2& v, int i) { return i == 0 ? v.x : v.y; }
__device__ inline float frag_get(const float4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
__device__ inline float frag_get(const float8& v, int i) { return i < 4 ? frag_get(v.lo, i) : frag_get(v.hi, i - 4); }

// Buffer descriptors give branch-free guarded loads: an offset at or beyond num_records reads 0
// without touching memory.
__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ inline float4 buffer_load_f4(__amdgpu_buffer_rsrc_t r, uint32_t byte_off)
{
    auto v = __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, 0);
    return *reinterpret_cast<float4*>(&v);
}
__device__ inline float2 buffer_load_f2(__amdgpu_buffer_rsrc_t r, uint32_t byte_off)
{
    auto v = __builtin_amdgcn_raw_buffer_load_b64(r, byte_off, 0, 0);
    return *reinterpret_cast<float2*>(&v);
}
__device__ inline float buffer_load_f1(__amdgpu_buffer_rsrc_t r, uint32_t byte_off, uint32_t s_off)
{
    return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, byte_off, s_off, 0));
}

// Waves per SIMD the register allocation must allow for 128-row waves (256-row waves get two), and
// the tile-walk band height in row tiles.  The 2:8 geometry (64-row windows, 16 kept) would take
// 134 registers at three waves per SIMD, six too many for the four workgroups per CU the run-time
// model counts on: it is compiled for four (128 registers, nothing spills; the dense geometry
// would spill, the others are below 128 anyway).
constexpr int kWavesPerSimd = 3;
constexpr int kBandTiles = 2;

// Tile shapes that exist in a second form for launches of at most one workgroup per CU, where
// each wave has its SIMD to itself (direct_unit's DEEP).
template <int WS, int RM, bool HIGH>
constexpr bool has_lone_form()
{
    return (HIGH && WS == 8 && RM <= 4) || (!HIGH && WS == 16 && RM == 4);
}

// KS: dense rows per window, WS: kept rows per window, QS: column vectors per preprocessed column
// block (Ns = 32*QS), WR: waves along M, RM: 32-row blocks per wave (2, 4 or 8), HIGH:
// high-sparsity layout (D holds ranks into the window's column_info list), DEEP: B operands are
// loaded two windows ahead (for launches that leave each wave alone on its SIMD), KW: waves along
// K.  With KW > 1 (WR == 1) the workgroup's KW waves compute the same RM*32 rows of ONE 32-column
// vector, each over its share of the windows, and add their results up through LDS in wave order;
// QS then only describes the index layout, and the tile walk counts vectors, not column blocks.
// KH: sets of QS * WR waves per workgroup (1 or 2).  With two, the workgroup computes the same
// whole tile twice over, each set over half of the windows, and the sets exchange half of their
// sums through LDS before they store.
template <int KS, int WS, int QS, int WR, int RM, bool HIGH, bool DEEP = false, int KW = 1, int KH = 1>
__device__ __forceinline__ void direct_unit(const DirectParams& p, const int logical, const int sub, const int sub_tiles)
{
    static_assert(RM == 2 || RM == 4 || RM == 8, "64-, 128- or 256-row waves");
    constexpr int IL = RM < 4 ? RM : 4;  // rows interleaved per lane: block b holds rows IL*r + b%IL (+128 for b >= 4)
    static_assert(WS % 2 == 0, "two kept rows per MFMA");
    typedef typename AFrag<RM>::type afrag_t;
    constexpr int MW = RM * 32;               // rows per wave
    constexpr int MS = WR * MW;               // rows per workgroup tile
    constexpr int NS = QS * 32;
    constexpr int CH = WS <= 16 ? WS : 16;    // kept rows per pipeline chunk
    constexpr int NCH = WS / CH;
    constexpr int CS = CH / 2;                // MFMA k-steps per chunk
    constexpr int ND = (WS * QS + 63) / 64;   // wave-wide loads per window of indices
    static_assert(WS % CH == 0, "whole chunks");

    // logical tile -> (tile_m, tile_n): bands of GROUP row tiles across all column blocks; with
    // sub_tiles > 1 the walk and tiles_m are those of tiles sub_tiles times as tall as MS
    constexpr int GROUP = kBandTiles;
    int tile_m, tile_n;
    {
        const int band = logical / (GROUP * p.tiles_n);
        const int first_m = band * GROUP;
        const int rows = min(GROUP, p.tiles_m - first_m);
        const int in_band = logical - band * GROUP * p.tiles_n;
        tile_m = first_m + in_band % rows;
        tile_n = in_band / rows;
    }
    const int lane = threadIdx.x & 63;
    static_assert(KH == 1 || (KH == 2 && KW == 1 && RM == 8), "two sets of waves only on whole 256-row waves");
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave = KH > 1 ? wave_all % (QS * WR) : wave_all;
    const int kh = KH > 1 ? wave_all / (QS * WR) : 0;
    int w_begin, w_count;
    if constexpr (KW > 1)
        split_windows(p.nwin, KW, wave, &w_begin, &w_count);
    else if constexpr (KH > 1)
        split_windows(p.nwin, KH, kh, &w_begin, &w_count);
    else
        split_windows(p.nwin, p.split_k, blockIdx.y, &w_begin, &w_count);
    const int w_last = w_begin + w_count - 1;

    // column vector inside its preprocessed column block, and that block.  With waves along K the
    // workgroup is either one vector of a walk over vectors, or (sub_tiles == 0) unit `sub` of the
    // WR * QS units, 128 rows of one vector each, of a whole tile of the walk over tiles
    const bool tile_unit = KW > 1 && sub_tiles == 0;
    const int vec = KW > 1 ? (tile_unit ? sub % QS : tile_n % QS) : wave % QS;
    const int wr = KW > 1 ? (tile_unit ? sub / QS : 0) : wave / QS;
    const int block_n = KW > 1 && !tile_unit ? tile_n / QS : tile_n;
    const int h = lane >> 5;
    const int j = lane & 31;
    const int M = p.M, N = p.N, lda = p.lda;
    const int bi = tile_unit ? tile_m * MS + wr * MW            // first row of this wave (may be >= M: loads nothing)
                             : (tile_m * sub_tiles + sub) * MS + wr * MW;
    const int bj = block_n * NS + vec * 32;

    const float* const Ablk = p.A + min(bi, lda);
    const float* const Bvec = p.B + bj;
    const int32_t* const Dblk = p.D + (size_t)block_n * p.W * QS;
    const int32_t* const Cinfo = HIGH ? p.cinfo + (size_t)block_n * p.nwin * KS : nullptr;
    // extents: the last dense row of a window ends with its lda floats (rows between M and lda are
    // padding that may be read and is never stored), the last kept row of B with this vector's 32
    // columns
    const uint32_t a_bytes = bi < M ? (uint32_t)(((size_t)(KS - 1) * lda + (size_t)(lda - bi)) * sizeof(float)) : 0u;
    const uint32_t b_bytes = (uint32_t)(((size_t)(WS - 1) * N + 32) * sizeof(float));
    const uint32_t row_bytes = (uint32_t)((size_t)lda * sizeof(float));
    const uint32_t a_vlane = (uint32_t)(j * IL * sizeof(float));  // this lane's run of IL rows inside the wave's rows
    const uint32_t b_chunk = (uint32_t)((size_t)CH * N * sizeof(float));
    // B operand of k-step s: this lane's element of kept row 2s + h.  The lane part sits in one
    // register, the k-step part is a scalar offset of the load
    const uint32_t b_lane = (uint32_t)(((size_t)h * N + j) * sizeof(float));
    const uint32_t b_step = (uint32_t)((size_t)2 * N * sizeof(float));

    // ---- index metadata: d_vec / ci_vec belong to the window whose operands are being loaded,
    // d_nxt / ci_nxt to the one after it
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
    // Byte offsets of this lane's A operands for the CS k-steps of chunk c of the window whose
    // metadata is in d_vec / ci_vec: lane half h of k-step s needs the dense row that index entry
    // (c*CH + 2s + h) * QS + vec selects.  ds_bpermute fetches that entry from the lane holding it
    // (a crossbar read, no LDS memory involved).  On the high-sparsity layout the entries are
    // ranks into the window's column_info list; resolve_ranks() turns all of them into rows with
    // one more permute per window.
    const int perm_addr = (h * QS + vec) * (int)sizeof(int32_t);
    uint32_t a_off[CS];
    auto resolve_ranks = [&]() {
        if constexpr (HIGH) {
            static_assert(!HIGH || ND == 1, "one register of ranks per window");
            d_vec[0] = __builtin_amdgcn_ds_bpermute(d_vec[0] << 2, ci_vec);
        }
    };
    auto form_offsets = [&](int c) {
#pragma unroll
        for (int s = 0; s < CS; ++s) {
            const int e = (c * CH + 2 * s) * QS;
            const int row = __builtin_amdgcn_ds_bpermute(perm_addr + (e % 64) * (int)sizeof(int32_t), d_vec[e / 64]);
            a_off[s] = __umul24((uint32_t)row, row_bytes) + a_vlane;
        }
    };

    // B operands are loaded BD chunks ahead of their use, A operands one chunk: B streams from HBM
    // (each element is read by the few workgroups of one column block), A is mostly served by the
    // L2.  A chunk of a 128-row wave is 4 to 8 k-steps, one to two thousand matrix-pipe cycles,
    // which covers an L2 hit but not always an HBM miss; two chunks do.  Measured on waves of 64
    // and 128 rows: 16 and 12 kept rows of 32, 3 to 12 % faster while a CU holds one or two
    // workgroups, level beyond (the 128-row wave with 16 kept rows would pass 128 registers and
    // lose its fourth workgroup per CU, so it takes the deeper form only when asked, DEEP); 8 kept
    // rows of 64, 4 to 20 % faster while each wave has its SIMD to itself and 2 to 5 % slower
    // otherwise (DEEP again); 16 kept rows of 64 run out of registers with it.  256-row waves
    // are level either way and keep one.
    constexpr bool kAlwaysDeep = !HIGH && NCH == 1 && RM <= 4 && !(WS == 16 && RM == 4);
    constexpr int BD = (kAlwaysDeep || (DEEP && has_lone_form<WS, RM, HIGH>())) ? 2 : 1;
    afrag_t a_op[CS];
    float b_op[BD][CS];
    // A operand of k-step s of chunk c of the window the descriptor points at
    auto load_a = [&](int s, __amdgpu_buffer_rsrc_t ra) {
        const uint32_t off = a_off[s];
        if constexpr (RM == 8) {
            a_op[s].lo = buffer_load_f4(ra, off);
            a_op[s].hi = buffer_load_f4(ra, off + 512);
        } else if constexpr (RM == 4) {
            a_op[s] = buffer_load_f4(ra, off);
        } else {
            a_op[s] = buffer_load_f2(ra, off);
        }
    };

    floatx16 acc[RM];
#pragma unroll
    for (int b = 0; b < RM; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v)
            acc[b][v] = 0.0f;

    if (w_count > 0) {
        // the loads are issued in the order of the loop (index metadata of the window after, then
        // the operands), so that the wait counts the compiler places at the loop head for the
        // metadata leave the operand loads in flight on the first pass as on every other
        load_meta(w_begin);
        take_meta();
        load_meta(min(w_begin + 1, w_last));
        resolve_ranks();
        form_offsets(0);
        const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ablk + (size_t)w_begin * KS * lda, a_bytes);
        const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bvec + (size_t)w_begin * WS * N, b_bytes);
#pragma unroll
        for (int s = 0; s < CS; ++s) {
            load_a(s, ra);
            b_op[0][s] = buffer_load_f1(rb, b_lane, s * b_step);
        }
        if constexpr (BD == 2) {
            const __amdgpu_buffer_rsrc_t rb1 = make_rsrc(Bvec + (size_t)min(w_begin + 1, w_last) * WS * N, b_bytes);
#pragma unroll
            for (int s = 0; s < CS; ++s)
                b_op[1][s] = buffer_load_f1(rb1, b_lane, s * b_step);
        }
    }
    // window t of this workgroup; PAR (a compile-time 0 or 1) selects the B operand set it uses
    auto window = [&](const int t, auto par) {
        constexpr int PAR = decltype(par)::value;
        const int w = w_begin + t;
        const int wn = min(w + 1, w_last);  // the last window reloads itself; nothing consumes it
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            // while chunk c is multiplied, chunk c+1 (or chunk 0 of the next window) is loaded
            const bool wrap = c == NCH - 1;
            if (wrap) {
                __builtin_amdgcn_sched_barrier(0);
                take_meta();
                resolve_ranks();
                load_meta(min(w + 2, w_last));
            }
            const int wl = wrap ? wn : w;
            const int cl = wrap ? 0 : c + 1;
            form_offsets(cl);
            const __amdgpu_buffer_rsrc_t ra = make_rsrc(Ablk + (size_t)wl * KS * lda, a_bytes);
            const int wb = BD == 2 ? min(w + 2, w_last) : wl;
            const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bvec + (size_t)wb * WS * N, b_bytes);
#pragma unroll
            for (int s = 0; s < CS; ++s) {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int b = 0; b < RM; ++b)
                    acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag_get(a_op[s], b), b_op[PAR][s], acc[b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                load_a(s, ra);
                b_op[PAR][s] = buffer_load_f1(rb, b_lane, s * b_step + cl * b_chunk);
            }
        }
    };
    if constexpr (BD == 2) {
        int t = 0;
        for (; t + 1 < w_count; t += 2) {
            window(t, std::integral_constant<int, 0>());
            window(t + 1, std::integral_constant<int, 1>());
        }
        if (t < w_count)
            window(t, std::integral_constant<int, 0>());
    } else {
        for (int t = 0; t < w_count; ++t)
            window(t, std::integral_constant<int, 0>());
    }

    // ---- epilogue: MFMA result register v of lane (h, j) is row 8*(v/4) + 4*h + v%4 of the block,
    // column j; block b of the wave holds rows (b/4)*128 + IL*r + b%IL.  Stores go through a
    // descriptor that ends with the last live row of this wave, so rows beyond M are dropped
    // without a branch; the per-register part of the offset is a scalar.
    float* const out = p.out + (size_t)blockIdx.y * p.slice_elems;
    const int rows_here = min(M - bi, MW);
    float* const c_base = out + (size_t)min(bi, M) * N + bj;
    const uint32_t c_bytes = rows_here > 0 ? (uint32_t)(((size_t)(rows_here - 1) * N + 32) * sizeof(float)) : 0u;
    const __amdgpu_buffer_rsrc_t rc = make_rsrc(c_base, c_bytes);
    const uint32_t c_lane = (uint32_t)(((size_t)4 * IL * h * N + j) * sizeof(float));
    const uint32_t n_bytes = (uint32_t)((size_t)N * sizeof(float));
    if constexpr (KW > 1) {
        // Waves along K: every wave leaves its sums in LDS, and the groups of four result registers
        // are dealt out to the waves, group g to wave g % KW, which adds the KW partial sums in wave
        // order (the order of the windows) and stores the group's four rows.
        static_assert(KW * RM <= 32, "128 KB of LDS for one workgroup per CU, 64 KB where two share a CU");
        __shared__ float4 partial[KW][RM * 4][64];
#pragma unroll
        for (int b = 0; b < RM; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                partial[wave][b * 4 + q][lane] = make_float4(acc[b][4 * q], acc[b][4 * q + 1], acc[b][4 * q + 2], acc[b][4 * q + 3]);
        __syncthreads();
#pragma unroll
        for (int b = 0; b < RM; ++b) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int g = b * 4 + q;
                if (g % KW != wave)
                    continue;
                float4 sum = partial[0][g][lane];
#pragma unroll
                for (int z = 1; z < KW; ++z) {
                    const float4 t = partial[z][g][lane];
                    sum.x += t.x;
                    sum.y += t.y;
                    sum.z += t.z;
                    sum.w += t.w;
                }
                const float out4[4] = {sum.x, sum.y, sum.z, sum.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t row = (b / 4) * 128 + IL * (8 * q + i) + (b % IL);
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(out4[i]), rc, c_lane + row * n_bytes, 0, 16);  // to C: see below
                }
            }
        }
        return;
    }
    // Results that go straight to C are stored with the system-coherent policy (sc1, bit 4 of the
    // cache-policy operand): nothing in this launch reads them again, and written through they cost
    // the launch 1 to 1.7 us less at its end than lines left dirty in L2 (4096 x 4096 x 1024 at 1:8:
    // 41.0 -> 39.3 us).  Slices of a cut reduction keep the default policy (stored this way too they
    // were measured within -6 to +1 %, most shapes level).
    const auto store_blocks = [&](auto policy, auto first, auto count) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
#pragma unroll
            for (int b = decltype(first)::value; b < decltype(first)::value + decltype(count)::value; ++b) {
                // row inside the wave, without the lane's 4*IL*h: IL * (8*(v/4) + v%4) + b%IL, second group + 128
                const uint32_t row = (b / 4) * 128 + IL * (8 * (v / 4) + (v % 4)) + (b % IL);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(acc[b][v]), rc, c_lane + row * n_bytes, 0,
                                                      decltype(policy)::value);
            }
        }
    };
    if constexpr (KH == 2) {
        // Two sets of waves, each over half of the windows: every wave hands the half of its result
        // blocks that the other set stores to its partner through LDS, adds what it is handed (one
        // addition per element, so the order does not matter) and stores its own half.
        constexpr int HB = RM / 2;
        __shared__ float4 handed[2][QS * WR][HB * 4][64];
        const auto hand = [&](auto first) {
#pragma unroll
            for (int b = 0; b < HB; ++b)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const floatx16& r = acc[decltype(first)::value + b];
                    handed[kh][wave][b * 4 + q][lane] = make_float4(r[4 * q], r[4 * q + 1], r[4 * q + 2], r[4 * q + 3]);
                }
        };
        const auto take = [&](auto first) {
#pragma unroll
            for (int b = 0; b < HB; ++b)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 t = handed[1 - kh][wave][b * 4 + q][lane];
                    floatx16& r = acc[decltype(first)::value + b];
                    r[4 * q] += t.x;
                    r[4 * q + 1] += t.y;
                    r[4 * q + 2] += t.z;
                    r[4 * q + 3] += t.w;
                }
        };
        typedef std::integral_constant<int, 0> lower;
        typedef std::integral_constant<int, HB> upper;
        if (kh == 0)
            hand(upper{});
        else
            hand(lower{});
        __syncthreads();
        if (kh == 0) {
            take(lower{});
            store_blocks(std::integral_constant<int, 16>{}, lower{}, upper{});
        } else {
            take(upper{});
            store_blocks(std::integral_constant<int, 16>{}, upper{}, upper{});
        }
        return;
    }
    typedef std::integral_constant<int, 0> first_block;
    typedef std::integral_constant<int, RM> all_blocks;
    if (p.split_k == 1)
        store_blocks(std::integral_constant<int, 16>{}, first_block{}, all_blocks{});
    else
        store_blocks(std::integral_constant<int, 0>{}, first_block{}, all_blocks{});
}

// Workgroup `id` of a launch whose workgroups all compute the same kind of unit.  Whole tiles: a
// walk that gives each XCD (consecutive ids go to different XCDs) a contiguous run of the
// p.head_units logical tiles.  In a launch of pieces along M (p.sub_tiles > 1) consecutive ids are
// the pieces of one tile.
template <int KS, int WS, int QS, int WR, int RM, bool HIGH, bool DEEP = false, int KW = 1, int KH = 1>
__device__ __forceinline__ void direct_uniform_launch(const DirectParams& p, const int id)
{
    int logical, sub = 0;
    if (p.sub_tiles > 1) {
        logical = p.tile_offset + id / p.sub_tiles;
        sub = id % p.sub_tiles;
    } else {
        const int total = p.head_units;
        const int q = total / p.xcds, r = total % p.xcds;
        const int xcd = id % p.xcds, loc = id / p.xcds;
        logical = p.tile_offset + (xcd < r ? xcd * (q + 1) + loc : r * (q + 1) + (xcd - r) * q + loc);
    }
    direct_unit<KS, WS, QS, WR, RM, HIGH, DEEP, KW, KH>(p, logical, sub, p.sub_tiles);
}

#define NMSPMM_DIRECT_BOUNDS __launch_bounds__(64 * QS * WR, RM == 8 ? 2 : (HIGH && WS == 16) ? 4 : kWavesPerSimd)

template <int KS, int WS, int QS, int WR, int RM, bool HIGH>
__global__ void NMSPMM_DIRECT_BOUNDS spmm_direct_kernel(const DirectParams p)
{
    direct_uniform_launch<KS, WS, QS, WR, RM, HIGH>(p, blockIdx.x);
}

// The same with B loaded two windows ahead, for launches of at most one workgroup per CU.
template <int KS, int WS, int QS, int WR, int RM, bool HIGH>
__global__ void NMSPMM_DIRECT_BOUNDS spmm_direct_lone_kernel(const DirectParams p)
{
    direct_uniform_launch<KS, WS, QS, WR, RM, HIGH, true>(p, blockIdx.x);
}

// Whole tiles of 256-row waves with two sets of waves, each over half of the windows (128 KB of
// LDS): for launches of at most one such workgroup per CU, which would otherwise leave every SIMD
// with a single wave.
template <int KS, int WS, int QS, int WR, bool HIGH>
__global__ void __launch_bounds__(128 * QS * WR, 1) spmm_direct_halves_kernel(const DirectParams p)
{
    direct_uniform_launch<KS, WS, QS, WR, 8, HIGH, false, 1, 2>(p, blockIdx.x);
}

// Four waves along K: one workgroup per RM*32 rows of one 32-column vector (p.tiles_n counts
// vectors), the reduction over K split between its waves and finished in LDS.  For problems of so
// few tiles that the reduction has to be cut to fill the GPU: no scratch, no second pass.
template <int KS, int WS, int QS, int RM, bool HIGH, bool DEEP>
__global__ void __launch_bounds__(256, 2) spmm_direct_inner_kernel(const DirectParams p)
{
    direct_uniform_launch<KS, WS, QS, 1, RM, HIGH, DEEP, 4>(p, blockIdx.x);
}

// Eight waves along K, 64 or 128 rows (64 or 128 KB of LDS): for launches of at most one such
// workgroup per CU.
template <int KS, int WS, int QS, int RM, bool HIGH, bool DEEP>
__global__ void __launch_bounds__(512, 1) spmm_direct_inner8_kernel(const DirectParams p)
{
    direct_uniform_launch<KS, WS, QS, 1, RM, HIGH, DEEP, 8>(p, blockIdx.x);
}

// The first p.head_units workgroups compute whole tiles; the ones after them the tiles from
// p.tail_offset on, four workgroups per tile, each 128 rows of one 32-column vector with the
// reduction shared between its four waves.  They are dispatched last and give the CUs that run out
// of whole tiles a quarter of a tile each.
template <int KS, int WS, int QS, int WR, bool HIGH>
__global__ void __launch_bounds__(256, 2) spmm_direct_mixed_inner_kernel(const DirectParams p)
{
    const int id = blockIdx.x;
    if (id >= p.head_units) {
        const int u = id - p.head_units;
        direct_unit<KS, WS, QS, WR, 4, HIGH, false, 4>(p, p.tail_offset + u / 4, u % 4, 0);
        return;
    }
    direct_uniform_launch<KS, WS, QS, WR, 4, HIGH>(p, id);
}

// The same with eight workgroups per leftover tile, each 64 rows of one 32-column vector (32 KB of
// LDS: a CU holds several at once).
template <int KS, int WS, int QS, int WR, bool HIGH>
__global__ void __launch_bounds__(256, 2) spmm_direct_mixed_eighths_kernel(const DirectParams p)
{
    const int id = blockIdx.x;
    if (id >= p.head_units) {
        const int u = id - p.head_units;
        direct_unit<KS, WS, QS, 2 * WR, 2, HIGH, false, 4>(p, p.tail_offset + u / 8, u % 8, 0);
        return;
    }
    direct_uniform_launch<KS, WS, QS, WR, 4, HIGH>(p, id);
}

// Every workgroup is one of the WRU * QS units of a whole tile of the walk over tiles (from
// p.tail_offset on), 64 rows of one 32-column vector, the reduction shared between its four waves:
// for the leftover tiles of a launch of several rounds, in a launch of their own.
template <int KS, int WS, int QS, int WRU, bool HIGH>
__global__ void __launch_bounds__(256, 2) spmm_direct_units_kernel(const DirectParams p)
{
    const int id = blockIdx.x;
    direct_unit<KS, WS, QS, WRU, 2, HIGH, false, 4>(p, p.tail_offset + id / (WRU * QS), id % (WRU * QS), 0);
}

// The first p.head_units workgroups compute whole tiles; the ones after them are the pieces, two
// per tile along M, of the tiles from p.tail_offset on, computed on waves of RM / 2 blocks.  They
// are dispatched last and fill the CUs that run out of whole tiles, in pieces fine enough to even
// out the end of the launch (same sums in the same order as whole tiles, no scratch).
template <int KS, int WS, int QS, int WR, int RM, bool HIGH, bool DEEP = false>
__global__ void NMSPMM_DIRECT_BOUNDS spmm_direct_mixed_kernel(const DirectParams p)
{
    const int id = blockIdx.x;
    if (id >= p.head_units) {
        const int u = id - p.head_units;
        direct_unit<KS, WS, QS, WR, RM / 2, HIGH, DEEP>(p, p.tail_offset + u / 2, u % 2, 2);
        return;
    }
    direct_uniform_launch<KS, WS, QS, WR, RM, HIGH, DEEP>(p, id);
}

// One launch of uniform workgroups.  A launch of at most one workgroup per CU (each wave alone on
// its SIMD) takes the form that loads B two windows ahead where the tile shape has one; a whole
// problem of at most that many tiles of 256-row waves the form with two sets of waves
// (wave_sets_pay).
template <int KS, int WS, int QS, int WR, int RM, bool HIGH>
static hipError_t launch_uniform(const dim3 grid, const dim3 block, hipStream_t stream, const DirectParams& p,
                                 const bool whole_problem = false)
{
    bool lone = false;
    if constexpr (has_lone_form<WS, RM, HIGH>())
        lone = (long long)grid.x * grid.y <= machine().cus;
    bool halves = false;
    if constexpr (RM == 8)
        halves = whole_problem && p.split_k == 1 && wave_sets_pay(grid.x, p.nwin, WS);
    if (halves) {
        if constexpr (RM == 8)
            spmm_direct_halves_kernel<KS, WS, QS, WR, HIGH><<<grid, dim3(2 * block.x), 0, stream>>>(p);
    } else if (lone) {
        if constexpr (has_lone_form<WS, RM, HIGH>())
            spmm_direct_lone_kernel<KS, WS, QS, WR, RM, HIGH><<<grid, block, 0, stream>>>(p);
    } else {
        spmm_direct_kernel<KS, WS, QS, WR, RM, HIGH><<<grid, block, 0, stream>>>(p);
    }
    return hipGetLastError();
}

template <int KS, int WS, int QS, int WR, int RM, bool HIGH>
static hipError_t launch_cfg(const SpmmArgs& a, const TailPlan& plan)
{
    constexpr int MS = WR * RM * 32;
    constexpr int NS = QS * 32;
    DirectParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.out = a.split_k > 1 ? a.partial : a.C;
    p.slice_elems = a.slice_stride;
    p.M = a.M;
    p.lda = a.lda;
    p.N = a.N;
    p.W = a.W;
    p.nwin = a.W / WS;
    p.split_k = a.split_k;
    p.tiles_m = (a.M + MS - 1) / MS;
    p.tiles_n = a.N / NS;
    p.tile_offset = 0;
    p.tail_offset = 0;
    p.sub_tiles = 1;
    p.xcds = machine().xcds;
    // the plan counts tiles of RM blocks per wave; it applies when that is this tile shape
    const bool own_tail = plan.separate && RM == plan.blocks;
    const dim3 block(64 * QS * WR);
    dim3 grid(p.tiles_m * p.tiles_n, a.split_k, 1);
    p.head_units = (int)grid.x;
    if (!own_tail)
        return launch_uniform<KS, WS, QS, WR, RM, HIGH>(grid, block, a.stream, p, true);
    p.head_units = (int)plan.head;
    if (plan.units && RM == 4) {
        // eight workgroups per leftover tile, dispatched after the whole tiles in the same launch (the
        // 128-row kernel's register allocation lets a CU hold four of them): against a launch of
        // their own 0 to 4 % faster at 1:8, -4 to +2 % at 2:8 and 3:8, more on short reductions
        p.tail_offset = (int)plan.head;
        grid.x = (unsigned)(plan.head + plan.tail * plan.sub);
        if constexpr (RM == 4)
            spmm_direct_mixed_eighths_kernel<KS, WS, QS, WR, HIGH><<<grid, block, 0, a.stream>>>(p);
        return hipGetLastError();
    }
    if (plan.sub > 1 && plan.fused) {
        // shorter waves for the leftovers, in the same launch: each leftover tile in two pieces
        // along M, so that the pieces fill the CUs more evenly than whole tiles would
        p.tail_offset = (int)plan.head;
        if (plan.along_k) {
            grid.x = (unsigned)(plan.head + plan.tail * (plan.eighths ? 8 : 4));
            if constexpr (RM == 4) {
                if (plan.eighths)
                    spmm_direct_mixed_eighths_kernel<KS, WS, QS, WR, HIGH><<<grid, block, 0, a.stream>>>(p);
                else
                    spmm_direct_mixed_inner_kernel<KS, WS, QS, WR, HIGH><<<grid, block, 0, a.stream>>>(p);
            }
            return hipGetLastError();
        }
        grid.x = (unsigned)(plan.head + plan.tail * plan.sub);
        if constexpr (RM == 4) {
            if (has_lone_form<WS, RM, HIGH>() && grid.x <= (unsigned)machine().cus)
                spmm_direct_mixed_kernel<KS, WS, QS, WR, RM, HIGH, has_lone_form<WS, RM, HIGH>()><<<grid, block, 0, a.stream>>>(p);
            else
                spmm_direct_mixed_kernel<KS, WS, QS, WR, RM, HIGH><<<grid, block, 0, a.stream>>>(p);
        }
        return hipGetLastError();
    }
    // head tiles, then the leftover tiles in a launch of their own
    grid.x = (unsigned)plan.head;
    hipError_t e = launch_uniform<KS, WS, QS, WR, RM, HIGH>(grid, block, a.stream, p);
    if (e != hipSuccess)
        return e;
    p.tile_offset = (int)plan.head;
    if (plan.units) {
        // (256-row waves) sixteen workgroups per leftover tile in a launch of their own, 64 rows of one
        // 32-column vector each, the reduction shared between its four waves
        p.tail_offset = (int)plan.head;
        grid.x = (unsigned)(plan.tail * plan.sub);
        p.head_units = (int)grid.x;
        if constexpr (RM == 8)
            spmm_direct_units_kernel<KS, WS, QS, 4 * WR, HIGH><<<grid, dim3(256), 0, a.stream>>>(p);
        return hipGetLastError();
    }
    if (plan.sub > 1) {
        // shorter waves for the leftovers, in a launch of the kernel built for such waves (which
        // more workgroups per CU can run): each tile in plan.sub pieces along M; same sums in the
        // same order as whole tiles
        p.sub_tiles = plan.sub;
        grid.x = (unsigned)(plan.tail * plan.sub);
        p.head_units = (int)grid.x;
        if (RM / plan.sub == 4) {
            if constexpr (RM >= 8)
                return launch_uniform<KS, WS, QS, WR, 4, HIGH>(grid, block, a.stream, p);
        } else {
            if constexpr (RM >= 4)
                return launch_uniform<KS, WS, QS, WR, 2, HIGH>(grid, block, a.stream, p);
        }
        return hipErrorInvalidValue;
    }
    grid.x = (unsigned)plan.tail;  // whole tiles
    p.head_units = (int)grid.x;
    return launch_uniform<KS, WS, QS, WR, RM, HIGH>(grid, block, a.stream, p);
}

// The launch with four waves along K (spmm_direct_inner_kernel), on 128- or 64-row tiles as
// plan_inner chooses.
template <int KS, int WS, int QS, bool HIGH>
static hipError_t launch_inner(const SpmmArgs& a)
{
    const long long vecs = a.N / 32;
    const InnerPlan plan = plan_inner(a.M, a.N, a.W / WS, WS);
    const int rows = plan.rows;
    const bool tall = rows == 128;
    const bool eight = plan.waves == 8;
    DirectParams p;
    p.A = a.A;
    p.B = a.B;
    p.D = a.D;
    p.cinfo = a.cinfo;
    p.out = a.C;
    p.slice_elems = 0;
    p.M = a.M;
    p.lda = a.lda;
    p.N = a.N;
    p.W = a.W;
    p.nwin = a.W / WS;
    p.split_k = 1;
    p.tiles_m = (a.M + rows - 1) / rows;
    p.tiles_n = (int)vecs;
    p.tile_offset = 0;
    p.tail_offset = 0;
    p.sub_tiles = 1;
    p.xcds = machine().xcds;
    const long long groups = (long long)p.tiles_m * p.tiles_n;
    if (groups > 0x7fffffffLL)
        return hipErrorInvalidValue;
    p.head_units = (int)groups;
    const dim3 grid((unsigned)groups), block(256);
    const bool lone = groups <= machine().cus;
    if (tall && eight) {
        spmm_direct_inner8_kernel<KS, WS, QS, 4, HIGH, has_lone_form<WS, 4, HIGH>()><<<grid, dim3(512), 0, a.stream>>>(p);
    } else if (tall) {
        if (lone && has_lone_form<WS, 4, HIGH>())
            spmm_direct_inner_kernel<KS, WS, QS, 4, HIGH, has_lone_form<WS, 4, HIGH>()><<<grid, block, 0, a.stream>>>(p);
        else
            spmm_direct_inner_kernel<KS, WS, QS, 4, HIGH, false><<<grid, block, 0, a.stream>>>(p);
    } else if (eight) {
        spmm_direct_inner8_kernel<KS, WS, QS, 2, HIGH, has_lone_form<WS, 2, HIGH>()><<<grid, dim3(512), 0, a.stream>>>(p);
    } else {
        if (lone && has_lone_form<WS, 2, HIGH>())
            spmm_direct_inner_kernel<KS, WS, QS, 2, HIGH, has_lone_form<WS, 2, HIGH>()><<<grid, block, 0, a.stream>>>(p);
        else
            spmm_direct_inner_kernel<KS, WS, QS, 2, HIGH, false><<<grid, block, 0, a.stream>>>(p);
    }
    return hipGetLastError();
}

// Every workgroup has four waves: 1 x 4, 2 x 2 or 4 x 1 (rows x column vectors), chosen by the
// column-block width the indices were preprocessed for.  A wave is 256 or 128 rows tall, whichever
// the run-time model expects to finish first: the taller wave halves the B and index loads per
// MFMA, but only two such workgroups fit a CU, which quantises badly on mid-sized problems.
// The tail handling is planned for a single reduction slice.
static TailPlan tail_plan_for(const SpmmArgs& a)
{
    TailPlan none;
    none.blocks = choose_wave_blocks(a.M, a.N, a.W / a.kept, a.kept, a.split_k);
    none.head = none.tail = 0;
    none.separate = false;
    none.sub = 1;
    none.fused = false;
    none.along_k = false;
    none.eighths = false;
    none.units = false;
    if (a.split_k != 1)
        return none;
    TailPlan t = plan_tail(a.M, a.N, a.W / a.kept, a.kept, 128 / a.Ns);
    if (t.head + t.tail * t.sub > 0x7fffffffLL)
        return none;
    return t;
}

template <int KS, int WS, bool HIGH>
static hipError_t launch_ns(const SpmmArgs& a)
{
    if (a.split_k == 1 && a.W / WS >= 4 && inner_split_pays(a.M, a.N, a.W / WS, WS)) {
        switch (a.Ns) {
        case 128: return launch_inner<KS, WS, 4, HIGH>(a);
        case 64: return launch_inner<KS, WS, 2, HIGH>(a);
        case 32: return launch_inner<KS, WS, 1, HIGH>(a);
        }
    }
    const TailPlan plan = tail_plan_for(a);
    const bool tall = plan.blocks == 8;
    if (!tall && a.Ns == 128 && short_waves_pay(a.M))
        return launch_cfg<KS, WS, 4, 1, 2, HIGH>(a, plan);
    switch (a.Ns) {
    case 128:
        return tall ? launch_cfg<KS, WS, 4, 1, 8, HIGH>(a, plan) : launch_cfg<KS, WS, 4, 1, 4, HIGH>(a, plan);
    case 64:
        return tall ? launch_cfg<KS, WS, 2, 2, 8, HIGH>(a, plan) : launch_cfg<KS, WS, 2, 2, 4, HIGH>(a, plan);
    case 32:
        return tall ? launch_cfg<KS, WS, 1, 4, 8, HIGH>(a, plan) : launch_cfg<KS, WS, 1, 4, 4, HIGH>(a, plan);
    }
    return hipErrorInvalidValue;
}

bool mfma_supported(const SpmmArgs& a)
{
    if (a.a_rowmajor)
        return false;
    if (a.vec_len != 32 || (a.Ns != 32 && a.Ns != 64 && a.Ns != 128))
        return false;
    // any pitch: 128-bit buffer loads only need their address on a 4-byte boundary, and their range
    // check is per 32-bit word (a pitch that is a multiple of four floats keeps them on 16-byte
    // boundaries, which is faster)
    if (a.lda < a.M || a.M < 32)
        return false;
    // 32-bit buffer offsets: one window of A and one window of B must stay below 2 GiB; the row
    // offset of A is formed with a 24-bit multiply
    if ((size_t)a.window * a.lda * sizeof(float) >= 0x80000000ull || (size_t)a.kept * a.N * sizeof(float) >= 0x80000000ull)
        return false;
    if ((size_t)a.lda * sizeof(float) >= (1u << 24))
        return false;
    // a wave's 256 rows of C are addressed with 32-bit offsets
    if ((size_t)256 * a.N * sizeof(float) >= 0x80000000ull)
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
