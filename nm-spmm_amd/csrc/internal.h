// Shared declarations between the C-ABI layer and the kernel translation units.
#ifndef NMSPMM_INTERNAL_H
#define NMSPMM_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace nmspmm {

// One multiplication, already validated by the C-ABI layer.
struct SpmmArgs {
    const float* A;        // column-major M x K: element (i,k) at A[i + k*lda]
    const float* B;        // row-major W x N
    const int32_t* D;      // [N/Ns][W][Ns/vec_len]
    const int32_t* cinfo;  // [N/Ns][W/kept][window] or nullptr (low-sparsity layout)
    const int32_t* row_index;  // optional row list [N/32][ceil(W/16)][4][4] (spmm_decode.hip) or nullptr
    bool stream_b;         // B is loaded with the non-temporal hint (decode kernel on the row list)
    float* decode_part;    // decode kernel on the row list: scratch for partial tiles when a vector's
    size_t decode_part_bytes;  // reduction is cut across workgroups, and one arrival counter per vector
    unsigned long long* decode_tickets;  // (epoch << 8 | arrivals); all three 0 / nullptr: never cut
    unsigned long long decode_epoch;     // this launch's epoch: never 0, never that of an earlier launch on the device
    int decode_ticket_count;
    float* C;              // row-major M x N
    float* partial;        // split_k slices of slice_stride floats when split_k > 1, else nullptr
    size_t slice_stride;   // M * N rounded up to a multiple of 4
    int M, N, K, W;
    int lda;               // floats between consecutive dense rows of A; M unless the copy of a
                           // row-major A was padded (matrix-core path only)
    bool a_rowmajor;       // A is row-major M x K instead, `lda` floats between its rows (taken by
                           // the one-block decode kernels only)
    int window, kept, vec_len, Ns;
    int split_k;
    bool accumulate;       // split_k > 1 only: the sum of the slices is added to what C holds (the
                           // reference's atomicAdd reduction, include/ptx.h:34-40) instead of replacing it
    hipStream_t stream;
};

// What the run-time models and the tile walks need to know about the GPU: read once per device
// from the HIP runtime (capi.hip); the figures of an MI355X in its single-partition mode when
// there is no device to ask (the planning entry points also work without a GPU).
struct Machine {
    int cus;        // compute units (hipDeviceAttributeMultiprocessorCount)
    int xcds;       // accelerator dies, each with its own L2 (hipDeviceAttributeNumberOfXccs)
    double clock;   // shader clock in Hz (hipDeviceAttributeClockRate)
};
const Machine& machine();

// Matrix-pipe time of one kept row of one 128-row x 128-column workgroup: 128.4 shader cycles
// (fitted on one MI355X at 2.39 GHz: 53.5 ns), i.e. kept/2 k-steps x 4 MFMAs x 64 cycles per window.
inline double kept_row_seconds() { return 128.4 / machine().clock; }

// Windows [begin, begin + count) of reduction slice `z` out of `split_k`: an even split when it
// divides, otherwise the first (nwin % split_k) slices take one extra window — the partition
// rule of the reference kernels (src/kernel_64x128_8x8.cu:20-37).
__host__ __device__ inline void split_windows(int nwin, int split_k, int z, int* begin, int* count)
{
    const int p = nwin / split_k, q = nwin % split_k;
    *begin = z < q ? z * (p + 1) : z * p + q;
    *count = z < q ? p + 1 : p;
}

// Pipe time of a 256-row wave relative to a 128-row one: twice the rows with half the B and index
// loads per MFMA.  Measured on eleven shapes from 2048 x 4096 x 4096 to 8192 cubed with every CU
// busy: 3 to 12 % less at 2:4, 2 to 7 % at 2:8, 1 to 7 % at 1:8, growing with the size of the
// problem (the tall waves' smaller traffic counts for more the longer the run); one figure per
// layout is used.
inline double tall_wave_cost(int kept) { return kept <= 8 ? 2.0 / 1.03 : 2.0 / 1.05; }

// Whether the last layer of a launch of fewer tiles than the GPU holds at once is computed by
// workgroups whose four waves share the reduction (four per tile, each a quarter of a tile's time
// and alone on its CU) rather than as two 64-row pieces per tile (0.55 of a tile's time each).
// Measured on 156 shapes of 288 to 640 tiles against the pieces: 10 to 13 % faster with one whole
// layer and at most 64 tiles after it (5 to 7 % at 1:8); level to 5 % slower with 65 to 128 tiles
// after it (two such workgroups per CU), and -7 to +3 % after two whole layers (that kernel's LDS
// lets a CU hold two workgroups only), so it is taken in the first case.  (Without a whole layer
// the whole problem takes the launch with waves along K, plan_inner.)
inline bool tail_along_k(long long tiles, int nwin)
{
    const long long cus = machine().cus;
    return tiles > cus && tiles <= cus + cus / 4 && nwin >= 8;
}
// With at least sixteen windows the last layer is cut finer: eight workgroups per tile, each 64 rows
// of one 32-column vector (32 KB of LDS, so that a CU holds the two or three that fall to it at
// once, next to whole tiles too), for up to 96 tiles after one to three whole layers.  Measured
// on 108 shapes (2:8, 2:4, 1:8, 3:8): after one whole layer 7 to 10 % faster than the four
// workgroups per tile with up to 32 tiles left, level to 3 % faster with 48 to 64, and 5 to 7 %
// faster than the 64-row pieces with 80 to 96 (2 to 4 % at 1:8; 512 x 11008 x 4096 at 2:8: 93.9 ->
// 88.3 us), level to 4 % slower with 128 (four to a CU); after two and three whole layers 11 to
// 14 % faster than the pieces with up to 32 tiles left, 4 to 10 % with 48 to 64, 0 to 3 % with 96;
// below sixteen windows slower at 1:8.  Same sums in the same order as the four per tile.
inline bool tail_along_k_eighths(long long tiles, int nwin)
{
    const long long cus = machine().cus;
    const long long whole = tiles / cus, layer = tiles % cus;
    return nwin >= 16 && whole >= 1 && whole <= 3 && layer > 0 && layer <= 3 * cus / 8;
}

// Leftover tiles of 256-row waves (two workgroups per CU) after at least one full round: `rest`
// tiles, each `unit` seconds of a CU's pipes.  Left in the launch they land packed on the CUs that
// free up first and the last round lasts as long as a full one (measured: 2752 tiles on 512 slots
// take six rounds, not 5.4; 768 tiles take two, not 1.5).  In a launch of their own they spread
// over all CUs, and cut into 2 or 4 pieces along M (128- or 64-row waves, 4 % and 20 % more loads
// per MFMA) they spread more evenly still: the piece count of the busiest CU, times the piece's
// share of a tile, decides.  A CU left with a single workgroup runs at about 0.9; the second
// launch costs about 12 us (the gap, and the first launch draining).  Returns the modelled time
// of the cheapest way and its piece count (0: leave the tiles in the launch).  Over 96 ragged
// LLM-layer shapes this choice is 4.1 % faster on average than leaving the tiles in the launch
// (best choice per shape: 4.3 %), up to 30 % on single shapes.  `pieces` 16 stands for the cut
// into workgroups of 64 rows of one vector (spmm_direct_units_kernel), measured against the
// pieces along M on 42 shapes of 16 to 96 leftover tiles (2:8, 1:8, 3:8): 6 to 9 % of the whole
// multiplication faster with 16 tiles left over, 4 to 8 % with 32, 2 to 5 % with 48, level beyond
// (4096 x 4224 x 4096 at 2:8: 276.7 -> 252.6 us); the same cut of 128-row tiles into eight
// (plan_tail), up to 96 tiles left over: 1 to 8 %.
inline double tall_tail_seconds(long long rest, double unit, int* pieces, int max_pieces = 4, int nwin = 0)
{
    static const double piece_cost[3] = {1.0, 1.04, 1.2};
    const long long cus = machine().cus;
    double best = 2.0 * unit;
    int best_sub = 0;
    for (int i = 0, sub = 1; i < 3 && sub <= max_pieces; ++i, sub *= 2) {
        const long long busiest = (rest * sub + cus - 1) / cus;
        const double s = busiest * unit / sub * piece_cost[i] / (busiest == 1 ? 0.9 : 1.0) + 12e-6;
        if (s < best) {
            best = s;
            best_sub = sub;
        }
    }
    // Or as sixteen workgroups per tile in that launch, each 64 rows of one 32-column vector with the
    // reduction shared between its four waves (from sixteen windows up; up to four to a CU): 0.13,
    // 0.21, 0.29 and 0.37 of a tile's time with one to four on the busiest CU.
    if (max_pieces >= 4 && nwin >= 16 && 16 * rest <= 4 * cus) {
        const long long busiest = (16 * rest + cus - 1) / cus;
        const double s = (0.05 + 0.08 * (double)busiest) * unit + 1e-6;  // their launch starts while the first drains
        if (s < best) {
            best = s;
            best_sub = 16;
        }
    }
    if (pieces)
        *pieces = best_sub;
    return best;
}
// Modelled run time in seconds of the matrix-core kernel for waves of `blocks` 32-row blocks (4 or
// 8; 2 for the 64-row waves of ragged row counts) and `split` reduction slices, without the second
// pass of a split.  A workgroup covers 32*blocks rows x 128 columns; per window it needs kept/2
// k-steps x blocks MFMAs x 64 cycles of each of its CU's four matrix pipes (2.39 GHz; taller and
// shorter waves differ by a few per cent in the loads they issue, tall_wave_cost).  A CU holds
// four workgroups of 128-row waves or two of 256-row waves at once and they share its pipes, so
// the 256 CUs retire the workgroups in rounds of 1024 or 512.  Fewer workgroups than that spread
// over the CUs and cost as much as the busiest CU (a CU left with one workgroup, one wave per
// SIMD, runs at about 0.9 of its rate).  After full rounds the leftovers land packed on the CUs
// that happen to free up first and cost a whole round, unless plan_tail (unsplit reductions only)
// gives them a launch of shorter pieces: tall_tail_seconds for 256-row waves, the piece costs
// below for 128-row ones.  Constants fitted to sweeps on one MI355X (mean error 6 %).
inline double model_kernel_seconds(int M, int N, int nwin, int kept, int blocks, int split)
{
    const long long cus = machine().cus;
    const double per_window = kept * kept_row_seconds() * (blocks == 8 ? tall_wave_cost(kept) : blocks == 2 ? 0.5 * 1.25 : 1.0);
    const double unit = per_window * ((nwin + split - 1) / split);
    const long long groups = (long long)((M + 32 * blocks - 1) / (32 * blocks)) * ((N + 127) / 128) * split;
    const int slots = blocks == 8 ? 2 : blocks == 2 ? 6 : 4;
    const long long full = groups / (cus * slots), rest = groups % (cus * slots);
    const long long busiest = (rest + cus - 1) / cus;
    if (blocks == 4 && split == 1) {
        // plan_tail computes the last tiles of such a launch as two 64-row pieces each.  Next to
        // whole tiles a piece costs 0.55 of a tile; alone on its CU (one 64-row wave per SIMD) it
        // hides less latency: 0.65 of a tile, 0.7 on the 1:8 geometry (in its form that loads B two
        // windows ahead)
        const double lone = kept <= 8 ? 0.7 : 0.65;
        const long long whole = rest / cus, layer = rest % cus;
        if (full == 0 && layer > 0 && layer <= cus / 2) {
            if (tail_along_k_eighths(rest, nwin))  // an eighth of a tile each: 0.105 of a tile's time per workgroup of the busiest CU
                return (whole + 0.105 * (double)((8 * layer + cus - 1) / cus)) * unit + 1e-6;
            if (tail_along_k(rest, nwin))  // a quarter of a tile each, one per CU at 0.9 of the rate
                return (whole + 0.25 / 0.9) * unit + 1e-6;
            return whole == 0 ? lone * unit : (whole + 0.55) * unit;
        }
        if (full >= 1 && rest > 0 && 8 * rest <= 3 * cus && nwin >= 16) {
            // eight workgroups per leftover tile at the end of the launch (plan_tail): 0.2, 0.35 and 0.5
            // of a tile's time with one, two and three on the busiest CU (measured after one round)
            const long long busiest_unit = (8 * rest + cus - 1) / cus;
            return (double)full * slots * unit + (0.05 + 0.15 * (double)busiest_unit) * unit + 1e-6;
        }
        if (full >= 1 && rest > 0 && rest <= cus / 2 * slots) {
            const long long busiest_piece = (2 * rest + cus - 1) / cus;
            return (double)full * slots * unit + (busiest_piece == 1 ? lone : 0.55 * busiest_piece) * unit + 10e-6;
        }
    }
    double t = (double)full * slots * unit;
    if (busiest > 0 && blocks == 8 && split == 1 && full >= 1) {
        t += tall_tail_seconds(rest, unit, nullptr, 4, nwin);  // plan_tail gives these leftovers a launch of shorter pieces
    } else if (busiest > 0) {
        // one workgroup per CU: a 128-row wave alone on its SIMD runs at 0.9 of the rate; a 256-row
        // wave with 16 or more kept rows per chunk keeps its pipe busy by itself (measured 3 to 5 %
        // ahead of two 128-row workgroups per CU at 2:4 and 2:8, behind at 1:8 and 3:8)
        const double lone_rate = blocks == 8 && kept >= 16 ? 1.0 : 0.9;
        const double spread = busiest * unit / (busiest == 1 ? lone_rate : 1.0);
        if (full < 2)
            t += spread;
        else if (split == 1 && rest <= cus / 2 * slots)
            t += spread + 6e-6;  // the leftovers get a launch of their own (plan_tail)
        else
            t += slots * unit;
    }
    return t;
}
// 64-row waves (two 32-row blocks) cost about 25 % more loads per MFMA; the kernel uses them, in
// place of 128-row ones on 128-wide column blocks, only where 128-row waves would multiply mostly
// padding (192 rows: three 64-row waves instead of two 128-row ones, +24 % measured).
inline bool short_waves_pay(int M)
{
    const int rows64 = (M + 63) / 64 * 64, rows128 = (M + 127) / 128 * 128;
    return rows64 * 8 <= rows128 * 7;
}
// Wave height (32-row blocks) the matrix-core kernel uses for a shape: the faster one by the model.
inline int choose_wave_blocks(int M, int N, int nwin, int kept, int split)
{
    if (M <= 128)
        return 4;
    return model_kernel_seconds(M, N, nwin, kept, 8, split) < model_kernel_seconds(M, N, nwin, kept, 4, split) ? 8 : 4;
}

// Tail handling of the tile kernel (split_k == 1): the 256 CUs retire 128 x 128 tiles 1024 at a
// time (256 x 128 tiles 512 at a time); when the last round is ragged, its `tail` tiles get a
// launch of their own, whole, in pieces along M, or as workgroups of 64 rows of one vector that
// share the reduction between their waves.  A launch of fewer than 1024 128-row tiles has no
// rounds; its last layer of tiles is cut in the same launch instead.
struct TailPlan {
    int blocks;      // 32-row blocks per wave (4 or 8)
    long long head;  // tiles computed whole
    long long tail;  // tiles computed apart from them
    int sub;         // > 1: the tail tiles run as `sub` pieces along M each, on waves of blocks / sub blocks
    bool fused;      // the pieces along M are part of the launch of the whole tiles, after them
    bool eighths;    // along_k with eight workgroups per tile (64 rows of one 32-column vector each)
    bool units;      // leftovers after full rounds run as `sub` workgroups each, 64 rows of one 32-column
                     // vector with the reduction shared between the four waves: in a launch of their
                     // own after 256-row waves, at the end of the same launch after 128-row waves
    bool along_k;    // fused, and the tail tiles run as four workgroups each (one per 128 rows of one
                     // 32-column vector) whose four waves share the reduction, instead of pieces along M
    bool separate;   // the tail tiles are planned apart from the whole tiles: in a launch of their own
                     // (they then spread over the CUs instead of landing packed on the ones that
                     // free up last) or, fused, as the last workgroups of the same launch
};
// `wr`: waves of a workgroup along M (1, 2 or 4 for column blocks of 128, 64 or 32): a tile is
// 32 * blocks * wr rows x 128 / wr columns.  `max_pieces`: the shortest waves the kernel has,
// as pieces of a 256-row wave.
inline TailPlan plan_tail(int M, int N, int nwin, int kept, int wr = 1, int max_pieces = 4)
{
    TailPlan t;
    t.blocks = choose_wave_blocks(M, N, nwin, kept, 1);
    const int tile_rows = 32 * t.blocks * wr, tile_cols = 128 / wr;
    const long long tiles = (long long)((M + tile_rows - 1) / tile_rows) * ((N + tile_cols - 1) / tile_cols);
    const long long cus = machine().cus;
    const long long slots = cus * (t.blocks == 8 ? 2 : 4);
    t.head = tiles;
    t.tail = 0;
    t.sub = 1;
    t.separate = false;
    t.fused = false;
    t.along_k = false;
    t.eighths = false;
    t.units = false;
    if (t.blocks == 4 && max_pieces >= 4) {
        // 128-row waves.  Fewer tiles than the CUs hold at once spread one per CU, then two per CU,
        // ..., and the launch lasts as long as the busiest CU: a last layer that covers at most half
        // of the CUs is computed as two 64-row pieces per tile, dispatched after the whole tiles in
        // the same launch, so that it covers twice as many CUs for about half as long (+25 to +40 %
        // up to 384 tiles, +17 % with two whole layers, +10 % with three).  After one or more full
        // rounds the workgroups of a CU finish close together and the dispatcher refills a CU's four
        // slots at once, so up to half a round of leftovers lands packed on a quarter of the CUs:
        // as pieces in a launch of their own they spread (+12 to +33 % at 2:8, up to +13 % at 1:8,
        // +6 to +21 % at 2:4 except around a quarter round, where whole tiles are 2 % better).
        // More than half a round left over: only its last layer, as above (+2 to +5 %).
        const long long rest = tiles % slots, layer = tiles % cus;
        t.separate = true;
        t.sub = 2;
        if (tiles >= slots && rest > 0 && rest <= slots / 2) {
            t.tail = rest;  // in a launch of their own: at the end of the first they would land packed too
            if (8 * rest <= 3 * cus && nwin >= 16) {  // eight workgroups per tile with the reduction shared between the waves
                t.units = true;
                t.sub = 8;
            }
        } else if (layer > 0 && layer <= cus / 2) {
            t.tail = layer;
            t.fused = true;
            t.eighths = tail_along_k_eighths(tiles, nwin);
            t.along_k = t.eighths || tail_along_k(tiles, nwin);
        } else {
            t.separate = false;
            t.sub = 1;
            return t;
        }
        t.head = tiles - t.tail;
        return t;
    }
    const long long rest = tiles % slots;
    if (tiles < slots || rest == 0)
        return t;
    if (t.blocks == 8) {
        int pieces = 0;
        tall_tail_seconds(rest, kept * kept_row_seconds() * tall_wave_cost(kept) * nwin, &pieces, max_pieces, nwin);
        if (pieces == 0)
            return t;
        t.separate = true;
        t.head = tiles - rest;
        t.tail = rest;
        t.sub = pieces;
        t.units = pieces == 16;
    } else {
        // 128-row form of the short-vector kernel (it has no 64-row pieces), four workgroups per
        // CU: the finer grain already fills the last round well after one full round (a launch of
        // their own was measured 0 to 16 % SLOWER there).  In steady state (two or more full
        // rounds) a launch of their own spreads few leftovers.
        if (tiles < 2 * slots || rest > slots / 2)
            return t;
        t.separate = true;
        t.head = tiles - rest;
        t.tail = rest;
    }
    return t;
}

// The launch with four waves along K (spmm_direct_inner_kernel): one workgroup per 128 or 64 rows
// of one 32-column vector, each of its four waves over a quarter of the windows, partial sums
// added in LDS.  It cuts the reduction without scratch or a second pass, for problems of at most
// 256 tiles of 128 x 128 (measured on 96 shapes, M = 192 ... 1024, against the best of the splits
// 1, 2, 4, 8 of the tile kernel: 2 to 56 % faster up to 256 tiles, 0 to 16 % slower at 512).
// Two workgroups of 128-row waves fit a CU (64 KB of LDS each): a layer of up to one per CU costs
// 1.17 of a workgroup's time (one wave per SIMD; 1.3 behind full pairs of layers), two layers
// together 2.16.  Workgroups of 64-row
// waves (32 KB) cost 0.56 of a taller one per layer, 0.62 when there is only one layer.  Both
// measured on 144 shapes (M = 160 ... 1024, four patterns, reductions of 2048 to 14336) with each
// form forced; the choice between them then lands within 1 % of the better one on average.
struct InnerPlan {
    bool pays;     // eligible at all
    int rows;      // 128 or 64 rows per workgroup
    int waves;     // 4, or 8 where every workgroup has a compute unit to itself
    double seconds;  // modelled kernel time
};
inline InnerPlan plan_inner(int M, int N, int nwin, int kept)
{
    InnerPlan r;
    r.pays = false;
    r.rows = 128;
    r.waves = 4;
    r.seconds = 0.0;
    const long long cus = machine().cus;
    const long long tiles = (long long)((M + 127) / 128) * ((N + 127) / 128);
    if (tiles > cus || nwin < 8 || M <= 32)
        return r;
    const long long vecs = N / 32;
    const long long g4 = (long long)((M + 127) / 128) * vecs, g2 = (long long)((M + 63) / 64) * vecs;
    const long long b4 = (g4 + cus - 1) / cus, b2 = (g2 + cus - 1) / cus;
    const double c4 = 2.16 * (double)(b4 / 2) + (b4 % 2 ? (b4 == 1 ? 1.17 : 1.3) : 0.0);
    const double c2 = 0.56 * (b2 == 1 ? 1.0 / 0.9 : (double)b2);
    const double unit = kept * kept_row_seconds() * ((nwin + 3) / 4);
    r.pays = true;
    r.rows = c2 < c4 ? 64 : 128;
    r.seconds = (c2 < c4 ? c2 : c4) * unit + 1e-6;
    // Eight waves along K (two per SIMD; 64 or 128 KB of LDS) where every workgroup gets a compute
    // unit to itself and there are at least 16 windows: on 64 rows if that is the form chosen and its
    // workgroups fit the compute units once, else on 128 rows if those do.  Measured: 64 rows 6 to
    // 16 % shorter than four waves with B in the caches and 12 to 30 % with B from HBM (K = 11008 on
    // 4096 columns at 1:8, 96 rows: 18.1 -> 15.2 and 23.7 -> 16.7 us); 128 rows against the two
    // 64-row workgroups per CU they replace (4096 columns, 129 to 256 rows) level with B in the
    // caches, 5 to 17 % shorter with B from HBM.  With more workgroups than compute units eight
    // waves are level to 5 % longer.
    if (nwin >= 16) {
        if (r.rows == 64 && g2 <= cus) {
            r.waves = 8;
        } else if (g4 <= cus) {
            r.rows = 128;
            r.waves = 8;
        }
    }
    // More than two layers of 64-row workgroups: the four forms (64 or 128 rows, four or eight
    // waves) are priced by a fit on 123 shapes with each form forced (320 to 2048 rows on 2048 to
    // 8192 columns, K = 4096 to 14336, 2:8, 2:4 and 1:8; mean error 1 to 2.5 % per form), in
    // `unit`s per workgroup per CU plus a fixed cost per layer and launch (the latter less the
    // 6 us that the tile kernel's launches of 100 to 256 tiles cost beyond their model, which
    // prices none: the two are compared).  A layer that is not
    // full costs 0.4 to 1 of a full one.  64-row workgroups cost 0.60 a layer; on four waves a CU
    // holds four of them and the few workgroups left after a full round of 1024 land packed on
    // the CUs that free up first (+0.38 and +0.12 with up to one and two layers left), on eight
    // waves it holds two and ends evenly.  128-row workgroups cost 0.95 a layer plus 0.155 per
    // workgroup; on four waves an odd layer runs one wave per SIMD (+0.22 with B in the caches, +0.6
    // to +0.8 with B streamed from HBM, which a single wave per SIMD hides badly: priced at 0.35,
    // which costs 0.2 % with B in the caches and halves the distance to the best form with B from
    // HBM, 1.1 -> 0.5 % on 51 shapes), on eight waves every layer has two, for 1.5 us more per layer
    // (the exchange between eight waves through 128 KB of LDS).  The choice lands within 0.3 % of the best form on average (2.2 % before, when only
    // the two four-wave forms were priced; 768 x 4096 x 14336 at 2:8: 194 -> 169 us, 640 x 4096 x
    // 8192 at 2:4: 189 -> 170 us).  Up to 128 rows the earlier pricing stays (the choice between this
    // kernel and the ones for few rows was fitted against it), and below 32 windows, where the fixed
    // costs decide and the forms were measured within 7 % of each other either way.
    if (g2 > 2 * cus && M > 128 && nwin >= 32) {
        const double q2 = (double)g2 / (double)cus, q4 = (double)g4 / (double)cus;
        const double frac2 = q2 - (double)(g2 / cus);
        const double layers2 = (double)(g2 / cus) + (frac2 > 0.0 ? 0.4 + 0.6 * frac2 : 0.0);
        const double left = q2 > 4.0 ? q2 - 4.0 * (double)(g2 / (4 * cus)) : 0.0;  // layers after full rounds of four
        const double packed = left > 0.0 && left <= 1.0 ? 0.38 : left > 1.0 && left <= 2.0 ? 0.12 : 0.0;
        const double c64 = 0.60 * layers2;
        const double c128 = 0.95 * (double)b4 + 0.155 * q4;
        const double odd = b4 % 2 == 1 && b4 >= 3 ? 0.35 : 0.0;
        struct Form { int rows, waves; double seconds; };
        const Form forms[4] = {
            {64, 4, (c64 + packed) * unit + 0.67e-6 * (double)b2 - 3.8e-6},
            {128, 4, (c128 + odd) * unit + 1.47e-6 * (double)b4 - 3.1e-6},
            {64, 8, c64 * unit + 1.13e-6 * (double)b2 - 3.3e-6},
            {128, 8, c128 * unit + 3.0e-6 * (double)b4 - 3.3e-6},
        };
        int best = 0;
        for (int i = 1; i < 4; ++i)
            if (forms[i].seconds < forms[best].seconds)
                best = i;
        r.rows = forms[best].rows;
        r.waves = forms[best].waves;
        // 0.97: where the two models tie (1024 rows on 4096 columns: 256 tiles, one per CU) the tile
        // kernel was measured level to 10 % behind this launch, never ahead
        r.seconds = 0.97 * forms[best].seconds;
    }
    return r;
}

// Whether an unsplit multiplication takes the launch with four waves along K.
inline bool inner_split_pays(int M, int N, int nwin, int kept)
{
    const InnerPlan inner = plan_inner(M, N, nwin, kept);
    if (!inner.pays)
        return false;
    int blocks = choose_wave_blocks(M, N, nwin, kept, 1);
    if (blocks == 4 && short_waves_pay(M))
        blocks = 2;
    return inner.seconds < model_kernel_seconds(M, N, nwin, kept, blocks, 1);
}

// Whether a launch of whole tiles of 256-row waves runs each workgroup as two sets of four waves,
// each set over half of the windows, added up in LDS (128 KB).  Such waves fit two to a SIMD, so a
// launch of at most one workgroup per CU leaves every SIMD with a single wave; with the second set
// the matrix pipe has another wave to issue from while one waits for its operands.  Measured over
// 2:8, 1:4 and 2:4 at 1024 to 4096 rows: 2 to 4 % shorter from 768 kept rows per vector up (2048 x
// 4096 x 4096 at 2:8: 126.8 -> 124.1 us; at 2:4: 246.7 -> 238.5), 1 to 3 % at 512, level at 384,
// 1 to 2 % longer at 256, where the second set's prologue and the exchange weigh more than the
// overlap gives.
inline bool wave_sets_pay(long long workgroups, int nwin, int kept)
{
    return workgroups <= machine().cus && (long long)nwin * kept >= 512;
}

// Whole multiplication on the tile kernel: 6 us per launch, C written at about 8 TB/s, the kernel,
// and for a split the second pass that moves (2 * split + 1) * M * N floats at about 8 TB/s (the
// slices are cache resident) plus 4 us for its launch behind the first.
inline double model_tile_seconds(int M, int N, int nwin, int kept, int split)
{
    const double c_bytes = (double)M * N * sizeof(float);
    int blocks = choose_wave_blocks(M, N, nwin, kept, split);
    if (blocks == 4 && short_waves_pay(M))
        blocks = 2;  // as launch_mfma does (the column-block width is taken to be 128)
    double kernel = model_kernel_seconds(M, N, nwin, kept, blocks, split);
    if (split == 1) {
        const InnerPlan inner = plan_inner(M, N, nwin, kept);
        if (inner.pays && inner.seconds < kernel)
            kernel = inner.seconds;  // launch_mfma takes that launch then
    }
    double t = 6e-6 + c_bytes / 8e12 + kernel;
    if (split > 1)
        t += (2.0 * split + 1.0) * c_bytes / 8e12 + 4e-6;
    return t;
}
// Rows per workgroup of the kernels that take one workgroup per 32-column vector: with at most
// half as many vectors as compute units, more than 16 rows are cut into parts of 16 rows, or of 32
// where 16-row parts would be more workgroups than compute units, one workgroup per vector and
// part.  The parts of a vector read the same B and disjoint rows of A and C, so nothing has to be
// added up.  Returns M where the rows are not cut.  (Parts of 64 rows for 65 to 128 rows were
// measured too: 4 to 12 % slower than the tile kernel on 4096 columns.)
inline int decode_part_rows(int M, int vectors)
{
    const long long cus = machine().cus;
    if (M <= 16 || 2LL * vectors > cus)
        return M;
    for (int rows = 16; rows <= 32 && rows < M; rows *= 2)
        if ((long long)((M + rows - 1) / rows) * vectors <= cus)
            return rows;
    return M;
}

// Whole multiplication on the decode kernel (M <= 128): one workgroup per 32-column vector (and
// part of the rows), 256 of them at a time, each needing kept/2 k-steps x (1, 2 or 4) MFMAs per
// window on the four matrix pipes of its CU (4.2 ns per kept row and 32-row block, measured),
// plus 5 us.
inline double model_decode_seconds(int M, int N, int nwin, int kept)
{
    const int vectors = (N + 31) / 32;
    const int rows = decode_part_rows(M, vectors);
    const int blocks = rows <= 32 ? 1 : rows <= 64 ? 2 : 4;
    const long long cus = machine().cus;
    const long long rounds = ((long long)vectors * ((M + rows - 1) / rows) + cus - 1) / cus;
    return 5e-6 + (double)rounds * nwin * kept * blocks * (10.08 / machine().clock);
}

// Matrix-core path (spmm_direct.hip).  Returns false when the geometry has no instantiation.
bool mfma_supported(const SpmmArgs& a);
hipError_t launch_mfma(const SpmmArgs& a);

// Matrix-core path for index vectors of 4, 8 or 16 columns (spmm_short.hip): low-sparsity layout,
// windows of 4, 8 or 16 rows, N a multiple of 128, K a multiple of 16.
bool short_supported(const SpmmArgs& a);
hipError_t launch_short(const SpmmArgs& a);

// Gathering matrix-core path for the same vector lengths at densities up to one half
// (spmm_gather.hip): multiplies kept rows only; K a multiple of 64 (32 for windows of 4 rows),
// N a multiple of 64, any M.
bool gather_supported(const SpmmArgs& a);
hipError_t launch_gather(const SpmmArgs& a);

// Decode-sized path (spmm_skinny.hip): M <= 32, the reference geometries, no workspace needed.
bool skinny_supported(const SpmmArgs& a);
hipError_t launch_skinny(const SpmmArgs& a);

// Decode-sized path on the row list (spmm_decode.hip): M <= 32 and a.row_index given.
bool decode_supported(const SpmmArgs& a);
hipError_t launch_decode(const SpmmArgs& a);
// Row list from the preprocessed D (and column_info on the high-sparsity layout).
hipError_t launch_row_index(const int32_t* D, const int32_t* cinfo, int32_t* R, int W, int N, int window, int kept,
                            int Ns, hipStream_t stream);

// Generic SIMT path (spmm_simt.hip): any window/kept, vec_len in {4, 8, 16, 32}, any M.
bool simt_supported(const SpmmArgs& a);
hipError_t launch_simt(const SpmmArgs& a);

// Sums split_k slices of `partial` in slice order (spmm_simt.hip) and stores the sum to C, or,
// with `accumulate`, adds it to what C holds.
hipError_t launch_splitk_reduce(const float* partial, float* C, size_t elems, size_t slice_stride,
                                int split_k, bool accumulate, hipStream_t stream);

// Index preprocessing kernels (preprocess.hip).
hipError_t launch_trans_index(int32_t* dDT, int W, int Q, int pN, int pM, hipStream_t stream);
// n0, m0, times: the pattern the indices were generated with and the transIndex doublings to fold
// into the read (times == 0: none).
hipError_t launch_reblock(const int32_t* in, int32_t* out, int W, int Q, int Qs, int n0, int m0, int times,
                          hipStream_t stream);
hipError_t launch_preprocess_high(int32_t* cinfo, int pM, int pN, const int32_t* in, int32_t* out,
                                  int W, int Q, int Qs, int n0, int m0, int times, hipStream_t stream);

// Dense <-> N:M vector-sparse conversion (compress.hip): m in {4, 8, 16, 32}, vec_len in {4, 8, 16, 32}.
bool compress_supported(int m, int vec_len);
hipError_t launch_compress(const float* B, float* BT, int32_t* DT, int K, int N, int n, int m, int vec_len,
                           hipStream_t stream);
hipError_t launch_decompress(const float* BT, const int32_t* DT, float* B, int K, int N, int n, int m, int vec_len,
                             hipStream_t stream);

// dst[c * dst_ld + r] = src[r * cols + c] for a rows x cols row-major src (transpose.hip).
hipError_t launch_transpose(const float* src, float* dst, int rows, int cols, int dst_ld, hipStream_t stream);

} // namespace nmspmm
#endif
