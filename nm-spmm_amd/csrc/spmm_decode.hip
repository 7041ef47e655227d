// Decode-sized multiplication (M <= 32, and 33 to 64 rows of a column-major A) on the row list: the index format this library adds for
// the memory-bound case, next to the reference's D / column_info buffers (which stay as they are).
//
// The reference layout makes a kernel chase two dependent loads before it can ask for a row of A:
// the window's ranks in D, then the window's column_info list (reference
// src/kernel_64x128_8x8.cu:371 and include/utils.h:82-95 for the meaning).  At decode sizes the
// whole launch lasts a few memory latencies, so that chain is a quarter of the run time.  The row
// list stores, per 32-column vector and kept row, the absolute dense row of A, in the order the
// lanes of this kernel consume it:
//
//   row_index[(v * G + g) * 16 + kq * 4 + t] = 1 + k(16 g + 4 t + kq, v),   0 where there is no such kept row
//
// with G = ceil(W / 16) groups of 16 kept rows per vector and k(r, v) the dense row that kept row
// r of vector v multiplies.  One 128-bit load per lane hands lane quarter kq the rows of its next
// four k-steps; no lane exchange, no second table, and the layout no longer depends on the window
// geometry or on Ns.
//
// Kernel: one workgroup per 32-column vector, 16 or 8 waves; wave w takes the groups w, w + 16,
// ... (so the waves of a workgroup, and with them the whole GPU, read one band of adjacent rows of
// B at a time).  A k-step is four kept rows on v_mfma_f32_16x16x4_f32: lane (kq, jl) = (l / 16, l % 16)
// loads B[4 s + kq][2 jl .. 2 jl + 1] with one 64-bit load (four 128-byte row segments per wave and
// instruction, each byte of B read once) and A[jl][row]; even and odd columns accumulate in two
// MFMA tiles.  17 to 32 rows take a second pair of tiles for the other 16 rows with the same B
// operands, 33 to 64 rows four pairs.  The waves add their tiles up through LDS in wave order (deterministic, one launch,
// no workspace).  Measured on the MI355X: more than one group per wave in flight does not help.
// The counters show a CU with about 64 requests outstanding whatever the kernel does, which looks
// like what its vector L1 keeps in flight: the 16 waves' one group each (256 lines of B plus their
// rows of A) already fill it, so the loop is: load a group, multiply it.
//
// Every workgroup asks for the same rows of A in the same order, and the workgroups of an XCD share
// its L2: in step, they all hit the same few cache lines (and L2 channels) at the same moment.  For
// long reductions (W >= 2048) of 8 to 16 rows the kernel therefore runs with 8 waves and lets
// workgroup j of an XCD start its walk 5 j groups further on, wrapping around (measured at
// K = Ncols = 8192, 2:8, M = 16, B resident in the Infinity Cache: 12.99 -> 12.22 us; with B
// streamed from HBM the 16 waves in step are 3 to 5 % ahead, which the caller can ask for with the
// non-temporal hint).  Fewer rows gather little of A and run faster on 16 waves either way, and so
// do shorter reductions and the 17-to-32-row form.
#include "internal.h"

namespace nmspmm {

typedef float dfloatx4 __attribute__((ext_vector_type(4)));
typedef int dintx4 __attribute__((ext_vector_type(4)));

struct DecodeParams {
    const float* A;
    const float* B;
    const int32_t* R;
    float* C;
    int M, N, W, G;
    // element (i, k) of A lies i * a_row_stride + k * a_k_stride bytes into its a_bytes bytes
    uint32_t a_row_stride, a_k_stride, a_bytes, b_bytes;
    int accumulate;
    int rotate;  // groups by which consecutive workgroups of an XCD stagger the start of their walk
    int xcds;    // accelerator dies: consecutive workgroup ids go to consecutive dies
    // cut reductions (SPLIT): workgroup id = slice * vectors + vector; each of the `slices` workgroups
    // of a vector leaves its partial tile in `part`, takes a ticket, and the last one adds them up.
    // A ticket word holds (epoch << 8) | arrivals and is zero between launches; `epoch` grows with
    // every launch on a device, so a word left behind by a launch that never finished is smaller
    // than epoch << 8 and counts as "no arrivals" too.
    float* part;
    unsigned long long* tickets;
    unsigned long long epoch;
    int slices, vectors;
    // rows cut across workgroups: the launch has `vectors` = Ncols / 32 x `parts` workgroups (per
    // slice), workgroup (v, q) computes rows [q * part_rows, min(M, (q + 1) * part_rows)) of vector v
    int parts, part_rows, real_vectors;
};

__device__ inline __amdgpu_buffer_rsrc_t dc_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// HB: 16-row halves (1: M <= 16, 2: M <= 32, 4: M <= 64).  WIDE (column-major A): one load fetches
// the rows of several halves at once, instead of one 32-bit load per half: HB = 2 a 64-bit load of
// rows 2 jl, 2 jl + 1; HB = 4 a 128-bit load of rows 4 jl .. 4 jl + 3 (half hb is then the rows
// HB t + hb, t the tile row).  The code is written for any multiple of four halves (two such loads
// 64 rows apart for eight), but eight halves were measured and dropped: at 128 rows and
// K = Ncols = 8192, 38.9 us on 16 waves and 41 us on 8 against the tile kernel's 36 at 2:8, 22.8
// against 24.3 us at 1:8.  NT: B is loaded with the non-temporal hint (it is not kept in the
// caches).  SPLIT: the reduction of a vector is cut across p.slices workgroups (fewer vectors than
// compute units would otherwise leave compute units idle).
template <int HB, bool WIDE, bool NT, int kDecodeWaves, bool SPLIT = false, int RING = 0>
__global__ void __launch_bounds__(64 * kDecodeWaves) spmm_decode_kernel(const DecodeParams p)
{
    constexpr int HBW = HB < 4 ? HB : 4;   // halves that one wide load serves
    constexpr int NW = HB / HBW;           // wide loads per lane and kept row
    constexpr int HBC = HB < 2 ? HB : 2;   // halves per pass of the reduction through LDS
    constexpr int kAux = NT ? 2 : 0;
    __shared__ float red[kDecodeWaves][8 * HBC][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4, jl = lane & 15;
    // vv: (vector, row part).  The parts of a vector get ids that differ by the number of XCDs, so
    // that they run on the same XCD at about the same time and share its L2's copy of B.
    const int vv = SPLIT ? (int)(blockIdx.x % (unsigned)p.vectors) : (int)blockIdx.x;
    const int slice = SPLIT ? (int)(blockIdx.x / (unsigned)p.vectors) : 0;
    int v = vv, part = 0;
    if (p.parts > 1) {
        if (p.real_vectors % p.xcds == 0) {
            const int slot = vv / p.xcds;
            part = slot % p.parts;
            v = (slot / p.parts) * p.xcds + vv % p.xcds;
        } else {
            part = vv % p.parts;
            v = vv / p.parts;
        }
    }
    const int m0 = part * p.part_rows;
    const int M = min(p.M - m0, p.part_rows), N = p.N;

    // every offset that relies on the descriptor's range check is a vector offset: the scalar
    // offset of a buffer load is not part of that check
    const __amdgpu_buffer_rsrc_t rb = dc_rsrc(p.B + (size_t)v * 32, p.b_bytes);
    const __amdgpu_buffer_rsrc_t rr = dc_rsrc(p.R + (size_t)v * p.G * 16, (uint32_t)p.G * 64u);
    const __amdgpu_buffer_rsrc_t ra = dc_rsrc(reinterpret_cast<const char*>(p.A) + (size_t)m0 * p.a_row_stride,
                                              p.a_bytes - (uint32_t)m0 * p.a_row_stride);
    const uint32_t a_stride = p.a_k_stride;
    // Lanes whose row of C does not exist read the last row that does (their tile rows are never
    // stored): out-of-range lanes would be dropped by the descriptor as well, but loads with most
    // lanes out of range are slow (M = 1, B streamed from HBM: 17.3 -> 13.6 us at K = Ncols = 8192,
    // 2:8).  The list holds row + 1; entry 0 (no such kept row, or a read beyond the list) selects
    // an offset beyond the descriptor, which loads 0.
    uint32_t a_lane[HB];
    if (WIDE) {
        // lane jl holds rows HBW jl .. HBW jl + HBW - 1 of each group of 16 HBW rows; a lane whose
        // rows all lie beyond M reads the last run that holds a live row (what a run reads beyond
        // row M - 1 is whatever follows it in A, or 0 beyond its end: those tile rows are never stored)
#pragma unroll
        for (int w = 0; w < NW; ++w)
            a_lane[w] = (uint32_t)min(16 * HBW * w + HBW * jl, (M - 1) / HBW * HBW) * (uint32_t)sizeof(float) - a_stride;
    } else {
#pragma unroll
        for (int hb = 0; hb < HB; ++hb)
            a_lane[hb] = (uint32_t)min(jl + 16 * hb, M - 1) * p.a_row_stride - a_stride;
    }
    auto a_offset = [&](uint32_t lane_part, int row) { return row > 0 ? lane_part + (uint32_t)row * a_stride : 0x80000000u; };
    const uint32_t b_lane = (uint32_t)(((size_t)kq * N + 2 * jl) * sizeof(float));
    const uint32_t b_step = (uint32_t)((size_t)4 * N * sizeof(float));

    dfloatx4 acc_e[HB], acc_o[HB];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
        acc_e[hb] = {0.0f, 0.0f, 0.0f, 0.0f};
        acc_o[hb] = {0.0f, 0.0f, 0.0f, 0.0f};
    }

    auto load_rows = [&](int g) -> dintx4 {
        const auto x = __builtin_amdgcn_raw_buffer_load_b128(rr, (uint32_t)(g * 64 + kq * 16), 0, 0);
        dintx4 r = {(int)x[0], (int)x[1], (int)x[2], (int)x[3]};
        return r;
    };

    // this wave's groups are wave, wave + kDecodeWaves, ...: cnt of them, walked from position
    // `first` on and around (consecutive workgroup ids go to different XCDs, so id / xcds counts the
    // workgroups of one XCD).  Positions advance by one with a wrap: the scalar work between a
    // group's MFMAs and the next group's loads is on every wave's critical path, so it is kept to
    // a compare and a select.
    // (a cut reduction: this workgroup's groups are [g_first, g_first + g_count), the partition rule
    // of every split here)
    int g_first = 0, g_count = p.G;
    if (SPLIT)
        split_windows(p.G, p.slices, slice, &g_first, &g_count);
    const int cnt = (g_count - wave + kDecodeWaves - 1) / kDecodeWaves;
    const int first = cnt > 0 ? (int)((blockIdx.x / (unsigned)p.xcds) * (unsigned)p.rotate % (unsigned)cnt) : 0;
    auto after = [&](int x) { return x + 1 >= cnt ? 0 : x + 1; };
    auto group_of = [&](int x) { return g_first + wave + x * kDecodeWaves; };
    auto load_a_step = [&](int row, float (&dst)[HB]) {
        if constexpr (WIDE && HBW == 2) {
            const auto x = __builtin_amdgcn_raw_buffer_load_b64(ra, a_offset(a_lane[0], row), 0, 0);
            dst[0] = __int_as_float(x[0]);
            dst[1] = __int_as_float(x[1]);
        } else if constexpr (WIDE) {
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const auto x = __builtin_amdgcn_raw_buffer_load_b128(ra, a_offset(a_lane[w], row), 0, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    dst[4 * w + e] = __int_as_float(x[e]);
            }
        } else {
#pragma unroll
            for (int hb = 0; hb < HB; ++hb)
                dst[hb] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(ra, a_offset(a_lane[hb], row), 0, 0));
        }
    };
    auto load_b_step = [&](int t, int g, float2& dst) {
        // rows at or beyond W (the tail of the last group) lie beyond the descriptor: 0
        const auto x = __builtin_amdgcn_raw_buffer_load_b64(rb, b_lane + (uint32_t)g * 4u * b_step + t * b_step, 0, kAux);
        dst = make_float2(__int_as_float(x[0]), __int_as_float(x[1]));
    };
    // A first: its addresses come from the row list, which has landed; the four loads of B follow
    // (measured against B first: 1 to 2 % faster)
    auto load_operands = [&](int g, const dintx4& rows, float (&av)[4][HB], float2 (&bv)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            load_a_step(rows[t], av[t]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t)
            load_b_step(t, g, bv[t]);
    };
    auto multiply_group = [&](const float (&av)[4][HB], const float2 (&bv)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int hb = 0; hb < HB; ++hb) {
                acc_e[hb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t][hb], bv[t].x, acc_e[hb], 0, 0, 0);
                acc_o[hb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t][hb], bv[t].y, acc_o[hb], 0, 0, 0);
            }
    };
    if constexpr (RING > 0) {
        // Short reductions (every wave has exactly RING groups): the launch lasts a few trips to
        // memory, so all of a wave's groups are requested at once - one trip for the lists, one for
        // the operands - instead of one trip per group.  Straight-line code: with wave-uniform
        // branches around the groups a wave does not have it was slower than the loop.
        dintx4 rows[RING];
        float av[RING][4][HB];
        float2 bv[RING][4];
#pragma unroll
        for (int r = 0; r < RING; ++r)
            rows[r] = load_rows(group_of(r));
#pragma unroll
        for (int r = 0; r < RING; ++r)
            load_operands(group_of(r), rows[r], av[r], bv[r]);
#pragma unroll
        for (int r = 0; r < RING; ++r)
            multiply_group(av[r], bv[r]);
    } else {
        // Software pipeline of depth one: while a group is multiplied the next group's operands and
        // the rows of the group after it are in flight.
        float2 b[4];
        float a[4][HB];
        dintx4 rows_next;
        int x_next = after(first);  // position whose rows are in rows_next
        if (cnt > 0) {
            const dintx4 rows = load_rows(group_of(first));
            rows_next = load_rows(group_of(x_next));
            load_operands(group_of(first), rows, a, b);
        }
        for (int i = 0; i < cnt; ++i) {
            multiply_group(a, b);
            if (i + 1 < cnt) {
                load_operands(group_of(x_next), rows_next, a, b);
                x_next = after(x_next);
                rows_next = load_rows(group_of(x_next));  // after the last group: a group that is not used
            }
        }
    }

    // The waves' tiles are added in wave order, HBC halves per pass through LDS.  Value x of a lane:
    // register x % 4 of the even (x % 8 < 4) or odd columns of half x / 8; register r of lane
    // (kq, jl) is tile row 4 kq + r.
    auto row_of = [&](int x) {
        const int tile_row = 4 * kq + (x % 4), hb = x / 8;
        return WIDE ? 16 * HBW * (hb / HBW) + HBW * tile_row + hb % HBW : 16 * hb + tile_row;
    };
    auto store_c = [&](int x, float s) {
        const int row = row_of(x);
        if (row < M) {
            float* const dst = p.C + (size_t)(m0 + row) * N + (size_t)v * 32 + 2 * jl + (x % 8) / 4;
            *dst = p.accumulate ? *dst + s : s;
        }
    };
    constexpr int kTile = 8 * HB * 64;
    float* const mine = SPLIT ? p.part + ((size_t)vv * p.slices + slice) * kTile : nullptr;
#pragma unroll
    for (int pass = 0; pass < HB / HBC; ++pass) {
        if (pass > 0)
            __syncthreads();  // the previous pass has been read
#pragma unroll
        for (int hh = 0; hh < HBC; ++hh)
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                red[wave][8 * hh + x][lane] = acc_e[pass * HBC + hh][x];
                red[wave][8 * hh + 4 + x][lane] = acc_o[pass * HBC + hh][x];
            }
        __syncthreads();
        for (int xl = wave; xl < 8 * HBC; xl += kDecodeWaves) {
            float s = red[0][xl][lane];
#pragma unroll
            for (int y = 1; y < kDecodeWaves; ++y)
                s += red[y][xl][lane];
            const int x = pass * 8 * HBC + xl;
            if constexpr (SPLIT)
                // partial tile to scratch with device-scope stores (they reach the point where the
                // other dies see them)
                __hip_atomic_store(&mine[x * 64 + lane], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else
                store_c(x, s);
        }
    }
    if constexpr (SPLIT) {
        // Publish, then take a ticket.  No workgroup ever waits for another: whoever draws the last
        // ticket of its vector finds all partial tiles complete.  What makes this true:
        //   - the partial tiles are written and read with agent-scope atomic stores and loads (sc1:
        //     written through to, and read from, the level at which all dies agree; no cache of
        //     this or another die can hold a stale copy for such a load to hit);
        //   - every wave waits until all its stores have been acknowledged (s_waitcnt vmcnt(0):
        //     on this GPU stores count in vmcnt) before it enters the barrier, so when lane 0 draws
        //     the ticket after the barrier every lane's part of the tile has arrived;
        //   - the last arrival reads the tiles only after it has seen its ticket (through LDS and a
        //     barrier): its loads are issued after every other slice's arrival, hence after their
        //     stores were acknowledged.
        // A release fence at workgroup scope does not wait for global stores here (all waves of a
        // workgroup share a CU), and the slices run on other CUs and dies.  A release fence at agent
        // scope would give the order as well, but it also writes back everything the die's L2 holds
        // dirty (other workgroups' rows of C): measured 12 -> 60 us at K = 11008 on 4096 columns.
        __shared__ unsigned int ticket;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            // Raise the word to this launch's epoch with no arrivals (a word of this epoch is larger
            // and stays), then arrive.  Both are read-modify-writes of one location by one lane, so
            // they take effect in this order, and only the second one's answer is waited for.
            (void)__hip_atomic_fetch_max(&p.tickets[vv], p.epoch << 8, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const unsigned long long before =
                __hip_atomic_fetch_add(&p.tickets[vv], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ticket = (unsigned int)(before & 0xffull);  // 0 for the first arrival
        }
        __syncthreads();
        if (ticket != (unsigned int)(p.slices - 1))
            return;
        asm volatile("" ::: "memory");
        // This is the last arrival, so nobody touches the word again in this launch: it goes back
        // to zero now (the store travels while the tiles are added up).  A HIP graph that replays
        // this launch carries this launch's epoch again and must find what the first run found; a
        // launch that is cut short leaves its word behind and the next launch's larger epoch
        // overrides it.
        if (tid == 0)
            __hip_atomic_store(&p.tickets[vv], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int x = wave; x < 8 * HB; x += kDecodeWaves) {
            float s = 0.0f;
            for (int z = 0; z < p.slices; ++z)
                s += __hip_atomic_load(&p.part[((size_t)vv * p.slices + z) * kTile + x * 64 + lane], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            store_c(x, s);
        }
    }
}

bool decode_supported(const SpmmArgs& a)
{
    // up to 32 rows either layout of A; 33 to 64 rows only column-major (wide loads of A); 65 to 128
    // rows where they are cut into parts of at most 32 rows (few column vectors)
    if (a.row_index == nullptr || a.M > 128 || a.vec_len != 32)
        return false;
    if (a.M > 64 && decode_part_rows(a.M, a.N / 32) > 32)
        return false;
    if (a.a_rowmajor) {
        if (a.M > 32)
            return false;
        if (a.lda < a.K || (size_t)a.M * a.lda * sizeof(float) >= 0x80000000ull)
            return false;
    } else {
        if (a.lda < a.M || (size_t)a.K * a.lda * sizeof(float) >= 0x80000000ull)
            return false;
    }
    // 32-bit offsets into B from a vector's first column, and into a vector's part of the list
    // (the last group's rows beyond W, and a group beyond the list, must stay beyond B's descriptor
    // without wrapping: 16 rows more)
    if (((size_t)a.W + 32) * a.N * sizeof(float) >= 0xffffffffull || (size_t)a.W * 4 + 64 >= 0xffffffffull)
        return false;
    return true;
}

hipError_t launch_decode(const SpmmArgs& a)
{
    DecodeParams p;
    p.A = a.A;
    p.B = a.B;
    p.R = a.row_index;
    p.C = a.C;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.G = (a.W + 15) / 16;
    p.a_row_stride = (uint32_t)(a.a_rowmajor ? a.lda * sizeof(float) : sizeof(float));
    p.a_k_stride = (uint32_t)(a.a_rowmajor ? sizeof(float) : a.lda * sizeof(float));
    p.a_bytes = (uint32_t)((size_t)(a.a_rowmajor ? a.M : a.K) * a.lda * sizeof(float));
    p.b_bytes = (uint32_t)(((size_t)(a.W - 1) * a.N + 32) * sizeof(float));
    p.accumulate = (a.accumulate && a.split_k > 1) ? 1 : 0;
    p.rotate = 0;
    p.xcds = machine().xcds;
    const int real_vectors = a.N / 32;
    const int cus = machine().cus;
    // More than 16 rows on few vectors: the rows are cut into parts of 16 (or 32) with a workgroup
    // each, as far as that fills compute units that would idle otherwise.  The parts of a vector read
    // the same B (the second one from the L2 of their XCD) and disjoint rows of A and C: nothing to
    // add up, and each CU keeps the request count of the 16-row form.
    int parts = 1, part_rows = a.M;
    if (decode_part_rows(a.M, real_vectors) < a.M) {
        part_rows = decode_part_rows(a.M, real_vectors);
        parts = (a.M + part_rows - 1) / part_rows;
        // Up to 32 rows, where the caller's flag allows cut reductions and there is room for either
        // two slices or two parts but not both, the slices win (K = 11008 on 4096 columns, 32 rows:
        // 12.9 us with two slices, 15.9 us with two parts, 17.7 us with neither)
        const bool scratch = a.decode_part != nullptr && a.decode_tickets != nullptr;
        if (scratch && a.M <= 32 && cus / real_vectors >= 2 && p.G / 64 >= 2 && cus / (real_vectors * parts) < 2)
            parts = 1;
        if (parts == 1)
            part_rows = a.M;
    }
    const int vectors = real_vectors * parts;  // workgroups per slice
    const int m_wg = parts > 1 ? part_rows : a.M;
    const bool pairs = m_wg > 16 && !a.a_rowmajor && a.lda % 2 == 0 && a.M % 2 == 0;
    const int halves = m_wg <= 16 ? 1 : m_wg <= 32 ? 2 : 4;  // 16-row halves per wave
    p.parts = parts;
    p.part_rows = part_rows;
    p.real_vectors = real_vectors;

    // Fewer vectors than compute units: with scratch from the caller's flag, cut each reduction
    // across as many workgroups as fill the GPU once, as long as every wave of a slice keeps at
    // least four groups (the partial tiles, the ticket and the final sum cost about 1.3 us; measured
    // at 128 vectors: K = 11008 at 2:8 gains 11 to 27 % re-reading one B and 26 to 33 % with B from
    // HBM, K = 4096 nothing).
    int slices = 1;
    if (a.decode_part != nullptr && a.decode_tickets != nullptr) {
        int s = cus / vectors;
        if (s > p.G / 64)
            s = p.G / 64;
        if (s > 8)
            s = 8;
        const size_t tile_bytes = (size_t)8 * halves * 64 * sizeof(float);
        if (s >= 2 && vectors <= a.decode_ticket_count && (size_t)vectors * s * tile_bytes <= a.decode_part_bytes)
            slices = s;
    }
    p.part = a.decode_part;
    p.tickets = a.decode_tickets;
    p.epoch = a.decode_epoch;
    p.slices = slices;
    p.vectors = vectors;
    const bool nt = a.stream_b;
#define NMSPMM_DECODE_LAUNCH(HB, WIDE, WAVES, SPLIT, GRID)                                                  \
    do {                                                                                                    \
        if (nt)                                                                                             \
            spmm_decode_kernel<HB, WIDE, true, WAVES, SPLIT><<<GRID, dim3(64 * WAVES), 0, a.stream>>>(p);   \
        else                                                                                                \
            spmm_decode_kernel<HB, WIDE, false, WAVES, SPLIT><<<GRID, dim3(64 * WAVES), 0, a.stream>>>(p);  \
    } while (0)
    if (slices > 1) {
        const dim3 grid((unsigned)(vectors * slices));
        if (halves == 1)
            NMSPMM_DECODE_LAUNCH(1, false, 16, true, grid);
        else if (halves == 2 && pairs)
            NMSPMM_DECODE_LAUNCH(2, true, 16, true, grid);
        else if (halves == 2)
            NMSPMM_DECODE_LAUNCH(2, false, 16, true, grid);
        else
            NMSPMM_DECODE_LAUNCH(4, true, 16, true, grid);
        return hipGetLastError();
    }

    const dim3 grid((unsigned)vectors);
    // Short reductions, the same two to four groups for every wave (K = 4096 at 2:8 and 1:8): every
    // group of a wave is requested at once.  Measured at K = 4096 on 14336 columns, 1 / 8 / 16 rows:
    // 1:8 (two groups per wave) 6.2 / 6.8 / 7.0 -> 5.2 / 5.7 / 5.9 us, 2:8 (four) 11.4 / 12.4 / 12.5 ->
    // 11.1 / 11.8 / 12.0 us; 17 to 32 rows gain at two groups per wave (9.3 -> 8.2 us) and nothing at four.
    if (p.G % 16 == 0 && p.G >= 32 && p.G <= (halves == 1 ? 64 : halves == 2 ? 32 : 0)) {
#define NMSPMM_DECODE_RING(HB, WIDE, RING)                                                                   \
    do {                                                                                                      \
        if (nt)                                                                                               \
            spmm_decode_kernel<HB, WIDE, true, 16, false, RING><<<grid, dim3(64 * 16), 0, a.stream>>>(p);      \
        else                                                                                                  \
            spmm_decode_kernel<HB, WIDE, false, 16, false, RING><<<grid, dim3(64 * 16), 0, a.stream>>>(p);     \
    } while (0)
#define NMSPMM_DECODE_RINGS(HB, WIDE)                                                                        \
    do {                                                                                                      \
        if (p.G == 32)                                                                                        \
            NMSPMM_DECODE_RING(HB, WIDE, 2);                                                                  \
        else if (p.G == 48)                                                                                   \
            NMSPMM_DECODE_RING(HB, WIDE, 3);                                                                  \
        else                                                                                                  \
            NMSPMM_DECODE_RING(HB, WIDE, 4);                                                                  \
    } while (0)
        if (halves == 1)
            NMSPMM_DECODE_RINGS(1, false);
        else if (pairs)
            NMSPMM_DECODE_RING(2, true, 2);
        else
            NMSPMM_DECODE_RING(2, false, 2);
#undef NMSPMM_DECODE_RINGS
#undef NMSPMM_DECODE_RING
        return hipGetLastError();
    }
    if (halves == 1) {
        if (!nt && a.W >= 2048 && a.M >= 8 && vectors >= cus) {
            // (with fewer workgroups than compute units 8 waves per CU are too few: 16 then)
            p.rotate = 5;
            spmm_decode_kernel<1, false, false, 8><<<grid, dim3(64 * 8), 0, a.stream>>>(p);
        } else {
            NMSPMM_DECODE_LAUNCH(1, false, 16, false, grid);
        }
    } else if (halves == 2 && pairs) {
        NMSPMM_DECODE_LAUNCH(2, true, 16, false, grid);
    } else if (halves == 2) {
        NMSPMM_DECODE_LAUNCH(2, false, 16, false, grid);
    } else {
        NMSPMM_DECODE_LAUNCH(4, true, 16, false, grid);
    }
#undef NMSPMM_DECODE_LAUNCH
    return hipGetLastError();
}

// Builds the row list from the preprocessed buffers (D in its blocked layout, column_info on the
// high-sparsity layout): one thread per list entry, writes coalesced.
__global__ void __launch_bounds__(256)
row_index_kernel(const int32_t* __restrict__ D, const int32_t* __restrict__ cinfo, int32_t* __restrict__ R, int W,
                 int Q, int Qs, int window, int kept, int G)
{
    const size_t total = (size_t)Q * G * 16;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const int nwin = W / kept;
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += stride) {
        const int e = (int)(o % 16);
        const size_t vg = o / 16;
        const int g = (int)(vg % G);
        const int v = (int)(vg / G);
        const int kq = e / 4, t = e % 4;
        const int r = 16 * g + 4 * t + kq;
        int out = 0;
        if (r < W) {
            const int jb = v / Qs, c = v % Qs;
            const int w = r / kept;
            int local = D[((size_t)jb * W + r) * Qs + c];
            if (cinfo != nullptr) {
                // a rank outside the window's list marks a malformed index: no row
                local = (unsigned)local < (unsigned)window ? cinfo[((size_t)jb * nwin + w) * window + local] : -1;
            }
            if ((unsigned)local < (unsigned)window)
                out = 1 + w * window + local;
        }
        R[o] = out;
    }
}

hipError_t launch_row_index(const int32_t* D, const int32_t* cinfo, int32_t* R, int W, int N, int window, int kept,
                            int Ns, hipStream_t stream)
{
    const int Q = N / 32, G = (W + 15) / 16;
    const size_t total = (size_t)Q * G * 16;
    size_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32)
        blocks = 256 * 32;
    if (blocks < 1)
        blocks = 1;
    row_index_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(D, cinfo, R, W, Q, Ns / 32, window, kept, G);
    return hipGetLastError();
}

} // namespace nmspmm
