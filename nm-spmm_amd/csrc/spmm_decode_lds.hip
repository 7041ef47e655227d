// Decode-sized multiplication (2 to 32 rows) on the row list with the rows of A staged in LDS.
//
// spmm_decode_kernel (spmm_decode.hip) gathers A from global memory: per kept row and 32-column
// vector one request of 4 M bytes, W of them per workgroup, every one an L1 miss that waits in the
// L2's queues behind B's misses to HBM.  Here a workgroup takes a slice of the reduction (a range
// of dense rows of A small enough for the LDS: the reference kernels stage A the same way,
// src/kernel_64x128_8x8.cu:139-159, and gather from shared memory, :371) and several column
// vectors.  It copies its rows of A into LDS once, with coalesced 128-bit loads that do not depend
// on the list, and every gather afterwards is an LDS read: the only requests left while B streams
// are B's own cache lines and the list.
//
//   workgroup id = slice * vgroups + vgroup; 16 waves; V = 1, 2, 4, 8 or 16 vectors per workgroup,
//   16 / V waves per vector, wave (vector j, sub s) takes the slice's groups s, s + 16 / V, ...
//
// The k-step is the one of spmm_decode_kernel (four kept rows on v_mfma_f32_16x16x4_f32, even and
// odd columns in two tiles; up to 16 rows one pair of tiles per wave, 17 to 32 rows two).  The
// waves of a vector add their tiles through LDS (the region that held A) in wave order; with more
// than one slice the sums go to scratch as partial tiles and the slice that arrives last adds them
// up in slice order (arrival words as in spmm_decode.hip): one launch, no workgroup waits for
// another, the same bits on every run.
#include "internal.h"

#include <algorithm>
#include <atomic>

namespace nmspmm {

typedef float lfloatx4 __attribute__((ext_vector_type(4)));
typedef int lintx4 __attribute__((ext_vector_type(4)));

struct DecodeLdsParams {
    const float* A;
    const float* B;
    const int32_t* R;
    float* C;
    int M, N, W, G, Q;
    int lda;         // floats between dense rows (column-major A) or between rows (row-major A)
    int rowmajor;    // A is row-major M x K
    int fill;        // 0: 128-bit copies of a column-major A (M and lda multiples of 4), 1: element by element
    uint32_t a_bytes, b_bytes;
    int accumulate;
    int window, kept;
    int V, vgroups, slices;
    int pitch;       // floats per dense row in LDS
    int lds_rows;    // dense rows the LDS region holds
    float* part;     // [Q][slices][HB][512] partial tiles (slices > 1)
    unsigned long long* tickets;
    unsigned long long epoch;
};

__device__ inline __amdgpu_buffer_rsrc_t dl_rsrc(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

constexpr int kLdsWaves = 16;

// HB: 16-row halves per wave (1: M <= 16, 2: M <= 32).  NT: B is loaded with the non-temporal hint.
template <int HB, bool NT>
__global__ void __launch_bounds__(64 * kLdsWaves) spmm_decode_lds_kernel(const DecodeLdsParams p)
{
    extern __shared__ float lds[];  // A[lds_rows][pitch], afterwards the waves' tiles [16][8 HB][64]
    __shared__ unsigned int arrival[kLdsWaves];
    constexpr int kAux = NT ? 2 : 0;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kq = lane >> 4, jl = lane & 15;
    const int vgroup = (int)(blockIdx.x % (unsigned)p.vgroups);
    const int slice = (int)(blockIdx.x / (unsigned)p.vgroups);
    const int M = p.M, N = p.N, pitch = p.pitch;

    // this slice's groups of 16 kept rows and the dense rows of A they can name
    int g_first = 0, g_count = p.G;
    split_windows(p.G, p.slices, slice, &g_first, &g_count);
    const int r_lo = 16 * g_first, r_hi = min(p.W, 16 * (g_first + g_count));
    const int k_lo = r_lo / p.kept * p.window;
    const int span = min((r_hi + p.kept - 1) / p.kept * p.window - k_lo, p.lds_rows);

    // ---- A[k_lo .. k_lo + span) into LDS --------------------------------------------------------
    const __amdgpu_buffer_rsrc_t ra = dl_rsrc(p.A, p.a_bytes);
    if (p.rowmajor) {
        // a wave instruction moves 4 rows x 64 dense rows: lane (il, kc) = (lane / 16, lane % 16)
        // loads A[4 ib + il][k_lo + 64 kb + 4 kc .. + 3] (256 contiguous bytes per row) and writes
        // four words `pitch` apart; pitch is odd, so the 64 lanes of a write hit 64 banks
        const int il = lane >> 4, kc = lane & 15;
        const int nI = (M + 3) / 4, nK = (span + 63) / 64;
        for (int u = wave; u < nI * nK; u += kLdsWaves) {
            const int i = 4 * (u % nI) + il, k = 64 * (u / nI) + 4 * kc;
            if (i < M && k < span) {
                const auto x = __builtin_amdgcn_raw_buffer_load_b128(
                    ra, (uint32_t)(((size_t)i * p.lda + k_lo + k) * sizeof(float)), 0, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    lds[(k + e) * pitch + i] = __int_as_float(x[e]);
            }
        }
    } else if (p.fill == 0) {
        // column-major, M and lda multiples of 4: chunk c is floats [4 part, 4 part + 4) of dense row k
        const int per_row = M / 4, chunks = span * per_row;
        constexpr int kUnroll = 4;
        for (int c0 = tid; c0 < chunks; c0 += 64 * kLdsWaves * kUnroll) {
            lintx4 x[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int c = c0 + u * 64 * kLdsWaves;
                const int k = c / per_row, part = c % per_row;
                // chunks beyond the slice land beyond the descriptor and load 0; they are not written
                const uint32_t off = c < chunks ? (uint32_t)(((size_t)(k_lo + k) * p.lda + 4 * part) * sizeof(float)) : 0xfffffff0u;
                const auto y = __builtin_amdgcn_raw_buffer_load_b128(ra, off, 0, 0);
                x[u] = {(int)y[0], (int)y[1], (int)y[2], (int)y[3]};
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int c = c0 + u * 64 * kLdsWaves;
                if (c < chunks) {
                    const int k = c / per_row, part = c % per_row;
                    *reinterpret_cast<lintx4*>(&lds[k * pitch + 4 * part]) = x[u];
                }
            }
        }
    } else {
        for (int e = tid; e < span * M; e += 64 * kLdsWaves) {
            const int k = e / M, i = e % M;
            lds[k * pitch + i] = __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(
                ra, (uint32_t)(((size_t)(k_lo + k) * p.lda + i) * sizeof(float)), 0, 0));
        }
    }

    // ---- this wave's vector and groups ----------------------------------------------------------
    const int wpv = kLdsWaves / p.V;  // waves per vector
    const int my_vec = wave / wpv, my_sub = wave % wpv;
    const int v = vgroup * p.V + my_vec;
    const bool live = v < p.Q;
    const int cnt = live ? (g_count - my_sub + wpv - 1) / wpv : 0;
    auto group_of = [&](int x) { return g_first + my_sub + x * wpv; };
    // every offset that relies on a descriptor's range check is a vector offset
    const __amdgpu_buffer_rsrc_t rb = dl_rsrc(p.B + (size_t)(live ? v : 0) * 32, p.b_bytes);
    const __amdgpu_buffer_rsrc_t rr = dl_rsrc(p.R + (size_t)(live ? v : 0) * p.G * 16, (uint32_t)p.G * 64u);
    const uint32_t b_lane = (uint32_t)(((size_t)kq * N + 2 * jl) * sizeof(float));
    const uint32_t b_step = (uint32_t)((size_t)4 * N * sizeof(float));
    // lanes whose row of C does not exist read the last row that does (their tile rows are never stored)
    int a_lane[HB];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb)
        a_lane[hb] = min(jl + 16 * hb, M - 1);

    auto load_rows = [&](int g) -> lintx4 {
        const auto x = __builtin_amdgcn_raw_buffer_load_b128(rr, (uint32_t)(g * 64 + kq * 16), 0, 0);
        lintx4 r = {(int)x[0], (int)x[1], (int)x[2], (int)x[3]};
        return r;
    };
    auto load_b = [&](int g, float2 (&dst)[4]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            // rows at or beyond W (the tail of the last group) lie beyond the descriptor: 0
            const auto x = __builtin_amdgcn_raw_buffer_load_b64(rb, b_lane + (uint32_t)g * 4u * b_step + t * b_step, 0, kAux);
            dst[t] = make_float2(__int_as_float(x[0]), __int_as_float(x[1]));
        }
    };
    lfloatx4 acc_e[HB], acc_o[HB];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
        acc_e[hb] = {0.0f, 0.0f, 0.0f, 0.0f};
        acc_o[hb] = {0.0f, 0.0f, 0.0f, 0.0f};
    }
    // the list holds row + 1; 0 (no such kept row) and rows outside the slice (a malformed list) give 0
    auto multiply = [&](const lintx4& rows, const float2 (&b)[4]) {
        float a[4][HB];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int rel = rows[t] - 1 - k_lo;
            const bool ok = (unsigned)rel < (unsigned)span;
            const int at = (ok ? rel : 0) * pitch;
#pragma unroll
            for (int hb = 0; hb < HB; ++hb) {
                const float x = lds[at + a_lane[hb]];
                a[t][hb] = ok ? x : 0.0f;
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int hb = 0; hb < HB; ++hb) {
                acc_e[hb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][hb], b[t].x, acc_e[hb], 0, 0, 0);
                acc_o[hb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t][hb], b[t].y, acc_o[hb], 0, 0, 0);
            }
    };

    // B and the list do not wait for A: the first two groups' requests go out before the barrier
    // that ends the fill, and from then on two groups are in flight while another is multiplied
    float2 b0[4], b1[4], b2[4];
    lintx4 r0, r1, r2;
    if (cnt > 0) {
        r0 = load_rows(group_of(0));
        load_b(group_of(0), b0);
    }
    if (cnt > 1) {
        r1 = load_rows(group_of(1));
        load_b(group_of(1), b1);
    }
    __syncthreads();
    for (int i = 0; i < cnt; ++i) {
        if (i + 2 < cnt) {
            r2 = load_rows(group_of(i + 2));
            load_b(group_of(i + 2), b2);
        }
        multiply(r0, b0);
        r0 = r1;
        r1 = r2;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            b0[t] = b1[t];
            b1[t] = b2[t];
        }
    }

    // ---- the waves of a vector add their tiles in wave order ------------------------------------
    // value x of a lane: register x % 4 of the even (x % 8 < 4) or odd columns of half x / 8;
    // register r of lane (kq, jl) is tile row 4 kq + r
    constexpr int kTile = 8 * HB * 64;
    __syncthreads();  // every wave is done with A
#pragma unroll
    for (int hb = 0; hb < HB; ++hb)
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            lds[(wave * 8 * HB + 8 * hb + x) * 64 + lane] = acc_e[hb][x];
            lds[(wave * 8 * HB + 8 * hb + 4 + x) * 64 + lane] = acc_o[hb][x];
        }
    __syncthreads();
    auto store_c = [&](int x, float s) {
        const int row = 16 * (x / 8) + 4 * kq + (x % 4);
        if (row < M) {
            float* const dst = p.C + (size_t)row * N + (size_t)v * 32 + 2 * jl + (x % 8) / 4;
            *dst = p.accumulate ? *dst + s : s;
        }
    };
    float* const mine = p.part + ((size_t)(live ? v : 0) * p.slices + slice) * kTile;
    if (live) {
        for (int x = my_sub; x < 8 * HB; x += wpv) {
            float s = lds[(my_vec * wpv * 8 * HB + x) * 64 + lane];
            for (int y = 1; y < wpv; ++y)
                s += lds[((my_vec * wpv + y) * 8 * HB + x) * 64 + lane];
            if (p.slices > 1)
                // partial tile to scratch with agent-scope stores: written through to where all dies agree
                __hip_atomic_store(&mine[x * 64 + lane], s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else
                store_c(x, s);
        }
    }
    if (p.slices == 1)
        return;
    // Publish, then arrive (the order is argued in spmm_decode.hip): every wave waits for the
    // acknowledgement of its stores before the barrier; after it one lane per vector raises the
    // vector's arrival word to this launch's epoch and adds one; the slice that arrives last reads
    // the partial tiles (agent-scope loads) after it has seen its number.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (live && my_sub == 0 && lane == 0) {
        (void)__hip_atomic_fetch_max(&p.tickets[v], p.epoch << 8, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long before = __hip_atomic_fetch_add(&p.tickets[v], 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        arrival[my_vec] = (unsigned int)(before & 0xffull);
    }
    __syncthreads();
    // Every wave helps with every vector of the workgroup whose last slice this is: item = (vector,
    // value).  The slices' values are requested together (eight at a time) and added in slice order.
    asm volatile("" ::: "memory");
    for (int item = wave; item < p.V * 8 * HB; item += kLdsWaves) {
        const int j = item / (8 * HB), x = item % (8 * HB);
        const int vj = vgroup * p.V + j;
        if (vj >= p.Q || arrival[j] != (unsigned int)(p.slices - 1))
            continue;
        const float* const tiles = p.part + (size_t)vj * p.slices * kTile + x * 64 + lane;
        float s = 0.0f;
        for (int z0 = 0; z0 < p.slices; z0 += 8) {
            float t[8];
#pragma unroll
            for (int z = 0; z < 8; ++z)
                t[z] = z0 + z < p.slices
                           ? __hip_atomic_load(&tiles[(size_t)(z0 + z) * kTile], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                           : 0.0f;
#pragma unroll
            for (int z = 0; z < 8; ++z)
                s += t[z];
        }
        const int row = 16 * (x / 8) + 4 * kq + (x % 4);
        if (row < M) {
            float* const dst = p.C + (size_t)row * N + (size_t)vj * 32 + 2 * jl + (x % 8) / 4;
            *dst = p.accumulate ? *dst + s : s;
        }
    }
    // the words go back to zero, so that a HIP graph that replays this launch (with this epoch)
    // finds what the first run found
    if (live && my_sub == 0 && lane == 0 && arrival[my_vec] == (unsigned int)(p.slices - 1))
        __hip_atomic_store(&p.tickets[v], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

namespace {

constexpr int kMaxLdsDevices = 64;
constexpr size_t kLdsBudget = 128 * 1024;  // of the 160 KB of a compute unit: one workgroup per CU
constexpr size_t kTilesBytes = (size_t)kLdsWaves * 8 * 64 * sizeof(float);

// dense rows of A that slice `z` of `slices` can name
int slice_span(int G, int W, int window, int kept, int slices, int z)
{
    int g_first = 0, g_count = G;
    split_windows(G, slices, z, &g_first, &g_count);
    const int r_lo = 16 * g_first, r_hi = std::min(W, 16 * (g_first + g_count));
    return (r_hi + kept - 1) / kept * window - r_lo / kept * window;
}

struct LdsPlan {
    int slices, V, pitch, lds_rows, fill;
    size_t lds_bytes;
};

bool plan_decode_lds(const SpmmArgs& a, LdsPlan* plan)
{
    const int G = (a.W + 15) / 16, Q = a.N / 32;
    const int halves = a.M <= 16 ? 1 : 2;
    int pitch, fill = 0;
    if (a.a_rowmajor) {
        pitch = (a.M + 3) / 4 * 4 + 1;
    } else if (a.M % 4 == 0 && a.lda % 4 == 0) {
        pitch = a.M;
    } else {
        pitch = a.M;
        fill = 1;
    }
    // fewest slices whose rows of A fit the LDS budget
    int slices = 0, rows = 0;
    for (int s = 1; s <= G && s <= 64; ++s) {
        int widest = 0;
        for (int z = 0; z < s; ++z)
            widest = std::max(widest, slice_span(G, a.W, a.window, a.kept, s, z));
        if ((size_t)widest * pitch * sizeof(float) <= kLdsBudget) {
            slices = s;
            rows = widest;
            break;
        }
    }
    if (slices == 0)
        return false;
    // as many vectors per workgroup as still give (nearly) one workgroup per compute unit; every
    // wave keeps at least one group
    const int cus = machine().cus;
    int V = 1;
    for (int cand = 16; cand >= 1; cand /= 2) {
        const int wgs = slices * ((Q + cand - 1) / cand);
        if (wgs * 10 >= cus * 8 && G / slices >= kLdsWaves / cand) {
            V = cand;
            break;
        }
    }
    plan->slices = slices;
    plan->V = V;
    plan->pitch = pitch;
    plan->lds_rows = rows;
    plan->fill = fill;
    plan->lds_bytes = std::max((size_t)rows * pitch * sizeof(float), kTilesBytes * halves);
    return true;
}

}  // namespace

bool decode_lds_supported(const SpmmArgs& a)
{
    if (a.row_index == nullptr || a.vec_len != 32 || a.M < 2 || a.M > 32 || !decode_supported(a))
        return false;
    LdsPlan plan;
    if (!plan_decode_lds(a, &plan))
        return false;
    if (plan.slices > 1) {
        const size_t tile_bytes = (size_t)8 * (a.M <= 16 ? 1 : 2) * 64 * sizeof(float);
        if (a.decode_part == nullptr || a.decode_tickets == nullptr || a.N / 32 > a.decode_ticket_count ||
            (size_t)(a.N / 32) * plan.slices * tile_bytes > a.decode_part_bytes || plan.slices > 255)
            return false;
    }
    return true;
}

hipError_t launch_decode_lds(const SpmmArgs& a)
{
    LdsPlan plan;
    if (!plan_decode_lds(a, &plan))
        return hipErrorInvalidValue;
    DecodeLdsParams p;
    p.A = a.A;
    p.B = a.B;
    p.R = a.row_index;
    p.C = a.C;
    p.M = a.M;
    p.N = a.N;
    p.W = a.W;
    p.G = (a.W + 15) / 16;
    p.Q = a.N / 32;
    p.lda = a.lda;
    p.rowmajor = a.a_rowmajor ? 1 : 0;
    p.fill = plan.fill;
    p.a_bytes = (uint32_t)((size_t)(a.a_rowmajor ? a.M : a.K) * a.lda * sizeof(float));
    p.b_bytes = (uint32_t)(((size_t)(a.W - 1) * a.N + 32) * sizeof(float));
    p.accumulate = (a.accumulate && a.split_k > 1) ? 1 : 0;
    p.window = a.window;
    p.kept = a.kept;
    p.V = plan.V;
    p.vgroups = (p.Q + plan.V - 1) / plan.V;
    p.slices = plan.slices;
    p.pitch = plan.pitch;
    p.lds_rows = plan.lds_rows;
    p.part = a.decode_part;
    p.tickets = a.decode_tickets;
    p.epoch = a.decode_epoch;
    const dim3 grid((unsigned)(p.vgroups * p.slices)), block(64 * kLdsWaves);
    const bool nt = a.stream_b;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxLdsDevices)
        return hipErrorInvalidDevice;
    // more than 64 KB of dynamic LDS has to be allowed once per kernel and device
#define NMSPMM_LDS_LAUNCH(HB, NT)                                                                                  \
    do {                                                                                                           \
        auto* const kernel = spmm_decode_lds_kernel<HB, NT>;                                                       \
        static std::atomic<bool> allowed[kMaxLdsDevices];                                                          \
        if (!allowed[dev].load(std::memory_order_acquire)) {                                                       \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),                        \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBudget); \
            if (e != hipSuccess)                                                                                   \
                return e;                                                                                          \
            allowed[dev].store(true, std::memory_order_release);                                                   \
        }                                                                                                          \
        kernel<<<grid, block, plan.lds_bytes, a.stream>>>(p);                                                      \
    } while (0)
    if (a.M <= 16) {
        if (nt)
            NMSPMM_LDS_LAUNCH(1, true);
        else
            NMSPMM_LDS_LAUNCH(1, false);
    } else {
        if (nt)
            NMSPMM_LDS_LAUNCH(2, true);
        else
            NMSPMM_LDS_LAUNCH(2, false);
    }
#undef NMSPMM_LDS_LAUNCH
    return hipGetLastError();
}

} // namespace nmspmm
