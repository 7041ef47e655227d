// C-ABI layer: argument validation, kernel-family dispatch and the per-device split-K workspace.
// Validation happens before any HIP call, so the error paths can be exercised without a GPU.
#include "../../include/nmspmm.h"
#include "internal.h"

#include <atomic>
#include <cmath>
#include <map>
#include <mutex>
#include <vector>

using namespace nmspmm;

namespace {

thread_local const char* g_last_kernel = "none";

struct Workspace {
    void* ptr = nullptr;
    size_t bytes = 0;
    std::vector<void*> retired;  // outgrown buffers: launches already enqueued may still use them
};
constexpr int kMaxDevices = 64;
Workspace g_workspace[kMaxDevices];
std::mutex g_workspace_mutex;

// Split-K slices for nmspmm_spmm_noalloc: device memory that exists from the moment the code object
// is loaded on a GPU until the process ends, one copy per GPU, so that entry point never allocates.
// Host code must not use the array's name as an address (on the host it is only a handle):
// noalloc_scratch() asks the runtime for the device address, once per device.
static __device__ __align__(256) unsigned char scratch[NMSPMM_NOALLOC_MAX_BYTES];
void* g_scratch_ptr[64] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device, or nullptr when the runtime cannot give it.
void* noalloc_scratch()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

// Arrival counters of the decode kernel's cut reductions (NMSPMM_DECODE_SPLIT), one 64-bit word per
// vector: (epoch << 8) | arrivals.  Every launch that cuts reductions draws a new epoch for its
// device, and a word that carries another epoch counts as "no arrivals yet": nothing has to be
// cleared between launches, and a launch that was cut short leaves nothing behind that a later
// one could trip over.  (56 bits of epoch: no wrap within a process's life.)
constexpr int kDecodeTickets = 1024;
static __device__ unsigned long long decode_tickets[kDecodeTickets];
unsigned long long* g_tickets_ptr[64] = {};
std::atomic<unsigned long long> g_decode_epoch[64];

unsigned long long next_decode_epoch()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        dev = 0;
    return (g_decode_epoch[dev].fetch_add(1, std::memory_order_relaxed) + 1) & 0x00ffffffffffffffull;
}

unsigned long long* decode_ticket_array()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_tickets_ptr[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(decode_tickets)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        g_tickets_ptr[dev] = (unsigned long long*)ptr;
    }
    return g_tickets_ptr[dev];
}

// The GPU's figures, asked once per device; without a device, an MI355X in single-partition mode.
Machine g_machine[kMaxDevices];
std::atomic<bool> g_machine_known[kMaxDevices];
const Machine kDefaultMachine = {256, 8, 2.4e9};
std::mutex g_machine_mutex;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t slice_stride(int M, int N) { return (((size_t)M * N + 3) / 4) * 4; }

int valid_vec_len(int v) { return v == 4 || v == 8 || v == 16 || v == 32; }

int check_index_shape(int W, int Q)
{
    return (W > 0 && Q > 0) ? NMSPMM_OK : NMSPMM_ERR_BAD_SHAPE;
}

// Grows (never shrinks) the calling device's cached workspace.  An outgrown buffer is kept until
// nmspmm_release(): another thread may have taken its address a moment ago and not launched yet,
// and launches already enqueued read it, so it is neither freed nor waited for here.  Growth is
// at least geometric, which bounds what the retired buffers hold to the size of the live one.
int cached_workspace(size_t bytes, void** out)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return NMSPMM_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    Workspace& ws = g_workspace[dev];
    if (ws.bytes < bytes) {
        const size_t want = bytes > 2 * ws.bytes ? bytes : 2 * ws.bytes;
        void* grown = nullptr;
        if (hipMalloc(&grown, want) != hipSuccess) {
            (void)hipGetLastError();
            if (want == bytes || hipMalloc(&grown, bytes) != hipSuccess)
                return NMSPMM_ERR_HIP;
            ws.bytes = bytes;
        } else {
            ws.bytes = want;
        }
        if (ws.ptr)
            ws.retired.push_back(ws.ptr);
        ws.ptr = grown;
    }
    *out = ws.ptr;
    return NMSPMM_OK;
}

// Device staging for the host-pointer preprocessing forms: one buffer per device, grown on demand
// and kept until nmspmm_release(), instead of an allocation per call.  Those calls are synchronous
// (they end with a copy back to the host), so a lease simply holds the lock for the duration of
// the call; an outgrown buffer has no work pending and is freed at once.
struct Staging {
    void* ptr = nullptr;
    size_t bytes = 0;
};
Staging g_staging[kMaxDevices];
std::mutex g_staging_mutex;

class StagingLease {
public:
    // `parts` regions of the given sizes, each on a 256-byte boundary
    StagingLease(const size_t* sizes, int parts) : lock_(g_staging_mutex)
    {
        int dev = 0;
        if (parts > kMaxParts || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
            return;
        size_t total = 0;
        size_t offset[kMaxParts];
        for (int i = 0; i < parts; ++i) {
            offset[i] = total;
            total += (sizes[i] + 255) / 256 * 256;
        }
        Staging& st = g_staging[dev];
        if (st.bytes < total) {
            if (st.ptr)
                (void)hipFree(st.ptr);
            st.ptr = nullptr;
            st.bytes = 0;
            if (hipMalloc(&st.ptr, total) != hipSuccess) {
                (void)hipGetLastError();
                st.ptr = nullptr;
                return;
            }
            st.bytes = total;
        }
        for (int i = 0; i < parts; ++i)
            part_[i] = (char*)st.ptr + offset[i];
        ok_ = true;
    }
    bool ok() const { return ok_; }
    void* part(int i) const { return part_[i]; }

private:
    static constexpr int kMaxParts = 3;
    std::lock_guard<std::mutex> lock_;
    void* part_[kMaxParts] = {nullptr, nullptr, nullptr};
    bool ok_ = false;
};

} // namespace

namespace nmspmm {

const Machine& machine()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return kDefaultMachine;
    }
    if (g_machine_known[dev].load(std::memory_order_acquire))
        return g_machine[dev];  // every call after the first on a device: no lock
    std::lock_guard<std::mutex> lock(g_machine_mutex);
    if (!g_machine_known[dev].load(std::memory_order_relaxed)) {
        Machine m = kDefaultMachine;
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            m.cus = v;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeNumberOfXccs, dev) == hipSuccess && v > 0)
            m.xcds = v;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeClockRate, dev) == hipSuccess && v > 0)
            m.clock = 1e3 * v;  // reported in kHz
        (void)hipGetLastError();
        if (m.cus % m.xcds != 0)
            m.xcds = 1;  // an odd partition: the walk then treats the GPU as one die
        g_machine[dev] = m;
        g_machine_known[dev].store(true, std::memory_order_release);
    }
    return g_machine[dev];
}

} // namespace nmspmm

extern "C" {

int nmspmm_version(void) { return 100; }

const char* nmspmm_status_string(int status)
{
    switch (status) {
    case NMSPMM_OK: return "ok";
    case NMSPMM_ERR_NULL_POINTER: return "null pointer";
    case NMSPMM_ERR_BAD_SHAPE: return "bad shape";
    case NMSPMM_ERR_BAD_PATTERN: return "unsupported sparsity pattern";
    case NMSPMM_ERR_WRONG_PATH: return "sparsity belongs to the other (low/high) entry point";
    case NMSPMM_ERR_BAD_SPLIT: return "bad split_k";
    case NMSPMM_ERR_WORKSPACE: return "workspace missing or too small";
    case NMSPMM_ERR_HIP: return "HIP runtime error";
    case NMSPMM_ERR_ALIGNMENT: return "pointer not 16-byte aligned";
    }
    return "unknown status";
}

const char* nmspmm_last_kernel(void) { return g_last_kernel; }

int nmspmm_pattern_from_sparsity(float sparsity, int* window, int* kept, int* is_high)
{
    if (!window || !kept || !is_high)
        return NMSPMM_ERR_NULL_POINTER;
    struct Row { float s; int window, kept, high; };
    static const Row table[] = {
        {0.0f, 32, 32, 0}, {0.5f, 32, 16, 0}, {0.625f, 32, 12, 0}, {0.75f, 64, 16, 1}, {0.875f, 64, 8, 1},
    };
    for (const Row& r : table) {
        if (std::fabs(sparsity - r.s) < 1e-6f) {
            *window = r.window;
            *kept = r.kept;
            *is_high = r.high;
            return NMSPMM_OK;
        }
    }
    return NMSPMM_ERR_BAD_PATTERN;
}

/* ---- preprocessing ------------------------------------------------------------------------- */

static int check_trans(const void* DT, int W, int N, int Q, const int* pN, const int* pM)
{
    if (!DT || !pN || !pM)
        return NMSPMM_ERR_NULL_POINTER;
    if (check_index_shape(W, Q) != NMSPMM_OK || N <= 0 || N % Q != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    if (*pN <= 0 || *pM <= 0 || *pN > *pM)
        return NMSPMM_ERR_BAD_PATTERN;
    if (W % (2 * *pN) != 0) /* an odd number of windows has no partner for the last one */
        return NMSPMM_ERR_BAD_SHAPE;
    return NMSPMM_OK;
}

int nmspmm_trans_index_device(int32_t* dDT, int W, int N, int Q, int* pruning_N, int* pruning_M, void* stream)
{
    const int st = check_trans(dDT, W, N, Q, pruning_N, pruning_M);
    if (st != NMSPMM_OK)
        return st;
    if (launch_trans_index(dDT, W, Q, *pruning_N, *pruning_M, (hipStream_t)stream) != hipSuccess)
        return NMSPMM_ERR_HIP;
    *pruning_N *= 2;
    *pruning_M *= 2;
    return NMSPMM_OK;
}

int nmspmm_trans_index_host(int32_t* DT, int W, int N, int Q, int* pruning_N, int* pruning_M)
{
    const int st = check_trans(DT, W, N, Q, pruning_N, pruning_M);
    if (st != NMSPMM_OK)
        return st;
    const size_t bytes = sizeof(int32_t) * (size_t)W * Q;
    const StagingLease d(&bytes, 1);
    if (!d.ok())
        return NMSPMM_ERR_HIP;
    if (hipMemcpy(d.part(0), DT, bytes, hipMemcpyHostToDevice) != hipSuccess)
        return NMSPMM_ERR_HIP;
    const int rc = nmspmm_trans_index_device((int32_t*)d.part(0), W, N, Q, pruning_N, pruning_M, nullptr);
    if (rc != NMSPMM_OK)
        return rc;
    if (hipMemcpy(DT, d.part(0), bytes, hipMemcpyDeviceToHost) != hipSuccess)
        return NMSPMM_ERR_HIP;
    return NMSPMM_OK;
}

static int check_reblock(const void* in, const void* out, int W, int Q, int Ns, int vec_len)
{
    if (!in || !out)
        return NMSPMM_ERR_NULL_POINTER;
    if (!valid_vec_len(vec_len))
        return NMSPMM_ERR_BAD_PATTERN;
    if (check_index_shape(W, Q) != NMSPMM_OK || Ns <= 0 || Ns % vec_len != 0 || Q % (Ns / vec_len) != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    return NMSPMM_OK;
}

int nmspmm_preprocess_low_device(const int32_t* dDT_in, int32_t* dDT_out, int W, int Q, int Ns, int vec_len,
                                 void* stream)
{
    const int st = check_reblock(dDT_in, dDT_out, W, Q, Ns, vec_len);
    if (st != NMSPMM_OK)
        return st;
    if (dDT_in == dDT_out)
        return NMSPMM_ERR_BAD_SHAPE;
    if (launch_reblock(dDT_in, dDT_out, W, Q, Ns / vec_len, 1, 0, 0, (hipStream_t)stream) != hipSuccess)
        return NMSPMM_ERR_HIP;
    return NMSPMM_OK;
}

int nmspmm_preprocess_low_host(int32_t* DT, int W, int Q, int Ns, int vec_len)
{
    const int st = check_reblock(DT, DT, W, Q, Ns, vec_len);
    if (st != NMSPMM_OK)
        return st;
    const size_t bytes = sizeof(int32_t) * (size_t)W * Q;
    const size_t sizes[2] = {bytes, bytes};
    const StagingLease d(sizes, 2);
    if (!d.ok())
        return NMSPMM_ERR_HIP;
    if (hipMemcpy(d.part(0), DT, bytes, hipMemcpyHostToDevice) != hipSuccess)
        return NMSPMM_ERR_HIP;
    const int rc =
        nmspmm_preprocess_low_device((const int32_t*)d.part(0), (int32_t*)d.part(1), W, Q, Ns, vec_len, nullptr);
    if (rc != NMSPMM_OK)
        return rc;
    if (hipMemcpy(DT, d.part(1), bytes, hipMemcpyDeviceToHost) != hipSuccess)
        return NMSPMM_ERR_HIP;
    return NMSPMM_OK;
}

size_t nmspmm_column_info_ints(int W, int pruning_N, int pruning_M, int N, int Ns)
{
    if (W <= 0 || pruning_N <= 0 || pruning_M <= 0 || N <= 0 || Ns <= 0 || W % pruning_N != 0 || N % Ns != 0)
        return 0;
    return (size_t)(N / Ns) * (size_t)(W / pruning_N) * (size_t)pruning_M;
}

static int check_high(const void* ci, const void* in, const void* out, int pM, int pN, int W, int Q, int N,
                      int Ns, int vec_len)
{
    if (!ci)
        return NMSPMM_ERR_NULL_POINTER;
    const int st = check_reblock(in, out, W, Q, Ns, vec_len);
    if (st != NMSPMM_OK)
        return st;
    if (pN <= 0 || pM <= 0 || pN > pM || pM > 1024)
        return NMSPMM_ERR_BAD_PATTERN;
    if (W % pN != 0 || N != Q * vec_len)
        return NMSPMM_ERR_BAD_SHAPE;
    return NMSPMM_OK;
}

int nmspmm_preprocess_high_device(int32_t* d_column_info, int pruning_M, int pruning_N, const int32_t* dDT_in,
                                  int32_t* dDT_out, int W, int Q, int N, int Ns, int vec_len, void* stream)
{
    const int st = check_high(d_column_info, dDT_in, dDT_out, pruning_M, pruning_N, W, Q, N, Ns, vec_len);
    if (st != NMSPMM_OK)
        return st;
    if (dDT_in == dDT_out)
        return NMSPMM_ERR_BAD_SHAPE;
    if (launch_preprocess_high(d_column_info, pruning_M, pruning_N, dDT_in, dDT_out, W, Q, Ns / vec_len, 1, 0, 0,
                               (hipStream_t)stream) != hipSuccess)
        return NMSPMM_ERR_HIP;
    return NMSPMM_OK;
}

int nmspmm_preprocess_high_host(int32_t* column_info, int pruning_M, int pruning_N, int32_t* DT, int W, int Q,
                                int N, int Ns, int vec_len)
{
    const int st = check_high(column_info, DT, DT, pruning_M, pruning_N, W, Q, N, Ns, vec_len);
    if (st != NMSPMM_OK)
        return st;
    const size_t bytes = sizeof(int32_t) * (size_t)W * Q;
    const size_t ci_bytes = sizeof(int32_t) * nmspmm_column_info_ints(W, pruning_N, pruning_M, N, Ns);
    const size_t sizes[3] = {bytes, bytes, ci_bytes};
    const StagingLease d(sizes, 3);
    if (!d.ok())
        return NMSPMM_ERR_HIP;
    if (hipMemcpy(d.part(0), DT, bytes, hipMemcpyHostToDevice) != hipSuccess)
        return NMSPMM_ERR_HIP;
    const int rc = nmspmm_preprocess_high_device((int32_t*)d.part(2), pruning_M, pruning_N, (const int32_t*)d.part(0),
                                                 (int32_t*)d.part(1), W, Q, N, Ns, vec_len, nullptr);
    if (rc != NMSPMM_OK)
        return rc;
    if (hipMemcpy(DT, d.part(1), bytes, hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(column_info, d.part(2), ci_bytes, hipMemcpyDeviceToHost) != hipSuccess)
        return NMSPMM_ERR_HIP;
    return NMSPMM_OK;
}

int nmspmm_preprocess_device(const int32_t* dDT_in, int n, int m, int W, int Q, int N, int Ns, int32_t* dD_out,
                             int32_t* d_column_info, int* window, int* kept, void* stream)
{
    if (!dDT_in || !dD_out || !window || !kept)
        return NMSPMM_ERR_NULL_POINTER;
    if (n <= 0 || m <= 0 || n > m)
        return NMSPMM_ERR_BAD_PATTERN;
    if (Q > 0 && N > 0 && N % Q == 0 && N / Q < 32) {
        // vectors of 4, 8 or 16 columns: the kernels take the window as generated, so the whole
        // preprocessing is the re-blocking
        const int vec_len = N / Q;
        if (!valid_vec_len(vec_len))
            return NMSPMM_ERR_BAD_PATTERN;
        const int st = check_reblock(dDT_in, dD_out, W, Q, Ns, vec_len);
        if (st != NMSPMM_OK)
            return st;
        if (dDT_in == dD_out || W % n != 0)
            return NMSPMM_ERR_BAD_SHAPE;
        if (launch_reblock(dDT_in, dD_out, W, Q, Ns / vec_len, n, m, 0, (hipStream_t)stream) != hipSuccess)
            return NMSPMM_ERR_HIP;
        *window = m;
        *kept = n;
        return NMSPMM_OK;
    }
    // the kernel geometry of the pattern's sparsity, reached by doubling the generated window
    int win = 0, kp = 0, high = 0;
    const int st0 = nmspmm_pattern_from_sparsity(1.0f - (float)n / (float)m, &win, &kp, &high);
    if (st0 != NMSPMM_OK)
        return st0;
    int times = 0;
    while ((m << times) < win)
        ++times;
    if ((m << times) != win || (n << times) != kp)
        return NMSPMM_ERR_BAD_PATTERN;
    const int st = check_reblock(dDT_in, dD_out, W, Q, Ns, 32);
    if (st != NMSPMM_OK)
        return st;
    if (dDT_in == dD_out || N != Q * 32 || W % kp != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    if (high && !d_column_info)
        return NMSPMM_ERR_NULL_POINTER;
    const hipError_t e = high ? launch_preprocess_high(d_column_info, win, kp, dDT_in, dD_out, W, Q, Ns / 32, n, m,
                                                       times, (hipStream_t)stream)
                              : launch_reblock(dDT_in, dD_out, W, Q, Ns / 32, n, m, times, (hipStream_t)stream);
    if (e != hipSuccess)
        return NMSPMM_ERR_HIP;
    *window = win;
    *kept = kp;
    return NMSPMM_OK;
}

/* ---- multiplication ------------------------------------------------------------------------ */

static int check_compress(const void* dense, const void* bt, const void* dt, int K, int N, int n, int m, int vec_len)
{
    if (!dense || !bt || !dt)
        return NMSPMM_ERR_NULL_POINTER;
    if (((uintptr_t)dense | (uintptr_t)bt) & 15u)
        return NMSPMM_ERR_ALIGNMENT;
    if (!compress_supported(m, vec_len) || n <= 0 || n >= m)
        return NMSPMM_ERR_BAD_PATTERN;
    // the kernels address a window of m rows through 32-bit byte offsets
    if (K <= 0 || N <= 0 || K % m != 0 || N % vec_len != 0 || (size_t)m * N * sizeof(float) > 0xffffffffull)
        return NMSPMM_ERR_BAD_SHAPE;
    return NMSPMM_OK;
}

int nmspmm_compress_device(const float* dB, int K, int N, int n, int m, int vec_len, float* dBT, int32_t* dDT,
                           void* stream)
{
    const int st = check_compress(dB, dBT, dDT, K, N, n, m, vec_len);
    if (st != NMSPMM_OK)
        return st;
    return launch_compress(dB, dBT, dDT, K, N, n, m, vec_len, (hipStream_t)stream) == hipSuccess ? NMSPMM_OK
                                                                                                   : NMSPMM_ERR_HIP;
}

int nmspmm_decompress_device(const float* dBT, const int32_t* dDT, int K, int N, int n, int m, int vec_len,
                             float* dB, void* stream)
{
    const int st = check_compress(dB, dBT, dDT, K, N, n, m, vec_len);
    if (st != NMSPMM_OK)
        return st;
    return launch_decompress(dBT, dDT, dB, K, N, n, m, vec_len, (hipStream_t)stream) == hipSuccess ? NMSPMM_OK
                                                                                                     : NMSPMM_ERR_HIP;
}

size_t nmspmm_workspace_bytes(int M, int N, int split_k)
{
    if (M <= 0 || N <= 0 || split_k <= 1)
        return 0;
    return sizeof(float) * slice_stride(M, N) * (size_t)split_k;
}

// lda: floats between consecutive dense rows of A; 0 lets the function choose (M, or M rounded up
// to 4 when `may_pad` allows it and that puts the shape on the matrix-core path) and reports it.
// a_rowmajor: A is row-major M x K with `lda` floats between rows; only the decode kernels take
// that, and kNotTaken comes back (nothing launched) when they do not take the shape.
constexpr int kNotTaken = -1000;
// Factor on model_decode_seconds when it is compared with model_tile_seconds (33 to 128 rows; see
// spmm_impl)
constexpr double kDecodeBias = 1.25;

static int spmm_impl(const float* A, const float* B, const int32_t* D, const int32_t* column_info, float* C, int M,
                     int N, int K, int W, int window, int kept, int vec_len, int Ns, int split_k, void* workspace,
                     size_t workspace_bytes, void* stream, int lda, bool dry_run, int* lda_out, bool a_rowmajor = false,
                     unsigned flags = 0, const int32_t* row_index = nullptr)
{
    if (flags & ~(unsigned)(NMSPMM_ACCUMULATE | NMSPMM_STREAM_B | NMSPMM_DECODE_SPLIT))
        return NMSPMM_ERR_BAD_SHAPE;
    if (!A || !B || !D || !C)
        return NMSPMM_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || W <= 0)
        return NMSPMM_ERR_BAD_SHAPE;
    if (window <= 0 || kept <= 0 || kept > window || !valid_vec_len(vec_len))
        return NMSPMM_ERR_BAD_PATTERN;
    if (Ns <= 0 || Ns % vec_len != 0 || N % Ns != 0 || W % kept != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    if ((long long)K * kept != (long long)W * window)
        return NMSPMM_ERR_BAD_SHAPE;
    if (split_k < 1 || split_k > W / kept)
        return NMSPMM_ERR_BAD_SPLIT;
    if (!aligned16(A) || !aligned16(B) || !aligned16(C))
        return NMSPMM_ERR_ALIGNMENT;
    if (split_k > 1) {
        if (!workspace || workspace_bytes < nmspmm_workspace_bytes(M, N, split_k) || !aligned16(workspace))
            return NMSPMM_ERR_WORKSPACE;
    }

    SpmmArgs a;
    a.A = A;
    a.B = B;
    a.D = D;
    a.cinfo = column_info;
    a.row_index = row_index;
    a.stream_b = (flags & NMSPMM_STREAM_B) != 0;
    a.decode_part = nullptr;
    a.decode_part_bytes = 0;
    a.decode_tickets = nullptr;
    a.decode_epoch = 0;
    a.decode_ticket_count = 0;
    a.C = C;
    a.partial = split_k > 1 ? (float*)workspace : nullptr;
    a.slice_stride = slice_stride(M, N);
    a.M = M;
    a.lda = lda > 0 ? lda : M;
    a.a_rowmajor = a_rowmajor;
    a.N = N;
    a.K = K;
    a.W = W;
    a.window = window;
    a.kept = kept;
    a.vec_len = vec_len;
    a.Ns = Ns;
    a.split_k = split_k;
    a.accumulate = (flags & NMSPMM_ACCUMULATE) != 0 && split_k > 1;
    a.stream = (hipStream_t)stream;

    if (lda == 0 && M > 32 && M % 4 != 0) {
        // a padded copy of A is only worth making if it reaches the matrix-core kernel
        a.lda = (M + 3) / 4 * 4;
        if (!mfma_supported(a) && !short_supported(a) && !gather_supported(a))
            a.lda = M;
    }
    if (lda_out)
        *lda_out = a.lda;
    if (dry_run)
        return NMSPMM_OK;

    if (a_rowmajor && !(M <= 32 && (skinny_supported(a) || decode_supported(a))))
        return kNotTaken;
    // A row count a little above a multiple of 128 (1 to 32 rows more): the tile kernel would spend a
    // whole layer of 128-row workgroups, mostly padding, on the last rows.  Where the models expect
    // it to be shorter, the rows up to the multiple go to the tile kernel and the last ones to the
    // kernels with one workgroup per vector, which read B once more at the rate of HBM.  The
    // comparison allows 3 us for what the two models both count.  Measured on 140 shapes (136 to 416
    // rows, 2048 to 11008 columns, four patterns) with the two parts launched by hand: the rule is
    // 0.8 % behind the better way on average where whole launches are 6.1 % behind (136 x 4096 x
    // 11008 at 2:4: 83.2 -> 67.4 us; on 2048 columns, where the last rows add no layer, the whole
    // launch stays).  With eight kept rows per window and fewer than 512 rows the two ways were
    // within 2 us of each other nearly everywhere and the models cannot tell them apart: whole
    // launches there (from 512 rows on the rule's choices were 1 to 10 % shorter on 15 of 17 shapes
    // and 1 % longer on two).  Every row of C is computed by one kernel, in its own order.
    const int last_rows = a_rowmajor || split_k != 1 || !mfma_supported(a) ? 0 : nmspmm_rows_apart(M, N, W, kept);
    if (last_rows > 0) {
        SpmmArgs tail = a;
        tail.M = last_rows;
        const bool tail_ok = (row_index && decode_supported(tail)) || skinny_supported(tail);
        const int head_rows = M - last_rows;
        if (tail_ok) {
            int st = spmm_impl(A, B, D, column_info, C, head_rows, N, K, W, window, kept, vec_len, Ns, 1, nullptr, 0,
                               stream, a.lda, false, nullptr, false, flags, row_index);
            if (st != NMSPMM_OK)
                return st;
            const char* const head_kernel = g_last_kernel;
            st = spmm_impl(A + head_rows, B, D, column_info, C + (size_t)head_rows * N, last_rows, N, K, W, window, kept,
                           vec_len, Ns, 1, nullptr, 0, stream, a.lda, false, nullptr, false, flags, row_index);
            g_last_kernel = head_kernel;  // the family that computed all rows but the last few
            return st;
        }
    }
    hipError_t e;
    // up to 32 rows the kernels with one workgroup per vector always win; up to 128 they compete
    // with the tile kernel at the caller's split.  The two models are compared with a bias: on 340
    // shapes of 33 to 128 rows (2048 to 28672 columns, reductions of 2048 to 11008, four patterns,
    // each kernel forced in turn, B re-read from the caches and, for 84 of them, streamed from HBM
    // too) the tile model is 10 to 12 % pessimistic at these row counts and the other 3 to 13 %
    // optimistic from 4096 columns on.  With the factor the choice is within 1 % of always taking
    // the faster kernel on average, without it 4 to 8 % behind (worst 54 %).  (Fitted before the tile
    // kernel's launches of at most one 64-row workgroup per CU got eight waves along K, which only
    // moved ties towards the tile kernel.)
    // (the models are only asked where they decide: 33 to 128 rows)
    const bool decode_wins = M > 32 && M <= 128 &&
                             kDecodeBias * model_decode_seconds(M, N, W / kept, kept) <
                                 model_tile_seconds(M, N, W / kept, kept, split_k);
    if (decode_supported(a) && (M <= 32 || decode_wins || !mfma_supported(a))) {
        // decode sizes with the row list: one launch, reduction inside the workgroup (or, on request,
        // across a few workgroups through the library's device-resident scratch)
        if (flags & NMSPMM_DECODE_SPLIT) {
            a.decode_part = (float*)noalloc_scratch();
            a.decode_tickets = decode_ticket_array();
            if (a.decode_part && a.decode_tickets) {
                a.decode_part_bytes = NMSPMM_NOALLOC_MAX_BYTES;
                a.decode_ticket_count = kDecodeTickets;
                a.decode_epoch = next_decode_epoch();
            } else {
                a.decode_part = nullptr;
                a.decode_tickets = nullptr;
            }
        }
        e = launch_decode(a);
        g_last_kernel = "decode";
        return e == hipSuccess ? NMSPMM_OK : NMSPMM_ERR_HIP;
    }
    if (skinny_supported(a) && (M <= 32 || decode_wins || !mfma_supported(a))) {
        // one launch, reduction inside the workgroup: split_k and the workspace are not needed
        e = launch_skinny(a);
        g_last_kernel = "skinny";
        return e == hipSuccess ? NMSPMM_OK : NMSPMM_ERR_HIP;
    }
    if (mfma_supported(a)) {
        e = launch_mfma(a);
        g_last_kernel = "mfma";
    } else if (gather_supported(a)) {
        // short vectors at densities up to one half: multiply the kept rows only
        e = launch_gather(a);
        g_last_kernel = "gather";
    } else if (short_supported(a)) {
        e = launch_short(a);
        g_last_kernel = "short";
    } else if (simt_supported(a)) {
        e = launch_simt(a);
        g_last_kernel = "simt";
    } else {
        return NMSPMM_ERR_BAD_PATTERN;
    }
    if (e != hipSuccess)
        return NMSPMM_ERR_HIP;
    if (split_k > 1) {
        e = launch_splitk_reduce(a.partial, C, (size_t)M * N, a.slice_stride, split_k, a.accumulate, a.stream);
        if (e != hipSuccess)
            return NMSPMM_ERR_HIP;
    }
    return NMSPMM_OK;
}

int nmspmm_transpose_device(const float* src, int rows, int cols, float* dst, void* stream)
{
    if (!src || !dst)
        return NMSPMM_ERR_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || src == dst || (rows + 63) / 64 > 65535)
        return NMSPMM_ERR_BAD_SHAPE;
    return launch_transpose(src, dst, rows, cols, rows, (hipStream_t)stream) == hipSuccess ? NMSPMM_OK
                                                                                            : NMSPMM_ERR_HIP;
}

// floats reserved at the head of the workspace for the column-major copy of a row-major A: K rows
// of M rounded up to 4
static size_t rowmajor_copy_floats(int M, int K) { return (size_t)K * ((size_t)(M + 3) / 4 * 4); }

size_t nmspmm_workspace_bytes_rowmajor(int M, int N, int K, int split_k)
{
    if (M <= 0 || N <= 0 || K <= 0 || split_k < 1)
        return 0;
    return sizeof(float) * rowmajor_copy_floats(M, K) + nmspmm_workspace_bytes(M, N, split_k);
}

int nmspmm_spmm_rowmajor_ex(const float* A_rowmajor, const float* B, const int32_t* D, const int32_t* column_info,
                            const int32_t* row_index, float* C, int M, int N, int K, int W, int window, int kept,
                            int vec_len, int Ns, int split_k, void* workspace, size_t workspace_bytes, unsigned flags,
                            void* stream)
{
    if (row_index && ((uintptr_t)row_index & 15u))
        return NMSPMM_ERR_ALIGNMENT;
    if (!A_rowmajor)
        return NMSPMM_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || (M + 63) / 64 > 65535)
        return NMSPMM_ERR_BAD_SHAPE;
    if (split_k < 1)
        return NMSPMM_ERR_BAD_SPLIT;
    if (!workspace || !aligned16(workspace) || workspace_bytes < nmspmm_workspace_bytes_rowmajor(M, N, K, split_k))
        return NMSPMM_ERR_WORKSPACE;
    float* const At = (float*)workspace;
    float* const slices = At + rowmajor_copy_floats(M, K);
    const size_t slice_bytes = workspace_bytes - sizeof(float) * rowmajor_copy_floats(M, K);
    // Up to 8 rows the decode kernel reads a row-major A in place: no copy, one launch.  (A lane
    // then fetches its operand from a cache line of its own row; measured against the copy, which
    // costs 2.5 to 4 us at these sizes: level up to 8 rows, 0.4 to 2 times slower from 16 on.)
    if (M <= 8 && aligned16(A_rowmajor)) {
        const int st = spmm_impl(A_rowmajor, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k,
                                 slices, slice_bytes, stream, K, false, nullptr, true, flags, row_index);
        if (st != kNotTaken)
            return st;
    }
    // check every argument and settle the row pitch of the copy before anything is launched
    int lda = M;
    const int st = spmm_impl(At, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k, slices,
                             slice_bytes, stream, 0, true, &lda, false, flags, row_index);
    if (st != NMSPMM_OK)
        return st;
    if (launch_transpose(A_rowmajor, At, M, K, lda, (hipStream_t)stream) != hipSuccess)
        return NMSPMM_ERR_HIP;
    return spmm_impl(At, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k, slices, slice_bytes,
                     stream, lda, false, nullptr, false, flags, row_index);
}

int nmspmm_spmm_rowmajor(const float* A_rowmajor, const float* B, const int32_t* D, const int32_t* column_info,
                         float* C, int M, int N, int K, int W, int window, int kept, int vec_len, int Ns,
                         int split_k, void* workspace, size_t workspace_bytes, void* stream)
{
    return nmspmm_spmm_rowmajor_ex(A_rowmajor, B, D, column_info, nullptr, C, M, N, K, W, window, kept, vec_len, Ns,
                                   split_k, workspace, workspace_bytes, 0, stream);
}

int nmspmm_spmm(const float* A, const float* B, const int32_t* D, const int32_t* column_info, float* C, int M,
                int N, int K, int W, int window, int kept, int vec_len, int Ns, int split_k, void* workspace,
                size_t workspace_bytes, void* stream)
{
    return spmm_impl(A, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k, workspace,
                     workspace_bytes, stream, M, false, nullptr);
}

int nmspmm_spmm_ex(const float* A, const float* B, const int32_t* D, const int32_t* column_info,
                   const int32_t* row_index, float* C, int M, int N, int K, int W, int window, int kept, int vec_len,
                   int Ns, int split_k, void* workspace, size_t workspace_bytes, unsigned flags, void* stream)
{
    if (row_index && ((uintptr_t)row_index & 15u))
        return NMSPMM_ERR_ALIGNMENT;
    return spmm_impl(A, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k, workspace,
                     workspace_bytes, stream, M, false, nullptr, false, flags, row_index);
}

size_t nmspmm_row_index_ints(int W, int N)
{
    if (W <= 0 || N <= 0 || N % 32 != 0)
        return 0;
    return (size_t)(N / 32) * (size_t)((W + 15) / 16) * 16;
}

int nmspmm_row_index_device(const int32_t* dD, const int32_t* d_column_info, int W, int N, int window, int kept,
                            int Ns, int32_t* d_row_index, void* stream)
{
    if (!dD || !d_row_index)
        return NMSPMM_ERR_NULL_POINTER;
    if (window <= 0 || kept <= 0 || kept > window)
        return NMSPMM_ERR_BAD_PATTERN;
    if (W <= 0 || N <= 0 || Ns <= 0 || Ns % 32 != 0 || N % Ns != 0 || W % kept != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    if ((long long)(W / kept) * window >= (1LL << 31) - 1)
        return NMSPMM_ERR_BAD_SHAPE;
    return launch_row_index(dD, d_column_info, d_row_index, W, N, window, kept, Ns, (hipStream_t)stream) == hipSuccess
               ? NMSPMM_OK
               : NMSPMM_ERR_HIP;
}

int nmspmm_spmm_noalloc(const float* A, const float* B, const int32_t* D, const int32_t* column_info, float* C,
                        int M, int N, int K, int W, int window, int kept, int vec_len, int Ns, int split_k,
                        void* stream)
{
    // every argument is checked before the scratch is looked up, so the error paths need no GPU
    // (the dry run only validates; C stands in for a workspace that is large enough and aligned)
    const int st = spmm_impl(A, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k,
                             split_k > 1 ? (void*)C : nullptr, (size_t)-1, stream, M, true, nullptr);
    if (st != NMSPMM_OK)
        return st;
    const size_t need = nmspmm_workspace_bytes(M, N, split_k);
    if (need > (size_t)NMSPMM_NOALLOC_MAX_BYTES)
        return NMSPMM_ERR_WORKSPACE;
    void* ws = nullptr;
    if (need > 0) {
        ws = noalloc_scratch();
        if (!ws)
            return NMSPMM_ERR_HIP;
    }
    return spmm_impl(A, B, D, column_info, C, M, N, K, W, window, kept, vec_len, Ns, split_k, ws, need, stream, M,
                     false, nullptr);
}

// Row lists attached to index buffers (nmspmm_row_index_attach): (device, address of D) -> list.
// The named launchers look their D up for decode-sized calls; the count lets every other call skip
// the lock.
static std::mutex g_attach_mutex;
static std::map<std::pair<int, const void*>, const int32_t*> g_attached;
static std::atomic<int> g_attached_count{0};

static const int32_t* attached_row_index(const int32_t* D)
{
    if (g_attached_count.load(std::memory_order_acquire) == 0)
        return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess)
        return nullptr;
    std::lock_guard<std::mutex> lock(g_attach_mutex);
    const auto it = g_attached.find({dev, D});
    return it == g_attached.end() ? nullptr : it->second;
}

int nmspmm_row_index_attach(const int32_t* dD, const int32_t* row_index)
{
    if (!dD)
        return NMSPMM_ERR_NULL_POINTER;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess)
        return NMSPMM_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_attach_mutex);
    if (row_index)
        g_attached[{dev, dD}] = row_index;
    else
        g_attached.erase({dev, dD});
    g_attached_count.store((int)g_attached.size(), std::memory_order_release);
    return NMSPMM_OK;
}

int nmspmm_row_index_detach(const int32_t* dD) { return nmspmm_row_index_attach(dD, nullptr); }

// `flags`: NMSPMM_ACCUMULATE for the reference launchers' replacements, whose SPLIT_K > 1 adds to C.
static int named_gemm(int want_high, int tile, const float* A, const float* B, const int32_t* D,
                      const int32_t* column_info, float* C, int M, int N, int K, int W, float sparsity,
                      int split_k, unsigned flags, void* stream)
{
    int window, kept, is_high;
    const int st = nmspmm_pattern_from_sparsity(sparsity, &window, &kept, &is_high);
    if (st != NMSPMM_OK)
        return st;
    if (is_high != want_high)
        return NMSPMM_ERR_WRONG_PATH;
    if (tile != 32 && tile != 64 && tile != 128)
        return NMSPMM_ERR_BAD_SHAPE;
    if (want_high && !column_info)
        return NMSPMM_ERR_NULL_POINTER;
    if (!A || !B || !D || !C)
        return NMSPMM_ERR_NULL_POINTER;
    if (M <= 0 || N <= 0 || W <= 0 || W % kept != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    if (split_k < 1 || split_k > W / kept)
        return NMSPMM_ERR_BAD_SPLIT;
    // Only a split reduction uses the library's per-device workspace: unsplit calls touch no shared
    // memory and may run on any number of streams.
    void* ws = nullptr;
    const size_t ws_bytes = nmspmm_workspace_bytes(M, N, split_k);
    if (ws_bytes > 0) {
        const int rc = cached_workspace(ws_bytes, &ws);
        if (rc != NMSPMM_OK)
            return rc;
    }
    // decode sizes: the row list the caller attached to this D, if any
    const int32_t* const row_index = M <= 128 ? attached_row_index(D) : nullptr;
    return nmspmm_spmm_ex(A, B, D, want_high ? column_info : nullptr, row_index, C, M, N, K, W, window, kept, 32, tile,
                          split_k, ws, ws_bytes, flags, stream);
}

int nmspmm_gemm_low_sparsity(int tile, const float* A, const float* B, const int32_t* D, float* C, int M, int N,
                             int K, int W, float sparsity, int split_k, void* stream)
{
    return named_gemm(0, tile, A, B, D, nullptr, C, M, N, K, W, sparsity, split_k, NMSPMM_ACCUMULATE, stream);
}

int nmspmm_gemm_high_sparsity(int tile, const float* A, const float* B, const int32_t* D,
                              const int32_t* column_info, float* C, int M, int N, int K, int W, float sparsity,
                              int split_k, void* stream)
{
    return named_gemm(1, tile, A, B, D, column_info, C, M, N, K, W, sparsity, split_k, NMSPMM_ACCUMULATE, stream);
}

int nmspmm_suggest_split_k(int M, int N, int W, int kept)
{
    if (M <= 0 || N <= 0 || W <= 0 || kept <= 0 || W % kept != 0)
        return 0;
    if (M <= 32)
        return 1;  // the decode kernel reduces inside its workgroups
    // The split with the smallest modelled time of the tile kernel (model_tile_seconds); a finer
    // split has to win by 5 %.  Fitted to sweeps of M in 48..4096, N and K in 512..14336 at 2:4,
    // 3:8, 2:8 and 1:8 on one MI355X: the choice is within 1 % of the best split on average, where
    // never splitting loses 32 %.  Up to 128 rows the one-launch decode kernel is the alternative;
    // where its model is faster no split is needed.
    const int nwin = W / kept;
    int best = 1;
    double best_t = 0.0;
    for (int split = 1; split <= 16 && split <= nwin; split *= 2) {
        const double t = model_tile_seconds(M, N, nwin, kept, split);
        if (split == 1 || t < 0.95 * best_t) {
            best = split;
            best_t = t;
        }
    }
    if (M <= 128 && kDecodeBias * model_decode_seconds(M, N, nwin, kept) < best_t)  // the dispatcher's comparison
        return 1;
    return best;
}

int nmspmm_waves_along_k_rows(int M, int N, int W, int kept)
{
    if (M <= 0 || N <= 0 || W <= 0 || kept <= 0 || W % kept != 0)
        return 0;
    return inner_split_pays(M, N, W / kept, kept) ? plan_inner(M, N, W / kept, kept).rows : 0;
}

int nmspmm_rows_apart(int M, int N, int W, int kept)
{
    if (M <= 128 || N <= 0 || W <= 0 || kept <= 0 || W % kept != 0)
        return 0;
    if (kept < 12 && M < 512)  // eight kept rows per window: the models only tell the two ways apart from 512 rows on
        return 0;
    const int last_rows = M % 128, nwin = W / kept;
    if (last_rows < 1 || last_rows > 32)
        return 0;
    return model_tile_seconds(M - last_rows, N, nwin, kept, 1) + model_decode_seconds(last_rows, N, nwin, kept) - 3e-6 <
                   model_tile_seconds(M, N, nwin, kept, 1)
               ? last_rows
               : 0;
}

int nmspmm_waves_along_k_count(int M, int N, int W, int kept)
{
    if (nmspmm_waves_along_k_rows(M, N, W, kept) == 0)
        return 0;
    return plan_inner(M, N, W / kept, kept).waves;
}

int nmspmm_device_figures(int* compute_units, int* dies, double* clock_hz)
{
    const Machine& m = machine();
    if (compute_units)
        *compute_units = m.cus;
    if (dies)
        *dies = m.xcds;
    if (clock_hz)
        *clock_hz = m.clock;
    return NMSPMM_OK;
}

int nmspmm_tile_wave_rows(int M, int N, int W, int kept, int Ns, int split_k)
{
    if (M <= 0 || N <= 0 || W <= 0 || kept <= 0 || W % kept != 0 || split_k < 1 || (Ns != 32 && Ns != 64 && Ns != 128))
        return 0;
    const int nwin = W / kept;
    if (split_k == 1 && nwin >= 4 && inner_split_pays(M, N, nwin, kept))
        return 0;  // the launch with waves along K: nmspmm_waves_along_k_rows() describes it
    const int blocks = choose_wave_blocks(M, N, nwin, kept, split_k);
    if (blocks == 4 && Ns == 128 && short_waves_pay(M))
        return 64;
    return 32 * blocks;
}

int nmspmm_tile_wave_sets(int M, int N, int W, int kept, int Ns, int split_k)
{
    const int rows = nmspmm_tile_wave_rows(M, N, W, kept, Ns, split_k);
    if (rows == 0)
        return 0;
    if (rows != 256 || split_k != 1)
        return 1;
    const int wr = 128 / Ns;  // waves along M: a workgroup is 256 * wr rows by Ns columns
    const long long tiles = (long long)((M + 256 * wr - 1) / (256 * wr)) * (N / Ns);
    const TailPlan t = plan_tail(M, N, W / kept, kept, wr);
    if (t.separate && t.blocks == 8)
        return 1;  // leftover tiles in a launch of their own: no launch is the whole problem
    return wave_sets_pay(tiles, W / kept, kept) ? 2 : 1;
}

int nmspmm_gemm_auto(const float* A, const float* B, const int32_t* D, const int32_t* column_info, float* C,
                     int M, int N, int K, int W, float sparsity, void* stream)
{
    int window, kept, is_high;
    const int st = nmspmm_pattern_from_sparsity(sparsity, &window, &kept, &is_high);
    if (st != NMSPMM_OK)
        return st;
    if (W <= 0 || W % kept != 0)
        return NMSPMM_ERR_BAD_SHAPE;
    const int split_k = nmspmm_suggest_split_k(M, N, W, kept);
    if (split_k < 1)
        return NMSPMM_ERR_BAD_SHAPE;
    return named_gemm(is_high, NMSPMM_TILE_HUGE, A, B, D, column_info, C, M, N, K, W, sparsity, split_k, 0, stream);
}

int nmspmm_release(void)
{
    {
        std::lock_guard<std::mutex> attach_lock(g_attach_mutex);
        g_attached.clear();
        g_attached_count.store(0, std::memory_order_release);
    }
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    int rc = NMSPMM_OK;
    int prev = 0;
    const bool have_dev = hipGetDevice(&prev) == hipSuccess;
    for (int d = 0; d < kMaxDevices; ++d) {
        Workspace& ws = g_workspace[d];
        if (!ws.ptr && ws.retired.empty())
            continue;
        // hipFree waits for the work enqueued on the device before it releases the memory
        if (hipSetDevice(d) != hipSuccess)
            rc = NMSPMM_ERR_HIP;
        if (ws.ptr && hipFree(ws.ptr) != hipSuccess)
            rc = NMSPMM_ERR_HIP;
        for (void* old : ws.retired)
            if (hipFree(old) != hipSuccess)
                rc = NMSPMM_ERR_HIP;
        ws.retired.clear();
        ws.ptr = nullptr;
        ws.bytes = 0;
    }
    {
        std::lock_guard<std::mutex> staging_lock(g_staging_mutex);
        for (int d = 0; d < kMaxDevices; ++d) {
            Staging& st = g_staging[d];
            if (!st.ptr)
                continue;
            if (hipSetDevice(d) != hipSuccess || hipFree(st.ptr) != hipSuccess)
                rc = NMSPMM_ERR_HIP;
            st.ptr = nullptr;
            st.bytes = 0;
        }
    }
    if (have_dev)
        (void)hipSetDevice(prev);
    return rc;
}

} // extern "C"
