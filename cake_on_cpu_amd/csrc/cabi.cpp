// cabi.cpp -- the extern "C" boundary (include/cake_hip.h): argument checks,
// host/device operand staging, workspace ownership, timing, kernel dispatch.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <chrono>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "blockdims.hpp"
#include "cake_hip.h"
#include "kernels.hpp"
#include "planner.hpp"

namespace {

using namespace cake;

thread_local std::string g_last_error;
thread_local double g_family_seconds[5] = {0, 0, 0, 0, 0};
thread_local int g_last_conv_route = CAKE_HIP_CONV_NONE;

int fail(int status, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return status;
}

#define HIP_TRY(expr)                                                                         \
    do {                                                                                      \
        hipError_t e_ = (expr);                                                               \
        if (e_ != hipSuccess)                                                                 \
            return fail(CAKE_HIP_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));     \
    } while (0)

// Grow-only device buffer.  A workspace that kernels of device-operand calls use (`keep_old`) is
// not freed when it grows: a caller may have captured earlier launches in a HIP graph, which
// holds the old address, so the outgrown allocation is kept until shutdown.  Such a buffer asks
// for at least twice its size, which bounds everything kept to the size of the live one (old
// blocks + live block < 2 x live block, i.e. at most 4 x the largest request while the doubling
// succeeds).  When memory does not allow that it falls back in steps: the request with a little
// slack, then the bare request, and as the last resort it waits for the device, gives the
// outgrown blocks and the present one back and asks again -- graphs captured before that point
// then hold addresses that are gone and must be captured anew (the call still succeeds whenever
// the request itself fits).  Staging copies of host operands are only touched by synchronous
// calls and are freed at once.
struct DeviceBuffer {
    void* ptr = nullptr;
    size_t cap = 0;
    bool keep_old = false;
    std::vector<void*> outgrown;
    static void* try_alloc(size_t bytes)
    {
        void* fresh = nullptr;
        if (hipMalloc(&fresh, bytes) == hipSuccess) return fresh;
        (void)hipGetLastError();
        return nullptr;
    }
    int reserve(size_t bytes)
    {
        if (bytes <= cap) return CAKE_HIP_OK;
        const size_t slack = bytes + (bytes >> 3) + 256;
        if (!keep_old && ptr) {
            (void)hipFree(ptr);
            ptr = nullptr;
            cap = 0;
        }
        size_t want = keep_old && slack < 2 * cap ? 2 * cap : slack;
        void* fresh = try_alloc(want);
        if (!fresh && want > slack) fresh = try_alloc(want = slack);
        if (!fresh) fresh = try_alloc(want = bytes + 256);
        if (!fresh && (ptr || !outgrown.empty())) {
            (void)hipDeviceSynchronize();   // nothing in flight may still use the blocks given back
            for (void* q : outgrown) (void)hipFree(q);
            outgrown.clear();
            if (ptr) (void)hipFree(ptr);
            ptr = nullptr;
            cap = 0;
            fresh = try_alloc(want = slack);
            if (!fresh) fresh = try_alloc(want = bytes + 256);
        }
        if (!fresh) return fail(CAKE_HIP_ERR_ALLOC, "device allocation of %zu bytes failed", bytes + 256);
        if (ptr) outgrown.push_back(ptr);
        ptr = fresh;
        cap = want;
        return CAKE_HIP_OK;
    }
    void release()
    {
        if (ptr) (void)hipFree(ptr);
        for (void* q : outgrown) (void)hipFree(q);
        outgrown.clear();
        ptr = nullptr;
        cap = 0;
    }
};

enum { STAGE_SLOTS = 6 };

// Everything a compute call needs besides its operands: workspaces, events, the pinned buffers
// and streams of host-operand transfers.  One default context exists per process (it is what
// cake_hip_init sets up); cake_hip_ctx_create makes further ones.  A context has a mutex of its
// own, so calls on different contexts run side by side, on different streams; calls on one
// context take turns because they share its workspaces.
struct Context {
    std::recursive_mutex mutex;        // one compute call at a time per context (an entry point may call another)
    std::atomic<bool> ready{false};
    int device = 0;
    cake_hip_device_t info{};
    DeviceModel model;
    DeviceBuffer stage[STAGE_SLOTS];  // device copies of host operands
    DeviceBuffer splitk, gemv, conv, conv_taps, conv_filters, tables, unpacked, linear, turned;
    hipStream_t own_stream = nullptr;   // what a NULL stream argument means on this context (default context: the null stream)
    hipEvent_t ev[2] = {nullptr, nullptr};
    hipEvent_t fam[2] = {nullptr, nullptr};
    std::vector<hipEvent_t> fam_pool;   // event pairs of the kernel families of one timed call, created on demand
    // host <-> device transfers of large host operands: two pinned buffers, a stream, an event each
    // (buffers 0, 1 and copy_stream: towards the device; 2, 3 and copy_back_stream: back, used
    // only when both directions run at once)
    void* pinned[4] = {nullptr, nullptr, nullptr, nullptr};
    hipStream_t copy_stream = nullptr, copy_back_stream = nullptr;
    hipEvent_t copy_done[2] = {nullptr, nullptr};
    // cake_hip_sgemm_noalloc in progress (set under `mutex`): partial sums and the turned operand
    // are carved from the file-scope array, `noalloc_used` bytes of it so far
    bool noalloc_call = false;
    size_t noalloc_used = 0;

    DeviceBuffer* compute_buffers[9] = {&splitk, &gemv, &conv, &conv_taps, &conv_filters, &tables, &unpacked, &linear, &turned};
    int create_events()
    {
        for (hipEvent_t* e : {&ev[0], &ev[1], &fam[0], &fam[1]})
            if (!*e) HIP_TRY(hipEventCreate(e));
        for (DeviceBuffer* b : compute_buffers) b->keep_old = true;
        return CAKE_HIP_OK;
    }
    void release_all()
    {
        for (DeviceBuffer& b : stage) b.release();
        for (DeviceBuffer* b : compute_buffers) b->release();
        for (hipEvent_t e : fam_pool) (void)hipEventDestroy(e);
        fam_pool.clear();
        for (hipEvent_t* e : {&ev[0], &ev[1], &fam[0], &fam[1], &copy_done[0], &copy_done[1]}) {
            if (*e) (void)hipEventDestroy(*e);
            *e = nullptr;
        }
        for (void*& p : pinned) {
            if (p) (void)hipHostFree(p);
            p = nullptr;
        }
        for (hipStream_t* cs : {&copy_stream, &copy_back_stream, &own_stream}) {
            if (*cs) (void)hipStreamDestroy(*cs);
            *cs = nullptr;
        }
    }
};

Context g_default_ctx;
thread_local Context* t_current_ctx = nullptr;   // set by cake_hip_ctx_set_current; nullptr: the default context
std::mutex g_ctx_registry_mutex;
std::vector<Context*> g_created_ctx;             // contexts from cake_hip_ctx_create that are still alive

inline Context& cur() { return t_current_ctx ? *t_current_ctx : g_default_ctx; }

// the stream argument of an entry point: NULL means the current context's own stream
inline hipStream_t pick_stream(void* stream_)
{
    return stream_ ? static_cast<hipStream_t>(stream_) : cur().own_stream;
}

// Partial sums (K slices of split-K, tail-split and streaming products, slices of the
// matrix-vector kernels) of cake_hip_sgemm_noalloc: a file-scope array instead of a buffer from
// hipMalloc.  The name is a host-side handle, not a device address; cake_hip_init asks the runtime
// for the address on each device it is called for and the kernels only ever get that pointer.
// Every context on a device shares the device's one array.
constexpr size_t NOALLOC_SCRATCH_BYTES = 64u << 20;
static __device__ __align__(256) unsigned char noalloc_scratch[NOALLOC_SCRATCH_BYTES];
enum { MAX_DEVICES = 64 };
unsigned char* g_noalloc_ptr[MAX_DEVICES] = {nullptr};

// Scratch memory of the current call: `buf` (grown when needed), or the next piece of the
// file-scope array during cake_hip_sgemm_noalloc, which never grows.
int scratch_space(DeviceBuffer& buf, size_t bytes, float** out)
{
    Context& c = cur();
    if (c.noalloc_call) {
        const size_t at = (c.noalloc_used + 255) & ~(size_t)255;
        if (bytes > NOALLOC_SCRATCH_BYTES || at + bytes > NOALLOC_SCRATCH_BYTES)
            return fail(CAKE_HIP_ERR_RANGE, "this product needs %zu bytes of partial sums; cake_hip_sgemm_noalloc has %zu",
                        at + bytes, (size_t)NOALLOC_SCRATCH_BYTES);
        *out = reinterpret_cast<float*>(g_noalloc_ptr[c.device] + at);
        c.noalloc_used = at + bytes;
        return CAKE_HIP_OK;
    }
    int st = buf.reserve(bytes);
    if (st) return st;
    *out = static_cast<float*>(buf.ptr);
    return CAKE_HIP_OK;
}

int ensure_init()
{
    if (cur().ready) return CAKE_HIP_OK;
    if (&cur() != &g_default_ctx) return fail(CAKE_HIP_ERR_ARG, "the current context has been destroyed");
    return cake_hip_init(0);
}

bool is_device_pointer(const void* p)
{
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();  // plain host memory is reported as an error
        return false;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged;
}

// An operand as the kernels see it.  Host memory is mirrored in a staging slot.
struct Operand {
    float* dev = nullptr;
    float* host = nullptr;  // non-null when staged
    size_t bytes = 0;
};

// Transfers between a caller's (pageable) host memory and the device.  hipMemcpy on pageable
// memory moves 17 (to the host) to 29 GB/s (to the device) on this platform, pinned memory 53 GB/s
// either way.  Large operands therefore travel in chunks through two pinned buffers: worker
// threads copy between the caller's memory and one buffer while the DMA engine moves the other.
constexpr size_t PIN_CHUNK = 32u << 20;
constexpr size_t PIN_THRESHOLD = 8u << 20;   // below this a plain hipMemcpy is as fast
constexpr int PIN_THREADS = 8;

static int pinned_ready()
{
    for (int i = 0; i < 2; ++i) {
        if (!cur().pinned[i]) HIP_TRY(hipHostMalloc(&cur().pinned[i], PIN_CHUNK, hipHostMallocDefault));
        if (!cur().copy_done[i]) HIP_TRY(hipEventCreateWithFlags(&cur().copy_done[i], hipEventDisableTiming));
    }
    if (!cur().copy_stream) HIP_TRY(hipStreamCreateWithFlags(&cur().copy_stream, hipStreamNonBlocking));
    return CAKE_HIP_OK;
}

static int pinned_both_ways_ready()
{
    int st = pinned_ready();
    if (st) return st;
    for (int i = 2; i < 4; ++i)
        if (!cur().pinned[i]) HIP_TRY(hipHostMalloc(&cur().pinned[i], PIN_CHUNK, hipHostMallocDefault));
    if (!cur().copy_back_stream) HIP_TRY(hipStreamCreateWithFlags(&cur().copy_back_stream, hipStreamNonBlocking));
    return CAKE_HIP_OK;
}

static void parallel_memcpy(void* dst, const void* src, size_t bytes)
{
    const size_t piece = ((bytes + PIN_THREADS - 1) / PIN_THREADS + 4095) & ~(size_t)4095;
    std::vector<std::thread> workers;
    for (size_t off = piece; off < bytes; off += piece)
        workers.emplace_back([=] { memcpy(static_cast<char*>(dst) + off, static_cast<const char*>(src) + off,
                                          bytes - off < piece ? bytes - off : piece); });
    memcpy(dst, src, bytes < piece ? bytes : piece);
    for (std::thread& t : workers) t.join();
}

static int host_to_device(void* dev, const void* host, size_t bytes)
{
    if (bytes < PIN_THRESHOLD) {
        HIP_TRY(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice));
        return CAKE_HIP_OK;
    }
    int st = pinned_ready();
    if (st) return st;
    int i = 0;
    for (size_t off = 0; off < bytes; off += PIN_CHUNK, ++i) {
        const size_t n = bytes - off < PIN_CHUNK ? bytes - off : PIN_CHUNK;
        const int b = i & 1;
        if (i >= 2) HIP_TRY(hipEventSynchronize(cur().copy_done[b]));   // the buffer's last transfer is over
        parallel_memcpy(cur().pinned[b], static_cast<const char*>(host) + off, n);
        HIP_TRY(hipMemcpyAsync(static_cast<char*>(dev) + off, cur().pinned[b], n, hipMemcpyHostToDevice, cur().copy_stream));
        HIP_TRY(hipEventRecord(cur().copy_done[b], cur().copy_stream));
    }
    HIP_TRY(hipStreamSynchronize(cur().copy_stream));
    return CAKE_HIP_OK;
}

static int device_to_host(void* host, const void* dev, size_t bytes)
{
    if (bytes < PIN_THRESHOLD) {
        HIP_TRY(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
        return CAKE_HIP_OK;
    }
    int st = pinned_ready();
    if (st) return st;
    const size_t chunks = (bytes + PIN_CHUNK - 1) / PIN_CHUNK;
    auto chunk_bytes = [&](size_t c) { return bytes - c * PIN_CHUNK < PIN_CHUNK ? bytes - c * PIN_CHUNK : PIN_CHUNK; };
    auto issue = [&](size_t c) -> hipError_t {
        const int b = (int)(c & 1);
        hipError_t e = hipMemcpyAsync(cur().pinned[b], static_cast<const char*>(dev) + c * PIN_CHUNK, chunk_bytes(c),
                                      hipMemcpyDeviceToHost, cur().copy_stream);
        return e != hipSuccess ? e : hipEventRecord(cur().copy_done[b], cur().copy_stream);
    };
    HIP_TRY(issue(0));
    for (size_t c = 0; c < chunks; ++c) {
        // the other buffer was emptied in the previous round: fill it while this one is copied out
        if (c + 1 < chunks) HIP_TRY(issue(c + 1));
        HIP_TRY(hipEventSynchronize(cur().copy_done[c & 1]));
        parallel_memcpy(static_cast<char*>(host) + c * PIN_CHUNK, cur().pinned[c & 1], chunk_bytes(c));
    }
    return CAKE_HIP_OK;
}

int stage_in(const float* p, size_t bytes, int slot, bool copy, Operand* op)
{
    op->bytes = bytes;
    if (bytes == 0 || is_device_pointer(p)) {
        op->dev = const_cast<float*>(p);
        op->host = nullptr;
        return CAKE_HIP_OK;
    }
    int st = cur().stage[slot].reserve(bytes);
    if (st) return st;
    op->dev = static_cast<float*>(cur().stage[slot].ptr);
    op->host = const_cast<float*>(p);
    if (copy) {
        // an earlier call may have left kernels in flight that still read this slot (device
        // outputs make a call asynchronous); hipMemcpy alone does not wait for non-blocking streams
        HIP_TRY(hipDeviceSynchronize());
        if ((st = host_to_device(op->dev, p, bytes))) return st;
    }
    return CAKE_HIP_OK;
}

int stage_out(const Operand& op, hipStream_t stream)
{
    if (!op.host) return CAKE_HIP_OK;
    HIP_TRY(hipStreamSynchronize(stream));
    return device_to_host(op.host, op.dev, op.bytes);
}

// Event bracket for `seconds`.
struct Timer {
    hipStream_t stream;
    double* out;
    bool on;
    int pairs = 0;              // event pairs of cur().fam_pool in use by this call
    int family_of[32];
    Timer(hipStream_t s, double* o) : stream(s), out(o), on(o != nullptr) {}
    int start()
    {
        for (double& f : g_family_seconds) f = 0;
        if (on) HIP_TRY(hipEventRecord(cur().ev[0], stream));
        return CAKE_HIP_OK;
    }
    int stop()
    {
        if (!on) return CAKE_HIP_OK;
        HIP_TRY(hipEventRecord(cur().ev[1], stream));
        HIP_TRY(hipEventSynchronize(cur().ev[1]));
        float ms = 0;
        HIP_TRY(hipEventElapsedTime(&ms, cur().ev[0], cur().ev[1]));
        *out = ms * 1e-3;
        // the families' events were recorded before ev[1] on the same stream: all of them are over
        for (int i = 0; i < pairs; ++i) {
            HIP_TRY(hipEventElapsedTime(&ms, cur().fam_pool[2 * i], cur().fam_pool[2 * i + 1]));
            g_family_seconds[family_of[i]] += ms * 1e-3;
        }
        pairs = 0;
        return CAKE_HIP_OK;
    }
    // Time one kernel family when timing is on.  The events are only read in stop(): waiting for
    // each family where it is launched would put a trip to the host between the kernels of a call
    // (the packed product of 4096^3, five launches: 1.18 ms per call with those waits, 1.09 without).
    template <class F>
    int family(int which, F&& launch)
    {
        const bool pooled = on && pairs < 32;
        if (pooled) {
            while ((int)cur().fam_pool.size() < 2 * pairs + 2) {
                hipEvent_t e = nullptr;
                HIP_TRY(hipEventCreate(&e));
                cur().fam_pool.push_back(e);
            }
            HIP_TRY(hipEventRecord(cur().fam_pool[2 * pairs], stream));
        } else if (on) {
            HIP_TRY(hipEventRecord(cur().fam[0], stream));
        }
        hipError_t e = launch();
        if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
        if (pooled) {
            HIP_TRY(hipEventRecord(cur().fam_pool[2 * pairs + 1], stream));
            family_of[pairs++] = which;
        } else if (on) {   // more families than the pool holds: wait for this one here
            HIP_TRY(hipEventRecord(cur().fam[1], stream));
            HIP_TRY(hipEventSynchronize(cur().fam[1]));
            float ms = 0;
            HIP_TRY(hipEventElapsedTime(&ms, cur().fam[0], cur().fam[1]));
            g_family_seconds[which] += ms * 1e-3;
        }
        return CAKE_HIP_OK;
    }
};

bool fits_int(double elems) { return elems < 2147483647.0; }


// The 16-byte loaders address a macro-tile with 32-bit byte offsets from its
// origin: 256 rows of A (stride K) and 32 rows of B (stride N) must stay below 2^31.
bool vec4_loadable(const float* A, const float* B, int K, int N)
{
    // the 16-byte buffer loads need 4-byte alignment only; what limits them is the 32-bit byte
    // offset inside a tile (up to 256 rows of A, 64 rows of B)
    (void)A; (void)B;
    return (double)K * 256 * 4 < 2147483648.0 && (double)N * 64 * 4 < 2147483648.0;
}

PackGeom make_geom(int M, int N, int K, int p, const cake_hip_blk_dims_t* d,
                   const cake_hip_cpu_cntx_t* cx, int sched)
{
    PackGeom g;
    g.d = *d;
    g.M = M; g.N = N; g.K = K; g.p = p;
    g.mr = cx->mr; g.nr = cx->nr;
    g.sch = sched;
    return g;
}

int check_geom(const cake_hip_blk_dims_t* d, const cake_hip_cpu_cntx_t* cx, int p, int sched)
{
    if (!d || !cx) return fail(CAKE_HIP_ERR_ARG, "block dims / cntx is NULL");
    if (p <= 0 || cx->mr <= 0 || cx->nr <= 0 || d->m_c <= 0 || d->k_c <= 0 || d->n_c <= 0)
        return fail(CAKE_HIP_ERR_ARG, "block dims are not initialised (p=%d mr=%d nr=%d m_c=%d k_c=%d n_c=%d)",
                    p, cx->mr, cx->nr, d->m_c, d->k_c, d->n_c);
    if (sched < CAKE_HIP_KMN || sched > CAKE_HIP_NKM) return fail(CAKE_HIP_ERR_ARG, "unknown schedule %d", sched);
    return CAKE_HIP_OK;
}

// Device index tables for one packed operand, carved from cur().tables at `at`.
int build_tables(int which, const PackGeom& g, size_t* at, IndexTables* out, hipStream_t stream)
{
    const int Mp = padded_rows(g), Np = padded_cols(g);
    const size_t nrows = (which == 1) ? g.K : Mp;
    const size_t ncols = (which == 0) ? g.K : Np;
    int4* base = reinterpret_cast<int4*>(static_cast<char*>(cur().tables.ptr) + *at);
    out->row = base;
    out->col = base + nrows;
    *at += (nrows + ncols) * sizeof(int4);
    hipError_t e = launch_build_index_tables(which, g, base, base + nrows, stream);
    if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "index table launch failed: %s", hipGetErrorString(e));
    return CAKE_HIP_OK;
}

size_t tables_bytes(int which, const PackGeom& g)
{
    const size_t nrows = (which == 1) ? g.K : padded_rows(g);
    const size_t ncols = (which == 0) ? g.K : padded_cols(g);
    return (nrows + ncols) * sizeof(int4);
}

// The GEMM proper on device operands.
int run_gemm(const float* A, const float* B, float* C, int M, int N, int K, int lda, int ldb, int ldc,
             int sched, int accumulate, const int* tile_override, int a_mode, int b_mode,
             hipStream_t stream, Timer& timer,
             const ConvGeom* conv = nullptr, const float* col_bias = nullptr,
             const TunedChoice* choice = nullptr)
{
    const bool vec = a_mode == LOAD_VEC4 && (b_mode == LOAD_VEC4 || b_mode == LOAD_VEC4_NCHW);
    const bool vec_plan = vec || (a_mode == LOAD_VEC4 && b_mode == LOAD_VEC4_T);  // planned (and tuned) alike
    // Products with a few rows or columns have streaming kernels of their own; a macro-tile is
    // only used for them on request or when the tuner measured one to be faster.
    const bool streaming_ok = vec && !conv && !choice && !tile_override && !tune_lookup(M, N, K, true, nullptr);
    if (streaming_ok && fewrows_applies(M, N, K, lda, ldb)) {
        // a few rows of A against a wide B: bound by reading B, served by the streaming kernel
        const int slices = fewrows_slices(M, N, K, cur().model.cus);
        float* partial = nullptr;
        if (slices > 1) {
            int st2 = scratch_space(cur().splitk, (size_t)slices * M * N * sizeof(float), &partial);
            if (st2) return st2;
        }
        return timer.family(0, [&] {
            return launch_sgemm_fewrows(A, B, C, partial, M, N, K, lda, ldb, ldc, accumulate, col_bias,
                                        cur().model.cus, stream);
        });
    }
    if (streaming_ok && fewrows_nt_applies(N, M, K, ldb, lda, true)) {
        // a tall A against a few columns of B: the same with A streamed along its rows.  Up to 16
        // columns of B (K x N, small next to A) are turned into N rows of K first where
        // fewrows_nt_turn_pays says so.
        const bool turn = ldb == N && K <= 64 * 65535 &&   // (what the transpose kernel's grid takes)
                          fewrows_nt_turn_pays(N, M, K, lda, cur().model.cus) && fewrows_nt_applies(N, M, K, K, lda, false);
        const float* Bx = B;
        if (turn) {
            float* bt = nullptr;
            int st2 = scratch_space(cur().turned, (size_t)K * N * sizeof(float), &bt);
            if (st2) return st2;
            st2 = timer.family(4, [&] { return launch_transpose(B, bt, K, N, stream); });
            if (st2) return st2;
            Bx = bt;
        }
        const int slices = fewrows_nt_slices(N, M, K, lda, !turn, cur().model.cus);
        float* partial = nullptr;
        if (slices > 1) {
            int st2 = scratch_space(cur().splitk, (size_t)slices * M * N * sizeof(float), &partial);
            if (st2) return st2;
        }
        return timer.family(0, [&] {
            return launch_sgemm_fewrows_nt(Bx, A, C, partial, N, M, K, turn ? K : ldb, lda, ldc, !turn, true, accumulate,
                                           col_bias, cur().model.cus, stream);
        });
    }
    // A short K under many tiles of C: workgroups that walk over tiles, the next tile's operands in flight
    // (plain operands only: with a convolution's gathered B the integer divisions that place a
    // tile's columns in the image, paid per tile instead of once per workgroup, cost more than
    // the overlap gives -- 1 x 1, 64 -> 256 channels on 56 x 56: 56 us against 50 us)
    // (beyond 64 k only where C is overwritten without a bias: that kernel has no other epilogue)
    const bool shortk_ok = vec && !conv && !choice && !tile_override && !tune_lookup(M, N, K, vec_plan, nullptr) &&
                           shortk_applies(M, N, K, cur().model.cus) && (K <= 64 || (!accumulate && !col_bias));
    // (with very many tiles and K in whole stages of 32 the walk over 256 x 128 tiles is the faster one)
    if (shortk_ok && !accumulate && !col_bias && b_mode == LOAD_VEC4 && resident_beats_shortk(M, N, K, cur().model.cus) &&
        (double)256 * ldc * 4.0 < 2147483648.0) {
        static const int big_tile[4] = {256, 128, 32, 1};
        GemmPlan plan;
        const char* route = std::getenv("CAKE_HIP_GEMM_ROUTE");
        if (!(route && !std::strcmp(route, "tile")) && plan_gemm(M, N, K, sched, big_tile, vec_plan, cur().model, &plan) == CAKE_HIP_OK &&
            plan.pub.split_k == 1 && plan.pub.tail_tiles == 0) {
            GemmArgs g{};
            g.A = A; g.B = B; g.C = C;
            g.M = M; g.N = N; g.K = K;
            g.lda = lda; g.ldb = ldb; g.ldc = ldc;
            g.tiles_m = plan.pub.tiles_m; g.tiles_n = plan.pub.tiles_n;
            g.split_k = 1; g.k_per_split = plan.k_per_split;
            g.group = plan.pub.group; g.group_along_n = plan.group_along_n;
            return timer.family(0, [&] { return launch_sgemm_resident(g, cur().model.cus, stream); });
        }
    }
    if (shortk_ok) {
        GemmArgs g{};
        g.A = A; g.B = B; g.C = C;
        g.M = M; g.N = N; g.K = K;
        g.lda = lda; g.ldb = ldb; g.ldc = ldc;
        const int tn = shortk_tile_n(M, N, K, cur().model.cus);
        g.tiles_m = (M + 63) / 64; g.tiles_n = (N + tn - 1) / tn;
        g.split_k = 1; g.k_per_split = K;
        // The tile sequence runs down bands of tile rows.  Up to 16 tile rows make one band: a
        // workgroup's tiles then share their rows of A and a column block of B is used up before the
        // next.  Taller products are cut into bands of 4 to 16 tile rows (a power of two, so that a
        // workgroup still keeps its rows of A from tile to tile): the tiles in flight then spread over
        // more columns of C, whose rows are a power of two apart more often than not, and with them
        // over more memory channels -- 16384^2 x 16: 230 -> 209 us, x 32: 284 -> 249 us, 8192^2 x 8:
        // 57 -> 45 us, x 32: 67 -> 60 us, 16384 x 4096 x 16: 57 -> 46 us, 12288^2 x 32: 160 -> 142 us,
        // 20000 x 10000 x 24: 277 -> 230 us; wider products want lower bands (4096 x 16384 x 16: 46.5 us
        // in bands of 4, 54.7 of 8, 58.6 of 16; 16384 x 4096 x 16: 53.6, 49.7, 46.1).
        g.group = shortk_band_rows(g.tiles_m, N);
        g.group_along_n = 0;
        g.accumulate = accumulate;
        g.col_bias = col_bias;
        return timer.family(0, [&] { return launch_sgemm_shortk(g, tn, cur().model.cus, stream); });
    }
    GemmPlan plan;
    int st = choice ? plan_gemm_choice(M, N, K, sched, *choice, vec_plan, cur().model, &plan)
                    : plan_gemm(M, N, K, sched, tile_override, vec_plan, cur().model, &plan);
    if (st) return fail(st, "no tile matches the requested override");
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.tiles_m = plan.pub.tiles_m; g.tiles_n = plan.pub.tiles_n;
    g.split_k = plan.pub.split_k; g.k_per_split = plan.k_per_split;
    g.group = plan.pub.group; g.group_along_n = plan.group_along_n;
    g.accumulate = accumulate;
    g.col_bias = col_bias;
    if (conv) g.conv = *conv;
    g.partial = nullptr;
    g.tail_tiles = plan.pub.tail_tiles;
    g.tail_split = plan.pub.tail_split;
    g.tail_k_per_split = plan.tail_k_per_split;
    g.tail_partial = nullptr;
    if (plan.pub.tail_tiles > 0) {
        st = scratch_space(cur().splitk, (size_t)plan.pub.tail_tiles * plan.pub.tail_split * plan.pub.tile_m *
                                             plan.pub.tile_n * sizeof(float), &g.tail_partial);
        if (st) return st;
    }
    if (plan.pub.split_k > 1) {
        st = scratch_space(cur().splitk, (size_t)plan.pub.split_k * M * N * sizeof(float), &g.partial);
        if (st) return st;
    }
    // A plain product on 256 x 128 tiles with a K below 1024 and two tiles per CU or more: one
    // workgroup per CU stays and walks over the tiles (sgemm_resident.hip).
    // CAKE_HIP_GEMM_ROUTE=tile keeps the macro-tile kernel (for tests and measurements; read at every call).
    if (plan.pub.tile_m == 256 && plan.pub.tile_n == 128 && plan.pub.split_k == 1 && plan.pub.tail_tiles == 0 && !conv &&
        a_mode == LOAD_VEC4 && b_mode == LOAD_VEC4 &&
        resident_applies(M, N, K, cur().model.cus, !accumulate && !col_bias, tile_override != nullptr)) {
        const char* route = std::getenv("CAKE_HIP_GEMM_ROUTE");
        if (!(route && !std::strcmp(route, "tile")))
            return timer.family(0, [&] { return launch_sgemm_resident(g, cur().model.cus, stream); });
    }
    st = timer.family(0, [&] { return launch_sgemm(plan.tile_id, a_mode, b_mode, g, plan.pub.grid, stream); });
    if (st) return st;
    if (plan.pub.split_k > 1)
        st = timer.family(1, [&] {
            return launch_splitk_reduce(g.partial, C, M, N, ldc, plan.pub.split_k, accumulate, stream, conv,
                                        col_bias);
        });
    else if (plan.pub.tail_tiles > 0)
        st = timer.family(1, [&] { return launch_tail_reduce(plan.tile_id, g, stream); });
    return st;
}

}  // namespace

extern "C" {

const char* cake_hip_strerror(int status)
{
    switch (status) {
        case CAKE_HIP_OK: return "ok";
        case CAKE_HIP_ERR_ARG: return "invalid argument";
        case CAKE_HIP_ERR_NO_DEVICE: return "no usable HIP device";
        case CAKE_HIP_ERR_HIP: return "HIP runtime error";
        case CAKE_HIP_ERR_ALLOC: return "allocation failed";
        case CAKE_HIP_ERR_RANGE: return "operand exceeds 32-bit element indexing";
        case CAKE_HIP_ERR_ARCH: return "device is not gfx950";
        default: return "unknown status";
    }
}

const char* cake_hip_last_error(void) { return g_last_error.c_str(); }

int cake_hip_init(int device)
{
    Context& c = g_default_ctx;
    std::lock_guard<std::recursive_mutex> lock(c.mutex);
    if (c.ready && c.device == device) return CAKE_HIP_OK;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(CAKE_HIP_ERR_NO_DEVICE, "hipGetDeviceCount found no device");
    }
    if (device < 0 || device >= count) return fail(CAKE_HIP_ERR_ARG, "device %d out of range (%d present)", device, count);
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(CAKE_HIP_ERR_ARCH, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    c.device = device;
    c.info = cake_hip_device_t{};
    c.info.device = device;
    c.info.cus = prop.multiProcessorCount;
    c.info.xcds = 8;
    c.info.lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
    c.info.l2_bytes = prop.l2CacheSize;
    c.info.wavefront = prop.warpSize;
    c.info.clock_khz = prop.clockRate;
    c.info.hbm_bytes = prop.totalGlobalMem;
    std::snprintf(c.info.arch, sizeof c.info.arch, "%s", prop.gcnArchName);
    c.model = DeviceModel{};
    if (c.info.cus > 0) c.model.cus = c.info.cus;
    if (c.info.lds_bytes_per_cu >= 64 * 1024) c.model.lds_per_cu = c.info.lds_bytes_per_cu;
    int st = c.create_events();
    if (st) return st;
    // this device's copy of the file-scope scratch array (every device has its own, at its own address)
    if (device < MAX_DEVICES && !g_noalloc_ptr[device]) {
        void* at = nullptr;
        HIP_TRY(hipGetSymbolAddress(&at, HIP_SYMBOL(noalloc_scratch)));
        g_noalloc_ptr[device] = static_cast<unsigned char*>(at);
    }
    if (const char* tuned = std::getenv("CAKE_HIP_TUNE_FILE")) (void)tune_load(tuned);  // optional
    c.ready = true;
    return CAKE_HIP_OK;
}

int cake_hip_shutdown(void)
{
    Context& c = g_default_ctx;
    std::lock_guard<std::recursive_mutex> lock(c.mutex);
    if (!c.ready) return CAKE_HIP_OK;
    (void)hipDeviceSynchronize();
    c.release_all();
    c.ready = false;
    return CAKE_HIP_OK;
}

int cake_hip_ctx_create(cake_hip_ctx_t* out)
{
    if (!out) return fail(CAKE_HIP_ERR_ARG, "out is NULL");
    *out = nullptr;
    if (!g_default_ctx.ready) {
        int st = cake_hip_init(0);
        if (st) return st;
    }
    Context* c = new (std::nothrow) Context;
    if (!c) return fail(CAKE_HIP_ERR_ALLOC, "out of host memory");
    c->device = g_default_ctx.device;
    c->info = g_default_ctx.info;
    c->model = g_default_ctx.model;
    int st = c->create_events();
    if (st == CAKE_HIP_OK && hipStreamCreateWithFlags(&c->own_stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        st = fail(CAKE_HIP_ERR_HIP, "hipStreamCreateWithFlags failed");
    }
    if (st) {
        c->release_all();
        delete c;
        return st;
    }
    c->ready = true;
    {
        std::lock_guard<std::mutex> lock(g_ctx_registry_mutex);
        g_created_ctx.push_back(c);
    }
    *out = c;
    return CAKE_HIP_OK;
}

static Context* find_created(cake_hip_ctx_t h)
{
    std::lock_guard<std::mutex> lock(g_ctx_registry_mutex);
    for (Context* c : g_created_ctx)
        if (c == h) return c;
    return nullptr;
}

int cake_hip_ctx_destroy(cake_hip_ctx_t h)
{
    if (!h) return CAKE_HIP_OK;
    Context* c = find_created(h);
    if (!c) return fail(CAKE_HIP_ERR_ARG, "not a context from cake_hip_ctx_create (or destroyed already)");
    if (t_current_ctx == c) t_current_ctx = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_ctx_registry_mutex);
        for (size_t i = 0; i < g_created_ctx.size(); ++i)
            if (g_created_ctx[i] == c) {
                g_created_ctx.erase(g_created_ctx.begin() + i);
                break;
            }
    }
    {
        // a call on another thread that still holds the context finishes first; the work it and
        // earlier calls enqueued (on the context's stream or a caller's) may still read the workspaces
        std::lock_guard<std::recursive_mutex> lock(c->mutex);
        (void)hipDeviceSynchronize();
        c->release_all();
        c->ready = false;
    }
    // The husk (a few hundred bytes, no device resources) is kept: a thread that still has the
    // context current then gets an error from its next call instead of touching freed memory.
    return CAKE_HIP_OK;
}

int cake_hip_ctx_set_current(cake_hip_ctx_t h)
{
    if (!h) {
        t_current_ctx = nullptr;
        return CAKE_HIP_OK;
    }
    Context* c = find_created(h);
    if (!c) return fail(CAKE_HIP_ERR_ARG, "not a context from cake_hip_ctx_create (or destroyed already)");
    t_current_ctx = c;
    return CAKE_HIP_OK;
}

cake_hip_ctx_t cake_hip_ctx_get_current(void) { return t_current_ctx; }

void* cake_hip_ctx_stream(cake_hip_ctx_t h)
{
    if (!h) return nullptr;
    Context* c = find_created(h);
    return c ? c->own_stream : nullptr;
}

int cake_hip_device_info(cake_hip_device_t* out)
{
    if (!out) return fail(CAKE_HIP_ERR_ARG, "out is NULL");
    int st = ensure_init();
    if (st) return st;
    *out = cur().info;
    return CAKE_HIP_OK;
}

int cake_hip_malloc(void** ptr, size_t bytes)
{
    if (!ptr) return fail(CAKE_HIP_ERR_ARG, "ptr is NULL");
    int st = ensure_init();
    if (st) return st;
    *ptr = nullptr;
    if (bytes == 0) return CAKE_HIP_OK;
    if (hipMalloc(ptr, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return fail(CAKE_HIP_ERR_ALLOC, "device allocation of %zu bytes failed", bytes);
    }
    return CAKE_HIP_OK;
}

int cake_hip_free(void* ptr)
{
    if (!ptr) return CAKE_HIP_OK;
    HIP_TRY(hipFree(ptr));
    return CAKE_HIP_OK;
}

// true for ordinary (pageable) host memory: neither device memory nor host memory the runtime knows
static bool is_pageable_host(const void* p)
{
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return attr.type == hipMemoryTypeUnregistered;
}

// Large copies from or to pageable memory travel through the library's pinned buffers like the
// operands of a compute call (a plain hipMemcpy of 256 MB: 30 GB/s to the device, 17.5 GB/s back).
// Both wait for the device first, as hipMemcpy on the null stream does for its own stream.
int cake_hip_memcpy_h2d(void* dst, const void* src, size_t bytes)
{
    if (bytes && (!dst || !src)) return fail(CAKE_HIP_ERR_ARG, "NULL pointer");
    if (bytes >= PIN_THRESHOLD && is_pageable_host(src)) {
        int st = ensure_init();
        if (st) return st;
        std::lock_guard<std::recursive_mutex> lock(cur().mutex);
        HIP_TRY(hipDeviceSynchronize());
        return host_to_device(dst, src, bytes);
    }
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return CAKE_HIP_OK;
}

int cake_hip_memcpy_d2h(void* dst, const void* src, size_t bytes)
{
    if (bytes && (!dst || !src)) return fail(CAKE_HIP_ERR_ARG, "NULL pointer");
    if (bytes >= PIN_THRESHOLD && is_pageable_host(dst)) {
        int st = ensure_init();
        if (st) return st;
        std::lock_guard<std::recursive_mutex> lock(cur().mutex);
        HIP_TRY(hipDeviceSynchronize());
        return device_to_host(dst, src, bytes);
    }
    HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return CAKE_HIP_OK;
}

int cake_hip_memset(void* dst, int value, size_t bytes)
{
    if (bytes && !dst) return fail(CAKE_HIP_ERR_ARG, "NULL pointer");
    HIP_TRY(hipMemset(dst, value, bytes));
    return CAKE_HIP_OK;
}

int cake_hip_synchronize(void)
{
    HIP_TRY(hipDeviceSynchronize());
    return CAKE_HIP_OK;
}

// Which kernel cake_hip_sgemm runs for dense row-major operands of this shape (CAKE_HIP_KERNEL_*)
static int kernel_family(int M, int N, int K, bool tile_forced, bool vec)
{
    if (tile_forced || M <= 0 || N <= 0 || K <= 0) return CAKE_HIP_KERNEL_TILE;
    if (M == 1 || N == 1) return CAKE_HIP_KERNEL_GEMV;
    if (vec && !tune_lookup(M, N, K, true, nullptr)) {
        if (fewrows_applies(M, N, K, K, N)) return CAKE_HIP_KERNEL_STREAM_ROWS;
        if (fewrows_nt_applies(N, M, K, N, K, true)) return CAKE_HIP_KERNEL_STREAM_COLS;
        if (shortk_applies(M, N, K, cur().ready ? cur().model.cus : DeviceModel{}.cus)) return CAKE_HIP_KERNEL_SHORT_K;
    }
    return CAKE_HIP_KERNEL_TILE;
}

int cake_hip_plan(int M, int N, int K, int sched, const int* tile_override, cake_hip_plan_t* out)
{
    if (!out) return fail(CAKE_HIP_ERR_ARG, "out is NULL");
    GemmPlan plan;
    const DeviceModel model = cur().ready ? cur().model : DeviceModel{};
    const bool vec = vec4_loadable(nullptr, nullptr, K, N);
    int st = plan_gemm(M, N, K, sched, tile_override, vec, model, &plan);
    if (st) return fail(st, "cake_hip_plan: bad shape, schedule or tile override");
    *out = plan.pub;
    out->kernel = kernel_family(M, N, K, tile_override != nullptr, vec);
    if (out->kernel == CAKE_HIP_KERNEL_SHORT_K && resident_beats_shortk(M, N, K, model.cus)) {
        // very many tiles, K in whole stages of 32: the walk over 256 x 128 tiles instead
        static const int big_tile[4] = {256, 128, 32, 1};
        GemmPlan big;
        if (plan_gemm(M, N, K, sched, big_tile, vec, model, &big) == CAKE_HIP_OK && big.pub.split_k == 1 && big.pub.tail_tiles == 0) {
            *out = big.pub;
            out->kernel = CAKE_HIP_KERNEL_TILE;   // (named below)
        }
    }
    if (out->kernel == CAKE_HIP_KERNEL_SHORT_K) {
        // what launch_sgemm_shortk does: 64 x 64 tiles with the whole K in one LDS stage, walked in
        // column blocks of B by the resident workgroups per CU
        const int tn = shortk_tile_n(M, N, K, model.cus);
        out->tile_m = 64; out->tile_n = tn; out->tile_k = K <= 32 || K > 64 ? 32 : 64;
        out->wave_m = 32; out->wave_n = tn / 2;
        out->threads = 256;
        out->split_k = 1; out->tail_tiles = 0; out->tail_split = 1;
        out->tiles_m = (M + 63) / 64; out->tiles_n = (N + tn - 1) / tn;
        out->group = shortk_band_rows(out->tiles_m, N);
        shortk_launch_shape((long)out->tiles_m * out->tiles_n, tn, K, model.cus, &out->grid, &out->lds_bytes);
    } else if (out->kernel == CAKE_HIP_KERNEL_TILE && vec && out->tile_m == 256 && out->tile_n == 128 && out->split_k == 1 &&
               out->tail_tiles == 0 &&
               (resident_applies(M, N, K, model.cus, true, tile_override != nullptr) || (!tile_override && resident_beats_shortk(M, N, K, model.cus)))) {
        // what launch_sgemm_resident does with the same tiles: one workgroup of 8 waves per CU
        // that walks over them, its operands loaded straight into LDS
        const long tiles = (long)out->tiles_m * out->tiles_n;
        out->kernel = CAKE_HIP_KERNEL_RESIDENT;
        out->threads = 512;
        out->grid = (int)(((tiles < model.cus ? tiles : (long)model.cus) + 7) / 8 * 8);
        out->lds_bytes = resident_lds_bytes();
    }
    return CAKE_HIP_OK;
}

int cake_hip_init_block_dims(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cntx, int sched,
                             int mcu, int kcu, int ncu, cake_hip_blk_dims_t* out)
{
    int st = init_block_dims(M, N, K, p, cntx, sched, mcu, kcu, ncu, out);
    if (st) return fail(st, "cake_hip_init_block_dims: invalid argument");
    return CAKE_HIP_OK;
}

int cake_hip_derive_schedule(int M, int N, int K, int p, int mc, const cake_hip_cpu_cntx_t* cntx)
{
    if (!cntx || p <= 0 || mc <= 0) return CAKE_HIP_KMN;
    return derive_schedule(M, N, K, p, mc, cntx);
}

int cake_hip_grid_dims_2d(int M, int N, int K, int p, int ncores) { return grid_dims_2d(M, N, K, p, ncores); }

int cake_hip_init_block_dims_2d(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cntx, int sched, float type_size,
                                int mcu, int kcu, int ncu, cake_hip_blk_dims_t* out)
{
    int st = init_block_dims_2d(M, N, K, p, cntx, sched, type_size, mcu, kcu, ncu, out);
    if (st) return fail(st, "cake_hip_init_block_dims_2d: invalid argument");
    return CAKE_HIP_OK;
}

int cake_hip_init_block_dims_2d_small(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cntx, int sched,
                                      float type_size, cake_hip_blk_dims_t* out)
{
    int st = init_block_dims_2d_small(M, N, K, p, cntx, sched, type_size, out);
    if (st) return fail(st, "cake_hip_init_block_dims_2d_small: invalid argument");
    return CAKE_HIP_OK;
}

int cake_hip_init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s,
                                  int p, cake_hip_cpu_cntx_t* cntx, cake_hip_blk_dims_t* out)
{
    int st = init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cntx, out);
    if (st) return fail(st, "cake_hip_init_block_dims_conv: invalid argument");
    return CAKE_HIP_OK;
}

// Rows of A (and of C) per block of the pipelined host path: about a quarter of the rows, whole
// macro-tile rows, and a block of either matrix fits a pinned buffer.  0: rows too long for this path.
static int host_row_block(int M, int K, int N)
{
    const size_t widest = (size_t)(K > N ? K : N) * sizeof(float);
    const int fit = (int)(PIN_CHUNK / widest / 256 * 256);
    const int quarter = (M / 4 + 255) / 256 * 256;
    return fit < quarter ? fit : quarter;
}

// C = A . B with A and C in host memory and large: instead of "upload all, multiply, download
// all", the rows of A travel in blocks through a three-stage pipeline.  While block i is
// multiplied, block i + 1 is copied into a pinned buffer and sent to the device, block i - 1 comes
// back into another pinned buffer and block i - 2 is copied out to the caller's C.  B (device
// memory by now) is needed by every block and goes first.  The products of the blocks are
// ordinary calls of the row-major kernel on device memory.
static int sgemm_host_pipelined(const float* A, const float* b_dev, float* C, int M, int N, int K, int sched,
                                const int* tile_override, hipStream_t stream, double* seconds)
{
    const int RB = host_row_block(M, K, N);
    const int nblk = (M + RB - 1) / RB;
    int st = pinned_both_ways_ready();
    if (st) return st;
    if ((st = cur().stage[0].reserve((size_t)M * K * 4))) return st;
    if ((st = cur().stage[2].reserve((size_t)M * N * 4))) return st;
    float* a_dev = static_cast<float*>(cur().stage[0].ptr);
    float* c_dev = static_cast<float*>(cur().stage[2].ptr);
    HIP_TRY(hipDeviceSynchronize());   // nothing of an earlier call still uses the staging slots

    struct Events {
        std::vector<hipEvent_t> ev;
        ~Events() { for (hipEvent_t e : ev) if (e) (void)hipEventDestroy(e); }
    } events;
    events.ev.assign((size_t)3 * nblk, nullptr);
    for (hipEvent_t& e : events.ev) HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    hipEvent_t* up = events.ev.data();            // block i has arrived on the device
    hipEvent_t* done = up + nblk;                 // block i has been multiplied
    hipEvent_t* back = done + nblk;               // block i of C sits in its pinned buffer

    auto rows_of = [&](int i) { return M - i * RB < RB ? M - i * RB : RB; };
    // `seconds`: from the first product's start to the last one's end on the stream (the waits for
    // arriving blocks included); no per-kernel timing, which would stop the host after every launch
    Timer timer(stream, seconds), untimed(stream, nullptr);
    if ((st = timer.start())) return st;
    for (int i = 0; i < nblk + 2; ++i) {
        if (i < nblk) {
            const size_t off = (size_t)i * RB * K, bytes = (size_t)rows_of(i) * K * 4;
            void* pin = cur().pinned[i & 1];
            if (i >= 2) HIP_TRY(hipEventSynchronize(up[i - 2]));   // the buffer's last transfer is over
            parallel_memcpy(pin, A + off, bytes);
            HIP_TRY(hipMemcpyAsync(a_dev + off, pin, bytes, hipMemcpyHostToDevice, cur().copy_stream));
            HIP_TRY(hipEventRecord(up[i], cur().copy_stream));
            HIP_TRY(hipStreamWaitEvent(stream, up[i], 0));
            const float* ai = a_dev + off;
            float* ci = c_dev + (size_t)i * RB * N;
            const int mode = vec4_loadable(ai, b_dev, K, N) ? LOAD_VEC4 : LOAD_SCALAR;
            if ((st = run_gemm(ai, b_dev, ci, rows_of(i), N, K, K, N, N, sched, 0, tile_override, mode, mode, stream, untimed)))
                return st;
            HIP_TRY(hipEventRecord(done[i], stream));
        }
        if (i >= 1 && i - 1 < nblk) {   // block i - 1 starts its way back (its buffer was emptied one round ago)
            const int j = i - 1;
            HIP_TRY(hipStreamWaitEvent(cur().copy_back_stream, done[j], 0));
            HIP_TRY(hipMemcpyAsync(cur().pinned[2 + (j & 1)], c_dev + (size_t)j * RB * N, (size_t)rows_of(j) * N * 4,
                                   hipMemcpyDeviceToHost, cur().copy_back_stream));
            HIP_TRY(hipEventRecord(back[j], cur().copy_back_stream));
        }
        if (i >= 2) {                   // block i - 2 has arrived: out to the caller's C
            const int j = i - 2;
            HIP_TRY(hipEventSynchronize(back[j]));
            parallel_memcpy(C + (size_t)j * RB * N, cur().pinned[2 + (j & 1)], (size_t)rows_of(j) * N * 4);
        }
    }
    return timer.stop();
}

// C = A . B on device operands: the matrix-vector kernels for a single row or column, run_gemm
// for everything else, a fill for an empty sum.
static int sgemm_on_device(const float* A, const float* B, float* C, int M, int N, int K, int sched, int accumulate,
                           const int* tile_override, hipStream_t stream, Timer& timer)
{
    int st = CAKE_HIP_OK;
    if (K == 0) {
        // empty sum: C = 0 (or unchanged when accumulating); a fill kernel, not a memset node
        if (!accumulate) {
            hipError_t e = launch_splitk_reduce(nullptr, C, M, N, N, 0, 0, stream);
            if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "zero fill failed: %s", hipGetErrorString(e));
        }
    } else if ((M == 1 || N == 1) && !tile_override) {
        // A product with a single row or column is a matrix-vector product: C[M] = A[M][K] . B[K]
        // reads A row-major; C[N] = A[K] . B[K][N] is B read as a column-major N x K matrix.
        const size_t floats = N == 1 ? sgemv_rowmajor_scratch_floats(M, K, cur().model.cus)
                                     : sgemv_colmajor_scratch_floats(N, K, cur().model.cus);
        float* scratch = nullptr;
        if (floats && (st = scratch_space(cur().gemv, floats * sizeof(float), &scratch))) return st;
        st = timer.family(2, [&] {
            return N == 1 ? launch_sgemv_rowmajor(A, B, C, M, K, accumulate, scratch, cur().model.cus, stream)
                          : launch_sgemv_colmajor(B, A, C, N, K, accumulate, scratch, cur().model.cus, stream);
        });
        if (st) return st;
    } else {
        const bool vec = vec4_loadable(A, B, K, N);
        const int mode = vec ? LOAD_VEC4 : LOAD_SCALAR;
        st = run_gemm(A, B, C, M, N, K, K, N, N, sched, accumulate, tile_override, mode,
                      mode, stream, timer);
        if (st) return st;
    }
    return CAKE_HIP_OK;
}

int cake_hip_sgemm(const float* A, const float* B, float* C, int M, int N, int K, int sched,
                   int accumulate, const int* tile_override, void* stream_, double* seconds)
{
    if (M < 0 || N < 0 || K < 0) return fail(CAKE_HIP_ERR_ARG, "negative dimension");
    if (sched < 0 || sched > CAKE_HIP_NA) return fail(CAKE_HIP_ERR_ARG, "unknown schedule %d", sched);
    if (seconds) *seconds = 0;
    if (M == 0 || N == 0) return CAKE_HIP_OK;
    if (!A || !B || !C) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if (!fits_int((double)M * K) || !fits_int((double)K * N) || !fits_int((double)M * N))
        return fail(CAKE_HIP_ERR_RANGE, "operand of %dx%dx%d exceeds 2^31 elements", M, K, N);
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand a, b, c;
    // large host operands: transfers and arithmetic overlap block by block
    const int RB = K > 0 ? host_row_block(M, K, N) : 0;
    if (RB > 0 && M >= 3 * RB && N > 32 && ((double)M * K + (double)M * N) * 4 >= 32.0 * (1 << 20) && !accumulate &&
        !is_device_pointer(A) && !is_device_pointer(C)) {
        if ((st = stage_in(B, (size_t)K * N * 4, 1, true, &b))) return st;
        return sgemm_host_pipelined(A, b.dev, C, M, N, K, sched, tile_override, stream, seconds);
    }
    if ((st = stage_in(A, (size_t)M * K * 4, 0, true, &a))) return st;
    if ((st = stage_in(B, (size_t)K * N * 4, 1, true, &b))) return st;
    if ((st = stage_in(C, (size_t)M * N * 4, 2, accumulate != 0, &c))) return st;

    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if ((st = sgemm_on_device(a.dev, b.dev, c.dev, M, N, K, sched, accumulate, tile_override, stream, timer))) return st;
    if ((st = timer.stop())) return st;
    return stage_out(c, stream);
}

int cake_hip_sgemm_noalloc(const float* A, const float* B, float* C, int M, int N, int K, int sched,
                           int accumulate, void* stream_)
{
    if (M < 0 || N < 0 || K < 0) return fail(CAKE_HIP_ERR_ARG, "negative dimension");
    if (sched < 0 || sched > CAKE_HIP_NA) return fail(CAKE_HIP_ERR_ARG, "unknown schedule %d", sched);
    if (M == 0 || N == 0) return CAKE_HIP_OK;
    if (!A || !B || !C) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if (!fits_int((double)M * K) || !fits_int((double)K * N) || !fits_int((double)M * N))
        return fail(CAKE_HIP_ERR_RANGE, "operand of %dx%dx%d exceeds 2^31 elements", M, K, N);
    // nothing is set up here: events, device model and the scratch address come from cake_hip_init
    Context& c = cur();
    std::lock_guard<std::recursive_mutex> lock(c.mutex);
    if (!c.ready)
        return fail(CAKE_HIP_ERR_NO_DEVICE, "cake_hip_sgemm_noalloc needs cake_hip_init to have run: it sets nothing up itself");
    if (c.device >= MAX_DEVICES || !g_noalloc_ptr[c.device])
        return fail(CAKE_HIP_ERR_NO_DEVICE, "no scratch address for device %d", c.device);
    if (!is_device_pointer(A) || !is_device_pointer(B) || !is_device_pointer(C))
        return fail(CAKE_HIP_ERR_ARG, "cake_hip_sgemm_noalloc takes device memory only (host operands need staging buffers)");
    hipStream_t stream = pick_stream(stream_);
    Timer untimed(stream, nullptr);
    c.noalloc_call = true;
    c.noalloc_used = 0;
    const int st = sgemm_on_device(A, B, C, M, N, K, sched, accumulate, nullptr, stream, untimed);
    c.noalloc_call = false;
    return st;
}

size_t cake_hip_packed_a_size(int M, int K, int p, const cake_hip_blk_dims_t* d,
                              const cake_hip_cpu_cntx_t* cx, int sched)
{
    if (check_geom(d, cx, p, sched)) return 0;
    PackGeom g = make_geom(M, 0, K, p, d, cx, sched);
    return (size_t)padded_rows(g) * (size_t)K * sizeof(float);
}

size_t cake_hip_packed_b_size(int K, int N, int p, const cake_hip_blk_dims_t* d,
                              const cake_hip_cpu_cntx_t* cx)
{
    if (check_geom(d, cx, p, CAKE_HIP_KMN)) return 0;
    PackGeom g = make_geom(0, N, K, p, d, cx, CAKE_HIP_KMN);
    return (size_t)K * (size_t)padded_cols(g) * sizeof(float);
}

size_t cake_hip_packed_c_size(int M, int N, int p, const cake_hip_blk_dims_t* d,
                              const cake_hip_cpu_cntx_t* cx, int sched)
{
    if (check_geom(d, cx, p, sched)) return 0;
    PackGeom g = make_geom(M, N, 0, p, d, cx, sched);
    return (size_t)padded_rows(g) * (size_t)padded_cols(g) * sizeof(float);
}

int64_t cake_hip_packed_offset(int which, int row, int col, int M, int N, int K, int p,
                               const cake_hip_blk_dims_t* d, const cake_hip_cpu_cntx_t* cx, int sched)
{
    if (check_geom(d, cx, p, sched)) return -1;
    PackGeom g = make_geom(M, N, K, p, d, cx, sched);
    if (row < 0 || col < 0) return -1;
    switch (which) {
        case 0: return (row < padded_rows(g) && col < K) ? packed_a_offset(g, row, col) : -1;
        case 1: return (row < K && col < padded_cols(g)) ? packed_b_offset(g, row, col) : -1;
        case 2: return (row < padded_rows(g) && col < padded_cols(g)) ? packed_c_offset(g, row, col) : -1;
        default: return -1;
    }
}

// which: 0 A (rows M, cols K), 1 B (rows K, cols N), 2 C (rows M, cols N); dir: 0 pack, 1 unpack
static int pack_common(int which, int dir, const float* src, float* dst, int M, int N, int K, int p,
                       const cake_hip_blk_dims_t* d, const cake_hip_cpu_cntx_t* cx, int sched,
                       void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    int st = check_geom(d, cx, p, sched);
    if (st) return st;
    if (!src || !dst) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    PackGeom g = make_geom(M, N, K, p, d, cx, sched);
    const int rows = (which == 1) ? K : M, cols = (which == 0) ? K : N;
    const int rows_p = (which == 1) ? K : padded_rows(g), cols_p = (which == 0) ? K : padded_cols(g);
    if (rows <= 0 || cols <= 0) return fail(CAKE_HIP_ERR_ARG, "empty operand");
    if (!fits_int((double)rows_p * cols_p)) return fail(CAKE_HIP_ERR_RANGE, "packed operand exceeds 2^31 elements");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    const size_t plain_bytes = (size_t)rows * cols * 4, packed_bytes = (size_t)rows_p * cols_p * 4;
    Operand in, out;
    if ((st = stage_in(src, dir == 0 ? plain_bytes : packed_bytes, 0, true, &in))) return st;
    // unpack writes only the real extent of C; a staged C must start from the caller's values
    if ((st = stage_in(dst, dir == 0 ? packed_bytes : plain_bytes, 1, false, &out))) return st;
    if ((st = cur().tables.reserve(tables_bytes(which, g)))) return st;

    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    size_t at = 0;
    IndexTables tab;
    if ((st = build_tables(which, g, &at, &tab, stream))) return st;
    st = timer.family(4, [&] {
        const int fast = which == 0 ? g.mr : g.nr;
        return dir == 0 ? launch_pack(in.dev, out.dev, rows, cols, cols, rows_p, cols_p, tab, fast, which == 0, stream)
                        : launch_unpack(in.dev, out.dev, rows, cols, cols, tab, fast, which == 0, stream);
    });
    if (st) return st;
    if ((st = timer.stop())) return st;
    return stage_out(out, stream);
}

int cake_hip_pack_a(const float* A, float* A_p, int M, int K, int p, const cake_hip_blk_dims_t* d,
                    const cake_hip_cpu_cntx_t* cx, int sched, void* stream, double* seconds)
{
    return pack_common(0, 0, A, A_p, M, 0, K, p, d, cx, sched, stream, seconds);
}

int cake_hip_pack_b(const float* B, float* B_p, int K, int N, int p, const cake_hip_blk_dims_t* d,
                    const cake_hip_cpu_cntx_t* cx, int sched, void* stream, double* seconds)
{
    return pack_common(1, 0, B, B_p, 0, N, K, p, d, cx, sched, stream, seconds);
}

int cake_hip_pack_c(const float* C, float* C_p, int M, int N, int p, const cake_hip_blk_dims_t* d,
                    const cake_hip_cpu_cntx_t* cx, int sched, void* stream, double* seconds)
{
    return pack_common(2, 0, C, C_p, M, N, 0, p, d, cx, sched, stream, seconds);
}

int cake_hip_unpack_c(float* C, const float* C_p, int M, int N, int p, const cake_hip_blk_dims_t* d,
                      const cake_hip_cpu_cntx_t* cx, int sched, void* stream, double* seconds)
{
    return pack_common(2, 1, C_p, C, M, N, 0, p, d, cx, sched, stream, seconds);
}

int cake_hip_sgemm_packed(const float* A, const float* B, float* C, int M, int N, int K, int p,
                          const cake_hip_blk_dims_t* d, const cake_hip_cpu_cntx_t* cx, int packedA,
                          int packedB, int accumulate, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    if (!packedA && !packedB) return cake_hip_sgemm(A, B, C, M, N, K, d ? d->sch : CAKE_HIP_NA, accumulate, nullptr, stream_, seconds);
    if (!d) return fail(CAKE_HIP_ERR_ARG, "block dims is NULL");
    const int sched = d->sch;
    int st = check_geom(d, cx, p, sched);
    if (st) return st;
    if (M <= 0 || N <= 0 || K <= 0) return fail(CAKE_HIP_ERR_ARG, "empty operand");
    if (!A || !B || !C) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    PackGeom g = make_geom(M, N, K, p, d, cx, sched);
    const size_t a_elems = packedA ? (size_t)padded_rows(g) * K : (size_t)M * K;
    const size_t b_elems = packedB ? (size_t)K * padded_cols(g) : (size_t)K * N;
    if (!fits_int((double)a_elems) || !fits_int((double)b_elems) || !fits_int((double)M * N))
        return fail(CAKE_HIP_ERR_RANGE, "operand exceeds 2^31 elements");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand a, b, c;
    if ((st = stage_in(A, a_elems * 4, 0, true, &a))) return st;
    if ((st = stage_in(B, b_elems * 4, 1, true, &b))) return st;
    if ((st = stage_in(C, (size_t)M * N * 4, 2, accumulate != 0, &c))) return st;
    if ((st = cur().tables.reserve((packedA ? tables_bytes(0, g) : 0) + (packedB ? tables_bytes(1, g) : 0)))) return st;
    // A packed operand is first copied back to row-major order (one pass at HBM speed through
    // the index tables); the product then runs on the row-major kernel, which is several times
    // faster than gathering packed elements inside the K walk.
    const size_t ua_floats = packedA ? (((size_t)M * K + 63) & ~(size_t)63) : 0;
    const size_t ub_floats = packedB ? (size_t)K * N : 0;
    if ((st = cur().unpacked.reserve((ua_floats + ub_floats) * sizeof(float)))) return st;
    float* ua = static_cast<float*>(cur().unpacked.ptr);
    float* ub = ua + ua_floats;

    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    size_t at = 0;
    IndexTables ta{}, tb{};
    if (packedA) {
        if ((st = build_tables(0, g, &at, &ta, stream))) return st;
        if ((st = timer.family(4, [&] { return launch_unpack(a.dev, ua, M, K, K, ta, g.mr, true, stream); }))) return st;
    }
    if (packedB) {
        if ((st = build_tables(1, g, &at, &tb, stream))) return st;
        if ((st = timer.family(4, [&] { return launch_unpack(b.dev, ub, K, N, N, tb, g.nr, false, stream); }))) return st;
    }
    const float* ga = packedA ? ua : a.dev;
    const float* gb = packedB ? ub : b.dev;
    const int mode = vec4_loadable(ga, gb, K, N) ? LOAD_VEC4 : LOAD_SCALAR;
    st = run_gemm(ga, gb, c.dev, M, N, K, K, N, N, sched, accumulate, nullptr, mode, mode, stream, timer);
    if (st) return st;
    if ((st = timer.stop())) return st;
    return stage_out(c, stream);
}

int cake_hip_sgemv(const float* A, const float* x, float* y, int M, int K, int a_col_major,
                   int accumulate, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    if (M < 0 || K < 0) return fail(CAKE_HIP_ERR_ARG, "negative dimension");
    if (M == 0) return CAKE_HIP_OK;
    if (!y || (K > 0 && (!A || !x))) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if (!fits_int((double)M * K)) return fail(CAKE_HIP_ERR_RANGE, "matrix of %dx%d exceeds 2^31 elements", M, K);
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand a, xv, yv;
    if ((st = stage_in(A, (size_t)M * K * 4, 0, true, &a))) return st;
    if ((st = stage_in(x, (size_t)K * 4, 1, true, &xv))) return st;
    if ((st = stage_in(y, (size_t)M * 4, 2, accumulate != 0, &yv))) return st;
    if (K > 0) {
        const size_t floats = a_col_major ? sgemv_colmajor_scratch_floats(M, K, cur().model.cus)
                                          : sgemv_rowmajor_scratch_floats(M, K, cur().model.cus);
        if (floats && (st = cur().gemv.reserve(floats * sizeof(float)))) return st;
    }
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if (K == 0) {
        if (!accumulate) {
            hipError_t e = launch_splitk_reduce(nullptr, yv.dev, M, 1, 1, 0, 0, stream);
            if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "zero fill failed: %s", hipGetErrorString(e));
        }
    } else {
        st = timer.family(2, [&] {
            return a_col_major ? launch_sgemv_colmajor(a.dev, xv.dev, yv.dev, M, K, accumulate,
                                                       static_cast<float*>(cur().gemv.ptr), cur().model.cus, stream)
                               : launch_sgemv_rowmajor(a.dev, xv.dev, yv.dev, M, K, accumulate,
                                                       static_cast<float*>(cur().gemv.ptr), cur().model.cus, stream);
        });
        if (st) return st;
    }
    if ((st = timer.stop())) return st;
    return stage_out(yv, stream);
}

static int conv_out_dims(int Hin, int Win, int Hf, int Wf, int stride, int pad, int* Hout, int* Wout)
{
    if (Hf <= 0 || Wf <= 0 || stride <= 0 || pad < 0) return 1;
    if (Hin + 2 * pad < Hf || Win + 2 * pad < Wf) return 1;
    *Hout = (Hin + 2 * pad - Hf) / stride + 1;
    *Wout = (Win + 2 * pad - Wf) / stride + 1;
    return 0;
}

int cake_hip_im2col(const float* in, float* cols, int batch, int Cin, int Hin, int Win, int Hf,
                    int Wf, int stride, int pad, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    int Hout, Wout;
    if (batch <= 0 || Cin <= 0 || Hin <= 0 || Win <= 0 || conv_out_dims(Hin, Win, Hf, Wf, stride, pad, &Hout, &Wout))
        return fail(CAKE_HIP_ERR_ARG, "bad convolution geometry");
    if (!in || !cols) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    const double krows = (double)Cin * Hf * Wf, ncols = (double)batch * Hout * Wout;
    if (!fits_int(krows * ncols) || !fits_int((double)batch * Cin * Hin * Win) || krows > 65535)
        return fail(CAKE_HIP_ERR_RANGE, "column matrix %gx%g out of range", krows, ncols);
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);
    Operand i, o;
    if ((st = stage_in(in, (size_t)batch * Cin * Hin * Win * 4, 0, true, &i))) return st;
    if ((st = stage_in(cols, (size_t)(krows * ncols) * 4, 1, false, &o))) return st;
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    st = timer.family(3, [&] {
        return launch_im2col(i.dev, o.dev, batch, Cin, Hin, Win, Hf, Wf, Hout, Wout, stride, pad, stream);
    });
    if (st) return st;
    if ((st = timer.stop())) return st;
    return stage_out(o, stream);
}

// How the input of a convolution is staged for the on-the-fly gather (conv_stage_input_kernel):
// zero padding written out, of every `stride` rows the RH reachable ones kept, every row split
// into its PW reachable column phases of Wq floats.
struct ConvStage {
    bool copy;      // false: stride 1 without padding reads the input as it lies
    int RH, PW, Hs, Wq, pitch;
    double elems;   // floats of the staged input
};

static ConvStage conv_stage(int batch, int Cin, int Hin, int Win, int Hf, int Wf, int stride, int pad)
{
    ConvStage s{};
    s.copy = pad > 0 || stride > 1;
    if (!s.copy) {
        s.RH = s.PW = 1; s.Hs = Hin; s.Wq = s.pitch = Win;
    } else {
        const int Hp = Hin + 2 * pad, Wp = Win + 2 * pad;
        s.RH = Hf < stride ? Hf : stride;
        s.PW = Wf < stride ? Wf : stride;
        s.Hs = (Hp + stride - 1) / stride * s.RH;
        s.Wq = ((Wp + stride - 1) / stride + 3) & ~3;
        s.pitch = s.PW * s.Wq;
    }
    s.elems = (double)batch * Cin * s.Hs * s.pitch;
    return s;
}

size_t cake_hip_conv2d_workspace(int batch, int Cin, int Hin, int Win, int Cout, int Hf, int Wf,
                                 int stride, int pad)
{
    int Hout, Wout;
    if (batch <= 0 || Cin <= 0 || Cout <= 0 || conv_out_dims(Hin, Win, Hf, Wf, stride, pad, &Hout, &Wout)) return 0;
    const size_t ncols = (size_t)batch * Hout * Wout;
    // two-step path: column matrix + a [Cout][ncols] product when the caller wants NCHW;
    // gather path: the staged copy of the input
    const size_t two_step = ((size_t)Cin * Hf * Wf * ncols + (size_t)Cout * ncols) * sizeof(float);
    const size_t staged = (size_t)conv_stage(batch, Cin, Hin, Win, Hf, Wf, stride, pad).elems * sizeof(float);
    return (two_step > staged ? two_step : staged) + 512;
}

// explicit == 0: gather the column matrix inside the GEMM when the geometry allows it
static int conv2d_common(const float* in, const float* weights, float* out, int batch, int Cin, int Hin,
                         int Win, int Cout, int Hf, int Wf, int stride, int pad, int out_nchw,
                         void* workspace, void* stream_, double* seconds, int explicit_cols, int accumulate = 0)
{
    if (seconds) *seconds = 0;
    g_last_conv_route = CAKE_HIP_CONV_NONE;
    int Hout, Wout;
    if (batch <= 0 || Cin <= 0 || Cout <= 0 || Hin <= 0 || Win <= 0 ||
        conv_out_dims(Hin, Win, Hf, Wf, stride, pad, &Hout, &Wout))
        return fail(CAKE_HIP_ERR_ARG, "bad convolution geometry");
    // A 1 x 1 filter at stride 1 without padding sees every plane as one row of Hin * Win pixels:
    // rows of the product are then padded to a multiple of 4 once per plane instead of once per
    // image row (7 x 7 maps: 52 columns for 49 instead of 56, 14 x 14 maps: none at all).
    if (Hf == 1 && Wf == 1 && stride == 1 && pad == 0 && (double)Hin * Win < 2147483647.0) {
        Win *= Hin;
        Hin = 1;
        Wout = Win;
        Hout = 1;
    }
    if (!in || !weights || !out) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if (accumulate && out_nchw && batch > 1) return fail(CAKE_HIP_ERR_ARG, "accumulation into a batched NCHW output is not offered");
    const double K_d = (double)Cin * Hf * Wf;
    const double ncols_d = (double)batch * Hout * Wout;
    const double in_elems = (double)batch * Cin * Hin * Win;
    if (!fits_int(K_d) || !fits_int(Cout * K_d) || !fits_int(ncols_d) || in_elems * 4 >= 1e15 || Cout * ncols_d * 4 >= 1e15)
        return fail(CAKE_HIP_ERR_RANGE, "convolution lowers to a %dx%gx%g product that is out of range", Cout, K_d, ncols_d);
    const int K = (int)K_d, N = (int)ncols_d;
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand i, w, o;
    if ((st = stage_in(in, (size_t)in_elems * 4, 0, true, &i))) return st;
    if ((st = stage_in(weights, (size_t)Cout * K * 4, 1, true, &w))) return st;
    if ((st = stage_in(out, (size_t)Cout * N * 4, 2, accumulate != 0, &o))) return st;

    // A 1 x 1 filter at a stride above 1 without padding reads every stride-th pixel of every
    // stride-th row.  Those are copied out densely first ([batch][Cin][Hout][Wout]: a quarter of
    // the input at stride 2) and the layer then is the 1 x 1 layer at stride 1 on that copy, one row
    // of Hout * Wout pixels per plane, with all the routes of such a layer -- where the staged
    // gather keeps rows padded to 4 columns and narrow maps went through a column matrix and a
    // layout pass.  The copy runs at the speed of the cache lines it touches (32 x 256 x 56 x 56:
    // 16 us, 32 x 512 x 28 x 28: 11.5 us), which is what the staged copy cost before, so the gain is
    // the narrow maps': batch 32, 512 -> 1024 channels 28 x 28 -> 14 x 14 87 -> 75 us; 256 -> 512
    // 56 x 56 -> 28 x 28 and 1024 -> 2048 14 x 14 -> 7 x 7 stay at 78 (the plain products take 58-60).
    const float* sub_src = nullptr;
    float* sub_dst = nullptr;
    int sub_Hin = 0, sub_Win = 0, sub_Hout = 0, sub_Wout = 0, sub_stride = 0;
    if (!explicit_cols && Hf == 1 && Wf == 1 && stride > 1 && pad == 0 &&
        (double)batch * Cin * Hout * Wout * 4.0 + 4096.0 < 2147483648.0 &&
        fits_int((double)Cout * batch * ((double)Hout * Wout + 4.0)) && (double)K * 256 * 4 < 2147483648.0) {
        const size_t bytes = (size_t)batch * Cin * Hout * Wout * sizeof(float);
        char* ws = static_cast<char*>(workspace);
        if (!ws) {
            if ((st = cur().conv.reserve(bytes + 256))) return st;
            ws = static_cast<char*>(cur().conv.ptr);
        } else if (!is_device_pointer(ws)) {
            return fail(CAKE_HIP_ERR_ARG, "workspace must be device memory");
        }
        sub_src = i.dev;
        sub_dst = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
        sub_Hin = Hin; sub_Win = Win; sub_Hout = Hout; sub_Wout = Wout; sub_stride = stride;
        i.dev = sub_dst;
        Win = Hout * Wout; Hin = 1; Wout = Win; Hout = 1; stride = 1;
    }
    // (launched by the route taken, behind its timer's start)
    auto subsample_first = [&](Timer& tm, hipStream_t sm) -> int {
        if (!sub_src) return 0;
        return tm.family(3, [&] {
            return launch_subsample_planes(sub_src, sub_dst, (size_t)batch * Cin, sub_Hin, sub_Win, sub_Hout, sub_Wout, sub_stride, sm);
        });
    };

    // The on-the-fly gather needs byte offsets into the staged input below 2^31
    // (a chunk of 4 columns must lie in one output row: the product is computed with rows of
    // row_n = Wout rounded up to 4 columns, and the columns past Wout are dropped when C is written.
    // That costs row_n / Wout - 1 of extra arithmetic, where the column matrix costs a write and a
    // read of K x N floats, a share of the product's time that falls with Cout: measured on 7x7 to
    // 30x30 maps the padded rows win while (row_n / Wout - 1) * Cout stays below about 60.)
    // The batch is cut into chunks of images when the whole of it does not meet those bounds:
    // images are independent, the chunks run one after the other through the same staged copy.
    const int row_n = (Wout + 3) & ~3;
    auto chunk_fits = [&](int nb) {
        return conv_stage(nb, Cin, Hin, Win, Hf, Wf, stride, pad).elems * 4 + 4096 < 2147483648.0 &&
               fits_int((double)Cout * nb * Hout * row_n) && fits_int((double)Cout * nb * Hout * Wout);
    };
    int chunk = batch;
    while (chunk > 1 && !chunk_fits(chunk)) chunk = (chunk + 1) / 2;
    const int chunks = (batch + chunk - 1) / chunk;
    chunk = (batch + chunks - 1) / chunks;
    const ConvStage sg = conv_stage(chunk, Cin, Hin, Win, Hf, Wf, stride, pad);
    // (a flattened 1 x 1 filter pads at most 3 columns per plane, which always costs less than a
    // column matrix that is a copy of the input)
    const bool flat_1x1 = Hf == 1 && Wf == 1 && stride == 1 && pad == 0;
    const bool implicit = !explicit_cols && (flat_1x1 || (double)(row_n - Wout) / Wout * Cout < 60.0) && chunk_fits(chunk) &&
                          (double)K * 256 * 4 < 2147483648.0;
    Timer timer(stream, seconds);
    // A 1 x 1 convolution at stride 1 without padding is one plain product per image on the input
    // as it lies, out[b] (Cout x HW) = weights (Cout x Cin) . in[b] (Cin x HW): with few input
    // channels and many tiles the images are walked as a batch by the short-K kernel
    // (64 -> 256 channels on 32 x 56 x 56: 50 -> 43 us).
    const int HW = Hout * Wout;
    // (up to 64 channels from 12 tiles per CU on; 65 to 256 channels -- the kernel whose operands go
    // straight into LDS -- from 2 tiles per CU on, for a product that overwrites C, and beyond 160
    // channels only where the planes fill their column tiles to 90 %)
    // Beyond 64 channels the column tiles run across image borders where that saves tiles (a plane's
    // pixels a multiple of 4 but not of 64, the whole input below 2 GiB): 256 -> 1024 channels on
    // 32 x 14 x 14 is 1568 tiles that way and 2048 with every image's last tile a quarter full.
    const bool across_images = K > 64 && HW % 4 == 0 && HW % 64 != 0 && (double)batch * Cin * HW * 4.0 < 2147483648.0 &&
                               fits_int((double)batch * HW);
    const long batch_tiles = (long)((Cout + 63) / 64) * (across_images ? ((long)batch * HW + 63) / 64 : (long)((HW + 63) / 64) * batch);
    const bool batch_pays = K <= 64 ? batch_tiles >= 12L * cur().model.cus
                                    : !accumulate && batch_tiles >= 2L * cur().model.cus &&
                                          (K <= SHORTK_MAX_K || across_images || 10L * ((HW + 63) / 64 * 64 - HW) <= (long)HW);
    if (!explicit_cols && Hf == 1 && Wf == 1 && stride == 1 && pad == 0 &&
        shortk_applies(Cout, HW, K, cur().model.cus, batch, true) && batch_pays &&
        vec4_loadable(w.dev, i.dev, K, HW)) {
        GemmArgs g{};
        g.A = w.dev; g.B = i.dev; g.C = o.dev;
        g.M = Cout; g.N = HW; g.K = K;
        g.lda = K; g.ldb = HW;
        g.ldc = out_nchw ? HW : N;                             // [batch][Cout][HW] or [Cout][batch*HW]
        g.b_batch_stride = (size_t)Cin * HW;
        g.c_batch_stride = out_nchw ? (size_t)Cout * HW : (size_t)HW;
        const int tn = shortk_tile_n(Cout, HW, K, cur().model.cus, batch, true);
        g.tiles_m = (Cout + 63) / 64;
        if (across_images) {
            g.N = batch * HW;
            g.batch_cols = HW;
            g.tiles_n = (g.N + tn - 1) / tn;
        } else {
            g.tiles_n_per_image = (HW + tn - 1) / tn;
            g.tiles_n = g.tiles_n_per_image * batch;
        }
        g.split_k = 1; g.k_per_split = K;
        g.group = g.tiles_m; g.group_along_n = 0;
        g.accumulate = accumulate;
        g_last_conv_route = CAKE_HIP_CONV_SHORTK_BATCH;
        if ((st = timer.start())) return st;
        if ((st = subsample_first(timer, stream))) return st;
        st = timer.family(0, [&] { return launch_sgemm_shortk(g, tn, cur().model.cus, stream); });
        if (st) return st;
        if ((st = timer.stop())) return st;
        return stage_out(o, stream);
    }
    // Stride 1 with whole blocks of 32 channels and maps up to about 60 pixels wide: the input is
    // read where it lies, patches of it per workgroup kept in LDS with the zero padding around them
    // (sgemm_conv_patch.hip) -- no padded copy, no table of tap offsets.
    // That kernel has one tile shape, 256 x 128, and one workgroup per CU.  Where its tiles fill
    // their rows and the machine it is 5-7 % ahead of the staged gather with the planner's choice
    // of tile, from 18 K steps on (batch 32 on 56 x 56 maps, us patch / staged: 64 -> 256 channels
    // 223 / 239, 128 -> 256 418 / 439, 256 -> 256 807 / 856, 256 -> 512 1614 / 1656); where they do not
    // it loses by what is left empty (256 -> 192: 805 / 661; batch 16, 1.5 rounds: 518 / 437; batch
    // 48, 4.6 rounds: 1302 / 1276).  So it is taken when 95 % of the tile rows are in use and its
    // rounds -- whole ones, plus what the planner's cut of a thin last round costs: sub-tiles at a
    // tenth of a round per 256 of them, K slices at a slice's share and a tenth -- come to no more
    // than 1.06 times (1.03 for filters other than 3 x 3, whose K walk keeps its places at run time)
    // the tiles' own count in rounds.
    int patch_rows = 0, patch_pitch = 0;
    bool patch_pays = false;
    {
        const int cus = cur().model.cus;
        const long tiles_m = (Cout + 255) / 256, tiles_n = ((long)batch * Hout * row_n + 127) / 128, tiles = tiles_m * tiles_n;
        const int taps = Hf * Wf, steps = conv_patch_k(Cin, Hf, Wf) / 32;
        const int tile[4] = {256, 128, 32, 0};
        GemmPlan pp;
        if (steps >= 18 && 20L * Cout >= 19L * 256 * tiles_m && tiles >= cus && fits_int((double)batch * Hout * row_n) &&
            plan_gemm(Cout, batch * Hout * row_n, steps * 32, CAKE_HIP_NA, tile, true, cur().model, &pp) == CAKE_HIP_OK) {
            const int tail = pp.pub.tail_tiles;
            double rounds = (double)((tiles - tail + cus - 1) / cus);
            if (tail > 0) {
                const int blocks = steps / taps;                  // K slices are whole blocks of 32 channels
                const int slices = std::min(blocks, std::max(1, pp.pub.tail_split));
                if (taps == 9 && tail * CONV_TAIL_SUBTILES_PER_TILE <= 2 * cus)
                    rounds += 0.1 * ((tail * CONV_TAIL_SUBTILES_PER_TILE + cus - 1) / cus);
                else
                    rounds += slices > 1 ? 1.0 / slices + 0.1 : 1.0;
            }
            patch_pays = rounds <= (Hf == 3 && Wf == 3 ? 1.06 : 1.03) * (double)tiles / cus;
        }
    }
    // CAKE_HIP_CONV_ROUTE=patch takes that kernel wherever its geometry allows, =staged never
    // (for tests and measurements; read at every call)
    const char* route = std::getenv("CAKE_HIP_CONV_ROUTE");
    const bool patch_wanted = route && !std::strcmp(route, "patch") ? true
                              : route && !std::strcmp(route, "staged") ? false : patch_pays;
    if (!explicit_cols && patch_wanted && fits_int((double)Cout * batch * Hout * row_n) && fits_int((double)Cout * conv_patch_lda(Cin, Hf, Wf)) &&
        conv_patch_geometry(batch, Cin, Hin, Win, Hf, Wf, stride, pad, Hout, Wout, &patch_rows, &patch_pitch)) {
        const int taps = Hf * Wf, Kp = conv_patch_k(Cin, Hf, Wf), Np = batch * Hout * row_n, ldw = conv_patch_lda(Cin, Hf, Wf);
        g_last_conv_route = CAKE_HIP_CONV_PATCH;
        // (the kernel built for 3 x 3 filters walks K in the filters' own order and reads them where they lie)
        const bool relay = !conv_patch_reads_filters_in_place(Hf, Wf);
        if (relay && (st = cur().conv_filters.reserve((size_t)Cout * ldw * sizeof(float)))) return st;
        const float* wt = relay ? static_cast<const float*>(cur().conv_filters.ptr) : w.dev;
        const int tile[4] = {256, 128, 32, 0};
        GemmPlan plan;
        if ((st = plan_gemm(Cout, Np, Kp, CAKE_HIP_NA, tile, true, cur().model, &plan))) return fail(st, "conv2d: no plan");
        GemmArgs g{};
        g.A = wt; g.B = nullptr; g.C = o.dev;
        g.M = Cout; g.N = Np; g.K = Kp;
        g.lda = relay ? ldw : Kp; g.ldb = Np; g.ldc = N;
        g.tiles_m = plan.pub.tiles_m; g.tiles_n = plan.pub.tiles_n;
        g.split_k = 1; g.k_per_split = Kp;
        g.group = plan.pub.group; g.group_along_n = plan.group_along_n;
        g.accumulate = accumulate;
        // tiles of a thin last round are cut along K in whole channel blocks
        // -- or, under 3 x 3 filters, not cut along K at all: 16 workgroups per tail tile compute
        // 64 rows x 32 pixels each over the whole K, no partial sums in memory and no second kernel
        // (CAKE_HIP_CONV_TAIL=slices|subtiles overrides the choice; for tests and measurements)
        int grid = g.tiles_m * g.tiles_n;
        const char* tail_env = std::getenv("CAKE_HIP_CONV_TAIL");
        const bool subtiles_fit = taps == 9 && plan.pub.tail_tiles > 0;
        const bool subtiles = tail_env && !std::strcmp(tail_env, "slices") ? false
                              : tail_env && !std::strcmp(tail_env, "subtiles") ? subtiles_fit
                              : subtiles_fit && plan.pub.tail_tiles * CONV_TAIL_SUBTILES_PER_TILE <= 2 * cur().model.cus;
        if (subtiles) {
            g.tail_tiles = plan.pub.tail_tiles;
            g.tail_split = CONV_TAIL_SUBTILES_PER_TILE;
            g.tail_k_per_split = Kp;
            g.conv.tail_mode = CONV_TAIL_SUBTILES;
            grid += g.tail_tiles * (CONV_TAIL_SUBTILES_PER_TILE - 1);
        } else if (plan.pub.tail_tiles > 0) {
            const int block_k = 32 * taps, blocks = Kp / block_k;
            const int per = (blocks + plan.pub.tail_split - 1) / plan.pub.tail_split;
            const int slices = (blocks + per - 1) / per;
            if (slices > 1) {
                g.tail_tiles = plan.pub.tail_tiles;
                g.tail_split = slices;
                g.tail_k_per_split = per * block_k;
                g.conv.tail_mode = CONV_TAIL_BLOCKS;
                if ((st = scratch_space(cur().splitk, (size_t)g.tail_tiles * slices * 256 * 128 * sizeof(float), &g.tail_partial)))
                    return st;
                grid += g.tail_tiles * (slices - 1);
            }
        }
        ConvGeom& cv = g.conv;
        cv.in = i.dev;
        cv.in_bytes = (unsigned)(in_elems * 4);
        cv.Cin = Cin; cv.Hout = Hout; cv.Wout = Wout; cv.row_n = row_n;
        cv.out_nchw = out_nchw ? 1 : 0;
        cv.batch = batch; cv.Hin = Hin; cv.Win = Win; cv.pad = pad; cv.Hf = Hf; cv.Wf = Wf;
        cv.patch_rows = patch_rows; cv.patch_pitch = patch_pitch;
        cv.stream_out = (reinterpret_cast<uintptr_t>(o.dev) & 127) == 0 && (out_nchw ? (Hout * Wout) % 32 == 0 : N % 32 == 0);
        cv.by_row_n = FastDiv::make(row_n); cv.by_hout = FastDiv::make(Hout); cv.by_vrows = FastDiv::make(Hin + 2 * pad);
        cv.by_channel_chunks = FastDiv::make(patch_rows * ((Win + 3) / 4)); cv.by_row_chunks = FastDiv::make((Win + 3) / 4);
        cv.margin_chunks = patch_pitch / 4 - (Win + 3) / 4;
        cv.by_margin_chunks = FastDiv::make(cv.margin_chunks); cv.by_channel_margin_chunks = FastDiv::make(patch_rows * cv.margin_chunks);
        if ((st = timer.start())) return st;
        if (relay && (st = timer.family(3, [&] { return launch_conv_filter_relayout(w.dev, static_cast<float*>(cur().conv_filters.ptr), Cout, Cin, Hf, Wf, stream); }))) return st;
        if ((st = timer.family(0, [&] { return launch_sgemm_conv_patch(g, grid, stream); }))) return st;
        if (g.tail_partial && (st = timer.family(1, [&] { return launch_tail_reduce(plan.tile_id, g, stream); }))) return st;
        if ((st = timer.stop())) return st;
        return stage_out(o, stream);
    }
    if (implicit) {
        g_last_conv_route = CAKE_HIP_CONV_GATHER;
        float* staged = nullptr;
        if (sg.copy) {
            char* ws = static_cast<char*>(workspace);
            if (!ws) {
                if ((st = cur().conv.reserve((size_t)sg.elems * 4 + 256))) return st;
                ws = static_cast<char*>(cur().conv.ptr);
            } else if (!is_device_pointer(ws)) {
                return fail(CAKE_HIP_ERR_ARG, "workspace must be device memory");
            }
            staged = reinterpret_cast<float*>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
        }
        if ((st = cur().conv_taps.reserve(((size_t)K + CONV_TAP_TABLE_EXTRA) * sizeof(int)))) return st;
        int* taps = static_cast<int*>(cur().conv_taps.ptr);
        if ((st = timer.start())) return st;
        if ((st = subsample_first(timer, stream))) return st;
        const bool one_by_one = Hf == 1 && Wf == 1;   // row k is channel k: no table of tap offsets
        // the table of tap offsets is written by the launch that stages the first chunk of images,
        // or by a launch of its own where the input is read as it lies
        bool table_due = !one_by_one;
        if (table_due && !sg.copy) {
            st = timer.family(3, [&] {
                return launch_conv_tap_table(taps, K, CONV_TAP_TABLE_EXTRA, sg.Hs, sg.pitch, sg.Wq, Hf, Wf, stride, sg.RH, stream);
            });
            if (st) return st;
            table_due = false;
        }
        const size_t HW = (size_t)Hout * Wout;
        for (int b0 = 0; b0 < batch; b0 += chunk) {
            const int nb = batch - b0 < chunk ? batch - b0 : chunk;
            const float* src = i.dev + (size_t)b0 * Cin * Hin * Win;
            if (sg.copy) {
                st = timer.family(3, [&] {
                    return launch_conv_stage_input(src, staged, (size_t)nb * Cin, Hin, Win, pad, stride, sg.RH, sg.PW, sg.Hs,
                                                   sg.Wq, table_due ? taps : nullptr, K, CONV_TAP_TABLE_EXTRA, Hf, Wf, stream);
                });
                if (st) return st;
                table_due = false;
            }
            ConvGeom cv{};
            cv.in = sg.copy ? staged : src;
            cv.in_bytes = (unsigned)((double)nb * Cin * sg.Hs * sg.pitch * 4);
            cv.Cin = Cin; cv.plane_rows = sg.Hs; cv.pitch = sg.pitch; cv.row_step = sg.RH;
            cv.Hout = Hout; cv.Wout = Wout; cv.row_n = row_n;
            cv.tap_table = taps;
            cv.tap_stride = sg.Hs * sg.pitch * 4;   // 1 x 1 filters: channel k starts k planes into the image
            cv.out_nchw = out_nchw ? 1 : 0;
            // [batch][Cout][HW]: the chunk's images are contiguous; [Cout][batch*HW]: its columns are
            float* dst = o.dev + (out_nchw ? (size_t)b0 * Cout * HW : (size_t)b0 * HW);
            const int Np = nb * Hout * row_n;
            st = run_gemm(w.dev, nullptr, dst, Cout, Np, K, K, Np, N, CAKE_HIP_NA, accumulate, nullptr, LOAD_VEC4,
                          one_by_one ? LOAD_IM2COL_1X1 : LOAD_IM2COL_ROW, stream, timer, &cv);
            if (st) return st;
        }
        if ((st = timer.stop())) return st;
        return stage_out(o, stream);
    }

    if (!fits_int(K_d * ncols_d) || !fits_int(Cout * ncols_d) || !fits_int(in_elems) || K > 65535)
        return fail(CAKE_HIP_ERR_RANGE, "column matrix %gx%g out of range", K_d, ncols_d);
    if (sub_src) return fail(CAKE_HIP_ERR_RANGE, "conv2d: a subsampled 1 x 1 layer that the gather does not take");   // (its bounds above rule this out)
    g_last_conv_route = CAKE_HIP_CONV_TWO_STEP;
    char* ws = static_cast<char*>(workspace);
    if (!ws) {
        if ((st = cur().conv.reserve(cake_hip_conv2d_workspace(batch, Cin, Hin, Win, Cout, Hf, Wf, stride, pad)))) return st;
        ws = static_cast<char*>(cur().conv.ptr);
    } else if (!is_device_pointer(ws)) {
        return fail(CAKE_HIP_ERR_ARG, "workspace must be device memory");
    }
    ws = reinterpret_cast<char*>((reinterpret_cast<uintptr_t>(ws) + 255) & ~(uintptr_t)255);
    float* cols = reinterpret_cast<float*>(ws);
    float* cn = cols + (size_t)K * N;  // [Cout][N] product, used only for NCHW output

    if ((st = timer.start())) return st;
    st = timer.family(3, [&] {
        return launch_im2col(i.dev, cols, batch, Cin, Hin, Win, Hf, Wf, Hout, Wout, stride, pad, stream);
    });
    if (st) return st;
    if (accumulate) out_nchw = 0;   // a single image: [Cout][HW] is its NCHW layout
    const bool vec = vec4_loadable(w.dev, cols, K, N);
    const int mode = vec ? LOAD_VEC4 : LOAD_SCALAR;
    // NCHW output: where an image's pixels are a multiple of 4 (its 16-byte chunks of columns then
    // never run from one image into the next) the GEMM's epilogue (and its slice reductions) write
    // the layout themselves, an image seen as one row of Hout * Wout pixels; otherwise the product
    // goes to [Cout][N] first and a layout pass follows
    ConvGeom nchw{};
    const bool fused_nchw = out_nchw && vec && (Hout * Wout) % 4 == 0 && Cout > 48 && K > 64;   // (the macro-tile kernel's shapes)
    if (fused_nchw) {
        nchw.in = cols;
        nchw.Hout = 1; nchw.Wout = Hout * Wout; nchw.row_n = Hout * Wout;
        nchw.out_nchw = 1;
        out_nchw = 0;
    }
    float* prod = out_nchw ? cn : o.dev;
    st = run_gemm(w.dev, cols, prod, Cout, N, K, K, N, N, CAKE_HIP_NA, accumulate, nullptr, mode,
                  fused_nchw ? LOAD_VEC4_NCHW : mode, stream, timer, fused_nchw ? &nchw : nullptr);
    if (st) return st;
    if (out_nchw) {
        st = timer.family(3, [&] { return launch_cn_to_nchw(cn, o.dev, batch, Cout, Hout * Wout, stream); });
        if (st) return st;
    }
    if ((st = timer.stop())) return st;
    return stage_out(o, stream);
}

int cake_hip_conv2d(const float* in, const float* weights, float* out, int batch, int Cin, int Hin,
                    int Win, int Cout, int Hf, int Wf, int stride, int pad, int out_nchw,
                    void* workspace, void* stream, double* seconds)
{
    return conv2d_common(in, weights, out, batch, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, out_nchw,
                         workspace, stream, seconds, 0);
}

int cake_hip_conv2d_im2col(const float* in, const float* weights, float* out, int batch, int Cin,
                           int Hin, int Win, int Cout, int Hf, int Wf, int stride, int pad,
                           int out_nchw, void* workspace, void* stream, double* seconds)
{
    return conv2d_common(in, weights, out, batch, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, out_nchw,
                         workspace, stream, seconds, 1);
}

int cake_hip_sconv(const float* filters, const float* in, float* out, int Wf, int Hf, int Win, int Hin,
                   int Wout, int Hout, int Cin, int Cout, int stride, void* stream, double* seconds)
{
    if (seconds) *seconds = 0;
    int ho = 0, wo = 0;
    if (Cin <= 0 || Cout <= 0 || Hin <= 0 || Win <= 0 || conv_out_dims(Hin, Win, Hf, Wf, stride, 0, &ho, &wo))
        return fail(CAKE_HIP_ERR_ARG, "bad convolution geometry");
    if (ho != Hout || wo != Wout)
        return fail(CAKE_HIP_ERR_ARG, "a %dx%d filter at stride %d maps %dx%d to %dx%d, not %dx%d", Hf, Wf, stride, Hin,
                    Win, ho, wo, Hout, Wout);
    return conv2d_common(in, filters, out, 1, Cin, Hin, Win, Cout, Hf, Wf, stride, 0, 0, nullptr, stream, seconds, 0, 1);
}

// ---- filters in the reference's packed layout ------------------------------------------

static int filter_geom(int Cout, int Cin, int taps, int p, const cake_hip_blk_dims_t* d, const cake_hip_cpu_cntx_t* cx,
                       PackGeom* g)
{
    int st = check_geom(d, cx, p, CAKE_HIP_KMN);
    if (st) return st;
    if (Cout <= 0 || Cin <= 0 || taps <= 0) return fail(CAKE_HIP_ERR_ARG, "empty filters");
    *g = make_geom(Cout, 0, Cin, p, d, cx, CAKE_HIP_KMN);
    // the block dims must be those of this Cout, Cin and p (init_block_dims_conv): the index map reads them
    if (d->sch != CAKE_HIP_KMN || padded_rows(*g) != d->M_padded || d->M_padded < Cout ||
        d->Kb != Cin / d->k_c + (Cin % d->k_c != 0) || (d->k_pad && d->k_c1 != Cin % d->k_c))
        return fail(CAKE_HIP_ERR_ARG, "block dims do not belong to %d x %d filters on %d cores", Cout, Cin, p);
    if (!fits_int((double)d->M_padded * Cin * taps)) return fail(CAKE_HIP_ERR_RANGE, "packed filters exceed 2^31 elements");
    return CAKE_HIP_OK;
}

size_t cake_hip_packed_filters_size(int Cout, int Cin, int taps, int p, const cake_hip_blk_dims_t* d,
                                    const cake_hip_cpu_cntx_t* cx)
{
    PackGeom g;
    if (filter_geom(Cout, Cin, taps, p, d, cx, &g)) return 0;
    return (size_t)d->M_padded * Cin * taps * sizeof(float);
}

int cake_hip_pack_filters(const float* filters, float* filters_p, int Cout, int Cin, int taps, int p,
                          const cake_hip_blk_dims_t* d, const cake_hip_cpu_cntx_t* cx, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    PackGeom g;
    int st = filter_geom(Cout, Cin, taps, p, d, cx, &g);
    if (st) return st;
    if (!filters || !filters_p) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);
    Operand in, out;
    if ((st = stage_in(filters, (size_t)Cout * Cin * taps * 4, 0, true, &in))) return st;
    if ((st = stage_in(filters_p, (size_t)d->M_padded * Cin * taps * 4, 1, false, &out))) return st;
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if ((st = timer.family(4, [&] { return launch_filter_layout(in.dev, out.dev, g, Cout, Cin, taps, 1, stream); }))) return st;
    if ((st = timer.stop())) return st;
    return stage_out(out, stream);
}

int cake_hip_sconv_packed(const float* filters_p, const float* in, float* out, int Wf, int Hf, int Win, int Hin,
                          int Wout, int Hout, int Cin, int Cout, int stride, int p, const cake_hip_blk_dims_t* d,
                          const cake_hip_cpu_cntx_t* cx, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    if (Wf <= 0 || Hf <= 0 || !fits_int((double)Wf * Hf)) return fail(CAKE_HIP_ERR_ARG, "bad convolution geometry");
    const int taps = Wf * Hf;
    PackGeom g;
    int st = filter_geom(Cout, Cin, taps, p, d, cx, &g);
    if (st) return st;
    if (!filters_p) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);   // held across the unpacking and the convolution
    hipStream_t stream = pick_stream(stream_);
    Operand fp;
    // (slot 3: the convolution stages its own operands in slots 0 to 2)
    if ((st = stage_in(filters_p, (size_t)d->M_padded * Cin * taps * 4, 3, true, &fp))) return st;
    if ((st = cur().unpacked.reserve((size_t)Cout * Cin * taps * sizeof(float)))) return st;
    float* plain = static_cast<float*>(cur().unpacked.ptr);
    // the filters go back to [Cout][Cin][Hf][Wf] (a few megabytes at most), then the convolution runs as cake_hip_sconv does
    hipError_t e = launch_filter_layout(fp.dev, plain, g, Cout, Cin, taps, 0, stream);
    if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "filter unpack launch failed: %s", hipGetErrorString(e));
    return cake_hip_sconv(plain, in, out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, stride, stream_, seconds);
}

int cake_hip_transpose(const float* src, float* dst, int rows, int cols, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    if (rows < 0 || cols < 0) return fail(CAKE_HIP_ERR_ARG, "negative dimension");
    if (rows == 0 || cols == 0) return CAKE_HIP_OK;
    if (!src || !dst) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if (src == dst) return fail(CAKE_HIP_ERR_ARG, "transpose in place is not supported");
    if (!fits_int((double)rows * cols)) return fail(CAKE_HIP_ERR_RANGE, "matrix of %dx%d exceeds 2^31 elements", rows, cols);
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);
    Operand in, out;
    const size_t bytes = (size_t)rows * cols * 4;
    if ((st = stage_in(src, bytes, 0, true, &in))) return st;
    if ((st = stage_in(dst, bytes, 1, false, &out))) return st;
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    st = timer.family(4, [&] { return launch_transpose(in.dev, out.dev, rows, cols, stream); });
    if (st) return st;
    if ((st = timer.stop())) return st;
    return stage_out(out, stream);
}

static int linear_dims_ok(int M, int N, int K)
{
    if (M < 0 || N < 0 || K < 0) return fail(CAKE_HIP_ERR_ARG, "negative dimension");
    if (!fits_int((double)M * K) || !fits_int((double)K * N) || !fits_int((double)M * N))
        return fail(CAKE_HIP_ERR_RANGE, "operand of %dx%dx%d exceeds 2^31 elements", M, K, N);
    return CAKE_HIP_OK;
}

// C = A.B on device operands with the planner's choice of everything; K == 0 gives C = bias or 0.
static int linear_gemm(const float* A, const float* B, float* C, int M, int N, int K, const float* col_bias,
                       hipStream_t stream, Timer& timer)
{
    if (M == 0 || N == 0) return CAKE_HIP_OK;
    if (K == 0) {
        hipError_t e = launch_splitk_reduce(nullptr, C, M, N, N, 0, 0, stream, nullptr, col_bias);
        return e == hipSuccess ? CAKE_HIP_OK : fail(CAKE_HIP_ERR_HIP, "fill failed: %s", hipGetErrorString(e));
    }
    const int mode = vec4_loadable(A, B, K, N) ? LOAD_VEC4 : LOAD_SCALAR;
    return run_gemm(A, B, C, M, N, K, K, N, N, CAKE_HIP_NA, 0, nullptr, mode, mode,
                    stream, timer, nullptr, col_bias);
}

// C[M][N] = (accumulate ? C : 0) + X[M][K] . W[N][K]^T (+ bias[N] on every row) on device operands,
// W read as it lies: a single row of X (or of W) is a row-major matrix-vector product, two rows
// against a mid-size W the two-vector sweep, up to 32 rows of either the streaming kernel, the
// rest the macro-tile kernel with 16-byte loads along k on both sides.  Only rows of 2^21 floats
// and more, beyond that kernel's 32-bit offsets, go through a transposed copy of W.
// tile_override != nullptr forces the macro-tile kernel.
static int gemm_nt(const float* X, const float* W, float* C, int M, int N, int K, int accumulate,
                   const int* tile_override, const float* bias, hipStream_t stream, Timer& timer)
{
    int st;
    if (K == 0) {
        if (accumulate && !bias) return CAKE_HIP_OK;
        hipError_t e = launch_splitk_reduce(nullptr, C, M, N, N, 0, accumulate, stream, nullptr, bias);
        return e == hipSuccess ? CAKE_HIP_OK : fail(CAKE_HIP_ERR_HIP, "fill failed: %s", hipGetErrorString(e));
    }
    const int cus = cur().model.cus;
    if ((M == 1 || N == 1) && !tile_override && !(bias && accumulate)) {
        // y = W . x (one row of X), or C[:, 0] = X . w (one row of W): the matrix is read row-major at
        // 7.2 TB/s where the streaming kernel reaches 6.4.  A bias goes first and the product is
        // added to it, which rounds as fl(sum + bias) does.
        const float* mat = M == 1 ? W : X;
        const float* vec = M == 1 ? X : W;
        const int rows = M == 1 ? N : M;
        const size_t floats = sgemv_rowmajor_scratch_floats(rows, K, cus);
        if (floats && (st = cur().gemv.reserve(floats * sizeof(float)))) return st;
        float* scratch = static_cast<float*>(cur().gemv.ptr);
        if (bias) {   // C[m][n] = bias[n], by a kernel (no copy or memset node for a captured graph)
            hipError_t e = launch_splitk_reduce(nullptr, C, M, N, N, 0, 0, stream, nullptr, bias);
            if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "fill failed: %s", hipGetErrorString(e));
        }
        return timer.family(2, [&] {
            return launch_sgemv_rowmajor(mat, vec, C, rows, K, bias ? 1 : accumulate, scratch, cus, stream);
        });
    }
    if (!tile_override && !accumulate && fewrows_nt_applies(M, N, K, K, K, false) &&
        sgemv_rowmajor_multi_applies(N, K, M, K, W, X, cus)) {
        // two rows against a mid-size W: one pass of the matrix-vector sweep over W serves both
        return timer.family(2, [&] { return launch_sgemv_rowmajor_multi(W, X, C, bias, N, K, M, K, N, stream); });
    }
    const bool few_x = !tile_override && fewrows_nt_applies(M, N, K, K, K, false);
    const bool few_w = !tile_override && !few_x && fewrows_nt_applies(N, M, K, K, K, false);
    if (few_x || few_w) {
        // a few rows on one side: the other operand is streamed once as it lies
        const int slices = few_x ? fewrows_nt_slices(M, N, K, K, false, cus) : fewrows_nt_slices(N, M, K, K, false, cus);
        float* partial = nullptr;
        if (slices > 1) {
            if ((st = scratch_space(cur().splitk, (size_t)slices * M * N * sizeof(float), &partial))) return st;
        }
        return timer.family(0, [&] {
            return few_x ? launch_sgemm_fewrows_nt(X, W, C, partial, M, N, K, K, K, N, false, false, accumulate, bias, cus, stream)
                         : launch_sgemm_fewrows_nt(W, X, C, partial, N, M, K, K, K, N, false, true, accumulate, bias, cus, stream);
        });
    }
    if ((double)K * 256 * 4 < 2147483648.0)
        return run_gemm(X, W, C, M, N, K, K, K, N, CAKE_HIP_NA, accumulate, tile_override, LOAD_VEC4, LOAD_VEC4_T,
                        stream, timer, nullptr, bias);
    if ((st = cur().linear.reserve((size_t)N * K * 4))) return st;
    float* wt = static_cast<float*>(cur().linear.ptr);
    st = timer.family(4, [&] { return launch_transpose(W, wt, N, K, stream); });
    if (st) return st;
    const int mode = vec4_loadable(X, wt, K, N) ? LOAD_VEC4 : LOAD_SCALAR;
    return run_gemm(X, wt, C, M, N, K, K, N, N, CAKE_HIP_NA, accumulate, tile_override, mode, mode, stream, timer,
                    nullptr, bias);
}

int cake_hip_sgemm_nt(const float* A, const float* Bt, float* C, int M, int N, int K, int accumulate,
                      const int* tile_override, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    if (M < 0 || N < 0 || K < 0) return fail(CAKE_HIP_ERR_ARG, "negative dimension");
    if (M == 0 || N == 0) return CAKE_HIP_OK;
    if (!C || (K > 0 && (!A || !Bt))) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if (!fits_int((double)M * K) || !fits_int((double)K * N) || !fits_int((double)M * N))
        return fail(CAKE_HIP_ERR_RANGE, "operand of %dx%dx%d exceeds 2^31 elements", M, K, N);
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);
    Operand a, b, c;
    if ((st = stage_in(A, (size_t)M * K * 4, 0, true, &a))) return st;
    if ((st = stage_in(Bt, (size_t)N * K * 4, 1, true, &b))) return st;
    if ((st = stage_in(C, (size_t)M * N * 4, 2, accumulate != 0, &c))) return st;
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if ((st = gemm_nt(a.dev, b.dev, c.dev, M, N, K, accumulate, tile_override, nullptr, stream, timer))) return st;
    if ((st = timer.stop())) return st;
    return stage_out(c, stream);
}

int cake_hip_linear_forward(const float* x, const float* w, const float* bias, float* y, int M, int N,
                            int K, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    int st = linear_dims_ok(M, N, K);
    if (st) return st;
    if (M == 0 || N == 0) return CAKE_HIP_OK;
    if (!y || (K > 0 && (!x || !w))) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand xo, wo, bo, yo;
    if ((st = stage_in(x, (size_t)M * K * 4, 0, true, &xo))) return st;
    if ((st = stage_in(w, (size_t)N * K * 4, 1, true, &wo))) return st;
    if (bias && (st = stage_in(bias, (size_t)N * 4, 2, true, &bo))) return st;
    if ((st = stage_in(y, (size_t)M * N * 4, 3, false, &yo))) return st;
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if ((st = gemm_nt(xo.dev, wo.dev, yo.dev, M, N, K, 0, nullptr, bias ? bo.dev : nullptr, stream, timer))) return st;
    if ((st = timer.stop())) return st;
    return stage_out(yo, stream);
}

int cake_hip_linear_forward_wt(const float* x, const float* wt, const float* bias, float* y, int M, int N,
                               int K, void* stream_, double* seconds)
{
    if (seconds) *seconds = 0;
    int st = linear_dims_ok(M, N, K);
    if (st) return st;
    if (M == 0 || N == 0) return CAKE_HIP_OK;
    if (!y || (K > 0 && (!x || !wt))) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand xo, wo, bo, yo;
    if ((st = stage_in(x, (size_t)M * K * 4, 0, true, &xo))) return st;
    if ((st = stage_in(wt, (size_t)N * K * 4, 1, true, &wo))) return st;
    if (bias && (st = stage_in(bias, (size_t)N * 4, 2, true, &bo))) return st;
    if ((st = stage_in(y, (size_t)M * N * 4, 3, false, &yo))) return st;
    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if ((st = linear_gemm(xo.dev, wo.dev, yo.dev, M, N, K, bias ? bo.dev : nullptr, stream, timer))) return st;
    if ((st = timer.stop())) return st;
    return stage_out(yo, stream);
}

int cake_hip_linear_backward(const float* grad_y, const float* x, const float* w, float* grad_x,
                             float* grad_w, float* grad_bias, int M, int N, int K, void* stream_,
                             double* seconds)
{
    if (seconds) *seconds = 0;
    int st = linear_dims_ok(M, N, K);
    if (st) return st;
    if (!grad_y && M > 0 && N > 0) return fail(CAKE_HIP_ERR_ARG, "NULL grad_y");
    if (grad_x && !w && N > 0) return fail(CAKE_HIP_ERR_ARG, "grad_x needs w");
    if (grad_w && !x && M > 0) return fail(CAKE_HIP_ERR_ARG, "grad_w needs x");
    if ((st = ensure_init())) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);

    Operand go, xo, wo, gxo, gwo, gbo;
    if ((st = stage_in(grad_y, (size_t)M * N * 4, 0, true, &go))) return st;
    if (grad_w && (st = stage_in(x, (size_t)M * K * 4, 1, true, &xo))) return st;
    if (grad_x && (st = stage_in(w, (size_t)N * K * 4, 2, true, &wo))) return st;
    if (grad_x && (st = stage_in(grad_x, (size_t)M * K * 4, 3, false, &gxo))) return st;
    if (grad_w && (st = stage_in(grad_w, (size_t)N * K * 4, 4, false, &gwo))) return st;
    if (grad_bias && (st = stage_in(grad_bias, (size_t)N * 4, 5, false, &gbo))) return st;
    // workspace: grad_y transposed (N x M), then a vector of M ones, then the GEMV's slice partials
    const size_t gt_floats = grad_w ? (((size_t)M * N + 63) & ~(size_t)63) : 0;
    const size_t ones_floats = grad_bias ? (((size_t)M + 63) & ~(size_t)63) : 0;
    const size_t gemv_floats = grad_bias && M > 0 && N > 0 ? sgemv_colmajor_scratch_floats(N, M, cur().model.cus) : 0;
    if ((st = cur().linear.reserve((gt_floats + ones_floats + gemv_floats) * 4 + 256))) return st;
    float* gt = static_cast<float*>(cur().linear.ptr);
    float* ones = gt + gt_floats;
    float* gemv_scratch = ones + ones_floats;

    Timer timer(stream, seconds);
    if ((st = timer.start())) return st;
    if (grad_x)  // grad_x[M][K] = grad_y[M][N] . w[N][K]   (src/linear.cpp:58-72)
        if ((st = linear_gemm(go.dev, wo.dev, gxo.dev, M, K, N, nullptr, stream, timer))) return st;
    if (grad_w) {  // grad_w[N][K] = grad_y^T[N][M] . x[M][K]   (src/linear.cpp:74-90)
        if (M > 0 && N > 0) {
            st = timer.family(4, [&] { return launch_transpose(go.dev, gt, M, N, stream); });
            if (st) return st;
        }
        if ((st = linear_gemm(gt, xo.dev, gwo.dev, N, K, M, nullptr, stream, timer))) return st;
    }
    if (grad_bias && N > 0) {  // column sums of grad_y   (src/linear.cpp:92-93)
        if (M == 0) {
            hipError_t e = launch_fill_value(gbo.dev, (size_t)N, 0.f, stream);
            if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "fill failed: %s", hipGetErrorString(e));
        } else {
            // grad_y read as a column-major N x M matrix times a vector of ones
            st = timer.family(2, [&] {
                hipError_t e = launch_fill_value(ones, (size_t)M, 1.f, stream);
                if (e != hipSuccess) return e;
                return launch_sgemv_colmajor(go.dev, ones, gbo.dev, N, M, 0, gemv_scratch, cur().model.cus, stream);
            });
            if (st) return st;
        }
    }
    if ((st = timer.stop())) return st;
    if (grad_x && (st = stage_out(gxo, stream))) return st;
    if (grad_w && (st = stage_out(gwo, stream))) return st;
    if (grad_bias && (st = stage_out(gbo, stream))) return st;
    return CAKE_HIP_OK;
}

// ---- autotuner -----------------------------------------------------------------------

int cake_hip_autotune(int M, int N, int K, double budget_seconds, cake_hip_plan_t* best_plan,
                      double* best_seconds, double* default_seconds)
{
    if (best_seconds) *best_seconds = 0;
    if (default_seconds) *default_seconds = 0;
    if (M <= 0 || N <= 0 || K <= 0) return fail(CAKE_HIP_ERR_ARG, "autotune needs a non-empty product");
    if (!fits_int((double)M * K) || !fits_int((double)K * N) || !fits_int((double)M * N))
        return fail(CAKE_HIP_ERR_RANGE, "operand of %dx%dx%d exceeds 2^31 elements", M, K, N);
    if (!(budget_seconds > 0)) budget_seconds = 2.0;
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = cur().own_stream;

    // synthetic operands in the staging slots (what a host caller's operands would use)
    if ((st = cur().stage[0].reserve((size_t)M * K * 4))) return st;
    if ((st = cur().stage[1].reserve((size_t)K * N * 4))) return st;
    if ((st = cur().stage[2].reserve((size_t)M * N * 4))) return st;
    float* A = static_cast<float*>(cur().stage[0].ptr);
    float* B = static_cast<float*>(cur().stage[1].ptr);
    float* C = static_cast<float*>(cur().stage[2].ptr);
    HIP_TRY(launch_fill_uniform(A, (size_t)M * K, 1, stream));
    HIP_TRY(launch_fill_uniform(B, (size_t)K * N, 2, stream));
    const bool vec = vec4_loadable(A, B, K, N);
    const int mode = vec ? LOAD_VEC4 : LOAD_SCALAR;

    // time one explicit choice: a warm-up launch, then the fastest of three batches of
    // back-to-back launches (clock ramps and other tenants only ever make a batch slower)
    auto measure = [&](const TunedChoice* c, double* secs) -> int {
        Timer untimed(stream, nullptr);
        double est = 0, best_batch = 1e30;
        for (int pass = 0; pass < 4; ++pass) {
            const int reps = pass == 0 ? 1 : (est < 2e-4 ? 20 : est < 5e-3 ? 5 : 2);
            HIP_TRY(hipEventRecord(cur().ev[0], stream));
            for (int r = 0; r < reps; ++r) {
                int e = run_gemm(A, B, C, M, N, K, K, N, N, CAKE_HIP_NA, 0, nullptr, mode, mode, stream, untimed, nullptr, nullptr, c);
                if (e) return e;
            }
            HIP_TRY(hipEventRecord(cur().ev[1], stream));
            HIP_TRY(hipEventSynchronize(cur().ev[1]));
            float ms = 0;
            HIP_TRY(hipEventElapsedTime(&ms, cur().ev[0], cur().ev[1]));
            est = ms * 1e-3 / reps;
            if (pass > 0 && est < best_batch) best_batch = est;
        }
        *secs = best_batch;
        return CAKE_HIP_OK;
    };

    // the model's own choice first: it is the baseline and the fallback
    GemmPlan model_plan;
    {
        const int any[4] = {0, 0, 0, 0};
        if ((st = plan_gemm(M, N, K, CAKE_HIP_NA, any, vec, cur().model, &model_plan))) return st;
    }
    TunedChoice best{model_plan.tile_id, model_plan.pub.split_k, 1, 0.0};
    if ((st = measure(&best, &best.seconds))) return st;
    // a product with a few rows or columns runs on a streaming kernel unless a tile is measured
    // to beat it: that kernel is the default here, and the table keeps no entry when it wins
    // (the same holds for the short-K kernel that walks over tiles)
    const bool streaming = vec && (fewrows_applies(M, N, K, K, N) || fewrows_nt_applies(N, M, K, N, K, true) ||
                                   shortk_applies(M, N, K, cur().model.cus));
    double streaming_seconds = 0;
    if (streaming) {
        tune_erase(M, N, K, true);
        if ((st = measure(nullptr, &streaming_seconds))) return st;
    }
    if (default_seconds) *default_seconds = streaming ? streaming_seconds : best.seconds;

    const auto t0 = std::chrono::steady_clock::now();
    auto spent = [&] { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count(); };
    bool out_of_time = false;
    for (int id = 0; id < TILE_COUNT && !out_of_time; ++id) {
        const TileInfo& t = tile_info(id);
        if (t.lds_bytes > cur().model.lds_per_cu) continue;
        const int max_split = std::max(1, K / (4 * t.bk));
        for (int split = 1; split <= max_split && split <= 1024; split *= 2) {
            for (int tail = (split == 1 ? 1 : 0); tail >= 0; --tail) {
                if (id == model_plan.tile_id && split == model_plan.pub.split_k && (tail == 1 || split > 1))
                    continue;  // the baseline itself
                if (spent() > budget_seconds) { out_of_time = true; break; }
                TunedChoice c{id, split, tail, 0.0};
                if (tail) {  // only a distinct candidate when the tile count leaves a thin round
                    GemmPlan probe;
                    if (plan_gemm_choice(M, N, K, CAKE_HIP_NA, c, vec, cur().model, &probe) || probe.pub.tail_tiles == 0)
                        continue;
                }
                // skip candidates the model already puts far behind: a split whose slices alone outweigh the product
                if ((double)split * M * N * 4.0 > 64.0 * ((double)M * K + (double)K * N) * 4.0 && split > 1) continue;
                double secs = 0;
                if ((st = measure(&c, &secs))) return st;
                c.seconds = secs;
                if (secs < best.seconds) best = c;
            }
            if (out_of_time) break;
        }
    }
    // the default was timed first, on a device that may not have reached its clocks yet: time it
    // once more now, so that it is not beaten by a candidate that merely ran later
    {
        double again = 0;
        if (streaming) {
            if ((st = measure(nullptr, &again))) return st;
            if (again < streaming_seconds) streaming_seconds = again;
        } else {
            TunedChoice model_choice{model_plan.tile_id, model_plan.pub.split_k, 1, 0.0};
            if ((st = measure(&model_choice, &again))) return st;
            if (again < best.seconds) {
                best = model_choice;
                best.seconds = again;
            }
            if (default_seconds && again < *default_seconds) *default_seconds = again;
        }
        if (streaming && default_seconds) *default_seconds = streaming_seconds;
    }
    if (streaming && streaming_seconds <= best.seconds) {
        if (best_seconds) *best_seconds = streaming_seconds;
        if (best_plan) {
            GemmPlan plan;
            if ((st = plan_gemm(M, N, K, CAKE_HIP_NA, nullptr, vec, cur().model, &plan))) return st;
            *best_plan = plan.pub;
            best_plan->kernel = kernel_family(M, N, K, false, vec);
        }
        return CAKE_HIP_OK;
    }
    tune_store(M, N, K, vec, best);
    if (vec) {
        // the same tile serves callers whose operands are not 16-byte loadable, unless measured separately
        TunedChoice other;
        if (!tune_lookup(M, N, K, false, &other)) tune_store(M, N, K, false, best);
    }
    if (best_seconds) *best_seconds = best.seconds;
    if (best_plan) {
        GemmPlan plan;
        if ((st = plan_gemm(M, N, K, CAKE_HIP_NA, nullptr, vec, cur().model, &plan))) return st;
        *best_plan = plan.pub;
        best_plan->kernel = kernel_family(M, N, K, false, vec);
    }
    return CAKE_HIP_OK;
}

int cake_hip_tune_save(const char* path)
{
    if (!path) return fail(CAKE_HIP_ERR_ARG, "path is NULL");
    const int st = tune_save(path);
    return st ? fail(st, "cannot write %s", path) : CAKE_HIP_OK;
}

int cake_hip_tune_load(const char* path, int* entries)
{
    if (entries) *entries = 0;
    if (!path) return fail(CAKE_HIP_ERR_ARG, "path is NULL");
    const int n = tune_load(path);
    if (n < 0) return fail(CAKE_HIP_ERR_ARG, "cannot read %s", path);
    if (entries) *entries = n;
    return CAKE_HIP_OK;
}

int cake_hip_tune_clear(void)
{
    tune_clear();
    return CAKE_HIP_OK;
}

int cake_hip_tune_count(void) { return tune_count(); }

int cake_hip_fill_uniform(float* dst, size_t n, uint64_t seed, void* stream_)
{
    if (n == 0) return CAKE_HIP_OK;
    if (!dst) return fail(CAKE_HIP_ERR_ARG, "NULL operand");
    int st = ensure_init();
    if (st) return st;
    std::lock_guard<std::recursive_mutex> lock(cur().mutex);
    hipStream_t stream = pick_stream(stream_);
    Operand o;
    if ((st = stage_in(dst, n * 4, 0, false, &o))) return st;
    hipError_t e = launch_fill_uniform(o.dev, n, seed, stream);
    if (e != hipSuccess) return fail(CAKE_HIP_ERR_HIP, "fill launch failed: %s", hipGetErrorString(e));
    return stage_out(o, stream);
}

int cake_hip_last_conv_route(void) { return g_last_conv_route; }

int cake_hip_last_kernel_seconds(double out[5])
{
    if (!out) return fail(CAKE_HIP_ERR_ARG, "out is NULL");
    for (int i = 0; i < 5; ++i) out[i] = g_family_seconds[i];
    return CAKE_HIP_OK;
}

}  // extern "C"
