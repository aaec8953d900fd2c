// cake_api.cpp -- libcake.so: the reference's C++ entry points for the fp32 GEMM
// path, forwarding to the C-ABI of libcake_hip.so.
//
// Error behaviour follows the reference (src/cake_sgemm.cpp:49-52,
// src/block_sizing.cpp:400-403): a failure prints a message and exit(1)s; there
// are no return codes at this level.  Return values are wall-clock seconds of
// the call, as in src/cake_sgemm.cpp:164-174.
#include "cake.h"

#include <math.h>
#include <time.h>

#include <mutex>

#include "cake_hip.h"

namespace {

double wall_seconds()
{
    struct timespec t;
    clock_gettime(CLOCK_REALTIME, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

void die_on(int status, const char* where)
{
    if (status == CAKE_HIP_OK) return;
    const char* detail = cake_hip_last_error();
    printf("%s: %s (%s)\n", where, cake_hip_strerror(status), detail ? detail : "");
    exit(1);
}

// blk_dims_t and cake_hip_blk_dims_t have the same 26 four-byte fields in the
// same order; the enum is an int.
static_assert(sizeof(blk_dims_t) == sizeof(cake_hip_blk_dims_t), "blk_dims_t layout");

cake_hip_blk_dims_t to_abi(const blk_dims_t* x)
{
    cake_hip_blk_dims_t d;
    memcpy(&d, x, sizeof d);
    return d;
}

cake_hip_cpu_cntx_t to_abi(const cake_cntx_t* c)
{
    cake_hip_cpu_cntx_t r;
    r.alpha_n = c->alpha_n;
    r.mr = c->mr; r.nr = c->nr;
    r.L1 = c->L1; r.L2 = c->L2; r.L3 = c->L3;
    r.ncores = c->ncores;
    return r;
}

long popen_number(const char* cmd)
{
    char buf[64] = {0};
    FILE* fp = popen(cmd, "r");
    if (!fp) return -1;
    char* got = fgets(buf, sizeof buf, fp);
    pclose(fp);
    return got ? atol(buf) : -1;
}

// Device-side state per cake_cntx_t.  The reference keeps its kernel library's context in
// cake_cntx_t::blis_cntx (include/common.h:139); here that field names the device context
// (workspaces, events, stream: cake_hip_ctx_create) the cntx works on, so that host threads that each
// use a cntx of their own do not wait for each other.  A cntx cannot be told when it is freed (callers
// free() it, examples/cake_sgemm_test.cpp:87), so contexts are not owned by it: they come from a
// small pool that lives as long as the process.  The first cntx seen works on the library's default
// context, the following ones on up to three created contexts, handed out in turn; whatever the
// field holds is only ever compared with the pool's entries, never followed.
enum { CONTEXT_POOL = 4 };
std::mutex g_pool_mutex;
char g_default_marker;                    // its address stands for the default context
void* g_pool[CONTEXT_POOL] = {&g_default_marker, NULL, NULL, NULL};
int g_pool_made = 1, g_pool_next = 0;

cake_hip_ctx_t context_of(cake_cntx_t* c)
{
    if (!c) return NULL;
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    void* mine = NULL;
    for (int i = 0; i < g_pool_made; ++i)
        if (c->blis_cntx == g_pool[i]) mine = g_pool[i];
    if (!mine) {
        if (g_pool_next >= g_pool_made && g_pool_made < CONTEXT_POOL) {
            cake_hip_ctx_t fresh = NULL;
            if (cake_hip_ctx_create(&fresh) == CAKE_HIP_OK && fresh) g_pool[g_pool_made++] = fresh;
        }
        mine = g_pool[g_pool_next % g_pool_made];
        g_pool_next = (g_pool_next + 1) % CONTEXT_POOL;
        c->blis_cntx = mine;
    }
    return mine == &g_default_marker ? NULL : mine;
}

// makes a cntx's device context the calling thread's for the duration of one call
struct OnContextOf {
    cake_hip_ctx_t before;
    explicit OnContextOf(cake_cntx_t* c) : before(cake_hip_ctx_get_current())
    {
        (void)cake_hip_ctx_set_current(context_of(c));
    }
    ~OnContextOf() { (void)cake_hip_ctx_set_current(before); }
};

// macro-tile override from the caller's mcu,kcu,ncu when such a tile exists
const int* tile_from_user(int M, int N, int K, int sch, int mcu, int kcu, int ncu, int out[4])
{
    if (!(mcu && kcu && ncu)) return NULL;
    out[0] = mcu; out[1] = ncu; out[2] = kcu; out[3] = 0;
    cake_hip_plan_t probe;
    return cake_hip_plan(M, N, K, sch, out, &probe) == CAKE_HIP_OK ? out : NULL;
}

double sgemm_common(float* A, float* B, float* C, int M, int N, int K, int p, cake_cntx_t* cntx,
                    char* argv[], bool packedA, bool packedB, float beta, enum sched sch, int mcu,
                    int kcu, int ncu)
{
    (void)argv;
    if (cntx == NULL) cntx = cake_query_cntx();  // leaked, as in the reference (:14-16)
    OnContextOf on(cntx);
    const double t0 = wall_seconds();
    if (packedA || packedB) {
        blk_dims_t x;
        init_block_dims(M, N, K, p, &x, cntx, sch, argv, 4, mcu, kcu, ncu);
        cake_hip_blk_dims_t d = to_abi(&x);
        cake_hip_cpu_cntx_t cx = to_abi(cntx);
        const int accumulate = (x.sch != KMN) && (beta != 0);
        double dev_s = 0;
        die_on(cake_hip_sgemm_packed(A, B, C, M, N, K, p, &d, &cx, packedA, packedB, accumulate, NULL, &dev_s),
               "cake_sgemm");
    } else {
        // beta != 0 means "start from C" only under the schedule the reference itself resolves
        // from the caller's cntx and p (src/cake_sgemm.cpp:34-35,114); the order in which the
        // GPU walks its tiles stays the planner's choice and does not change the result.
        int resolved = sch;
        if (M > 0 && N > 0 && K > 0) {
            blk_dims_t x;
            init_block_dims(M, N, K, p, &x, cntx, sch, argv, 4, mcu, kcu, ncu);
            resolved = x.sch;
        } else if (sch == NA) {
            resolved = KMN;   // nothing to size for an empty product: K-first, which assigns C
        }
        const int accumulate = (resolved != KMN) && (beta != 0);
        int ov[4];
        double dev_s = 0;
        die_on(cake_hip_sgemm(A, B, C, M, N, K, sch, accumulate, tile_from_user(M, N, K, sch, mcu, kcu, ncu, ov),
                              NULL, &dev_s),
               "cake_sgemm");
    }
    return wall_seconds() - t0;
}

}  // namespace

// ---- machine description ----------------------------------------------------

int get_num_physical_cores()
{
    long logical = popen_number("grep -c ^processor /proc/cpuinfo");
    long tpc = popen_number("lscpu | grep Thread -m 1 | tr -dc '0-9'");
    long sockets = popen_number("lscpu | grep Socket -m 1 | tr -dc '0-9'");
    if (logical <= 0) logical = 1;
    if (tpc <= 0) tpc = 1;
    if (sockets <= 0) sockets = 1;
    long c = logical / (tpc * sockets);
    return c > 0 ? (int)c : 1;
}

int get_cache_size(int level)
{
    char cmd[256], buf[64] = {0};
    snprintf(cmd, sizeof cmd,
             "lscpu --caches=NAME,%s | grep L%d | grep -Eo '[0-9]*M|[0-9]*K|[0-9]*G' | tr -d '\\n'",
             level < 3 ? "ONE-SIZE" : "ALL-SIZE", level);
    FILE* fp = popen(cmd, "r");
    if (!fp) return 0;
    char* got = fgets(buf, sizeof buf, fp);
    pclose(fp);
    size_t len = got ? strlen(buf) : 0;
    if (len < 2) return level == 1 ? 32 << 10 : level == 2 ? 1 << 20 : 32 << 20;
    int shift = buf[len - 1] == 'K' ? 10 : buf[len - 1] == 'M' ? 20 : 30;
    buf[len - 1] = 0;
    return atoi(buf) << shift;
}

cake_cntx_t* cake_query_cntx_torch(int L2, int L3)
{
    cake_cntx_t* c = (cake_cntx_t*)calloc(1, sizeof(cake_cntx_t));
    c->alpha_n = 1.0;
    c->mr = 6;
    c->nr = 16;
    c->L2 = L2;
    c->L3 = L3;
    c->ncores = get_num_physical_cores();
    c->peak_dram_bw = 8.0e12;
    c->peak_flops = 157.3e12;
    return c;
}

cake_cntx_t* cake_query_cntx()
{
    cake_cntx_t* c = cake_query_cntx_torch(get_cache_size(2), get_cache_size(3));
    c->L1 = get_cache_size(1);
    return c;
}

void update_mr_nr(cake_cntx_t* cake_cntx, int m_r, int n_r)
{
    cake_cntx->mr = m_r;
    cake_cntx->nr = n_r;
    cake_cntx->m_map = 0;
    cake_cntx->n_map = 0;
}

// ---- block sizing -------------------------------------------------------------

void init_block_dims(int M, int N, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx,
                     enum sched sch, char* argv[], float type_size, int mcu, int kcu, int ncu)
{
    (void)argv; (void)type_size;
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    cake_hip_blk_dims_t d;
    int st = cake_hip_init_block_dims(M, N, K, p, &cx, sch, mcu, kcu, ncu, &d);
    if (st != CAKE_HIP_OK) {
        printf("unknown schedule\n");
        exit(1);
    }
    memcpy(x, &d, sizeof d);
    cake_cntx->alpha_n = cx.alpha_n;
}

cache_dims_t* get_cache_dims(int M, int N, int K, int p, cake_cntx_t* cake_cntx, enum sched sch,
                             char* argv[], float type_size, int mcu, int kcu, int ncu)
{
    blk_dims_t x;
    init_block_dims(M, N, K, p, &x, cake_cntx, sch, argv, type_size, mcu, kcu, ncu);
    cache_dims_t* r = (cache_dims_t*)malloc(sizeof(cache_dims_t));
    r->m_c = x.m_c; r->k_c = x.k_c; r->n_c = x.n_c; r->sch = x.sch;
    return r;
}

int grid_dims_2d(int M, int N, int K, int p, int ncores) { return cake_hip_grid_dims_2d(M, N, K, p, ncores); }

void init_block_dims_2d(int M, int N, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch,
                        char* argv[], float type_size, int mcu, int kcu, int ncu)
{
    (void)argv;
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    cake_hip_blk_dims_t d;
    die_on(cake_hip_init_block_dims_2d(M, N, K, p, &cx, sch, type_size, mcu, kcu, ncu, &d), "init_block_dims_2d");
    memcpy(x, &d, sizeof d);
    cake_cntx->alpha_n = cx.alpha_n;
}

void init_block_dims_2d_small(int M, int N, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch,
                              char* argv[], float type_size)
{
    (void)argv;
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    cake_hip_blk_dims_t d;
    die_on(cake_hip_init_block_dims_2d_small(M, N, K, p, &cx, sch, type_size, &d), "init_block_dims_2d_small");
    memcpy(x, &d, sizeof d);
}

void init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s, int p,
                          blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch, char* argv[], float density,
                          float type_size)
{
    (void)argv; (void)density; (void)type_size;
    if (sch != KMN && sch != MKN && sch != NKM) {
        printf("unknown schedule\n");
        exit(1);
    }
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    cake_hip_blk_dims_t d;
    die_on(cake_hip_init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, &cx, &d), "init_block_dims_conv");
    if (sch != KMN) {   // the reference sizes m_c, k_c, n_c and fills in nothing else for these (cake_conv.cpp:404-416)
        cake_hip_blk_dims_t only = cake_hip_blk_dims_t();
        only.m_c = d.m_c; only.k_c = d.k_c; only.n_c = d.n_c;
        d = only;
    }
    d.sch = sch;
    memcpy(x, &d, sizeof d);
}

cache_dims_t* get_cache_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s,
                                  int p, cake_cntx_t* cake_cntx, enum sched sch, char* argv[], float density,
                                  float type_size)
{
    blk_dims_t x;
    init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, &x, cake_cntx, KMN, argv, density, type_size);
    cache_dims_t* r = (cache_dims_t*)malloc(sizeof(cache_dims_t));
    r->m_c = x.m_c; r->k_c = x.k_c; r->n_c = x.n_c; r->sch = sch;
    return r;
}

enum sched derive_schedule(int M, int N, int K, int p, int mc_ret, cake_cntx_t* cake_cntx)
{
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    return (enum sched)cake_hip_derive_schedule(M, N, K, p, mc_ret, &cx);
}

// ---- GEMM -----------------------------------------------------------------------

double cake_sgemm(float* A, float* B, float* C, int M, int N, int K, int p, cake_cntx_t* cake_cntx,
                  char* argv[], bool packedA, bool packedB, float alpha, float beta, enum sched sch,
                  int mcu, int kcu, int ncu)
{
    (void)alpha;  // never read by the reference either
    return sgemm_common(A, B, C, M, N, K, p, cake_cntx, argv, packedA, packedB, beta, sch, mcu, kcu, ncu);
}

// The pack-on-the-fly and 2-D entry points always run K-first on row-major operands: they set
// sch = KMN before sizing their blocks and never look at packedA / packedB or beta
// (src/cake_sgemm.cpp:200,273,418), so C is assigned whatever the caller passed.
double cake_sgemm_online(float* A, float* B, float* C, int M, int N, int K, int p,
                         cake_cntx_t* cake_cntx, char* argv[], bool packedA, bool packedB, float alpha,
                         float beta, enum sched sch, int mcu, int kcu, int ncu)
{
    (void)alpha; (void)beta; (void)sch; (void)packedA; (void)packedB;
    return sgemm_common(A, B, C, M, N, K, p, cake_cntx, argv, 0, 0, 0.f, KMN, mcu, kcu, ncu);
}

double cake_sgemm_2d(float* A, float* B, float* C, int M, int N, int K, int p, cake_cntx_t* cake_cntx,
                     char* argv[], bool packedA, bool packedB, float alpha, float beta, enum sched sch,
                     int mcu, int kcu, int ncu)
{
    (void)alpha; (void)beta; (void)sch; (void)packedA; (void)packedB;
    return sgemm_common(A, B, C, M, N, K, p, cake_cntx, argv, 0, 0, 0.f, KMN, mcu, kcu, ncu);
}

double cake_sgemm_2d_small(float* A, float* B, float* C, int M, int N, int K, int p,
                           cake_cntx_t* cake_cntx, char* argv[], bool packedA, bool packedB,
                           float alpha, float beta, enum sched sch)
{
    (void)alpha; (void)beta; (void)sch; (void)packedA; (void)packedB;
    return sgemm_common(A, B, C, M, N, K, p, cake_cntx, argv, 0, 0, 0.f, KMN, 0, 0, 0);
}

// The timing variant sets sch = KMN and otherwise runs cake_sgemm's steps, packed operands
// included (src/cake_sgemm.cpp:472-600); K-first assigns C whatever beta says.
double cake_sgemm_test(float* A, float* B, float* C, int M, int N, int K, int p, cake_cntx_t* cake_cntx,
                       char* argv[], bool packedA, bool packedB, float alpha, float beta, enum sched sch)
{
    (void)alpha; (void)sch;
    return sgemm_common(A, B, C, M, N, K, p, cake_cntx, argv, packedA, packedB, beta, KMN, 0, 0, 0);
}

// ---- packing ----------------------------------------------------------------------

size_t cake_sgemm_packed_A_size(int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    return cake_hip_packed_a_size(M, K, p, &d, &cx, sch);
}

size_t cake_sgemm_packed_B_size(int K, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    return cake_hip_packed_b_size(K, N, p, &d, &cx);
}

size_t cake_sgemm_packed_C_size(int M, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    return cake_hip_packed_c_size(M, N, p, &d, &cx, sch);
}

double pack_A(float* A, float* A_p, int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    OnContextOf on(cake_cntx);
    const double t0 = wall_seconds();
    die_on(cake_hip_pack_a(A, A_p, M, K, p, &d, &cx, sch, NULL, NULL), "pack_A");
    die_on(cake_hip_synchronize(), "pack_A");
    return wall_seconds() - t0;
}

void pack_B(float* B, float* B_p, int K, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    OnContextOf on(cake_cntx);
    die_on(cake_hip_pack_b(B, B_p, K, N, p, &d, &cx, sch, NULL, NULL), "pack_B");
}

void pack_C(float* C, float* C_p, int M, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    OnContextOf on(cake_cntx);
    die_on(cake_hip_pack_c(C, C_p, M, N, p, &d, &cx, sch, NULL, NULL), "pack_C");
}

void unpack_C(float* C, float* C_p, int M, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    OnContextOf on(cake_cntx);
    die_on(cake_hip_unpack_c(C, C_p, M, N, p, &d, &cx, sch, NULL, NULL), "unpack_C");
}

// ---- GEMV -------------------------------------------------------------------------

double cake_sgemv(float* A, float* B, float* C, int M, int K, int p, cake_cntx_t* cake_cntx,
                  char* argv[], bool packedA, float alpha, float beta, enum sched sch)
{
    (void)p; (void)argv; (void)packedA; (void)alpha; (void)beta; (void)sch;
    OnContextOf on(cake_cntx);
    const double t0 = wall_seconds();
    double dev_s = 0;
    // column-major A, accumulate into y: examples/cake_gemv.cpp:89-140
    die_on(cake_hip_sgemv(A, B, C, M, K, 1, 1, NULL, &dev_s), "cake_sgemv");
    return wall_seconds() - t0;
}

// ---- im2col -----------------------------------------------------------------------

float* im_2_col(float* In, int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s)
{
    (void)Cout; (void)s;  // neither is used by the reference's im_2_col
    if (Hout != Hin - Hf + 1 || Wout != Win - Wf + 1) {
        printf("im_2_col: Hout/Wout must be Hin-Hf+1 / Win-Wf+1\n");
        exit(1);
    }
    float* cols = (float*)malloc(sizeof(float) * (size_t)Cin * Hf * Wf * Hout * Wout);
    if (!cols) {
        printf("im_2_col: out of memory\n");
        exit(1);
    }
    die_on(cake_hip_im2col(In, cols, 1, Cin, Hin, Win, Hf, Wf, 1, 0, NULL, NULL), "im_2_col");
    return cols;
}

// ---- direct convolution --------------------------------------------------------------

// pack_filters (examples/cake_conv.cpp:536-610) is written for 3 x 3 filters: K = Cin * 9
double pack_filters(float* A, float* A_p, int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx)
{
    cake_hip_blk_dims_t d = to_abi(x);
    cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
    OnContextOf on(cake_cntx);
    const double t0 = wall_seconds();
    die_on(cake_hip_pack_filters(A, A_p, M, K / 9, 9, p, &d, &cx, NULL, NULL), "pack_filters");
    die_on(cake_hip_synchronize(), "pack_filters");
    return wall_seconds() - t0;
}

double cake_sconv(float* A, float* B, float* C, int Wf, int Hf, int Win, int Hin, int Wout, int Hout,
                  int Cin, int Cout, int s, int p, cake_cntx_t* cake_cntx, char* argv[], bool packedA,
                  enum sched sch)
{
    (void)sch;   // always K-first in the reference (cake_conv.cpp:790)
    if (cake_cntx == NULL) cake_cntx = cake_query_cntx();  // leaked, as in the reference (:770-772)
    OnContextOf on(cake_cntx);
    const double t0 = wall_seconds();
    if (packedA) {
        // A was written by pack_filters for the blocks the reference derives here (:791-799)
        blk_dims_t x;
        init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, &x, cake_cntx, KMN, argv, 0, 4);
        cake_hip_blk_dims_t d = to_abi(&x);
        cake_hip_cpu_cntx_t cx = to_abi(cake_cntx);
        die_on(cake_hip_sconv_packed(A, B, C, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, &d, &cx, NULL, NULL),
               "cake_sconv");
    } else {
        die_on(cake_hip_sconv(A, B, C, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, NULL, NULL), "cake_sconv");
    }
    return wall_seconds() - t0;
}

void conv_gemm_checker(float* conv, float* gemm, int M, int N)
{
    const float eps = 1e-3f;  // cake_conv.cpp:1219
    long wrong = 0, correct = 0;
    for (size_t i = 0; i < (size_t)M * N; ++i) (fabsf(gemm[i] - conv[i]) > eps ? wrong : correct)++;
    if (wrong)
        printf("WRONG = %ld , CORRECT = %ld\n", wrong, correct);
    else
        printf("CORRECT!\n");
}

// ---- test helpers (host code) -------------------------------------------------------

void rand_init(float* mat, int r, int c)
{
    for (size_t i = 0; i < (size_t)r * c; ++i) mat[i] = (float)rand() / (float)RAND_MAX * 2.0f - 1.0f;
}

bool mat_equals(float* C, float* C_check, int M, int N)
{
    const float eps = 1e-3f;  // util.cpp:144
    long bad = 0;
    for (size_t i = 0; i < (size_t)M * N; ++i)
        if (fabsf(C_check[i] - C[i]) > eps) ++bad;
    if (!bad) {
        printf("CORRECT!\n");
        return 0;
    }
    printf("WRONG!\n%ld\n", bad);
    return 1;
}

bool cake_sgemm_checker(float* A, float* B, float* C, int N, int M, int K)
{
    float* ref = (float*)calloc((size_t)M * N, sizeof(float));
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int k = 0; k < K; ++k) {
            const float a = A[(size_t)m * K + k];
            const float* b = B + (size_t)k * N;
            float* r = ref + (size_t)m * N;
            for (int n = 0; n < N; ++n) r[n] += a * b[n];
        }
    bool ret = mat_equals(C, ref, M, N);
    free(ref);
    return ret;
}

void print_schedule(enum sched sch)
{
    static const char* names[] = {"KMN", "MKN", "NKM", "NA"};
    printf("%s Cake Schedule\n", names[(int)sch & 3]);
}

void print_array(float* arr, int len)
{
    for (int i = 0; i < len; ++i) printf("%f ", arr[i]);
    printf("\n");
}

void print_mat(float* arr, int r, int c)
{
    for (int i = 0; i < r; ++i) print_array(arr + (size_t)i * c, c);
}

bool add_checker(float** C_arr, float* C, int M, int N, int p)
{
    const float eps = 1e-3f;
    long bad = 0;
    for (size_t i = 0; i < (size_t)M * N; ++i) {
        float sum = 0.f;
        for (int c = 0; c < p; ++c) sum += C_arr[c][i];
        if (fabsf(sum - C[i]) > eps) ++bad;
    }
    if (!bad) {
        printf("ADD CORRECT!\n");
        return 0;
    }
    printf("ADD WRONG!\n%ld\n", bad);
    return 1;
}

float rand_gen() { return ((float)rand() + 1.f) / ((float)RAND_MAX + 1.f); }

float normalRandom()
{
    const float u = rand_gen(), v = rand_gen();
    return cosf(2.f * 3.14159265358979323846f * v) * sqrtf(-2.f * logf(u));
}

void transpose_mat(float* A_old, float* At, int K, int N, int Kt, int Nt)
{
    (void)Kt; (void)Nt;
    die_on(cake_hip_transpose(A_old, At, K, N, NULL, NULL), "transpose_mat");
}

// ---- the reference's self-test over the five entry points ---------------------------

namespace {

typedef double (*sgemm_entry)(float*, float*, float*, int, int, int, int, cake_cntx_t*, char**, bool, bool,
                              float, float, enum sched, int, int, int);

struct EntryCase {
    const char* name;
    sgemm_entry fn;
    enum sched sch;
};

}  // namespace

int run_tests()
{
    static const int dims[6] = {1, 10, 96, 111, 960, 2111};  // util.cpp:11-13
    static const EntryCase entries[5] = {
        {"2d K-first", cake_sgemm_2d, KMN},   {"M-first", cake_sgemm, MKN}, {"online K-first", cake_sgemm_online, KMN},
        {"K-first", cake_sgemm, KMN},         {"N-first", cake_sgemm, NKM},
    };
    cake_cntx_t* cntx = cake_query_cntx();
    const int ps[2] = {2, cntx->ncores > 2 ? cntx->ncores : 0};
    int failed = 0;
    srand((unsigned)time(NULL));
    for (int pi = 0; pi < 2; ++pi) {
        const int p = ps[pi];
        if (p == 0) continue;
        for (int mi = 0; mi < 6; ++mi)
            for (int ki = 0; ki < 6; ++ki)
                for (int ni = 0; ni < 6; ++ni) {
                    const int M = dims[mi], K = dims[ki], N = dims[ni];
                    float* A = (float*)malloc(sizeof(float) * (size_t)M * K);
                    float* B = (float*)malloc(sizeof(float) * (size_t)K * N);
                    float* C = (float*)malloc(sizeof(float) * (size_t)M * N);
                    rand_init(A, M, K);
                    rand_init(B, K, N);
                    for (const EntryCase& e : entries) {
                        memset(C, 0, sizeof(float) * (size_t)M * N);
                        e.fn(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 0, e.sch, 0, 0, 0);
                        if (cake_sgemm_checker(A, B, C, N, M, K)) {
                            printf("TESTS FAILED on %s p=%d M=%d K=%d N=%d\n", e.name, p, M, K, N);
                            ++failed;
                        }
                    }
                    free(A); free(B); free(C);
                }
    }
    free(cntx);
    printf(failed ? "FAILED\n" : "ALL TESTS PASSED!\n");
    return 0;
}
