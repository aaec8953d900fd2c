/*
 * cake_oracle.c -- CPU restatement of the CAKE fp32 GEMM hot path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the GPU library is
 * compared against and the CPU baseline that is timed beside it.  Nothing in
 * the shipped library links, loads or calls it.
 *
 * Every function names the file:line of vnatesh/CAKE_on_CPU it restates.
 * The code is written from the algorithm, not transcribed: block walks are
 * expressed as (block, core) -> (source offset, destination offset) maps and
 * one generic panel copier per operand.
 *
 * Pin status (which independent check would catch a mistake in each part):
 *   planner (orc_get_cache_dims / orc_derive_schedule / orc_init_block_dims)
 *       - known answers measured on the real reference build for four shapes,
 *         coverage invariants on the 6^3 edge-shape grid, and end-to-end
 *         products against the fp64 closed form (a wrong remainder breaks C).
 *   packing / unpacking (orc_pack_A/B/C, orc_unpack_C, panel copiers)
 *       - bit-exact against the reference's own pack_*.cpp / unpack_*.cpp
 *         compiled from /root/reference (oracle/_ref), permutation and
 *         zero-padding properties, packed sizes.
 *   micro-kernel (orc_ukernel)
 *       - bit-exact against the reference's 6x16 AVX2 kernel (oracle/_ref).
 *   schedules (orc_schedule_KMN/MKN/NKM) and orc_cake_sgemm
 *       - fp64 triple loop, identity / all-ones / single-non-zero cases on the
 *         reference's own edge-shape list {1,10,96,111,960,2111}.
 *   orc_cake_sgemv
 *       - bit-exact against the reference's schedule_mvm + 8-row kernel
 *         (oracle/_ref) where M is a multiple of 8, fp64 dot products.
 *   orc_im_2_col / orc_im2col
 *       - bit-exact against the reference's im_2_col (oracle/_ref), brute-force
 *         definition, naive 7-loop convolution.
 *   The outputs of the compiled reference parts on seeded inputs are also
 *   committed (tests/golden/reference_vectors.npz), so the packing, kernel, gemv
 *   and im_2_col comparisons run where the reference sources are absent too.
 *   orc_init_block_dims_conv / orc_pack_filters
 *       - bit-exact against the reference's init_block_dims_conv and pack_filters
 *         (oracle/_ref) and their committed outputs, a hand-computed block table,
 *         and the permutation property (every filter value lands exactly once).
 *   The linear layer (oracle/__init__.py, a caller of orc_cake_sgemm) is pinned
 *   against torch.nn.functional.linear and its autograd in fp64.
 *   No function here is "parity unpinned".
 */
#define _GNU_SOURCE
#include <immintrin.h>
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

enum { ORC_KMN = 0, ORC_MKN = 1, ORC_NKM = 2, ORC_NA = 3 };

/* Same fields, same order as blk_dims_t (include/common.h:108-135). */
typedef struct orc_blk_dims {
    int m_c, k_c, n_c;
    int m_c1, k_c1, n_c1;
    int m_c1_last_core, n_c1_last_core, k_c1_last_core;
    int mr_rem, nr_rem, k_rem;
    int p_l, pm_l, pn_l, pm, pn;
    int m_pad, k_pad, n_pad;
    int Mb, Kb, Nb;
    int M_padded, N_padded;
    int sch;
} orc_blk_dims;

/* The planner inputs of cake_cntx_t (include/common.h:138-151). */
typedef struct orc_cntx {
    double alpha_n;
    int mr, nr;
    int L1, L2, L3;
    int ncores;
} orc_cntx;

static double now_s(void)
{
    struct timespec t;
    clock_gettime(CLOCK_REALTIME, &t);
    return (double)t.tv_sec + 1e-9 * (double)t.tv_nsec;
}

/* ------------------------------------------------------------------------ */
/* Seeded inputs: counter-based splitmix64, 24 random bits -> [-1, 1).       */
/* Element i of stream `seed` is mix(seed + (i+1)*GOLDEN); every value is an  */
/* exact multiple of 2^-23, so host, numpy and device generators agree to     */
/* the bit.                                                                   */
/* ------------------------------------------------------------------------ */
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t i)
{
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void orc_fill_uniform(float *dst, size_t n, uint64_t seed)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        uint32_t bits24 = (uint32_t)(splitmix64_at(seed, i) >> 40);
        dst[i] = (float)bits24 * 0x1p-23f - 1.0f;
    }
}

/* ------------------------------------------------------------------------ */
/* Machine description (cake_query_cntx, src/block_sizing.cpp:40-75;          */
/* get_num_physical_cores :91-143; get_cache_size :148-298).  The reference   */
/* shells out to lscpu; so does this.  Its per-CPU-model size table is a      */
/* special case for a handful of parts and is not restated.                   */
/* ------------------------------------------------------------------------ */
static long run_number(const char *cmd)
{
    char buf[64] = {0};
    FILE *fp = popen(cmd, "r");
    if (!fp) return -1;
    if (!fgets(buf, sizeof buf, fp)) { pclose(fp); return -1; }
    pclose(fp);
    return atol(buf);
}

static int lscpu_cache_bytes(int level)
{
    char cmd[256], buf[64] = {0};
    snprintf(cmd, sizeof cmd,
             "lscpu --caches=NAME,%s | grep L%d | grep -Eo '[0-9]*M|[0-9]*K|[0-9]*G' | tr -d '\\n'",
             level < 3 ? "ONE-SIZE" : "ALL-SIZE", level);
    FILE *fp = popen(cmd, "r");
    if (!fp) return 0;
    if (!fgets(buf, sizeof buf, fp)) { pclose(fp); return 0; }
    pclose(fp);
    size_t len = strlen(buf);
    if (len == 0) return 0;
    char unit = buf[len - 1];
    buf[len - 1] = 0;
    long v = atol(buf);
    if (unit == 'K') return (int)(v << 10);
    if (unit == 'M') return (int)(v << 20);
    if (unit == 'G') return (int)(v << 30);
    return 0;
}

int orc_physical_cores(void)
{
    long logical = run_number("grep -c ^processor /proc/cpuinfo");
    long tpc = run_number("lscpu | grep Thread -m 1 | tr -dc '0-9'");
    long sockets = run_number("lscpu | grep Socket -m 1 | tr -dc '0-9'");
    if (logical <= 0) logical = omp_get_num_procs();
    if (tpc <= 0) tpc = 1;
    if (sockets <= 0) sockets = 1;
    long c = logical / (tpc * sockets);
    return c > 0 ? (int)c : 1;
}

void orc_query_cntx(orc_cntx *c)
{
    c->alpha_n = 1.0;
    c->mr = 6;  /* MR_MIN / NR_MIN of the Haswell build (python/kernel_gen.py:421-465) */
    c->nr = 16;
    c->L1 = lscpu_cache_bytes(1);
    c->L2 = lscpu_cache_bytes(2);
    c->L3 = lscpu_cache_bytes(3);
    c->ncores = orc_physical_cores();
    if (c->L1 <= 0) c->L1 = 32 << 10;
    if (c->L2 <= 0) c->L2 = 1 << 20;
    if (c->L3 <= 0) c->L3 = 32 << 20;
}

/* ------------------------------------------------------------------------ */
/* Planner                                                                    */
/* ------------------------------------------------------------------------ */

/* derive_schedule, src/block_sizing.cpp:434-462.  The cut-offs are kept in
 * single precision exactly as there (float m,k,n; double intermediate). */
int orc_derive_schedule(int M, int N, int K, int p, int mc, const orc_cntx *cx)
{
    (void)p;
    float side = (float)(p * mc);
    float K_cut_M = (float)((2.0 * M) / (1.0 + (M * ((2.0 / side) - (1.0 / side)))));
    float K_cut_N = (float)((2.0 * N) / (1.0 + (N * ((2.0 / side) - (1.0 / side)))));
    float wide = (float)(cx->alpha_n * p * mc);
    float N_cut_M = (float)(M / (1.0 + (M * ((1.0 / wide) - (1.0 / wide)))));
    float M_cut_N = (float)(N / (1.0 + (N * ((1.0 / wide) - (1.0 / wide)))));
    if ((float)N <= N_cut_M && (float)K <= K_cut_M) return ORC_MKN;
    if ((float)M <= M_cut_N && (float)K <= K_cut_N) return ORC_NKM;
    return ORC_KMN;
}

static int round_down(int v, int q) { return v - (v % q); }

/* get_cache_dims, src/block_sizing.cpp:304-429.  Writes alpha_n into *cx like
 * the reference does. */
void orc_get_cache_dims(int M, int N, int K, int p, orc_cntx *cx, int sch,
                        int mcu, int kcu, int ncu,
                        int *m_c, int *k_c, int *n_c, int *sch_out)
{
    const double ts = 4.0;
    const int mr = cx->mr, nr = cx->nr;

    /* L2: 2*ts*(x^2 + 2*nr*x) <= L2  ->  positive root, rounded down to mr (:316-321). */
    int b = 2 * nr;
    int mc_L2 = (int)((-b + sqrt((double)(b * b) + 4.0 * ((double)cx->L2 / (2.0 * ts)))) / 2.0);
    mc_L2 = round_down(mc_L2, mr);

    /* L3 (:329-331). */
    int nt = cx->ncores;
    int mc_L3 = (int)sqrt(((double)cx->L3 / (2.0 * ts)) / (nt * (1 + 1.0 + 1.0 * nt)));
    mc_L3 = round_down(mc_L3, mr);

    cx->alpha_n = (double)mc_L3 / mc_L2; /* :336 */

    /* Shrink m_c when M cannot fill p blocks (:340-352).  Note: an exact
     * multiple of mr still gains a full extra mr. */
    int mc = mc_L2;
    if (M < p * mr) {
        mc = mr;
    } else if (M < p * mc_L2) {
        int a = M / p;
        mc = (a < mr) ? mr : a + (mr - (a % mr));
    }

    int s = (sch == ORC_NA) ? orc_derive_schedule(M, N, K, p, mc, cx) : sch;
    *sch_out = s;

    if (mcu && ncu && kcu) { /* user tiles (:363-368) */
        *m_c = mcu; *k_c = kcu; *n_c = ncu;
        cx->alpha_n = 1.0;
        return;
    }

    int nc;
    if (s == ORC_KMN || s == ORC_MKN) { /* :376-386 */
        nc = round_down((int)(cx->alpha_n * p * mc), nr);
        if (nc == 0) nc = nr;
    } else if (s == ORC_NKM) { /* :389-397 */
        nc = round_down(mc, nr);
        if (nc == 0) nc = nr;
        mc = round_down((int)(cx->alpha_n * mc), mr);
        if (mc == 0) mc = mr;
    } else {
        fprintf(stderr, "unknown schedule\n");
        exit(1);
    }
    *m_c = mc; *k_c = mc; *n_c = nc; /* k_c = m_c, :407 */
}

static int ceil_ratio(int a, int b) { return (int)ceil((double)a / (double)b); }

/* init_block_dims, src/block_sizing.cpp:465-595.  Fields the reference leaves
 * untouched for a schedule are zero here. */
void orc_init_block_dims(int M, int N, int K, int p, orc_blk_dims *x, orc_cntx *cx,
                         int sch, int mcu, int kcu, int ncu)
{
    const int mr = cx->mr, nr = cx->nr;
    memset(x, 0, sizeof *x);
    orc_get_cache_dims(M, N, K, p, cx, sch, mcu, kcu, ncu, &x->m_c, &x->k_c, &x->n_c, &x->sch);

    /* N side is the same in all three schedules. */
    x->n_pad = (N % x->n_c) ? 1 : 0;
    x->nr_rem = ceil_ratio(N % x->n_c, nr);
    x->n_c1 = x->nr_rem * nr;
    x->Nb = N / x->n_c + x->n_pad;
    x->N_padded = (N - N % x->n_c) + x->n_c1;

    if (x->sch == ORC_KMN) { /* :481-516: M is split over the p cores */
        int span = p * x->m_c;
        x->k_pad = (K % x->k_c) ? 1 : 0;
        x->m_pad = (M % span) ? 1 : 0;
        x->mr_rem = ceil_ratio(M % span, mr);
        int per_core = ceil_ratio(x->mr_rem, p);
        x->p_l = per_core ? ceil_ratio(x->mr_rem, per_core) : 0;
        x->m_c1 = per_core * mr;
        x->m_c1_last_core = (per_core - (x->p_l * per_core - x->mr_rem)) * mr;
        x->k_c1 = K % x->k_c;
        x->Mb = M / span + x->m_pad;
        x->Kb = K / x->k_c + x->k_pad;
        x->M_padded = mr * x->mr_rem + (M / span) * span;
        x->pm = p; x->pn = 1;
    } else if (x->sch == ORC_MKN || x->sch == ORC_NKM) { /* :519-590: K is split over the cores */
        int kspan = p * x->k_c;
        int mspan = (x->sch == ORC_MKN) ? x->m_c : p * x->m_c;
        x->k_pad = (K % kspan) ? 1 : 0;
        x->m_pad = (M % mspan) ? 1 : 0;
        x->k_rem = K % kspan;
        x->k_c1 = ceil_ratio(x->k_rem, p);
        x->p_l = x->k_c1 ? ceil_ratio(x->k_rem, x->k_c1) : 0;
        x->k_c1_last_core = x->k_rem - x->k_c1 * (x->p_l - 1);
        x->mr_rem = ceil_ratio(M % mspan, mr);
        x->m_c1 = x->mr_rem * mr;
        x->Mb = M / mspan + x->m_pad;
        x->Kb = K / kspan + x->k_pad;
        x->M_padded = (M / mspan) * mspan + x->m_c1;
        if (x->sch == ORC_MKN) { x->pm = p; x->pn = 1; } else { x->pm = 1; x->pn = p; }
    } else {
        fprintf(stderr, "unknown schedule\n");
        exit(1);
    }
}

/* cake_sgemm_packed_{A,B,C}_size, src/pack_helper.cpp:5-87 (bytes). */
size_t orc_packed_A_size(int M, int K, int p, const orc_blk_dims *x, const orc_cntx *cx, int sch)
{
    int span = (sch == ORC_MKN) ? x->m_c : p * x->m_c;
    int rem = ceil_ratio(M % span, cx->mr);
    size_t Mp = (size_t)cx->mr * rem + (size_t)(M / span) * span;
    return Mp * (size_t)K * sizeof(float);
}

size_t orc_packed_B_size(int K, int N, int p, const orc_blk_dims *x, const orc_cntx *cx)
{
    (void)p;
    int rem = ceil_ratio(N % x->n_c, cx->nr);
    size_t Np = (size_t)(N - N % x->n_c) + (size_t)rem * cx->nr;
    return (size_t)K * Np * sizeof(float);
}

size_t orc_packed_C_size(int M, int N, int p, const orc_blk_dims *x, const orc_cntx *cx, int sch)
{
    size_t a = orc_packed_A_size(M, 1, p, x, cx, sch) / sizeof(float);
    size_t b = orc_packed_B_size(1, N, p, x, cx) / sizeof(float);
    return a * b * sizeof(float);
}

/* ------------------------------------------------------------------------ */
/* Panel copiers (pack_ob_A_single_buf, src/pack_ob.cpp:40-60;               */
/* pack_ob_B_single_buf :105-140; pack_ob_C_single_buf :253-288;              */
/* unpack_ob_C_single_buf :393-411).  rows_left / cols_left = how many real   */
/* rows / columns remain from the block's origin; the rest is zero padding.   */
/* ------------------------------------------------------------------------ */
static void copy_A_block(const float *src, float *dst, int ld, int rows_left,
                         int rows, int kc, int mr)
{
    size_t o = 0;
    for (int r0 = 0; r0 < rows; r0 += mr)
        for (int kk = 0; kk < kc; ++kk)
            for (int j = 0; j < mr; ++j, ++o)
                dst[o] = (r0 + j < rows_left) ? src[(size_t)(r0 + j) * ld + kk] : 0.0f;
}

static void copy_B_block(const float *src, float *dst, int ld, int cols_left,
                         int kc, int cols, int nr)
{
    size_t o = 0;
    for (int c0 = 0; c0 < cols; c0 += nr)
        for (int kk = 0; kk < kc; ++kk)
            for (int j = 0; j < nr; ++j, ++o)
                dst[o] = (c0 + j < cols_left) ? src[(size_t)kk * ld + c0 + j] : 0.0f;
}

static void copy_C_block(float *c, float *cp, int ld, int rows_left, int cols_left,
                         int rows, int cols, int mr, int nr, int to_packed)
{
    size_t o = 0;
    for (int c0 = 0; c0 < cols; c0 += nr)
        for (int r0 = 0; r0 < rows; r0 += mr)
            for (int i = 0; i < mr; ++i)
                for (int j = 0; j < nr; ++j, ++o) {
                    int inside = (r0 + i < rows_left) && (c0 + j < cols_left);
                    float *g = c + (size_t)(r0 + i) * ld + c0 + j;
                    if (to_packed) cp[o] = inside ? *g : 0.0f;
                    else if (inside) *g = cp[o];
                }
}

/* Geometry of one "core" slice in the split dimension of the last block. */
typedef struct { int used, span; } split_t;

static split_t split_of(int is_last, int p, int p_l, int full, int rem_span)
{
    split_t s;
    s.used = is_last ? p_l : p;
    s.span = is_last ? rem_span : p * full;
    return s;
}

/* ------------------------------------------------------------------------ */
/* pack_A                                                                     */
/*   KMN: pack_A_single_buf_k_first, src/pack_k_first.cpp:7-76                */
/*   MKN: pack_A_single_buf_m_first, src/pack_m_first.cpp:7-78                */
/*   NKM: pack_A_single_buf_n_first, src/pack_n_first.cpp:8-79                */
/* ------------------------------------------------------------------------ */
double orc_pack_A(const float *A, float *Ap, int M, int K, int p,
                  const orc_blk_dims *x, const orc_cntx *cx, int sch)
{
    const int mr = cx->mr;
    double t0 = now_s();
    size_t off = 0;
    if (sch == ORC_KMN) {
        for (int mb = 0; mb < x->Mb; ++mb) {
            int last = (mb == x->Mb - 1) && x->m_pad;
            split_t s = split_of(last, p, x->p_l, x->m_c, mr * x->mr_rem);
            int slice = last ? x->m_c1 : x->m_c;
            for (int kb = 0; kb < x->Kb; ++kb) {
                int kc = ((kb == x->Kb - 1) && x->k_pad) ? x->k_c1 : x->k_c;
#pragma omp parallel for
                for (int core = 0; core < s.used; ++core) {
                    int rows = last ? (core == x->p_l - 1 ? x->m_c1_last_core : x->m_c1) : x->m_c;
                    size_t row0 = (size_t)mb * p * x->m_c + (size_t)core * slice;
                    copy_A_block(A + row0 * K + (size_t)kb * x->k_c,
                                 Ap + off + (size_t)core * slice * kc,
                                 K, M - (int)row0, rows, kc, mr);
                }
                off += (size_t)s.span * kc;
            }
        }
    } else if (sch == ORC_MKN || sch == ORC_NKM) {
        /* the two differ only in which loop is outermost and in the M block height */
        int mspan = (sch == ORC_MKN) ? x->m_c : p * x->m_c;
        int outerN = (sch == ORC_MKN) ? x->Kb : x->Mb;
        int innerN = (sch == ORC_MKN) ? x->Mb : x->Kb;
        for (int o = 0; o < outerN; ++o)
            for (int i = 0; i < innerN; ++i) {
                int kb = (sch == ORC_MKN) ? o : i;
                int mb = (sch == ORC_MKN) ? i : o;
                int lastk = (kb == x->Kb - 1) && x->k_pad;
                split_t s = split_of(lastk, p, x->p_l, x->k_c, x->k_rem);
                int slice = lastk ? x->k_c1 : x->k_c;
                int rows = ((mb == x->Mb - 1) && x->m_pad) ? x->m_c1 : mspan;
#pragma omp parallel for
                for (int core = 0; core < s.used; ++core) {
                    int kc = lastk ? (core == x->p_l - 1 ? x->k_c1_last_core : x->k_c1) : x->k_c;
                    size_t row0 = (size_t)mb * mspan;
                    copy_A_block(A + row0 * K + (size_t)kb * p * x->k_c + (size_t)core * slice,
                                 Ap + off + (size_t)core * slice * rows,
                                 K, M - (int)row0, rows, kc, mr);
                }
                off += (size_t)s.span * rows;
            }
    } else {
        fprintf(stderr, "unknown schedule\n");
        exit(1);
    }
    return now_s() - t0;
}

/* ------------------------------------------------------------------------ */
/* pack_B                                                                     */
/*   KMN: pack_B_k_first, src/pack_k_first.cpp:187-283                        */
/*   MKN: pack_B_m_first, src/pack_m_first.cpp:83-144                         */
/*   NKM: pack_B_n_first, src/pack_n_first.cpp:84-144                         */
/* Columns >= N are always written as zero here.  The MKN/NKM reference code  */
/* passes a K-derived flag as pad_n (pack_m_first.cpp:128-139), so outside    */
/* the last core of the last K block it fills that padding with wrapped reads */
/* of B instead; the padding columns never reach C, so results agree.         */
/* ------------------------------------------------------------------------ */
void orc_pack_B(const float *B, float *Bp, int K, int N, int p,
                const orc_blk_dims *x, const orc_cntx *cx, int sch)
{
    const int nr = cx->nr;
    if (sch == ORC_KMN) {
        /* n-block nb starts at nb*K*n_c; inside it k-block kb starts at kb*k_c*n_c_t */
        for (int nb = 0; nb < x->Nb; ++nb) {
            int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
#pragma omp parallel for
            for (int kb = 0; kb < x->Kb; ++kb) {
                int kc = ((kb == x->Kb - 1) && x->k_pad) ? x->k_c1 : x->k_c;
                copy_B_block(B + (size_t)kb * x->k_c * N + (size_t)nb * x->n_c,
                             Bp + (size_t)nb * K * x->n_c + (size_t)kb * x->k_c * cols,
                             N, N - nb * x->n_c, kc, cols, nr);
            }
        }
        return;
    }
    if (sch != ORC_MKN && sch != ORC_NKM) {
        fprintf(stderr, "unknown schedule\n");
        exit(1);
    }
    size_t off = 0;
    int outerN = (sch == ORC_MKN) ? x->Nb : x->Kb;
    int innerN = (sch == ORC_MKN) ? x->Kb : x->Nb;
    for (int o = 0; o < outerN; ++o)
        for (int i = 0; i < innerN; ++i) {
            int nb = (sch == ORC_MKN) ? o : i;
            int kb = (sch == ORC_MKN) ? i : o;
            int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
            int lastk = (kb == x->Kb - 1) && x->k_pad;
            split_t s = split_of(lastk, p, x->p_l, x->k_c, x->k_rem);
            int slice = lastk ? x->k_c1 : x->k_c;
#pragma omp parallel for
            for (int core = 0; core < s.used; ++core) {
                int kc = lastk ? (core == x->p_l - 1 ? x->k_c1_last_core : x->k_c1) : x->k_c;
                size_t k0 = (size_t)kb * p * x->k_c + (size_t)core * slice;
                copy_B_block(B + k0 * N + (size_t)nb * x->n_c,
                             Bp + off + (size_t)core * slice * cols,
                             N, N - nb * x->n_c, kc, cols, nr);
            }
            off += (size_t)s.span * cols;
        }
}

/* ------------------------------------------------------------------------ */
/* pack_C / unpack_C                                                          */
/*   KMN: src/pack_k_first.cpp:404-476, src/unpack_k_first.cpp:5-67           */
/*   MKN: src/pack_m_first.cpp:150-204, src/unpack_m_first.cpp:5-49           */
/*   NKM: src/pack_n_first.cpp:150-213, src/unpack_n_first.cpp:5-49           */
/* For NKM the block offset follows unpack_n_first / schedule_NKM             */
/* (n * m_c_t * n_c); pack_n_first.cpp:205 uses n*p*m_c*n_c_t, which only     */
/* differs in the last, partial M block and disagrees with the schedule.      */
/* ------------------------------------------------------------------------ */
static void walk_C(float *C, float *Cp, int M, int N, int p,
                   const orc_blk_dims *x, const orc_cntx *cx, int sch, int to_packed)
{
    const int mr = cx->mr, nr = cx->nr;
    if (sch == ORC_KMN) {
        size_t off = 0;
        for (int nb = 0; nb < x->Nb; ++nb) {
            int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
            for (int mb = 0; mb < x->Mb; ++mb) {
                int last = (mb == x->Mb - 1) && x->m_pad;
                split_t s = split_of(last, p, x->p_l, x->m_c, mr * x->mr_rem);
                int slice = last ? x->m_c1 : x->m_c;
#pragma omp parallel for
                for (int core = 0; core < s.used; ++core) {
                    int rows = last ? (core == x->p_l - 1 ? x->m_c1_last_core : x->m_c1) : x->m_c;
                    int row0 = mb * p * x->m_c + core * slice;
                    copy_C_block(C + (size_t)row0 * N + (size_t)nb * x->n_c,
                                 Cp + off + (size_t)core * slice * cols, N,
                                 M - row0, N - nb * x->n_c, rows, cols, mr, nr, to_packed);
                }
                off += (size_t)s.span * cols;
            }
        }
    } else if (sch == ORC_MKN) {
        for (int nb = 0; nb < x->Nb; ++nb) {
            int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
#pragma omp parallel for
            for (int mb = 0; mb < x->Mb; ++mb) {
                int rows = ((mb == x->Mb - 1) && x->m_pad) ? x->m_c1 : x->m_c;
                copy_C_block(C + (size_t)mb * x->m_c * N + (size_t)nb * x->n_c,
                             Cp + (size_t)x->M_padded * nb * x->n_c + (size_t)mb * x->m_c * cols, N,
                             M - mb * x->m_c, N - nb * x->n_c, rows, cols, mr, nr, to_packed);
            }
        }
    } else if (sch == ORC_NKM) {
        int mspan = p * x->m_c;
        for (int mb = 0; mb < x->Mb; ++mb) {
            int rows = ((mb == x->Mb - 1) && x->m_pad) ? x->m_c1 : mspan;
#pragma omp parallel for
            for (int nb = 0; nb < x->Nb; ++nb) {
                int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
                copy_C_block(C + (size_t)mb * mspan * N + (size_t)nb * x->n_c,
                             Cp + (size_t)x->N_padded * mb * mspan + (size_t)nb * rows * x->n_c, N,
                             M - mb * mspan, N - nb * x->n_c, rows, cols, mr, nr, to_packed);
            }
        }
    } else {
        fprintf(stderr, "unknown schedule\n");
        exit(1);
    }
}

void orc_pack_C(float *C, float *Cp, int M, int N, int p,
                const orc_blk_dims *x, const orc_cntx *cx, int sch)
{
    walk_C(C, Cp, M, N, p, x, cx, sch, 1);
}

void orc_unpack_C(float *C, float *Cp, int M, int N, int p,
                  const orc_blk_dims *x, const orc_cntx *cx, int sch)
{
    walk_C(C, Cp, M, N, p, x, cx, sch, 0);
}

/* ------------------------------------------------------------------------ */
/* Micro-kernel: C[mr x nr] += sum_kk A[kk*mr + i] * B[kk*nr + j], one fused   */
/* multiply-add chain per element in ascending kk                             */
/* (cake_sgemm_haswell_6x16, src/kernels/haswell/dense.cpp:8-204).            */
/* ------------------------------------------------------------------------ */
static void ukernel_generic(const float *A, const float *B, float *C, int mr, int nr, int k)
{
    for (int kk = 0; kk < k; ++kk)
        for (int i = 0; i < mr; ++i) {
            float a = A[(size_t)kk * mr + i];
            for (int j = 0; j < nr; ++j)
                C[i * nr + j] = fmaf(a, B[(size_t)kk * nr + j], C[i * nr + j]);
        }
}

static void ukernel_6x16(const float *A, const float *B, float *C, int k)
{
    __m256 acc[6][2];
    for (int i = 0; i < 6; ++i) {
        acc[i][0] = _mm256_loadu_ps(C + 16 * i);
        acc[i][1] = _mm256_loadu_ps(C + 16 * i + 8);
    }
    for (int kk = 0; kk < k; ++kk, A += 6, B += 16) {
        __m256 lo = _mm256_loadu_ps(B), hi = _mm256_loadu_ps(B + 8);
#pragma GCC unroll 6
        for (int i = 0; i < 6; ++i) {
            __m256 a = _mm256_broadcast_ss(A + i);
            acc[i][0] = _mm256_fmadd_ps(a, lo, acc[i][0]);
            acc[i][1] = _mm256_fmadd_ps(a, hi, acc[i][1]);
        }
    }
    for (int i = 0; i < 6; ++i) {
        _mm256_storeu_ps(C + 16 * i, acc[i][0]);
        _mm256_storeu_ps(C + 16 * i + 8, acc[i][1]);
    }
}

void orc_ukernel(const float *A, const float *B, float *C, int mr, int nr, int k)
{
    if (mr == 6 && nr == 16) ukernel_6x16(A, B, C, k);
    else ukernel_generic(A, B, C, mr, nr, k);
}

/* One packed operation block: all (n_reg, m_reg) register tiles of an
 * rows x cols x kc block (inner loops of src/cake_sgemm_k_first.cpp:113-126). */
static void block_product(const float *a, const float *b, float *c,
                          int rows, int cols, int kc, int mr, int nr)
{
    for (int nreg = 0; nreg < cols / nr; ++nreg)
        for (int mreg = 0; mreg < rows / mr; ++mreg)
            orc_ukernel(a + (size_t)mreg * mr * kc, b + (size_t)nreg * kc * nr,
                        c + (size_t)nreg * rows * nr + (size_t)mreg * mr * nr, mr, nr, kc);
}

/* Boustrophedon index: position `step` of a walk over `count` items that
 * runs backwards when `reverse` is set. */
static int snake(int step, int count, int reverse) { return reverse ? count - 1 - step : step; }

/* ------------------------------------------------------------------------ */
/* schedule_KMN, src/cake_sgemm_k_first.cpp:9-153.  C tile stationary in a    */
/* per-core scratch across the whole K walk, then assigned (not added) to C.  */
/* ------------------------------------------------------------------------ */
void orc_schedule_KMN(const float *Ap, const float *Bp, float *C, int M, int N, int K, int p,
                      const orc_cntx *cx, const orc_blk_dims *x)
{
    const int mr = cx->mr, nr = cx->nr;
    float **scratch = (float **)malloc(sizeof(float *) * p);
    for (int i = 0; i < p; ++i) scratch[i] = (float *)calloc((size_t)x->m_c * x->n_c, sizeof(float));

    for (int nb = 0; nb < x->Nb; ++nb) {
        int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
        for (int ms = 0; ms < x->Mb; ++ms) {
            int mb = snake(ms, x->Mb, nb & 1);
            int k_reverse = (nb & 1) != (mb & 1);
            int last = (mb == x->Mb - 1) && x->m_pad;
            split_t s = split_of(last, p, x->p_l, x->m_c, mr * x->mr_rem);
            int slice = last ? x->m_c1 : x->m_c;
#pragma omp parallel for
            for (int core = 0; core < s.used; ++core) {
                int rows = last ? (core == x->p_l - 1 ? x->m_c1_last_core : x->m_c1) : x->m_c;
                float *cp = scratch[core];
                for (int ks = 0; ks < x->Kb; ++ks) {
                    int kb = snake(ks, x->Kb, k_reverse);
                    int kc = ((kb == x->Kb - 1) && x->k_pad) ? x->k_c1 : x->k_c;
                    const float *a = Ap + (size_t)mb * p * x->m_c * K + (size_t)kb * s.span * x->k_c
                                   + (size_t)core * slice * kc;
                    const float *b = Bp + (size_t)nb * K * x->n_c + (size_t)kb * x->k_c * cols;
                    block_product(a, b, cp, rows, cols, kc, mr, nr);
                }
                int row0 = mb * p * x->m_c + core * slice;
                copy_C_block(C + (size_t)row0 * N + (size_t)nb * x->n_c, cp, N,
                             M - row0, N - nb * x->n_c, rows, cols, mr, nr, 0);
                memset(cp, 0, sizeof(float) * (size_t)x->m_c * x->n_c);
            }
        }
    }
    for (int i = 0; i < p; ++i) free(scratch[i]);
    free(scratch);
}

/* ------------------------------------------------------------------------ */
/* schedule_MKN, src/cake_sgemm_m_first.cpp:4-113, and schedule_NKM,          */
/* src/cake_sgemm_n_first.cpp:4-113.  K is cut into p slices per block that   */
/* one thread walks in order; threads own whole M (resp. N) blocks of a       */
/* packed C.                                                                  */
/* ------------------------------------------------------------------------ */
void orc_schedule_MKN(const float *Ap, const float *Bp, float *Cp, int M, int N, int K, int p,
                      const orc_cntx *cx, const orc_blk_dims *x)
{
    (void)M; (void)N;
    const int mr = cx->mr, nr = cx->nr;
    for (int nb = 0; nb < x->Nb; ++nb) {
        int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
        for (int ks = 0; ks < x->Kb; ++ks) {
            int kb = snake(ks, x->Kb, nb & 1);
            int lastk = (kb == x->Kb - 1) && x->k_pad;
            split_t s = split_of(lastk, p, x->p_l, x->k_c, x->k_rem);
            int slice = lastk ? x->k_c1 : x->k_c;
#pragma omp parallel for
            for (int mb = 0; mb < x->Mb; ++mb) {
                int rows = ((mb == x->Mb - 1) && x->m_pad) ? x->m_c1 : x->m_c;
                float *c = Cp + (size_t)nb * x->M_padded * x->n_c + (size_t)mb * x->m_c * cols;
                for (int core = 0; core < s.used; ++core) {
                    int kc = lastk ? (core == x->p_l - 1 ? x->k_c1_last_core : x->k_c1) : x->k_c;
                    const float *a = Ap + (size_t)kb * x->M_padded * p * x->k_c
                                   + (size_t)mb * x->m_c * s.span + (size_t)core * rows * slice;
                    const float *b = Bp + (size_t)nb * K * x->n_c + (size_t)kb * p * x->k_c * cols
                                   + (size_t)core * slice * cols;
                    block_product(a, b, c, rows, cols, kc, mr, nr);
                }
            }
        }
    }
}

void orc_schedule_NKM(const float *Ap, const float *Bp, float *Cp, int M, int N, int K, int p,
                      const orc_cntx *cx, const orc_blk_dims *x)
{
    (void)M; (void)N;
    const int mr = cx->mr, nr = cx->nr;
    const int mspan = p * x->m_c;
    for (int mb = 0; mb < x->Mb; ++mb) {
        int rows = ((mb == x->Mb - 1) && x->m_pad) ? x->m_c1 : mspan;
        for (int ks = 0; ks < x->Kb; ++ks) {
            int kb = snake(ks, x->Kb, mb & 1);
            int lastk = (kb == x->Kb - 1) && x->k_pad;
            split_t s = split_of(lastk, p, x->p_l, x->k_c, x->k_rem);
            int slice = lastk ? x->k_c1 : x->k_c;
#pragma omp parallel for
            for (int nb = 0; nb < x->Nb; ++nb) {
                int cols = ((nb == x->Nb - 1) && x->n_pad) ? x->n_c1 : x->n_c;
                float *c = Cp + (size_t)mb * mspan * x->N_padded + (size_t)rows * nb * x->n_c;
                for (int core = 0; core < s.used; ++core) {
                    int kc = lastk ? (core == x->p_l - 1 ? x->k_c1_last_core : x->k_c1) : x->k_c;
                    const float *a = Ap + (size_t)mb * mspan * K + (size_t)rows * kb * p * x->k_c
                                   + (size_t)core * rows * slice;
                    const float *b = Bp + (size_t)kb * p * x->k_c * x->N_padded
                                   + (size_t)nb * x->n_c * s.span + (size_t)core * slice * cols;
                    block_product(a, b, c, rows, cols, kc, mr, nr);
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------ */
/* cake_sgemm, src/cake_sgemm.cpp:9-175.  Returns wall seconds of             */
/* plan + pack + compute + unpack like the reference.  alpha is ignored; beta */
/* is only tested against zero and only for MKN/NKM, where it means "start    */
/* from the existing C" (:114).  KMN assigns.                                 */
/* ------------------------------------------------------------------------ */
double orc_cake_sgemm(float *A, float *B, float *C, int M, int N, int K, int p, orc_cntx *cx,
                      int packedA, int packedB, float alpha, float beta, int sch,
                      int mcu, int kcu, int ncu, orc_blk_dims *dims_out)
{
    (void)alpha;
    orc_cntx local;
    if (!cx) { orc_query_cntx(&local); cx = &local; }
    omp_set_num_threads(p);
    double t0 = now_s();

    orc_blk_dims x;
    orc_init_block_dims(M, N, K, p, &x, cx, sch, mcu, kcu, ncu);
    sch = x.sch;
    if (dims_out) *dims_out = x;

    float *Ap = A, *Bp = B;
    if (!packedA) {
        if (posix_memalign((void **)&Ap, 64, orc_packed_A_size(M, K, p, &x, cx, sch) + 64)) exit(1);
        orc_pack_A(A, Ap, M, K, p, &x, cx, sch);
    }
    if (!packedB) {
        if (posix_memalign((void **)&Bp, 64, orc_packed_B_size(K, N, p, &x, cx) + 64)) exit(1);
        orc_pack_B(B, Bp, K, N, p, &x, cx, sch);
    }

    if (sch == ORC_KMN) {
        orc_schedule_KMN(Ap, Bp, C, M, N, K, p, cx, &x);
    } else {
        size_t csz = orc_packed_C_size(M, N, p, &x, cx, sch);
        float *Cp;
        if (beta != 0) {
            if (posix_memalign((void **)&Cp, 64, csz + 64)) exit(1);
            orc_pack_C(C, Cp, M, N, p, &x, cx, sch);
        } else {
            Cp = (float *)calloc(csz / sizeof(float) + 16, sizeof(float));
        }
        if (sch == ORC_MKN) orc_schedule_MKN(Ap, Bp, Cp, M, N, K, p, cx, &x);
        else orc_schedule_NKM(Ap, Bp, Cp, M, N, K, p, cx, &x);
        orc_unpack_C(C, Cp, M, N, p, &x, cx, sch);
        free(Cp);
    }
    double dt = now_s() - t0;
    if (!packedA) free(Ap);
    if (!packedB) free(Bp);
    return dt;
}

/* ------------------------------------------------------------------------ */
/* cake_sgemv (examples/cake_gemv.cpp): y[m] += sum_k A[k*M + m] * x[k],      */
/* A column-major, sequential fused multiply-add over ascending k.            */
/*   get_cache_dims_mvm :273-340, init_block_dims_mvm :344-418,               */
/*   schedule_mvm :424-490, cake_sgemv_haswell_8x8_col :89-140,               */
/*   cake_sgemv :716-767 (always KMN).                                        */
/* The reference's row kernel is 8 wide whatever cntx->mr says and runs past  */
/* row M when M is not a multiple of mr; here the tail rows are masked.       */
/* ------------------------------------------------------------------------ */
void orc_init_block_dims_mvm(int M, int K, int p, orc_blk_dims *x, const orc_cntx *cx)
{
    const int mr = cx->mr;
    memset(x, 0, sizeof *x);
    int mc = (int)((-2 + sqrt(4.0 + 4.0 * ((double)cx->L2 / 4.0))) / 2.0);
    mc += 64 - (mc % 64);
    int mc_ret = mc;
    if (M < p * mr) {
        mc_ret = mr;
    } else if (M < p * mc) {
        int a = M / p;
        mc_ret = (a < mr) ? mr : a + (mr - (a % mr));
    }
    x->m_c = x->k_c = mc_ret;
    x->sch = ORC_KMN;
    int span = p * x->m_c;
    x->k_pad = (K % x->k_c) ? 1 : 0;
    x->m_pad = (M % span) ? 1 : 0;
    x->mr_rem = ceil_ratio(M % span, mr);
    int per_core = ceil_ratio(x->mr_rem, p);
    x->p_l = per_core ? ceil_ratio(x->mr_rem, per_core) : 0;
    x->m_c1 = per_core * mr;
    x->m_c1_last_core = (per_core - (x->p_l * per_core - x->mr_rem)) * mr;
    x->k_c1 = K % x->k_c;
    x->Mb = M / span + x->m_pad;
    x->Kb = K / x->k_c + x->k_pad;
    x->M_padded = mr * x->mr_rem + (M / span) * span;
}

static void gemv_rows(const float *A, const float *xv, float *y, int rows, int k, int M)
{
    if (rows == 8) {
        __m256 acc = _mm256_loadu_ps(y);
        for (int kk = 0; kk < k; ++kk)
            acc = _mm256_fmadd_ps(_mm256_loadu_ps(A + (size_t)kk * M), _mm256_broadcast_ss(xv + kk), acc);
        _mm256_storeu_ps(y, acc);
        return;
    }
    for (int kk = 0; kk < k; ++kk)
        for (int i = 0; i < rows; ++i)
            y[i] = fmaf(A[(size_t)kk * M + i], xv[kk], y[i]);
}

double orc_cake_sgemv(const float *A, const float *xv, float *y, int M, int K, int p, orc_cntx *cx)
{
    orc_cntx local;
    if (!cx) { orc_query_cntx(&local); local.mr = 8; cx = &local; }
    omp_set_num_threads(p);
    orc_blk_dims x;
    orc_init_block_dims_mvm(M, K, p, &x, cx);
    const int mr = cx->mr;
    double t0 = now_s();
    for (int mb = 0; mb < x.Mb; ++mb) {
        int last = (mb == x.Mb - 1) && x.m_pad;
        int used = last ? x.p_l : p;
        int slice = last ? x.m_c1 : x.m_c;
#pragma omp parallel for
        for (int core = 0; core < used; ++core) {
            int rows = last ? (core == x.p_l - 1 ? x.m_c1_last_core : x.m_c1) : x.m_c;
            int row0 = mb * p * x.m_c + core * slice;
            for (int kb = 0; kb < x.Kb; ++kb) {
                int kc = ((kb == x.Kb - 1) && x.k_pad) ? x.k_c1 : x.k_c;
                for (int r = 0; r < rows; r += mr) {
                    int live = M - (row0 + r);
                    if (live <= 0) break;
                    if (live > mr) live = mr;
                    gemv_rows(A + (size_t)kb * x.k_c * M + row0 + r, xv + (size_t)kb * x.k_c,
                              y + row0 + r, live, kc, M);
                }
            }
        }
    }
    return now_s() - t0;
}

/* ------------------------------------------------------------------------ */
/* im_2_col, examples/cake_conv.cpp:1178-1213: one CHW image, no padding,     */
/* unit stride (the stride argument is accepted and never used there):        */
/*   out[(c*Hf*Wf + h*Wf + w) * (Hout*Wout) + ho*Wout + wo]                   */
/*       = In[c][ho + h][wo + w].                                             */
/* orc_im2col generalises it to a batch (column n = b*Hout*Wout + ho*Wout+wo),*/
/* zero padding and stride; with batch 1, pad 0, stride 1 it is the same map. */
/* ------------------------------------------------------------------------ */
void orc_im2col(const float *in, float *out, int batch, int Cin, int Hin, int Win,
                int Hf, int Wf, int Hout, int Wout, int stride, int pad)
{
    const size_t Ncols = (size_t)batch * Hout * Wout;
#pragma omp parallel for collapse(2)
    for (int c = 0; c < Cin; ++c)
        for (int h = 0; h < Hf; ++h)
            for (int w = 0; w < Wf; ++w) {
                float *row = out + ((size_t)c * Hf * Wf + (size_t)h * Wf + w) * Ncols;
                for (int b = 0; b < batch; ++b)
                    for (int ho = 0; ho < Hout; ++ho)
                        for (int wo = 0; wo < Wout; ++wo) {
                            int hi = ho * stride + h - pad, wi = wo * stride + w - pad;
                            float v = 0.0f;
                            if (hi >= 0 && hi < Hin && wi >= 0 && wi < Win)
                                v = in[(((size_t)b * Cin + c) * Hin + hi) * Win + wi];
                            row[((size_t)b * Hout + ho) * Wout + wo] = v;
                        }
            }
}

void orc_im_2_col(const float *in, float *out, int Wf, int Hf, int Win, int Hin,
                  int Wout, int Hout, int Cin)
{
    orc_im2col(in, out, 1, Cin, Hin, Win, Hf, Wf, Hout, Wout, 1, 0);
}

/* ------------------------------------------------------------------------ */
/* Closed-form checkers (not restatements): fp64 product with the             */
/* normaliser S[m][n] = sum_k |a||b|, the error metric, naive convolution.    */
/* ------------------------------------------------------------------------ */
void orc_gemm_f64(const float *A, const float *B, int M, int N, int K, double *C64, double *S)
{
#pragma omp parallel for schedule(dynamic, 4)
    for (int m = 0; m < M; ++m) {
        double *c = C64 + (size_t)m * N, *s = S ? S + (size_t)m * N : NULL;
        for (int n = 0; n < N; ++n) { c[n] = 0.0; if (s) s[n] = 0.0; }
        for (int k = 0; k < K; ++k) {
            double a = A[(size_t)m * K + k], aa = fabs(a);
            const float *b = B + (size_t)k * N;
            if (s) for (int n = 0; n < N; ++n) { c[n] += a * b[n]; s[n] += aa * fabs((double)b[n]); }
            else   for (int n = 0; n < N; ++n) c[n] += a * b[n];
        }
    }
}

/* max over elements of |C - C64| / S (elements with S == 0 must match exactly). */
double orc_max_rel_err(const float *C, const double *C64, const double *S, size_t n)
{
    double worst = 0.0;
#pragma omp parallel for reduction(max : worst)
    for (size_t i = 0; i < n; ++i) {
        double d = fabs((double)C[i] - C64[i]);
        double e = (S[i] > 0.0) ? d / S[i] : (d == 0.0 ? 0.0 : INFINITY);
        if (!(e <= worst)) worst = e; /* NaN propagates as the worst case */
    }
    return worst;
}

/* y64[m] = sum_k A(m,k) x[k], S[m] = sum_k |A||x|; A row- or column-major. */
void orc_gemv_f64(const float *A, const float *xv, int M, int K, int col_major, double *y64, double *S)
{
#pragma omp parallel for
    for (int m = 0; m < M; ++m) {
        double acc = 0.0, s = 0.0;
        for (int k = 0; k < K; ++k) {
            double a = col_major ? A[(size_t)k * M + m] : A[(size_t)m * K + k];
            acc += a * xv[k];
            s += fabs(a) * fabs((double)xv[k]);
        }
        y64[m] = acc;
        if (S) S[m] = s;
    }
}

/* out[b][co][ho][wo] in fp64 from NCHW input and OIHW weights. */
void orc_conv_naive_f64(const float *in, const float *wt, double *out, double *S, int batch,
                        int Cin, int Hin, int Win, int Cout, int Hf, int Wf,
                        int Hout, int Wout, int stride, int pad)
{
#pragma omp parallel for collapse(2)
    for (int b = 0; b < batch; ++b)
        for (int co = 0; co < Cout; ++co)
            for (int ho = 0; ho < Hout; ++ho)
                for (int wo = 0; wo < Wout; ++wo) {
                    double acc = 0.0, s = 0.0;
                    for (int ci = 0; ci < Cin; ++ci)
                        for (int h = 0; h < Hf; ++h)
                            for (int w = 0; w < Wf; ++w) {
                                int hi = ho * stride + h - pad, wi = wo * stride + w - pad;
                                if (hi < 0 || hi >= Hin || wi < 0 || wi >= Win) continue;
                                double a = wt[(((size_t)co * Cin + ci) * Hf + h) * Wf + w];
                                double v = in[(((size_t)b * Cin + ci) * Hin + hi) * Win + wi];
                                acc += a * v;
                                s += fabs(a) * fabs(v);
                            }
                    size_t o = (((size_t)b * Cout + co) * Hout + ho) * Wout + wo;
                    out[o] = acc;
                    if (S) S[o] = s;
                }
}

/* ------------------------------------------------------------------------ */
/* Blocks of the direct convolution and the packed filters of cake_sconv.    */
/*   get_cache_dims_conv   examples/cake_conv.cpp:262-329                     */
/*   init_block_dims_conv  examples/cake_conv.cpp:333-425 (K-first case)      */
/*   pack_filters          examples/cake_conv.cpp:536-610                     */
/*   pack_ob_A_single_buf_conv  examples/cake_conv.cpp:430-454                */
/* Pinned bit for bit against those functions compiled from the reference    */
/* (oracle/_ref) and their committed outputs (tests/golden), and by a        */
/* hand-computed block table.                                                 */
/* ------------------------------------------------------------------------ */
void orc_init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout,
                              int s, int p, orc_blk_dims *x, const orc_cntx *cx)
{
    (void)Hin; (void)s;
    const int mr = cx->mr;
    memset(x, 0, sizeof *x);
    /* output channels per core: an even share, whole m_r panels */
    int share = (int)ceil((double)Cout / p);
    share -= share % mr;
    int mc = share;
    if (Cout < p * mr) mc = mr;
    else if (Cout < p * share) {
        int a = Cout / p;
        mc = a < mr ? mr : a + (mr - a % mr);
    }
    /* rows of the output image per block, then the channels that still fit the L2 */
    int rows = (int)floor((cx->alpha_n * p * mc) / Wout);
    if (rows == 0) rows = 1;
    int ck = (int)ceil((((double)cx->L2) / 4.0 - (double)rows * Wout * mc) /
                       ((double)mc * Wf * Hf + (double)rows * Win));
    if (ck > Cin) ck = Cin;
    else if (ck < 0) ck = 128;
    if (ck == 0) ck = 1;   /* the reference would go on to divide by it */
    x->m_c = mc; x->k_c = ck; x->n_c = rows; x->sch = ORC_KMN;

    const int block_rows = p * mc;
    const int left = Cout % block_rows;
    x->m_pad = left != 0;
    x->k_pad = Cin % ck != 0;
    x->n_pad = Hout % rows != 0;
    x->mr_rem = ceil_ratio(left, mr);
    int panels = ceil_ratio(x->mr_rem, p);
    x->p_l = panels ? ceil_ratio(x->mr_rem, panels) : 0;
    x->m_c1 = panels * mr;
    x->m_c1_last_core = (panels - (x->p_l * panels - x->mr_rem)) * mr;
    x->k_c1 = Cin % ck;
    x->n_c1 = Hout % rows;
    x->Mb = Cout / block_rows + x->m_pad;
    x->Kb = Cin / ck + x->k_pad;
    x->Nb = Hout / rows + x->n_pad;
    x->M_padded = mr * x->mr_rem + (Cout / block_rows) * block_rows;
    x->N_padded = (Hout - Hout % rows) + x->n_c1;
}

/* F[Cout][Cin][taps] -> K-first blocks whose m_r panels hold [tap][channel][m_r]. */
void orc_pack_filters(const float *F, float *Fp, int Cout, int Cin, int taps, int p,
                      const orc_blk_dims *x, const orc_cntx *cx)
{
    const int mr = cx->mr;
    const size_t K = (size_t)Cin * taps;
    size_t off = 0;
    for (int mb = 0; mb < x->Mb; ++mb) {
        int last = (mb == x->Mb - 1) && x->m_pad;
        split_t sp = split_of(last, p, x->p_l, x->m_c, mr * x->mr_rem);
        int slice = last ? x->m_c1 : x->m_c;
        for (int kb = 0; kb < x->Kb; ++kb) {
            int kc = ((kb == x->Kb - 1) && x->k_pad) ? x->k_c1 : x->k_c;
            for (int core = 0; core < sp.used; ++core) {
                int rows = last ? (core == x->p_l - 1 ? x->m_c1_last_core : x->m_c1) : x->m_c;
                size_t row0 = (size_t)mb * p * x->m_c + (size_t)core * slice;
                float *dst = Fp + off + (size_t)core * slice * kc * taps;
                for (int panel = 0; panel < rows; panel += mr)
                    for (int t = 0; t < taps; ++t)
                        for (int c = 0; c < kc; ++c)
                            for (int j = 0; j < mr; ++j) {
                                size_t r = row0 + panel + j;
                                *dst++ = r < (size_t)Cout
                                             ? F[r * K + ((size_t)kb * x->k_c + c) * taps + t] : 0.f;
                            }
            }
            off += (size_t)sp.span * kc * taps;
        }
    }
}

int orc_sizeof_blk_dims(void) { return (int)sizeof(orc_blk_dims); }
