// dropin_test.cpp -- a caller written the way the reference's example mains are
// (examples/cake_sgemm_test.cpp, examples/cake_gemv.cpp, examples/cake_conv.cpp:
// query the context, rand_init, call, check against a naive host loop), compiled
// against include/cake.h and linked to libcake.so only.  Prints one line per
// case and "ALL PASS" at the end; exit status 0 only if every case passed.
#include <math.h>

#include <thread>

#include "cake.h"

static int failures = 0;

static void report(const char* what, bool ok)
{
    printf("%-58s %s\n", what, ok ? "ok" : "FAILED");
    fflush(stdout);
    if (!ok) ++failures;
}

static bool close_to_naive(float* A, float* B, float* C, int M, int N, int K)
{
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double acc = 0, mag = 0;
            for (int k = 0; k < K; ++k) {
                acc += (double)A[(size_t)m * K + k] * B[(size_t)k * N + n];
                mag += fabs((double)A[(size_t)m * K + k] * B[(size_t)k * N + n]);
            }
            if (fabs(acc - C[(size_t)m * N + n]) > 1e-4 * (mag > 0 ? mag : 1)) return false;
        }
    return true;
}

static void sgemm_case(int M, int K, int N, int p, enum sched sch, cake_cntx_t* cntx)
{
    float* A = (float*)malloc(sizeof(float) * M * K);
    float* B = (float*)malloc(sizeof(float) * K * N);
    float* C = (float*)calloc((size_t)M * N, sizeof(float));
    rand_init(A, M, K);
    rand_init(B, K, N);
    double t = cake_sgemm(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 0, sch);
    char what[128];
    snprintf(what, sizeof what, "cake_sgemm M=%d K=%d N=%d p=%d sch=%d (%.4f s)", M, K, N, p, (int)sch, t);
    report(what, close_to_naive(A, B, C, M, N, K));
    free(A); free(B); free(C);
}

static void variants_case(cake_cntx_t* cntx)
{
    const int M = 111, K = 96, N = 213, p = 3;
    float* A = (float*)malloc(sizeof(float) * M * K);
    float* B = (float*)malloc(sizeof(float) * K * N);
    rand_init(A, M, K);
    rand_init(B, K, N);
    float* C = (float*)calloc((size_t)M * N, sizeof(float));
    cake_sgemm_2d(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 0, KMN);
    report("cake_sgemm_2d", close_to_naive(A, B, C, M, N, K));
    memset(C, 0, sizeof(float) * M * N);
    cake_sgemm_online(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 0, KMN);
    report("cake_sgemm_online", close_to_naive(A, B, C, M, N, K));
    memset(C, 0, sizeof(float) * M * N);
    cake_sgemm_test(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 1, NKM);   // K-first whatever is asked: C assigned
    report("cake_sgemm_test", close_to_naive(A, B, C, M, N, K));
    memset(C, 0, sizeof(float) * M * N);
    cake_sgemm(A, B, C, M, N, K, p, NULL);  // NULL context, all defaults
    report("cake_sgemm default arguments, NULL context", !cake_sgemm_checker(A, B, C, N, M, K));
    free(A); free(B); free(C);
}

// the packed path of examples/cake_conv.cpp:1007-1066
static void conv_case(cake_cntx_t* cntx)
{
    const int Cin = 8, Cout = 20, Hf = 3, Wf = 3, Hout = 12, Wout = 10, Hin = Hout + 2, Win = Wout + 2, p = 4;
    const int M = Cout, K = Cin * Hf * Wf, N = Hout * Wout;
    float* F = (float*)malloc(sizeof(float) * M * K);
    float* In = (float*)malloc(sizeof(float) * Cin * Hin * Win);
    rand_init(F, M, K);
    rand_init(In, Cin, Hin * Win);
    float* Bm = im_2_col(In, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, 1);
    bool cols_ok = true;
    for (int c = 0; c < Cin && cols_ok; ++c)
        for (int h = 0; h < Hf; ++h)
            for (int w = 0; w < Wf; ++w)
                for (int ho = 0; ho < Hout; ++ho)
                    for (int wo = 0; wo < Wout; ++wo)
                        if (Bm[(size_t)(c * Hf * Wf + h * Wf + w) * N + ho * Wout + wo] !=
                            In[(size_t)c * Hin * Win + (ho + h) * Win + wo + w])
                            cols_ok = false;
    report("im_2_col layout", cols_ok);

    enum sched sch = KMN;
    blk_dims_t* x = (blk_dims_t*)malloc(sizeof(blk_dims_t));
    init_block_dims(M, N, K, p, x, cntx, sch, NULL, 0);
    float* A_p = (float*)malloc(cake_sgemm_packed_A_size(M, K, p, x, cntx, sch));
    float* B_p = (float*)malloc(cake_sgemm_packed_B_size(K, N, p, x, cntx));
    pack_A(F, A_p, M, K, p, x, cntx, sch);
    pack_B(Bm, B_p, K, N, p, x, cntx, sch);
    float* C = (float*)calloc((size_t)M * N, sizeof(float));
    cake_sgemm(A_p, B_p, C, M, N, K, p, cntx, NULL, 1, 1, 1, 0, KMN);
    report("cake_sgemm(packedA=1, packedB=1) after pack_A/pack_B", close_to_naive(F, Bm, C, M, N, K));

    // direct convolution as the independent answer
    bool conv_ok = true;
    for (int co = 0; co < Cout && conv_ok; ++co)
        for (int ho = 0; ho < Hout; ++ho)
            for (int wo = 0; wo < Wout; ++wo) {
                double acc = 0;
                for (int c = 0; c < Cin; ++c)
                    for (int h = 0; h < Hf; ++h)
                        for (int w = 0; w < Wf; ++w)
                            acc += (double)F[(size_t)co * K + c * Hf * Wf + h * Wf + w] *
                                   In[(size_t)c * Hin * Win + (ho + h) * Win + wo + w];
                if (fabs(acc - C[(size_t)co * N + ho * Wout + wo]) > 1e-3) conv_ok = false;
            }
    report("im2col GEMM equals direct convolution", conv_ok);

    // pack_C / unpack_C round trip
    float* C_p = (float*)malloc(cake_sgemm_packed_C_size(M, N, p, x, cntx, sch));
    float* C2 = (float*)calloc((size_t)M * N, sizeof(float));
    pack_C(C, C_p, M, N, p, x, cntx, sch);
    unpack_C(C2, C_p, M, N, p, x, cntx, sch);
    report("unpack_C(pack_C(C)) == C", memcmp(C, C2, sizeof(float) * M * N) == 0);
    free(F); free(In); free(Bm); free(x); free(A_p); free(B_p); free(C); free(C_p); free(C2);
}

// examples/cake_conv.cpp main: the direct convolution against the im2col product of the same
// filters and image (conv_gemm_checker, :1216-1234), on a geometry whose sizes agree
static void sconv_case(cake_cntx_t* cntx, int Cin, int Cout, int Hin, int Win, int Hf, int Wf)
{
    const int Hout = Hin - Hf + 1, Wout = Win - Wf + 1, p = 4, s = 1;
    const int M = Cout, K = Cin * Hf * Wf, N = Hout * Wout;
    float* F = (float*)malloc(sizeof(float) * M * K);
    float* In = (float*)malloc(sizeof(float) * Cin * Hin * Win);
    rand_init(F, M, K);
    rand_init(In, Cin, Hin * Win);
    float* Out = (float*)calloc((size_t)M * N, sizeof(float));
    cake_sconv(F, In, Out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cntx);
    float* Bm = im_2_col(In, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s);
    float* C = (float*)calloc((size_t)M * N, sizeof(float));
    cake_sgemm(F, Bm, C, M, N, K, p, cntx, NULL, 0, 0, 1, 0, KMN);
    conv_gemm_checker(Out, C, M, N);
    bool ok = close_to_naive(F, Bm, Out, M, N, K);
    for (size_t i = 0; i < (size_t)M * N && ok; ++i)
        if (fabsf(Out[i] - C[i]) > 1e-3f) ok = false;
    cake_sconv(F, In, Out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cntx);   // adds to Out
    for (size_t i = 0; i < (size_t)M * N && ok; ++i)
        if (fabsf(Out[i] - 2 * C[i]) > 2e-3f) ok = false;
    char what[128];
    snprintf(what, sizeof what, "cake_sconv %dx%d filters, %d->%d channels on %dx%d", Hf, Wf, Cin, Cout, Hin, Win);
    report(what, ok);
    free(F); free(In); free(Out); free(Bm); free(C);
}

// cake_sconv with packedA: the reference's sequence (examples/cake_conv.cpp:791-805) -- blocks from
// init_block_dims_conv, a buffer of cake_sgemm_packed_A_size bytes, pack_filters, then the call.
static void packed_sconv_case(cake_cntx_t* cntx, int Cin, int Cout, int Hin, int Win)
{
    const int Hf = 3, Wf = 3, Hout = Hin - 2, Wout = Win - 2, p = 4, s = 1;
    const int M = Cout, K = Cin * 9, N = Hout * Wout;
    float* F = (float*)malloc(sizeof(float) * M * K);
    float* In = (float*)malloc(sizeof(float) * Cin * Hin * Win);
    rand_init(F, M, K);
    rand_init(In, Cin, Hin * Win);
    float* plain = (float*)calloc((size_t)M * N, sizeof(float));
    float* packed = (float*)calloc((size_t)M * N, sizeof(float));
    cake_sconv(F, In, plain, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cntx);
    blk_dims_t x;
    init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, &x, cntx, KMN, NULL);
    const size_t bytes = cake_sgemm_packed_A_size(Cout, K, p, &x, cntx, KMN);
    float* F_p = (float*)malloc(bytes);
    pack_filters(F, F_p, Cout, K, p, &x, cntx);
    // the layout, from its definition: the first m_r panel of the first block holds [tap][channel][m_r]
    bool layout = bytes == sizeof(float) * (size_t)x.M_padded * K;
    const int kc = x.Kb == 1 && x.k_pad ? x.k_c1 : x.k_c;
    for (int t = 0; t < 9 && layout; ++t)
        for (int c = 0; c < kc; ++c)
            for (int j = 0; j < cntx->mr; ++j) {
                const float want = j < Cout ? F[(size_t)j * K + c * 9 + t] : 0.f;
                if (F_p[((size_t)t * kc + c) * cntx->mr + j] != want) layout = false;
            }
    cake_sconv(F_p, In, packed, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cntx, NULL, 1);
    char what[128];
    snprintf(what, sizeof what, "pack_filters layout, %d->%d channels", Cin, Cout);
    report(what, layout);
    snprintf(what, sizeof what, "cake_sconv packedA=1 equals packedA=0, %d->%d on %dx%d", Cin, Cout, Hin, Win);
    report(what, memcmp(plain, packed, sizeof(float) * M * N) == 0);
    free(F); free(In); free(plain); free(packed); free(F_p);
}

// The 2-D block sizing is host arithmetic; 3000^3 on 8 cores with L1 = 32 KiB, L2 = 1 MiB, worked
// out by hand from src/block_sizing.cpp:639-779: a 4 x 2 grid of 354 x 368 blocks, k_c = 368.
static void dims_2d_case(cake_cntx_t* cntx)
{
    cake_cntx_t c = *cntx;
    c.mr = 6; c.nr = 16; c.L1 = 32 << 10; c.L2 = 1 << 20; c.ncores = 8;
    report("grid_dims_2d", grid_dims_2d(3000, 3000, 3000, 8, 8) == 2 && grid_dims_2d(1000, 1600, 1, 10, 10) == 5);
    blk_dims_t x;
    init_block_dims_2d(3000, 3000, 3000, 8, &x, &c, KMN, NULL);
    report("init_block_dims_2d", x.pm == 4 && x.pn == 2 && x.m_c == 354 && x.n_c == 368 && x.k_c == 368 && x.Mb == 3 &&
                                     x.Nb == 5 && x.Kb == 9 && x.m_c1 == 42 && x.n_c1 == 32 && x.N_padded == 3008);
    init_block_dims_2d_small(100, 200, 500, 8, &x, &c, KMN, NULL);
    report("init_block_dims_2d_small", x.pm == 2 && x.pn == 4 && x.m_c == 54 && x.n_c == 64 && x.k_c == 54 &&
                                           x.m_c1 == 48 && x.n_c1 == 16 && x.Kb == 10);
}

// Two host threads, each with a cntx of its own: each cntx works on a device context of its own
// (its blis_cntx field names it), so the calls do not take turns; the results are those of the same
// calls made one after the other.
static void two_cntx_case()
{
    const int M = 700, K = 900, N = 500, p = 4;
    float* A = (float*)malloc(sizeof(float) * M * K);
    float* B = (float*)malloc(sizeof(float) * K * N);
    rand_init(A, M, K);
    rand_init(B, K, N);
    float* alone = (float*)calloc((size_t)M * N, sizeof(float));
    cake_cntx_t* c0 = cake_query_cntx();
    cake_sgemm(A, B, alone, M, N, K, p, c0);
    cake_cntx_t* cx[2] = {cake_query_cntx(), cake_query_cntx()};
    float* C[2] = {(float*)calloc((size_t)M * N, sizeof(float)), (float*)calloc((size_t)M * N, sizeof(float))};
    bool same[2] = {true, true};
    std::thread t[2];
    for (int i = 0; i < 2; ++i)
        t[i] = std::thread([&, i] {
            for (int rep = 0; rep < 5; ++rep) {
                cake_sgemm(A, B, C[i], M, N, K, p, cx[i]);
                if (memcmp(C[i], alone, sizeof(float) * M * N) != 0) same[i] = false;
            }
        });
    for (int i = 0; i < 2; ++i) t[i].join();
    report("two threads, a cntx each: results of the single calls", same[0] && same[1]);
    report("each cntx names a device context of its own", cx[0]->blis_cntx && cx[1]->blis_cntx &&
                                                              cx[0]->blis_cntx != cx[1]->blis_cntx &&
                                                              c0->blis_cntx != cx[0]->blis_cntx);
    free(A); free(B); free(alone); free(C[0]); free(C[1]); free(c0); free(cx[0]); free(cx[1]);
}

// beta with the default schedule: whether C is added to follows the schedule init_block_dims
// resolves from the caller's cntx and p (src/cake_sgemm.cpp:34-35,114), not the device's tiling.
static void beta_case(int M, int K, int N, int p, cake_cntx_t* cntx)
{
    float* A = (float*)malloc(sizeof(float) * M * K);
    float* B = (float*)malloc(sizeof(float) * K * N);
    float* C0 = (float*)malloc(sizeof(float) * M * N);
    float* C = (float*)malloc(sizeof(float) * M * N);
    float* P = (float*)calloc((size_t)M * N, sizeof(float));
    rand_init(A, M, K);
    rand_init(B, K, N);
    rand_init(C0, M, N);
    memcpy(C, C0, sizeof(float) * M * N);
    blk_dims_t x;
    init_block_dims(M, N, K, p, &x, cntx, NA, NULL);
    cake_sgemm(A, B, P, M, N, K, p, cntx, NULL, 0, 0, 1, 0, KMN);    // the plain product
    cake_sgemm(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 1);         // sch = NA, beta = 1
    const bool adds = x.sch != KMN;
    bool ok = true;
    for (size_t i = 0; i < (size_t)M * N && ok; ++i)
        if (fabs((double)C[i] - ((double)P[i] + (adds ? C0[i] : 0.f))) > 1e-4 * (fabs(P[i]) + 1)) ok = false;
    char what[128];
    snprintf(what, sizeof what, "cake_sgemm beta=1 sch=NA M=%d K=%d N=%d p=%d: %s C", M, K, N, p,
             adds ? "adds to" : "assigns");
    report(what, ok);
    // the pack-on-the-fly entry point is K-first whatever it is asked for: it assigns
    memcpy(C, C0, sizeof(float) * M * N);
    cake_sgemm_online(A, B, C, M, N, K, p, cntx, NULL, 0, 0, 1, 1, MKN);
    report("cake_sgemm_online beta=1 sch=MKN assigns C", memcmp(C, P, sizeof(float) * M * N) == 0);
    free(A); free(B); free(C0); free(C); free(P);
}

// K = 0: the sum is empty.  With sch = NA there is nothing to size a block for and the product is
// K-first, which assigns (C becomes zero whatever beta says); M-first asked for by name keeps C.
static void empty_k_case(cake_cntx_t* cntx)
{
    const int M = 5, N = 7;
    float A[1] = {0}, B[1] = {0};
    float C[M * N];
    for (int i = 0; i < M * N; ++i) C[i] = 3.f;
    cake_sgemm(A, B, C, M, N, 0, 4, cntx, NULL, 0, 0, 1, 1);
    bool zero = true;
    for (int i = 0; i < M * N; ++i) zero = zero && C[i] == 0.f;
    report("cake_sgemm K=0 beta=1 sch=NA assigns zero", zero);
    for (int i = 0; i < M * N; ++i) C[i] = 3.f;
    cake_sgemm(A, B, C, M, N, 0, 4, cntx, NULL, 0, 0, 1, 1, MKN);
    bool kept = true;
    for (int i = 0; i < M * N; ++i) kept = kept && C[i] == 3.f;
    report("cake_sgemm K=0 beta=1 sch=MKN keeps C", kept);
}

// examples/cake_gemv.cpp main: column-major A, mr = 8, y accumulates
static void gemv_case(cake_cntx_t* cntx, int M, int K)
{
    float* A = (float*)malloc(sizeof(float) * M * K);
    float* x = (float*)malloc(sizeof(float) * K);
    float* y = (float*)calloc(M, sizeof(float));
    rand_init(A, M, K);
    rand_init(x, K, 1);
    cntx->mr = 8;
    cake_sgemv(A, x, y, M, K, 4, cntx);
    cake_sgemv(A, x, y, M, K, 4, cntx);  // second call doubles y
    bool ok = true;
    for (int m = 0; m < M && ok; ++m) {
        double acc = 0, mag = 0;
        for (int k = 0; k < K; ++k) {
            acc += (double)A[(size_t)k * M + m] * x[k];
            mag += fabs((double)A[(size_t)k * M + m] * x[k]);
        }
        if (fabs(2 * acc - y[m]) > 2e-4 * (mag > 0 ? mag : 1)) ok = false;
    }
    char what[96];
    snprintf(what, sizeof what, "cake_sgemv M=%d K=%d (column-major, accumulating)", M, K);
    report(what, ok);
    cntx->mr = 6;
    free(A); free(x); free(y);
}

static void transpose_case(int K, int N)
{
    float* A = (float*)malloc(sizeof(float) * K * N);
    float* At = (float*)malloc(sizeof(float) * K * N);
    rand_init(A, K, N);
    transpose_mat(A, At, K, N, 8, 8);
    bool ok = true;
    for (int k = 0; k < K && ok; ++k)
        for (int n = 0; n < N; ++n)
            if (At[(size_t)n * K + k] != A[(size_t)k * N + n]) ok = false;
    char what[64];
    snprintf(what, sizeof what, "transpose_mat K=%d N=%d", K, N);
    report(what, ok);
    free(A); free(At);
}

int main(int argc, char** argv)
{
    if (argc > 1 && strcmp(argv[1], "run_tests") == 0) return run_tests();  // the reference's own sweep
    srand(1);
    cake_cntx_t* cntx = cake_query_cntx();
    printf("cntx: mr=%d nr=%d L2=%d L3=%d ncores=%d\n", cntx->mr, cntx->nr, cntx->L2, cntx->L3, cntx->ncores);
    const int dims[] = {1, 10, 96, 111, 300};  // subset of src/util.cpp:11-13
    for (int mi = 0; mi < 5; ++mi)
        for (int ki = 0; ki < 5; ++ki)
            for (int ni = 0; ni < 5; ++ni) {
                enum sched sch = (enum sched)((mi + ki + ni) % 4);
                sgemm_case(dims[mi], dims[ki], dims[ni], 2 + (mi + ni) % 3, sch, cntx);
            }
    sgemm_case(960, 2111, 333, 8, NA, cntx);
    variants_case(cntx);
    {
        // a fixed host description, so the resolved schedules do not depend on the test machine:
        // 1024^3 with p = 8 is M-first and 200 x 300 x 3000 N-first for it, 300 x 3000 x 300 K-first
        cake_cntx_t fixed = *cntx;
        fixed.L2 = 2 << 20; fixed.L3 = 105 << 20; fixed.ncores = 8;
        beta_case(1024, 1024, 1024, 8, &fixed);
        beta_case(200, 300, 3000, 4, &fixed);
        beta_case(300, 3000, 300, 4, &fixed);
        empty_k_case(&fixed);
    }
    conv_case(cntx);
    sconv_case(cntx, 16, 24, 34, 34, 3, 3);
    sconv_case(cntx, 5, 130, 21, 37, 5, 3);
    packed_sconv_case(cntx, 16, 24, 34, 34);
    packed_sconv_case(cntx, 40, 100, 21, 37);
    dims_2d_case(cntx);
    two_cntx_case();
    gemv_case(cntx, 1024, 777);
    gemv_case(cntx, 37, 5);
    transpose_case(130, 77);
    transpose_case(1, 1000);

    blk_dims_t x;
    init_block_dims(8192, 8192, 8192, 8, &x, cntx, NA, NULL);
    report("init_block_dims fills blk_dims_t", x.m_c > 0 && x.k_c == x.m_c && x.Mb > 0 && x.M_padded >= 8192);
    update_mr_nr(cntx, 8, 12);
    report("update_mr_nr", cntx->mr == 8 && cntx->nr == 12);
    free(cntx);
    printf(failures ? "%d FAILED\n" : "ALL PASS\n", failures);
    return failures ? 1 : 0;
}
