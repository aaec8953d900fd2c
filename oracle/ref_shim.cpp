// ref_shim.cpp -- C-linkage doorways into the parts of vnatesh/CAKE_on_CPU that
// compile straight from their own sources (no generated kernels.h / grid table).
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/build_ref.sh into oracle/_ref/ when
// /root/reference is present; used by tests to check the C restatement in
// cake_oracle.c bit for bit.  Nothing here is reference code: each function
// forwards to a symbol defined in a reference .cpp that the script compiles
// where it lies.
#include "cake.h"

// defined in src/kernels/haswell/dense.cpp
void cake_sgemm_haswell_6x16(float* A, float* B, float* C, int m, int n, int k);
// defined in examples/cake_gemv.cpp
void cake_sgemv_haswell_8x8_col(float* A, float* B, float* C, int m, int k, int M);
void schedule_mvm(float* A_p, float* B_p, float* C_p, int M, int K, int p,
                  cake_cntx_t* cake_cntx, blk_dims_t* x);
// defined in examples/cake_conv.cpp
float* im_2_col(float* In, int Wf, int Hf, int Win, int Hin, int Wout, int Hout,
                int Cin, int Cout, int s);

void init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s, int p,
                          blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch, char* argv[], float density,
                          float type_size);
double pack_filters(float* A, float* A_p, int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx);

#define EXPORT extern "C" __attribute__((visibility("default")))

namespace {
// 26 ints in blk_dims_t field order -> the reference's struct
blk_dims_t dims_from(const int* v)
{
    blk_dims_t x;
    int* f = reinterpret_cast<int*>(&x);
    for (int i = 0; i < 25; ++i) f[i] = v[i];
    x.sch = static_cast<enum sched>(v[25]);
    return x;
}

cake_cntx_t cntx_from(int mr, int nr)
{
    cake_cntx_t c;
    memset(&c, 0, sizeof c);
    c.mr = mr;
    c.nr = nr;
    c.alpha_n = 1.0;
    return c;
}
}  // namespace

EXPORT int ref_sizeof_blk_dims() { return (int)sizeof(blk_dims_t); }

EXPORT size_t ref_packed_A_size(int M, int K, int p, const int* dims, int mr, int nr, int sch)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    return cake_sgemm_packed_A_size(M, K, p, &x, &c, (enum sched)sch);
}

EXPORT size_t ref_packed_B_size(int K, int N, int p, const int* dims, int mr, int nr)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    return cake_sgemm_packed_B_size(K, N, p, &x, &c);
}

EXPORT size_t ref_packed_C_size(int M, int N, int p, const int* dims, int mr, int nr, int sch)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    return cake_sgemm_packed_C_size(M, N, p, &x, &c, (enum sched)sch);
}

EXPORT void ref_pack_A(float* A, float* A_p, int M, int K, int p, const int* dims, int mr, int nr, int sch)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    omp_set_num_threads(p);
    pack_A(A, A_p, M, K, p, &x, &c, (enum sched)sch);
}

EXPORT void ref_pack_B(float* B, float* B_p, int K, int N, int p, const int* dims, int mr, int nr, int sch)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    omp_set_num_threads(p);
    pack_B(B, B_p, K, N, p, &x, &c, (enum sched)sch);
}

EXPORT void ref_pack_C(float* Cm, float* C_p, int M, int N, int p, const int* dims, int mr, int nr, int sch)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    omp_set_num_threads(p);
    pack_C(Cm, C_p, M, N, p, &x, &c, (enum sched)sch);
}

EXPORT void ref_unpack_C(float* Cm, float* C_p, int M, int N, int p, const int* dims, int mr, int nr, int sch)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    omp_set_num_threads(p);
    unpack_C(Cm, C_p, M, N, p, &x, &c, (enum sched)sch);
}

EXPORT void ref_ukernel_6x16(float* A, float* B, float* Ct, int k)
{
    cake_sgemm_haswell_6x16(A, B, Ct, 6, 16, k);
}

EXPORT void ref_schedule_mvm(float* A, float* xv, float* y, int M, int K, int p, const int* dims, int mr)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, 16);
    omp_set_num_threads(p);
    schedule_mvm(A, xv, y, M, K, p, &c, &x);
}

EXPORT void ref_im_2_col(float* In, float* out, int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin)
{
    float* m = im_2_col(In, Wf, Hf, Win, Hin, Wout, Hout, Cin, 1, 1);
    memcpy(out, m, sizeof(float) * (size_t)Cin * Wf * Hf * Wout * Hout);
    free(m);
}

// 26 ints in blk_dims_t field order out of the reference's struct (fields the reference leaves
// unset are zeroed first, so that the comparison is defined)
EXPORT void ref_init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout,
                                     int s, int p, int mr, int nr, int L2, double alpha_n, int* dims_out)
{
    blk_dims_t x;
    memset(&x, 0, sizeof x);
    cake_cntx_t c = cntx_from(mr, nr);
    c.L2 = L2;
    c.alpha_n = alpha_n;
    init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, &x, &c, KMN, NULL, 0, 4);
    const int* f = reinterpret_cast<const int*>(&x);
    for (int i = 0; i < 25; ++i) dims_out[i] = f[i];
    dims_out[25] = (int)x.sch;
}

// 3 x 3 filters only: the reference's pack_filters has Wf = Hf = 3 written into it
EXPORT void ref_pack_filters(float* F, float* F_p, int Cout, int K, int p, const int* dims, int mr, int nr)
{
    blk_dims_t x = dims_from(dims);
    cake_cntx_t c = cntx_from(mr, nr);
    omp_set_num_threads(p);
    pack_filters(F, F_p, Cout, K, p, &x, &c);
}
