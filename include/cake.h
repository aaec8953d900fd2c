// cake.h -- C++ interface of the fp32 GEMM path of CAKE, served by an MI355X.
//
// Source-compatible with the part of vnatesh/CAKE_on_CPU's include/cake.h,
// include/common.h, include/tiling.h, include/packing.h and include/util.h that
// the cake_sgemm / cake_sgemv / im2col-convolution path uses: same type names,
// field order, function names, argument order and default arguments, so a
// caller written against the reference recompiles against this header and
// links libcake.so unchanged.  Underneath, every function forwards to the C-ABI
// of libcake_hip.so (include/cake_hip.h); the product, the packing and im2col
// all run on the GPU.  Only the test helpers at the end are host code, as an
// independent checker has to be.
//
// Matrices are row-major float.  Pointers may be ordinary host memory (as in
// the reference) or device memory.
#pragma once

#include <stdbool.h>
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

// ---- types (reference: include/common.h:105-159) ---------------------------

enum sched { KMN, MKN, NKM, NA };

typedef struct blk_dims_t {
    int m_c, k_c, n_c;
    int m_c1, k_c1, n_c1;
    int m_c1_last_core, n_c1_last_core, k_c1_last_core;
    int mr_rem, nr_rem, k_rem;
    int p_l, pm_l, pn_l, pm, pn;
    int m_pad, k_pad, n_pad;
    int Mb, Kb, Nb;
    int M_padded, N_padded;
    enum sched sch;
} blk_dims_t;

typedef struct cake_cntx_t {
    void* blis_cntx;      // names the device context this cntx works on (set on first use; zero it in a cntx you build yourself)
    double alpha_n;
    double peak_dram_bw;  // bytes/s of the device the library runs on
    double peak_flops;    // fp32 matrix FLOP/s of that device
    int mr, nr;           // register-tile shape that defines the packed layouts
    int m_map, n_map;
    int L1, L2, L3;       // host cache sizes: inputs of the CB-block sizing
    int ncores;           // host physical cores
} cake_cntx_t;

typedef struct cache_dims_t {
    int m_c, k_c, n_c;
    enum sched sch;
} cache_dims_t;

#define cake_max(x, y) (((x) >= (y)) ? (x) : (y))
#define cake_min(x, y) (((x) <= (y)) ? (x) : (y))

// ---- machine description and block sizing (reference: include/tiling.h) -----

cake_cntx_t* cake_query_cntx();                                    // block_sizing.cpp:40
cake_cntx_t* cake_query_cntx_torch(int L2, int L3);                // block_sizing.cpp:10
void update_mr_nr(cake_cntx_t* cake_cntx, int m_r, int n_r);        // block_sizing.cpp:78
int get_cache_size(int level);                                     // block_sizing.cpp:148
int get_num_physical_cores();                                      // block_sizing.cpp:91

enum sched derive_schedule(int M, int N, int K, int p, int mc_ret, cake_cntx_t* cake_cntx);

cache_dims_t* get_cache_dims(int M, int N, int K, int p, cake_cntx_t* cake_cntx, enum sched sch,
                             char* argv[], float type_size = 4, int mcu = 0, int kcu = 0, int ncu = 0);

void init_block_dims(int M, int N, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx,
                     enum sched sch, char* argv[], float type_size = 4,
                     int mcu = 0, int kcu = 0, int ncu = 0);

// Block sizing of the reference's 2-D grid of cores (include/tiling.h:43-51,
// src/block_sizing.cpp:596-841): host arithmetic, as in the reference.  grid_dims_2d returns pn,
// the factor of p closest to sqrt(p N / M); the reference's generated factor table is replaced by
// a divisibility test, so `ncores` is not read.
int grid_dims_2d(int M, int N, int K, int p, int ncores);
void init_block_dims_2d(int M, int N, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx,
                        enum sched sch, char* argv[], float type_size = 4,
                        int mcu = 0, int kcu = 0, int ncu = 0);
void init_block_dims_2d_small(int M, int N, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx,
                              enum sched sch, char* argv[], float type_size = 4);

// ---- GEMM (reference: include/cake.h:12-14,36-47) ---------------------------

double cake_sgemm(float* A, float* B, float* C, int M, int N, int K, int p,
                  cake_cntx_t* cake_cntx, char* argv[] = NULL, bool packedA = 0, bool packedB = 0,
                  float alpha = 1, float beta = 0, enum sched sch = NA,
                  int mcu = 0, int kcu = 0, int ncu = 0);

// The pack-on-the-fly and 2-D core-grid entry points of the reference.  On the
// GPU operands are always staged on the fly and the grid is the device's, so
// these run the same kernel as cake_sgemm.
double cake_sgemm_online(float* A, float* B, float* C, int M, int N, int K, int p,
                         cake_cntx_t* cake_cntx, char* argv[] = NULL, bool packedA = 0,
                         bool packedB = 0, float alpha = 1, float beta = 0, enum sched sch = NA,
                         int mcu = 0, int kcu = 0, int ncu = 0);
double cake_sgemm_2d(float* A, float* B, float* C, int M, int N, int K, int p,
                     cake_cntx_t* cake_cntx, char* argv[] = NULL, bool packedA = 0,
                     bool packedB = 0, float alpha = 1, float beta = 0, enum sched sch = NA,
                     int mcu = 0, int kcu = 0, int ncu = 0);
double cake_sgemm_2d_small(float* A, float* B, float* C, int M, int N, int K, int p,
                           cake_cntx_t* cake_cntx, char* argv[] = NULL, bool packedA = 0,
                           bool packedB = 0, float alpha = 1, float beta = 0, enum sched sch = NA);

// The reference's timing variant (include/cake.h:39-41, src/cake_sgemm.cpp:472-600): cake_sgemm
// with the schedule forced to K-first, packedA / packedB honoured, returning the time of the
// product alone.
double cake_sgemm_test(float* A, float* B, float* C, int M, int N, int K, int p,
                       cake_cntx_t* cake_cntx, char* argv[] = NULL, bool packedA = 0,
                       bool packedB = 0, float alpha = 1, float beta = 0, enum sched sch = NA);

// ---- packing (reference: include/packing.h:6-13,70-72) ----------------------

size_t cake_sgemm_packed_A_size(int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch);
size_t cake_sgemm_packed_B_size(int K, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx);
size_t cake_sgemm_packed_C_size(int M, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch);

double pack_A(float* A, float* A_p, int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch);
void pack_B(float* B, float* B_p, int K, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch);
void pack_C(float* C, float* C_p, int M, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch);
void unpack_C(float* C, float* C_p, int M, int N, int p, blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch);

// ---- GEMV (reference: examples/cake_gemv.cpp:7-9) ---------------------------
// y += A.x with A column-major, A[k*M + m].

double cake_sgemv(float* A, float* B, float* C, int M, int K, int p, cake_cntx_t* cake_cntx,
                  char* argv[] = NULL, bool packedA = 0, float alpha = 1, float beta = 0,
                  enum sched sch = NA);

// ---- convolution through im2col (reference: examples/cake_conv.cpp:24-25) ---
// Returns a malloc'd [Cin*Hf*Wf][Hout*Wout] matrix; the caller frees it.

float* im_2_col(float* In, int Wf, int Hf, int Win, int Hin, int Wout, int Hout,
                int Cin, int Cout, int s);

// Direct convolution of one CHW image (reference: examples/cake_conv.cpp:5-8,765-848):
// C[Cout][Hout][Wout] += A[Cout][Cin][Hf][Wf] * B[Cin][Hin][Win], no padding,
// Hout = (Hin - Hf) / s + 1 and Wout = (Win - Wf) / s + 1.  On the GPU the windows are gathered
// inside the product, so there is no column matrix either.  With packedA the filters are in the
// layout of pack_filters for the blocks of init_block_dims_conv (same Cout, Cin, p and cntx), as in
// the reference (:791-799); they are brought back to [Cout][Cin][Hf][Wf] on the device first.
double cake_sconv(float* A, float* B, float* C, int Wf, int Hf, int Win, int Hin, int Wout, int Hout,
                  int Cin, int Cout, int s, int p, cake_cntx_t* cake_cntx, char* argv[] = NULL,
                  bool packedA = 0, enum sched sch = NA);
// examples/cake_conv.cpp:10-18,262-420: blocks of that convolution (K-first only), and
// examples/cake_conv.cpp:536-610: 3 x 3 filters, A[M = Cout][K = Cin * 9], into those blocks;
// A_p holds x->M_padded * K floats.  Returns seconds.
cache_dims_t* get_cache_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout,
                                  int s, int p, cake_cntx_t* cake_cntx, enum sched sch, char* argv[],
                                  float density = 0, float type_size = 4);
void init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s, int p,
                          blk_dims_t* x, cake_cntx_t* cake_cntx, enum sched sch, char* argv[],
                          float density = 0, float type_size = 4);
double pack_filters(float* A, float* A_p, int M, int K, int p, blk_dims_t* x, cake_cntx_t* cake_cntx);
void conv_gemm_checker(float* conv, float* gemm, int M, int N);    // cake_conv.cpp:1216

// ---- test helpers (reference: include/util.h) -------------------------------

void rand_init(float* mat, int r, int c);                          // util.cpp:259
bool cake_sgemm_checker(float* A, float* B, float* C, int N, int M, int K);  // util.cpp:173
bool mat_equals(float* C, float* C_check, int M, int N);           // util.cpp:139
bool add_checker(float** C_arr, float* C, int M, int N, int p);     // util.cpp:205
void print_schedule(enum sched sch);
void print_mat(float* arr, int r, int c);
void print_array(float* arr, int len);
float rand_gen();                                                  // util.cpp:251, uniform (0,1]
float normalRandom();                                              // util.cpp:270, N(0,1) by Box-Muller
// At[n][k] = A_old[k][n] for a K x N matrix, on the GPU; Kt, Nt (host blocking) are unused.
void transpose_mat(float* A_old, float* At, int K, int N, int Kt, int Nt);  // transpose.cpp:5
// The reference's self-test (util.cpp:3-136): every M, K, N in {1,10,96,111,960,2111}
// through cake_sgemm_2d, cake_sgemm MKN, cake_sgemm_online, cake_sgemm KMN and
// cake_sgemm NKM, each checked against a host loop.  p has no effect on the
// device, so the sweep runs p = 2 and p = ncores (the two ends of the reference's
// range) instead of every value between.  Prints "ALL TESTS PASSED!" or "FAILED";
// returns 0 like the reference.
int run_tests();
