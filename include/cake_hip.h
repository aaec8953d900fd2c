/*
 * cake_hip.h -- C-ABI of the MI355X (gfx950) implementation of CAKE's fp32
 * GEMM hot path: cake_sgemm, cake_sgemv and the im2col -> GEMM convolution.
 *
 * Plain C: pointers, ints, sizes and status codes only.  This is the surface a
 * foreign-function binding (ctypes, cgo, JNI, N-API) or the C++ drop-in
 * library (include/cake.h) binds to.  Each entry point names the interface of
 * vnatesh/CAKE_on_CPU it replaces.
 *
 * Pointers.  Every matrix/vector argument may be a device pointer (memory from
 * cake_hip_malloc, hipMalloc or a torch ROCm tensor) or a plain host pointer.
 * Host operands are staged through device buffers owned by the library and
 * results copied back before the call returns.  `seconds`, when not NULL,
 * receives the device time of the kernels alone (HIP events on the stream the
 * kernels ran on); staging copies are not part of it.
 *
 * Streams.  `stream` is a hipStream_t passed as void*; NULL is the default
 * stream.  With device operands and seconds == NULL a call only enqueues work.
 *
 * Every function returns CAKE_HIP_OK (0) or an error code; no function calls
 * exit().  cake_hip_last_error() gives the text of the last failure on the
 * calling thread.
 */
#ifndef CAKE_HIP_H
#define CAKE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* enum sched of the reference (include/common.h:105), same values. */
enum { CAKE_HIP_KMN = 0, CAKE_HIP_MKN = 1, CAKE_HIP_NKM = 2, CAKE_HIP_NA = 3 };

enum {
    CAKE_HIP_OK = 0,
    CAKE_HIP_ERR_ARG = 1,       /* NULL pointer, negative size, unknown schedule */
    CAKE_HIP_ERR_NO_DEVICE = 2, /* no usable gfx950 device                       */
    CAKE_HIP_ERR_HIP = 3,       /* a HIP runtime call failed                     */
    CAKE_HIP_ERR_ALLOC = 4,     /* device or host allocation failed              */
    CAKE_HIP_ERR_RANGE = 5,     /* an operand does not fit 32-bit element indexing */
    CAKE_HIP_ERR_ARCH = 6       /* device is not gfx950                          */
};

/* blk_dims_t of the reference (include/common.h:108-135): same fields, same order. */
typedef struct cake_hip_blk_dims_t {
    int m_c, k_c, n_c;
    int m_c1, k_c1, n_c1;
    int m_c1_last_core, n_c1_last_core, k_c1_last_core;
    int mr_rem, nr_rem, k_rem;
    int p_l, pm_l, pn_l, pm, pn;
    int m_pad, k_pad, n_pad;
    int Mb, Kb, Nb;
    int M_padded, N_padded;
    int sch;
} cake_hip_blk_dims_t;

/* The CPU-cache description the reference's block sizing reads from
 * cake_cntx_t (include/common.h:138-151). */
typedef struct cake_hip_cpu_cntx_t {
    double alpha_n; /* written back by cake_hip_init_block_dims */
    int mr, nr;
    int L1, L2, L3;
    int ncores;
} cake_hip_cpu_cntx_t;

/* Kernel families of cake_hip_plan_t.kernel.  Dense row-major operands without a tile override:
 * a product with a single row or column runs on the matrix-vector kernels, one with at most 32
 * rows of A (K >= 256) or columns of B (K >= 64) and at least 512 of the other on the streaming kernels
 * where those are ahead of the 32 x 128 and 128 x 32 macro-tiles: 17 to 32 rows or columns from 100
 * million elements of the other operand on (rows also against fewer than 1024 columns), up to 16 rows
 * always, up to 16 columns outside 8 to 60 million elements with rows of 2048 to 8192 floats;
 * as does one with 33 to 48 rows of A against a B of 48 million elements or more, 49 to 64
 * rows against 100 million, 65 to 80 against 30 million, 97 to 112 against 64 million,
 * one with K <= 64 and at least one tile of 64 x 64 per CU on workgroups that walk over tiles
 * (tile, grid and LDS fields then describe that launch; K up to 32 and, when it is a multiple of 4,
 * K from 65 to 160 in stages of 32 k loaded straight into LDS -- the latter only for a product
 * that overwrites C, the plan of one that adds to C or carries a bias is the macro-tile's),
 * everything else on the macro-tile kernel the other fields describe. */
enum {
    CAKE_HIP_KERNEL_TILE = 0,
    CAKE_HIP_KERNEL_GEMV = 1,
    CAKE_HIP_KERNEL_STREAM_ROWS = 2, /* few rows of A: B streamed once    */
    CAKE_HIP_KERNEL_STREAM_COLS = 3, /* few columns of B: A streamed once */
    CAKE_HIP_KERNEL_SHORT_K = 4,     /* short K (up to 160), many tiles: 64 x 64 tiles, next tile's operands in flight */
    CAKE_HIP_KERNEL_RESIDENT = 5     /* K below 1024 on 256 x 128 tiles, two or more per CU: one workgroup per CU walks over them */
};

/* What the GPU planner decided for one GEMM: the successor of
 * get_cache_dims / derive_schedule (src/block_sizing.cpp:304-462). */
typedef struct cake_hip_plan_t {
    int sched;        /* resolved reuse order: KMN, MKN or NKM                   */
    int tile_m, tile_n, tile_k; /* macro-tile held by one workgroup               */
    int wave_m, wave_n;         /* sub-tile held by one 64-lane wavefront         */
    int threads;      /* workgroup size                                           */
    int split_k;      /* K slices reduced in a second, fixed-order pass (1 = none) */
    int tail_tiles;   /* tiles of the thin last round that are cut along K instead (0 = none) */
    int tail_split;   /* K slices per tail tile                                   */
    int tiles_m, tiles_n;
    int group;        /* CB-block edge in tiles: tiles that run together share panels */
    int grid;         /* workgroups launched                                      */
    int lds_bytes;    /* LDS per workgroup (double buffered)                      */
    int vector_loads; /* 1: 16-byte global loads usable (K below 2M and N below 8M floats) */
    int cus;          /* compute units the plan was made for                      */
    int kernel;       /* CAKE_HIP_KERNEL_*: which kernel family cake_hip_sgemm runs for this shape */
    double flops;     /* 2*M*N*K                                                  */
    double min_bytes; /* compulsory traffic 4*(MK+KN+MN)                          */
    double model_bytes; /* modelled HBM traffic of the chosen order and CB block  */
} cake_hip_plan_t;

typedef struct cake_hip_device_t {
    int device;
    int cus;
    int xcds;
    int lds_bytes_per_cu;
    int l2_bytes;
    int wavefront;
    int clock_khz;
    size_t hbm_bytes;
    char arch[32];
} cake_hip_device_t;

/* ---- lifetime ---------------------------------------------------------- */
/* Selects `device`, checks that it is gfx950 and creates the library context.
 * Compute entry points call it with device 0 on first use. */
int cake_hip_init(int device);
int cake_hip_shutdown(void);
int cake_hip_device_info(cake_hip_device_t* out);
const char* cake_hip_strerror(int status);
const char* cake_hip_last_error(void);

/* ---- contexts ------------------------------------------------------------ */
/* A context owns what a compute call needs besides its operands: the workspaces (split-K and
 * streaming slices, the convolution's column matrix or staged input, staging copies of host
 * operands, pinned transfer buffers), its timing events and a stream of its own.  The library has
 * one default context, which cake_hip_init sets up and every entry point uses unless the calling
 * thread has made another one current.  Calls on one context take turns (they share its
 * workspaces); calls on different contexts hold different locks and, given different streams and
 * device operands, run side by side on the device.  This is the device-side state the reference
 * keeps per cake_cntx_t in its blis_cntx field (include/common.h:138-151); the C++ layer hangs a
 * context off that field.
 *
 * cake_hip_ctx_create needs an initialised library (it calls cake_hip_init(0) when none is) and
 * makes a context for the device of the default one, with a non-blocking stream of its own.
 * cake_hip_ctx_set_current(ctx) makes it the calling thread's context (NULL: back to the default);
 * from then on a NULL `stream` argument means the context's own stream (cake_hip_ctx_stream), where
 * on the default context it means the HIP null stream.  cake_hip_ctx_destroy waits for the device
 * and frees the context's device memory, events and stream; a thread that still has it current
 * gets CAKE_HIP_ERR_ARG from its next call.  cake_hip_sgemm_noalloc on any context uses the
 * device's one scratch array. */
typedef void* cake_hip_ctx_t;
int cake_hip_ctx_create(cake_hip_ctx_t* out);
int cake_hip_ctx_destroy(cake_hip_ctx_t ctx);
int cake_hip_ctx_set_current(cake_hip_ctx_t ctx);
cake_hip_ctx_t cake_hip_ctx_get_current(void);
void* cake_hip_ctx_stream(cake_hip_ctx_t ctx);

/* ---- device memory for callers without a HIP runtime of their own ------- */
int cake_hip_malloc(void** ptr, size_t bytes);
int cake_hip_free(void* ptr);
int cake_hip_memcpy_h2d(void* dst, const void* src, size_t bytes);
int cake_hip_memcpy_d2h(void* dst, const void* src, size_t bytes);
int cake_hip_memset(void* dst, int value, size_t bytes);
int cake_hip_synchronize(void);

/* ---- planner ------------------------------------------------------------ */
/* GPU tile / wave-layout / reuse-order plan.  Needs no device: when the
 * library is not initialised it plans for 256 CUs with 160 KB of LDS each.
 * tile_override = {tile_m, tile_n, tile_k, split_k} or NULL; zero entries mean
 * "choose" (the mcu,kcu,ncu arguments of cake_sgemm, include/cake.h:12-14). */
int cake_hip_plan(int M, int N, int K, int sched, const int* tile_override,
                  cake_hip_plan_t* out);

/* The reference's own CPU block sizing, init_block_dims
 * (src/block_sizing.cpp:465-595; include/tiling.h:39-41), kept because callers
 * read blk_dims_t fields and because it defines the packed layouts below. */
int cake_hip_init_block_dims(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cntx,
                             int sched, int mcu, int kcu, int ncu,
                             cake_hip_blk_dims_t* out);

/* derive_schedule (src/block_sizing.cpp:434-462): the reference's IO-optimal
 * reuse order for a CB block of side p*mc.  Returns KMN, MKN or NKM. */
int cake_hip_derive_schedule(int M, int N, int K, int p, int mc, const cake_hip_cpu_cntx_t* cntx);

/* Block sizing of the reference's 2-D grid of cores: grid_dims_2d, init_block_dims_2d and
 * init_block_dims_2d_small (include/tiling.h:43-51, src/block_sizing.cpp:596-841).  Host integer
 * arithmetic; no device is needed.  grid_dims_2d returns pn, the number of cores along N (pm = p / pn):
 * the factor of p closest to sqrt(p N / M).  The reference reads the factors of p from a table
 * generated at build time for the machine's core count (python/grid_gen.py); here divisibility is
 * tested directly and `ncores` is not used.  Fields of blk_dims_t that the reference leaves
 * unset are zero. */
int cake_hip_grid_dims_2d(int M, int N, int K, int p, int ncores);
int cake_hip_init_block_dims_2d(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cntx, int sched,
                                float type_size, int mcu, int kcu, int ncu, cake_hip_blk_dims_t* out);
int cake_hip_init_block_dims_2d_small(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cntx, int sched,
                                      float type_size, cake_hip_blk_dims_t* out);
/* Blocks of the direct convolution: get_cache_dims_conv + init_block_dims_conv
 * (examples/cake_conv.cpp:262-420): m_c output channels per core, k_c input channels, n_c rows of
 * the output image; always K-first.  cntx->alpha_n is read (cake_query_cntx sets 1.0). */
int cake_hip_init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout,
                                  int s, int p, cake_hip_cpu_cntx_t* cntx, cake_hip_blk_dims_t* out);

/* ---- GEMM ---------------------------------------------------------------- */
/* C[MxN] = A[MxK] . B[KxN], all row-major fp32: cake_sgemm
 * (src/cake_sgemm.cpp:9-175).  accumulate != 0 starts from the existing C
 * (what beta != 0 means in the reference's MKN/NKM paths, :114). */
int cake_hip_sgemm(const float* A, const float* B, float* C, int M, int N, int K,
                   int sched, int accumulate, const int* tile_override,
                   void* stream, double* seconds);

/* cake_hip_sgemm for callers that must not allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The same kernels as cake_hip_sgemm run on the planner's own choice of tile, with the same slice
 * counts, so the results are the same bits; the partial sums that split-K, tail-split and
 * streaming products and the matrix-vector kernels need, and the few columns of B that a tall
 * product turns into rows first, go into a 64 MiB array that is part of the library's device image
 * instead of buffers that grow, and the call makes no hipMalloc or hipFree.  A, B and C must be device memory; cake_hip_init must have run
 * (it looks up the array's address on its device); a product whose partial sums would not fit
 * returns CAKE_HIP_ERR_RANGE and touches nothing.  Every call on a device uses that device's one
 * array: calls that overlap on one device (different streams) race, calls on one stream do not. */
int cake_hip_sgemm_noalloc(const float* A, const float* B, float* C, int M, int N, int K,
                           int sched, int accumulate, void* stream);

/* Same product with A and/or B already in the reference's packed layouts
 * (cake_sgemm with packedA / packedB, src/cake_sgemm.cpp:42-44,64-66), as
 * written by cake_hip_pack_a / cake_hip_pack_b for the same (dims, p, cntx). */
int cake_hip_sgemm_packed(const float* A, const float* B, float* C, int M, int N, int K,
                          int p, const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx,
                          int packedA, int packedB, int accumulate,
                          void* stream, double* seconds);

/* ---- packing (reference layouts, bit-exact) ------------------------------ */
/* cake_sgemm_packed_{A,B,C}_size, src/pack_helper.cpp:5-87 (bytes). */
size_t cake_hip_packed_a_size(int M, int K, int p, const cake_hip_blk_dims_t* dims,
                              const cake_hip_cpu_cntx_t* cntx, int sched);
size_t cake_hip_packed_b_size(int K, int N, int p, const cake_hip_blk_dims_t* dims,
                              const cake_hip_cpu_cntx_t* cntx);
size_t cake_hip_packed_c_size(int M, int N, int p, const cake_hip_blk_dims_t* dims,
                              const cake_hip_cpu_cntx_t* cntx, int sched);
/* pack_A / pack_B / pack_C / unpack_C, src/pack_helper.cpp:92-184. */
int cake_hip_pack_a(const float* A, float* A_p, int M, int K, int p,
                    const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx,
                    int sched, void* stream, double* seconds);
int cake_hip_pack_b(const float* B, float* B_p, int K, int N, int p,
                    const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx,
                    int sched, void* stream, double* seconds);
int cake_hip_pack_c(const float* C, float* C_p, int M, int N, int p,
                    const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx,
                    int sched, void* stream, double* seconds);
int cake_hip_unpack_c(float* C, const float* C_p, int M, int N, int p,
                      const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx,
                      int sched, void* stream, double* seconds);
/* Packed offset of element (row, col) of A (which=0), B (1) or C (2): the
 * index map the pack kernels implement, evaluated on the host. */
int64_t cake_hip_packed_offset(int which, int row, int col, int M, int N, int K, int p,
                               const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx,
                               int sched);

/* ---- GEMV ---------------------------------------------------------------- */
/* y[M] = A . x (accumulate == 0) or y += A . x (accumulate != 0).
 * a_col_major != 0: A[k*M + m], the layout cake_sgemv reads
 * (examples/cake_gemv.cpp:89-140,716-767; it always accumulates);
 * a_col_major == 0: A[m*K + k]. */
int cake_hip_sgemv(const float* A, const float* x, float* y, int M, int K,
                   int a_col_major, int accumulate, void* stream, double* seconds);

/* ---- convolution through im2col ------------------------------------------ */
/* NCHW input -> cols[Cin*Hf*Wf][batch*Hout*Wout], row k = c*Hf*Wf + h*Wf + w,
 * column n = b*Hout*Wout + ho*Wout + wo, zero where the window hangs over the
 * edge: im_2_col (examples/cake_conv.cpp:1178-1213) generalised to a batch,
 * padding and stride.  Hout = (Hin + 2*pad - Hf)/stride + 1, same for W. */
int cake_hip_im2col(const float* in, float* cols, int batch, int Cin, int Hin, int Win,
                    int Hf, int Wf, int stride, int pad, void* stream, double* seconds);

/* out = conv(in, weights) computed as weights[Cout x Cin*Hf*Wf] . cols: the
 * im2col path of examples/cake_conv.cpp:1007-1066.  weights are OIHW.
 * out_nchw == 0: out is [Cout][batch*Hout*Wout] (the GEMM's own layout, which
 * is what the reference produces for its single image); != 0: NCHW.
 *
 * cake_hip_conv2d gathers the column matrix inside the GEMM's B loader, so the
 * K x N intermediate is never written.  With padding or a stride above 1 the
 * input is first copied once into a staged image (zero padding written out,
 * rows split into their column phases, so that 4 neighbouring output pixels
 * read 4 neighbouring floats); an output width that is not a multiple of 4 is
 * computed with rows padded to one and the extra columns dropped.  It runs the
 * two-step path instead when that padding would cost more than the column
 * matrix (narrow maps with many output channels).  A 1 x 1 filter at stride 1
 * without padding needs neither: a plane is then one row of Hin * Win pixels,
 * gathered from the input as it lies, and with at most 64 input channels and
 * enough tiles the images run as one batch of plain products on the short-K
 * kernel.  A 1 x 1 filter at a stride above 1 without padding has the pixels
 * it reads copied out densely first and then runs as such a layer on the copy.
 * Stride-1 layers with whole blocks of 32 input channels, a filter of
 * 7 taps or more, up to 4 columns of padding and maps up to about 60 pixels
 * wide have a kernel that reads the input where it lies (no staged copy:
 * patches of the input per workgroup in LDS, zero padding in place; under a
 * 3 x 3 filter the filters are read where they lie as well and the call is
 * that one kernel); it has a single 256 x 128 tile and is taken where that
 * pays -- 18 K steps or more, 95 % of the tile rows in use, and rounds of tiles
 * that fill the device (a thin last round cut into sub-tiles or K slices
 * counted for what it costs).  The environment variable CAKE_HIP_CONV_ROUTE (read
 * at every call) overrides that choice: "patch" takes this kernel wherever
 * its geometry allows, "staged" never.
 * A batch whose staged input
 * would reach 2 GiB, or whose product 2^31 elements, is run in chunks of whole
 * images through the same staged buffer, so input and output may be as large
 * as memory holds; only a single image of 2 GiB takes the two-step path, whose
 * column matrix is limited to 2^31 elements (CAKE_HIP_ERR_RANGE beyond).
 * cake_hip_conv2d_im2col always runs the two steps the reference runs: im2col
 * into a column matrix, then the GEMM.  Both give the same result.
 * workspace (device, cake_hip_conv2d_workspace bytes: the column matrix of the
 * two-step path or the staged image of the gather path) may be NULL: the
 * library then uses a buffer of its own. */
size_t cake_hip_conv2d_workspace(int batch, int Cin, int Hin, int Win, int Cout,
                                 int Hf, int Wf, int stride, int pad);
int cake_hip_conv2d(const float* in, const float* weights, float* out,
                    int batch, int Cin, int Hin, int Win, int Cout, int Hf, int Wf,
                    int stride, int pad, int out_nchw, void* workspace,
                    void* stream, double* seconds);
int cake_hip_conv2d_im2col(const float* in, const float* weights, float* out,
                           int batch, int Cin, int Hin, int Win, int Cout, int Hf, int Wf,
                           int stride, int pad, int out_nchw, void* workspace,
                           void* stream, double* seconds);

/* Which of the routes above the calling thread's last convolution call took (cake_hip_conv2d,
 * cake_hip_conv2d_im2col, cake_hip_sconv); CAKE_HIP_CONV_NONE when it failed its argument checks. */
enum {
    CAKE_HIP_CONV_NONE = 0,
    CAKE_HIP_CONV_SHORTK_BATCH = 1, /* 1 x 1 layer as a batch of plain products on the short-K kernel */
    CAKE_HIP_CONV_PATCH = 2,        /* input read where it lies, patches of 16 channels in LDS        */
    CAKE_HIP_CONV_GATHER = 3,       /* columns gathered inside the product (staged copy where needed) */
    CAKE_HIP_CONV_TWO_STEP = 4      /* column matrix written out, then the product                    */
};
int cake_hip_last_conv_route(void);

/* out[Cout][Hout][Wout] += filters[Cout][Cin][Hf][Wf] * in[Cin][Hin][Win]: the direct convolution
 * of one CHW image without padding, cake_sconv (examples/cake_conv.cpp:5-8,765-848), whose
 * micro-kernel starts from the values out already holds (:36-47).  Runs as cake_hip_conv2d does
 * (columns gathered inside the product, no column matrix).  Hout and Wout must be
 * (Hin - Hf) / stride + 1 and (Win - Wf) / stride + 1. */
int cake_hip_sconv(const float* filters, const float* in, float* out, int Wf, int Hf, int Win, int Hin,
                   int Wout, int Hout, int Cin, int Cout, int stride, void* stream, double* seconds);

/* Filters [Cout][Cin][taps] (taps = Hf * Wf) into the layout of the reference's pack_filters
 * (examples/cake_conv.cpp:430-454,536-610; it is written for 3 x 3 filters, taps = 9): K-first
 * blocks over output channels and input channels, and inside an m_r panel
 * [tap][channel][m_r]; rows past Cout are zero.  dims from cake_hip_init_block_dims_conv for the
 * same Cout, Cin, p and cntx.  The size in bytes is M_padded * Cin * taps * 4. */
size_t cake_hip_packed_filters_size(int Cout, int Cin, int taps, int p, const cake_hip_blk_dims_t* dims,
                                    const cake_hip_cpu_cntx_t* cntx);
int cake_hip_pack_filters(const float* filters, float* filters_p, int Cout, int Cin, int taps, int p,
                          const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx, void* stream,
                          double* seconds);
/* cake_hip_sconv with the filters in that layout: cake_sconv with packedA = 1
 * (examples/cake_conv.cpp:797-799).  The filters are copied back to [Cout][Cin][Hf][Wf] in a
 * library workspace first (one small kernel). */
int cake_hip_sconv_packed(const float* filters_p, const float* in, float* out, int Wf, int Hf, int Win, int Hin,
                          int Wout, int Hout, int Cin, int Cout, int stride, int p,
                          const cake_hip_blk_dims_t* dims, const cake_hip_cpu_cntx_t* cntx, void* stream,
                          double* seconds);

/* ---- transpose and the linear layer ---------------------------------------- */
/* dst[c][r] = src[r][c] for a rows x cols row-major matrix; dst is cols x rows.
 * Replaces transpose_mat (include/util.h:32, src/transpose.cpp:5-29; its blocking
 * arguments Kt, Nt have no meaning here).  src and dst must not overlap. */
int cake_hip_transpose(const float* src, float* dst, int rows, int cols, void* stream,
                       double* seconds);

/* y[M][N] = x[M][K] . w[N][K]^T (+ bias[N] on every row when bias != NULL).
 * Replaces linear_forward (src/linear.cpp:12-50), which transposes the weights
 * into a K x N matrix, calls cake_sgemm and adds the bias afterwards.  Here w is
 * read as it lies: a single sample is a matrix-vector product, up to 32 samples
 * stream w once, larger batches run on the macro-tile kernel with 16-byte loads
 * along k for both operands.  (Only rows of 2^21 floats and more still go
 * through a transposed copy in a library workspace.)  The bias is added to the
 * finished fp32 product in every case (same rounding: fl(fl(sum) + bias)). */
int cake_hip_linear_forward(const float* x, const float* w, const float* bias, float* y, int M,
                            int N, int K, void* stream, double* seconds);

/* C[M][N] = (accumulate ? C : 0) + A[M][K] . Bt[N][K]^T: the product above without the bias, for
 * any caller whose second operand lies transposed (rows of length K).  It has no counterpart in
 * the reference's API, which can only transpose such an operand first (transpose_mat,
 * src/linear.cpp:26-36); here Bt is read as it lies by the same kernels as the linear layer.
 * tile_override as for cake_hip_sgemm (it forces the macro-tile kernel). */
int cake_hip_sgemm_nt(const float* A, const float* Bt, float* C, int M, int N, int K, int accumulate,
                      const int* tile_override, void* stream, double* seconds);

/* The same with the weights already transposed: wt is [K][N] (input x output
 * features), y = x . wt (+ bias).  This is the product of linear_forward alone
 * (the cake_sgemm call of src/linear.cpp:38 with its bias loop), for callers
 * whose weights stay the same over many calls and who keep the transposed copy
 * (cake_hip_transpose).  cake_hip_linear_forward needs no such copy. */
int cake_hip_linear_forward_wt(const float* x, const float* wt, const float* bias, float* y, int M,
                               int N, int K, void* stream, double* seconds);

/* Gradients of the layer above for grad_y[M][N] (src/linear.cpp:53-102):
 *   grad_x[M][K] = grad_y . w,   grad_w[N][K] = grad_y^T . x,
 *   grad_bias[N] = column sums of grad_y (summed in a fixed order).
 * Any of the three outputs may be NULL and is then skipped (x may be NULL when
 * grad_w is, w when grad_x is). */
int cake_hip_linear_backward(const float* grad_y, const float* x, const float* w, float* grad_x,
                             float* grad_w, float* grad_bias, int M, int N, int K, void* stream,
                             double* seconds);

/* ---- autotuner --------------------------------------------------------------- */
/* Times macro-tile x split-K x tail-split candidates for an M x N x K product on
 * the device (synthetic operands in library memory, default stream) for at most
 * about budget_seconds (<= 0: 2 s), and records the fastest in a process-wide
 * table keyed by (M, N, K).  From then on cake_hip_plan / cake_hip_sgemm and the
 * other products use that choice whenever the caller gives no tile override.
 * The planner's own choice is always measured first, so the result is never
 * slower than the default by more than timing noise.  A product with few rows of A
 * or columns of B (CAKE_HIP_KERNEL_STREAM_*) or a short K under many tiles
 * (CAKE_HIP_KERNEL_SHORT_K) runs on a kernel of its own instead of a macro-tile:
 * that kernel is then the default that is measured, and the table only gets an
 * entry (which from then on replaces that kernel) when a tile beats it.
 * best_plan, best_seconds, default_seconds may be NULL.
 * Successor of the reference's user-tile hook and stubbed simulated-annealing
 * tuner (mcu,kcu,ncu of cake_sgemm, src/block_sizing.cpp:363-368;
 * src/autotune_sa.cpp:36-81). */
int cake_hip_autotune(int M, int N, int K, double budget_seconds, cake_hip_plan_t* best_plan,
                      double* best_seconds, double* default_seconds);
/* The table as a text file, one line per product:
 *   M N K vec tile_m tile_n tile_k split_k tail_ok seconds
 * Loading merges into the table (entries for tiles this build lacks are skipped)
 * and needs no device.  cake_hip_init also loads the file named by the
 * environment variable CAKE_HIP_TUNE_FILE when it is set and readable. */
int cake_hip_tune_save(const char* path);
int cake_hip_tune_load(const char* path, int* entries);
int cake_hip_tune_clear(void);
int cake_hip_tune_count(void);

/* ---- seeded inputs -------------------------------------------------------- */
/* dst[i] = uniform[-1,1) value i of the counter-based splitmix64 stream `seed`
 * (24 random bits, exact in fp32).  Stands in for rand_init (src/util.cpp:259-267),
 * which is time-seeded and not reproducible. */
int cake_hip_fill_uniform(float* dst, size_t n, uint64_t seed, void* stream);

/* Average duration in seconds of the kernels of the last compute call on this
 * thread, per kernel family: [0] GEMM macro-tile, [1] split-K reduce,
 * [2] GEMV, [3] im2col, [4] pack/unpack/transpose.  Zero where none ran. */
int cake_hip_last_kernel_seconds(double out[5]);

#ifdef __cplusplus
}
#endif
#endif /* CAKE_HIP_H */
