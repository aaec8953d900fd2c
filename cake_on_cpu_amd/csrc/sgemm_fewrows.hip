// sgemm_fewrows.hip -- products in which one operand has at most 32 rows or
// columns, or A up to 112 rows against a large B ("a few vectors times a matrix":
// small-batch linear layers, blocks of matrix-vector products).
//
// Such a product is bound by reading the large operand once from HBM, not by
// arithmetic, and a 64-row macro-tile would spend most of the matrix pipe on
// zero rows while reading the large operand in short pieces.  The kernels here
// stream the large operand once, 16 bytes per lane, into the operand registers
// of v_mfma_f32_16x16x4_f32, whose 16 rows fit the problem (17 to 32 rows or
// columns run two MFMA groups per value loaded): no barrier inside the k loop,
// so every wave keeps its loads in flight on its own.  The small operand comes
// from L2 with one load per 4 to 16 loads of the large one.
//
//   sgemm_fewrows_nn_kernel   C[M<=112][N] = A[M][K] . B[K][N]      streams B (n contiguous),
//                             straight from global memory into MFMA operands
//   sgemm_fewrows_nt_kernel   C'[i<=32][n] = sum_k X[i][k] W[n][k]  streams W (k contiguous)
//                             through a wave-private LDS area that turns rows into MFMA
//                             operands: the linear layer y = x w^T for a small batch without
//                             transposing w, and C[M][N<=32] = A.B with W = A, X = B^T
//
// A workgroup owns 64 or 128 columns of B (64 rows of W) and a slice of k; its four
// waves share the slice and add their sums in LDS in wave order; K slices are summed
// by splitk_reduce_kernel in slice order, so results are run-to-run identical.
//
// Operand layout of v_mfma_f32_16x16x4_f32: lane l supplies A[l % 16][l / 16]
// and B[l / 16][l % 16]; result register r of lane l is C[4 * (l / 16) + r][l % 16].
// The order of k inside a product is free as long as both operands agree, so a
// lane that loads 4 consecutive k of its row (16 bytes) feeds them to 4
// successive MFMAs: MFMA e of a group of 16 k works on k = 4 (l / 16) + e.
#include "sgemm_tile.hpp"
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

namespace cake {

// 16-byte load marked non-temporal: the large operand is read once and should not push the small
// one or the partial sums out of the caches on its way through
__device__ __forceinline__ f32x4 stream_load_f32x4(const float* base, int byte_offset, unsigned records)
{
    __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)records, 0x00020000);
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, /*nt*/ 2));
}

__device__ __forceinline__ float load_f32(const float* base, int byte_offset, unsigned records)
{
    __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)records, 0x00020000);
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 0));
}

static constexpr int FR_K_UNIT = 256;   // K slices are multiples of this: 64 k per wave

// The part of [kbeg, kend) that wave `wave` of 4 walks: quarters rounded up to 16 k
__device__ __forceinline__ void wave_part(int kbeg, int kend, int wave, int& kw0, int& kw1)
{
    const int part = (((kend - kbeg + 3) >> 2) + 15) & ~15;
    kw0 = min(kend, kbeg + wave * part);
    kw1 = min(kend, kw0 + part);
}

// MG groups of 16 rows of A (M <= 16 MG) against NJ pieces of 64 columns per workgroup: every
// B value loaded feeds MG MFMAs, so the arithmetic per byte grows with MG.  One and two groups
// (up to 32 rows) stay bound by memory; three (up to 48 rows) need about as long for the matrix
// work as for the memory and still beat the 64-row macro-tile on large operands (48 x 16384 x
// 16384: 220 us against 289 us).  Four groups (up to 64 rows) are bound by the matrix pipe: against
// 100 million elements of B and more they are 4 to 11 % ahead of the macro-tile (64 x 16384 x
// 16384: 265-277 us against 288-298 us; 64 x 10240 x 10240: 121 against 137 us), below that behind
// it (64 x 8192 x 8192: 76 against 73 us).  The matrix pipe is busy in 84-85 % of that launch's
// cycles (counters); more loads in flight, a load behind every piece of B that the MFMAs are done
// with instead of behind the whole unit, and leaving the scheduling to the compiler did not
// raise that.
// Five and seven groups (65 to 80 and 97 to 112 rows) run on 64 columns per workgroup with four
// units in flight, which is what the registers hold.  They win where the macro-tiles would pad
// the rows to 96 or 128: 80 x 16384 x 16384 320 us against 374 us, 72 x 8192 x 8192 89 against
// 98 us, 112 x 16384 x 16384 430 against 475 us (N x K, us for 65/72/80 rows, tiles -> here:
// 8192 x 4096 54-56 -> 50-52, 4096 x 4096 31-32 -> 31-33, 2048 x 2048 16 -> 16-18; for 104/112
// rows: 12288 x 12288 278-281 -> 254-256, 8192 x 8192 124-125 -> 120-122, 8192 x 4096 63 -> 69).
// Six groups tie with the 96-row macro-tile, which pads nothing there (96 x 16384 x 16384: 374
// against 388 us, 8192 x 8192: 106 against 102 us), and are not instantiated.
template <int MG, int NJ>
__global__ void __launch_bounds__(256, 2) sgemm_fewrows_nn_kernel(const float* __restrict__ A,
                                                               const float* __restrict__ B,
                                                               float* __restrict__ out, int M, int N, int K,
                                                               int lda, int ldb, int k_per_slice,
                                                               int out_ld, size_t out_slice_stride,
                                                               int accumulate, const float* __restrict__ col_bias)
{
    constexpr int COLS = 64 * NJ;                     // columns of B per workgroup
    constexpr int STAGES = MG > 4 ? 4 : 8 / NJ;       // units in flight per wave: 16 loads of B (8 from five groups on)
    __shared__ __align__(16) float red[16 * MG * COLS];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    const int n0 = blockIdx.x * COLS;
    const int kbeg = blockIdx.y * k_per_slice;
    const int kend = min(K, kbeg + k_per_slice);
    int kw0, kw1;
    wave_part(kbeg, kend, wave, kw0, kw1);

    const unsigned a_elems = clamp_elems((long long)(M - 1) * lda + K);
    const unsigned b_elems = clamp_elems((long long)(K - 1) * ldb + N - n0);
    // A: rows 16 g + li, k = 4 lq .. 4 lq + 3 of the group.  B: rows 4 lq + e of the group (e = 0..3
    // by moving the base), and of each row NJ 16-byte pieces: piece j is columns 64 j + 4 li .. + 3,
    // so that the 16 lanes of a row read 256 contiguous bytes per load instruction.
    int a_off[MG];
#pragma unroll
    // rows at and past M repeat the last row (their results are never written): lanes that ask for
    // an out-of-range offset instead make every load of A slower (33 x 16384 x 16384: 258 us
    // against 224 us)
    for (int g = 0; g < MG; ++g) a_off[g] = (min(16 * g + li, M - 1) * lda + 4 * lq) * 4;
    int b_off[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        b_off[j] = n0 + 64 * j + 4 * li < N ? (4 * lq * ldb + 64 * j + 4 * li) * 4 : BUF_OOB;

    f32x4 acc[MG][4 * NJ];
#pragma unroll
    for (int g = 0; g < MG; ++g)
#pragma unroll
        for (int c = 0; c < 4 * NJ; ++c) acc[g][c] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Groups of 16 k that lie wholly below kw1 <= K, in units of half a group (2 NJ loads of B,
    // 8 MG NJ MFMAs).  STAGES units are in flight: each is multiplied and its registers refilled
    // with the unit STAGES further on.  A unit past the end gets a record count of 0, which turns
    // its loads into zeros without a memory access, so the loop body needs no branch and the
    // wait counts in front of the MFMAs are exact.  Every row asked for below the end exists, so
    // those record counts are exact too (records_left must not be asked about a start past the
    // end of an operand: its difference would wrap to "everything in range").
    const int units = 2 * ((kw1 - kw0) >> 4);
    auto load_a = [&](int q, f32x4 (&a)[MG]) {
        const int kq = kw0 + 16 * (q >> 1);
        const unsigned rec = q < units ? records_left(a_elems, (unsigned)kq) : 0u;
#pragma unroll
        for (int g = 0; g < MG; ++g) a[g] = buffer_load_f32x4(A + kq, a_off[g], rec);
    };
    auto load_unit = [&](int q, int h, f32x4 (&b)[2][NJ]) {
        const int kq = kw0 + 16 * (q >> 1) + 2 * h;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const unsigned skip = (unsigned)(kq + e) * (unsigned)ldb;
            const unsigned rec = q < units ? records_left(b_elems, skip) : 0u;
#pragma unroll
            for (int j = 0; j < NJ; ++j) b[e][j] = stream_load_f32x4(B + n0 + (size_t)skip, b_off[j], rec);
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the loads in front of the MFMAs they overlap
    };
    auto mma_unit = [&](const f32x4 (&a)[MG], int h, const f32x4 (&b)[2][NJ]) {
#pragma unroll
        for (int e = 0; e < 2; ++e)
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int g = 0; g < MG; ++g)
                        acc[g][4 * j + c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g][2 * h + e], b[e][j][c],
                                                                                 acc[g][4 * j + c], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    if (units > 0) {
        f32x4 a[STAGES / 2][MG];
        f32x4 b[STAGES][2][NJ];
#pragma unroll
        for (int i = 0; i < STAGES; ++i) {
            if (i % 2 == 0) load_a(i, a[i / 2]);
            load_unit(i, i % 2, b[i]);
        }
        for (int q = 0; q < units; q += STAGES) {
#pragma unroll
            for (int i = 0; i < STAGES; ++i) {
                mma_unit(a[i / 2], i % 2, b[i]);
                if (i % 2 == 1) load_a(q + i + STAGES, a[i / 2]);  // both halves of the group are done
                load_unit(q + i + STAGES, i % 2, b[i]);
            }
        }
    }
    const int k = kw0 + 8 * units;
    if (k < kw1) {
        // the last 1..15 k of the wave's part, element by element: k at or past kw1 reads as zero
        // on both sides (rows of B between kw1 and K belong to another wave or slice)
#pragma nounroll
        for (int e = 0; e < 4; ++e) {
            const bool below = k + 4 * lq + e < kw1;
            float a[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g)
                a[g] = buffer_load_f32(A + k, below && 16 * g + li < M ? ((16 * g + li) * lda + 4 * lq + e) * 4 : BUF_OOB);
            const float* row = B + n0 + (size_t)(k + e) * ldb;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const bool col = n0 + 64 * j + 4 * li < N;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    // element loads: a 16-byte load of the last row could hang over the end of B
                    const bool ok = below && col && n0 + 64 * j + 4 * li + c < N;
                    const float b = buffer_load_f32(row, ok ? b_off[j] + 4 * c : BUF_OOB);
#pragma unroll
                    for (int g = 0; g < MG; ++g)
                        acc[g][4 * j + c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[g], b, acc[g][4 * j + c], 0, 0, 0);
                }
            }
        }
    }

    // register r of MFMA (g, 4j+c) holds C[16 g + 4 lq + r][n0 + 64 j + 4 li + c].  Wave sums meet in
    // LDS in wave order: red[row][column].
    for (int w = 0; w < 4; ++w) {
        if (w) __syncthreads();
        if (wave == w) {
#pragma unroll
            for (int g = 0; g < MG; ++g)
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        f32x4* p = reinterpret_cast<f32x4*>(red + (16 * g + 4 * lq + r) * COLS + 64 * j + 4 * li);
                        const f32x4 v = {acc[g][4 * j][r], acc[g][4 * j + 1][r], acc[g][4 * j + 2][r], acc[g][4 * j + 3][r]};
                        *p = w == 0 ? v : *p + v;
                    }
        }
    }
    __syncthreads();
    // a thread per column, the rows dealt over the 256 / COLS threads that share it
    const int cl = tid % COLS, n = n0 + cl;
    if (n >= N) return;
    float* dst = out + (size_t)blockIdx.y * out_slice_stride + n;
    const float bias = col_bias ? col_bias[n] : 0.f;
    for (int m = tid / COLS; m < M; m += 256 / COLS) {
        float v = red[m * COLS + cl];
        if (accumulate) v += dst[(size_t)m * out_ld];
        if (col_bias) v += bias;
        dst[(size_t)m * out_ld] = v;
    }
}

// out[i * ld_i + n * ld_n] = sum_k X(i, k) W[n][k] for i < M <= 16, n < N.
// X_KMAJOR: X(i, k) = X[k * ldx + i] (the B of a product with few columns), else X[i * ldx + k].
//
// The MFMA wants lane (lq, li) to hold 4 consecutive k of row li: loaded that way, the four
// lanes of every quad would touch four different rows, and the texture path serves a quad per
// cycle only when its lanes fall into one cache line.  So the wave loads with its lanes along k
// (8 rows x 128 bytes per instruction), passes the data through an LDS area of its own and reads
// it back in MFMA order: no barrier, LDS operations of one wave complete in order.  The waves
// of a workgroup take the steps of 32 k in turn, so together they read 512 contiguous bytes of
// every row at a time.
__device__ __forceinline__ f32x4 keep_below(f32x4 v, int valid)  // zero the elements at and past `valid`
{
    if (valid < 4) v[3] = 0.f;
    if (valid < 3) v[2] = 0.f;
    if (valid < 2) v[1] = 0.f;
    if (valid < 1) v[0] = 0.f;
    return v;
}

// XG groups of 16 rows of X (M <= 16 XG): every W value staged feeds XG MFMAs.
// R rows of W per workgroup (64, 32 or 16), KSTEP k per step of a wave (32 or 64: a load
// instruction covers 8 rows x 128 bytes or 4 rows x 256 bytes), STAGES steps in flight per wave.
// Staged rows are KSTEP + 4 floats apart: the 16-byte reads of 16 rows in MFMA order spread
// over all banks.
template <bool X_KMAJOR, int XG, int R, int KSTEP, int STAGES>
__global__ void __launch_bounds__(256) sgemm_fewrows_nt_kernel(const float* __restrict__ X,
                                                               const float* __restrict__ W,
                                                               float* __restrict__ out, int M, int N, int K,
                                                               int ldx, int ldw, int k_per_slice,
                                                               long long ld_i, long long ld_n,
                                                               size_t out_slice_stride, int accumulate,
                                                               const float* __restrict__ bias_n,
                                                               const float* __restrict__ bias_i)
{
    constexpr int XROWS = 16 * XG;
    constexpr int PITCH = KSTEP + 4;
    constexpr int LPR = KSTEP / 4;                    // lanes along a row in load order
    constexpr int RPI = 64 / LPR;                     // rows per load instruction
    constexpr int NW = R / RPI, NX = XROWS / RPI;     // load instructions per step: W, X (row-major)
    constexpr int NK = KSTEP / 4;                     // k-major X: 4 k per instruction and group
    constexpr int WAVE_FLOATS = (R + XROWS) * PITCH;  // R rows of W and 16 XG of X
    __shared__ __align__(16) float smem[4 * WAVE_FLOATS];
    static_assert(4 * WAVE_FLOATS >= XROWS * R, "the reduction buffer fits the staging memory");
    static_assert(R % 16 == 0 && R % RPI == 0 && XROWS % RPI == 0 && (XROWS * R) % 256 == 0, "shape");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;       // MFMA order: row li, k = 4 lq .. + 3 of a group of 16
    const int lr = lane / LPR, lc = lane % LPR;     // load order: row lr of RPI, k = 4 lc .. + 3 of the step
    const int n0 = blockIdx.x * R;
    const int kbeg = blockIdx.y * k_per_slice;
    const int kend = min(K, kbeg + k_per_slice);
    float* Ws = smem + wave * WAVE_FLOATS;      // [R][PITCH]
    float* Xs = Ws + R * PITCH;                 // [16 XG][PITCH]

    const float* Wb = W + (size_t)n0 * ldw;
    const int rows_left = N - n0;
    const unsigned w_elems = clamp_elems((long long)(rows_left - 1) * ldw + K);
    const unsigned x_elems = clamp_elems(X_KMAJOR ? (long long)(K - 1) * ldx + M : (long long)(M - 1) * ldx + K);
    const int w_off = (lr * ldw + 4 * lc) * 4;
    const int x_off = X_KMAJOR ? (lq * ldx + li) * 4 : (lr * ldx + 4 * lc) * 4;

    f32x4 acc[XG][R / 16];
#pragma unroll
    for (int xg = 0; xg < XG; ++xg)
#pragma unroll
        for (int g = 0; g < R / 16; ++g) acc[xg][g] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Rows at and past N (or M) are not masked: what they bring only reaches results that are
    // never written.  Their addresses are kept inside the operands by exact record counts, and
    // a group of rows that starts past the end gets a count of 0 (records_left must not be asked
    // about a start past the end: its difference would wrap to "everything in range").
    // TAIL: the last, partial step of the slice; k at and past kend reads as zero on both sides.
    // live = false: a step past the end of the wave's share, loaded as zeros without a memory
    // access (record count 0), so that the loop below needs no branch
    auto load_step = [&](int k, bool live, auto tail, f32x4 (&gw)[NW], f32x4 (&gx)[NX], float (&gk)[NK * XG]) {
        constexpr bool TAIL = decltype(tail)::value;
        const int below = kend - (k + 4 * lc);   // of this lane's 4 k, how many lie below kend
#pragma unroll
        for (int t = 0; t < NW; ++t) {
            const unsigned used = (unsigned)(RPI * t) * (unsigned)ldw + (unsigned)k;
            const unsigned rec = live && RPI * t < rows_left ? records_left(w_elems, used) : 0u;
            gw[t] = stream_load_f32x4(Wb + (size_t)(RPI * t) * ldw + k, TAIL && below <= 0 ? BUF_OOB : w_off, rec);
            if (TAIL) gw[t] = keep_below(gw[t], below);
        }
        if constexpr (!X_KMAJOR) {
#pragma unroll
            for (int t = 0; t < NX; ++t) {
                const unsigned used = (unsigned)(RPI * t) * (unsigned)ldx + (unsigned)k;
                const unsigned rec = live && RPI * t < M ? records_left(x_elems, used) : 0u;
                gx[t] = buffer_load_f32x4(X + (size_t)(RPI * t) * ldx + k, TAIL && below <= 0 ? BUF_OOB : x_off, rec);
                if (TAIL) gx[t] = keep_below(gx[t], below);
            }
        } else {
#pragma unroll
            for (int t = 0; t < NK; ++t) {   // k = 4 t + lq of the step, i = 16 xg + li
                const unsigned used = (unsigned)(k + 4 * t) * (unsigned)ldx;
                const unsigned rec = live && (!TAIL || k + 4 * t < kend) ? records_left(x_elems, used) : 0u;
                const int off = TAIL && k + 4 * t + lq >= kend ? BUF_OOB : x_off;
#pragma unroll
                for (int xg = 0; xg < XG; ++xg)  // BUF_OOB plus 64 bytes stays out of range
                    gk[XG * t + xg] = load_f32(X + (size_t)(k + 4 * t) * ldx, off + 64 * xg, rec);
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // keep the loads in front of the MFMAs they overlap
    };
    auto store_step = [&](const f32x4 (&gw)[NW], const f32x4 (&gx)[NX], const float (&gk)[NK * XG]) {
#pragma unroll
        for (int t = 0; t < NW; ++t) *reinterpret_cast<f32x4*>(Ws + (RPI * t + lr) * PITCH + 4 * lc) = gw[t];
        if constexpr (!X_KMAJOR) {
#pragma unroll
            for (int t = 0; t < NX; ++t) *reinterpret_cast<f32x4*>(Xs + (RPI * t + lr) * PITCH + 4 * lc) = gx[t];
        } else {
#pragma unroll
            for (int t = 0; t < NK; ++t)
#pragma unroll
                for (int xg = 0; xg < XG; ++xg) Xs[(16 * xg + li) * PITCH + 4 * t + lq] = gk[XG * t + xg];
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto compute_step = [&]() {
#pragma unroll
        for (int u = 0; u < KSTEP / 16; ++u) {
            f32x4 x[XG];
#pragma unroll
            for (int xg = 0; xg < XG; ++xg)
                x[xg] = *reinterpret_cast<const f32x4*>(Xs + (16 * xg + li) * PITCH + 16 * u + 4 * lq);
#pragma unroll
            for (int g = 0; g < R / 16; ++g) {
                const f32x4 w = *reinterpret_cast<const f32x4*>(Ws + (16 * g + li) * PITCH + 16 * u + 4 * lq);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int xg = 0; xg < XG; ++xg)
                        acc[xg][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[xg][e], w[e], acc[xg][g], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    {
        // The wave's steps are wave, wave + 4, ... below `full`; STAGES of them are in flight.
        f32x4 gw[STAGES][NW], gx[STAGES][NX];
        float gk[STAGES][NK * XG];
        const int full = (kend - kbeg) / KSTEP;
        const int mine = full > wave ? (full - wave + 3) >> 2 : 0;
        // Workgroups start their walk at different steps and wrap around: rows of W are a power
        // of two apart more often than not, and workgroups that all read the same k of their rows
        // at the same time meet in the same memory channels (a pure read of 8192 x 8192 in this
        // shape: 56 us from a common start, 38 us rotated).
        const int rot = full > 0 ? (int)((blockIdx.x * 7u) % (unsigned)full) : 0;
        auto step_k = [&](int j) {
            int s = wave + 4 * j + rot;
            if (s >= full) s -= full;
            return kbeg + KSTEP * s;
        };
        if (mine > 0) {
#pragma unroll
            for (int i = 0; i < STAGES; ++i) load_step(step_k(i), i < mine, std::false_type{}, gw[i], gx[i], gk[i]);
            for (int j = 0; j < mine; j += STAGES) {
#pragma unroll
                for (int i = 0; i < STAGES; ++i) {
                    store_step(gw[i], gx[i], gk[i]);
                    load_step(step_k(j + i + STAGES), j + i + STAGES < mine, std::false_type{}, gw[i], gx[i], gk[i]);
                    compute_step();
                }
            }
        }
        if (((kend - kbeg) & (KSTEP - 1)) && wave == (full & 3)) {
            load_step(kbeg + KSTEP * full, true, std::true_type{}, gw[0], gx[0], gk[0]);
            store_step(gw[0], gx[0], gk[0]);
            compute_step();
        }
    }

    // register r of acc[xg][g] holds C'[16 xg + 4 lq + r][n0 + 16 g + li]; wave sums meet in LDS in
    // wave order
    float* red = smem;
    for (int w = 0; w < 4; ++w) {
        __syncthreads();  // the first: every wave is done with its staging area
        if (wave == w) {
#pragma unroll
            for (int xg = 0; xg < XG; ++xg)
#pragma unroll
                for (int g = 0; g < R / 16; ++g)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float* p = red + (16 * xg + 4 * lq + r) * R + 16 * g + li;
                        *p = w == 0 ? acc[xg][g][r] : *p + acc[xg][g][r];
                    }
        }
    }
    __syncthreads();
    constexpr int PER_THREAD = XROWS * R / 256;     // rows of C' per thread: thread (tid / R) owns PER_THREAD of them
    const int n = n0 + tid % R;
    if (n >= N) return;
    float* dst = out + (size_t)blockIdx.y * out_slice_stride + (long long)n * ld_n;
    const float bn = bias_n ? bias_n[n] : 0.f;
#pragma unroll
    for (int r = 0; r < PER_THREAD; ++r) {
        const int i = PER_THREAD * (tid / R) + r;
        if (i >= M) break;
        float v = red[i * R + tid % R];
        if (accumulate) v += dst[i * ld_i];
        if (bias_n) v += bn;
        if (bias_i) v += bias_i[i];
        dst[i * ld_i] = v;
    }
}

static int slice_length(int K, int slices, int* used)
{
    int k_per = (K + slices - 1) / slices;
    k_per = (k_per + FR_K_UNIT - 1) / FR_K_UNIT * FR_K_UNIT;
    *used = (K + k_per - 1) / k_per;
    return k_per;
}

// Columns of B per workgroup of the nn kernel: 128, or 64 for small products, which then spread
// over more workgroups with fewer K slices (measured: 16 x 4096 x 4096 17 us against 21 us;
// 256 columns were slower throughout, 16 x 8192 x 8192: 63 us against 49 us), and for more than
// 64 rows, whose sums leave registers for no more.
static int nn_cols(int M, int N, int K) { return M > 64 || (double)N * K <= 24.0e6 ? 64 : 128; }

// workgroups per CU: what the registers of the nn kernel and the LDS of the nt kernel allow
int fewrows_slices(int M, int N, int K, int cus)
{
    // Workgroups = column blocks x slices, up to three per CU.  What decides is how evenly they
    // fill the CUs: the slice count whose workgroups come closest to whole rounds of one per CU
    // wins, the smaller count among equals (16 rows, N x K, us by slices: 16384^2 158.7 in 2,
    // 166.6 in 4; 20000^2 304 in 2, 241 in 3, 259 in 4; 24576^2 427 in 2, 440 in 3, 379 in 4;
    // 14336^2 140.6 in 2, 172 in 3, 143.5 in 4; 30000 x 12000 229 in 1, 239 in 2).
    const int blocks = (N + nn_cols(M, N, K) - 1) / nn_cols(M, N, K);
    const int max_slices = std::max(1, std::min((K + FR_K_UNIT - 1) / FR_K_UNIT, std::max(1, 3 * cus / blocks)));
    int best = 1;
    double best_fill = 0.0;
    for (int s = 1; s <= max_slices; ++s) {
        const long wgs = (long)blocks * s;
        const double fill = (double)wgs / (double)((wgs + cus - 1) / cus * cus);
        if (fill > best_fill + 0.03) { best_fill = fill; best = s; }
    }
    return best;
}
// Shape of the nt kernel for a product: rows of W per workgroup (64 with steps of 32 k, 32 or 16
// with steps of 64 k and two of them in flight; with two groups of rows of X, whose matrix work per
// byte of W is twice as long, two steps of 32 k in flight for 64 and 32 rows: 32 x 16384 x 16384
// 208 -> 189 us, 32 x 8192 x 8192 60 -> 54 us) and K slices.  Every pair is priced by a small model
// of what a sweep of 48 products showed (16 and 32 rows of X, W from 2048^2 to 20000^2, both
// layouts of X; us on one device) and the cheapest is taken:
//  * the stream of W runs at the rate of a plain read times how evenly the workgroups fill the
//    CUs -- rounds of one per CU, and rounds of as many as the LDS lets a CU hold (16 x 8192 x 8192:
//    32 rows in 256 workgroups 41.5, 64 rows in 2 x 128: 45.0; 16 x 10000 x 10000: 64 rows in 3 slices,
//    471 workgroups, 91; in 1 slice, 157 workgroups, 102);
//  * two groups of 16 rows of X want more than one workgroup per CU (32 x 16384 x 16384: 512
//    workgroups 202, 256 workgroups 223);
//  * fewer rows per workgroup fetch X more often: 16 rows cost 8-10 % over 64 with X in rows, twice
//    that with X k-major, whose loads are single floats (16 x 16384 x 16384: 64 rows 153, 32 rows 161);
//  * K slices cost the kernel that adds them up, and more with every slice (16 x 4096 x 4096: 16 rows
//    in one slice 14.1, 64 rows in 4 slices 17.6; 16 x 1024 x 8192: 16 rows in 4 slices 12.1, 64 rows
//    in 16 slices 15.4);
//  * a workgroup spends about 1.5 us before its stream is up to speed, so short rows want few
//    workgroups (16 x 100000 x 512: 64 rows 36.9, 32 rows 42.4: rows of up to 1024 k keep 64 rows
//    per workgroup when that fills the device);
//  * rows of W that are not 16-byte aligned cost the 128-byte pieces of the 64-row shape more
//    (16 x 16385 x 4097: 32 rows 60.6, 64 rows 66.8).
// Over the sweep the choice is within 1.7 % of the best shape measured on average, 15 % at worst.
struct NtConfig { int rows, kstep, stages, slices; };
static NtConfig nt_config(int M, int N, int K, int ldw, bool x_kmajor, int cus)
{
    static const NtConfig shapes1[3] = {{64, 32, 1, 1}, {32, 64, 2, 1}, {16, 64, 2, 1}};
    static const NtConfig shapes2[3] = {{64, 32, 2, 1}, {32, 32, 2, 1}, {16, 64, 2, 1}};   // two groups: two steps in flight throughout
    const int groups = M <= 16 ? 1 : 2;
    const NtConfig (&shapes)[3] = groups == 1 ? shapes1 : shapes2;
    const double stream_us = (double)N * K * 4.0 / 7.0e6;
    const double need = groups == 2 ? 1.5 * cus : 1.0 * cus;
    NtConfig best = shapes[0];
    double best_us = 1e30;
    for (const NtConfig& shape : shapes) {
        const long blocks = (N + shape.rows - 1) / shape.rows;
        // rows too short to pay for a workgroup's start twice as often, and 64-row blocks fill the device anyway
        if (shape.rows < 64 && K <= 1024 && (N + 63) / 64 >= cus) continue;
        const long lds = (long)(shape.rows + 16 * groups) * (shape.kstep + 4) * 16;
        const long resident = std::max(1L, std::min(4L, 163840L / lds)) * cus;
        const double refetch = 1.0 + (x_kmajor ? 0.6 : 0.3) * 16.0 * groups / shape.rows;
        const double unaligned = shape.rows == 64 && ldw % 4 != 0 ? 1.15 : 1.0;
        const int max_slices = std::max(1, std::min((K + FR_K_UNIT - 1) / FR_K_UNIT, (int)((3L * cus + blocks - 1) / blocks)));
        for (int s = 1; s <= max_slices; ++s) {
            int used;
            (void)slice_length(K, s, &used);
            if (used != s) continue;     // the rounding of slices to whole units gives this count no launch of its own
            const long wgs = blocks * s;
            const double per_cu = wgs < cus ? (double)wgs / cus : (double)wgs / (double)((wgs + cus - 1) / cus * cus);
            const double per_round = wgs > resident ? (double)wgs / (double)((wgs + resident - 1) / resident * resident) : 1.0;
            const double busy = std::min(per_cu, per_round) * std::pow(std::min(1.0, wgs / need), 0.2);
            const double rounds = (double)((wgs + resident - 1) / resident);     // every round starts its stream anew
            const double us = stream_us / busy * refetch * unaligned + 1.5 * rounds + (s > 1 ? 4.5 + 0.4 * s : 0.0);
            if (us < best_us) {
                best_us = us; best = shape; best.slices = s;
                // a second step in flight pays once a wave has a dozen steps to walk (32 x 3000 x 5000 in
                // 5 slices of 64 rows: 24.2 us with one step in flight, 26.7 with two)
                if (shape.rows == 64 && slice_length(K, s, &used) < 1536) best.stages = 1;
            }
        }
    }
    return best;
}
int fewrows_nt_slices(int M, int N, int K, int ldw, bool x_kmajor, int cus) { return nt_config(M, N, K, ldw, x_kmajor, cus).slices; }

// A tall A (rows x K, row pitch lda) against up to 16 columns of B (K x cols): whether to turn B
// into `cols` rows of K first, so that the kernel loads it 16 bytes at a time and stages it with a
// quarter of the LDS stores.  That costs a small kernel in front (about 3 us) and pays where
// workgroups of fewer than 64 rows, which fetch B more often, would fetch it k-major at twice the
// price: a single K slice, rows of 4096 k and more (us, B as it lies -> turned: 8192 x 16 x 4096
// 30.7 -> 27.0, 4096 x 16 x 4096 20.8 -> 18.1, 8192 x 16 x 8192 48.7 -> 45.7, 7000 x 16 x 7000
// 53.2 -> 48.6; not with 64-row workgroups, K slices or short rows: 16384 x 16 x 4096 45.1 ->
// 45.6, 10000 x 16 x 10000 91.7 -> 96.5, 32768 x 16 x 1024 24.2 -> 27.0, 3000 x 16 x 5000 20 -> 24),
// and against 200 million elements and more with rows of 16384 k (16384 x 16 x 16384: 166 -> 158).
// Over 28 products from 2048^2 to 20000^2 the choice is 0.6 % off the better of the two on
// average and 4.5 % at worst.
bool fewrows_nt_turn_pays(int cols, int rows, int K, int lda, int cus)
{
    if (cols > 16 || K < 4096) return false;
    if (K >= 16384 && (double)rows * K >= 200.0e6) return true;
    if (rows < 4096 || lda % 4 != 0) return false;
    const NtConfig turned = nt_config(cols, rows, K, lda, false, cus);
    return turned.slices == 1 && turned.rows < 64;
}

bool fewrows_applies(int M, int N, int K, int lda, int ldb)
{
    // byte offsets inside a group (15 rows of B plus 256 columns, 111 rows of A) must stay below 2^31
    // 33 to 48 rows only against a large B: at 4096 x 4096 the macro-tile is the faster one (23 against
    // 26 us); 49 to 64 rows against a larger one still; 65 to 80 and 97 to 112 rows where the
    // macro-tiles would pad to 96 and 128 (81 to 96 rows fill the 96-row tile)
    const double big = (double)N * K;
    // 17 to 32 rows stream from 100 million elements of B on; below, the 32 x 128 macro-tile in its
    // K slices is ahead at every size (us, here / tile: 32 x 8192 x 8192 52 / 46, 32 x 4096 x 4096
    // 20 / 16, 32 x 3333 x 3333 24 / 14.5, 32 x 1000 x 1000 12 / 11; 32 x 10000 x 10000 81 on either).
    // Up to 16 rows stay here: the tile gains and loses 5-10 % from size to size (16 x 6144 x 6144
    // 34 / 31, 16 x 11008 x 4096 37 / 38.5, 8 x 9000 x 3000 27 / 30, 16 x 8192 x 1024 10 / 12).
    const bool few = M <= 16 || (M <= 32 && (big >= 100.0e6 || N < 1024));   // (a B of few columns has too few tiles: 24 x 640 x 20000 19 / 21)
    const bool rows_ok = M >= 1 && (few || (M > 32 && M <= 48 && big >= 48.0e6) || (M > 48 && M <= 64 && big >= 100.0e6) ||
                                    (M > 64 && M <= 80 && big >= 30.0e6) || (M > 96 && M <= 112 && big >= 64.0e6));
    // (a short K walk is over before the stream is up to speed: 32 x 6512 x 76 takes 6.4 us here
    // and 5.1 us on a 64 x 64 tile, 32 x 2882 x 216 7.5 against 6.9 us; with a single group of 16
    // rows it pays from a shorter K on, 13 x 2236 x 184: 5.5 against 6.8 us)
    return rows_ok && N >= 512 && K >= (M <= 16 ? 128 : 256) && (double)ldb * 16 * 4 + 1024 < 2147483648.0 &&
           (double)lda * 112 * 4 < 2147483648.0;
}

bool fewrows_nt_applies(int M, int N, int K, int ldx, int ldw, bool x_kmajor)
{
    // 64 rows of W, and 32 rows (or 32 k) of X, within 2^31 bytes of the block's origin.
    // X as the rows of a small batch (a linear layer, W as it lies): up to 32 rows; a third group
    // of 16 was measured and lost to the macro-tile kernel that reads W along k (48 x 8192 x 8192:
    // 82 against 72 us).
    // X as the few columns of a product (k-major), against the 128 x 32 macro-tile with its K
    // slices (us, here / tile): 17 to 32 columns from 100 million elements of W on (16384 x 32 x
    // 8192 102 / 140, 32768 x 32 x 4096 97 / 123, 16384 x 32 x 16384 190 / 213; below: 16384 x 32 x
    // 4096 68 / 47, 8192 x 32 x 8192 59 / 53, 100000 x 20 x 512 62 / 41, 8192 x 32 x 4096 38 / 26);
    // up to 16 columns everywhere but between 8 and 60 million elements with rows of 2048 to
    // 8192 k (8192 x 8 x 4096 27 / 25, 4096 x 16 x 4096 18 / 16, 3000 x 8 x 3000 17.5 / 13, 2048 x 16 x
    // 8192 22 / 17; outside: 16384 x 16 x 4096 45 / 45, 1000 x 5 x 1000 8.8 / 11.8, 4096 x 8 x 1024
    // 7.7 / 9.4, 1024 x 16 x 16384 21 / 23).
    const double big = (double)N * K;
    const bool cols_ok = M <= 16 ? !(big >= 8.0e6 && big <= 60.0e6 && K >= 2048 && K <= 8192) : (M <= 32 && big >= 100.0e6);
    // X as rows, 17 to 32 of them: from 100 million elements of W on, and for small layers and short
    // rows; between, the 32 x 128 macro-tile that reads W along k is ahead (us, here / tile: 32 x 8192
    // x 8192 56 / 50, 32 x 4096 x 11008 45 / 38, 32 x 14336 x 4096 56 / 41, 32 x 4096 x 4096 22 / 16.5, 32 x
    // 100000 x 512 59 / 42; 32 x 1000 x 1000 9.8 / 11.2, 32 x 512 x 512 5.7 / 9.2, 32 x 8192 x 1024 11.5 / 12.9)
    const bool batch_ok = M <= 16 || (M <= 32 && (big >= 100.0e6 || big < 4.0e6 || (K < 2048 && big < 30.0e6)));
    const bool rows_ok = x_kmajor ? cols_ok : batch_ok;
    return M >= 1 && rows_ok && N >= 512 && K >= 64 && (double)ldw * 64 * 4 < 2147483648.0 &&
           (double)ldx * 32 * 4 + (x_kmajor ? 128 : 0) < 2147483648.0;
}

// partial: [slices][M][N] floats when fewrows_slices(M, N, K, cus) > 1, else unused
hipError_t launch_sgemm_fewrows(const float* A, const float* B, float* C, float* partial, int M, int N,
                                int K, int lda, int ldb, int ldc, int accumulate, const float* col_bias,
                                int cus, hipStream_t stream)
{
    if (M > 112) return hipErrorInvalidValue;   // seven groups of 16 rows are the most there are
    int used;
    const int k_per = slice_length(K, fewrows_slices(M, N, K, cus), &used);
    const int cols = nn_cols(M, N, K);
    const dim3 grid((N + cols - 1) / cols, used), block(256);
    float* out = used > 1 ? partial : C;
    const int out_ld = used > 1 ? N : ldc;
    const size_t stride = used > 1 ? (size_t)M * N : 0;
    auto kernel = M <= 16 ? (cols == 128 ? sgemm_fewrows_nn_kernel<1, 2> : sgemm_fewrows_nn_kernel<1, 1>)
                : M <= 32 ? (cols == 128 ? sgemm_fewrows_nn_kernel<2, 2> : sgemm_fewrows_nn_kernel<2, 1>)
                : M <= 48 ? (cols == 128 ? sgemm_fewrows_nn_kernel<3, 2> : sgemm_fewrows_nn_kernel<3, 1>)
                : M <= 64 ? (cols == 128 ? sgemm_fewrows_nn_kernel<4, 2> : sgemm_fewrows_nn_kernel<4, 1>)
                : M <= 80 ? sgemm_fewrows_nn_kernel<5, 1> : sgemm_fewrows_nn_kernel<7, 1>;
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, A, B, out, M, N, K, lda, ldb, k_per,
                       out_ld, stride, used > 1 ? 0 : accumulate, used > 1 ? nullptr : col_bias);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || used == 1) return e;
    return launch_splitk_reduce(partial, C, M, N, ldc, used, accumulate, stream, nullptr, col_bias);
}

// C'(i, n) = sum_k X(i, k) W[n][k] for i < M <= 32, n < N.
// c_is_n_by_m = false: C is M x N (C[i * ldc + n], bias per n);  true: C is N x M (C[n * ldc + i],
// bias per i): in both cases `bias` runs along the columns of C.
// partial: [slices] copies of C without padding when fewrows_nt_slices(M, N, K, cus) > 1
hipError_t launch_sgemm_fewrows_nt(const float* X, const float* W, float* C, float* partial, int M, int N,
                                   int K, int ldx, int ldw, int ldc, bool x_kmajor, bool c_is_n_by_m,
                                   int accumulate, const float* bias, int cus, hipStream_t stream)
{
    int used;
    const NtConfig cfg = nt_config(M, N, K, ldw, x_kmajor, cus);
    const int k_per = slice_length(K, cfg.slices, &used);
    const dim3 grid((N + cfg.rows - 1) / cfg.rows, used), block(256);
    const bool split = used > 1;
    float* out = split ? partial : C;
    const long long ld_i = c_is_n_by_m ? 1 : (split ? N : ldc);
    const long long ld_n = c_is_n_by_m ? (split ? M : ldc) : 1;
    const size_t stride = split ? (size_t)M * N : 0;
    const float* bias_n = split || c_is_n_by_m ? nullptr : bias;
    const float* bias_i = split || !c_is_n_by_m ? nullptr : bias;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, block, 0, stream, X, W, out, M, N, K, ldx, ldw, k_per, ld_i, ld_n, stride,
                           split ? 0 : accumulate, bias_n, bias_i);
    };
    auto pick = [&](auto rows, auto kstep, auto stages) {
        constexpr int R = decltype(rows)::value, KS = decltype(kstep)::value, ST = decltype(stages)::value;
        if (M <= 16) x_kmajor ? launch(sgemm_fewrows_nt_kernel<true, 1, R, KS, ST>) : launch(sgemm_fewrows_nt_kernel<false, 1, R, KS, ST>);
        else x_kmajor ? launch(sgemm_fewrows_nt_kernel<true, 2, R, KS, ST>) : launch(sgemm_fewrows_nt_kernel<false, 2, R, KS, ST>);
    };
    using std::integral_constant;
    switch (cfg.rows * 1000 + cfg.kstep * 10 + cfg.stages) {
    case 64321: pick(integral_constant<int, 64>{}, integral_constant<int, 32>{}, integral_constant<int, 1>{}); break;
    case 64322: pick(integral_constant<int, 64>{}, integral_constant<int, 32>{}, integral_constant<int, 2>{}); break;
    case 32642: pick(integral_constant<int, 32>{}, integral_constant<int, 64>{}, integral_constant<int, 2>{}); break;
    case 32322: pick(integral_constant<int, 32>{}, integral_constant<int, 32>{}, integral_constant<int, 2>{}); break;
    default: pick(integral_constant<int, 16>{}, integral_constant<int, 64>{}, integral_constant<int, 2>{}); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !split) return e;
    return c_is_n_by_m ? launch_splitk_reduce(partial, C, N, M, ldc, used, accumulate, stream, nullptr, bias)
                       : launch_splitk_reduce(partial, C, M, N, ldc, used, accumulate, stream, nullptr, bias);
}

}  // namespace cake
