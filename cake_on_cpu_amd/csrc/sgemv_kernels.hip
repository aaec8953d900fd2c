// sgemv_kernels.hip -- bandwidth-bound fp32 matrix-vector kernels for gfx950.
//
// They replace cake_sgemv's schedule_mvm + cake_sgemv_haswell_8x8_col
// (examples/cake_gemv.cpp:89-140,424-490).  A is read exactly once with
// 16-byte, fully coalesced loads; x is small and is served from cache.
//
//   row-major  A[m*K + k]: long rows (K >= 2048): one workgroup per 2 rows,
//              all its lanes stride over k (each row is read as one
//              sequential stream, which is what keeps the HBM pages open);
//              short rows: one wavefront per 4 rows.  64-lane butterfly
//              reduction at the end.
//   col-major  A[k*M + m] (the reference's layout): lanes own 4 consecutive m,
//              K is cut into slices across workgroups and waves; slices are
//              summed in a fixed order (no atomics), so results are
//              run-to-run identical.
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace cake {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// ---------------------------------------------------------------------------
// row-major
// ---------------------------------------------------------------------------
template <int ROWS, bool VEC>
__global__ void __launch_bounds__(256) sgemv_rowmajor_kernel(const float* __restrict__ A,
                                                             const float* __restrict__ x,
                                                             float* __restrict__ y, int M, int K,
                                                             int accumulate)
{
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = wave * ROWS;
    if (row0 >= M) return;

    float acc[ROWS];
    const float* rowp[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        acc[r] = 0.f;
        // rows past the end re-read the last row; their sums are dropped below
        rowp[r] = A + (size_t)min(row0 + r, M - 1) * K;
    }

    if (VEC) {
        const int K4 = K >> 2;
        const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
        // Rows are a power of two of bytes apart more often than not, and the same k of the ROWS rows
        // of a wave then lies in the same memory channel: each row is walked one step further along
        // than the one before (whole steps of 64 lanes, wrapping around; the rest of a row after them).
        const int whole = K4 >> 6;
        const int skew = whole >= ROWS ? 1 : 0;    // (so that one subtraction wraps every row)
#pragma unroll 4
        for (int i = 0; i < whole; ++i) {
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                int it = i + r * skew;
                if (it >= whole) it -= whole;
                const int c = it * 64 + lane;
                const f32x4 xv = x4[c];
                const f32x4 av = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(rowp[r]) + c);
                acc[r] += av.x * xv.x + av.y * xv.y + av.z * xv.z + av.w * xv.w;
            }
        }
        const int c = whole * 64 + lane;
        if (c < K4) {
            const f32x4 xv = x4[c];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const f32x4 av = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(rowp[r]) + c);
                acc[r] += av.x * xv.x + av.y * xv.y + av.z * xv.z + av.w * xv.w;
            }
        }
    } else {
#pragma unroll 4
        for (int c = lane; c < K; c += 64) {
            const float xv = x[c];
#pragma unroll
            for (int r = 0; r < ROWS; ++r) acc[r] += rowp[r][c] * xv;
        }
    }

#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float s = wave_sum(acc[r]);
        if (lane == 0 && row0 + r < M) y[row0 + r] = accumulate ? y[row0 + r] + s : s;
    }
}

// Long rows: the whole workgroup walks ROWS rows front to back, so each row is
// one sequential 16-byte-per-lane stream; wave sums meet in LDS in wave order.
template <int ROWS, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) sgemv_rowmajor_wg_kernel(const float* __restrict__ A,
                                                                       const float* __restrict__ x,
                                                                       float* __restrict__ y, int M,
                                                                       int K, int accumulate,
                                                                       int k4_per_slice)
{
    // grid.y > 1: few rows and very long ones -- each workgroup takes a slice of k and writes
    // its sums to y[slice][M] (a scratch array that sgemv_slice_reduce_kernel adds up in order)
    __shared__ float red[WAVES][ROWS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = blockIdx.x * ROWS;
    y += (size_t)blockIdx.y * M;
    float acc[ROWS];
    const f32x4* rowp[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        acc[r] = 0.f;
        rowp[r] = reinterpret_cast<const f32x4*>(A + (size_t)min(row0 + r, M - 1) * K);
    }
    const int c_begin = blockIdx.y * k4_per_slice;
    const int c_end = min(K >> 2, c_begin + k4_per_slice);
    const f32x4* x4 = reinterpret_cast<const f32x4*>(x);
#pragma unroll 4
    for (int c = c_begin + tid; c < c_end; c += WAVES * 64) {
        const f32x4 xv = x4[c];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const f32x4 av = __builtin_nontemporal_load(rowp[r] + c);
            acc[r] += av.x * xv.x + av.y * xv.y + av.z * xv.z + av.w * xv.w;
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const float s = wave_sum(acc[r]);
        if (lane == 0) red[wave][r] = s;
    }
    __syncthreads();
    if (tid < ROWS && row0 + tid < M) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) s += red[w][tid];
        y[row0 + tid] = accumulate ? y[row0 + tid] + s : s;
    }
}

// The same sweep against NV vectors at once (a linear layer on two samples):
// Y[v][row] = bias[row] + sum_k A[row][k] * X[v][k].  A is read once for all of them, but every
// workgroup reads all of X through the caches, NV/ROWS bytes for each byte of A, and that
// traffic is what limits it: measured at 4096 x 4096, 2 vectors take 11.6 us (one: 10.8) where 4
// take 17.5 us and 8 take 24 us or more, which is no better than the streaming matrix-core
// kernel for few rows.  Vectors past `vectors` repeat the last one and are not written.
template <int ROWS, int NV>
__global__ void __launch_bounds__(512) sgemv_rowmajor_multi_kernel(const float* __restrict__ A,
                                                                   const float* __restrict__ X,
                                                                   float* __restrict__ Y,
                                                                   const float* __restrict__ bias, int M,
                                                                   int K, int vectors, int ldx, int ldy)
{
    constexpr int WAVES = 8;
    __shared__ float red[WAVES][ROWS * NV];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = blockIdx.x * ROWS;
    float acc[ROWS][NV];
    const f32x4* rowp[ROWS];
    const f32x4* xp[NV];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        rowp[r] = reinterpret_cast<const f32x4*>(A + (size_t)min(row0 + r, M - 1) * K);
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[r][v] = 0.f;
    }
#pragma unroll
    for (int v = 0; v < NV; ++v)
        xp[v] = reinterpret_cast<const f32x4*>(X + (size_t)min(v, vectors - 1) * ldx);
    const int c_end = K >> 2;
#pragma unroll 2
    for (int c = tid; c < c_end; c += WAVES * 64) {
        f32x4 av[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) av[r] = __builtin_nontemporal_load(rowp[r] + c);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const f32x4 xv = xp[v][c];
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
                acc[r][v] += av[r].x * xv.x + av[r].y * xv.y + av[r].z * xv.z + av[r].w * xv.w;
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const float s = wave_sum(acc[r][v]);
            if (lane == 0) red[wave][r * NV + v] = s;
        }
    __syncthreads();
    if (tid < ROWS * NV) {
        // consecutive threads write consecutive rows of one vector
        const int v = tid / ROWS, r = tid % ROWS;
        if (row0 + r < M && v < vectors) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) s += red[w][r * NV + v];
            if (bias) s += bias[row0 + r];
            Y[(size_t)v * ldy + row0 + r] = s;
        }
    }
}

// Very short rows (K <= 32): a thread per row.  Neighbouring threads read neighbouring rows, so a
// wave still touches one contiguous piece of A, and the few loads of a row hit the same lines.
template <bool VEC>
__global__ void __launch_bounds__(256) sgemv_rowmajor_thread_kernel(const float* __restrict__ A,
                                                                    const float* __restrict__ x,
                                                                    float* __restrict__ y, int M, int K,
                                                                    int accumulate)
{
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row >= M) return;
    const float* a = A + (size_t)row * K;
    float acc = 0.f;
    if (VEC) {
        for (int k = 0; k < K; k += 4) {
            const f32x4 av = *reinterpret_cast<const f32x4*>(a + k);
            acc += av.x * x[k] + av.y * x[k + 1] + av.z * x[k + 2] + av.w * x[k + 3];
        }
    } else {
        for (int k = 0; k < K; ++k) acc += a[k] * x[k];
    }
    y[row] = accumulate ? y[row] + acc : acc;
}

__global__ void sgemv_slice_reduce_kernel(const float* __restrict__ part, float* __restrict__ y, int M,
                                          int slices, int accumulate);

// K slices for the long-row kernel when the rows alone do not fill the device.
static int rowmajor_slices(int M, int K, int cus)
{
    const int wgs = (M + 1) / 2;
    if (K < 16384 || wgs >= cus) return 1;
    int want = (2 * cus + wgs - 1) / wgs;
    const int max_slices = K / 8192;  // at least 8192 k per slice
    return want < max_slices ? want : max_slices;
}

size_t sgemv_rowmajor_scratch_floats(int M, int K, int cus)
{
    const int s = rowmajor_slices(M, K, cus);
    return s > 1 ? (size_t)s * M : 0;
}

hipError_t launch_sgemv_rowmajor(const float* A, const float* x, float* y, int M, int K,
                                 int accumulate, float* scratch, int cus, hipStream_t stream)
{
    if (M <= 0) return hipSuccess;
    constexpr int ROWS = 4;
    const bool vec = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(x)) % 16 == 0);
    const int waves = (M + ROWS - 1) / ROWS;
    const int blocks = (waves + 3) / 4;
    if (K <= 32) {
        if (vec)
            hipLaunchKernelGGL((sgemv_rowmajor_thread_kernel<true>), dim3((M + 255) / 256), dim3(256), 0, stream, A, x, y, M, K, accumulate);
        else
            hipLaunchKernelGGL((sgemv_rowmajor_thread_kernel<false>), dim3((M + 255) / 256), dim3(256), 0, stream, A, x, y, M, K, accumulate);
        return hipGetLastError();
    }
    if (vec && K >= 8192) {
        const int slices = scratch ? rowmajor_slices(M, K, cus) : 1;
        if (slices > 1) {
            const int k4_per = ((K / 4 + slices - 1) / slices + 511) & ~511;  // whole sweeps of the workgroup
            hipLaunchKernelGGL((sgemv_rowmajor_wg_kernel<2, 8>), dim3((M + 1) / 2, slices), dim3(512), 0, stream, A, x, scratch, M, K, 0, k4_per);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            hipLaunchKernelGGL(sgemv_slice_reduce_kernel, dim3((M + 63) / 64), dim3(256), 0, stream, scratch, y, M, slices, accumulate);
            return hipGetLastError();
        }
        hipLaunchKernelGGL((sgemv_rowmajor_wg_kernel<2, 8>), dim3((M + 1) / 2), dim3(512), 0, stream, A, x, y, M, K, accumulate, K / 4);
        return hipGetLastError();
    }
    if (vec && K >= 2048) {
        hipLaunchKernelGGL((sgemv_rowmajor_wg_kernel<2, 4>), dim3((M + 1) / 2), dim3(256), 0, stream, A, x, y, M, K, accumulate, K / 4);
        return hipGetLastError();
    }
    if (vec)
        hipLaunchKernelGGL((sgemv_rowmajor_kernel<ROWS, true>), dim3(blocks), dim3(256), 0, stream, A, x, y, M, K, accumulate);
    else
        hipLaunchKernelGGL((sgemv_rowmajor_kernel<ROWS, false>), dim3(blocks), dim3(256), 0, stream, A, x, y, M, K, accumulate);
    return hipGetLastError();
}

bool sgemv_rowmajor_multi_applies(int M, int K, int vectors, int ldx, const float* A, const float* X, int cus)
{
    if (vectors != 2 || K < 2048 || K % 4 != 0 || ldx % 4 != 0) return false;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(X)) % 16 != 0) return false;
    // no K slices here: the rows alone have to fill the device.  Beyond about 2^27 elements the
    // streaming kernel for few rows is the faster one (16384 x 16384: 166 us against 180 us).
    return (M + 3) / 4 >= cus && (double)M * K <= 140e6;
}

hipError_t launch_sgemv_rowmajor_multi(const float* A, const float* X, float* Y, const float* bias, int M,
                                       int K, int vectors, int ldx, int ldy, hipStream_t stream)
{
    if (M <= 0 || vectors <= 0) return hipSuccess;
    if (vectors > 2) return hipErrorInvalidValue;
    hipLaunchKernelGGL((sgemv_rowmajor_multi_kernel<4, 2>), dim3((M + 3) / 4), dim3(512), 0, stream, A, X, Y, bias, M, K, vectors, ldx, ldy);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// column-major
// ---------------------------------------------------------------------------
static constexpr int COL_BLOCK_M = 256;  // columns of y per workgroup
static constexpr int COL_MAX_FILL_SLICES = 3;

static int colmajor_slices(int M, int K, int cus)
{
    const int mblocks = (M + COL_BLOCK_M - 1) / COL_BLOCK_M;
    int want = 2 * cus / mblocks;                  // at most 2 workgroups (8 waves) per CU in one round: more concurrent
                                                    // strided streams than that lose HBM page locality
    if (mblocks > cus && mblocks <= 4 * cus) {
        // More blocks of columns than CUs, up to four per CU (beyond that slices only add traffic:
        // 300000 x 500, 1172 blocks: 89 us in 1 slice, 93 in 3): the count whose workgroups come closest to whole rounds
        // of one per CU, the smaller among near-equals, as for the streaming-rows kernel
        // (70000 x 3000, 274 blocks: 180 us in 1 slice, 154 in 2; 80000 x 8000, 313 blocks: 448 and
        // 391 us, 373 in 3; 100000 x 2000, 391 blocks: 122 and 136 us).
        double best = 0.0;
        for (int s = 1; s <= COL_MAX_FILL_SLICES && s * 128 <= K; ++s) {
            const long wgs = (long)mblocks * s;
            const double fill = (double)wgs / (double)((wgs + cus - 1) / cus * cus);
            if (fill > best + 0.03) { best = fill; want = s; }
        }
    }
    // Few blocks of columns: up to 64 slices, more when one or two blocks would otherwise leave most
    // CUs idle (us by slices, with the slices added up by four waves per 64 columns -- one thread per
    // column adding them in turn had made every count above 64 slower: 256 x 262144 88 in 64, 49 in
    // 191, 55 in 255; 300 x 100000 44 in 64, 31 in 127; 512 x 131072 52 in 64, 43 in 96, 45 in 127;
    // 1024 x 65536 42 in 64, 47 in 96; 1000 x 30000 24 in 64, 28 in 96; 2048 x 32768 42 in 64, 48 in 96).
    const int most = mblocks == 1 ? 192 : mblocks == 2 ? 128 : 64;
    if (want > most) want = most;
    int max_slices = (K + 127) / 128;              // at least 128 k per slice (3000^2: 18.8 us in 42 slices, 16.6 in 23)
    if (want > max_slices) want = max_slices;
    if (want < 1) want = 1;
    // Slices that start a power of two of 8 MB or more apart meet in the same memory channels:
    // half as many again moves them off that grid (8192^2: 54.8 us in 16 slices, 45.7 in 24;
    // 8192 x 4096: 36.9 in 16, 25.5 in 24; 16384 x 4096: 51.0 in 8, 42.4 in 12; 32768 x 2048:
    // 47.9 in 4, 41.8 in 6; 16384^2: 158.8 in 8, 156.9 in 12).
    if (want >= 4 && (want & (want - 1)) == 0) {
        const double apart = (double)((K + want - 1) / want) * M * 4.0;
        if (apart >= 8.0 * 1048576.0 && want * 3 / 2 <= max_slices) want = want * 3 / 2;
    }
    return want;
}

size_t sgemv_colmajor_scratch_floats(int M, int K, int cus)
{
    // a single slice writes y itself and touches no workspace
    const int slices = colmajor_slices(M, K, cus);
    return slices > 1 ? (size_t)slices * (size_t)M : 0;
}

// grid = (m blocks, k slices).  VEC: each wave covers all 256 columns of the
// block with one 16-byte load per lane and takes a quarter of the slice's k
// range; the four waves are summed through LDS in wave order.  Scalar: each
// thread owns one column over the whole slice.  A launch of a single slice has `out` = y and
// adds to it or overwrites it itself (`accumulate`); slices go to the workspace, overwriting.
//
// Summing the slices inside this kernel -- every workgroup publishes its partial sums, draws a
// ticket of its block of columns, and the last one adds them up in slice order -- was measured and
// costs far more than the second launch it saves (16384^2: 157 -> 293 us, 4096^2: 15 -> 98 us): the
// device-scope fences it needs write back and invalidate the whole L2 of the workgroup's XCD, and
// with them the stream of A and the vector x that the other workgroups are reading.
template <bool VEC>
__global__ void __launch_bounds__(256) sgemv_colmajor_kernel(const float* __restrict__ A,
                                                             const float* __restrict__ x,
                                                             float* __restrict__ out, int M, int K,
                                                             int k_per_slice, int accumulate)
{
    __shared__ float red[4][COL_BLOCK_M];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kbeg = blockIdx.y * k_per_slice;
    const int kend = min(K, kbeg + k_per_slice);
    float* dst = out + (size_t)blockIdx.y * M;

    if (VEC) {
        const int m = blockIdx.x * COL_BLOCK_M + lane * 4;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        if (m < M) {
            const int span = (kend - kbeg + 3) / 4;
            const int k0 = kbeg + wave * span, k1 = min(kend, k0 + span);
            const float* col = A + (size_t)k0 * M + m;
#pragma unroll 16
            for (int k = k0; k < k1; ++k, col += M) {
                const f32x4 av = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(col));
                const float xv = x[k];
                acc.x += av.x * xv; acc.y += av.y * xv; acc.z += av.z * xv; acc.w += av.w * xv;
            }
        }
        *reinterpret_cast<f32x4*>(&red[wave][lane * 4]) = acc;
        __syncthreads();
        const int mm = blockIdx.x * COL_BLOCK_M + tid;
        if (mm < M) {
            const float sum = ((red[0][tid] + red[1][tid]) + red[2][tid]) + red[3][tid];
            dst[mm] = accumulate ? dst[mm] + sum : sum;
        }
    } else {
        const int m = blockIdx.x * COL_BLOCK_M + tid;
        if (m >= M) return;
        float acc = 0.f;
        const float* col = A + (size_t)kbeg * M + m;
#pragma unroll 8
        for (int k = kbeg; k < kend; ++k, col += M) acc += *col * x[k];
        dst[m] = accumulate ? dst[m] + acc : acc;
    }
}

__global__ void sgemv_slice_reduce_kernel(const float* __restrict__ part, float* __restrict__ y, int M,
                                          int slices, int accumulate)
{
    // 64 columns per workgroup; its four waves each add every fourth slice, several loads in
    // flight, and meet in LDS in wave order: a fixed order, so the same sums from run to run.
    // (One thread per column adding all slices in turn took as long as the slices' loads one after
    // the other: 256 columns in 255 slices 105 us for a product that the main kernel does in 40.)
    __shared__ float red[4][64];
    const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int m = blockIdx.x * 64 + c;
    float acc = 0.f;
    if (m < M) {
#pragma unroll 8
        for (int s = g; s < slices; s += 4) acc += part[(size_t)s * M + m];
    }
    red[g][c] = acc;
    __syncthreads();
    // the slices first, then one addition to what y held: y += A.x rounds the same way whether
    // or not K was cut into slices
    if (g == 0 && m < M) {
        const float sum = ((red[0][c] + red[1][c]) + red[2][c]) + red[3][c];
        y[m] = accumulate ? y[m] + sum : sum;
    }
}

hipError_t launch_sgemv_colmajor(const float* A, const float* x, float* y, int M, int K,
                                 int accumulate, float* scratch, int cus, hipStream_t stream)
{
    if (M <= 0) return hipSuccess;
    const int slices = colmajor_slices(M, K, cus);
    int k_per_slice = (K + slices - 1) / slices;
    k_per_slice = (k_per_slice + 3) & ~3;
    const bool vec = (M % 4 == 0) && (reinterpret_cast<uintptr_t>(A) % 16 == 0);
    const dim3 grid((M + COL_BLOCK_M - 1) / COL_BLOCK_M, slices);
    float* out = slices == 1 ? y : scratch;          // a single slice needs no second launch
    const int acc = slices == 1 ? accumulate : 0;
    if (vec)
        hipLaunchKernelGGL((sgemv_colmajor_kernel<true>), grid, dim3(256), 0, stream, A, x, out, M, K, k_per_slice, acc);
    else
        hipLaunchKernelGGL((sgemv_colmajor_kernel<false>), grid, dim3(256), 0, stream, A, x, out, M, K, k_per_slice, acc);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || slices == 1) return e;
    hipLaunchKernelGGL(sgemv_slice_reduce_kernel, dim3((M + 63) / 64), dim3(256), 0, stream, scratch, y, M, slices, accumulate);
    return hipGetLastError();
}

}  // namespace cake
