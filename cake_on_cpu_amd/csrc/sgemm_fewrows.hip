// sgemm_fewrows.hip -- C[M][N] = A[M][K] . B[K][N] for M <= 16 ("a few vectors
// times a matrix": small-batch linear layers, blocks of matrix-vector products).
//
// Such a product is bound by reading B once from HBM, not by arithmetic, and a
// 64-row macro-tile would waste most of the matrix pipe on zero rows while
// reading B in 256-byte pieces.  Here B is streamed the way the column-major
// matrix-vector kernel streams its operand: a workgroup owns 256 consecutive
// columns and a slice of k; each of its four waves takes a quarter of every k
// chunk and reads whole 1 KB row pieces, 64 bytes per lane.  The arithmetic
// runs on v_mfma_f32_16x16x4_f32, whose 16 rows fit the problem: the 16 columns
// a lane loads feed 16 MFMAs, A comes from a
// k-major copy of the current chunk in LDS.  Wave sums meet in LDS in wave
// order and K slices are summed by splitk_reduce_kernel in slice order, so
// results are run-to-run identical.
//
// Operand layout of v_mfma_f32_16x16x4_f32: lane l supplies A[l % 16][l / 16]
// and B[l / 16][l % 16]; result register r of lane l is C[4 * (l / 16) + r][l % 16].
#include "sgemm_tile.hpp"

namespace cake {

// 16-byte load marked non-temporal: B is read once and should not push A or the partial sums
// out of the caches on its way through
__device__ __forceinline__ f32x4 stream_load_f32x4(const float* base, int byte_offset, unsigned records)
{
    __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)records, 0x00020000);
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, /*nt*/ 2));
}

static constexpr int FR_COLS = 256;   // columns per workgroup
static constexpr int FR_KC = 1024;    // k per LDS chunk of A (a quarter per wave)
static constexpr int FR_PITCH = 17;   // floats per k in the LDS copy of A: odd, so staging writes spread over banks

__global__ void __launch_bounds__(256) sgemm_fewrows_kernel(const float* __restrict__ A,
                                                            const float* __restrict__ B,
                                                            float* __restrict__ out, int M, int N, int K,
                                                            int lda, int ldb, int k_per_slice,
                                                            int out_ld, size_t out_slice_stride,
                                                            int accumulate, const float* __restrict__ col_bias)
{
    __shared__ __align__(16) float smem[FR_KC * FR_PITCH];   // At[k][m] while walking, then the wave sums
    static_assert(FR_KC * FR_PITCH >= 16 * FR_COLS, "the reduction buffer fits the A chunk's memory");
    float* At = smem;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lq = lane >> 4;
    const int n0 = blockIdx.x * FR_COLS;
    const int kbeg = blockIdx.y * k_per_slice;
    const int kend = min(K, kbeg + k_per_slice);
    const unsigned b_elems = clamp_elems((long long)(K - 1) * ldb + N - n0);
    // The lane's four 16-byte pieces of its row of B: piece j is columns 64 j + 4 li .. + 3, so that
    // the 16 lanes of a row read 256 contiguous bytes per load instruction.
    int b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b_off[j] = n0 + 64 * j + 4 * li < N ? (64 * j + 4 * li + lq * ldb) * 4 : BUF_OOB;

    f32x4 acc[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = kbeg; k0 < kend; k0 += FR_KC) {
        __syncthreads();  // the previous chunk has been consumed
        for (int kt = tid; kt < FR_KC; kt += 256) {
            const int k = k0 + kt;
#pragma unroll
            for (int m = 0; m < 16; ++m)
                At[kt * FR_PITCH + m] = (m < M && k < kend) ? A[(size_t)m * lda + k] : 0.f;
        }
        __syncthreads();
        // This wave's quarter of the chunk, as far as it lies below kend.  The groups of 4 rows
        // start below kend <= K, so their record counts are exact (records_left must not be asked
        // about a start past the end of B: its difference would wrap to "everything in range");
        // rows of the last group that reach past K are outside those records and read as zero,
        // rows between kend and K meet zeros of A.
        const int kw = k0 + wave * (FR_KC / 4);
        const int kk_end = min(FR_KC / 4, kend - kw);
        // U groups of 4 rows of B against 4 k of A each: all the loads first, so that 4 U loads of
        // 16 bytes are in flight per lane before the first MFMA needs one
        auto groups = [&](int kk, auto u_count) {
            constexpr int U = decltype(u_count)::value;
            f32x4 b[U][4];
            float a[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const unsigned skip = (unsigned)(kw + kk + 4 * u) * (unsigned)ldb;
                const unsigned rec = records_left(b_elems, skip);
#pragma unroll
                for (int j = 0; j < 4; ++j) b[u][j] = stream_load_f32x4(B + n0 + (size_t)skip, b_off[j], rec);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) a[u] = At[(wave * (FR_KC / 4) + kk + 4 * u + lq) * FR_PITCH + li];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[4 * j + e] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u], b[u][j][e], acc[4 * j + e], 0, 0, 0);
        };
        int kk = 0;
        for (; kk + 16 <= kk_end; kk += 16) groups(kk, std::integral_constant<int, 4>{});
        for (; kk < kk_end; kk += 4) groups(kk, std::integral_constant<int, 1>{});
    }

    // register r of MFMA 4j+e holds C[4*lq + r][n0 + 64 j + 4 li + e].  Wave sums meet in LDS in
    // wave order: red[row][column].
    float* red = smem;
    for (int w = 0; w < 4; ++w) {
        __syncthreads();
        if (wave == w) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    f32x4* p = reinterpret_cast<f32x4*>(red + (4 * lq + r) * FR_COLS + 64 * j + 4 * li);
                    const f32x4 v = {acc[4 * j][r], acc[4 * j + 1][r], acc[4 * j + 2][r], acc[4 * j + 3][r]};
                    *p = w == 0 ? v : *p + v;
                }
        }
    }
    __syncthreads();
    const int n = n0 + tid;
    if (n >= N) return;
    float* dst = out + (size_t)blockIdx.y * out_slice_stride + n;
    const float bias = col_bias ? col_bias[n] : 0.f;
    for (int m = 0; m < M; ++m) {
        float v = red[m * FR_COLS + tid];
        if (accumulate) v += dst[(size_t)m * out_ld];
        if (col_bias) v += bias;
        dst[(size_t)m * out_ld] = v;
    }
}

int fewrows_slices(int N, int K, int cus)
{
    const int nblocks = (N + FR_COLS - 1) / FR_COLS;
    int want = (2 * cus + nblocks - 1) / nblocks;
    const int max_slices = (K + FR_KC - 1) / FR_KC;  // at least one chunk per slice
    if (want > max_slices) want = max_slices;
    return want < 1 ? 1 : want;
}

bool fewrows_applies(int M, int N, int K)
{
    // byte offsets inside a chunk (3 rows of B plus 256 columns) must stay below 2^31
    return M >= 1 && M <= 16 && N >= 512 && K >= 64 && (double)N * 4 * 4 < 2147483648.0;
}

// partial: [slices][M][N] floats when fewrows_slices(N, K, cus) > 1, else unused
hipError_t launch_sgemm_fewrows(const float* A, const float* B, float* C, float* partial, int M, int N,
                                int K, int lda, int ldb, int ldc, int accumulate, const float* col_bias,
                                int cus, hipStream_t stream)
{
    const int slices = fewrows_slices(N, K, cus);
    int k_per = (K + slices - 1) / slices;
    k_per = (k_per + FR_KC - 1) / FR_KC * FR_KC;
    const int used = (K + k_per - 1) / k_per;
    const dim3 grid((N + FR_COLS - 1) / FR_COLS, used), block(256);
    float* out = used > 1 ? partial : C;
    const int out_ld = used > 1 ? N : ldc;
    const size_t stride = used > 1 ? (size_t)M * N : 0;
    hipLaunchKernelGGL(sgemm_fewrows_kernel, grid, block, 0, stream, A, B, out, M, N, K, lda, ldb, k_per, out_ld,
                       stride, used > 1 ? 0 : accumulate, used > 1 ? nullptr : col_bias);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || used == 1) return e;
    return launch_splitk_reduce(partial, C, M, N, ldc, used, accumulate, stream, 0, col_bias);
}

}  // namespace cake
