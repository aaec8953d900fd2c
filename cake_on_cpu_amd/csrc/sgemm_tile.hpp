// sgemm_tile.hpp -- fp32 MFMA macro-tile GEMM kernel for gfx950 (CDNA4).
//
// This one kernel is what CAKE's pack_* -> schedule_{KMN,MKN,NKM} -> 6x16
// outer-product micro-kernel -> unpack_* pipeline becomes on the GPU
// (src/pack_ob.cpp:40-140, src/cake_sgemm_k_first.cpp:9-153,
// src/kernels/haswell/dense.cpp:8-204, src/pack_ob.cpp:393-411):
//
//   * packing          -> the global->LDS stage loaders (16-byte coalesced
//                         loads, LDS rows padded so the MFMA operand reads are
//                         bank-conflict free); nothing is written back to HBM
//   * K-first schedule -> the C macro-tile stays in accumulator registers over
//                         the whole K walk of the workgroup (C_p[core] of the
//                         reference is the register file here)
//   * M-/N-first and the CB block -> the order in which workgroup ids visit
//                         tiles (decode_tile): tiles that are resident together
//                         on one XCD form a compact block sharing A/B panels
//                         in that XCD's L2
//   * micro-kernel     -> v_mfma_f32_32x32x2_f32, WM/32 x WN/32 of them per wave
//   * unpack           -> masked stores straight from the accumulators
//
// Workgroup = (BM/WM)*(BN/WN) wavefronts of 64 lanes; each wave owns a WM x WN
// sub-tile.  LDS holds two stages (double buffer) of A[BM][BK+4] and
// B[BK][BN+8]; one barrier per K step.
#pragma once

#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace cake {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    static constexpr int THREADS = WAVES_M * WAVES_N * 64;
    static constexpr int TM = WM / 32, TN = WN / 32;   // 32x32 MFMA tiles per wave
    static constexpr int LDA = BK + 4;                 // floats; 16-byte reads of 8 consecutive rows hit 8 distinct bank quads
    static constexpr int LDB = BN + 8;                 // floats; rows k and k+4 land 32 banks apart
    static constexpr int A_STAGE = BM * LDA;
    static constexpr int B_STAGE = BK * LDB;
    static constexpr int LDS_BYTES = 2 * (A_STAGE + B_STAGE) * 4;
    static constexpr int A_CHUNKS = BM * BK / 4;       // 16-byte chunks per stage
    static constexpr int B_CHUNKS = BK * BN / 4;
    static constexpr int A_ITERS = A_CHUNKS / THREADS;
    static constexpr int B_ITERS = B_CHUNKS / THREADS;
    static_assert(BM % WM == 0 && BN % WN == 0 && WM % 32 == 0 && WN % 32 == 0, "wave tiling");
    static_assert(BK % 8 == 0, "K step is consumed 8 deep");
    static_assert(A_CHUNKS % THREADS == 0 && B_CHUNKS % THREADS == 0, "stage loaders");
};

// Workgroup id -> (tile_m, tile_n, k-slice).
//
// Hardware deals consecutive workgroup ids round-robin to the 8 XCDs, each
// with its own L2.  Undo that first, so that each XCD works through one
// contiguous run of the tile sequence; then walk the sequence in bands of
// `group` tile rows (or columns), fastest along the band's short side, so that
// the ~32 tiles an XCD holds at any moment cover a compact block of C and share
// their A and B panels in L2.  group = tiles_m with group_along_n = 0 is a pure
// M-first walk, group = tiles_n with group_along_n = 1 a pure N-first walk.
__device__ __forceinline__ void decode_tile(const GemmArgs& g, int wg, int& tile_m, int& tile_n,
                                            int& split)
{
    const int tiles = g.tiles_m * g.tiles_n;
    const int total = tiles * g.split_k;
    const int q = total >> 3, r = total & 7;
    const int xcd = wg & 7, idx = wg >> 3;
    int lid = (xcd < r) ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
    split = lid / tiles;
    int t = lid - split * tiles;
    const int slow_n = g.group_along_n ? g.tiles_n : g.tiles_m;  // extent of the grouped dimension
    const int fast_n = g.group_along_n ? g.tiles_m : g.tiles_n;
    const int band_sz = g.group * fast_n;
    const int band = t / band_sz;
    const int rem = t - band * band_sz;
    const int first = band * g.group;
    const int gsz = min(g.group, slow_n - first);
    const int fast = rem / gsz;
    const int slow = first + (rem - fast * gsz);
    tile_m = g.group_along_n ? fast : slow;
    tile_n = g.group_along_n ? slow : fast;
}

// ---------------------------------------------------------------------------
// Stage loaders: global memory -> registers.  Chunk c of a stage is 4
// consecutive k (A) or 4 consecutive n (B).
// ---------------------------------------------------------------------------
template <class T, int MODE>
__device__ __forceinline__ void load_a_stage(const GemmArgs& g, int m0, int k0, int kend, int tid,
                                             f32x4 (&ra)[T::A_ITERS])
{
    constexpr int CPR = T::BK / 4;  // chunks per tile row
#pragma unroll
    for (int it = 0; it < T::A_ITERS; ++it) {
        const int c = tid + it * T::THREADS;
        const int row = m0 + c / CPR;
        const int col = k0 + (c % CPR) * 4;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (MODE == LOAD_VEC4) {
            if (row < g.M && col < kend)
                v = *reinterpret_cast<const f32x4*>(g.A + (size_t)row * g.lda + col);
        } else if (MODE == LOAD_SCALAR) {
            if (row < g.M) {
                const float* src = g.A + (size_t)row * g.lda + col;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < kend) v[e] = src[e];
            }
        } else {
            if (row < g.M) {
                const int4 R = g.a_tab.row[row];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < kend) {
                        const int4 Cc = g.a_tab.col[col + e];
                        v[e] = g.A[(size_t)(R.x + Cc.x + R.y * Cc.y + R.z * Cc.z + R.w * Cc.w)];
                    }
            }
        }
        ra[it] = v;
    }
}

template <class T, int MODE>
__device__ __forceinline__ void load_b_stage(const GemmArgs& g, int n0, int k0, int kend, int tid,
                                             f32x4 (&rb)[T::B_ITERS])
{
    constexpr int CPR = T::BN / 4;
#pragma unroll
    for (int it = 0; it < T::B_ITERS; ++it) {
        const int c = tid + it * T::THREADS;
        const int row = k0 + c / CPR;
        const int col = n0 + (c % CPR) * 4;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (MODE == LOAD_VEC4) {
            if (row < kend && col < g.N)
                v = *reinterpret_cast<const f32x4*>(g.B + (size_t)row * g.ldb + col);
        } else if (MODE == LOAD_SCALAR) {
            if (row < kend) {
                const float* src = g.B + (size_t)row * g.ldb + col;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < g.N) v[e] = src[e];
            }
        } else {
            if (row < kend) {
                const int4 R = g.b_tab.row[row];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < g.N) {
                        const int4 Cc = g.b_tab.col[col + e];
                        v[e] = g.B[(size_t)(R.x + Cc.x + R.y * Cc.y + R.z * Cc.z + R.w * Cc.w)];
                    }
            }
        }
        rb[it] = v;
    }
}

// registers -> LDS stage
template <class T>
__device__ __forceinline__ void store_stage(float* As, float* Bs, int tid,
                                            const f32x4 (&ra)[T::A_ITERS],
                                            const f32x4 (&rb)[T::B_ITERS])
{
#pragma unroll
    for (int it = 0; it < T::A_ITERS; ++it) {
        const int c = tid + it * T::THREADS;
        *reinterpret_cast<f32x4*>(As + (c / (T::BK / 4)) * T::LDA + (c % (T::BK / 4)) * 4) = ra[it];
    }
#pragma unroll
    for (int it = 0; it < T::B_ITERS; ++it) {
        const int c = tid + it * T::THREADS;
        *reinterpret_cast<f32x4*>(Bs + (c / (T::BN / 4)) * T::LDB + (c % (T::BN / 4)) * 4) = rb[it];
    }
}

// One LDS stage of MFMA work for a wave.
//
// v_mfma_f32_32x32x2_f32 takes A[i][kk] from lane i + 32*kk and B[kk][j] from
// lane j + 32*kk.  The sum over k does not care which two k meet in one
// instruction as long as A and B agree, so within a group of 8 k the lower 32
// lanes take k = 0..3 and the upper 32 lanes k = 4..7: each lane then fetches
// its four A values with a single 16-byte LDS read.
template <class T>
__device__ __forceinline__ void mma_stage(const float* As, const float* Bs, int a_row, int b_col,
                                          int lh, f32x16 (&acc)[T::TM][T::TN])
{
#pragma unroll
    for (int kg = 0; kg < T::BK / 8; ++kg) {
        f32x4 a[T::TM];
        float b[T::TN][4];
        const int kk = kg * 8 + lh * 4;
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
            a[tm] = *reinterpret_cast<const f32x4*>(As + (a_row + tm * 32) * T::LDA + kk);
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int i = 0; i < 4; ++i) b[tn][i] = Bs[(kk + i) * T::LDB + b_col + tn * 32];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < T::TN; ++tn)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm][i], b[tn][i], acc[tm][tn], 0, 0, 0);
    }
}

template <class T, int A_MODE, int B_MODE>
__global__ void __launch_bounds__(T::THREADS) sgemm_tile_kernel(const GemmArgs g)
{
    extern __shared__ __align__(16) float smem[];
    float* As = smem;
    float* Bs = smem + 2 * T::A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = (wave / T::WAVES_N) * T::WM;
    const int wn0 = (wave % T::WAVES_N) * T::WN;

    int tile_m, tile_n, split;
    decode_tile(g, blockIdx.x, tile_m, tile_n, split);
    const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int steps = (kend - kbeg + T::BK - 1) / T::BK;

    f32x16 acc[T::TM][T::TN];
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.f;

    f32x4 ra[T::A_ITERS], rb[T::B_ITERS];
    if (steps > 0) {
        load_a_stage<T, A_MODE>(g, m0, kbeg, kend, tid, ra);
        load_b_stage<T, B_MODE>(g, n0, kbeg, kend, tid, rb);
        store_stage<T>(As, Bs, tid, ra, rb);
    }
    __syncthreads();

    int cur = 0;
    for (int s = 0; s < steps; ++s) {
        const bool more = s + 1 < steps;
        if (more) {
            const int k0 = kbeg + (s + 1) * T::BK;
            load_a_stage<T, A_MODE>(g, m0, k0, kend, tid, ra);
            load_b_stage<T, B_MODE>(g, n0, k0, kend, tid, rb);
        }
        mma_stage<T>(As + cur * T::A_STAGE, Bs + cur * T::B_STAGE, wm0 + l32, wn0 + l32, lh, acc);
        if (more) store_stage<T>(As + (cur ^ 1) * T::A_STAGE, Bs + (cur ^ 1) * T::B_STAGE, tid, ra, rb);
        __syncthreads();
        cur ^= 1;
    }

    // Epilogue.  Accumulator register r of a 32x32 tile holds row
    // 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
    float* out = g.partial ? g.partial + (size_t)split * g.M * g.N : g.C;
    const int ldo = g.partial ? g.N : g.ldc;
    const bool add = (g.partial == nullptr) && g.accumulate;
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn) {
            const int col = n0 + wn0 + tn * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + tm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                if (row < g.M && col < g.N) {
                    float* dst = out + (size_t)row * ldo + col;
                    *dst = add ? *dst + acc[tm][tn][r] : acc[tm][tn][r];
                }
            }
        }
}

template <class T, int A_MODE, int B_MODE>
inline hipError_t launch_tile(const GemmArgs& args, int grid, hipStream_t stream)
{
    auto kern = sgemm_tile_kernel<T, A_MODE, B_MODE>;
    static bool attr_set = false;  // per instantiation
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::THREADS), T::LDS_BYTES, stream, args);
    return hipGetLastError();
}

using Tile256x256x32 = Tile<256, 256, 32, 128, 64>;
using Tile256x256x16 = Tile<256, 256, 16, 128, 128>;
using Tile256x128x32 = Tile<256, 128, 32, 64, 64>;
using Tile128x256x32 = Tile<128, 256, 32, 64, 64>;
using Tile128x128x32 = Tile<128, 128, 32, 64, 64>;
using Tile64x64x32 = Tile<64, 64, 32, 32, 32>;

}  // namespace cake
