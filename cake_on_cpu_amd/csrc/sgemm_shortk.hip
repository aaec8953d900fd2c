// Products with a short K (at most 64) and many tiles of C: the macro-tile kernel spends a
// workgroup per tile, and with two k steps per tile the load latency of every tile sits in front
// of its few MFMAs (measured 256 x 100352 x 64: 37 us for loads and arithmetic where the matrix
// work alone takes 21 us, plus 6 us of stores).  Here a workgroup stays and walks over tiles: the
// whole K of a tile is one stage of LDS, and the operands of the NEXT tile are already on their
// way into registers while the current tile is multiplied and written out (256 x 100352 x 64:
// 48 -> 40 us, 38 us with A's stage kept across tiles; 16384 x 16384 x 16: 308 -> 263 us).  Loaders, LDS layout, operand reads and the
// epilogue are the macro-tile kernel's.
// Measured and left out: the same with K up to 128 in one stage (71 KB of LDS, two workgroups per
// CU: 85 us against 73 us at 256 x 100352 x 128), K up to 128 as two unrolled stages of 64 with
// the second stage loaded while the first is multiplied (95 against 73 us at the same shape,
// 185 against 165 us at 8192 x 8192 x 128), and an epilogue that stores 4 bytes per lane
// straight from the accumulators instead of 16 through LDS (43 against 40 us).
#include "sgemm_tile.hpp"

namespace cake {

// 64 x 64 tiles of C, 4 waves of 32 x 32; BK is the longest K it takes
using TileShortK64 = Tile<64, 64, 64, 32, 32>;

template <class T>
static constexpr int shortk_lds_bytes() { return (T::A_STAGE + T::B_STAGE) * 4; }  // one stage

// PLAIN: C is overwritten and there is no bias, so the epilogue loads nothing and the next
// tile's operands stay in flight across it
// (Non-temporal stores for C were measured and left out: where rows of C are whole cache lines
// they gained 4-6 % on one device and lost 3 % on another, and where they are not -- a row pitch
// that is no multiple of 128 bytes -- they cost 35-45 %: 4096 x 4100 x 64 27 -> 39 us.)
template <class T, int B_MODE, bool PLAIN>
__global__ void __launch_bounds__(T::THREADS) sgemm_shortk_kernel(const GemmArgs g)
{
    static_assert(B_MODE == LOAD_VEC4, "row-major operands");
    using L = VecLoader<T>;
    static_assert(T::KSPLIT == 1, "one wave per block of C");
    static_assert(T::WAVES_M * T::WAVES_N * 32 * (T::WN + 4) <= T::B_STAGE, "the epilogue's staging blocks fit B's stage");
    extern __shared__ __align__(16) float smem[];
    float* As = smem;
    float* Bs = smem + T::A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = (wave / T::WAVES_N) * T::WM;
    const int wn0 = (wave % T::WAVES_N) * T::WN;
    const int a_lane = (wm0 + l32) * T::LDA;
    const int b_lane = wn0 + l32;

    const int groups = (g.K + 7) >> 3;        // operand groups of 8 k that hold anything
    // Hardware deals workgroup ids round-robin to the 8 XCDs.  Each XCD takes one contiguous
    // eighth of the tile sequence, and its workgroups walk through it side by side, so that the
    // tiles in flight on an XCD at any moment are neighbours and share their panels in its L2.
    const int tiles_all = g.tiles_m * g.tiles_n;
    const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;   // the grid is a multiple of 8
    const int first = xcd * (tiles_all >> 3) + min(xcd, tiles_all & 7);
    const int tiles = first + (tiles_all >> 3) + (xcd < (tiles_all & 7) ? 1 : 0);   // end of this XCD's run
    int t = first + (blockIdx.x >> 3);
    if (t >= tiles) return;                   // before any barrier: the whole workgroup leaves
    // tile number -> origin of the tile and, for a batch of products, the image's B and C
    GemmArgs gt = g, gt_next = g;
    auto place = [&](int tile, GemmArgs& ga, int& m0_, int& n0_) {
        int tile_m, tile_n;
        raster_tile(g, tile, tile_m, tile_n);
        if (g.tiles_n_per_image) {
            const int b = tile_n / g.tiles_n_per_image;
            tile_n -= b * g.tiles_n_per_image;
            ga.B = g.B + (size_t)b * g.b_batch_stride;
            ga.C = g.C + (size_t)b * g.c_batch_stride;
        }
        m0_ = tile_m * T::BM;
        n0_ = tile_n * T::BN;
    };
    int m0, n0;
    place(t, gt, m0, n0);

    L ld;
    f32x4 ra[T::A_ITERS], rb[T::B_ITERS];
    ld.init(gt, m0, n0, tid);
    ld.load_first_stage(g.K, ra, rb);
    // A's stage outlives a tile (the epilogue turns C around inside B's stage): a workgroup whose
    // next tile has the same rows of A -- every time when the walk's stride is a multiple of
    // tiles_m -- neither loads nor stores them again
    bool a_fresh = true;
    for (;;) {
        __syncthreads();   // every wave is done with the staging reads of the previous tile's epilogue
        if (a_fresh) {     // the same for every thread of the workgroup
            // an A chunk that straddles K is loaded whole: zero its tail (chunks past K read as zero)
#pragma unroll
            for (int it = 0; it < T::A_ITERS; ++it) ra[it] = a_chunk_below<T>(ra[it], it, tid, 0, g.K);
            store_stage_a<T>(As, tid, ra);
        }
        store_stage_b<T>(Bs, tid, rb);
        __syncthreads();

        // the next tile's operands start their way into the registers just emptied
        const int t_next = t + stride;
        const bool more = t_next < tiles;   // the same for every thread of the workgroup
        int m0_next = 0, n0_next = 0;
        if (more) {
            place(t_next, gt_next, m0_next, n0_next);
            ld.init(gt_next, m0_next, n0_next, tid);
            a_fresh = m0_next != m0;
            if (a_fresh) ld.load_first_stage(g.K, ra, rb);
            else ld.load_first_stage_b(g.K, ra, rb);
        }

        f32x16 acc[T::TM][T::TN];
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.f;
        Frag<T> frag[2];
        load_frag<T>(As, Bs, a_lane, b_lane, lh, 0, frag[0]);
#pragma unroll
        for (int kg = 0; kg < T::BK / 8; ++kg) {
            if (kg < groups) {   // uniform: K is the same for everyone
                if (kg + 1 < T::BK / 8) load_frag<T>(As, Bs, a_lane, b_lane, lh, kg + 1, frag[(kg + 1) & 1]);
                mma_frag<T>(frag[kg & 1], acc);
            }
        }
        store_c_tile<T, B_MODE, PLAIN>(gt, Bs, acc, m0, n0, 0, wave, wm0, wn0, lane, l32, lh);
        if (!more) break;
        t = t_next;
        m0 = m0_next;
        n0 = n0_next;
        gt.B = gt_next.B;
        gt.C = gt_next.C;
    }
}

template <class T, int B_MODE, bool PLAIN>
static hipError_t launch_shortk_as(const GemmArgs& args, int grid, hipStream_t stream)
{
    auto kern = sgemm_shortk_kernel<T, B_MODE, PLAIN>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       shortk_lds_bytes<T>());
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::THREADS), shortk_lds_bytes<T>(), stream, args);
    return hipGetLastError();
}

template <class T, int B_MODE>
static hipError_t launch_shortk(const GemmArgs& args, int grid, hipStream_t stream)
{
    return !args.accumulate && !args.col_bias ? launch_shortk_as<T, B_MODE, true>(args, grid, stream)
                                              : launch_shortk_as<T, B_MODE, false>(args, grid, stream);
}

// K at most 64, 16-byte-loadable row-major operands, no K slices, and at least a 64 x 64 tile per
// CU.  Measured against the macro-tile kernel's own choice at K = 16 to 64: 0.79-0.98 of its time
// from 1 to 16 tiles per CU (1024^2 x 64: 5.3 -> 4.7 us, 3000^2 x 48: 20.1 -> 15.9 us,
// 4096^2 x 64: 30.5 -> 26.5 us); with up to four tiles per CU every workgroup has one tile and
// the gain is the single LDS stage and the load-free epilogue.
// Tiles 128 wide (four waves of 32 x 64, three workgroups per CU) were measured against these on
// the same device from K = 16 to 64 and lost everywhere (16384^2 x 16: 260 against 231 us,
// 256 x 100352 x 64: 58 against 46 us): the width is a parameter of the launch, with one value.
int shortk_tile_n(int M, int N, int K, int cus, int batch)
{
    if (K < 1 || K > 64) return 0;
    const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64) * batch;
    if (tiles < (long)cus) return 0;
    return 64;
}

int shortk_band_rows(int tiles_m, int N)
{
    return tiles_m <= 16 ? tiles_m : N >= 12288 ? 4 : N >= 6144 ? 8 : 16;
}

// args: tiles_m, tiles_n, group, group_along_n set for 64 x tile_n tiles; split_k = 1, no tail tiles
hipError_t launch_sgemm_shortk(const GemmArgs& args, int tile_n, int cus, hipStream_t stream)
{
    const long tiles = (long)args.tiles_m * args.tiles_n;
    if (tiles <= 0) return hipSuccess;
    if (args.K > 64 || args.split_k != 1 || args.tail_tiles != 0 || args.partial) return hipErrorInvalidValue;
    int grid, lds;
    if (tile_n != 64) return hipErrorInvalidValue;
    shortk_launch_shape(tiles, tile_n, cus, &grid, &lds);
    return launch_shortk<TileShortK64, LOAD_VEC4>(args, grid, stream);
}

// Workgroups launched for `tiles` tiles of 64 x tile_n, and the LDS each of them takes
void shortk_launch_shape(long tiles, int tile_n, int cus, int* grid, int* lds_bytes)
{
    (void)tile_n;
    const long slots = (long)cus * 4;   // what the LDS of a CU holds: 35 KB per workgroup
    *grid = (int)(((tiles < slots ? tiles : slots) + 7) / 8 * 8);   // whole rows of 8 XCDs
    *lds_bytes = shortk_lds_bytes<TileShortK64>();
}

}  // namespace cake
