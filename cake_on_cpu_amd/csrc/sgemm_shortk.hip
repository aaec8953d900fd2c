// Three kernels for products with a short K (up to 160; up to 256 for a batch that shares A) and
// many tiles of C, in this order: K at most 64 with operands staged through registers (any
// epilogue); K at most 32, C overwritten, B loaded straight into LDS; K from 65 up, C overwritten,
// both operands loaded straight into LDS stage by stage.  What they share: a workgroup stays
// resident and walks over 64 x 64 tiles, with the next tile's (or stage's) operands on their way
// while the current one is multiplied.
//
// The first kernel.  With K at most 64 and many tiles of C the macro-tile kernel spends a
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

// The four pieces of a wave's 32 x 32 block (8 rows x 32 columns each, a lane holding 16 bytes of a
// row) stored into a tile whose rows of C are whole 16-byte chunks: through a buffer resource that
// starts at the tile's first element and ends with C, so rows past M are out of range by
// themselves, a lane past N gets an out-of-range offset, and the rest of a piece's address is a
// scalar -- no vector arithmetic per piece (every regular vector instruction costs the matrix
// pipe four cycles on this hardware: none is issued beside an MFMA).
// c_lane: bytes from a piece's first element to the lane's 16 bytes, (row in piece * ldc + column) * 4.
__device__ __forceinline__ void store_block_pieces(const GemmArgs& g, float* c, int m0, int n0, int wm0, int wn0, int rd_col, int c_lane,
                                                   const f32x4 (&v)[4])
{
    const __amdgpu_buffer_rsrc_t rc = __builtin_amdgcn_make_buffer_rsrc(
        c + (size_t)m0 * g.ldc + n0, 0, (int)records_left(clamp_elems((long long)(g.M - 1 - m0) * g.ldc + g.N - n0), 0u), 0x00020000);
    const int off = n0 + wn0 + rd_col < g.N ? c_lane : BUF_OOB;
#pragma unroll
    for (int P = 0; P < 4; ++P)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v[P]), rc, off, ((wm0 + 8 * P) * g.ldc + wn0) * 4, 0);
}
// whole 16-byte chunks per row of C, and offsets within a tile that fit 31 bits
__device__ __forceinline__ bool c_in_whole_chunks(const GemmArgs& g, int tile_rows)
{
    return (g.N & 3) == 0 && (long long)tile_rows * g.ldc * 4 < 2147483647ll;
}

// one stage of each operand and, behind them, 8 rows of staging per wave for the epilogue that overwrites C
template <class T>
static constexpr int shortk_lds_bytes() { return (T::A_STAGE + T::B_STAGE + T::WAVES_M * T::WAVES_N * 8 * (T::WN + 4)) * 4; }

// PLAIN: C is overwritten and there is no bias, so the epilogue loads nothing and the next
// tile's operands stay in flight across it
// (Non-temporal stores for C were measured and left out: where rows of C are whole cache lines
// they gained 4-6 % on one device and lost 3 % on another, and where they are not -- a row pitch
// that is no multiple of 128 bytes -- they cost 35-45 %: 4096 x 4100 x 64 27 -> 39 us.)
//
// What a workgroup does between two tiles is a chain that nothing of its own overlaps (the other
// workgroups of the CU fill the matrix pipe meanwhile), so the chain is kept short:
//   * a thread's chunk offsets do not depend on the tile: rows of A at and past M fall outside the
//     buffer's record count, which is set per tile; columns of B at and past N bring in values of
//     the next row, which only reach columns of the tile that are never stored; chunks at and past
//     K are out of range from the start.  Placing a tile is scalar work: three divisions by
//     invariants (multiplications with reciprocals from the host), two base addresses, two
//     record counts;
//   * the next tile's operands are waited for right after the tile's MFMAs and before its stores
//     are issued: loads and stores share one counter of outstanding operations, so a wait placed
//     after the stores would wait for their round trip to memory as well.
template <class T, int B_MODE, bool PLAIN>
__global__ void __launch_bounds__(T::THREADS) __attribute__((amdgpu_waves_per_eu(4))) sgemm_shortk_kernel(const GemmArgs g)
{
    static_assert(B_MODE == LOAD_VEC4, "row-major operands");
    static_assert(T::KSPLIT == 1, "one wave per block of C");
    static_assert(T::WAVES_M * T::WAVES_N * 32 * (T::WN + 4) <= T::B_STAGE, "the epilogue's staging blocks fit B's stage");
    extern __shared__ __align__(16) float smem[];
    float* As = smem;
    float* Bs = smem + T::A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar for the compiler too
    const int l32 = lane & 31, lh = lane >> 5;
    // (through readfirstlane: derived from the thread id, the compiler would take the wave's place in
    // the tile for a per-lane value and loop over every store whose scalar offset it enters)
    const int wm0 = __builtin_amdgcn_readfirstlane((wave / T::WAVES_N) * T::WM);
    const int wn0 = __builtin_amdgcn_readfirstlane((wave % T::WAVES_N) * T::WN);
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

    // per thread, for every tile: where its chunks lie relative to the tile's origin
    int a_off[T::A_ITERS], b_off[T::B_ITERS];
#pragma unroll
    for (int it = 0; it < T::A_ITERS; ++it) {
        const int c = tid + it * T::THREADS, k = (c % (T::BK / 4)) * 4;
        a_off[it] = k < g.K ? ((c / (T::BK / 4)) * g.lda + k) * 4 : BUF_OOB;
    }
#pragma unroll
    for (int it = 0; it < T::B_ITERS; ++it) {
        const int c = tid + it * T::THREADS, k = c / (T::BN / 4);
        b_off[it] = k < g.K ? (k * g.ldb + (c % (T::BN / 4)) * 4) * 4 : BUF_OOB;
    }
    const bool ragged_k = (g.K & 3) != 0;     // then an A chunk can straddle K and is masked when it is stored
    const bool c_whole_chunks = c_in_whole_chunks(g, T::BM);
    const int c_lane = (((tid & 63) >> 3) * g.ldc + (tid & 7) * 4) * 4;   // bytes from a piece's first element to the lane's 16 bytes

    // tile number -> origin of the tile, the operands' base addresses and record counts
    struct Place {
        int m0, n0;
        const float* a;
        const float* b;
        float* c;
        unsigned a_bytes, b_bytes;
    };
    auto place = [&](int tile) {
        // raster_tile with the grouped dimension along M, its divisions by invariants
        const int band_sz = g.group * g.tiles_n;
        const int band = (int)g.by_band.div((unsigned)tile), rem = tile - band * band_sz;
        const int row0 = band * g.group;
        const bool whole_band = g.tiles_m - row0 >= g.group;
        const int gsz = whole_band ? g.group : g.tiles_m - row0;
        int tile_n = (int)(whole_band ? g.by_group.div((unsigned)rem) : g.by_last_group.div((unsigned)rem));
        const int tile_m = row0 + rem - tile_n * gsz;
        Place p;
        p.b = g.B;
        p.c = g.C;
        if (g.tiles_n_per_image) {
            const int img = (int)g.by_image_tiles.div((unsigned)tile_n);
            tile_n -= img * g.tiles_n_per_image;
            p.b += (size_t)img * g.b_batch_stride;
            p.c += (size_t)img * g.c_batch_stride;
        }
        p.m0 = tile_m * T::BM;
        p.n0 = tile_n * T::BN;
        p.a = g.A + (size_t)p.m0 * g.lda;
        p.b += p.n0;
        p.a_bytes = records_left(clamp_elems((long long)(g.M - 1 - p.m0) * g.lda + g.K), 0u);
        p.b_bytes = records_left(clamp_elems((long long)(g.K - 1) * g.ldb + g.N - p.n0), 0u);
        return p;
    };
    f32x4 ra[T::A_ITERS], rb[T::B_ITERS];
    auto load_a = [&](const Place& p) {
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[it] = buffer_load_f32x4(p.a, a_off[it], p.a_bytes);
    };
    auto load_b = [&](const Place& p) {
#pragma unroll
        for (int it = 0; it < T::B_ITERS; ++it) rb[it] = buffer_load_f32x4(p.b, b_off[it], p.b_bytes);
    };

    Place cur = place(t);
    load_a(cur);
    load_b(cur);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): from here on the loop waits for loads where it says so
    GemmArgs gt = g;                      // what the epilogue that reads C sees: C and, for a batch, the image's part of it
    // A's stage outlives a tile (no epilogue touches it): a workgroup whose next tile has the same
    // rows of A -- every time when the walk's stride is a multiple of tiles_m -- neither loads nor
    // stores them again
    bool a_fresh = true;
    for (;;) {
        __syncthreads();   // every wave has read the previous tile's last operands (and is done with staging reads inside B's stage)
        if (a_fresh) {     // the same for every thread of the workgroup
            if (ragged_k) {
#pragma unroll
                for (int it = 0; it < T::A_ITERS; ++it) ra[it] = a_chunk_below<T>(ra[it], it, tid, 0, g.K);
            }
            store_stage_a<T>(As, tid, ra);
        }
        store_stage_b<T>(Bs, tid, rb);
        __syncthreads();

        // the next tile's operands start their way into the registers just emptied
        const int t_next = t + stride;
        const bool more = t_next < tiles;   // the same for every thread of the workgroup
        Place nxt = cur;
        if (more) {
            nxt = place(t_next);
            a_fresh = nxt.m0 != cur.m0;
            if (a_fresh) load_a(nxt);
            load_b(nxt);
        }

        // (the tile's first MFMA starts from a constant zero: nothing is cleared.  Every regular
        // vector instruction costs the matrix pipe four cycles on this hardware -- none is issued
        // beside an MFMA -- and a tile has only 32 MFMAs per wave to set against them.)
        f32x16 acc[T::TM][T::TN];
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        Frag<T> frag[2];
        load_frag<T>(As, Bs, a_lane, b_lane, lh, 0, frag[0]);
#pragma unroll
        for (int kg = 0; kg < T::BK / 8; ++kg) {
            if (kg < groups) {   // uniform: K is the same for everyone
                if (kg + 1 < T::BK / 8) load_frag<T>(As, Bs, a_lane, b_lane, lh, kg + 1, frag[(kg + 1) & 1]);
                if (kg == 0) {
#pragma unroll
                    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
                        for (int tn = 0; tn < T::TN; ++tn)
                            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag[0].a[tm][0], frag[0].b[tn][0], zero, 0, 0, 0);
#pragma unroll
                    for (int i = 1; i < 4; ++i)
#pragma unroll
                        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
                            for (int tn = 0; tn < T::TN; ++tn)
                                acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(frag[0].a[tm][i], frag[0].b[tn][i], acc[tm][tn], 0, 0, 0);
                } else {
                    mma_frag<T>(frag[kg & 1], acc);
                }
            }
        }
        if (PLAIN) {
            // the next tile's operands have had the tile's MFMAs to arrive; no store is outstanding
            // but the previous tile's, issued a whole tile ago
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (PLAIN) {
            // The wave turns its block around in pieces of 8 rows through a staging block of its own,
            // next to the operand stages: no barrier in front of the epilogue, so a wave that has
            // finished its MFMAs stores while the others of the workgroup are still multiplying.
            static_assert(T::TM == 1 && T::TN == 1 && T::WN == 32, "one 32 x 32 block of C per wave");
            constexpr int PITCH = T::WN + 4;
            float* stg = smem + T::A_STAGE + T::B_STAGE + wave * (8 * PITCH);
            const int rd_row = lane >> 3, rd_col = (lane & 7) * 4;
            // LDS serves a wave's requests in order: a piece's read sees its writes, and the next
            // piece's writes come after it.  All four pieces are therefore issued back to back and
            // the stores follow as the reads return.
            f32x4 v[4];
#pragma unroll
            for (int P = 0; P < 4; ++P) {
#pragma unroll
                for (int j = 0; j < 4; ++j) stg[(4 * lh + j) * PITCH + l32] = acc[0][0][4 * P + j];
                v[P] = *reinterpret_cast<const f32x4*>(stg + rd_row * PITCH + rd_col);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (c_whole_chunks) {
                store_block_pieces(g, cur.c, cur.m0, cur.n0, wm0, wn0, rd_col, c_lane, v);
            } else {
                const int row = cur.m0 + wm0 + rd_row, col = cur.n0 + wn0 + rd_col;
                float* dst = cur.c + (size_t)row * g.ldc + col;
                const int rows = g.M - row, valid = min(4, g.N - col);
#pragma unroll
                for (int P = 0; P < 4; ++P) {
                    if (8 * P < rows && valid > 0) {
                        float* d = dst + (size_t)(8 * P) * g.ldc;
                        if (valid == 4) {
                            *reinterpret_cast<f32x4_u*>(d) = v[P];
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                if (e < valid) d[e] = v[P][e];
                        }
                    }
                }
            }
        } else {
            gt.C = cur.c;
            store_c_tile<T, B_MODE, PLAIN>(gt, Bs, acc, cur.m0, cur.n0, 0, wave, wm0, wn0, lane, l32, lh);
        }
        if (!more) break;
        t = t_next;
        cur = nxt;
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

// C overwritten, no bias: the same walk with B loaded straight into LDS (buffer loads with the
// LDS bit: a wave's 64 lanes x 16 bytes land in 1 KB of consecutive LDS, lane by lane, so a lane
// asks for the chunk that belongs at its place: 4 rows of 64 columns per instruction, rows
// unpadded -- the 4-byte operand reads of a half-wave cover 32 consecutive floats of a row either
// way).  B has two buffers: while tile t is multiplied out of one, tile t + 1 arrives in the
// other, without passing through registers and without a store pass, and one barrier per tile is
// left (two when the rows of A change).  A's rows are unpadded as well, their 16-byte chunks
// swizzled (chunk c of row r sits at c ^ (r & 7)) so that the 16-byte operand reads of 8
// consecutive rows still hit 8 different bank groups.  With stages of 32 k that is 29 KB of LDS and
// 84 registers: five workgroups share a CU, and products with K up to 32 that overwrite C run
// here (against the kernel above, us: 256 x 100352 x 32 27.4 -> 25.6, 8192^2 x 32 56.7 -> 53.7,
// 4096 x 8192 x 25 30.1 -> 28.9, 1100 x 65536 x 32 63.6 -> 61.2; the same bits).  With stages of
// 64 k it is 53 KB and three workgroups per CU against four: measured level with the kernel
// above (256 x 100352 x 64: 39.5 against 39.3 us) and not instantiated.
template <int BK>
__device__ __forceinline__ void shortk_direct_body(const GemmArgs& g, float* As, float* B0, float* B1, float* Stg)
{
    using T = Tile<64, 64, BK, 32, 32>;
    constexpr int PITCH = T::WN + 4;
    constexpr int CPR = BK / 4;                      // 16-byte chunks per row of A
    constexpr int B_LOADS = BK * 64 / 4 / 256;       // load instructions per thread and stage

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar for the compiler too
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = __builtin_amdgcn_readfirstlane((wave / T::WAVES_N) * T::WM);   // (scalars: see sgemm_shortk_kernel)
    const int wn0 = __builtin_amdgcn_readfirstlane((wave % T::WAVES_N) * T::WN);
    const int a_row = (wm0 + l32) * BK, a_swz = l32 & 7;
    const int b_lane = wn0 + l32;
    float* stg = Stg + wave * (8 * PITCH);
    const bool c_whole_chunks = c_in_whole_chunks(g, 64);
    const int c_lane = ((lane >> 3) * g.ldc + (lane & 7) * 4) * 4;

    const int groups = (g.K + 7) >> 3;
    const int tiles_all = g.tiles_m * g.tiles_n;
    const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;
    const int first = xcd * (tiles_all >> 3) + min(xcd, tiles_all & 7);
    const int tiles = first + (tiles_all >> 3) + (xcd < (tiles_all & 7) ? 1 : 0);
    int t = first + (blockIdx.x >> 3);
    if (t >= tiles) return;

    int a_off[T::A_ITERS], a_lds[T::A_ITERS], b_off[B_LOADS];
#pragma unroll
    for (int it = 0; it < T::A_ITERS; ++it) {
        const int c = tid + it * T::THREADS, r = c / CPR, cc = c % CPR;
        a_off[it] = cc * 4 < g.K ? (r * g.lda + cc * 4) * 4 : BUF_OOB;
        a_lds[it] = r * BK + ((cc ^ (r & 7)) * 4);
    }
    // load instruction q = wave + 4 it of a stage fills rows 4 q .. 4 q + 3 of B's buffer
#pragma unroll
    for (int it = 0; it < B_LOADS; ++it) {
        const int k = 4 * (wave + 4 * it) + (lane >> 4);
        b_off[it] = k < g.K ? (k * g.ldb + (lane & 15) * 4) * 4 : BUF_OOB;
    }
    const bool ragged_k = (g.K & 3) != 0;
    // rows at and past K of both buffers are never loaded: zero once (a value left there would
    // meet a zero of A, but zero times a stray NaN is not zero)
    for (int i = tid; i < BK * 64 / 4; i += T::THREADS) {
        reinterpret_cast<f32x4*>(B0)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        reinterpret_cast<f32x4*>(B1)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    __syncthreads();

    struct Place {
        int m0, n0;
        const float* a;
        const float* b;
        float* c;
        unsigned a_bytes, b_bytes;
    };
    auto place = [&](int tile) {
        const int band_sz = g.group * g.tiles_n;
        const int band = (int)g.by_band.div((unsigned)tile), rem = tile - band * band_sz;
        const int row0 = band * g.group;
        const bool whole_band = g.tiles_m - row0 >= g.group;
        const int gsz = whole_band ? g.group : g.tiles_m - row0;
        int tile_n = (int)(whole_band ? g.by_group.div((unsigned)rem) : g.by_last_group.div((unsigned)rem));
        const int tile_m = row0 + rem - tile_n * gsz;
        Place p;
        p.b = g.B;
        p.c = g.C;
        if (g.tiles_n_per_image) {
            const int img = (int)g.by_image_tiles.div((unsigned)tile_n);
            tile_n -= img * g.tiles_n_per_image;
            p.b += (size_t)img * g.b_batch_stride;
            p.c += (size_t)img * g.c_batch_stride;
        }
        p.m0 = tile_m * T::BM;
        p.n0 = tile_n * T::BN;
        p.a = g.A + (size_t)p.m0 * g.lda;
        p.b += p.n0;
        p.a_bytes = records_left(clamp_elems((long long)(g.M - 1 - p.m0) * g.lda + g.K), 0u);
        p.b_bytes = records_left(clamp_elems((long long)(g.K - 1) * g.ldb + g.N - p.n0), 0u);
        return p;
    };
    f32x4 ra[T::A_ITERS];
    auto load_a = [&](const Place& p) {
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[it] = buffer_load_f32x4(p.a, a_off[it], p.a_bytes);
    };
    auto issue_b = [&](float* Bdst, const Place& p) {
        __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.b), 0, (int)p.b_bytes, 0x00020000);
#pragma unroll
        for (int it = 0; it < B_LOADS; ++it)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(Bdst + (wave + 4 * it) * 256),
                                                     16, b_off[it], 0, 0, 0);
    };

    Place cur = place(t), nxt = cur;
    load_a(cur);
    issue_b(B0, cur);
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
    bool a_fresh = true, more = true;

    auto step = [&](const float* Bc, float* Bn) {
        if (a_fresh) {
            __syncthreads();   // every wave has read its last operands of A's previous rows
#pragma unroll
            for (int it = 0; it < T::A_ITERS; ++it) {
                f32x4 v = ra[it];
                if (ragged_k) v = a_chunk_below<T>(v, it, tid, 0, g.K);   // a chunk that straddles K was loaded whole
                *reinterpret_cast<f32x4*>(As + a_lds[it]) = v;
            }
        }
        // every wave's share of this tile's B has landed (each waited for its own loads), A is
        // stored, and nobody reads the other buffer any more
        __syncthreads();
        const int t_next = t + stride;
        more = t_next < tiles;
        if (more) {
            nxt = place(t_next);
            a_fresh = nxt.m0 != cur.m0;
            if (a_fresh) load_a(nxt);
            issue_b(Bn, nxt);
        }
        f32x16 acc;   // (the tile's first MFMA starts from a constant zero: nothing is cleared)
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        f32x4 fa[2];
        float fb[2][4];
        auto fetch = [&](int kg, f32x4& a, float (&b)[4]) {
            a = *reinterpret_cast<const f32x4*>(As + a_row + (((kg * 2 + lh) ^ a_swz) * 4));
            const int kk = kg * 8 + lh * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = Bc[(kk + i) * 64 + b_lane];
        };
        fetch(0, fa[0], fb[0]);
#pragma unroll
        for (int kg = 0; kg < BK / 8; ++kg) {
            if (kg < groups) {
                if (kg + 1 < BK / 8) fetch(kg + 1, fa[(kg + 1) & 1], fb[(kg + 1) & 1]);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[kg & 1][i], fb[kg & 1][i], kg == 0 && i == 0 ? zero : acc, 0, 0, 0);
            }
        }
        // the next tile's operands have had the tile's MFMAs to arrive; no store is outstanding
        // but the previous tile's
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        __builtin_amdgcn_sched_barrier(0);
        // the wave's block, turned around in pieces of 8 rows through its own staging block
        const int rd_row = lane >> 3, rd_col = (lane & 7) * 4;
        f32x4 v[4];
#pragma unroll
        for (int P = 0; P < 4; ++P) {
#pragma unroll
            for (int j = 0; j < 4; ++j) stg[(4 * lh + j) * PITCH + l32] = acc[4 * P + j];
            v[P] = *reinterpret_cast<const f32x4*>(stg + rd_row * PITCH + rd_col);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (c_whole_chunks) {
            store_block_pieces(g, cur.c, cur.m0, cur.n0, wm0, wn0, rd_col, c_lane, v);
            return;
        }
        const int row = cur.m0 + wm0 + rd_row, col = cur.n0 + wn0 + rd_col;
        float* dst = cur.c + (size_t)row * g.ldc + col;
        const int rows = g.M - row, valid = min(4, g.N - col);
#pragma unroll
        for (int P = 0; P < 4; ++P) {
            if (8 * P < rows && valid > 0) {
                float* d = dst + (size_t)(8 * P) * g.ldc;
                if (valid == 4) {
                    *reinterpret_cast<f32x4_u*>(d) = v[P];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (e < valid) d[e] = v[P][e];
                }
            }
        }
    };
    for (;;) {
        step(B0, B1);
        if (!more) break;
        t += stride;
        cur = nxt;
        step(B1, B0);
        if (!more) break;
        t += stride;
        cur = nxt;
    }
}

// (the LDS arrays are separate objects on purpose: the compiler then knows that reads of one B
// buffer need not wait for loads into the other)
#define SHORTK_DIRECT_KERNEL(BK)                                                                    \
    __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5))) sgemm_shortk_direct_kernel_##BK(const GemmArgs g)        \
    {                                                                                               \
        __shared__ __align__(16) float As[64 * BK];                                                 \
        __shared__ __align__(16) float B0[BK * 64];                                                 \
        __shared__ __align__(16) float B1[BK * 64];                                                 \
        __shared__ __align__(16) float Stg[4 * 8 * 36];                                             \
        shortk_direct_body<BK>(g, As, B0, B1, Stg);                                                 \
    }
SHORTK_DIRECT_KERNEL(32)
#undef SHORTK_DIRECT_KERNEL

// K from 65 to 160 (a multiple of 4), C overwritten, no bias: the walk over tiles continued into K.
// A workgroup's work is a sequence of units -- (tile, stage of 32 k) -- and BOTH operands of a unit
// go straight into LDS (A's rows swizzled as above, by the choice of which chunk a lane asks for);
// each operand has two buffers, the loads of unit u + 1 are issued when unit u starts, across tile
// borders, so a tile has no prologue of its own; one barrier per unit; the epilogue as above.
// 37 KB of LDS and 76 registers: four workgroups per CU.  Nothing passes through registers, and
// lanes past the operands' ends write zeros into LDS (the hardware does that for out-of-range
// lanes of such loads).  K must be a multiple of 4: a chunk of A that straddled K would bring in
// the next row's values where B holds zeros, and zero times a stray NaN is not zero.
// Measured against the macro-tile kernel's choice for the same product (us): 1000 x 30000 x 128
// 81.6 -> 72.1, 4096^2 x 128 46.8 -> 42.9, 8192^2 x 96 139 -> 129, 3000^2 x 100 27.4 -> 22.4,
// 2000 x 20000 x 80 87.9 -> 70.2, 8192 x 2048 x 132 51.9 -> 44.1, 2048 x 8192 x 144 52.1 -> 46.4,
// 4096^2 x 160 51.6 -> 49.5, 1024^2 x 128 6.7 -> 5.6; level at K = 192 (1024 x 16384: 57.7 / 57.2)
// and behind at 256 (4096^2: 72.0 / 73.5), and behind the kernel at the top of this file at K = 64
// (256 x 100352: 38.6 / 40.2).  With three buffers per operand and the loads two units ahead
// (54 KB, three workgroups per CU) it was 2-8 % slower on all of them, and with the unit's barrier
// moved in front of its last group of MFMAs (operands in registers, the next unit's first operands
// read behind them) 0-8 % slower.
// A batch of products with one A (a 1 x 1 convolution on the input as it lies) runs here up to
// 256 channels: against the gather inside the macro-tile kernel, batch 32, us: 128 -> 512 on 28 x 28
// 41.9 -> 37.3, 128 -> 256 on 56 x 56 74.1 -> 65.6, 80 -> 480 on 56 x 56 105 -> 84, 128 -> 128 on
// 28 x 28 16.2 -> 13.9, 256 -> 128 on 56 x 56 63.3 -> 59.4, 256 -> 512 on 28 x 28 62.6 -> 59.8,
// 128 -> 512 on 14 x 14 (196 pixels in four tiles of 64: a quarter of the columns is padding)
// 15.7 -> 13.5, but 256 -> 1024 on 14 x 14 39.0 -> 41.7: with that much padding the gather stays
// from 161 channels on.
// That padding goes away when the column tiles run across image borders (FLAT: the columns of all
// images form one sequence, a lane's offset into B is recomputed per tile -- one division by the
// plane size as a multiplication -- and a 16-byte chunk never spans two images because the plane
// size is a multiple of 4): 256 -> 1024 on 14 x 14 is 1568 tiles instead of 2048, 38.5 -> 36.2 us
// against the gather; 128 -> 512 on 14 x 14 16.7 -> 14.3, 192 -> 384 16.1 -> 14.4, 128 -> 512 on 28 x 28
// 38.3 -> 33.8, 96 -> 256 on 28 x 28 19.5 -> 17.1, 128 -> 256 on 20 x 20 15.5 -> 13.3, batch 128
// 256 -> 512 on 10 x 10 35.5 -> 34.0.  (The divisor of that division must stay in scalar
// registers: a record count computed with an integer division of the arguments lands in a vector
// register and the compiler then loops over every load.)
template <int NSTAGE, bool FLAT>
__device__ __forceinline__ void shortk_staged_body(const GemmArgs& g, float* const (&Ab)[NSTAGE], float* const (&Bb)[NSTAGE],
                                                   float* Stg)
{
    constexpr int BK = 32, PITCH = 36, PF = NSTAGE - 1;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar for the compiler too
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = __builtin_amdgcn_readfirstlane((wave >> 1) * 32), wn0 = __builtin_amdgcn_readfirstlane((wave & 1) * 32);   // (scalars: see sgemm_shortk_kernel)
    const int a_row = (wm0 + l32) * BK, a_swz = l32 & 7;
    const int b_lane = wn0 + l32;
    float* stg = Stg + wave * (8 * PITCH);
    const bool c_whole_chunks = !FLAT && c_in_whole_chunks(g, 64);   // (across image borders a lane's place in C is not the tile's plus a constant)
    const int c_lane = ((lane >> 3) * g.ldc + (lane & 7) * 4) * 4;

    const int stages = (g.K + BK - 1) / BK;
    const int tiles_all = g.tiles_m * g.tiles_n;
    const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;
    const int first = xcd * (tiles_all >> 3) + min(xcd, tiles_all & 7);
    const int tiles = first + (tiles_all >> 3) + (xcd < (tiles_all & 7) ? 1 : 0);
    const int t0 = first + (blockIdx.x >> 3);
    if (t0 >= tiles) return;

    // load instruction q = wave + 4 it fills rows 8 q .. 8 q + 7 of A's buffer (8 chunks of 16 bytes
    // per row, chunk c of row r at place c ^ (r & 7)) and rows 4 q .. 4 q + 3 of B's
    int a_off[2], a_off_last[2], b_off[2];
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int q = wave + 4 * it;
        const int r = 8 * q + (lane >> 3), c = (lane & 7) ^ (r & 7);
        a_off[it] = (r * g.lda + c * 4) * 4;
        a_off_last[it] = (stages - 1) * BK + c * 4 < g.K ? a_off[it] : BUF_OOB;
        b_off[it] = ((4 * q + (lane >> 4)) * g.ldb + (lane & 15) * 4) * 4;
    }
    // A batch whose column tiles run across image borders: B's base stays the first image, the
    // lane's offset moves with the tile (b_flat, below), and rows at and past K -- which the record
    // count cannot cut off there, the next image follows -- are cut off per lane.
    constexpr bool flat = FLAT;   // g.batch_cols != 0
    const bool b_row_past_k[2] = {(stages - 1) * BK + 4 * wave + (lane >> 4) >= g.K,
                                  (stages - 1) * BK + 4 * (wave + 4) + (lane >> 4) >= g.K};

    // byte offset of the lane's first chunk of B in a tile that starts at column n0 of the whole batch
    // (columns at and past N belong to images past the last one: out of range)
    auto flat_offset = [&](int n0) {
        const unsigned n = (unsigned)n0 + (lane & 15) * 4;
        const unsigned img = g.by_batch_cols.div(n);
        return (int)((img * (unsigned)g.b_batch_stride + (n - img * (unsigned)g.batch_cols) +
                      (unsigned)(4 * wave + (lane >> 4)) * (unsigned)g.ldb) * 4u);
    };
    struct Place {
        int m0, n0;
        const float* a;
        const float* b;
        float* c;
        unsigned a_elems, b_elems;
        int b_flat;   // per lane: flat_offset(n0)
    };
    auto place = [&](int tile) {
        const int band_sz = g.group * g.tiles_n;
        const int band = (int)g.by_band.div((unsigned)tile), rem = tile - band * band_sz;
        const int row0 = band * g.group;
        const bool whole_band = g.tiles_m - row0 >= g.group;
        const int gsz = whole_band ? g.group : g.tiles_m - row0;
        int tile_n = (int)(whole_band ? g.by_group.div((unsigned)rem) : g.by_last_group.div((unsigned)rem));
        const int tile_m = row0 + rem - tile_n * gsz;
        Place p;
        p.b = g.B;
        p.c = g.C;
        if (g.tiles_n_per_image) {   // a batch of products with one A: the image's B and C
            const int img = (int)g.by_image_tiles.div((unsigned)tile_n);
            tile_n -= img * g.tiles_n_per_image;
            p.b += (size_t)img * g.b_batch_stride;
            p.c += (size_t)img * g.c_batch_stride;
        }
        p.m0 = tile_m * 64;
        p.n0 = tile_n * 64;
        p.a = g.A + (size_t)p.m0 * g.lda;
        p.a_elems = clamp_elems((long long)(g.M - 1 - p.m0) * g.lda + g.K);
        p.b_flat = 0;
        if (flat) {
            p.b_elems = (unsigned)g.b_batch_stride * g.by_batch_cols.div((unsigned)g.N);   // all images: below 2^29 elements
            p.b_flat = flat_offset(p.n0);
        } else {
            p.b += p.n0;
            p.b_elems = clamp_elems((long long)(g.K - 1) * g.ldb + g.N - p.n0);
        }
        return p;
    };
    auto issue = [&](float* Ad, float* Bd, const Place& p, int ks) {
        const unsigned ka = (unsigned)ks * BK, kb = (unsigned)ks * BK * (unsigned)g.ldb;
        __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.a + ka), 0,
                                                                      (int)records_left(p.a_elems, ka), 0x00020000);
        __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.b + kb), 0,
                                                                      (int)records_left(p.b_elems, kb), 0x00020000);
        const bool last = ks == stages - 1;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (__attribute__((address_space(3))) void*)(Ad + (wave + 4 * it) * 256), 16,
                                                     last ? a_off_last[it] : a_off[it], 0, 0, 0);
            const int bo = !flat ? b_off[it] : last && b_row_past_k[it] ? BUF_OOB : p.b_flat + it * (16 * 4) * g.ldb;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)(Bd + (wave + 4 * it) * 256), 16,
                                                     bo, 0, 0, 0);
        }
    };

    // consumer and producer positions in the unit sequence
    int t = t0, ks = 0, tp = t0, kp = 0;
    Place cur = place(t0), pp = cur;
    bool producing = true;
    auto produce = [&](float* Ad, float* Bd) {
        if (!producing) return;
        issue(Ad, Bd, pp, kp);
        if (++kp == stages) {
            kp = 0;
            tp += stride;
            producing = tp < tiles;
            if (producing) pp = place(tp);
        }
    };
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;

    // returns false after the workgroup's last unit
    auto unit = [&](const float* Ac, const float* Bc, float* Ad, float* Bd) -> bool {
        // this unit's loads have landed: at most the PF - 1 younger units' loads (4 instructions each) are outstanding
        if (producing) {
            if constexpr (PF == 1) __builtin_amdgcn_s_waitcnt(0x0F70);
            else __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
        } else {
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        __syncthreads();   // everybody's share has landed, and nobody reads the buffer that is filled next
        produce(Ad, Bd);
        const int groups = min(4, (g.K - ks * BK + 7) >> 3);
        f32x4 fa[2];
        float fb[2][4];
        auto fetch = [&](int kg, f32x4& a, float (&b)[4]) {
            a = *reinterpret_cast<const f32x4*>(Ac + a_row + (((kg * 2 + lh) ^ a_swz) * 4));
            const int kk = kg * 8 + lh * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) b[i] = Bc[(kk + i) * 64 + b_lane];
        };
        fetch(0, fa[0], fb[0]);
#pragma unroll
        for (int kg = 0; kg < 4; ++kg) {
            if (kg < groups) {
                if (kg + 1 < 4) fetch(kg + 1, fa[(kg + 1) & 1], fb[(kg + 1) & 1]);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[kg & 1][i], fb[kg & 1][i], acc, 0, 0, 0);
            }
        }
        if (++ks < stages) return true;
        // the tile is finished: the wave's block, turned around in pieces of 8 rows through its own staging block
        const int rd_row = lane >> 3, rd_col = (lane & 7) * 4;
        f32x4 v[4];
#pragma unroll
        for (int P = 0; P < 4; ++P) {
#pragma unroll
            for (int j = 0; j < 4; ++j) stg[(4 * lh + j) * PITCH + l32] = acc[4 * P + j];
            v[P] = *reinterpret_cast<const f32x4*>(stg + rd_row * PITCH + rd_col);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (c_whole_chunks) {
            store_block_pieces(g, cur.c, cur.m0, cur.n0, wm0, wn0, rd_col, c_lane, v);
        } else {
            const int row = cur.m0 + wm0 + rd_row, col = cur.n0 + wn0 + rd_col;
            float* dst = cur.c + (size_t)row * g.ldc + col;
            if (flat) {   // the chunk's image and pixel (a chunk never spans two images: batch_cols is a multiple of 4)
                const unsigned img = g.by_batch_cols.div((unsigned)col);
                dst = cur.c + (size_t)img * g.c_batch_stride + (size_t)row * g.ldc + ((unsigned)col - img * (unsigned)g.batch_cols);
            }
            const int rows = g.M - row, valid = min(4, g.N - col);
#pragma unroll
            for (int P = 0; P < 4; ++P) {
                if (8 * P < rows && valid > 0) {
                    float* d = dst + (size_t)(8 * P) * g.ldc;
                    if (valid == 4) {
                        *reinterpret_cast<f32x4_u*>(d) = v[P];
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (e < valid) d[e] = v[P][e];
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        ks = 0;
        t += stride;
        if (t >= tiles) return false;
        cur = place(t);
        return true;
    };

    // the first PF units' loads
#pragma unroll
    for (int i = 0; i < PF; ++i) produce(Ab[i], Bb[i]);
    for (;;) {
        if constexpr (NSTAGE == 2) {
            if (!unit(Ab[0], Bb[0], Ab[1], Bb[1])) break;
            if (!unit(Ab[1], Bb[1], Ab[0], Bb[0])) break;
        } else {
            if (!unit(Ab[0], Bb[0], Ab[2], Bb[2])) break;
            if (!unit(Ab[1], Bb[1], Ab[0], Bb[0])) break;
            if (!unit(Ab[2], Bb[2], Ab[1], Bb[1])) break;
        }
    }
}

// (kernels by macro, not by template: with __shared__ arrays inside a kernel template the host
// side of the launch did not link)
#define SHORTK_STAGED_KERNEL(NAME, FLAT)                                                            \
    __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) NAME(const GemmArgs g)                                   \
    {                                                                                               \
        __shared__ __align__(16) float A0[2048];                                                    \
        __shared__ __align__(16) float A1[2048];                                                    \
        __shared__ __align__(16) float B0[2048];                                                    \
        __shared__ __align__(16) float B1[2048];                                                    \
        __shared__ __align__(16) float Stg[4 * 8 * 36];                                             \
        float* const Ab[2] = {A0, A1};                                                              \
        float* const Bb[2] = {B0, B1};                                                              \
        shortk_staged_body<2, FLAT>(g, Ab, Bb, Stg);                                                \
    }
SHORTK_STAGED_KERNEL(sgemm_shortk_staged_kernel, false)
SHORTK_STAGED_KERNEL(sgemm_shortk_staged_flat_kernel, true)   // a batch whose column tiles run across image borders

// K at most 64, 16-byte-loadable row-major operands, no K slices, and at least a 64 x 64 tile per
// CU.  Measured against the macro-tile kernel's own choice at K = 16 to 64: 0.79-0.98 of its time
// from 1 to 16 tiles per CU (1024^2 x 64: 5.3 -> 4.7 us, 3000^2 x 48: 20.1 -> 15.9 us,
// 4096^2 x 64: 30.5 -> 26.5 us); with up to four tiles per CU every workgroup has one tile and
// the gain is the single LDS stage and the load-free epilogue.
// Tiles 128 wide (four waves of 32 x 64, three workgroups per CU) were measured against these on
// the same device from K = 16 to 64 and lost everywhere (16384^2 x 16: 260 against 231 us,
// 256 x 100352 x 64: 58 against 46 us): the width is a parameter of the launch, with one value.
int shortk_tile_n(int M, int N, int K, int cus, int batch, bool shared_a)
{
    // beyond 64 k: stages of 32 k with both operands loaded straight into LDS, K a multiple of 4
    if (K < 1 || K > (shared_a ? SHORTK_MAX_K_BATCH : SHORTK_MAX_K) || (K > 64 && K % 4 != 0)) return 0;
    const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64) * batch;
    if (tiles < (long)cus) return 0;
    if (!shared_a && stores_in_pieces_of_lines(M, N, K)) return 0;
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
    if (args.K > (args.tiles_n_per_image || args.batch_cols ? SHORTK_MAX_K_BATCH : SHORTK_MAX_K) || args.split_k != 1 || args.tail_tiles != 0 || args.partial) return hipErrorInvalidValue;
    int grid, lds;
    if (tile_n != 64) return hipErrorInvalidValue;
    const bool plain = !args.accumulate && !args.col_bias;
    if (args.K > 64 && (!plain || args.K % 4 != 0)) return hipErrorInvalidValue;
    const bool direct = args.K <= 32 && plain;
    shortk_launch_shape(tiles, tile_n, direct || args.K > 64 ? args.K : 64, cus, &grid, &lds);
    GemmArgs a2 = args;
    {
        const int group = args.group > 0 ? args.group : 1;
        const int nbands = (args.tiles_m + group - 1) / group;
        a2.by_band = FastDiv::make((unsigned)(group * args.tiles_n));
        a2.by_group = FastDiv::make((unsigned)group);
        a2.by_last_group = FastDiv::make((unsigned)(args.tiles_m - (nbands - 1) * group));
        a2.by_image_tiles = FastDiv::make((unsigned)args.tiles_n_per_image);
        a2.by_batch_cols = FastDiv::make((unsigned)args.batch_cols);
    }
    if (args.batch_cols && (args.K <= 64 || args.batch_cols % 4 != 0 || args.tiles_n_per_image != 0 || args.N % args.batch_cols != 0 ||
                            (double)args.b_batch_stride * (args.N / args.batch_cols) * 4.0 >= 2147483648.0))
        return hipErrorInvalidValue;
    if (direct || args.K > 64) {
        if (direct) hipLaunchKernelGGL(sgemm_shortk_direct_kernel_32, dim3(grid), dim3(256), 0, stream, a2);
        else if (args.batch_cols) hipLaunchKernelGGL(sgemm_shortk_staged_flat_kernel, dim3(grid), dim3(256), 0, stream, a2);
        else hipLaunchKernelGGL(sgemm_shortk_staged_kernel, dim3(grid), dim3(256), 0, stream, a2);
        return hipGetLastError();
    }
    return launch_shortk<TileShortK64, LOAD_VEC4>(a2, grid, stream);
}

// Workgroups launched for `tiles` tiles of 64 x tile_n of a product that overwrites C, and the LDS
// each of them takes: K up to 32 runs on the kernel that loads B straight into LDS
void shortk_launch_shape(long tiles, int tile_n, int K, int cus, int* grid, int* lds_bytes)
{
    (void)tile_n;
    const bool direct = K <= 32;
    const long slots = (long)cus * (direct ? 5 : 4);   // what the LDS of a CU holds: 28.5, 39.5 or (K above 64) 36.5 KB per workgroup
    *grid = (int)(((tiles < slots ? tiles : slots) + 7) / 8 * 8);   // whole rows of 8 XCDs
    *lds_bytes = direct ? (64 * 32 + 2 * 32 * 64 + 4 * 8 * 36) * 4
                        : K > 64 ? (4 * 2048 + 4 * 8 * 36) * 4 : shortk_lds_bytes<TileShortK64>();
}

}  // namespace cake
