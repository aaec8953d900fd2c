// sgemm_conv_patch.hip -- stride-1 convolution as an implicit GEMM that reads the NCHW input
// where it lies (the direct convolution of examples/cake_conv.cpp:31-258,614-716 on the MFMA
// macro-tile): no padded copy, no column matrix, no table of tap offsets.
//
// out[co][n] = sum_k' Wt[co][k'] * B[k'][n] with the sum walked channel block by channel block:
//     k' = (cb * taps + tap) * 32 + c,   channel = cb * 32 + c,   tap = h * Wf + w
// (the order of a sum is free as long as both operands agree; the filters are re-laid to it by
// conv_filter_relayout_kernel, 2 MB for 256 x 256 x 3 x 3).  A K stage of 32 is then 32 channels
// under ONE filter tap, so B[k'][n] = patch[c][row(n) + h][col(n) + w] for a patch of the input
// that stays in LDS for all taps of a channel block:
//   * the patch holds, for 32 channels, the R input rows the tile's pixels can reach and whole
//     rows of P floats: 4 + Win + pad columns, the image's own starting at column 4 so that the
//     16-byte global loads land 16-byte aligned in LDS.  Rows above and below an image and the
//     margins left and right of a row are zero: the padding exists in LDS only.  Rows come from
//     the "virtual" sequence image 0 padded, image 1 padded, ...: a tile whose pixels straddle two
//     images sees the lower margin of one and the upper margin of the next as distinct rows;
//   * the MFMA's B operand of lane n for stage (tap, group of 8 channels) is a 4-byte LDS read at
//     pixel(n) + tap offset + channel * PLANE: the pixel part is fixed per lane, the tap part per
//     stage, the channel part an immediate -- no integer work between the MFMAs;
//   * A (the filters) walks through the usual double-buffered stages; the patch is loaded once per
//     channel block (8 x 16 bytes per thread for 9 stages, where the gather from a staged copy
//     issued 2 per stage), at the start of the block's second-to-last stage, and swapped in
//     between the last stage's barrier and its last operand group.
// Everything else -- tile raster, tail tiles cut along K, epilogue with the NCHW layout -- is the
// macro-tile kernel's (sgemm_tile.hpp).
#include "sgemm_tile.hpp"

namespace cake {

namespace {

using TilePatch = Tile<256, 128, 32, 64, 64, 2, 1, 1>;   // 8 waves of 64 x 64, two register stages for A

constexpr int PATCH_PLANE_FLOATS = CONV_PATCH_PLANE;      // floats per channel of the patch (rows x pitch fit in it)
constexpr int PATCH_CHANNELS = 32;                        // = BK: one tap of 32 channels per K stage
constexpr int PATCH_FLOATS = PATCH_PLANE_FLOATS * PATCH_CHANNELS;

template <class T>
constexpr int patch_smem_bytes() { return (2 * T::A_STAGE + PATCH_FLOATS) * 4; }

// A thread's share of a patch: where its 16-byte chunks come from and where they go.
template <int THREADS>
struct PatchFetch {
    static constexpr int PATCH_ITERS = PATCH_FLOATS / 4 / THREADS;   // 16-byte chunks of a patch per thread
    static_assert(PATCH_FLOATS / 4 % THREADS == 0, "patch chunks are dealt evenly");
    int p_off[PATCH_ITERS];     // byte offset of the chunk inside channel block 0 of the input, or BUF_OOB
    int p_lds[PATCH_ITERS];     // where it goes in the patch (floats, a multiple of 4), or -1; the two low bits
                                // say how many of its 4 floats hang over the end of the row (the last chunk may)
    f32x4 pr[PATCH_ITERS];      // the next block's patch on its way
    const float* in;
    unsigned in_bytes;
    unsigned block_bytes;       // bytes of the input between channel blocks

    // v0: virtual row the patch starts at; rows_used: how many of its rows this tile's pixels reach
    __device__ __forceinline__ void init_patch(const ConvGeom& cv, int v0, int rows_used, int tid)
    {
        in = cv.in;
        in_bytes = cv.in_bytes;
        block_bytes = (unsigned)PATCH_CHANNELS * cv.Hin * cv.Win * 4u;
        const int wc = (cv.Win + 3) >> 2;                 // chunks per input row
        const int per_channel = cv.patch_rows * wc;
        const int total = PATCH_CHANNELS * per_channel;
        const int vrows = cv.Hin + 2 * cv.pad;            // rows of a padded image
#pragma unroll
        for (int it = 0; it < PATCH_ITERS; ++it) {
            const int q = tid + it * THREADS;
            const int c = (int)cv.by_channel_chunks.div(q), rem = q - c * per_channel;
            const int r = (int)cv.by_row_chunks.div(rem), j = rem - r * wc;
            const int v = v0 + r;
            const int b = (int)cv.by_vrows.div(v), hi = v - b * vrows - cv.pad;
            const bool data = q < total && r < rows_used && b < cv.batch && hi >= 0 && hi < cv.Hin;
            p_off[it] = data ? (((b * cv.Cin + c) * cv.Hin + hi) * cv.Win + 4 * j) * 4 : BUF_OOB;
            p_lds[it] = q < total ? c * PATCH_PLANE_FLOATS + r * cv.patch_pitch + 4 + 4 * j + max(0, 4 * j + 4 - cv.Win) : -1;
        }
    }

    // chunk `it` of channel block cb's patch (rows outside an image read as zero).  cb must be a
    // block of the input: the record count is a plain difference on purpose (a saturating one only
    // exists as a vector instruction, and a record count in a vector register makes the compiler
    // loop over the load).
    template <int IT>
    __device__ __forceinline__ void load_patch_chunk(int cb)
    {
        const unsigned skip = (unsigned)cb * block_bytes;
        pr[IT] = buffer_load_f32x4(reinterpret_cast<const float*>(reinterpret_cast<const char*>(in) + skip), p_off[IT],
                                   in_bytes - skip);
    }
    template <int IT = 0>
    __device__ __forceinline__ void load_patch(int cb)
    {
        if constexpr (IT < PATCH_ITERS) {
            load_patch_chunk<IT>(cb);
            load_patch<IT + 1>(cb);
        }
    }

    __device__ __forceinline__ void store_patch_to(float* patch)
    {
#pragma unroll
        for (int it = 0; it < PATCH_ITERS; ++it) {
            f32x4 v = pr[it];
            const int over = p_lds[it] & 3;
            if (over > 0) v[3] = 0.f;
            if (over > 1) v[2] = 0.f;
            if (over > 2) v[1] = 0.f;
            if (p_lds[it] >= 0) *reinterpret_cast<f32x4*>(patch + (p_lds[it] & ~3)) = v;
        }
    }
};

// Everything about the operands that is fixed per thread for a whole tile.
template <class T>
struct PatchLoader : PatchFetch<T::THREADS> {
    using PatchFetch<T::THREADS>::PATCH_ITERS;
    int a_off[T::A_ITERS];      // byte offset from the A tile origin, or BUF_OOB for rows >= M
    const float* a_base;        // Wt + m0 * lda
    unsigned a_elems;
    float* patch;

    __device__ __forceinline__ void init(const GemmArgs& g, int m0, int v0, int rows_used, int tid, float* patch_)
    {
        a_base = g.A + (size_t)m0 * g.lda;
        a_elems = clamp_elems((long long)(g.M - 1 - m0) * g.lda + g.K);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) {
            const int c = tid + it * T::THREADS;
            const int r = c / (T::BK / 4);
            a_off[it] = (m0 + r < g.M) ? (r * g.lda + (c % (T::BK / 4)) * 4) * 4 : BUF_OOB;
        }
        patch = patch_;
        this->init_patch(g.conv, v0, rows_used, tid);
    }

    __device__ __forceinline__ f32x4 load_a(int k0, int off) const
    {
        return buffer_load_f32x4(a_base + k0, off, records_left(a_elems, (unsigned)k0));
    }

    __device__ __forceinline__ void store_patch() { this->store_patch_to(patch); }
};

// One K step as the slot machinery of sgemm_tile.hpp sees it.
// PAIRED: one of two consecutive taps inside a channel block, which alternate between the two
// register stages of A so that their loads are dealt over the whole step.
// PAIRED_FETCH: the second tap of a block's last pair; it also fetches the next block's patch, in
// its first operand group, so that the patch has a whole step and more to arrive.
// SINGLE: a tap on its own (a block with an even number of taps starts with one): its loads of A
// follow its stores, into the registers just stored.
// LAST: the last tap of a channel block, as SINGLE; it swaps the fetched patch in between its
// barrier and its last operand group.
enum PatchStepKind { PATCH_PAIRED, PATCH_PAIRED_FETCH, PATCH_SINGLE, PATCH_LAST };
template <class T, int KIND>
struct PatchStep {
    using PL = PatchLoader<T>;
    static constexpr int NUM_LOADS = T::A_ITERS;
    static constexpr int EARLY_LOADS = KIND == PATCH_PAIRED_FETCH ? PL::PATCH_ITERS : 0;
    static constexpr bool SINGLE_STAGE = KIND == PATCH_SINGLE || KIND == PATCH_LAST;
    static constexpr bool MASK_A_STORES = false;   // K' is a whole number of stages
    static constexpr bool B_ALONG_K = false;
    static constexpr int PATCH_PLANE = PATCH_PLANE_FLOATS;
    static constexpr bool END_OF_BLOCK = KIND == PATCH_LAST;
    PL& pl;
    int next_block;
    template <int OP, class RA, class RB>
    __device__ __forceinline__ void load_one(int k0, int /*kend*/, RA& ra, RB& /*rb*/) const
    {
        if constexpr (OP < T::A_ITERS)
            ra[OP] = pl.load_a(k0, pl.a_off[OP]);
        else
            pl.template load_patch_chunk<OP - T::A_ITERS>(next_block);
    }
    __device__ __forceinline__ void swap_patch() const { pl.store_patch(); }
};

// A tail tile without K slices in memory.  A thin last round (config 5: 16 tiles for 256 CUs) used
// to be cut along K into one slice per CU, each slice paying a tile's whole prologue for four or
// five steps, writing its 128 KB of partial sums and leaving them to a second kernel.  Here a tile
// is cut into 16 sub-tiles of 64 rows x 32 pixels instead, one workgroup each, over the whole K:
//   * wave (blk, kq) of the 8 owns 32 x 32 block blk and quarter kq (8 channels) of every stage,
//     so each SIMD holds two independent chains of MFMAs, and the four quarters meet in LDS at the
//     end, summed in quarter order;
//   * A never touches LDS: a lane's 16 bytes of filters per stage (row blk * 32 + lane % 32, four
//     consecutive channels) are exactly its MFMA operands, loaded a whole channel block ahead
//     into a ring of TAPS registers;
//   * the patch (32 pixels' worth of rows, same layout and loader as the large tile's) is double
//     buffered, so a channel block ends with one barrier and no swap;
//   * the result goes to C from the summing pass, 32 consecutive pixels per row.
// TAPS is a template argument because the ring is indexed by tap and because the compiler can
// only count how many younger loads may stay in flight at each wait when the block is unrolled.
template <class T, int TAPS>
__device__ __forceinline__ void patch_tail_subtile(const GemmArgs& g, float* smem, const WorkItem& w)
{
    static_assert(T::THREADS == 512 && T::BM == 256 && T::BN == 128, "16 sub-tiles of 64 x 32, 8 waves each");
    static_assert(2 * PATCH_FLOATS * 4 <= patch_smem_bytes<T>(), "two patches fit the kernel's LDS");
    using PF = PatchFetch<T::THREADS>;
    const ConvGeom& cv = g.conv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int blk = wave & 1, kq = wave >> 1;
    const int m0 = w.tile_m * T::BM + (w.slice & 3) * 64;
    const int n0 = w.tile_n * T::BN + (w.slice >> 2) * 32;
    if (m0 >= g.M || n0 >= g.N) return;                   // the whole workgroup

    // the patch: as for the large tile, for 32 pixels
    const int vrows = cv.Hin + 2 * cv.pad;
    const int g0 = (int)cv.by_row_n.div(n0), img0 = (int)cv.by_hout.div(g0);
    const int v0 = img0 * vrows + (g0 - img0 * cv.Hout);
    int pix;
    {
        int n = n0 + l32;
        if (n >= g.N) n = n0;                              // computed and dropped
        const int gr = (int)cv.by_row_n.div(n), wo = n - gr * cv.row_n;
        const int b = (int)cv.by_hout.div(gr), ho = gr - b * cv.Hout;
        pix = (b * vrows + ho - v0) * cv.patch_pitch + (4 - cv.pad) + wo + (kq * 8 + lh * 4) * PATCH_PLANE_FLOATS;
    }
    const int n_last = min(n0 + 32, g.N) - 1;
    const int g_last = (int)cv.by_row_n.div(n_last), img_last = (int)cv.by_hout.div(g_last);
    const int rows_used = img_last * vrows + (g_last - img_last * cv.Hout) - v0 + cv.Hf;
    PF pf;
    pf.init_patch(cv, v0, rows_used, tid);
    // (the two patches are addressed by offsets into the one LDS array: pointers picked from a table
    // would lose their address space and become flat accesses)

    // A: the lane's row of the filters, its 4 channels of the wave's quarter
    const float* a_base = g.A + (size_t)m0 * g.lda;
    const unsigned a_elems = clamp_elems((long long)(g.M - 1 - m0) * g.lda + g.K);
    const int a_row = blk * 32 + l32;
    const int a_off = (m0 + a_row < g.M) ? (a_row * g.lda + kq * 8 + lh * 4) * 4 : BUF_OOB;
    auto load_a = [&](int step) {
        return buffer_load_f32x4(a_base + step * PATCH_CHANNELS, a_off, records_left(a_elems, (unsigned)(step * PATCH_CHANNELS)));
    };

    int toff[TAPS];
    {
        int th = 0, tw = 0;
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
            toff[t] = th * cv.patch_pitch + tw;
            if (++tw == cv.Wf) { tw = 0; ++th; }
        }
    }
    const int blocks = cv.Cin / PATCH_CHANNELS, last_block = blocks - 1;

    pf.load_patch(0);
    f32x4 ring[TAPS];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) ring[t] = load_a(t);
    // margins (and rows no chunk writes) are zero for the whole walk, in both patches
    for (int i = tid; i < 2 * PATCH_FLOATS / 4; i += T::THREADS)
        reinterpret_cast<f32x4*>(smem)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    pf.store_patch_to(smem);
    pf.load_patch(min(1, last_block));
    __syncthreads();

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;

    auto read_b = [&](float (&b)[4], int patch, int off) {
#pragma unroll
        for (int i = 0; i < 4; ++i) b[i] = smem[i * PATCH_PLANE_FLOATS + pix + patch + off];
    };
    // one channel block out of `patch`; with PREFETCH the filters of the block after it follow
    // their predecessors into the ring
    auto block = [&](int cb, int patch, auto prefetch) {
        float bq[2][4];
        read_b(bq[0], patch, toff[0]);
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
            const f32x4 a = ring[t];
            if constexpr (decltype(prefetch)::value) ring[t] = load_a((cb + 1) * TAPS + t);
            if (t + 1 < TAPS) read_b(bq[(t + 1) & 1], patch, toff[t + 1]);
            // (pinned: left to itself the compiler reads each operand right in front of its MFMA and
            // the chain waits out an LDS round trip per pair)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], bq[t & 1][i], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    for (int cb = 0; cb < last_block; ++cb) {
        block(cb, (cb & 1) * PATCH_FLOATS, std::true_type{});
        // (the other patch was last read a block ago, before the barrier that ended that block)
        pf.store_patch_to(smem + ((cb + 1) & 1) * PATCH_FLOATS);
        __syncthreads();
        pf.load_patch(min(cb + 2, last_block));
    }
    block(last_block, (last_block & 1) * PATCH_FLOATS, std::false_type{});

    // the four K quarters of each block meet in LDS; register r of a 32 x 32 block holds row
    // 8 * (r / 4) + 4 * (lane / 32) + r % 4, column lane % 32
    __syncthreads();                                       // nobody reads a patch any more
    float* red = smem;
#pragma unroll
    for (int r = 0; r < 16; ++r) red[(wave * 16 + r) * 64 + lane] = acc[r];
    __syncthreads();
    const int n = n0 + l32;
    size_t off = 0, row_stride = 0;
    const int valid = n < g.N ? conv_out_map(cv, g.M, g.ldc, n, 1, off, row_stride) : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = tid + i * T::THREADS;
        const int b = e >> 10, r = (e >> 6) & 15;
        float s = red[((0 * 2 + b) * 16 + r) * 64 + lane];
#pragma unroll
        for (int q = 1; q < 4; ++q) s += red[((q * 2 + b) * 16 + r) * 64 + lane];
        const int m = m0 + b * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (valid > 0 && m < g.M) {
            float* dst = g.C + (size_t)m * row_stride + off;
            *dst = g.accumulate ? *dst + s : s;
        }
    }
}

template <class T>
__global__ void __launch_bounds__(T::THREADS) sgemm_conv_patch_kernel(const GemmArgs g)
{
    static_assert(T::KSPLIT == 1 && T::REG_STAGES == 2 && T::BK == PATCH_CHANNELS && T::TN <= 2, "tile shape");
    using PL = PatchLoader<T>;
    extern __shared__ __align__(16) float smem[];
    float* As = smem;
    float* patch = smem + 2 * T::A_STAGE;
    const ConvGeom& cv = g.conv;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = (wave / T::WAVES_N) * T::WM;
    const int wn0 = (wave % T::WAVES_N) * T::WN;
    const int a_lane = (wm0 + l32) * T::LDA;

    const WorkItem w = decode_tile(g, blockIdx.x);
    const int m0 = w.tile_m * T::BM, n0 = w.tile_n * T::BN;
    const int taps = cv.Hf * cv.Wf;
    if (w.tail_tile >= 0 && cv.tail_mode == CONV_TAIL_SUBTILES) {
        patch_tail_subtile<T, 9>(g, smem, w);
        return;
    }
    // K slices are whole channel blocks, or the first or second half of one block's taps
    int kbeg = w.kbeg, kend = w.kend;
    if (w.tail_tile >= 0 && cv.tail_mode == CONV_TAIL_HALVES) {
        const int first = (taps + 1) >> 1, cb = w.slice >> 1;
        kbeg = (cb * taps + (w.slice & 1) * first) * T::BK;
        kend = (w.slice & 1) ? (cb + 1) * taps * T::BK : kbeg + first * T::BK;
    }
    const int steps = (kend - kbeg) / T::BK;
    const int cb0 = kbeg / (T::BK * taps);
    const int tap_lo = kbeg / T::BK - cb0 * taps;         // the first tap of the walk (0 unless half a block)
    const int tap_n = steps < taps ? steps : taps;        // taps walked per channel block
    const int th0 = tap_lo / cv.Wf, tw0 = tap_lo - th0 * cv.Wf;
    const int off0 = th0 * cv.patch_pitch + tw0;
    const int last_block = cv.Cin / PATCH_CHANNELS - 1;

    // the tile's first pixel fixes which virtual row the patch starts at
    const int vrows = cv.Hin + 2 * cv.pad;
    const int g0 = (int)cv.by_row_n.div(n0), img0 = (int)cv.by_hout.div(g0);
    const int v0 = img0 * vrows + (g0 - img0 * cv.Hout);
    // where the lane's pixels (one per 32-column block of the wave) sit in the patch under tap (0, 0);
    // the lane's half of an operand group (channels 0..3 or 4..7) is folded in
    int pix[2] = {0, 0};
#pragma unroll
    for (int tn = 0; tn < T::TN; ++tn) {
        int n = n0 + wn0 + tn * 32 + l32;
        if (n >= g.N) n = n0;                              // computed and dropped
        const int gr = (int)cv.by_row_n.div(n), wo = n - gr * cv.row_n;
        const int b = (int)cv.by_hout.div(gr), ho = gr - b * cv.Hout;
        pix[tn] = (b * vrows + ho - v0) * cv.patch_pitch + (4 - cv.pad) + wo + lh * 4 * PATCH_PLANE_FLOATS;
    }

    f32x16 acc[T::TM][T::TN];
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.f;

    if (steps > 0) {
        // the rows below the last pixel's window are never read: not fetched either
        const int n_last = min(n0 + T::BN, g.N) - 1;
        const int g_last = (int)cv.by_row_n.div(n_last), img_last = (int)cv.by_hout.div(g_last);
        const int rows_used = img_last * vrows + (g_last - img_last * cv.Hout) - v0 + cv.Hf;
        PL pl;
        pl.init(g, m0, v0, rows_used, tid, patch);
        // ra[1] holds the stage that the next step stores, at every step that is not the second of a pair
        f32x4 ra[2][T::A_ITERS], rb_unused[T::B_ITERS];
        Frag<T> frag[2];
        // prologue: the first block's patch and the first stage of A
        pl.load_patch(cb0);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[1][it] = pl.load_a(kbeg, pl.a_off[it]);
        // margins (and rows no chunk writes) are zero for the whole walk
        for (int i = tid; i < PATCH_FLOATS / 4; i += T::THREADS)
            reinterpret_cast<f32x4*>(patch)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
        pl.store_patch();
        store_stage_a<T>(As, tid, ra[1]);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[1][it] = pl.load_a(kbeg + T::BK, pl.a_off[it]);
        __syncthreads();
        // operands of the first group: A from stage 0, B from the patch under the first tap
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
            frag[0].a[tm] = *reinterpret_cast<const f32x4*>(As + a_lane + tm * 32 * T::LDA + lh * 4);
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int i = 0; i < 4; ++i) frag[0].b[tn][i] = patch[i * PATCH_PLANE_FLOATS + pix[tn] + off0];

        // One loop per kind of step: two step bodies chosen inside one loop would make the compiler
        // copy the accumulators wherever the bodies' register assignments meet, i.e. after every step.
        int cur = 0, s = 0;
        auto step_with = [&](const auto& loader, int off_cur, int off_next, f32x4 (&sa)[T::A_ITERS], f32x4 (&fa)[T::A_ITERS]) {
            using LD = std::remove_cv_t<std::remove_reference_t<decltype(loader)>>;
            const WalkCtx<T, LD> c{loader, kbeg + (s + 2) * T::BK, kend,
                                   As + cur * T::A_STAGE, patch + off_cur,
                                   As + (cur ^ 1) * T::A_STAGE, patch + off_next,
                                   tid, a_lane, pix[0], lh, sa, rb_unused, fa, rb_unused, pix[T::TN - 1]};
            __builtin_amdgcn_sched_barrier(0);
            step_groups<T, LD>(c, frag, acc);
            cur ^= 1;
            ++s;
        };
        const int blocks = steps < taps ? 1 : steps / taps;
        for (int cb = cb0; cb < cb0 + blocks; ++cb) {
            int th = th0, tw = tw0, off = off0;
            // offset of the next stage's tap, whose first operands a step reads
            auto next_tap = [&] {
                if (++tw == cv.Wf) { tw = 0; ++th; }
                return th * cv.patch_pitch + tw;
            };
            int tap = 0;
            if ((tap_n - 1) & 1) {
                const int off_next = next_tap();
                step_with(PatchStep<T, PATCH_SINGLE>{pl, cb}, off, off_next, ra[1], ra[1]);
                off = off_next;
                ++tap;
            }
            // (after the last channel block its own patch is fetched once more and never used)
            const int fetch = min(cb + 1, last_block);
            for (; tap < tap_n - 3; tap += 2) {
                const int off1 = next_tap();
                step_with(PatchStep<T, PATCH_PAIRED>{pl, cb}, off, off1, ra[1], ra[0]);
                const int off2 = next_tap();
                step_with(PatchStep<T, PATCH_PAIRED>{pl, cb}, off1, off2, ra[0], ra[1]);
                off = off2;
            }
            const int off1 = next_tap();
            step_with(PatchStep<T, PATCH_PAIRED>{pl, cb}, off, off1, ra[1], ra[0]);
            const int off2 = next_tap();
            step_with(PatchStep<T, PATCH_PAIRED_FETCH>{pl, fetch}, off1, off2, ra[0], ra[1]);
            step_with(PatchStep<T, PATCH_LAST>{pl, fetch}, off2, 0, ra[1], ra[1]);
        }
    }

    if (w.tail_tile >= 0) {
        // a K slice of a tail tile: the whole BM x BN block, tile-local, no masking
        float* out = g.tail_partial + ((size_t)w.slice * g.tail_tiles + w.tail_tile) * (T::BM * T::BN);
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    out[(wm0 + tm * 32 + 8 * (r >> 2) + 4 * lh + (r & 3)) * T::BN + wn0 + tn * 32 + l32] = acc[tm][tn][r];
        return;
    }
    // (streamed out where its rows are whole cache lines: C then drains while the other tiles are
    // multiplied instead of staying dirty in the L2s until the kernel ends -- config 5: 846 -> 840 us)
    store_c_tile<T, LOAD_IM2COL_ROW, false, true>(g, smem, acc, m0, n0, w.slice, wave, wm0, wn0, lane, l32, lh);
}

// Wt[co][(cb * taps + tap) * 32 + c] = W[co][(cb * 32 + c) * taps + tap], zero for channels past Cin
__global__ void __launch_bounds__(256) conv_filter_relayout_kernel(const float* __restrict__ W, float* __restrict__ Wt,
                                                                   int Cout, int Cin, int taps, int kp)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)Cout * kp) return;
    const int co = (int)(i / kp), k = (int)(i - (size_t)co * kp);
    const int c = k & 31, bt = k >> 5;
    const int cb = bt / taps, tap = bt - cb * taps;
    const int ch = cb * 32 + c;
    Wt[i] = ch < Cin ? W[((size_t)co * Cin + ch) * taps + tap] : 0.f;
}

}  // namespace

// Rows and row pitch of the patch for this geometry, or false when the kernel does not take it:
// stride 1 only, at least three taps, padding of at most 4, whole blocks of 32 channels, and a patch plane of at most 512 floats
// (56 x 56 maps under a 3 x 3 filter use all of it; wider images keep the staged-copy path).
bool conv_patch_geometry(int batch, int Cin, int Hin, int Win, int Hf, int Wf, int stride, int pad, int Hout, int Wout,
                         int* rows, int* pitch)
{
    if (stride != 1 || Hf * Wf < 3 || pad > 4 || Cin % 32 != 0) return false;
    const int row_n = (Wout + 3) & ~3;
    const int bn = TilePatch::BN;
    const int out_rows = (row_n - 1 + bn - 1) / row_n + 1;               // output rows a tile's pixels can lie in
    int images = (bn - 1) / (Hout * row_n) + 1;                          // image borders a tile can cross
    if (images > batch - 1) images = batch - 1;
    // consecutive output rows of one image are one virtual row apart, the first row of the next
    // image Hf - 1 more (a padded image has Hout + Hf - 1 rows); a window reaches Hf - 1 rows down
    const int R = out_rows + (Hf - 1) * images + Hf - 1;
    const int data = 4 + Win + pad, reach = 4 - pad + row_n + Wf - 1;     // last column written / read, + 1
    const int P = ((data > reach ? data : reach) + 3) & ~3;
    if (R * P > PATCH_PLANE_FLOATS) return false;
    // byte offsets into the input are 32-bit
    if ((double)batch * Cin * Hin * Win * 4.0 >= 2147483648.0) return false;
    *rows = R;
    *pitch = P;
    return true;
}

int conv_patch_k(int Cin, int Hf, int Wf) { return (Cin + 31) / 32 * 32 * Hf * Wf; }

hipError_t launch_conv_filter_relayout(const float* W, float* Wt, int Cout, int Cin, int taps, hipStream_t stream)
{
    const int kp = (Cin + 31) / 32 * 32 * taps;
    const size_t n = (size_t)Cout * kp;
    hipLaunchKernelGGL(conv_filter_relayout_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, W, Wt, Cout,
                       Cin, taps, kp);
    return hipGetLastError();
}

hipError_t launch_sgemm_conv_patch(const GemmArgs& args, int grid, hipStream_t stream)
{
    using T = TilePatch;
    auto kern = sgemm_conv_patch_kernel<T>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, patch_smem_bytes<T>());
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::THREADS), patch_smem_bytes<T>(), stream, args);
    return hipGetLastError();
}

}  // namespace cake
