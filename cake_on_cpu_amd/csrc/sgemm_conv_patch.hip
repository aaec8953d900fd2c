// sgemm_conv_patch.hip -- stride-1 convolution as an implicit GEMM that reads the NCHW input
// where it lies (the direct convolution of examples/cake_conv.cpp:31-258,614-716 on the MFMA
// macro-tile): no padded copy, no column matrix, no table of tap offsets.
//
// out[co][n] = sum_k' Wt[co][k'] * B[k'][n] with the sum walked in half blocks of 16 channels:
//     k' = (hb * taps + tap) * 16 + c,   channel = hb * 16 + c,   tap = h * Wf + w
// (the order of a sum is free as long as both operands agree; the filters are re-laid to it by
// conv_filter_relayout_kernel, 2 MB for 256 x 256 x 3 x 3).  A K stage of 32 is then two *pairs*
// of operand groups, each pair 16 channels under ONE filter tap, so
// B[k'][n] = patch[c][row(n) + h][col(n) + w] for a patch of the input that stays in LDS for all
// taps of its half block:
//   * a patch holds, for 16 channels, the R input rows the tile's pixels can reach and whole
//     rows of P floats: 4 + Win + pad columns, the image's own starting at column 4 so that the
//     16-byte global loads land 16-byte aligned in LDS.  Rows above and below an image and the
//     margins left and right of a row are zero: the padding exists in LDS only.  Rows come from
//     the "virtual" sequence image 0 padded, image 1 padded, ...: a tile whose pixels straddle two
//     images sees the lower margin of one and the upper margin of the next as distinct rows;
//   * the MFMA's B operand of lane n for a group (tap, 8 channels) is a 4-byte LDS read at
//     pixel(n) + tap offset + channel * PLANE: the pixel part is fixed per lane, the tap part per
//     pair, the channel part an immediate -- no integer work between the MFMAs;
//   * LDS has room for two such patches, and half blocks alternate between them: while the taps
//     of half block hb are walked out of one, half block hb + 1 waits in the other and hb + 2 is
//     fetched (4 x 16 bytes per thread) and written over hb's predecessor -- behind a stage's
//     barrier, two stages after its loads were issued, with no barrier of its own.  (One patch of
//     32 channels, swapped between two barriers at the end of its taps, stalled every wave of the
//     workgroup once per 9 stages: 11 us of config 5's 841.)
//   * A (the filters) walks through the usual double-buffered stages.
// Built for a known filter shape (3 x 3), the kernel walks K in the filters' own order instead,
// k = channel * taps + tap, and reads them where they lie as well: a pair of groups is then 16
// consecutive k, i.e. one or two channels under runs of taps, and since everything about a k is
// known when the code is compiled, a lane's read address is a register per filter tap of its
// first k (where its pixel sits under that tap's row, with the difference to the tap four k
// further on folded in for the upper half of the lanes) plus an immediate.  Half blocks of 16
// channels are still 16 * taps consecutive k, so the patches take turns exactly as above.
// Everything else -- tile raster, tail tiles cut along K, epilogue with the NCHW layout -- is the
// macro-tile kernel's (sgemm_tile.hpp).
#include "sgemm_tile.hpp"

namespace cake {

namespace {

using TilePatch = Tile<256, 128, 32, 64, 64, 2, 1, 1>;   // 8 waves of 64 x 64, two register stages for A

constexpr int PATCH_PLANE_FLOATS = CONV_PATCH_PLANE;      // floats per channel of the patch (rows x pitch fit in it)
constexpr int PATCH_CHANNELS = 32;                        // channels per block: two patches of 16, a whole number of K stages
constexpr int HALF_CHANNELS = 16;                         // channels per patch: a pair of operand groups per tap
constexpr int PATCH_FLOATS = PATCH_PLANE_FLOATS * PATCH_CHANNELS;   // both patches
constexpr int HALF_FLOATS = PATCH_PLANE_FLOATS * HALF_CHANNELS;

template <class T>
constexpr int patch_smem_bytes() { return (2 * T::A_STAGE + PATCH_FLOATS) * 4; }

// Zeroes what the walk reads of `planes` channel planes but never writes: per row, the 16 bytes left
// of the image's columns and the chunks right of them (the zero padding lives there; every other
// chunk of a row, rows outside an image included, is written anew with each patch).
template <int THREADS>
__device__ __forceinline__ void zero_patch_margins(const ConvGeom& cv, float* patch, int planes, int tid)
{
    const int per_channel = cv.patch_rows * cv.margin_chunks;
    const int first_right = 4 + 4 * ((cv.Win + 3) >> 2);
    for (int q = tid; q < planes * per_channel; q += THREADS) {
        const int c = (int)cv.by_channel_margin_chunks.div(q), rem = q - c * per_channel;
        const int r = (int)cv.by_margin_chunks.div(rem), m = rem - r * cv.margin_chunks;
        const int col = m == 0 ? 0 : first_right + 4 * (m - 1);
        *reinterpret_cast<f32x4*>(patch + c * PATCH_PLANE_FLOATS + r * cv.patch_pitch + col) = f32x4{0.f, 0.f, 0.f, 0.f};
    }
}

// A thread's share of a patch: where its 16-byte chunks come from and where they go.
template <int THREADS, int CHANNELS>
struct PatchFetch {
    static constexpr int PATCH_ITERS = PATCH_PLANE_FLOATS * CHANNELS / 4 / THREADS;   // 16-byte chunks of a patch per thread
    static_assert(PATCH_PLANE_FLOATS * CHANNELS / 4 % THREADS == 0, "patch chunks are dealt evenly");
    int p_off[PATCH_ITERS];     // byte offset of the chunk inside the first CHANNELS channels of the input, or BUF_OOB
    int p_lds[PATCH_ITERS];     // where it goes in the patch (floats, a multiple of 4); the two low bits say how
                                // many of its 4 floats hang over the end of the row (the last chunk may).  A
                                // chunk that does not exist is fetched as zeros and goes to the left margin
                                // of the patch's first row, which is zero anyway: no branch around the store
    f32x4 pr[PATCH_ITERS];      // a patch on its way
    const float* in;
    unsigned in_bytes;
    unsigned block_bytes;       // bytes of the input between blocks of CHANNELS channels

    // v0: virtual row the patch starts at; rows_used: how many of its rows this tile's pixels reach
    __device__ __forceinline__ void init_patch(const ConvGeom& cv, int v0, int rows_used, int tid)
    {
        in = cv.in;
        in_bytes = cv.in_bytes;
        block_bytes = (unsigned)CHANNELS * cv.Hin * cv.Win * 4u;
        const int wc = (cv.Win + 3) >> 2;                 // chunks per input row
        const int per_channel = cv.patch_rows * wc;
        const int total = CHANNELS * per_channel;
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
            p_lds[it] = q < total ? c * PATCH_PLANE_FLOATS + r * cv.patch_pitch + 4 + 4 * j + max(0, 4 * j + 4 - cv.Win) : 0;
        }
    }

    // chunk `it` of the patch of block cb of CHANNELS channels (rows outside an image read as zero).
    // cb must be a block of the input: the record count is a plain difference on purpose (a saturating one only
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

    template <int IT>
    __device__ __forceinline__ void store_patch_chunk_to(float* patch)
    {
        f32x4 v = pr[IT];
        const int over = p_lds[IT] & 3;
        if (over > 0) v[3] = 0.f;
        if (over > 1) v[2] = 0.f;
        if (over > 2) v[1] = 0.f;
        *reinterpret_cast<f32x4*>(patch + (p_lds[IT] & ~3)) = v;
    }
    template <int IT = 0>
    __device__ __forceinline__ void store_patch_to(float* patch)
    {
        if constexpr (IT < PATCH_ITERS) {
            store_patch_chunk_to<IT>(patch);
            store_patch_to<IT + 1>(patch);
        }
    }
};

// Where lane half lh (k + 4 lh of a group) reads under the tap of the group's k in the filters'
// own order, relative to the lane's pixel under tap (0, 0) and apart from the immediate part
// channel(k) * PLANE + column(tap(k)): the lower lanes read in the row of tap(k); the upper lanes
// four k further on, which is another tap and possibly the next channel.
template <int HF, int WF>
__device__ __forceinline__ int natural_place(int tap, int lh, int pitch)
{
    constexpr int TAPS = HF * WF;
    const int tap_b = (tap + 4) % TAPS, ch_b = (tap + 4) / TAPS;
    const int lower = (tap / WF) * pitch;
    const int upper = (tap_b / WF) * pitch + ch_b * PATCH_PLANE_FLOATS + tap_b % WF - tap % WF;
    return lh ? upper : lower;
}

// Everything about the operands that is fixed per thread for a whole tile.  NPLACE > 0: the
// filters' own K order; place[tn][tap] then says where the lane reads for a k under that tap.
template <class T, int NPLACE = 0>
struct PatchLoader : PatchFetch<T::THREADS, HALF_CHANNELS> {
    using PatchFetch<T::THREADS, HALF_CHANNELS>::PATCH_ITERS;
    int a_off[T::A_ITERS];      // byte offset from the A tile origin, or BUF_OOB for rows >= M
    const float* a_base;        // the filters (re-laid or not) + m0 * lda
    unsigned a_elems;
    const float* patch;
    int place[T::TN][NPLACE > 0 ? NPLACE : 1];

    __device__ __forceinline__ void init(const GemmArgs& g, int m0, int v0, int rows_used, int tid, const float* patch_)
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
};

// One K step as the slot machinery of sgemm_tile.hpp sees it.  Steps come in pairs that alternate
// between the two register stages of A, so that their loads are dealt over the whole step; a
// SINGLE step stands alone (a block with an odd number of steps ends with one): its loads of A
// follow its stores, into the registers just stored.  FETCH: the step also issues the loads of a
// patch (half block `hb`), in its first operand group.  STORE: the step writes the patch fetched
// two or three steps earlier to `dst`, chunk by chunk between the MFMAs of its last group.
// HF x WF > 0: the filters' own K order, and J is the step's number in its channel block.
template <class T, bool SINGLE, bool FETCH, bool STORE, int HF = 0, int WF = 0, int J = 0>
struct PatchStep {
    using PL = PatchLoader<T, HF * WF>;
    static constexpr int NUM_LOADS = T::A_ITERS;
    static constexpr int EARLY_LOADS = FETCH ? PL::PATCH_ITERS : 0;
    static constexpr bool SINGLE_STAGE = SINGLE;
    static constexpr bool MASK_A_STORES = false;   // K' is a whole number of stages
    static constexpr bool B_ALONG_K = false;
    static constexpr int PATCH_PLANE = PATCH_PLANE_FLOATS;
    static constexpr int PATCH_STORES = STORE ? PL::PATCH_ITERS : 0;
    static constexpr bool READS_PATCH_ITSELF = HF > 0;
    PL& pl;
    int hb;          // FETCH: the half block whose patch this step fetches
    float* dst;      // STORE: where the fetched patch goes
    template <int OP, class RA, class RB>
    __device__ __forceinline__ void load_one(int k0, int /*kend*/, RA& ra, RB& /*rb*/) const
    {
        if constexpr (OP < T::A_ITERS)
            ra[OP] = pl.load_a(k0, pl.a_off[OP]);
        else
            pl.template load_patch_chunk<OP - T::A_ITERS>(hb);
    }
    template <int IT>
    __device__ __forceinline__ void store_patch_chunk() const { pl.template store_patch_chunk_to<IT>(dst); }
    // operand i of the lane for column block TN_ and group NG of this step (WRAP: of the next step):
    // k = 8 * group + 4 * (lane / 32) + i, counted from the start of the channel block
    template <int NG, bool WRAP, int TN_, int I>
    __device__ __forceinline__ float patch_read() const
    {
        constexpr int TAPS = HF * WF;
        constexpr int G = (4 * (WRAP ? J + 1 : J) + NG) % (4 * TAPS);
        constexpr int k = 8 * G + I, ch = k / TAPS, tap = k % TAPS;
        return pl.patch[pl.place[TN_][tap] + ch * PATCH_PLANE_FLOATS + tap % WF];
    }
};

// A tail tile without K slices in memory.  A thin last round (config 5: 16 tiles for 256 CUs) used
// to be cut along K into one slice per CU, each slice paying a tile's whole prologue for four or
// five steps, writing its 128 KB of partial sums and leaving them to a second kernel.  Here a tile
// is cut into 16 sub-tiles of 64 rows x 32 pixels instead, one workgroup each, over the whole K:
//   * wave (blk, kq) of the 8 owns 32 x 32 block blk and quarter kq (8 channels) of every channel
//     block, so each SIMD holds two independent chains of MFMAs, and the four quarters meet in
//     LDS at the end, summed in quarter order;
//   * A never touches LDS: a lane's 16 bytes of filters per tap (row blk * 32 + lane % 32, four
//     consecutive channels) are exactly its MFMA operands, loaded a whole channel block ahead
//     into a ring of TAPS registers;
//   * the patch (32 channels, 32 pixels' worth of rows, same layout and loader as the large
//     tile's) is double buffered: block cb + 1's is written during the first taps of block cb,
//     between the MFMAs, most of a block after its loads were issued, so a block ends with one
//     barrier;
//   * the result goes to C from the summing pass, 32 consecutive pixels per row.
// TAPS is a template argument because the ring is indexed by tap and because the compiler can
// only count how many younger loads may stay in flight at each wait when the block is unrolled.
// With the filter's shape known as well (HF x WF > 0) K runs in the filters' own order, a quarter
// is 8 * TAPS consecutive k, and a lane's read addresses are a register per patch and tap plus
// immediates (natural_place).
template <class T, int TAPS, int HF, int WF>
__device__ __forceinline__ void patch_tail_subtile(const GemmArgs& g, float* smem, const WorkItem& w)
{
    static_assert(T::THREADS == 512 && T::BM == 256 && T::BN == 128, "16 sub-tiles of 64 x 32, 8 waves each");
    static_assert(2 * PATCH_FLOATS * 4 <= patch_smem_bytes<T>(), "two patches fit the kernel's LDS");
    static_assert(HF == 0 || HF * WF == TAPS, "filter shape");
    using PF = PatchFetch<T::THREADS, PATCH_CHANNELS>;
    static_assert(PF::PATCH_ITERS == 8 && TAPS >= 4, "the patch's chunks are written four per tap in taps 0 and 1, the next ones fetched four per tap in taps 2 and 3");
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
        pix = (b * vrows + ho - v0) * cv.patch_pitch + (4 - cv.pad) + wo + (kq * 8 + (HF > 0 ? 0 : lh * 4)) * PATCH_PLANE_FLOATS;
    }
    const int n_last = min(n0 + 32, g.N) - 1;
    const int g_last = (int)cv.by_row_n.div(n_last), img_last = (int)cv.by_hout.div(g_last);
    const int rows_used = img_last * vrows + (g_last - img_last * cv.Hout) - v0 + cv.Hf;
    PF pf;
    pf.init_patch(cv, v0, rows_used, tid);
    // (the two patches are addressed by offsets into the one LDS array: pointers picked from a table
    // would lose their address space and become flat accesses)

    // A: the lane's row of the filters, 4 consecutive k of the wave's quarter.  Quarter kq is channels
    // 8 kq .. 8 kq + 7 of the block.  In the re-laid order these are channels (kq & 1) * 8 .. + 7 of
    // half block kq >> 1, whose taps lie 16 floats apart, and load t is tap t; in the filters' own
    // order they are 8 * TAPS consecutive k, and load t is the t-th group of 8.
    const float* a_base = g.A + (size_t)m0 * g.lda;
    const unsigned a_elems = clamp_elems((long long)(g.M - 1 - m0) * g.lda + g.K);
    const int a_row = blk * 32 + l32;
    const int a_first = HF > 0 ? kq * 8 * TAPS + lh * 4 : (kq >> 1) * TAPS * HALF_CHANNELS + (kq & 1) * 8 + lh * 4;
    const int a_off = (m0 + a_row < g.M) ? (a_row * g.lda + a_first) * 4 : BUF_OOB;
    auto load_a = [&](int cb, int t) {
        const int k0 = cb * PATCH_CHANNELS * TAPS + t * (HF > 0 ? 8 : HALF_CHANNELS);
        return buffer_load_f32x4(a_base + k0, a_off, records_left(a_elems, (unsigned)k0));
    };

    // where the lane reads in patch number p: in the filters' own order place[p][tap of the first of
    // its 4 k] + channel * PLANE + column; in the re-laid order place[p][0] + the tap's offset + i * PLANE
    constexpr int NPLACE = HF > 0 ? TAPS : 1;
    int place[2][NPLACE], toff[TAPS];
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
        for (int e = 0; e < NPLACE; ++e) {
            if constexpr (HF > 0) place[p][e] = p * PATCH_FLOATS + pix + natural_place<HF, WF>(e, lh, cv.patch_pitch);
            else place[p][e] = p * PATCH_FLOATS + pix;
        }
    if constexpr (HF == 0) {
        int th = 0, tw = 0;
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
            toff[t] = th * cv.patch_pitch + tw;
            if (++tw == cv.Wf) { tw = 0; ++th; }
        }
    }
    const int last_block = cv.Cin / PATCH_CHANNELS - 1;

    pf.load_patch(0);
    f32x4 ring[TAPS];
#pragma unroll
    for (int t = 0; t < TAPS; ++t) ring[t] = load_a(0, t);
    // margins are zero for the whole walk, in both patches
    zero_patch_margins<T::THREADS>(cv, smem, 2 * PATCH_CHANNELS, tid);
    __syncthreads();
    pf.store_patch_to(smem);
    pf.load_patch(min(1, last_block));
    __syncthreads();

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;

    auto read_b = [&](float (&b)[4], auto P, int t) {     // (t is a constant once the taps are unrolled)
        constexpr int p = decltype(P)::value;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (HF > 0) {
                const int k = 8 * t + i, tap = k % TAPS;   // counted from the quarter's first k
                b[i] = smem[place[p][tap] + (k / TAPS) * PATCH_PLANE_FLOATS + tap % WF];
            } else {
                b[i] = smem[place[p][0] + toff[t] + i * PATCH_PLANE_FLOATS];
            }
        }
    };
    // One channel block out of patch P.  With MORE, the filters of the block after it follow their
    // predecessors into the ring, the next block's patch (fetched a block ago) is written into the
    // other patch and the one after that is fetched.
    auto block = [&](int cb, auto P, auto more) {
        constexpr int p = decltype(P)::value;
        constexpr bool MORE = decltype(more)::value;
        float bq[2][4];
        read_b(bq[0], P, 0);
#pragma unroll
        for (int t = 0; t < TAPS; ++t) {
            if (t + 1 < TAPS) read_b(bq[(t + 1) & 1], P, t + 1);
            // (pinned: left to itself the compiler reads each operand right in front of its MFMA and
            // the chain waits out an LDS round trip per pair)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ring[t][i], bq[t & 1][i], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (MORE) {
                ring[t] = load_a(cb + 1, t);
                float* other = smem + (1 - p) * PATCH_FLOATS;
                if (t == 0) { pf.template store_patch_chunk_to<0>(other); pf.template store_patch_chunk_to<1>(other); pf.template store_patch_chunk_to<2>(other); pf.template store_patch_chunk_to<3>(other); }
                if (t == 1) { pf.template store_patch_chunk_to<4>(other); pf.template store_patch_chunk_to<5>(other); pf.template store_patch_chunk_to<6>(other); pf.template store_patch_chunk_to<7>(other); }
                const int fetch = min(cb + 2, last_block);
                if (t == 2) { pf.template load_patch_chunk<0>(fetch); pf.template load_patch_chunk<1>(fetch); pf.template load_patch_chunk<2>(fetch); pf.template load_patch_chunk<3>(fetch); }
                if (t == 3) { pf.template load_patch_chunk<4>(fetch); pf.template load_patch_chunk<5>(fetch); pf.template load_patch_chunk<6>(fetch); pf.template load_patch_chunk<7>(fetch); }
            }
        }
        // the other patch is complete, and nobody reads this one any more
        if constexpr (MORE) __syncthreads();
    };
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    int cb = 0;
    for (; cb + 2 <= last_block; cb += 2) {
        block(cb, P0{}, std::true_type{});
        block(cb + 1, P1{}, std::true_type{});
    }
    if (cb < last_block) {
        block(cb, P0{}, std::true_type{});
        block(cb + 1, P1{}, std::false_type{});
    } else {
        block(cb, P0{}, std::false_type{});
    }

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

// HF x WF: the filter's shape when the kernel is built for one (3 x 3), 0 x 0: any, read from the arguments
template <class T, int HF, int WF>
__global__ void __launch_bounds__(T::THREADS) sgemm_conv_patch_kernel(const GemmArgs g)
{
    static_assert(T::KSPLIT == 1 && T::REG_STAGES == 2 && T::BK == PATCH_CHANNELS && T::TN <= 2, "tile shape");
    using PL = PatchLoader<T, HF * WF>;
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
        patch_tail_subtile<T, 9, HF, WF>(g, smem, w);
        return;
    }
    // K slices are whole channel blocks
    const int kbeg = w.kbeg, kend = w.kend;
    const int block_k = PATCH_CHANNELS * taps;             // k' per channel block: `taps` steps
    const int blocks = (kend - kbeg) / block_k;
    const int cb0 = kbeg / block_k;
    const int last_half = cv.Cin / HALF_CHANNELS - 1;

    // the tile's first pixel fixes which virtual row the patches start at
    const int vrows = cv.Hin + 2 * cv.pad;
    const int g0 = (int)cv.by_row_n.div(n0), img0 = (int)cv.by_hout.div(g0);
    const int v0 = img0 * vrows + (g0 - img0 * cv.Hout);
    // where the lane's pixels (one per 32-column block of the wave) sit in a patch under tap (0, 0);
    // in the re-laid K order the lane's half of an operand group (channels 0..3 or 4..7) is folded in
    int pix[2] = {0, 0};
#pragma unroll
    for (int tn = 0; tn < T::TN; ++tn) {
        int n = n0 + wn0 + tn * 32 + l32;
        if (n >= g.N) n = n0;                              // computed and dropped
        const int gr = (int)cv.by_row_n.div(n), wo = n - gr * cv.row_n;
        const int b = (int)cv.by_hout.div(gr), ho = gr - b * cv.Hout;
        pix[tn] = (b * vrows + ho - v0) * cv.patch_pitch + (4 - cv.pad) + wo + (HF > 0 ? 0 : lh * 4 * PATCH_PLANE_FLOATS);
    }

    f32x16 acc[T::TM][T::TN];
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.f;

    if (blocks > 0) {
        // the rows below the last pixel's window are never read: not fetched either
        const int n_last = min(n0 + T::BN, g.N) - 1;
        const int g_last = (int)cv.by_row_n.div(n_last), img_last = (int)cv.by_hout.div(g_last);
        const int rows_used = img_last * vrows + (g_last - img_last * cv.Hout) - v0 + cv.Hf;
        PL pl;
        pl.init(g, m0, v0, rows_used, tid, patch);
        if constexpr (HF > 0) {
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                for (int tap = 0; tap < HF * WF; ++tap) pl.place[tn][tap] = pix[tn] + natural_place<HF, WF>(tap, lh, cv.patch_pitch);
        }
        // ra[1] holds the stage that the next step stores, at every step that is not the second of a pair
        f32x4 ra[2][T::A_ITERS], rb_unused[T::B_ITERS];
        Frag<T> frag[2];
        // prologue: the first half block's patch, the second one's on its way, the first stage of A
        pl.load_patch(2 * cb0);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[1][it] = pl.load_a(kbeg, pl.a_off[it]);
        // margins are zero for the whole walk, in both patches
        zero_patch_margins<T::THREADS>(cv, patch, PATCH_CHANNELS, tid);
        __syncthreads();
        pl.store_patch_to(patch);
        pl.load_patch(2 * cb0 + 1);
        store_stage_a<T>(As, tid, ra[1]);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[1][it] = pl.load_a(kbeg + T::BK, pl.a_off[it]);
        __syncthreads();
        // operands of the first group: A from stage 0, B from the first patch under the first tap
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
            frag[0].a[tm] = *reinterpret_cast<const f32x4*>(As + a_lane + tm * 32 * T::LDA + lh * 4);
        if constexpr (HF > 0) {
            const PatchStep<T, false, false, false, HF, WF, 0> first{pl, 0, nullptr};
            frag[0].b[0][0] = first.template patch_read<0, false, 0, 0>();
            frag[0].b[0][1] = first.template patch_read<0, false, 0, 1>();
            frag[0].b[0][2] = first.template patch_read<0, false, 0, 2>();
            frag[0].b[0][3] = first.template patch_read<0, false, 0, 3>();
            if constexpr (T::TN > 1) {
                frag[0].b[T::TN - 1][0] = first.template patch_read<0, false, T::TN - 1, 0>();
                frag[0].b[T::TN - 1][1] = first.template patch_read<0, false, T::TN - 1, 1>();
                frag[0].b[T::TN - 1][2] = first.template patch_read<0, false, T::TN - 1, 2>();
                frag[0].b[T::TN - 1][3] = first.template patch_read<0, false, T::TN - 1, 3>();
            }
        } else {
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                for (int i = 0; i < 4; ++i) frag[0].b[tn][i] = patch[i * PATCH_PLANE_FLOATS + pix[tn]];
        }

        // A step is two pairs of operand groups.  In the re-laid order a pair is (half block, tap),
        // and pairs follow each other tap by tap, half block by half block, alternating between
        // the two patches: pair p of a block is tap p % taps of half block p / taps and reads at
        // (p / taps) * HALF_FLOATS + (tap / Wf) * pitch + tap % Wf (off0 for the step's first pair,
        // off1 for its second, off2 for the next step's first).  In the filters' own order the
        // step's loader knows the places itself.
        // One code copy per kind of step and place in the block: two step bodies chosen inside one
        // loop would make the compiler copy the accumulators wherever the bodies' register
        // assignments meet, i.e. after every step.
        int cur = 0, s = 0;
        auto step_with = [&](const auto& loader, f32x4 (&sa)[T::A_ITERS], f32x4 (&fa)[T::A_ITERS], int off0, int off1, int off2) {
            using LD = std::remove_cv_t<std::remove_reference_t<decltype(loader)>>;
            const WalkCtx<T, LD> c{loader, kbeg + (s + 2) * T::BK, kend,
                                   As + cur * T::A_STAGE, patch + off0,
                                   As + (cur ^ 1) * T::A_STAGE, patch + off2,
                                   tid, a_lane, pix[0], lh, sa, rb_unused, fa, rb_unused, pix[T::TN - 1], patch + off1};
            __builtin_amdgcn_sched_barrier(0);
            step_groups<T, LD>(c, frag, acc);
            cur ^= 1;
            ++s;
        };
        // Block cb walks half blocks 2 cb (out of the first patch) and 2 cb + 1 (out of the second).
        // The second one's patch is on its way when the block starts and is written in the block's
        // second step (third, with an even number of taps), which nothing reads before the step
        // after it; the next block's first patch is fetched five steps before the block ends and
        // written three steps before it ends, when the first half block's last tap is two steps or
        // more behind; its second patch is fetched in the last step.  (Half blocks past the last
        // are fetched as the last one again and never used.)
        if constexpr (HF > 0) {
            // The filter's shape is known: the steps of a block are written out, each knowing its
            // number in the block and with it the channel and tap of every k it multiplies; the
            // lanes' read addresses are registers computed once per tile plus immediates -- no
            // address arithmetic between the MFMAs at all.  (Kept up at run time, the places of a
            // step's operand groups cost 40 scalar and 6 vector instructions in front of its first
            // MFMA: 20 us of config 5's 840.)
            constexpr int TAPS = HF * WF;
            static_assert(TAPS >= 7 && TAPS % 2 == 1, "the block's steps are written out for an odd number of taps");
            auto step_at = [&](auto J, auto single, auto fetch, auto store, int hb, float* dst) {
                constexpr int j = decltype(J)::value;
                const PatchStep<T, decltype(single)::value, decltype(fetch)::value, decltype(store)::value, HF, WF, j> loader{pl, hb, dst};
                if constexpr (decltype(single)::value) step_with(loader, ra[1], ra[1], 0, 0, 0);
                else if constexpr (j % 2 == 0) step_with(loader, ra[1], ra[0], 0, 0, 0);
                else step_with(loader, ra[0], ra[1], 0, 0, 0);
            };
            constexpr std::false_type no{};
            constexpr std::true_type yes{};
            auto plain_steps = [&](auto self, auto J, auto END) {
                if constexpr (decltype(J)::value < decltype(END)::value) {
                    step_at(J, no, no, no, 0, nullptr);
                    self(self, std::integral_constant<int, decltype(J)::value + 1>{}, END);
                }
            };
            for (int cb = cb0; cb < cb0 + blocks; ++cb) {
                const int hx = min(2 * cb + 2, last_half), hy = min(2 * cb + 3, last_half);
                step_at(std::integral_constant<int, 0>{}, no, no, no, 0, nullptr);
                step_at(std::integral_constant<int, 1>{}, no, no, yes, 0, patch + HALF_FLOATS);
                plain_steps(plain_steps, std::integral_constant<int, 2>{}, std::integral_constant<int, TAPS - 5>{});
                step_at(std::integral_constant<int, TAPS - 5>{}, no, yes, no, hx, nullptr);
                step_at(std::integral_constant<int, TAPS - 4>{}, no, no, no, 0, nullptr);
                step_at(std::integral_constant<int, TAPS - 3>{}, no, no, yes, 0, patch);
                step_at(std::integral_constant<int, TAPS - 2>{}, no, no, no, 0, nullptr);
                step_at(std::integral_constant<int, TAPS - 1>{}, yes, yes, no, hy, nullptr);
            }
        } else {
            using Plain = PatchStep<T, false, false, false>;
            using Fetch = PatchStep<T, false, true, false>;
            using Store = PatchStep<T, false, false, true>;
            using Single = PatchStep<T, true, false, false>;
            using SingleFetch = PatchStep<T, true, true, false>;
            // `where` is the place in LDS of the pair that the next step starts with
            int th = 0, tw = 0, half = 0, where = 0;
            auto next_pair = [&] {
                if (++tw == cv.Wf) {
                    tw = 0;
                    if (++th == cv.Hf) { th = 0; half ^= 1; }
                }
                where = half * HALF_FLOATS + th * cv.patch_pitch + tw;
                return where;
            };
            auto step_next = [&](const auto& loader, f32x4 (&sa)[T::A_ITERS], f32x4 (&fa)[T::A_ITERS]) {
                const int off0 = where, off1 = next_pair(), off2 = next_pair();
                step_with(loader, sa, fa, off0, off1, off2);
            };
            auto first_of_pair = [&](const auto& loader) { step_next(loader, ra[1], ra[0]); };
            auto second_of_pair = [&](const auto& loader) { step_next(loader, ra[0], ra[1]); };
            auto single = [&](const auto& loader) { step_next(loader, ra[1], ra[1]); };
            const int middle_pairs = (taps - 7) >> 1;
            for (int cb = cb0; cb < cb0 + blocks; ++cb) {
                const int hx = min(2 * cb + 2, last_half), hy = min(2 * cb + 3, last_half);
                if (!(taps & 1)) single(Single{pl, 0, nullptr});
                first_of_pair(Plain{pl, 0, nullptr});
                second_of_pair(Store{pl, 0, patch + HALF_FLOATS});
                for (int i = 0; i < middle_pairs; ++i) {
                    first_of_pair(Plain{pl, 0, nullptr});
                    second_of_pair(Plain{pl, 0, nullptr});
                }
                first_of_pair(Fetch{pl, hx, nullptr});
                second_of_pair(Plain{pl, 0, nullptr});
                first_of_pair(Store{pl, 0, patch});
                second_of_pair(Plain{pl, 0, nullptr});
                single(SingleFetch{pl, hy, nullptr});
            }
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

// Wt[co][(hb * taps + tap) * 16 + c] = W[co][(hb * 16 + c) * taps + tap], zero for channels past Cin
__global__ void __launch_bounds__(256) conv_filter_relayout_kernel(const float* __restrict__ W, float* __restrict__ Wt,
                                                                   int Cout, int Cin, int taps, int kp, int ld)
{
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)Cout * kp) return;
    const int co = (int)(i / kp), k = (int)(i - (size_t)co * kp);
    const int c = k & 15, bt = k >> 4;
    const int hb = bt / taps, tap = bt - hb * taps;
    const int ch = hb * 16 + c;
    Wt[(size_t)co * ld + k] = ch < Cin ? W[((size_t)co * Cin + ch) * taps + tap] : 0.f;
}

}  // namespace

// Rows and row pitch of the patch for this geometry, or false when the kernel does not take it:
// stride 1 only, at least seven taps (the walk fetches and writes its patches at fixed steps of a block), padding of at most 4,
// whole blocks of 32 channels, and a patch plane of at most 512 floats
// (56 x 56 maps under a 3 x 3 filter use all of it; wider images keep the staged-copy path).
bool conv_patch_geometry(int batch, int Cin, int Hin, int Win, int Hf, int Wf, int stride, int pad, int Hout, int Wout,
                         int* rows, int* pitch)
{
    if (stride != 1 || Hf * Wf < 7 || pad > 4 || Cin % 32 != 0) return false;
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

// Floats between the rows of the re-laid filters: an odd number of 128-byte lines.  With an even
// number (config 5: 72) the same k' of 64 consecutive rows, which the sub-tiles of a last round
// load straight into MFMA operands, falls into 8 sets of the vector cache and every load misses.
int conv_patch_lda(int Cin, int Hf, int Wf)
{
    const int kp = conv_patch_k(Cin, Hf, Wf);
    return (kp / 32) % 2 ? kp : kp + 32;
}

bool conv_patch_reads_filters_in_place(int Hf, int Wf) { return Hf == 3 && Wf == 3; }

hipError_t launch_conv_filter_relayout(const float* W, float* Wt, int Cout, int Cin, int Hf, int Wf, hipStream_t stream)
{
    const int kp = conv_patch_k(Cin, Hf, Wf);
    const size_t n = (size_t)Cout * kp;
    hipLaunchKernelGGL(conv_filter_relayout_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, W, Wt, Cout,
                       Cin, Hf * Wf, kp, conv_patch_lda(Cin, Hf, Wf));
    return hipGetLastError();
}

hipError_t launch_sgemm_conv_patch(const GemmArgs& args, int grid, hipStream_t stream)
{
    using T = TilePatch;
    auto any = sgemm_conv_patch_kernel<T, 0, 0>;
    auto k3x3 = sgemm_conv_patch_kernel<T, 3, 3>;
    static const hipError_t attr_any = hipFuncSetAttribute(reinterpret_cast<const void*>(any),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, patch_smem_bytes<T>());
    static const hipError_t attr_3x3 = hipFuncSetAttribute(reinterpret_cast<const void*>(k3x3),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, patch_smem_bytes<T>());
    if (attr_any != hipSuccess) return attr_any;
    if (attr_3x3 != hipSuccess) return attr_3x3;
    if (args.conv.Hf == 3 && args.conv.Wf == 3)
        hipLaunchKernelGGL(k3x3, dim3(grid), dim3(T::THREADS), patch_smem_bytes<T>(), stream, args);
    else
        hipLaunchKernelGGL(any, dim3(grid), dim3(T::THREADS), patch_smem_bytes<T>(), stream, args);
    return hipGetLastError();
}

}  // namespace cake
