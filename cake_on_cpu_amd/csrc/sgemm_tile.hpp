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

#include <type_traits>

#include "kernels.hpp"

namespace cake {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));  // 16 bytes at any 4-byte address

// REG_STAGES: how many K stages' worth of registers sit between the global loads
// and the LDS stores (the 16-byte loaders only).  With 2, a step's loads go into
// the set the previous step emptied, so they can be issued anywhere in the step,
// for 6-8 more float4 registers per lane.
// STORE_LEAD: how many operand groups (of 8 k) before the step's barrier the
// register -> LDS stores are issued.  1 puts them in the group that ends at the
// barrier; 2 gives them a whole group to land first, which matters when a group
// is only a few MFMAs long and nothing else would cover the wait at the barrier.
// KSPLIT: how many waves share each WM x WN block of C, each taking its own
// BK / KSPLIT slice of every K stage (summed once through LDS after the walk).
// A 32x32 wave tile has only 16 MFMAs per 32 k, too few to hide its own LDS and
// barrier latencies when it is alone on its SIMD; with KSPLIT = 2 every SIMD
// holds two waves of the workgroup even when the grid is one workgroup per CU.
template <int BM_, int BN_, int BK_, int WM_, int WN_, int REG_STAGES_ = 1, int STORE_LEAD_ = 1, int KSPLIT_ = 1>
struct Tile {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
    static constexpr int REG_STAGES = REG_STAGES_;
    static constexpr int STORE_LEAD = STORE_LEAD_;
    static constexpr int KSPLIT = KSPLIT_;
    static constexpr int WAVE_BK = BK / KSPLIT;        // k extent of a stage that one wave multiplies
    static constexpr int WAVES_M = BM / WM, WAVES_N = BN / WN;
    static constexpr int THREADS = WAVES_M * WAVES_N * KSPLIT * 64;
    static constexpr int TM = WM / 32, TN = WN / 32;   // 32x32 MFMA tiles per wave
    static constexpr int LDA = BK + 4;                 // floats; 16-byte reads of 8 consecutive rows hit 8 distinct bank quads
    static constexpr int LDB = BN + 8;                 // floats; rows k and k+4 land 32 banks apart
    static constexpr int A_STAGE = BM * LDA;
    // B as [k][n] rows of LDB floats, or (B handed over as its transpose, VecLoaderNT) as [n][k]
    // rows of LDA floats like A: room for either
    static constexpr int B_STAGE = BK * LDB > BN * LDA ? BK * LDB : BN * LDA;
    static constexpr int LDS_BYTES = 2 * (A_STAGE + B_STAGE) * 4;
    static constexpr int A_CHUNKS = BM * BK / 4;       // 16-byte chunks per stage
    static constexpr int B_CHUNKS = BK * BN / 4;
    static constexpr int A_ITERS = A_CHUNKS / THREADS;
    static constexpr int B_ITERS = B_CHUNKS / THREADS;
    static_assert(BM % WM == 0 && BN % WN == 0 && WM % 32 == 0 && WN % 32 == 0, "wave tiling");
    static_assert(BK % KSPLIT == 0 && WAVE_BK % 8 == 0, "K step is consumed 8 deep");
    static_assert(KSPLIT == 1 || BM * BN * 4 <= LDS_BYTES, "the K halves are summed through the stage memory");
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
__device__ __forceinline__ void raster_tile(const GemmArgs& g, int t, int& tile_m, int& tile_n)
{
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

// Position in a sequence of `count` items of the item that workgroup `wg`
// takes when each XCD is to own one contiguous run of the sequence.
__device__ __forceinline__ int xcd_contiguous(int wg, int count)
{
    const int q = count >> 3, r = count & 7;
    const int xcd = wg & 7, idx = wg >> 3;
    return (xcd < r) ? xcd * (q + 1) + idx : r * (q + 1) + (xcd - r) * q + idx;
}

// Which tile and which K range a workgroup computes.
struct WorkItem {
    int tile_m, tile_n;
    int kbeg, kend;
    int slice;      // K slice number (split-K or tail), 0 otherwise
    int tail_tile;  // >= 0: index among the tail tiles, result goes to tail_partial
};

__device__ __forceinline__ WorkItem decode_tile(const GemmArgs& g, int wg)
{
    const int tiles = g.tiles_m * g.tiles_n;
    const int full = tiles - g.tail_tiles;
    // Whole tiles first, then the (much shorter) tail slices, each set dealt
    // evenly over the XCDs on its own so that every XCD gets the same work.
    const int whole = g.tail_tiles ? full : tiles * g.split_k;
    const int lid = wg < whole ? xcd_contiguous(wg, whole)
                               : whole + xcd_contiguous(wg - whole, g.tail_tiles * g.tail_split);
    WorkItem w;
    int t, per;
    if (g.tail_tiles && lid >= full) {
        const int rr = lid - full;
        w.tail_tile = rr / g.tail_split;
        w.slice = rr - w.tail_tile * g.tail_split;
        t = full + w.tail_tile;
        per = g.tail_k_per_split;
    } else if (g.tail_tiles) {
        w.tail_tile = -1;
        w.slice = 0;
        t = lid;
        per = g.K;
    } else {
        w.tail_tile = -1;
        w.slice = lid / tiles;
        t = lid - w.slice * tiles;
        per = g.k_per_split;
    }
    w.kbeg = w.slice * per;
    w.kend = min(g.K, w.kbeg + per);
    raster_tile(g, t, w.tile_m, w.tile_n);
    return w;
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
        } else {
            if (row < g.M) {
                const float* src = g.A + (size_t)row * g.lda + col;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < kend) v[e] = src[e];
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
        } else {
            if (row < kend) {
                const float* src = g.B + (size_t)row * g.ldb + col;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < g.N) v[e] = src[e];
            }
        }
        rb[it] = v;
    }
}

// registers -> LDS stage
template <class T>
__device__ __forceinline__ void store_b_chunk_along_k(float* Bs, int W, int tid, const f32x4& v);

template <class T>
__device__ __forceinline__ void store_stage_a(float* As, int tid, const f32x4 (&ra)[T::A_ITERS])
{
#pragma unroll
    for (int it = 0; it < T::A_ITERS; ++it) {
        const int c = tid + it * T::THREADS;
        *reinterpret_cast<f32x4*>(As + (c / (T::BK / 4)) * T::LDA + (c % (T::BK / 4)) * 4) = ra[it];
    }
}

template <class T, bool B_ALONG_K = false>
__device__ __forceinline__ void store_stage_b(float* Bs, int tid, const f32x4 (&rb)[T::B_ITERS])
{
#pragma unroll
    for (int it = 0; it < T::B_ITERS; ++it) {
        if constexpr (B_ALONG_K) {
            store_b_chunk_along_k<T>(Bs, it, tid, rb[it]);
        } else {
            const int c = tid + it * T::THREADS;
            *reinterpret_cast<f32x4*>(Bs + (c / (T::BN / 4)) * T::LDB + (c % (T::BN / 4)) * 4) = rb[it];
        }
    }
}

template <class T, bool B_ALONG_K = false>
__device__ __forceinline__ void store_stage(float* As, float* Bs, int tid,
                                            const f32x4 (&ra)[T::A_ITERS],
                                            const f32x4 (&rb)[T::B_ITERS])
{
    store_stage_a<T>(As, tid, ra);
    store_stage_b<T, B_ALONG_K>(Bs, tid, rb);
}

// MFMA operands of one wave for a group of 8 consecutive k.
//
// v_mfma_f32_32x32x2_f32 takes A[i][kk] from lane i + 32*kk and B[kk][j] from
// lane j + 32*kk.  The sum over k does not care which two k meet in one
// instruction as long as A and B agree, so within a group of 8 k the lower 32
// lanes take k = 0..3 and the upper 32 lanes k = 4..7: each lane then fetches
// its four A values with a single 16-byte LDS read.
template <class T>
struct Frag {
    f32x4 a[T::TM];
    float b[T::TN][4];
};

template <class T, bool B_ALONG_K = false>
// a_lane / b_lane: where the lane's operands start inside a stage (floats):
// its row of A (times LDA) and its column of B, plus the wave's K slice of the
// stage when several waves share a block of C.
// B_ALONG_K: the B stage is laid out like A ([n][k], rows of LDA floats) and b_lane is the lane's
// row of it times LDA.
__device__ __forceinline__ void load_frag(const float* As, const float* Bs, int a_lane, int b_lane,
                                          int lh, int kg, Frag<T>& f)
{
    const int kk = kg * 8 + lh * 4;
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
        f.a[tm] = *reinterpret_cast<const f32x4*>(As + a_lane + tm * 32 * T::LDA + kk);
#pragma unroll
    for (int tn = 0; tn < T::TN; ++tn) {
        if constexpr (B_ALONG_K) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(Bs + b_lane + tn * 32 * T::LDA + kk);
#pragma unroll
            for (int i = 0; i < 4; ++i) f.b[tn][i] = v[i];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) f.b[tn][i] = Bs[(kk + i) * T::LDB + b_lane + tn * 32];
        }
    }
}

template <class T>
__device__ __forceinline__ void mma_frag(const Frag<T>& f, f32x16 (&acc)[T::TM][T::TN])
{
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
                acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[tm][i], f.b[tn][i], acc[tm][tn], 0, 0, 0);
}

// ---------------------------------------------------------------------------
// 16-byte loader through buffer instructions.
//
// buffer_load_dwordx4 range-checks the byte offset against the resource's
// num_records and returns zero when it is outside, so an element that must
// read as zero (row >= M, column >= N, k >= kend) is requested at an offset
// past num_records instead of being branched around.  The K walk of a
// workgroup is therefore one straight-line basic block, which is what lets the
// instruction scheduler interleave memory operations with MFMAs.
// The resource is re-based every K step (tile origin + k0), so per-thread
// offsets are constants and stay below 2^31 bytes for lda < 2M, ldb < 16M.
// ---------------------------------------------------------------------------
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

static constexpr unsigned BUF_RECORDS = 0x80000000u;  // every legal offset is below, BUF_OOB is not
static constexpr int BUF_OOB = (int)0x80000000u;

__device__ __forceinline__ f32x4 buffer_load_f32x4(const float* base, int byte_offset,
                                                   unsigned records = BUF_RECORDS)
{
    __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)records, 0x00020000);
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0));
}

// Buffer record count (bytes) for a resource that starts `used` elements into an operand of
// `total` elements: loads are range-checked per 4 bytes, so a 16-byte load that hangs over the
// end of the operand reads zeros there instead of touching memory past the allocation.
// 32-bit scalar arithmetic only: this sits between MFMAs in front of every load.
__device__ __forceinline__ unsigned records_left(unsigned total_elems, unsigned used_elems)
{
    // used > total only happens for stages past K, whose lanes all ask for the out-of-range
    // offset: the difference then wraps to a large count, which is as good as any.  (Written
    // without a saturating subtraction on purpose: that only exists as a vector instruction,
    // and a record count in a vector register makes the compiler loop over the load.)
    return min(total_elems - used_elems, BUF_RECORDS / 4) * 4;
}

// element count as records_left takes it (operands here stay below 2^31 elements; larger counts
// only need to stay "large")
__device__ __forceinline__ unsigned clamp_elems(long long n)
{
    return n <= 0 ? 0u : n > 0xffffffffll ? 0xffffffffu : (unsigned)n;
}

// 4-byte load at base + voffset (per lane) + soffset (same for the wave): the wave-uniform part of
// an address rides in a scalar register and costs no vector ALU work
__device__ __forceinline__ int buffer_load_i32(const int* base, int voffset_bytes, int soffset_bytes)
{
    __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(base), 0, (int)BUF_RECORDS, 0x00020000);
    return __builtin_amdgcn_raw_buffer_load_b32(rsrc, voffset_bytes, soffset_bytes, 0);
}

// Row-major operands through 16-byte buffer loads.  Only 4-byte alignment is
// needed, so any K, N, leading dimension and base address qualify.  A chunk is
// 4 consecutive k of one A row, or 4 consecutive n of one B row:
//  * rows >= M of A, columns >= N of B (whole chunks) and k >= kend read as
//    zero through an out-of-range offset;
//  * an A chunk that straddles kend is loaded whole and its elements past kend
//    are zeroed when the stage is stored to LDS (by then the data has arrived,
//    so the test never waits on memory);
//  * a B chunk that straddles N brings in values of the next row: they only
//    reach columns >= N of the tile, which are never stored;
//  * the record count of each load ends at the operand's last element.
template <class T>
struct VecLoader {
    static constexpr int NUM_LOADS = T::A_ITERS + T::B_ITERS;  // load instructions per stage
    static constexpr bool MASK_A_STORES = true;
    static constexpr bool B_ALONG_K = false;     // a chunk of B is 4 consecutive n of one k
    int a_off[T::A_ITERS];  // byte offset from the A tile origin, or BUF_OOB for rows >= M
    int a_k[T::A_ITERS];    // first k of the chunk inside a stage
    int b_off[T::B_ITERS];  // byte offset from the B tile origin per stage, or BUF_OOB for cols >= N
    int b_k[T::B_ITERS];    // k row of the chunk inside a stage
    const float* a_base;    // A + m0*lda
    const float* b_base;    // B + n0
    unsigned a_elems;       // from a_base to the end of A
    unsigned b_elems;       // from b_base to the end of B
    int ldb;

    __device__ __forceinline__ void init(const GemmArgs& g, int m0, int n0, int tid)
    {
        a_base = g.A + (size_t)m0 * g.lda;
        b_base = g.B + n0;
        ldb = g.ldb;
        a_elems = clamp_elems((long long)(g.M - 1 - m0) * g.lda + g.K);
        b_elems = clamp_elems((long long)(g.K - 1) * g.ldb + g.N - n0);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) {
            const int c = tid + it * T::THREADS;
            const int r = c / (T::BK / 4);
            a_k[it] = (c % (T::BK / 4)) * 4;
            a_off[it] = (m0 + r < g.M) ? (r * g.lda + a_k[it]) * 4 : BUF_OOB;
        }
#pragma unroll
        for (int it = 0; it < T::B_ITERS; ++it) {
            const int c = tid + it * T::THREADS;
            const int col = (c % (T::BN / 4)) * 4;
            b_k[it] = c / (T::BN / 4);
            b_off[it] = (n0 + col < g.N) ? (b_k[it] * g.ldb + col) * 4 : BUF_OOB;
        }
    }

    __device__ __forceinline__ void prime(int) {}  // nothing to fetch ahead

    __device__ __forceinline__ f32x4 load_a(int k0, int off) const
    {
        return buffer_load_f32x4(a_base + k0, off, records_left(a_elems, (unsigned)k0));
    }
    __device__ __forceinline__ f32x4 load_b(int k0, int off) const
    {
        const unsigned skip = (unsigned)k0 * (unsigned)ldb;  // below 2^32: K*ldb < 2^31 and the walk
                                                             // runs a few stages of 32 rows past K
        return buffer_load_f32x4(b_base + skip, off, records_left(b_elems, skip));
    }

    // chunk OP (A chunks first, then B chunks) of a stage that lies wholly below
    // kend: no per-lane test, no vector ALU work
    template <int OP>
    __device__ __forceinline__ void load_one_inside(int k0, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < T::A_ITERS)
            ra[OP] = load_a(k0, a_off[OP]);
        else
            rb[OP - T::A_ITERS] = load_b(k0, b_off[OP - T::A_ITERS]);
    }

    // chunk OP of the stage starting at k0; chunks that start at or past kend read as zero
    template <int OP>
    __device__ __forceinline__ void load_one(int k0, int kend, f32x4 (&ra)[T::A_ITERS],
                                             f32x4 (&rb)[T::B_ITERS]) const
    {
        const int left = kend - k0;
        if constexpr (OP < T::A_ITERS)
            ra[OP] = load_a(k0, a_k[OP] < left ? a_off[OP] : BUF_OOB);
        else
            rb[OP - T::A_ITERS] = load_b(k0, b_k[OP - T::A_ITERS] < left ? b_off[OP - T::A_ITERS] : BUF_OOB);
    }

    __device__ __forceinline__ void load(int k0, int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        load_all<0>(k0, kend, ra, rb);
    }
    // the stage that starts at k = 0, for a kernel whose every stage does (sgemm_shortk.hip)
    __device__ __forceinline__ void load_first_stage(int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        load_all<0>(0, kend, ra, rb);
    }
    // only its B chunks: the A chunks are the previous tile's and already lie in LDS
    __device__ __forceinline__ void load_first_stage_b(int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        load_all<T::A_ITERS>(0, kend, ra, rb);
    }

    template <int OP>
    __device__ __forceinline__ void load_all(int k0, int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < NUM_LOADS) {
            load_one<OP>(k0, kend, ra, rb);
            load_all<OP + 1>(k0, kend, ra, rb);
        }
    }
};

// A chunk W of the stage that starts at k_stage, with the elements at or past kend zeroed.
template <class T>
__device__ __forceinline__ f32x4 a_chunk_below(const f32x4& v, int W, int tid, int k_stage, int kend)
{
    const int valid = kend - k_stage - ((tid + W * T::THREADS) % (T::BK / 4)) * 4;  // elements below kend
    f32x4 r = v;
    if (valid < 4) r[3] = 0.f;
    if (valid < 3) r[2] = 0.f;
    if (valid < 2) r[1] = 0.f;
    if (valid < 1) r[0] = 0.f;
    return r;
}

// B handed over as its transpose: Bt[n][k], rows ldb apart (the weights of a linear layer as
// they lie, y = x . w^T).  Both operands are then read like A: a chunk of B is 4 consecutive k
// of one row n (chunk c: n = c / (BK/4), k = 4 (c % (BK/4))), loaded with one 16-byte load and
// stored to an [n][k] stage of LDS laid out like A's, from which a lane fetches its four B values
// of a group with one 16-byte read.  (Stored as scalars into the [k][n] stage the 8 lanes of a row
// hit 2 banks: measured 5 % slower than the plain kernel at 8192^3 and 40 % at 64 x 16384^2.)
// Rows at and past N read as zero; a chunk that straddles kend is masked when stored.
template <class T>
struct VecLoaderNT {
    static constexpr int NUM_LOADS = T::A_ITERS + T::B_ITERS;
    static constexpr bool MASK_A_STORES = true;
    static constexpr bool B_ALONG_K = true;
    int a_off[T::A_ITERS];
    int a_k[T::A_ITERS];
    int b_off[T::B_ITERS];  // byte offset from the B tile origin, or BUF_OOB for rows >= N
    int b_k[T::B_ITERS];    // first k of the chunk inside a stage
    const float* a_base;    // A + m0*lda
    const float* b_base;    // Bt + n0*ldb
    unsigned a_elems;
    unsigned b_elems;

    __device__ __forceinline__ void init(const GemmArgs& g, int m0, int n0, int tid)
    {
        a_base = g.A + (size_t)m0 * g.lda;
        b_base = g.B + (size_t)n0 * g.ldb;
        a_elems = clamp_elems((long long)(g.M - 1 - m0) * g.lda + g.K);
        b_elems = clamp_elems((long long)(g.N - 1 - n0) * g.ldb + g.K);
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) {
            const int c = tid + it * T::THREADS;
            const int r = c / (T::BK / 4);
            a_k[it] = (c % (T::BK / 4)) * 4;
            a_off[it] = (m0 + r < g.M) ? (r * g.lda + a_k[it]) * 4 : BUF_OOB;
        }
#pragma unroll
        for (int it = 0; it < T::B_ITERS; ++it) {
            const int c = tid + it * T::THREADS;
            const int r = c / (T::BK / 4);
            b_k[it] = (c % (T::BK / 4)) * 4;
            b_off[it] = (n0 + r < g.N) ? (r * g.ldb + b_k[it]) * 4 : BUF_OOB;
        }
    }

    __device__ __forceinline__ void prime(int) {}

    __device__ __forceinline__ f32x4 load_a(int k0, int off) const
    {
        return buffer_load_f32x4(a_base + k0, off, records_left(a_elems, (unsigned)k0));
    }
    __device__ __forceinline__ f32x4 load_b(int k0, int off) const
    {
        return buffer_load_f32x4(b_base + k0, off, records_left(b_elems, (unsigned)k0));
    }

    template <int OP>
    __device__ __forceinline__ void load_one_inside(int k0, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < T::A_ITERS)
            ra[OP] = load_a(k0, a_off[OP]);
        else
            rb[OP - T::A_ITERS] = load_b(k0, b_off[OP - T::A_ITERS]);
    }

    template <int OP>
    __device__ __forceinline__ void load_one(int k0, int kend, f32x4 (&ra)[T::A_ITERS],
                                             f32x4 (&rb)[T::B_ITERS]) const
    {
        const int left = kend - k0;
        if constexpr (OP < T::A_ITERS)
            ra[OP] = load_a(k0, a_k[OP] < left ? a_off[OP] : BUF_OOB);
        else
            rb[OP - T::A_ITERS] = load_b(k0, b_k[OP - T::A_ITERS] < left ? b_off[OP - T::A_ITERS] : BUF_OOB);
    }

    __device__ __forceinline__ void load(int k0, int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        load_all<0>(k0, kend, ra, rb);
    }

    template <int OP>
    __device__ __forceinline__ void load_all(int k0, int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < NUM_LOADS) {
            load_one<OP>(k0, kend, ra, rb);
            load_all<OP + 1>(k0, kend, ra, rb);
        }
    }
};

// chunk number W of a B stage whose chunks run along k (VecLoaderNT): the stage is [n][k], rows of
// LDA floats, exactly like A's
template <class T>
__device__ __forceinline__ void store_b_chunk_along_k(float* Bs, int W, int tid, const f32x4& v)
{
    const int c = tid + W * T::THREADS;
    *reinterpret_cast<f32x4*>(Bs + (c / (T::BK / 4)) * T::LDA + (c % (T::BK / 4)) * 4) = v;
}

__device__ __forceinline__ float buffer_load_f32(const float* base, int byte_offset)
{
    __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, (int)BUF_RECORDS, 0x00020000);
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 0));
}

// A through 16-byte buffer loads as in VecLoader; B = the column matrix of a
// convolution, gathered from a staged copy of the NCHW input ("implicit im2col":
// examples/cake_conv.cpp:1178-1213 without the K x N intermediate).
// The staged input (conv_stage_input_kernel) has its zero padding written out and,
// for a strided convolution, its rows split into column phases, so that every
// window position is inside the copy and the 4 consecutive output pixels of a
// chunk read 4 consecutive floats: a chunk is ONE 16-byte load (4-byte aligned,
// which buffer loads allow).  A thread's chunk is 4 consecutive n at one k; they
// lie in one output row (rows of n are a multiple of 4 long), so one (image, row,
// column) triple per thread serves the whole K walk and only the filter tap
// (c, h, w) of each k changes from stage to stage.
template <class T, bool LINEAR_TAPS = false>
struct ConvRowLoader {
    static constexpr int NUM_LOADS = T::A_ITERS + T::B_ITERS;
    static constexpr bool MASK_A_STORES = true;   // K need not be a multiple of 4 (see VecLoader)
    static constexpr bool B_ALONG_K = false;
    int a_off[T::A_ITERS];
    int a_k[T::A_ITERS];
    int b_k[T::B_ITERS];  // k row of the chunk inside a stage
    int b_k4[T::B_ITERS]; // the same in bytes of the tap table
    const float* a_base;
    unsigned a_elems;     // from a_base to the end of A
    ConvGeom cv;
    int pix4;             // byte offset of the chunk's first pixel under tap (0, 0, 0); BUF_OOB for n >= N
                          // (adding a tap offset, which is below 2^31, keeps it out of range)
    // Byte offset of the filter tap of the chunk's k inside an image, for the
    // stage the NEXT load call fetches.  It comes from a small table in memory,
    // read one stage ahead so that its latency never sits in front of a gather.
    mutable int tap_next[T::B_ITERS];

    __device__ __forceinline__ void init(const GemmArgs& g, int m0, int n0, int tid)
    {
        a_base = g.A + (size_t)m0 * g.lda;
        a_elems = clamp_elems((long long)(g.M - 1 - m0) * g.lda + g.K);
        cv = g.conv;
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) {
            const int c = tid + it * T::THREADS;
            const int r = c / (T::BK / 4);
            a_k[it] = (c % (T::BK / 4)) * 4;
            a_off[it] = (m0 + r < g.M) ? (r * g.lda + a_k[it]) * 4 : BUF_OOB;
        }
#pragma unroll
        for (int it = 0; it < T::B_ITERS; ++it) {
            b_k[it] = (tid + it * T::THREADS) / (T::BN / 4);
            b_k4[it] = b_k[it] * 4;
        }
        static_assert(T::THREADS % (T::BN / 4) == 0, "a thread keeps the same 4 columns in every chunk");
        const int n = n0 + (tid % (T::BN / 4)) * 4;
        const int per_image = cv.Hout * cv.row_n;
        const int b = n / per_image, r = n - b * per_image;
        const int ho = r / cv.row_n, wo = r - ho * cv.row_n;
        pix4 = n < g.N ? (((b * cv.Cin) * cv.plane_rows + ho * cv.row_step) * cv.pitch + wo) * 4 : BUF_OOB;
    }

    __device__ __forceinline__ f32x4 load_a(int k0, int off) const
    {
        return buffer_load_f32x4(a_base + k0, off, records_left(a_elems, (unsigned)k0));
    }

    // before the first load: the stages are then fetched at k0, k0 + BK, k0 + 2 BK, ...
    __device__ __forceinline__ void prime(int k0)
    {
        if constexpr (LINEAR_TAPS) return;   // a 1 x 1 filter: the offset of row k is k * tap_stride
#pragma unroll
        for (int it = 0; it < T::B_ITERS; ++it) tap_next[it] = buffer_load_i32(cv.tap_table, b_k4[it], k0 * 4);
    }

    // byte offset of the window start of chunk `it` at stage k0, or BUF_OOB past the edges
    __device__ __forceinline__ int tap_offset(int it, int k0, int kend) const
    {
        const int k = k0 + b_k[it];
        if constexpr (LINEAR_TAPS) return k < kend ? pix4 + k * cv.tap_stride : BUF_OOB;
        const int off = k < kend ? pix4 + tap_next[it] : BUF_OOB;
        tap_next[it] = buffer_load_i32(cv.tap_table, b_k4[it], (k0 + T::BK) * 4);  // the table has spare entries past K
        return off;
    }

    // the same for a stage that lies wholly below kend
    __device__ __forceinline__ int tap_offset_inside(int it, int k0) const
    {
        if constexpr (LINEAR_TAPS) return pix4 + (k0 + b_k[it]) * cv.tap_stride;
        const int off = pix4 + tap_next[it];
        tap_next[it] = buffer_load_i32(cv.tap_table, b_k4[it], (k0 + T::BK) * 4);
        return off;
    }

    template <int OP>
    __device__ __forceinline__ void load_one(int k0, int kend, f32x4 (&ra)[T::A_ITERS],
                                             f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < T::A_ITERS)
            ra[OP] = load_a(k0, a_k[OP] < kend - k0 ? a_off[OP] : BUF_OOB);
        else
            rb[OP - T::A_ITERS] = buffer_load_f32x4(cv.in, tap_offset(OP - T::A_ITERS, k0, kend), cv.in_bytes);
    }

    template <int OP>
    __device__ __forceinline__ void load_one_inside(int k0, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < T::A_ITERS)
            ra[OP] = load_a(k0, a_off[OP]);
        else
            rb[OP - T::A_ITERS] = buffer_load_f32x4(cv.in, tap_offset_inside(OP - T::A_ITERS, k0), cv.in_bytes);
    }

    __device__ __forceinline__ void load(int k0, int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        load_all<0>(k0, kend, ra, rb);
    }
    template <int OP>
    __device__ __forceinline__ void load_all(int k0, int kend, f32x4 (&ra)[T::A_ITERS], f32x4 (&rb)[T::B_ITERS]) const
    {
        if constexpr (OP < NUM_LOADS) {
            load_one<OP>(k0, kend, ra, rb);
            load_all<OP + 1>(k0, kend, ra, rb);
        }
    }
};

// Where `count` (<= 4) consecutive columns of a convolution's product go, starting at GEMM
// column col (they lie in one output row: rows of n are a multiple of 4 long, and columns at and
// past Wout inside a row are computed but dropped).  Returns how many of them exist; the
// destination of row m is C + m * row_stride + off.
__device__ __forceinline__ int conv_out_map(const ConvGeom& cv, int M, int ldc, int col, int count,
                                            size_t& off, size_t& row_stride)
{
    const int row_id = col / cv.row_n, wo = col - row_id * cv.row_n;
    if (cv.out_nchw) {
        const int b = row_id / cv.Hout, ho = row_id - b * cv.Hout, HW = cv.Hout * cv.Wout;
        off = (size_t)b * M * HW + ho * cv.Wout + wo;
        row_stride = HW;
    } else {
        off = (size_t)row_id * cv.Wout + wo;
        row_stride = ldc;
    }
    return min(count, cv.Wout - wo);
}

// K walk for 16-byte-loadable operands.
//
// Per K step a wave issues 4*TM*TN*NKG MFMAs and a few dozen memory
// instructions.  Two waves share a SIMD and run the same code in lockstep, so
// memory instructions issued in a block stall BOTH waves' matrix work; spread
// between MFMAs they ride in the shadow of the 64-cycle matrix instruction
// instead.  Each group of 8 k is therefore cut into slots of a few MFMAs plus
// ONE memory instruction, and __builtin_amdgcn_sched_barrier(0) after every
// slot keeps the compiler from regrouping them.  With NKG = WAVE_BK/8 groups:
//     groups 0..    : LDS reads of the next group's operands
//     group NKG-2   : ... + registers (stage s+1) -> the other LDS buffer
//     ---- the step's one barrier ----
//     group NKG-1   : LDS reads of the NEXT step's first operand group
//                     + the global loads of stage s+2 into the registers just
//                     freed, which gives every load NKG-1 groups to complete
// The barrier sits before the last group on purpose: the last group's operands
// are already in registers, so its MFMAs keep the matrix pipe busy while the
// first operands of the new stage come in from LDS, instead of the pipe
// draining after every barrier.  (By then nobody reads the current buffer any
// more, and it is only overwritten a whole step later.)
// Loaders whose B operand is not staged per K step: B is read from patches of the convolution's
// input that stay in LDS for a whole block of channels (sgemm_conv_patch.hip).  Such a loader
// declares PATCH_PLANE, the distance in floats between the planes of two consecutive k of an
// operand group.  A stage is then two pairs of groups, each pair 16 channels under one filter tap
// with a place of its own in LDS (WalkCtx::Bc for groups 0 and 1, Bc2 for groups 2 and 3).  The
// loader may declare PATCH_STORES: the step then writes that many 16-byte chunks of a fetched
// patch to LDS between the MFMAs of its last group, i.e. behind its barrier, into a place that
// nobody reads before the next step's barrier.
template <class L, class = void>
struct patch_plane : std::integral_constant<int, 0> {};
template <class L>
struct patch_plane<L, std::void_t<decltype(L::PATCH_PLANE)>> : std::integral_constant<int, L::PATCH_PLANE> {};
// EARLY_LOADS: that many more load instructions (numbered after the stage's own) go into the
// step's first operand group, so that what they fetch is there when the patch is swapped.
template <class L, class = void>
struct early_loads : std::integral_constant<int, 0> {};
template <class L>
struct early_loads<L, std::void_t<decltype(L::EARLY_LOADS)>> : std::integral_constant<int, L::EARLY_LOADS> {};
// SINGLE_STAGE: the step keeps to one register stage (its loads follow its stores) although the
// tile has two.
template <class L, class = void>
struct single_stage : std::false_type {};
template <class L>
struct single_stage<L, std::void_t<decltype(L::SINGLE_STAGE)>> : std::bool_constant<L::SINGLE_STAGE> {};
// READS_PATCH_ITSELF: the loader knows where each operand of a group lies in its patches
// (patch_read<group, wrap, column block, i>()) and the step's Bc, Bc2 and Bn are not used.
template <class L, class = void>
struct reads_patch_itself : std::false_type {};
template <class L>
struct reads_patch_itself<L, std::void_t<decltype(L::READS_PATCH_ITSELF)>> : std::bool_constant<L::READS_PATCH_ITSELF> {};
template <class L, class = void>
struct patch_stores : std::integral_constant<int, 0> {};
template <class L>
struct patch_stores<L, std::void_t<decltype(L::PATCH_STORES)>> : std::integral_constant<int, L::PATCH_STORES> {};

template <class T, class L>
struct Slots {
    static constexpr int NKG = T::WAVE_BK / 8;      // operand groups of 8 k a wave walks per stage
    static constexpr int MFMA_PER_KG = 4 * T::TM * T::TN;
    static constexpr int FRAG_OPS = T::TM + (L::B_ALONG_K ? 1 : 4) * T::TN;   // LDS reads that fill one Frag
    static constexpr int LOAD_OPS = L::NUM_LOADS;               // global load instructions per stage
    static constexpr int PLANE = patch_plane<L>::value;         // > 0: B comes from a resident patch
    static constexpr int STORE_OPS = T::A_ITERS + (PLANE ? 0 : T::B_ITERS);   // 16-byte LDS stores per stage
    static constexpr int STORE_KG = NKG - 1 - T::STORE_LEAD;
    static_assert(STORE_KG >= 0, "stores must follow the previous step's barrier");
    static_assert(NKG >= 3, "the walk needs three operand groups per K step");
    // With two register stages the loads of a step fill the set that the PREVIOUS
    // step stored, so they can go anywhere in the step and are dealt evenly over
    // its groups: issued in one burst by all the waves at once they queue up at
    // the memory pipe and hold back the MFMAs behind them.  With one register
    // stage they have to follow the step's own stores.
    static constexpr bool SPREAD_LOADS = T::REG_STAGES >= 2 && !single_stage<L>::value;
    static constexpr int EARLY = early_loads<L>::value;
    // the stage's own loads in group kg, and which of the stage's loads the first of them is
    static constexpr int own_begin(int kg) { return SPREAD_LOADS ? kg * LOAD_OPS / NKG : 0; }
    static constexpr int own_in(int kg)
    {
        return SPREAD_LOADS ? (kg + 1) * LOAD_OPS / NKG - kg * LOAD_OPS / NKG : (kg == NKG - 1 ? LOAD_OPS : 0);
    }
    static constexpr int loads_in(int kg) { return own_in(kg) + (kg == 0 ? EARLY : 0); }
    // number (as the loader counts them) of load j of group kg: the early ones follow the stage's own
    static constexpr int load_index(int kg, int j) { return j < own_in(kg) ? own_begin(kg) + j : LOAD_OPS + j - own_in(kg); }
    static constexpr int stage_stores_in(int kg) { return kg == STORE_KG ? STORE_OPS : 0; }
    static constexpr int patch_stores_in(int kg) { return kg == NKG - 1 ? patch_stores<L>::value : 0; }
    // memory instructions riding in group kg: operand reads, then loads, then stores
    static constexpr int ops(int kg) { return FRAG_OPS + loads_in(kg) + stage_stores_in(kg) + patch_stores_in(kg); }
};

// A loader seen through this wrapper fetches stages that lie wholly below kend,
// which takes the per-lane "k < kend" tests (compares and selects between the
// MFMAs) out of the bulk of the K walk.
template <class L>
struct InsideStages {
    static constexpr int NUM_LOADS = L::NUM_LOADS;
    static constexpr bool MASK_A_STORES = false;
    static constexpr bool B_ALONG_K = L::B_ALONG_K;
    const L& ld;
    template <int OP, class RA, class RB>
    __device__ __forceinline__ void load_one(int k0, int /*kend*/, RA& ra, RB& rb) const
    {
        ld.template load_one_inside<OP>(k0, ra, rb);
    }
};

// Everything a slot needs, so the recursive templates below stay readable.
template <class T, class L>
struct WalkCtx {
    const L& ld;
    int k_next, kend;
    const float* Ac;
    const float* Bc;
    float* An;
    float* Bn;
    int tid, a_lane, b_lane, lh;
    f32x4 (&ra)[T::A_ITERS];  // register stage that this step stores to LDS
    f32x4 (&rb)[T::B_ITERS];
    f32x4 (&la)[T::A_ITERS];  // register stage that this step's global loads fill
    f32x4 (&lb)[T::B_ITERS];
    int b_lane2 = 0;          // patch loaders: where the lane's second column block starts (b_lane: the first)
    const float* Bc2 = nullptr;   // patch loaders: where the stage's groups 2 and 3 read (Bc: groups 0 and 1)
};

// Memory instruction number OP of group KG (compile-time indices, so every
// register array access is static).
template <class T, class L, int KG, int OP>
__device__ __forceinline__ void slot_op(const WalkCtx<T, L>& c, Frag<T>& next)
{
    using S = Slots<T, L>;
    constexpr int N_FRAG = S::FRAG_OPS;
    constexpr int N_LOAD = S::loads_in(KG);
    if constexpr (OP < N_FRAG) {
        // operands of the next group; the last group reads group 0 of the next stage
        constexpr bool wrap = (KG + 1 == S::NKG);
        const float* A = wrap ? c.An : c.Ac;
        const float* B = wrap ? c.Bn : c.Bc;
        const int kk = (wrap ? 0 : KG + 1) * 8 + c.lh * 4;
        if constexpr (OP < T::TM) {
            next.a[OP] = *reinterpret_cast<const f32x4*>(A + c.a_lane + OP * 32 * T::LDA + kk);
        } else if constexpr (L::B_ALONG_K) {
            constexpr int tn = OP - T::TM;
            const f32x4 v = *reinterpret_cast<const f32x4*>(B + c.b_lane + tn * 32 * T::LDA + kk);
#pragma unroll
            for (int i = 0; i < 4; ++i) next.b[tn][i] = v[i];
        } else if constexpr (S::PLANE > 0) {
            // k = plane of the patch; the lane's half (k 0..3 or 4..7 of the group) is part of b_lane
            constexpr int tn = (OP - T::TM) / 4, i = (OP - T::TM) % 4;
            static_assert(T::TN <= 2 && S::NKG == 4, "two column blocks per wave at most, two pairs of groups per stage");
            constexpr int ng = wrap ? 0 : KG + 1;          // the group these operands belong to
            if constexpr (reads_patch_itself<L>::value) {
                next.b[tn][i] = c.ld.template patch_read<ng, wrap, tn, i>();
            } else {
                const float* P = wrap ? c.Bn : (ng < 2 ? c.Bc : c.Bc2);
                next.b[tn][i] = P[((ng & 1) * 8 + i) * S::PLANE + (tn == 0 ? c.b_lane : c.b_lane2)];
            }
        } else {
            constexpr int tn = (OP - T::TM) / 4, i = (OP - T::TM) % 4;
            next.b[tn][i] = B[(kk + i) * T::LDB + c.b_lane + tn * 32];
        }
    } else if constexpr (OP < N_FRAG + N_LOAD) {
        c.ld.template load_one<S::load_index(KG, OP - N_FRAG)>(c.k_next, c.kend, c.la, c.lb);
    } else if constexpr (OP >= N_FRAG + N_LOAD + S::stage_stores_in(KG)) {
        c.ld.template store_patch_chunk<OP - N_FRAG - N_LOAD - S::stage_stores_in(KG)>();
    } else {
        constexpr int W = OP - N_FRAG - N_LOAD;  // store number W of the stage
        if constexpr (W < T::A_ITERS) {
            const int ch = c.tid + W * T::THREADS;
            f32x4 v = c.ra[W];
            // the stage stored here starts one K step before the one being fetched
            if constexpr (L::MASK_A_STORES) v = a_chunk_below<T>(v, W, c.tid, c.k_next - T::BK, c.kend);
            *reinterpret_cast<f32x4*>(c.An + (ch / (T::BK / 4)) * T::LDA + (ch % (T::BK / 4)) * 4) = v;
        } else {
            if constexpr (L::B_ALONG_K) {
                f32x4 v = c.rb[W - T::A_ITERS];
                // same chunk geometry as A: the k tail is zeroed here
                if constexpr (L::MASK_A_STORES) v = a_chunk_below<T>(v, W - T::A_ITERS, c.tid, c.k_next - T::BK, c.kend);
                store_b_chunk_along_k<T>(c.Bn, W - T::A_ITERS, c.tid, v);
            } else {
                const int ch = c.tid + (W - T::A_ITERS) * T::THREADS;
                *reinterpret_cast<f32x4*>(c.Bn + (ch / (T::BN / 4)) * T::LDB + (ch % (T::BN / 4)) * 4) = c.rb[W - T::A_ITERS];
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);
}

// Memory instruction OP of group KG is issued after MFMA number slot_of(OP)
// of the group (0 = before the first): the ops are spread evenly over it.
template <class T, class L, int KG>
constexpr int slot_of(int op)
{
    return ((op + 1) * Slots<T, L>::MFMA_PER_KG) / (Slots<T, L>::ops(KG) + 1);
}

template <class T, class L, int KG, int SLOT, int OP = 0>
__device__ __forceinline__ void issue_ops_of_slot(const WalkCtx<T, L>& c, Frag<T>& next)
{
    if constexpr (OP < Slots<T, L>::ops(KG)) {
        if constexpr (slot_of<T, L, KG>(OP) == SLOT) slot_op<T, L, KG, OP>(c, next);
        if constexpr (slot_of<T, L, KG>(OP) <= SLOT) issue_ops_of_slot<T, L, KG, SLOT, OP + 1>(c, next);
    }
}

template <class T, class L, int KG, int IDX = 0>
__device__ __forceinline__ void mfma_group(const WalkCtx<T, L>& c, const Frag<T>& f, Frag<T>& next,
                                           f32x16 (&acc)[T::TM][T::TN])
{
    if constexpr (IDX == 0) issue_ops_of_slot<T, L, KG, 0>(c, next);
    if constexpr (IDX < Slots<T, L>::MFMA_PER_KG) {
        constexpr int i = IDX / (T::TM * T::TN), tm = (IDX / T::TN) % T::TM, tn = IDX % T::TN;
        acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[tm][i], f.b[tn][i], acc[tm][tn], 0, 0, 0);
        issue_ops_of_slot<T, L, KG, IDX + 1>(c, next);
        mfma_group<T, L, KG, IDX + 1>(c, f, next, acc);
    }
}

template <class T, class L, int KG = 0>
__device__ __forceinline__ void step_groups(const WalkCtx<T, L>& c, Frag<T> (&frag)[2],
                                            f32x16 (&acc)[T::TM][T::TN])
{
    if constexpr (KG < Slots<T, L>::NKG) {
        if constexpr (KG == Slots<T, L>::NKG - 1) {
            __syncthreads();  // every wave has stored its share of the next stage
            __builtin_amdgcn_sched_barrier(0);
        }
        mfma_group<T, L, KG>(c, frag[KG & 1], frag[(KG + 1) & 1], acc);
        __builtin_amdgcn_sched_barrier(0);
        step_groups<T, L, KG + 1>(c, frag, acc);
    }
}

template <class T, class L>
__device__ __forceinline__ void k_walk_vec(const GemmArgs& g, float* As, float* Bs, int m0, int n0,
                                           int kbeg, int kend, int steps, int tid, int a_lane,
                                           int b_lane, int lh, f32x16 (&acc)[T::TM][T::TN])
{
    static_assert(Slots<T, L>::NKG % 2 == 0, "operand double buffer must come back to slot 0 every step");
    constexpr int RS = T::REG_STAGES;
    static_assert(RS == 1 || RS == 2, "one or two register stages");
    L ld;
    ld.init(g, m0, n0, tid);
    ld.prime(kbeg);
    f32x4 ra[RS][T::A_ITERS], rb[RS][T::B_ITERS];
    Frag<T> frag[2];
    if (steps <= 0) return;
    ld.load(kbeg, kend, ra[0], rb[0]);
    if constexpr (L::MASK_A_STORES) {
#pragma unroll
        for (int it = 0; it < T::A_ITERS; ++it) ra[0][it] = a_chunk_below<T>(ra[0][it], it, tid, kbeg, kend);
        if constexpr (L::B_ALONG_K) {
#pragma unroll
            for (int it = 0; it < T::B_ITERS; ++it) rb[0][it] = a_chunk_below<T>(rb[0][it], it, tid, kbeg, kend);
        }
    }
    store_stage<T, L::B_ALONG_K>(As, Bs, tid, ra[0], rb[0]);
    ld.load(kbeg + T::BK, kend, ra[1 % RS], rb[1 % RS]);
    __syncthreads();
    load_frag<T, L::B_ALONG_K>(As, Bs, a_lane, b_lane, lh, 0, frag[0]);

    // One K step s: stage s is in LDS, stage s+1 waits in registers.  The step
    // stores stage s+1 to the other LDS buffer and fetches stage s+2 -- with two
    // register stages into the set the previous step emptied, with one into the
    // set it has just stored.  Stages past the end are fetched as zeros and parked
    // in the idle buffer, so the walk has no branch.
    int cur = 0;
    const InsideStages<L> inside{ld};
    auto step_with = [&](const auto& loader, int s, f32x4 (&sa)[T::A_ITERS], f32x4 (&sb)[T::B_ITERS],
                         f32x4 (&fa)[T::A_ITERS], f32x4 (&fb)[T::B_ITERS]) {
        using LD = std::remove_cv_t<std::remove_reference_t<decltype(loader)>>;
        const WalkCtx<T, LD> c{loader, kbeg + (s + 2) * T::BK, kend,
                               As + cur * T::A_STAGE, Bs + cur * T::B_STAGE,
                               As + (cur ^ 1) * T::A_STAGE, Bs + (cur ^ 1) * T::B_STAGE,
                               tid, a_lane, b_lane, lh, sa, sb, fa, fb};
        __builtin_amdgcn_sched_barrier(0);
        step_groups<T, LD>(c, frag, acc);
        cur ^= 1;
    };
    // steps 0 .. bulk-1 fetch stages s+2 that end at or below kend
    const int bulk = min(steps, max(0, (kend - kbeg) / T::BK - 2));
    if constexpr (RS == 1) {
        int s = 0;
        for (; s < bulk; ++s) step_with(inside, s, ra[0], rb[0], ra[0], rb[0]);
        for (; s < steps; ++s) step_with(ld, s, ra[0], rb[0], ra[0], rb[0]);
    } else {
        int s = 0;
        for (; s + 1 < bulk; s += 2) {
            step_with(inside, s, ra[1], rb[1], ra[0], rb[0]);
            step_with(inside, s + 1, ra[0], rb[0], ra[1], rb[1]);
        }
        for (; s + 1 < steps; s += 2) {
            step_with(ld, s, ra[1], rb[1], ra[0], rb[0]);
            step_with(ld, s + 1, ra[0], rb[0], ra[1], rb[1]);
        }
        if (s < steps) step_with(ld, s, ra[1], rb[1], ra[0], rb[0]);
    }
}

// K walk for operands that need per-element addressing (any alignment, or the
// K far beyond the 16-byte loader.s reach).  Same double-buffered pipeline with the loads of
// the next stage issued first; correctness path, not tuned.
template <class T, int A_MODE, int B_MODE>
__device__ __forceinline__ void k_walk_generic(const GemmArgs& g, float* As, float* Bs, int m0, int n0,
                                               int kbeg, int kend, int steps, int tid, int a_lane,
                                               int b_lane, int lh, f32x16 (&acc)[T::TM][T::TN])
{
    constexpr int NKG = T::WAVE_BK / 8;
    f32x4 ra[T::A_ITERS], rb[T::B_ITERS];
    Frag<T> frag[2];
    if (steps > 0) {
        load_a_stage<T, A_MODE>(g, m0, kbeg, kend, tid, ra);
        load_b_stage<T, B_MODE>(g, n0, kbeg, kend, tid, rb);
        store_stage<T>(As, Bs, tid, ra, rb);
    }
    __syncthreads();
    if (steps > 0) load_frag<T>(As, Bs, a_lane, b_lane, lh, 0, frag[0]);

    int cur = 0;
    for (int s = 0; s < steps; ++s) {
        const bool more = s + 1 < steps;
        const float* Ac = As + cur * T::A_STAGE;
        const float* Bc = Bs + cur * T::B_STAGE;
        if (more) {
            const int k0 = kbeg + (s + 1) * T::BK;
            load_a_stage<T, A_MODE>(g, m0, k0, kend, tid, ra);
            load_b_stage<T, B_MODE>(g, n0, k0, kend, tid, rb);
        }
#pragma unroll
        for (int kg = 0; kg < NKG; ++kg) {
            if (kg + 1 < NKG) load_frag<T>(Ac, Bc, a_lane, b_lane, lh, kg + 1, frag[(kg + 1) & 1]);
            if (kg == NKG - 1 && more)
                store_stage<T>(As + (cur ^ 1) * T::A_STAGE, Bs + (cur ^ 1) * T::B_STAGE, tid, ra, rb);
            mma_frag<T>(frag[kg & 1], acc);
        }
        __syncthreads();
        cur ^= 1;
        if (more) load_frag<T>(As + cur * T::A_STAGE, Bs + cur * T::B_STAGE, a_lane, b_lane, lh, 0, frag[0]);
    }
}

// Epilogue of one macro-tile: the accumulators of every wave go to C (or to the tile's split-K
// slice), through the stage memory, which nobody may be reading any more after the barrier at
// the start.  PLAIN: the caller knows that C is overwritten and no bias is added, so the epilogue
// holds no load at all (a load here would make a kernel that has other loads in flight wait for
// all of them: the counter of outstanding loads is served in order).
// STREAM_OUT: when the caller's geometry says so (ConvGeom::stream_out), whole 16-byte pieces at
// 16-byte-aligned addresses leave with non-temporal stores.
template <class T, int B_MODE, bool PLAIN = false, bool STREAM_OUT = false>
__device__ __forceinline__ void store_c_tile(const GemmArgs& g, float* smem, const f32x16 (&acc)[T::TM][T::TN],
                                             int m0, int n0, int slice, int wblk, int wm0, int wn0, int lane,
                                             int l32, int lh)
{
    float* out = g.partial ? g.partial + (size_t)slice * g.M * g.N : g.C;
    const int ldo = g.partial ? g.N : g.ldc;
    const bool add = !PLAIN && (g.partial == nullptr) && g.accumulate;
    const float* bias = !PLAIN && g.partial == nullptr ? g.col_bias : nullptr;  // split-K adds it in the reduce
    // a convolution's columns n = (image, output row, column of a row padded to 4) go to
    // [M][batch*Hout*Wout] or NCHW: see conv_out_map
    // (LOAD_VEC4_NCHW: the product on an explicit column matrix writes NCHW itself)
    const bool conv_out = (B_MODE == LOAD_IM2COL_ROW || B_MODE == LOAD_IM2COL_1X1 || B_MODE == LOAD_VEC4_NCHW) &&
                          g.partial == nullptr;
    // The accumulators hold columns of C across lanes (one column per lane, 4 rows per
    // register group).  Each wave turns its block around through LDS, 32 rows at a time, so
    // that a lane owns 4 consecutive columns of a row and C moves in 16-byte pieces: a
    // quarter of the store instructions, and rows written in runs of WN floats.
    constexpr int PITCH = T::WN + 4;            // floats between rows of the wave's staging block
    constexpr int CH = T::WN / 4;               // 16-byte pieces per row
    constexpr int ROWS = 64 / CH;               // rows one wave-wide 16-byte read covers
    static_assert(T::WAVES_M * T::WAVES_N * 32 * PITCH * 4 <= T::LDS_BYTES, "staging blocks fit the stage memory");
    __syncthreads();  // nobody reads operand stages any more
    float* wbuf = smem + wblk * (32 * PITCH);
    const int rd_row = lane / CH, rd_col = (lane % CH) * 4;
    const int col = n0 + wn0 + rd_col;          // first of the lane's 4 columns
    size_t col_off = col;
    size_t row_stride = ldo;
    int valid = min(4, g.N - col);              // how many of the 4 columns exist (<= 0: none)
    if (conv_out && valid > 0) valid = conv_out_map(g.conv, g.M, g.ldc, col, valid, col_off, row_stride);
    f32x4 bias_v = {0.f, 0.f, 0.f, 0.f};
    if (bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < valid) bias_v[e] = bias[col + e];
    }
    const bool whole = valid == 4;
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm) {
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                wbuf[(8 * (r >> 2) + 4 * lh + (r & 3)) * PITCH + tn * 32 + l32] = acc[tm][tn][r];
        // LDS serves a wave's requests in order, so the reads below see the writes above.  All of
        // them are issued before the first store: behind the stores' branches each read would wait
        // out its own latency.
        f32x4 turned[32 / ROWS];
#pragma unroll
        for (int pass = 0; pass < 32 / ROWS; ++pass)
            turned[pass] = *reinterpret_cast<const f32x4*>(wbuf + (pass * ROWS + rd_row) * PITCH + rd_col);
#pragma unroll
        for (int pass = 0; pass < 32 / ROWS; ++pass) {
            const int lr = pass * ROWS + rd_row;
            const int row = m0 + wm0 + tm * 32 + lr;
            f32x4 v = turned[pass];
            if (row < g.M && valid > 0) {
                float* dst = out + (size_t)row * row_stride + col_off;
                if (whole) {
                    f32x4_u* d4 = reinterpret_cast<f32x4_u*>(dst);
                    if (add) v += *d4;
                    if (bias) v += bias_v;
                    if (STREAM_OUT && g.conv.stream_out && (reinterpret_cast<uintptr_t>(dst) & 15) == 0)
                        __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dst));
                    else
                        *d4 = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (e < valid) {
                            float x = add ? dst[e] + v[e] : v[e];
                            if (bias) x += bias_v[e];
                            dst[e] = x;
                        }
                }
            }
        }
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
    // waves that share a block of C sit WAVES_M * WAVES_N apart, i.e. on the same SIMD
    const int ks = wave / (T::WAVES_M * T::WAVES_N);
    const int wblk = wave % (T::WAVES_M * T::WAVES_N);
    const int wm0 = (wblk / T::WAVES_N) * T::WM;
    const int wn0 = (wblk % T::WAVES_N) * T::WN;
    const int a_lane = (wm0 + l32) * T::LDA + ks * T::WAVE_BK;
    const int b_lane = B_MODE == LOAD_VEC4_T ? (wn0 + l32) * T::LDA + ks * T::WAVE_BK
                                             : wn0 + l32 + ks * T::WAVE_BK * T::LDB;

    const WorkItem w = decode_tile(g, blockIdx.x);
    const int m0 = w.tile_m * T::BM, n0 = w.tile_n * T::BN;
    const int kbeg = w.kbeg, kend = w.kend;
    const int steps = (kend - kbeg + T::BK - 1) / T::BK;

    f32x16 acc[T::TM][T::TN];
#pragma unroll
    for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
        for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.f;

    if constexpr (A_MODE == LOAD_VEC4 && (B_MODE == LOAD_VEC4 || B_MODE == LOAD_VEC4_NCHW))
        k_walk_vec<T, VecLoader<T>>(g, As, Bs, m0, n0, kbeg, kend, steps, tid, a_lane, b_lane, lh, acc);
    else if constexpr (A_MODE == LOAD_VEC4 && B_MODE == LOAD_IM2COL_ROW)
        k_walk_vec<T, ConvRowLoader<T>>(g, As, Bs, m0, n0, kbeg, kend, steps, tid, a_lane, b_lane, lh, acc);
    else if constexpr (A_MODE == LOAD_VEC4 && B_MODE == LOAD_IM2COL_1X1)
        k_walk_vec<T, ConvRowLoader<T, true>>(g, As, Bs, m0, n0, kbeg, kend, steps, tid, a_lane, b_lane, lh, acc);
    else if constexpr (A_MODE == LOAD_VEC4 && B_MODE == LOAD_VEC4_T)
        k_walk_vec<T, VecLoaderNT<T>>(g, As, Bs, m0, n0, kbeg, kend, steps, tid, a_lane, b_lane, lh, acc);
    else
        k_walk_generic<T, A_MODE, B_MODE>(g, As, Bs, m0, n0, kbeg, kend, steps, tid, a_lane, b_lane, lh, acc);

    // Accumulator register r of a 32x32 tile holds row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
    if constexpr (T::KSPLIT > 1) {
        // sum the K slices of each block of C in slice order, through the stage memory
        static_assert(T::KSPLIT == 2, "two waves per block of C");
        __syncthreads();  // nobody reads operands any more
        float* red = smem + ((wm0 + 4 * lh) * T::BN + wn0 + l32);
        if (ks == 1) {
#pragma unroll
            for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
                for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        red[(tm * 32 + 8 * (r >> 2) + (r & 3)) * T::BN + tn * 32] = acc[tm][tn][r];
        }
        __syncthreads();
        if (ks == 1) return;
#pragma unroll
        for (int tm = 0; tm < T::TM; ++tm)
#pragma unroll
            for (int tn = 0; tn < T::TN; ++tn)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    acc[tm][tn][r] += red[(tm * 32 + 8 * (r >> 2) + (r & 3)) * T::BN + tn * 32];
    }

    // Epilogue.
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
    store_c_tile<T, B_MODE>(g, smem, acc, m0, n0, w.slice, wblk, wm0, wn0, lane, l32, lh);
}

// C tile = (accumulate ? C : 0) + sum over the K slices of a tail tile, in
// ascending slice order.  grid = (tail tiles, 1024-element chunks of a tile);
// each thread sums 4 consecutive elements of a tile row.
template <class T>
__global__ void __launch_bounds__(256) tail_reduce_kernel(const GemmArgs g)
{
    static_assert(T::BN % 4 == 0 && (T::BM * T::BN) % 1024 == 0, "tile is cut into float4 chunks");
    const int j = blockIdx.x;
    int tile_m, tile_n;
    raster_tile(g, g.tiles_m * g.tiles_n - g.tail_tiles + j, tile_m, tile_n);
    const int e = (blockIdx.y * 256 + threadIdx.x) * 4;
    const int r = e / T::BN, c = e - r * T::BN;
    const int row = tile_m * T::BM + r, col = tile_n * T::BN + c;
    if (row >= g.M || col >= g.N) return;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const float* src = g.tail_partial + (size_t)j * (T::BM * T::BN) + e;
    const size_t slice_stride = (size_t)g.tail_tiles * (T::BM * T::BN);
    float* dst = g.C + (size_t)row * g.ldc + col;
    int valid = min(4, g.N - col);
    if (g.conv.in) {
        size_t off, row_stride;
        valid = conv_out_map(g.conv, g.M, g.ldc, col, valid, off, row_stride);
        dst = g.C + (size_t)row * row_stride + off;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
        if (g.accumulate && q < valid) acc[q] = dst[q];
    for (int s = 0; s < g.tail_split; ++s) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(src + s * slice_stride);
        acc += v;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
        if (q < valid) dst[q] = g.col_bias ? acc[q] + g.col_bias[col + q] : acc[q];
}

template <class T, int A_MODE, int B_MODE>
inline hipError_t launch_tile(const GemmArgs& args, int grid, hipStream_t stream)
{
    auto kern = sgemm_tile_kernel<T, A_MODE, B_MODE>;
    // once per instantiation; the initialiser of a function-local static runs once even when
    // several host threads launch at the same time
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS_BYTES);
    if (attr != hipSuccess) return attr;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::THREADS), T::LDS_BYTES, stream, args);
    return hipGetLastError();
}

using Tile256x256x32 = Tile<256, 256, 32, 128, 64>;
using Tile256x128x32 = Tile<256, 128, 32, 64, 64, 2>;
using Tile128x256x32 = Tile<128, 256, 32, 64, 64, 2>;
using Tile128x128x32 = Tile<128, 128, 32, 64, 64, 2>;
using Tile64x64x32 = Tile<64, 64, 32, 32, 32, 2, 2>;
using Tile64x64x64 = Tile<64, 64, 64, 32, 32, 2, 2, 2>;
using Tile96x128x32 = Tile<96, 128, 32, 96, 32, 2>;
using Tile128x32x32 = Tile<128, 32, 32, 32, 32, 2>;
using Tile32x128x32 = Tile<32, 128, 32, 32, 32, 2>;

}  // namespace cake
