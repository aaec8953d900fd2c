// 256 x 128 tiles of a plain product (C overwritten, no bias, row-major operands, K a multiple of
// 4) computed by workgroups that stay: one per CU, walking over (tile, stage of 32 k) units of the
// tile sequence.  The macro-tile kernel spends a workgroup per tile, and with one workgroup per CU
// nothing hides a tile's first loads or its epilogue: about 15 000 cycles per tile next to 8300
// per stage, a fifth of the time at K = 256 and a tenth at K = 512.  Here both operands of a unit
// go straight into LDS (16-byte buffer loads with the LDS bit, two buffers per operand), the loads
// of unit u + 1 are issued when unit u starts -- across tile borders, so a tile has no prologue of
// its own -- and nothing passes through registers on its way in.
//
// LDS: A's stage is 256 rows of 32 floats, unpadded, the 16-byte chunks of a row swizzled (chunk
// c of row r at place c ^ ((r ^ (r >> 3)) & 7)) so that the operand reads of 16 consecutive rows
// hit different banks, whether the LDS serves them 8 or 16 lanes at a time; B's stage is 32 rows of 128 floats, rows whose k has bit 2 set stored with their halves
// of 32 columns exchanged (column n at n ^ 32), because the two halves of a wave read rows k and
// k + 4 of the same columns at once.  Both layouts are made by the choice of which chunk a lane
// asks for: a load instruction fills 1 KB of consecutive LDS, lane by lane.
#include "sgemm_tile.hpp"

namespace cake {

namespace {

constexpr int RES_BM = 256, RES_BN = 128, RES_BK = 32;
constexpr int RES_STG_PITCH = 36;   // floats per row of a wave's staging block (8 rows of 32 columns)

__device__ __forceinline__ void resident_body(const GemmArgs& g, float* const (&Ab)[2], float* const (&Bb)[2], float* Stg)
{
    constexpr int BK = RES_BK, PITCH = RES_STG_PITCH;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // 8 waves, 64 x 64 of C each; in a scalar register, and so is all that follows from it
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
    const int a_swz = (l32 ^ (l32 >> 3)) & 7;   // of the lane's row in the first block row; the second's has bit 2 flipped
    float* stg = Stg + wave * (8 * PITCH);

    const int stages = (g.K + BK - 1) / BK;
    const int tiles_all = g.tiles_m * g.tiles_n;
    // every XCD owns one contiguous run of the tile sequence; its workgroups walk through it side by side
    const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;
    const int first = xcd * (tiles_all >> 3) + min(xcd, tiles_all & 7);
    const int tiles = first + (tiles_all >> 3) + (xcd < (tiles_all & 7) ? 1 : 0);
    const int t0 = first + (blockIdx.x >> 3);
    if (t0 >= tiles) return;

    // A: load instruction q = wave + 8 it (it < 4) fills rows 8 q .. 8 q + 7 of the stage;
    // B: instruction q = wave + 8 it (it < 2) fills rows 2 q and 2 q + 1
    int a_off[4], a_off_last[4], b_off[2];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int q = wave + 8 * it;
        const int r = 8 * q + (lane >> 3), c = (lane & 7) ^ ((r ^ (r >> 3)) & 7);
        a_off[it] = (r * g.lda + c * 4) * 4;
        a_off_last[it] = (stages - 1) * BK + c * 4 < g.K ? a_off[it] : BUF_OOB;
    }
#pragma unroll
    for (int it = 0; it < 2; ++it) {
        const int q = wave + 8 * it;
        const int r = 2 * q + (lane >> 5), c = (lane & 31) ^ (((r >> 2) & 1) << 3);
        b_off[it] = (r * g.ldb + c * 4) * 4;
    }

    struct Place {
        int m0, n0;
        const float* a;
        const float* b;
        unsigned a_elems, b_elems;
    };
    const int fast_n = g.group_along_n ? g.tiles_m : g.tiles_n;
    const int slow_n = g.group_along_n ? g.tiles_n : g.tiles_m;
    auto place = [&](int tile) {
        const int band_sz = g.group * fast_n;
        const int band = (int)g.by_band.div((unsigned)tile), rem = tile - band * band_sz;
        const int slow0 = band * g.group;
        const bool whole_band = slow_n - slow0 >= g.group;
        const int gsz = whole_band ? g.group : slow_n - slow0;
        const int fast = (int)(whole_band ? g.by_group.div((unsigned)rem) : g.by_last_group.div((unsigned)rem));
        const int slow = slow0 + rem - fast * gsz;
        Place p;
        p.m0 = (g.group_along_n ? fast : slow) * RES_BM;
        p.n0 = (g.group_along_n ? slow : fast) * RES_BN;
        p.a = g.A + (size_t)p.m0 * g.lda;
        p.b = g.B + p.n0;
        p.a_elems = clamp_elems((long long)(g.M - 1 - p.m0) * g.lda + g.K);
        p.b_elems = clamp_elems((long long)(g.K - 1) * g.ldb + g.N - p.n0);
        return p;
    };
    // The six load instructions of a unit are not issued in one go: eight waves doing that at the
    // same moment fill the address queue of the memory pipeline and stall behind it with their
    // MFMAs unissued.  begin_produce prepares a unit's loads, load_one issues one of them.
    struct Loads {
        __amdgpu_buffer_rsrc_t ra, rb;
        bool last;
    };
    int tp = t0, kp = 0;
    Place cur = place(t0), pp = cur;
    bool producing = true;
    auto begin_produce = [&]() {
        Loads L;
        const unsigned ka = (unsigned)kp * BK, kb = (unsigned)kp * BK * (unsigned)g.ldb;
        // (past the workgroup's last unit the loads are still issued, with no records: every lane is
        // then out of range, nothing is fetched and zeros go into a stage nobody reads again.  Loads
        // behind a branch cost more than that: the compiler loses track of which LDS array each one
        // fills where the branches join and makes every later LDS read wait for all of them.)
        L.ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(pp.a + ka), 0, producing ? (int)records_left(pp.a_elems, ka) : 0, 0x00020000);
        L.rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(pp.b + kb), 0, producing ? (int)records_left(pp.b_elems, kb) : 0, 0x00020000);
        L.last = kp == stages - 1;
        if (producing && ++kp == stages) {
            kp = 0;
            tp += stride;
            producing = tp < tiles;
            if (producing) pp = place(tp);
        }
        return L;
    };
    auto load_one = [&](const Loads& L, float* Ad, float* Bd, int idx) {   // idx 0..3: A, 4..5: B
        if (idx < 4)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(L.ra, (__attribute__((address_space(3))) void*)(Ad + (wave + 8 * idx) * 256), 16,
                                                     L.last ? a_off_last[idx] : a_off[idx], 0, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(L.rb, (__attribute__((address_space(3))) void*)(Bd + (wave + 8 * (idx - 4)) * 256), 16,
                                                     b_off[idx - 4], 0, 0, 0);
    };
    int t = t0, ks = 0;   // the consumer's position in the unit sequence

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // operands of a group of 8 k: per 32 x 32 block row four k of the lane's row of A (one 16-byte
    // read), per block column the lane's column of B at four k (4-byte reads, two rows per instruction)
    f32x4 fa[2][2];
    float fb[2][2][4];
    // one of the six LDS reads that fetch group kg of a stage: 0, 1: A's block rows; 2..5: two k of a block column of B
    auto fetch_op = [&](const float* Ac, const float* Bc, int kg, int op, f32x4 (&a)[2], float (&b)[2][4]) {
        if (op < 2) {
            a[op] = *reinterpret_cast<const f32x4*>(Ac + (wm0 + 32 * op + l32) * BK + (((kg * 2 + lh) ^ a_swz ^ (4 * op)) * 4));
        } else {
            const int tn = (op - 2) >> 1, i0 = ((op - 2) & 1) * 2;
            const float* src = Bc + (kg * 8 + lh * 4 + i0) * RES_BN + ((wn0 + 32 * tn + l32) ^ (lh << 5));
            b[tn][i0] = src[0];
            b[tn][i0 + 1] = src[RES_BN];
        }
    };
    // The 16 MFMAs of a group with the operands in fa[cur], fb[cur]; between them, one at a time and
    // in a fixed order, the six LDS reads that fetch the next group (from An, Bn at group kg_next)
    // and -- in a unit's last group -- the six loads of the unit after the next.  Every memory
    // operation is pinned to its place: left to itself the compiler moves reads next to the MFMAs
    // that use them, and a wave then waits for LDS with nothing else to issue.
    auto group = [&](int cur, const float* An, const float* Bn, int kg_next, bool with_loads, const Loads& L, float* Ad, float* Bd) {
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) {
            const int i = idx >> 2, tm = (idx >> 1) & 1, tn = idx & 1;
            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][tm][i], fb[cur][tn][i], acc[tm][tn], 0, 0, 0);
            if (!(idx & 1) && (idx >> 1) < 6) {
                fetch_op(An, Bn, kg_next, idx >> 1, fa[cur ^ 1], fb[cur ^ 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (with_loads && (idx & 1) && (idx >> 1) < 6) {
                load_one(L, Ad, Bd, idx >> 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // One unit.  Its first group's operands are in fa[0], fb[0] already.  The barrier sits in front
    // of the LAST group's MFMAs, whose operands are in registers by then: behind it the stage is
    // free for the loads of the unit after the next, the next unit's stage (whose loads were
    // issued a unit ago) is complete, and its first operands are read under those MFMAs (past the
    // workgroup's last unit they are read all the same, and not used).
    // Returns false after the workgroup's last unit.
    auto unit = [&](float* Ac, float* Bc, const float* An, const float* Bn) -> bool {
        // (the scalar work that prepares the loads comes first, in the shadow of the first MFMAs:
        // behind the barrier it would hold up all eight waves at once)
        const Loads L = begin_produce();
        const Loads none{};
        group(0, Ac, Bc, 1, false, none, nullptr, nullptr);
        group(1, Ac, Bc, 2, false, none, nullptr, nullptr);
        group(0, Ac, Bc, 3, false, none, nullptr, nullptr);
        const bool tile_done = ks + 1 == stages;
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the next unit's operands have landed (and the last tile's stores have left)
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        group(1, An, Bn, 0, true, L, Ac, Bc);
        ++ks;
        if (!tile_done) return true;
        // the tile is finished: each 32 x 32 block of the wave, turned around in pieces of 8 rows
        // through the wave's own staging block (no barrier: a wave's LDS operations stay in order)
        const int rd_row = lane >> 3, rd_col = (lane & 7) * 4;
#pragma unroll
        for (int tm = 0; tm < 2; ++tm) {
#pragma unroll
            for (int tn = 0; tn < 2; ++tn) {
                const int row = cur.m0 + wm0 + 32 * tm + rd_row, col = cur.n0 + wn0 + 32 * tn + rd_col;
                float* dst = g.C + (size_t)row * g.ldc + col;
                const int rows = g.M - row, valid = min(4, g.N - col);
                f32x4 v[4];
#pragma unroll
                for (int P = 0; P < 4; ++P) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) stg[(4 * lh + j) * PITCH + l32] = acc[tm][tn][4 * P + j];
                    v[P] = *reinterpret_cast<const f32x4*>(stg + rd_row * PITCH + rd_col);
                    __builtin_amdgcn_sched_barrier(0);
                }
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
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[tm][tn][r] = 0.f;
            }
        }
        ks = 0;
        t += stride;
        if (t >= tiles) return false;
        cur = place(t);
        return true;
    };

    {
        const Loads L0 = begin_produce();
#pragma unroll
        for (int idx = 0; idx < 6; ++idx) load_one(L0, Ab[0], Bb[0], idx);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        const Loads L1 = begin_produce();
#pragma unroll
        for (int idx = 0; idx < 6; ++idx) load_one(L1, Ab[1], Bb[1], idx);
    }
#pragma unroll
    for (int op = 0; op < 6; ++op) fetch_op(Ab[0], Bb[0], 0, op, fa[0], fb[0]);
    for (;;) {
        if (!unit(Ab[0], Bb[0], Ab[1], Bb[1])) break;
        if (!unit(Ab[1], Bb[1], Ab[0], Bb[0])) break;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // no load into LDS outlives the wave
}

// (the LDS arrays are separate objects on purpose: the compiler then knows that operand reads of
// one buffer need not wait for the loads into the other)
__global__ void __launch_bounds__(512) sgemm_resident_kernel(const GemmArgs g)
{
    __shared__ __align__(16) float A0[RES_BM * RES_BK];
    __shared__ __align__(16) float A1[RES_BM * RES_BK];
    __shared__ __align__(16) float B0[RES_BK * RES_BN];
    __shared__ __align__(16) float B1[RES_BK * RES_BN];
    __shared__ __align__(16) float Stg[8 * 8 * RES_STG_PITCH];
    float* const Ab[2] = {A0, A1};
    float* const Bb[2] = {B0, B1};
    resident_body(g, Ab, Bb, Stg);
}

}  // namespace

// Where the walk pays: a plain product on 256 x 128 tiles, two or more of them per CU (with one
// there is nothing to walk to) and a K below 1024.  Measured against the macro-tile kernel on the
// same tiles, one device, us: 8192^2 x 256 273 -> 253, x 384 385 -> 367, x 512 496 -> 483, x 768
// 720 -> 713, x 1024 945 -> 944, x 2048 1844 -> 1861, 8192^3 7190 -> 7340; 4096^2 x 256 78.6 -> 73.5,
// x 512 128.9 -> 125.6; 16384 x 320 x 4096 331 -> 312; 1024 x 192 x 30000 110.5 -> 100.0 -- what
// the walk saves per tile is worth 7 % at K = 256 and nothing at 1024, and beyond that its K loop
// is the slower of the two by 1-2 %.  `forced`: the caller named the tile; then any tile count.
bool resident_applies(int M, int N, int K, int cus, bool plain, bool forced)
{
    if (!plain || K < RES_BK || K >= RESIDENT_MAX_K || K % 4 != 0) return false;
    const long tiles = (long)((M + RES_BM - 1) / RES_BM) * ((N + RES_BN - 1) / RES_BN);
    return forced || tiles >= 2L * cus;
}

int resident_lds_bytes() { return (2 * RES_BM * RES_BK + 2 * RES_BK * RES_BN + 8 * 8 * RES_STG_PITCH) * 4; }

// args: tiles_m, tiles_n, group, group_along_n set for 256 x 128 tiles; split_k = 1, no tail tiles
hipError_t launch_sgemm_resident(const GemmArgs& args, int cus, hipStream_t stream)
{
    const long tiles = (long)args.tiles_m * args.tiles_n;
    if (tiles <= 0) return hipSuccess;
    if (args.split_k != 1 || args.tail_tiles != 0 || args.partial || args.accumulate || args.col_bias || args.K % 4 != 0 ||
        args.tiles_m != (args.M + RES_BM - 1) / RES_BM || args.tiles_n != (args.N + RES_BN - 1) / RES_BN)
        return hipErrorInvalidValue;
    GemmArgs a2 = args;
    const int group = args.group > 0 ? args.group : 1;
    a2.group = group;
    const int fast_n = args.group_along_n ? args.tiles_m : args.tiles_n;
    const int slow_n = args.group_along_n ? args.tiles_n : args.tiles_m;
    const int nbands = (slow_n + group - 1) / group;
    a2.by_band = FastDiv::make((unsigned)(group * fast_n));
    a2.by_group = FastDiv::make((unsigned)group);
    a2.by_last_group = FastDiv::make((unsigned)(slow_n - (nbands - 1) * group));
    const int grid = (int)(((tiles < cus ? tiles : (long)cus) + 7) / 8 * 8);   // whole rows of 8 XCDs, one workgroup per CU
    hipLaunchKernelGGL(sgemm_resident_kernel, dim3(grid), dim3(512), 0, stream, a2);
    return hipGetLastError();
}

}  // namespace cake
