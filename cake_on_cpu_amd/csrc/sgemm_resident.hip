// 256 x 128 tiles of a plain product (C overwritten, no bias, row-major operands, K and N
// multiples of 4) computed by workgroups that stay: one per CU, walking over (tile, stage of 32 k)
// units of the tile sequence.  The macro-tile kernel spends a workgroup per tile, and with one
// workgroup per CU nothing hides a tile's first loads or its epilogue: about 5.6 us per tile next
// to 3.56 us per stage, a fifth of the time at K = 256 and a tenth at K = 512.  Here
//   * both operands of a unit go straight into LDS (16-byte buffer loads with the LDS bit, two
//     stages per operand); the loads of the unit after the next are issued behind this unit's
//     barrier, across tile borders, so a tile has no prologue of its own;
//   * a finished tile's accumulators move to a second set and are written out between the MFMAs
//     of the next tile's first unit, so a tile has no epilogue of its own either;
//   * every memory operation has a fixed place between two MFMAs, one at a time: eight waves
//     issuing their loads in one go fill the address queue of the memory pipeline and stall
//     behind it, and reads left to the compiler's scheduler end up next to the MFMAs that use them.
// What is left per tile is 1.8 us, and a stage takes 3.62 us: ahead of the macro-tile kernel below
// K = 1024, level there, 2 % behind at 8192 (resident_applies).
//
// LDS: A's stage is 256 rows of 32 floats, unpadded, the 16-byte chunks of a row swizzled (chunk
// c of row r at place c ^ ((r ^ (r >> 3)) & 7)) so that the operand reads of 16 consecutive rows
// hit different banks, whether the LDS serves them 8 or 16 lanes at a time; B's stage is 32 rows
// of 128 floats, rows whose k has bit 2 set stored with their halves of 32 columns exchanged
// (column n at n ^ 32), because the two halves of a wave read rows k and k + 4 of the same columns
// at once.  Both layouts are made by the choice of which chunk a lane asks for: a load
// instruction fills 1 KB of consecutive LDS, lane by lane.
#include "sgemm_tile.hpp"

namespace cake {

namespace {

constexpr int RES_BM = 256, RES_BN = 128, RES_BK = 32;
constexpr int RES_STG_PITCH = 36;   // floats per row of a wave's staging block (8 rows of 32 columns)

// Every LDS read in here is an instruction written out by hand, with the wait that goes with it.
// The compiler cannot tell which LDS array a pending load from memory fills once control flow has
// joined (a load behind a branch was enough), and then makes every later LDS read wait for all
// loads in flight -- the next unit's operands.  Reads it does not see cannot be made to wait; the
// stages can then be addressed by numbers that move from a stage to its twin every unit, so there
// is one copy of a unit's code per kind of unit (a tile's first, with and without a finished tile
// to write out, and the others) instead of one per stage as well.
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ unsigned lds_address(const float* p)
{
    return (unsigned)(__UINTPTR_TYPE__)(__attribute__((address_space(3))) const float*)p;
}

__device__ __forceinline__ void resident_body(const GemmArgs& g, float* lds)
{
    constexpr int BK = RES_BK, PITCH = RES_STG_PITCH;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // 8 waves, 64 x 64 of C each
    const int l32 = lane & 31, lh = lane >> 5;
    const int wm0 = (wave >> 1) * 64, wn0 = (wave & 1) * 64;
    float* stg = lds + (98304 / 4) + wave * (8 * PITCH);   // behind the four stages
    const unsigned lds0 = lds_address(lds);

    const int stages = (g.K + BK - 1) / BK;
    const int tiles_all = g.tiles_m * g.tiles_n;
    const int xcd = blockIdx.x & 7, stride = gridDim.x >> 3;
    const int first = xcd * (tiles_all >> 3) + min(xcd, tiles_all & 7);
    const int tiles = first + (tiles_all >> 3) + (xcd < (tiles_all & 7) ? 1 : 0);
    const int t0 = first + (blockIdx.x >> 3);
    if (t0 >= tiles) return;

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

    // LDS (one array, laid out here): A's two stages at 0 and 32 KB, B's at 64 and 80 KB, the staging
    // blocks behind them.  Every regular vector instruction in the loop costs the matrix pipe
    // about four cycles (nothing is issued beside an MFMA on this hardware), so the reads carry
    // their offsets within a stage as immediates, a lane's read addresses move from a stage to
    // its twin with one addition each per unit, and the loop computes no other addresses.
    constexpr int A_TWIN = 32768, B_AT = 65536, B_TWIN = 16384;
    unsigned a_to_twin = lds0 + A_TWIN, b_to_twin = lds0 + B_AT + B_TWIN;   // the stage that is not being multiplied (scalar: where loads go)
    int a_step = A_TWIN, b_step = B_TWIN;                                     // from the stage being multiplied to its twin

    struct Loads {
        __amdgpu_buffer_rsrc_t ra, rb;
        bool last;
    };
    int tp = t0, kp = 0;
    Place cur = place(t0), pp = cur;
    bool producing = true;
    // (past the workgroup's last unit the loads are still issued, with no records: every lane is
    // then out of range, nothing is fetched and zeros go into a stage nobody reads again)
    auto begin_produce = [&]() {
        Loads L;
        const unsigned ka = (unsigned)kp * BK, kb = (unsigned)kp * BK * (unsigned)g.ldb;
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
    // one of a unit's six loads into the stage at LDS addresses a_to, b_to: idx 0..3 A, 4..5 B
    auto load_one = [&](const Loads& L, unsigned a_to, unsigned b_to, int idx) {
        if (idx < 4)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(L.ra, (__attribute__((address_space(3))) void*)(__UINTPTR_TYPE__)(a_to + (wave + 8 * idx) * 1024), 16,
                                                     L.last ? a_off_last[idx] : a_off[idx], 0, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(L.rb, (__attribute__((address_space(3))) void*)(__UINTPTR_TYPE__)(b_to + (wave + 8 * (idx - 4)) * 1024), 16,
                                                     b_off[idx - 4], 0, 0, 0);
    };

    // the tile being multiplied (a tile's first MFMAs start from zero) and the finished one on its way out
    f32x16 acc[2][2], fin[2][2];

    // operands of a group of 8 k: fa[set][block row] four k of the lane's row of A, fb[set][block column][pair] two k of the lane's column of B
    f32x4 fa[2][2];
    f32x2 fb[2][2][2];
    // The lane's read addresses in the stage being multiplied.  A: chunk 2 kg + lh of its row sits
    // at place (2 kg + lh) ^ swz, and in the second block row (32 rows = 4 KB further) at that
    // place with bit 2 flipped, which is the first block row's place for group kg ^ 2: four
    // addresses, one per group.  B: the lane's column in either block column, at the first of its
    // four k of group 0; further k and groups are whole rows further (512 bytes each).
    unsigned a_rd[4], b_rd[2];
    {
        const unsigned swz = (unsigned)((l32 ^ (l32 >> 3)) & 7);
#pragma unroll
        for (int kg = 0; kg < 4; ++kg) a_rd[kg] = lds0 + (unsigned)((wm0 + l32) * BK * 4) + ((((unsigned)(kg * 2 + lh)) ^ swz) << 4);
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) b_rd[tn] = lds0 + B_AT + (unsigned)((lh * 4 * RES_BN + ((wn0 + 32 * tn + l32) ^ (lh << 5))) * 4);
    }
    auto swap_stages = [&]() {
#pragma unroll
        for (int kg = 0; kg < 4; ++kg) a_rd[kg] += a_step;
        b_rd[0] += b_step;
        b_rd[1] += b_step;
        a_to_twin -= a_step;
        b_to_twin -= b_step;
        a_step = -a_step;
        b_step = -b_step;
    };
    // one of the six LDS reads that fetch group kg of a stage -- 0, 1: A's block rows; 2..5: two k
    // of a block column of B -- of the stage being multiplied
#define RES_READ_B(ROW2)                                                                                   \
    asm volatile("ds_read2st64_b32 %0, %1 offset0:" #ROW2 " offset1:" #ROW2 "+2" : "=v"(b[tn][pair]) : "v"(at) : "memory")
    auto fetch_op = [&](int kg, int op, f32x4 (&a)[2], f32x2 (&b)[2][2]) {
        if (op < 2) {
            const unsigned at = a_rd[kg ^ (2 * op)];
            if (op == 0) asm volatile("ds_read_b128 %0, %1" : "=v"(a[0]) : "v"(at) : "memory");
            else asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(a[1]) : "v"(at) : "memory");
        } else {
            const int tn = (op - 2) >> 1, pair = (op - 2) & 1;
            const unsigned at = b_rd[tn];
            switch (kg * 2 + pair) {   // rows 8 kg + 2 pair and the next, in units of half rows (64 dwords)
            case 0: RES_READ_B(0); break;
            case 1: RES_READ_B(4); break;
            case 2: RES_READ_B(16); break;
            case 3: RES_READ_B(20); break;
            case 4: RES_READ_B(32); break;
            case 5: RES_READ_B(36); break;
            case 6: RES_READ_B(48); break;
            default: RES_READ_B(52); break;
            }
        }
    };
#undef RES_READ_B
    // all reads issued so far have returned; the operands of `set` are tied to it, so that no MFMA is placed in front
    auto fetched = [&](int set) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(fa[set][0]), "+v"(fa[set][1]), "+v"(fb[set][0][0]), "+v"(fb[set][0][1]), "+v"(fb[set][1][0]), "+v"(fb[set][1][1])
                     :
                     : "memory");
    };

    // The finished tile is stored through a buffer resource that starts at its first element and
    // ends with C: rows past M fall out of range by themselves, lanes whose columns lie past N get
    // an offset that is out of range, and what is left of a piece's address is a scalar.
    __amdgpu_buffer_rsrc_t fin_rsrc = __builtin_amdgcn_make_buffer_rsrc(g.C, 0, 0, 0x00020000);
    const int rd_row = lane >> 3, rd_col = (lane & 7) * 4;
    const int c_lane = (rd_row * g.ldc + rd_col) * 4;   // bytes from a piece's first element to the lane's 16 bytes
    int c_off[2] = {BUF_OOB, BUF_OOB};                  // the same, or out of range: per block column of the finished tile
    const unsigned stg_read = lds_address(stg + rd_row * PITCH + rd_col);
    f32x4 piece[3];
    auto piece_turn = [&](int q) {   // q = 0..15: block row q / 8, block column (q / 4) % 2, rows 8 (q % 4) ..
        const int tm = q >> 3, tn = (q >> 2) & 1, P = q & 3;
#pragma unroll
        for (int j = 0; j < 4; ++j) stg[(4 * lh + j) * PITCH + l32] = fin[tm][tn][4 * P + j];
        asm volatile("ds_read_b128 %0, %1" : "=v"(piece[q % 3]) : "v"(stg_read) : "memory");
    };
    // in_step: three or more LDS operations were issued behind the piece's read (the next piece's
    // turn), so it has returned once at most three are outstanding; otherwise everything is waited for
    auto piece_store = [&](int q, bool in_step) {
        const int tm = q >> 3, tn = (q >> 2) & 1, P = q & 3;
        if (in_step) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(piece[q % 3]) : : "memory");
        else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(piece[q % 3]) : : "memory");
        const int at = ((wm0 + 32 * tm + 8 * P) * g.ldc + wn0 + 32 * tn) * 4;   // scalar
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, piece[q % 3]), fin_rsrc, c_off[tn], at, 0);
    };

    // The 16 MFMAs of a group with the operands in set `cur_set`; between them, one at a time and in
    // a fixed order, the six LDS reads that fetch the next group (group kg_next of the stage being
    // multiplied) into the other set and, in a unit's last group, the six loads of the unit after
    // the next.  fresh: the first MFMA of each block starts from zero (a tile's first group).
    // drain = 1: the finished tile's 16 pieces, one turned behind every MFMA and stored two MFMAs
    // later; drain = 2: the last two stores of that.
    auto group = [&](int cur_set, int kg_next, bool with_loads, const Loads& L, bool fresh, int drain) {
        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int idx = 0; idx < 16; ++idx) {
            const int i = idx >> 2, tm = (idx >> 1) & 1, tn = idx & 1;
            acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur_set][tm][i], fb[cur_set][tn][i >> 1][i & 1],
                                                               fresh && idx < 4 ? zero : acc[tm][tn], 0, 0, 0);
            if (drain == 1 && idx >= 2) {
                piece_store(idx - 2, true);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (drain == 2 && idx < 2) {
                piece_store(14 + idx, false);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (!(idx & 1) && (idx >> 1) < 6) {
                fetch_op(kg_next, idx >> 1, fa[cur_set ^ 1], fb[cur_set ^ 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (with_loads && (idx & 1) && (idx >> 1) < 6) {
                load_one(L, a_to_twin, b_to_twin, idx >> 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (drain == 1) {
                piece_turn(idx);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // One unit; its first group's operands are in set 0.  The barrier sits in front of the LAST
    // group's MFMAs, whose operands are in registers by then: behind it the stage is free for the
    // loads of the unit after the next, the next unit's stage (whose loads were issued a unit ago)
    // is complete, and its first operands are read under those MFMAs (past the workgroup's last
    // unit they are read all the same, and not used).  fresh: a tile's first unit; drain: a
    // finished tile is waiting in `fin` and is written out under the first group.
    auto unit = [&](bool fresh, bool drain) {
        const Loads L = begin_produce();
        const Loads none{};
        fetched(0);
        __builtin_amdgcn_sched_barrier(0);
        group(0, 1, false, none, fresh, drain ? 1 : 0);
        fetched(1);
        __builtin_amdgcn_sched_barrier(0);
        group(1, 2, false, none, false, drain ? 2 : 0);
        fetched(0);
        __builtin_amdgcn_sched_barrier(0);
        group(0, 3, false, none, false, 0);
        fetched(1);                           // and with that every read of this stage
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the next unit's operands have landed (and a finished tile's stores have left)
        __syncthreads();
        swap_stages();                        // the next unit's stage is the one being multiplied from here on, this unit's the twin that loads fill
        __builtin_amdgcn_sched_barrier(0);
        group(1, 0, true, L, false, 0);
    };
    auto finish_tile = [&]() {
#pragma unroll
        for (int tm = 0; tm < 2; ++tm)
#pragma unroll
            for (int tn = 0; tn < 2; ++tn) fin[tm][tn] = acc[tm][tn];   // (the next tile's first MFMAs start from zero)
        fin_rsrc = __builtin_amdgcn_make_buffer_rsrc(g.C + (size_t)cur.m0 * g.ldc + cur.n0, 0,
                                                     (int)records_left(clamp_elems((long long)(g.M - 1 - cur.m0) * g.ldc + g.N - cur.n0), 0u), 0x00020000);
#pragma unroll
        for (int tn = 0; tn < 2; ++tn) c_off[tn] = cur.n0 + wn0 + 32 * tn + rd_col < g.N ? c_lane : BUF_OOB;
    };

    {
        const Loads L0 = begin_produce();
#pragma unroll
        for (int idx = 0; idx < 6; ++idx) load_one(L0, lds0, lds0 + B_AT, idx);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        const Loads L1 = begin_produce();
#pragma unroll
        for (int idx = 0; idx < 6; ++idx) load_one(L1, a_to_twin, b_to_twin, idx);
    }
#pragma unroll
    for (int op = 0; op < 6; ++op) fetch_op(0, op, fa[0], fb[0]);
    // the first tile: nothing to write out yet
    unit(true, false);
    for (int ks = 1; ks < stages; ++ks) unit(false, false);
    int t = t0;
    for (;;) {
        finish_tile();
        t += stride;
        if (t >= tiles) break;
        cur = place(t);
        unit(true, true);
        for (int ks = 1; ks < stages; ++ks) unit(false, false);
    }
    // the workgroup's last tile
#pragma unroll
    for (int q = 0; q < 16; ++q) {
        piece_turn(q);
        piece_store(q, false);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);   // no load into LDS outlives the wave
}

// 105 KB of LDS, 192 registers: one workgroup of 8 waves per CU
__global__ void __launch_bounds__(512) sgemm_resident_kernel(const GemmArgs g)
{
    __shared__ __align__(16) float lds[2 * RES_BM * RES_BK + 2 * RES_BK * RES_BN + 8 * 8 * RES_STG_PITCH];
    resident_body(g, lds);
}

}  // namespace

// Where the walk pays: a plain product on 256 x 128 tiles, two or more of them per CU (with one
// there is nothing to walk to) and a K below 1024.  Measured against the macro-tile kernel on the
// same tiles, one device, us: 8192^2 x 256 272.7 -> 246.4, x 512 498.0 -> 476.7, x 768 724.0 ->
// 708.0, x 1020 956.2 -> 941.3, x 1024 947 -> 939, x 1536 1392 -> 1401, x 2048 1841 -> 1862, 8192^3
// 7223 -> 7391; 4096^2 x 256 76.3 -> 71.8, x 512 129.0 -> 124.5; 16384 x 320 x 4096 330.4 -> 306.1;
// 1024 x 192 x 30000 110.0 -> 96.5 (the same bits everywhere: both sum k in order) -- what the walk
// saves per tile is worth 10 % at K = 256 and nothing at 1024, and beyond that its K loop is the
// slower of the two by 2 %.  `forced`: the caller named the tile; then any tile count.
bool resident_applies(int M, int N, int K, int cus, bool plain, bool forced)
{
    if (!plain || K < RES_BK || K >= RESIDENT_MAX_K || K % 4 != 0 || N % 4 != 0) return false;   // (16-byte chunks of C's rows end with the row)
    const long tiles = (long)((M + RES_BM - 1) / RES_BM) * ((N + RES_BN - 1) / RES_BN);
    return forced || tiles >= 2L * cus;
}

// A short K (32 to 160) under very many tiles, where the 64 x 64 walks of sgemm_shortk.hip apply:
// this kernel's larger tiles win when K is whole stages (those kernels multiply only the groups
// of 8 k that exist, this one whole stages of 32), the tiles fill their rounds and the matrix to
// 90 %, and there are three rounds or more -- two from K = 96 on.  Measured, same device and run,
// us 64 x 64 walk -> this kernel: 8192^2 x 32 59.1 -> 53.5, x 64 91.3 -> 85.3, x 96 128.1 -> 109.3,
// x 128 163.5 -> 136.5, x 160 192.9 -> 163.8; 12288^2 x 64 206.1 -> 182.4; 16384^2 x 64 365.3 -> 326.2;
// 4096 x 16384 x 96 129.3 -> 113.2; 3072 x 8192 x 128 62.0 -> 55.7; 7000 x 9000 x 64 87.8 -> 80.5;
// 4096^2 x 128 41.7 -> 39.7 (two rounds); against it: 8192^2 x 48 75.3 -> 81.9 (a stage half
// empty), 5120^2 x 64 35.6 -> 40.8 (3.1 rounds cost 4), 4096^2 x 64 27.9 -> 28.2 and x 32 18.4 ->
// 19.6 (two rounds), 256 x 100352 x 64 36.9 -> 42.2 (3.06 rounds), 2048^2 x 64 9.7 -> 13.8.
bool resident_beats_shortk(int M, int N, int K, int cus)
{
    if (K < RES_BK || K > SHORTK_MAX_K || K % RES_BK != 0 || N % 4 != 0) return false;
    const long tiles_m = (M + RES_BM - 1) / RES_BM, tiles_n = (N + RES_BN - 1) / RES_BN, tiles = tiles_m * tiles_n;
    const long rounds = (tiles + cus - 1) / cus;
    if (10 * tiles < 9 * rounds * cus) return false;                                           // the rounds filled to 90 %
    if (10.0 * M * N < 9.0 * (double)(tiles_m * RES_BM) * (double)(tiles_n * RES_BN)) return false;   // and the tiles
    return tiles >= 3L * cus || (K >= 96 && tiles >= 2L * cus);
}

int resident_lds_bytes() { return (2 * RES_BM * RES_BK + 2 * RES_BK * RES_BN + 8 * 8 * RES_STG_PITCH) * 4; }

// args: tiles_m, tiles_n, group, group_along_n set for 256 x 128 tiles; split_k = 1, no tail tiles
hipError_t launch_sgemm_resident(const GemmArgs& args, int cus, hipStream_t stream)
{
    const long tiles = (long)args.tiles_m * args.tiles_n;
    if (tiles <= 0) return hipSuccess;
    if (args.split_k != 1 || args.tail_tiles != 0 || args.partial || args.accumulate || args.col_bias || args.K % 4 != 0 || args.N % 4 != 0 ||
        (double)RES_BM * args.ldc * 4.0 >= 2147483648.0 ||
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
