// planner.cpp -- see planner.hpp.
#include "planner.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "kernels.hpp"

namespace cake {

namespace {

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Fraction of a CU's MFMA peak a workgroup of this shape sustains in the
// middle of a long K walk (measured on MI355X; larger tiles amortise the
// stage loads and the barrier over more matrix work).
double tile_efficiency(int tile_id)
{
    switch (tile_id) {
        case TILE_256x256x32_W128x64: return 0.925;  // one register stage: no room for a second
        case TILE_256x128x32_W64x64: return 0.94;
        case TILE_128x256x32_W64x64: return 0.94;
        case TILE_128x128x32_W64x64: return 0.93;
        case TILE_96x128x32_W96x32: return 0.86;  // 0.90 on a long K walk (192 x 16384^2); rated lower so that it is taken where it
                                                  // saves a quarter of padded rows, not for 512 rows as 6 x 96 (measured 68 against 60 us)
        case TILE_32x128x32_W32x32:
        case TILE_128x32x32_W32x32: return 0.82;  // as the 64 x 64 tile per MFMA; rated below it so that it is taken where it saves padded columns
        case TILE_64x64x32_W32x32: return 0.85;  // one wave per SIMD per workgroup, 16 MFMAs between barriers
        default: return 0.80;  // 64x64x64 with two waves per block of C: see model_seconds
    }
}

struct Candidate {
    int tile_id, split;
    double seconds;
};

// Tail splitting: when the tiles do not fill the last round of the machine, the
// leftover tiles are cut along K so that the last round is short instead of
// thin.  Returns the slice count for `rem` leftover tiles (1 = leave them whole).
int tail_split_for(int rem, int ksteps, const DeviceModel& dev)
{
    if (rem <= 0 || rem > dev.cus / 2) return 1;
    // (up to 16 slices: 16 leftover tiles of 256 x 100352 x 2304 in 16 slices take 815 us in all, in 8 slices 825 us)
    int split = std::min({16, dev.cus / rem, ksteps / 4});
    return split >= 2 ? split : 1;
}

// Workgroups of this tile that a CU holds at the same time (LDS and wave slots).
int resident_per_cu(const TileInfo& t, const DeviceModel& dev)
{
    return std::max(1, std::min(dev.lds_per_cu / t.lds_bytes, 2048 / t.threads));
}

// Tiles left over when every CU has had the same number of them, when they are few enough (at
// most half a CU's worth) to be worth cutting along K; 0 otherwise.  Counted per CU, not per
// resident slot: workgroups that share a CU share its matrix pipes, so what sets the time is how
// many tiles the fullest CU has, however many of them it holds at once (128 x 25088 x 1152 on
// 64 x 64 tiles, 784 = 3 x 256 + 16: 63.5 us with the 16 cut, 72.1 us with the 784 counted as
// less than one round of 1024 slots; 681 x 1544 x 1187: 30.0 against 38.5 us).
int thin_tail_tiles(int tiles, const DeviceModel& dev)
{
    const int rem = tiles % dev.cus;
    return tiles > dev.cus && rem > 0 && rem <= dev.cus / 2 ? rem : 0;
}

// Modelled seconds of one workgroup's K walk with a CU to itself.
double tile_seconds(int M, int N, int K, int tile_id, int split, const DeviceModel& dev)
{
    const TileInfo& t = tile_info(tile_id);
    const int tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
    const long wgs = (long)tiles * split;
    const int ksteps = ceil_div(ceil_div(K, split), t.bk);
    const double extra = 64.0 / t.bk;  // prologue and epilogue cost about as much as 64 k of the walk
    const double wg_flops = 2.0 * t.bm * t.bn * t.bk * (ksteps + extra);
    double eff = tile_efficiency(tile_id);
    // The K-split 64x64 tile pays off when the grid leaves a CU with a single workgroup: its two
    // waves per SIMD hide each other's latencies.  With more workgroups than that the plain
    // 64x64 tile does the same with half the LDS, so four of them share a CU.
    // (measured, 512 x 25088 x 256, 3136 workgroups: 70 us against 59 us), so there it is kept out of the way --
    // unless the K walk is long enough to carry the final sum of the K halves through LDS (32 steps
    // and more; measured 512 x 11008 x 4096: 336 us against 364 us, 512 x 14336 x 4096: 432 against 443).
    if (tile_id == TILE_64x64x64_W32x32) eff = wgs <= dev.cus ? 0.88 : (ksteps >= 32 ? 0.87 : 0.75);
    // The 96 x 128 tile with two workgroups on every CU and a long K walk does as well as the
    // 128 x 128 tile (3000^3: 386 us, where 256 x 128 with its thin last round takes 417 us;
    // 4352 x 4096 x 1024: 270 against 290 us).
    if (tile_id == TILE_96x128x32_W96x32 && wgs >= 2 * dev.cus && ksteps >= 32) eff = 0.93;
    return wg_flops / (dev.mfma_flops / dev.cus * eff);
}

// What the second kernel of a tail split costs (its launch, the gap in front of it, the slices
// written and read back): cutting the leftover tiles has to save more than that.
constexpr double TAIL_SPLIT_SECONDS = 8e-6;

// Slices for the leftover tiles of a thin last round, 1 when cutting them does not pay
// (1024 x 6272 x 256 on 64 x 64 tiles, 1568 = 6 x 256 + 32 with 5 us per tile: 33.2 us whole,
// 36.4 us with the 32 cut; 128 x 25088 x 1152, 13 us per tile: 71.8 whole, 61.3 us cut).
int tail_split_that_pays(int M, int N, int K, int tile_id, const DeviceModel& dev)
{
    const TileInfo& t = tile_info(tile_id);
    const int tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
    const int ksteps = ceil_div(K, t.bk);
    const int tt = thin_tail_tiles(tiles, dev);
    const int ts = tt ? tail_split_for(tt, ksteps, dev) : 1;
    if (ts <= 1) return 1;
    const double extra = 64.0 / t.bk;
    const double saved = (1.0 - (ceil_div(ksteps, ts) + extra) / (ksteps + extra)) * tile_seconds(M, N, K, tile_id, 1, dev);
    return saved > TAIL_SPLIT_SECONDS ? ts : 1;
}

// K slices for the 128 x 32 and 32 x 128 tiles.  Their products are bound by reading the large
// operand, not by the matrix pipe (13 FLOP per byte), so what counts is how many workgroups keep
// loads in flight and how long each one's walk is, which the round count below does not see: at
// least one workgroup per CU -- two for a K of 8192 and more while slices stay 512 k long (rows a
// power of two apart put workgroups that walk in step into the same memory channels) -- and
// slices of about 1024 k rather than 2048 while that still adds workgroups (us by slices
// 1/2/4/8/16: 8192 x 32 x 4096 69 40 26 27 34; 4096 x 32 x 4096 69 39 24 16 19; 8192 x 32 x 8192 160
// 84 69 53 60; 4096 x 16 x 8192 133 72 40 35 28; 16384 x 32 x 4096 82 54 47 56 67; 16384 x 32 x 2048
// 37 26 29 36 43; 32768 x 32 x 1024 23 29 37; a linear layer at batch 32, 4096 -> 4096 66 38 24 16 19,
// 11008 -> 4096 170 91 51 35 38, 8192 -> 2048 127 69 39 23 17).
int narrow_tile_split(int M, int N, int K, int tile_id, const DeviceModel& dev)
{
    const TileInfo& t = tile_info(tile_id);
    const long tiles = (long)ceil_div(M, t.bm) * ceil_div(N, t.bn);
    int split = 1;
    while (tiles * split < dev.cus && K / (2 * split) >= 256) split *= 2;
    if (K >= 8192)
        while (tiles * split < 2L * dev.cus && K / (2 * split) >= 512) split *= 2;
    if (K / split >= 2048 && tiles * split < 2L * dev.cus) split *= 2;
    return split;
}

// Modelled time of one tile shape with one split factor.
double model_seconds(int M, int N, int K, int tile_id, int split, const DeviceModel& dev)
{
    const TileInfo& t = tile_info(tile_id);
    const int tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
    const long wgs = (long)tiles * split;
    const int ksteps = ceil_div(ceil_div(K, split), t.bk);
    const double extra = 64.0 / t.bk;
    // Time in units of one tile on a CU: the fullest CU decides.  (Counting rounds in resident
    // slots, with a penalty for a four-wave workgroup left alone on its CU, was tried and lost on a
    // set of 130 shapes: 14 of them more than 5 % off the best of four planner variants against 7
    // for this count.)
    double rounds = (double)((wgs + dev.cus - 1) / dev.cus);
    bool tail = false;
    if (split == 1) {
        const int ts = tail_split_that_pays(M, N, K, tile_id, dev);
        if (ts > 1) {
            rounds = (double)(wgs / dev.cus) + (ceil_div(ksteps, ts) + extra) / (ksteps + extra);
            tail = true;
        }
    }
    double s = rounds * tile_seconds(M, N, K, tile_id, split, dev);
    // never faster than streaming the operands once
    const double bytes = 4.0 * ((double)M * K + (double)K * N + (double)M * N);
    s = std::max(s, bytes / (0.7 * dev.hbm_bytes_per_s));
    if ((tile_id == TILE_128x32x32_W32x32 || tile_id == TILE_32x128x32_W32x32) && split != narrow_tile_split(M, N, K, tile_id, dev))
        s *= 1.3;   // see there
    // the slices are written, read back and summed by a second kernel
    // (the second kernel and the gap in front of it: 1020 x 108 x 731 takes 14.6 us whole, 10.6 us in 4 slices;
    // 3.5 us since that kernel keeps the loads of eight slices in flight -- with 5 us the choice was more than 5 %
    // off the best of three settings on 6 of 130 shapes, 140 x 2611 x 830 by 16 %, with 3.5 us on none)
    if (split > 1) s += 4.0 * (double)M * N * (split + 1) / (0.5 * dev.hbm_bytes_per_s) + 3.5e-6;
    if (tail) s += TAIL_SPLIT_SECONDS;
    return s + 3e-6;  // launch
}

}  // namespace

// ---- measured choices ------------------------------------------------------------
namespace {

struct TuneKey {
    int M, N, K, vec;
    bool operator<(const TuneKey& o) const
    {
        return std::tie(M, N, K, vec) < std::tie(o.M, o.N, o.K, o.vec);
    }
};

std::map<TuneKey, TunedChoice> g_tuned;
std::mutex g_tuned_mutex;

}  // namespace

bool tune_lookup(int M, int N, int K, bool vector_ok, TunedChoice* out)
{
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    auto it = g_tuned.find(TuneKey{M, N, K, vector_ok ? 1 : 0});
    if (it == g_tuned.end()) return false;
    if (out) *out = it->second;
    return true;
}

void tune_store(int M, int N, int K, bool vector_ok, const TunedChoice& c)
{
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    g_tuned[TuneKey{M, N, K, vector_ok ? 1 : 0}] = c;
}

void tune_erase(int M, int N, int K, bool vector_ok)
{
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    g_tuned.erase(TuneKey{M, N, K, vector_ok ? 1 : 0});
}

void tune_clear()
{
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    g_tuned.clear();
}

int tune_count()
{
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    return (int)g_tuned.size();
}

// One line per entry: M N K vec tile_m tile_n tile_k split_k tail_ok seconds
int tune_save(const char* path)
{
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    FILE* f = std::fopen(path, "w");
    if (!f) return CAKE_HIP_ERR_ARG;
    std::fprintf(f, "# cake_hip tuned macro-tiles: M N K vec tile_m tile_n tile_k split_k tail_ok seconds\n");
    for (const auto& kv : g_tuned) {
        const TileInfo& t = tile_info(kv.second.tile_id);
        std::fprintf(f, "%d %d %d %d %d %d %d %d %d %.9g\n", kv.first.M, kv.first.N, kv.first.K, kv.first.vec,
                     t.bm, t.bn, t.bk, kv.second.split_k, kv.second.tail_ok, kv.second.seconds);
    }
    return std::fclose(f) == 0 ? CAKE_HIP_OK : CAKE_HIP_ERR_ARG;
}

// Entries naming a tile this build does not have, or malformed lines, are skipped.
// Returns the number of entries taken, or -1 when the file cannot be read.
int tune_load(const char* path)
{
    FILE* f = std::fopen(path, "r");
    if (!f) return -1;
    char line[256];
    int taken = 0;
    while (std::fgets(line, sizeof line, f)) {
        if (line[0] == '#') continue;
        int M, N, K, vec, bm, bn, bk, split, tail;
        double secs;
        if (std::sscanf(line, "%d %d %d %d %d %d %d %d %d %lf", &M, &N, &K, &vec, &bm, &bn, &bk, &split, &tail,
                        &secs) != 10)
            continue;
        if (M <= 0 || N <= 0 || K <= 0 || split < 1 || split > ceil_div(K, bk > 0 ? bk : 1)) continue;
        int id = -1;
        for (int i = 0; i < TILE_COUNT; ++i) {
            const TileInfo& t = tile_info(i);
            if (t.bm == bm && t.bn == bn && t.bk == bk) id = i;
        }
        if (id < 0) continue;
        tune_store(M, N, K, vec != 0, TunedChoice{id, split, tail != 0, secs});
        ++taken;
    }
    std::fclose(f);
    return taken;
}

static int finish_plan(int M, int N, int K, int sched, int tile_id, int split, bool tail_allowed,
                       bool vector_ok, const DeviceModel& dev, GemmPlan* out);

int plan_gemm_choice(int M, int N, int K, int sched, const TunedChoice& c, bool vector_ok,
                     const DeviceModel& dev, GemmPlan* out)
{
    if (!out || M <= 0 || N <= 0 || K <= 0 || sched < 0 || sched > CAKE_HIP_NA) return CAKE_HIP_ERR_ARG;
    if (c.tile_id < 0 || c.tile_id >= TILE_COUNT || c.split_k < 1) return CAKE_HIP_ERR_ARG;
    if (tile_info(c.tile_id).lds_bytes > dev.lds_per_cu) return CAKE_HIP_ERR_ARG;
    std::memset(out, 0, sizeof *out);
    return finish_plan(M, N, K, sched, c.tile_id, c.split_k, c.tail_ok != 0, vector_ok, dev, out);
}

int plan_gemm(int M, int N, int K, int sched, const int* ov, bool vector_ok, const DeviceModel& dev,
              GemmPlan* out)
{
    if (!out || M <= 0 || N <= 0 || K <= 0 || sched < 0 || sched > CAKE_HIP_NA) return CAKE_HIP_ERR_ARG;
    std::memset(out, 0, sizeof *out);

    int want_m = ov ? ov[0] : 0, want_n = ov ? ov[1] : 0, want_k = ov ? ov[2] : 0;
    int want_split = ov ? ov[3] : 0;
    if (want_m < 0 || want_n < 0 || want_k < 0 || want_split < 0) return CAKE_HIP_ERR_ARG;

    // a measured choice for exactly this product wins over the model
    TunedChoice tuned;
    if (!ov && tune_lookup(M, N, K, vector_ok, &tuned) && tile_info(tuned.tile_id).lds_bytes <= dev.lds_per_cu)
        return finish_plan(M, N, K, sched, tuned.tile_id, tuned.split_k, tuned.tail_ok != 0, vector_ok, dev, out);

    if (!want_m && !want_n && !want_k && !want_split && stores_in_pieces_of_lines(M, N, K)) {   // (kernels.hpp)
        want_m = 96; want_n = 128; want_k = 32; want_split = 1;
    }
    Candidate best = {-1, 1, 1e30};
    for (int id = 0; id < TILE_COUNT; ++id) {
        const TileInfo& t = tile_info(id);
        if (want_m && t.bm != want_m) continue;
        if (want_n && t.bn != want_n) continue;
        if (want_k && t.bk != want_k) continue;
        if (t.lds_bytes > dev.lds_per_cu) continue;
        const int max_split = std::max(1, K / (4 * t.bk));
        for (int split = 1; split <= 1024; split *= 2) {
            if (want_split && split != want_split) continue;
            if (!want_split && split > max_split) break;
            const double s = model_seconds(M, N, K, id, split, dev);
            if (s < best.seconds) best = {id, split, s};
        }
        if (want_split && (want_split & (want_split - 1))) {  // non power of two asked for
            const double s = model_seconds(M, N, K, id, want_split, dev);
            if (s < best.seconds) best = {id, want_split, s};
        }
    }
    if (best.tile_id < 0) return CAKE_HIP_ERR_ARG;  // no tile matches the override
    const bool tail_allowed = !(ov && ov[3]);  // an explicit split request is taken literally
    return finish_plan(M, N, K, sched, best.tile_id, best.split, tail_allowed, vector_ok, dev, out);
}

static int finish_plan(int M, int N, int K, int sched, int tile_id, int split, bool tail_allowed,
                       bool vector_ok, const DeviceModel& dev, GemmPlan* out)
{
    const Candidate best = {tile_id, split, 0.0};
    const TileInfo& t = tile_info(best.tile_id);
    cake_hip_plan_t& p = out->pub;
    out->tile_id = best.tile_id;
    p.tile_m = t.bm; p.tile_n = t.bn; p.tile_k = t.bk;
    p.wave_m = t.wm; p.wave_n = t.wn;
    p.threads = t.threads;
    p.lds_bytes = t.lds_bytes;
    p.tiles_m = ceil_div(M, t.bm);
    p.tiles_n = ceil_div(N, t.bn);
    p.split_k = best.split;
    out->k_per_split = ceil_div(ceil_div(K, best.split), t.bk) * t.bk;
    // drop slices that would start past K
    p.split_k = ceil_div(K, out->k_per_split);
    p.grid = p.tiles_m * p.tiles_n * p.split_k;
    p.tail_tiles = 0;
    p.tail_split = 1;
    out->tail_k_per_split = 0;
    const int tiles = p.tiles_m * p.tiles_n;
    if (p.split_k == 1 && tail_allowed) {
        const int ksteps = ceil_div(K, t.bk);
        const int tt = thin_tail_tiles(tiles, dev);
        const int ts = tail_split_that_pays(M, N, K, tile_id, dev);
        if (ts > 1) {
            out->tail_k_per_split = ceil_div(ksteps, ts) * t.bk;
            p.tail_split = ceil_div(K, out->tail_k_per_split);
            p.tail_tiles = tt;
            p.grid = tiles - p.tail_tiles + p.tail_tiles * p.tail_split;
        }
    }
    p.vector_loads = vector_ok ? 1 : 0;
    p.cus = dev.cus;
    p.flops = 2.0 * M * N * (double)K;
    p.min_bytes = 4.0 * ((double)M * K + (double)K * N + (double)M * N);

    // Reuse order.  `resident` tiles run at the same time on one XCD and share
    // its L2: a gm x gn block of them re-reads each A panel ceil(tiles_n/gn)
    // times and each B panel ceil(tiles_m/gm) times from HBM.
    const int resident = std::max(1, dev.cus / dev.xcds * resident_per_cu(t, dev));
    auto traffic = [&](int gm, int gn) {
        return 4.0 * ((double)M * K * ceil_div(p.tiles_n, gn) + (double)K * N * ceil_div(p.tiles_m, gm) +
                      (double)M * N);
    };
    int gm, gn;
    int resolved = sched;
    if (sched == CAKE_HIP_NA) {
        // pick the block shape with the least modelled traffic; name it after
        // the reference schedule it corresponds to
        double best_bytes = 1e300;
        gm = 1; gn = resident;
        for (int g = 1; g <= resident; g *= 2) {
            const int cm = std::min(g, p.tiles_m), cn = std::min(std::max(1, resident / g), p.tiles_n);
            const double b = traffic(cm, cn);
            if (b < best_bytes) { best_bytes = b; gm = cm; gn = cn; }
        }
        if (gn == 1 && p.tiles_m > 1) resolved = CAKE_HIP_MKN;       // a column of tiles
        else if (gm == 1 && p.tiles_n > 1) resolved = CAKE_HIP_NKM;  // a row of tiles
        else resolved = CAKE_HIP_KMN;
    }
    if (resolved == CAKE_HIP_MKN) {          // M-first: walk down a tile column, B panel shared
        out->group_along_n = 1;
        p.group = 1;
        gm = std::min(resident, p.tiles_m); gn = 1;
    } else if (resolved == CAKE_HIP_NKM) {   // N-first: walk along a tile row, A panel shared
        out->group_along_n = 0;
        p.group = 1;
        gm = 1; gn = std::min(resident, p.tiles_n);
    } else {                                 // K-first with a compact CB block
        if (sched != CAKE_HIP_NA) {
            gm = std::max(1, (int)std::lround(std::sqrt((double)resident * t.bn / t.bm)));
            int pow2 = 1;
            while (pow2 * 2 <= gm) pow2 *= 2;
            gm = std::min(pow2, p.tiles_m);
            gn = std::min(std::max(1, resident / gm), p.tiles_n);
        }
        out->group_along_n = 0;
        p.group = gm;
    }
    p.sched = resolved;
    p.model_bytes = traffic(gm, gn);
    return CAKE_HIP_OK;
}

}  // namespace cake
