// planner.hpp -- tile, wave-layout and reuse-order planner for the MFMA GEMM.
//
// The successor of CAKE's get_cache_dims / derive_schedule
// (src/block_sizing.cpp:304-462).  The reference sizes a CB block
// p*m_c x k_c x n_c from L2/L3 so that DRAM traffic per unit of compute stays
// constant as cores are added, and picks K-, M- or N-first reuse from an IO
// model.  Here the unit of compute is a workgroup's macro-tile, the "cores" are
// the CUs of one XCD (which share an L2), and the CB block is the set of tiles
// those CUs hold at the same time.
#pragma once

#include "cake_hip.h"

namespace cake {

struct DeviceModel {
    int cus = 256;               // MI355X: 8 XCDs x 32 CUs
    int xcds = 8;
    int lds_per_cu = 160 * 1024;
    int l2_per_xcd = 4 << 20;
    double mfma_flops = 157.3e12;  // fp32 matrix peak
    double hbm_bytes_per_s = 8.0e12;
};

struct GemmPlan {
    cake_hip_plan_t pub;   // what the C-ABI reports
    int tile_id;           // kernels.hpp TileId
    int k_per_split;       // multiple of tile_k
    int tail_k_per_split;  // multiple of tile_k; meaningful when pub.tail_tiles > 0
    int group_along_n;
};

// vector_ok: operands allow 16-byte loads (K%4==0, N%4==0, aligned bases).
// tile_override: {tile_m, tile_n, tile_k, split_k} or nullptr, zeros = choose.
// Returns a CAKE_HIP_* status.
int plan_gemm(int M, int N, int K, int sched, const int* tile_override, bool vector_ok,
              const DeviceModel& dev, GemmPlan* out);

// A measured choice for one product (the autotuner's result): which macro-tile,
// how many K slices for every tile, and whether a thin last round may be cut.
struct TunedChoice {
    int tile_id;
    int split_k;
    int tail_ok;
    double seconds;  // the measurement that won
};

// plan for an explicit choice (what the autotuner times)
int plan_gemm_choice(int M, int N, int K, int sched, const TunedChoice& c, bool vector_ok,
                     const DeviceModel& dev, GemmPlan* out);

// Table of measured choices keyed by (M, N, K, vector_ok); plan_gemm consults it
// when the caller gives no override.  Thread-safe.
bool tune_lookup(int M, int N, int K, bool vector_ok, TunedChoice* out);
void tune_store(int M, int N, int K, bool vector_ok, const TunedChoice& c);
void tune_erase(int M, int N, int K, bool vector_ok);
void tune_clear();
int tune_count();
int tune_save(const char* path);  // CAKE_HIP_* status
int tune_load(const char* path);  // entries taken, or -1 when unreadable

}  // namespace cake
