// blockdims.hpp -- the reference's CPU block sizing (blk_dims_t) and the packed
// operand layouts it implies, as index maps usable on host and device.
//
// The GPU kernels do not need CB blocks sized for CPU caches; this exists
// because the drop-in API exposes init_block_dims / blk_dims_t / pack_A / pack_B
// (include/tiling.h:39-41, include/packing.h:6-13 of the reference) and callers
// hand packed buffers back to cake_sgemm (examples/cake_conv.cpp:1028-1055).
#pragma once

#include <cstddef>
#include <cstdint>

#include "cake_hip.h"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define CAKE_HD __host__ __device__ __forceinline__
#else
#define CAKE_HD inline
#endif

namespace cake {

// Everything a packed-offset computation needs, flattened so it can be passed
// to a kernel by value.
struct PackGeom {
    cake_hip_blk_dims_t d;
    int M, N, K, p, mr, nr, sch;
};

// src/block_sizing.cpp:304-595
int init_block_dims(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cx, int sched,
                    int mcu, int kcu, int ncu, cake_hip_blk_dims_t* out);
// src/block_sizing.cpp:434-462
int derive_schedule(int M, int N, int K, int p, int mc, const cake_hip_cpu_cntx_t* cx);

// src/block_sizing.cpp:596-841: sizing for the reference's 2-D grid of cores
int grid_dims_2d(int M, int N, int K, int p, int ncores);
int init_block_dims_2d(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cx, int sched, float type_size,
                       int mcu, int kcu, int ncu, cake_hip_blk_dims_t* out);
int init_block_dims_2d_small(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cx, int sched, float type_size,
                             cake_hip_blk_dims_t* out);
// examples/cake_conv.cpp:262-420: blocks of the direct convolution (K-first)
int init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s, int p,
                         cake_hip_cpu_cntx_t* cx, cake_hip_blk_dims_t* out);

// Padded extents of the packed operands (src/pack_helper.cpp:5-87).
CAKE_HD int padded_rows(const PackGeom& g)
{
    int span = (g.sch == CAKE_HIP_MKN) ? g.d.m_c : g.p * g.d.m_c;
    int rem = g.M % span;
    return (g.M / span) * span + ((rem + g.mr - 1) / g.mr) * g.mr;
}

CAKE_HD int padded_cols(const PackGeom& g)
{
    int rem = g.N % g.d.n_c;
    return (g.N - rem) + ((rem + g.nr - 1) / g.nr) * g.nr;
}

// How a coordinate along the dimension that is divided among the p cores
// decomposes: which CB block, which core's slice, where inside it, and how
// long that slice and the whole block are.
struct SplitPos {
    int block;     // CB block index
    int core;      // slice within the block
    int inner;     // offset inside the slice
    int slice;     // nominal slice length in this block (stride between cores)
    int length;    // actual length of this core's slice
    int span;      // total length of this block
};

// Dimension split over cores with per-core length `full`; the last block
// (when `pad`) holds `rem_span` elements in `used` slices of `slice1`, the
// last of which has `last_len`.
CAKE_HD SplitPos split_pos(int x, int p, int full, int nblocks, int pad,
                           int rem_span, int slice1, int used, int last_len)
{
    SplitPos s;
    int span = p * full;
    s.block = x / span;
    int r = x - s.block * span;
    bool last = pad && (s.block == nblocks - 1);
    s.slice = last ? slice1 : full;
    s.span = last ? rem_span : span;
    s.core = r / s.slice;
    s.inner = r - s.core * s.slice;
    s.length = last ? (s.core == used - 1 ? last_len : slice1) : full;
    return s;
}

// Offset of A(row, col) in the packed A of schedule g.sch.
//   KMN [m-blk][k-blk][core][m_r-panel][k][m_r]   src/pack_k_first.cpp:27-68
//   MKN [k-blk][m-blk][core(k)][m_r-panel][k][m_r] src/pack_m_first.cpp:29-69
//   NKM [m-blk][k-blk][core(k)][m_r-panel][k][m_r] src/pack_n_first.cpp:30-70
// panel layout: src/pack_ob.cpp:40-60.  row < padded_rows, col < K.
CAKE_HD int64_t packed_a_offset(const PackGeom& g, int row, int col)
{
    const cake_hip_blk_dims_t& d = g.d;
    const int mr = g.mr;
    if (g.sch == CAKE_HIP_KMN) {
        SplitPos m = split_pos(row, g.p, d.m_c, d.Mb, d.m_pad, mr * d.mr_rem, d.m_c1, d.p_l,
                               d.m_c1_last_core);
        int kb = col / d.k_c, kk = col - kb * d.k_c;
        int kc = (d.k_pad && kb == d.Kb - 1) ? d.k_c1 : d.k_c;
        int panel = m.inner / mr, j = m.inner - panel * mr;
        return (int64_t)m.block * g.p * d.m_c * g.K + (int64_t)kb * m.span * d.k_c +
               (int64_t)m.core * m.slice * kc + (int64_t)panel * mr * kc + (int64_t)kk * mr + j;
    }
    SplitPos k = split_pos(col, g.p, d.k_c, d.Kb, d.k_pad, d.k_rem, d.k_c1, d.p_l,
                           d.k_c1_last_core);
    int mspan = (g.sch == CAKE_HIP_MKN) ? d.m_c : g.p * d.m_c;
    int mb = row / mspan, r = row - mb * mspan;
    int rows = (d.m_pad && mb == d.Mb - 1) ? d.m_c1 : mspan;
    int panel = r / mr, j = r - panel * mr;
    int64_t base = (g.sch == CAKE_HIP_MKN)
                       ? (int64_t)k.block * padded_rows(g) * g.p * d.k_c + (int64_t)mb * d.m_c * k.span
                       : (int64_t)mb * mspan * g.K + (int64_t)k.block * g.p * d.k_c * rows;
    return base + (int64_t)k.core * k.slice * rows + (int64_t)panel * mr * k.length +
           (int64_t)k.inner * mr + j;
}

// Offset of filter element (row = output channel, channel, tap) in the layout of the reference's
// pack_filters (examples/cake_conv.cpp:430-454,536-610): K-first blocks of A with K = input
// channels, and inside an m_r panel the taps outermost, [m-blk][channel-blk][core][m_r-panel][tap][channel][m_r].
// g.d from init_block_dims_conv, g.K = Cin.  row < padded rows (d.M_padded), channel < Cin.
CAKE_HD int64_t packed_filter_offset(const PackGeom& g, int row, int channel, int tap, int taps)
{
    const cake_hip_blk_dims_t& d = g.d;
    const int mr = g.mr;
    SplitPos m = split_pos(row, g.p, d.m_c, d.Mb, d.m_pad, mr * d.mr_rem, d.m_c1, d.p_l, d.m_c1_last_core);
    const int kb = channel / d.k_c, i = channel - kb * d.k_c;
    const int kc = (d.k_pad && kb == d.Kb - 1) ? d.k_c1 : d.k_c;
    const int panel = m.inner / mr, j = m.inner - panel * mr;
    return ((int64_t)m.block * g.p * d.m_c * g.K + (int64_t)kb * m.span * d.k_c + (int64_t)m.core * m.slice * kc +
            (int64_t)panel * mr * kc) * taps + (int64_t)tap * kc * mr + (int64_t)i * mr + j;
}

// Offset of B(row = k, col = n) in the packed B.
//   KMN [n-blk][k-blk][n_r-panel][k][n_r]          src/pack_k_first.cpp:187-283
//   MKN [n-blk][k-blk][core(k)][n_r-panel][k][n_r] src/pack_m_first.cpp:99-142
//   NKM [k-blk][n-blk][core(k)][n_r-panel][k][n_r] src/pack_n_first.cpp:99-142
// panel layout: src/pack_ob.cpp:105-140.  row < K, col < padded_cols.
CAKE_HD int64_t packed_b_offset(const PackGeom& g, int row, int col)
{
    const cake_hip_blk_dims_t& d = g.d;
    const int nr = g.nr;
    int nb = col / d.n_c, c = col - nb * d.n_c;
    int cols = (d.n_pad && nb == d.Nb - 1) ? d.n_c1 : d.n_c;
    int panel = c / nr, j = c - panel * nr;
    if (g.sch == CAKE_HIP_KMN) {
        int kb = row / d.k_c, kk = row - kb * d.k_c;
        int kc = (d.k_pad && kb == d.Kb - 1) ? d.k_c1 : d.k_c;
        return (int64_t)nb * g.K * d.n_c + (int64_t)kb * d.k_c * cols + (int64_t)panel * kc * nr +
               (int64_t)kk * nr + j;
    }
    SplitPos k = split_pos(row, g.p, d.k_c, d.Kb, d.k_pad, d.k_rem, d.k_c1, d.p_l,
                           d.k_c1_last_core);
    int64_t base = (g.sch == CAKE_HIP_MKN)
                       ? (int64_t)nb * g.K * d.n_c + (int64_t)k.block * g.p * d.k_c * cols
                       : (int64_t)k.block * g.p * d.k_c * padded_cols(g) + (int64_t)nb * d.n_c * k.span;
    return base + (int64_t)k.core * k.slice * cols + (int64_t)panel * k.length * nr +
           (int64_t)k.inner * nr + j;
}

// Offset of C(row, col) in the packed C: blocks of [n_r-panel][m_r-panel][m_r][n_r]
// (src/pack_ob.cpp:253-288) ordered per schedule
//   KMN src/pack_k_first.cpp:404-476, MKN src/unpack_m_first.cpp:5-49,
//   NKM src/unpack_n_first.cpp:5-49.
CAKE_HD int64_t packed_c_offset(const PackGeom& g, int row, int col)
{
    const cake_hip_blk_dims_t& d = g.d;
    const int mr = g.mr, nr = g.nr;
    int nb = col / d.n_c, c = col - nb * d.n_c;
    int cols = (d.n_pad && nb == d.Nb - 1) ? d.n_c1 : d.n_c;
    int pn = c / nr, j = c - pn * nr;
    int64_t base;
    int rows, r;
    if (g.sch == CAKE_HIP_KMN) {
        SplitPos m = split_pos(row, g.p, d.m_c, d.Mb, d.m_pad, mr * d.mr_rem, d.m_c1, d.p_l,
                               d.m_c1_last_core);
        base = (int64_t)nb * d.n_c * padded_rows(g) + (int64_t)m.block * g.p * d.m_c * cols +
               (int64_t)m.core * m.slice * cols;
        rows = m.length;
        r = m.inner;
    } else if (g.sch == CAKE_HIP_MKN) {
        int mb = row / d.m_c;
        r = row - mb * d.m_c;
        rows = (d.m_pad && mb == d.Mb - 1) ? d.m_c1 : d.m_c;
        base = (int64_t)padded_rows(g) * nb * d.n_c + (int64_t)mb * d.m_c * cols;
    } else {
        int mspan = g.p * d.m_c, mb = row / mspan;
        r = row - mb * mspan;
        rows = (d.m_pad && mb == d.Mb - 1) ? d.m_c1 : mspan;
        base = (int64_t)padded_cols(g) * mb * mspan + (int64_t)nb * rows * d.n_c;
    }
    int pm = r / mr, i = r - pm * mr;
    return base + (int64_t)pn * rows * nr + (int64_t)pm * mr * nr + (int64_t)i * nr + j;
}

}  // namespace cake
