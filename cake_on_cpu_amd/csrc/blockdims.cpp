// blockdims.cpp -- the reference's CPU block sizing, kept for API compatibility
// (callers read blk_dims_t; the packed layouts are defined in terms of it).
#include "blockdims.hpp"

#include <cmath>
#include <cstring>

namespace cake {

namespace {
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline int floor_to(int v, int q) { return (v / q) * q; }
}  // namespace

// IO-optimal reuse order for a CB block of side p*mc (src/block_sizing.cpp:434-462).
// The thresholds are single precision in the reference and are kept so, because
// the comparison decides the schedule at exact ties.
int derive_schedule(int M, int N, int K, int p, int mc, const cake_hip_cpu_cntx_t* cx)
{
    const float cube = (float)(p * mc);
    const float wide = (float)(cx->alpha_n * p * mc);
    auto k_cut = [&](int X) { return (float)((2.0 * X) / (1.0 + (X * ((2.0 / cube) - (1.0 / cube))))); };
    auto x_cut = [&](int X) { return (float)(X / (1.0 + (X * ((1.0 / wide) - (1.0 / wide))))); };
    if ((float)N <= x_cut(M) && (float)K <= k_cut(M)) return CAKE_HIP_MKN;
    if ((float)M <= x_cut(N) && (float)K <= k_cut(N)) return CAKE_HIP_NKM;
    return CAKE_HIP_KMN;
}

int init_block_dims(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cx, int sched,
                    int mcu, int kcu, int ncu, cake_hip_blk_dims_t* x)
{
    if (!cx || !x || M <= 0 || N <= 0 || K <= 0 || p <= 0 || cx->mr <= 0 || cx->nr <= 0 ||
        cx->ncores <= 0 || cx->L2 <= 0 || cx->L3 <= 0 || sched < 0 || sched > CAKE_HIP_NA)
        return CAKE_HIP_ERR_ARG;
    const int mr = cx->mr, nr = cx->nr;
    std::memset(x, 0, sizeof *x);

    // get_cache_dims (src/block_sizing.cpp:304-429): square m_c = k_c from the L2
    // capacity, L3-derived width factor alpha_n.
    const double elem = 4.0;
    const double two_nr = 2.0 * nr;
    int mc_l2 = floor_to((int)((-two_nr + std::sqrt(two_nr * two_nr + 4.0 * (cx->L2 / (2.0 * elem)))) / 2.0), mr);
    int mc_l3 = floor_to((int)std::sqrt((cx->L3 / (2.0 * elem)) / (cx->ncores * (2.0 + cx->ncores))), mr);
    if (mc_l2 <= 0) return CAKE_HIP_ERR_ARG;
    cx->alpha_n = (double)mc_l3 / (double)mc_l2;

    int mc = mc_l2;
    if (M < p * mr) {
        mc = mr;
    } else if (M < p * mc_l2) {
        int share = M / p;
        mc = share < mr ? mr : share + (mr - share % mr);
    }

    x->sch = (sched == CAKE_HIP_NA) ? derive_schedule(M, N, K, p, mc, cx) : sched;

    if (mcu && kcu && ncu) {
        x->m_c = mcu; x->k_c = kcu; x->n_c = ncu;
        cx->alpha_n = 1.0;
    } else {
        int nc;
        if (x->sch == CAKE_HIP_NKM) {
            nc = floor_to(mc, nr);
            mc = floor_to((int)(cx->alpha_n * mc), mr);
            if (mc == 0) mc = mr;
        } else {
            nc = floor_to((int)(cx->alpha_n * p * mc), nr);
        }
        if (nc == 0) nc = nr;
        x->m_c = mc; x->k_c = mc; x->n_c = nc;
    }

    // init_block_dims (src/block_sizing.cpp:465-595): remainders and padding.
    x->n_pad = N % x->n_c != 0;
    x->nr_rem = ceil_div(N % x->n_c, nr);
    x->n_c1 = x->nr_rem * nr;
    x->Nb = N / x->n_c + x->n_pad;
    x->N_padded = N - N % x->n_c + x->n_c1;

    if (x->sch == CAKE_HIP_KMN) {
        const int span = p * x->m_c;
        x->m_pad = M % span != 0;
        x->k_pad = K % x->k_c != 0;
        x->mr_rem = ceil_div(M % span, mr);
        const int panels_per_core = ceil_div(x->mr_rem, p);
        x->p_l = panels_per_core ? ceil_div(x->mr_rem, panels_per_core) : 0;
        x->m_c1 = panels_per_core * mr;
        x->m_c1_last_core = (x->mr_rem - (x->p_l - 1) * panels_per_core) * mr;
        if (!panels_per_core) x->m_c1_last_core = 0;
        x->k_c1 = K % x->k_c;
        x->Mb = M / span + x->m_pad;
        x->Kb = K / x->k_c + x->k_pad;
        x->M_padded = (M / span) * span + x->mr_rem * mr;
        x->pm = p; x->pn = 1;
    } else {
        const int kspan = p * x->k_c;
        const int mspan = (x->sch == CAKE_HIP_MKN) ? x->m_c : p * x->m_c;
        x->m_pad = M % mspan != 0;
        x->k_pad = K % kspan != 0;
        x->k_rem = K % kspan;
        x->k_c1 = ceil_div(x->k_rem, p);
        x->p_l = x->k_c1 ? ceil_div(x->k_rem, x->k_c1) : 0;
        x->k_c1_last_core = x->k_rem - x->k_c1 * (x->p_l - 1);
        x->mr_rem = ceil_div(M % mspan, mr);
        x->m_c1 = x->mr_rem * mr;
        x->Mb = M / mspan + x->m_pad;
        x->Kb = K / kspan + x->k_pad;
        x->M_padded = (M / mspan) * mspan + x->m_c1;
        if (x->sch == CAKE_HIP_MKN) { x->pm = p; x->pn = 1; } else { x->pm = 1; x->pn = p; }
    }
    return CAKE_HIP_OK;
}

}  // namespace cake
