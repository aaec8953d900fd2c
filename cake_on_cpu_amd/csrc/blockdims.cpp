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

// grid_dims_2d (src/block_sizing.cpp:596-634): the factor of p closest to the IO-optimal number
// of cores along N, sqrt(p N / M).  The reference looks the factors up in a table that its build
// generates for the machine's core count (python/grid_gen.py:19-42: row ncores - p marks the
// divisors of p); here divisibility is tested directly, so `ncores` is not needed and every
// p >= 1 has an answer.  Where the reference finds no factor below the optimum other than 1 it reads
// an uninitialised variable; that case is resolved as "the lower neighbour is 1".
int grid_dims_2d(int M, int N, int K, int p, int ncores)
{
    (void)K; (void)ncores;
    if (M <= 0 || N <= 0 || p <= 0) return 1;
    int pn = (int)roundf((float)std::sqrt(((double)p * N) / M));
    if (pn == 0) pn = 1;
    if (pn > p) pn = p;
    if (p % pn == 0) return pn;
    int high = p, low = 1;     // as factors, not table indices
    for (int f = pn + 1; f <= p; ++f)
        if (p % f == 0) { high = f; break; }
    for (int f = pn - 1; f >= 2; --f)
        if (p % f == 0) { low = f; break; }
    // the reference compares distances of table indices (factor - 1) to pn - 1: the same distances
    const int ret = (high - pn) < (pn - low) ? high : low;
    return ret < p ? ret : p;
}

namespace {
// k_c that keeps an m_r x k_c and a k_c x n_r panel plus the m_r x n_r tile in L1
// (src/block_sizing.cpp:657, :790), in the reference's single-precision arithmetic
int kc_from_l1(const cake_hip_cpu_cntx_t* cx, float type_size)
{
    return (int)((((float)cx->L1 / type_size) - (float)(cx->mr * cx->nr)) / (float)(cx->mr + cx->nr));
}
inline int round_up_to(int v, int q) { return v % q ? v + (q - v % q) : v; }
}  // namespace

// init_block_dims_2d (src/block_sizing.cpp:639-779): blocks for a pm x pn grid of cores.
int init_block_dims_2d(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cx, int sched, float type_size,
                       int mcu, int kcu, int ncu, cake_hip_blk_dims_t* x)
{
    if (!cx || !x || M <= 0 || N <= 0 || K <= 0 || p <= 0 || cx->mr <= 0 || cx->nr <= 0 || cx->L1 <= 0 ||
        cx->L2 <= 0 || !(type_size > 0) || sched < 0 || sched > CAKE_HIP_NA)
        return CAKE_HIP_ERR_ARG;
    const int mr = cx->mr, nr = cx->nr;
    std::memset(x, 0, sizeof *x);
    int pn = grid_dims_2d(M, N, K, p, cx->ncores);
    int pm = p / pn;
    const int M_up = round_up_to(M, mr), N_up = round_up_to(N, nr);
    int m_c, k_c;
    if (mcu && ncu && kcu) {
        m_c = mcu;
        k_c = kcu;
        cx->alpha_n = 1.0;
    } else {
        // m_c k_c + n_r k_c + m_c n_c <= L2 with n_c = m_c
        m_c = (int)((-nr + std::sqrt(1.0 * nr * nr + 4.0 * 2 * (((double)cx->L2) / 4.0))) / (2.0 * 2));
        m_c -= m_c % mr;
        k_c = kc_from_l1(cx, type_size);
    }
    if (m_c <= 0 || k_c <= 0) return CAKE_HIP_ERR_ARG;
    if (M_up == pm * mr) {
        m_c = mr;
        pm = 1;
    } else if (M_up < pm * m_c) {
        const int share = M_up / pm;
        if (share < mr) {
            m_c = mr;
            pm = M_up / mr;
        } else {
            m_c = round_up_to(share, mr);
        }
    }
    int n_c = round_up_to(m_c, nr);      // square tiles; a caller's ncu is overwritten here, as in the reference
    if (N_up == pn * nr) {
        n_c = nr;
        pn = 1;
    } else if (N_up < pn * n_c) {
        const int share = N_up / pn;
        if (share < nr) {
            n_c = nr;
            pn = N_up / nr;
        } else {
            n_c = round_up_to(share, nr);
        }
    }
    const int mspan = pm * m_c, nspan = pn * n_c;
    x->mr_rem = ceil_div(M % mspan, mr);
    const int mr_per_core = ceil_div(x->mr_rem, pm);
    x->pm_l = mr_per_core ? ceil_div(x->mr_rem, mr_per_core) : 0;
    x->m_c1 = mr_per_core * mr;
    x->m_c1_last_core = (mr_per_core - (x->pm_l * mr_per_core - x->mr_rem)) * mr;
    x->nr_rem = ceil_div(N % nspan, nr);
    const int nr_per_core = ceil_div(x->nr_rem, pn);
    x->pn_l = nr_per_core ? ceil_div(x->nr_rem, nr_per_core) : 0;
    x->n_c1 = nr_per_core * nr;
    x->n_c1_last_core = (nr_per_core - (x->pn_l * nr_per_core - x->nr_rem)) * nr;
    x->m_pad = M % mspan != 0;
    x->k_pad = K % k_c != 0;
    x->n_pad = N % nspan != 0;
    x->Mb = M / mspan + x->m_pad;
    x->Nb = N / nspan + x->n_pad;
    x->Kb = K / k_c + x->k_pad;
    x->M_padded = mr * x->mr_rem + (M / mspan) * mspan;
    x->N_padded = nr * x->nr_rem + (N / nspan) * nspan;
    x->m_c = m_c; x->k_c = k_c; x->n_c = n_c;
    x->k_c1 = K % k_c;
    x->pm = pm; x->pn = pn;
    x->sch = sched;
    return CAKE_HIP_OK;
}

// init_block_dims_2d_small (src/block_sizing.cpp:785-841): one block per core of the grid.
int init_block_dims_2d_small(int M, int N, int K, int p, cake_hip_cpu_cntx_t* cx, int sched, float type_size,
                             cake_hip_blk_dims_t* x)
{
    if (!cx || !x || M <= 0 || N <= 0 || K <= 0 || p <= 0 || cx->mr <= 0 || cx->nr <= 0 || cx->L1 <= 0 ||
        !(type_size > 0) || sched < 0 || sched > CAKE_HIP_NA)
        return CAKE_HIP_ERR_ARG;
    const int mr = cx->mr, nr = cx->nr;
    std::memset(x, 0, sizeof *x);
    const int pn = grid_dims_2d(M, N, K, p, cx->ncores);
    const int pm = p / pn;
    const int M_up = round_up_to(M, mr), N_up = round_up_to(N, nr);
    int m_c = M_up / pm;
    m_c += mr - m_c % mr;               // (a whole panel more when it already is a multiple: as the reference)
    int n_c = N_up / pn;
    n_c += nr - n_c % nr;
    const int kc_max = kc_from_l1(cx, type_size);
    if (kc_max <= 0) return CAKE_HIP_ERR_ARG;
    const int k_c = m_c > kc_max ? kc_max : m_c;
    x->M_padded = M_up;
    x->N_padded = N_up;
    x->m_c = m_c; x->k_c = k_c; x->n_c = n_c;
    x->m_c1 = M_up - (pm - 1) * m_c;
    x->n_c1 = N_up - (pn - 1) * n_c;
    x->k_c1 = K % k_c;
    x->k_pad = K % k_c != 0;
    x->n_pad = N % n_c != 0;
    x->m_pad = M % m_c != 0;
    x->Kb = K / k_c + x->k_pad;
    x->pm = pm; x->pn = pn;
    x->sch = sched;
    return CAKE_HIP_OK;
}

// get_cache_dims_conv + init_block_dims_conv (examples/cake_conv.cpp:262-420): blocks of the direct
// convolution -- M = Cout over the cores, K = input channels (k_c channels, each with all its
// filter taps), N = rows of the output image.  K-first only, like the reference.
int init_block_dims_conv(int Wf, int Hf, int Win, int Hin, int Wout, int Hout, int Cin, int Cout, int s, int p,
                         cake_hip_cpu_cntx_t* cx, cake_hip_blk_dims_t* x)
{
    (void)Hin; (void)s;
    if (!cx || !x || Wf <= 0 || Hf <= 0 || Win <= 0 || Wout <= 0 || Hout <= 0 || Cin <= 0 || Cout <= 0 || p <= 0 ||
        cx->mr <= 0 || cx->nr <= 0 || cx->L2 <= 0)
        return CAKE_HIP_ERR_ARG;
    const int mr = cx->mr;
    std::memset(x, 0, sizeof *x);
    int Cm = ceil_div(Cout, p);
    Cm -= Cm % mr;
    int mc = Cm;
    if (Cout < p * mr) {
        mc = mr;
    } else if (Cout < p * Cm) {
        const int share = Cout / p;
        mc = share < mr ? mr : share + (mr - share % mr);
    }
    int nc = (int)std::floor((cx->alpha_n * p * mc) / Wout);
    if (nc == 0) nc = 1;
    // 4 (Cm Wf Hf Ck + Hc Win Ck + Hc Wout Cm) <= L2
    int Ck = (int)std::ceil(((((double)cx->L2) / 4.0) - (double)nc * Wout * mc) / ((double)mc * Wf * Hf + (double)nc * Win));
    if (Ck > Cin) Ck = Cin;
    else if (Ck < 0) Ck = 128;
    if (Ck == 0) Ck = 1;     // (the reference would divide by zero)
    x->m_c = mc; x->k_c = Ck; x->n_c = nc;
    x->sch = CAKE_HIP_KMN;
    const int M = Cout, N = Hout, K = Cin, span = p * mc;
    x->k_pad = K % Ck != 0;
    x->n_pad = N % nc != 0;
    x->m_pad = M % span != 0;
    x->mr_rem = ceil_div(M % span, mr);
    const int mr_per_core = ceil_div(x->mr_rem, p);
    x->p_l = mr_per_core ? ceil_div(x->mr_rem, mr_per_core) : 0;
    x->n_c1 = N % nc;
    x->m_c1 = mr_per_core * mr;
    x->m_c1_last_core = (mr_per_core - (x->p_l * mr_per_core - x->mr_rem)) * mr;
    x->k_c1 = K % Ck;
    x->Mb = M / span + x->m_pad;
    x->Nb = N / nc + x->n_pad;
    x->Kb = K / Ck + x->k_pad;
    x->M_padded = mr * x->mr_rem + (M / span) * span;
    x->N_padded = (N - N % nc) + x->n_c1;
    return CAKE_HIP_OK;
}

}  // namespace cake
