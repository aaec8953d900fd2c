"""grid_dims_2d, init_block_dims_2d and init_block_dims_2d_small (src/block_sizing.cpp:596-841): host
arithmetic of the shipped library against answers worked out by hand from the reference's formulas
(the derivations are in the comments) and against the invariants a block table has to satisfy.
The reference's own functions need a table its build generates and do not compile here."""
import numpy as np
import pytest

import cake_on_cpu_amd as cake


def _cx(L1=32 << 10, L2=1 << 20):
    return cake.CpuCntx(alpha_n=1.0, mr=6, nr=16, L1=L1, L2=L2, L3=32 << 20, ncores=8)


@pytest.mark.parametrize("M,N,p,want", [
    (3000, 3000, 8, 2),     # sqrt(8) = 2.83 -> 3, not a factor of 8: 4 and 2 are equally far, the lower one wins
    (1000, 4000, 8, 4),     # sqrt(32) = 5.66 -> 6: 8 and 4 equally far -> 4
    (3000, 3000, 12, 3),    # sqrt(12) = 3.46 -> 3 divides 12
    (10, 100000, 8, 8),     # sqrt(80000) capped at p
    (100000, 10, 8, 1),     # rounds to 0 -> 1
    (1000, 3000, 6, 3),     # sqrt(18) = 4.24 -> 4: 6 is 2 away, 3 is 1 away
    (1000, 2500, 10, 5),    # sqrt(25) = 5
    (1000, 1600, 10, 5),    # sqrt(16) = 4: 5 is 1 away, 2 is 2 away
    (5, 5, 7, 1),           # p prime, optimum 3: 7 is 4 away, 1 is 2 away
    (7, 7, 1, 1),
])
def test_grid_dims_2d_by_hand(M, N, p, want):
    assert cake.grid_dims_2d(M, N, 123, p, 8) == want


def test_grid_dims_2d_returns_a_factor_nearest_the_optimum():
    rng = np.random.default_rng(3)
    for _ in range(2000):
        M, N, p = int(rng.integers(1, 5000)), int(rng.integers(1, 5000)), int(rng.integers(1, 65))
        pn = cake.grid_dims_2d(M, N, 1, p, 64)
        assert 1 <= pn <= p and p % pn == 0
        opt = min(max(int(np.float32(np.sqrt(p * N / M)).round()), 1), p)
        nearest = min(abs(f - opt) for f in range(1, p + 1) if p % f == 0)
        assert abs(pn - opt) == nearest, (M, N, p, pn, opt)


def _fields(x, names):
    return {n: getattr(x, n) for n in names}


def test_init_block_dims_2d_by_hand():
    """L1 = 32 KiB: k_c = (8192 - 96) / 22 = 368.  L2 = 1 MiB: m_c = floor((-16 + sqrt(256 + 8 * 262144)) / 4)
    = 358 -> 354 (multiple of 6); n_c = 354 rounded up to 16 = 368.
    3000^3 on 8 cores: pn = 2, pm = 4; blocks of 1416 x 736: 3000 = 2 * 1416 + 168 (28 panels, 7 per core),
    3000 = 4 * 736 + 56 (4 panels of 16, 2 per core); K = 8 * 368 + 56."""
    x = cake.init_block_dims_2d(3000, 3000, 3000, 8, _cx())
    want = dict(m_c=354, k_c=368, n_c=368, m_c1=42, k_c1=56, n_c1=32, m_c1_last_core=42, n_c1_last_core=32,
                mr_rem=28, nr_rem=4, pm_l=4, pn_l=2, pm=4, pn=2, m_pad=1, k_pad=1, n_pad=1, Mb=3, Kb=9, Nb=5,
                M_padded=3000, N_padded=3008)
    assert _fields(x, want) == want
    # 20 x 100 x 5000: all 8 cores along N; M rounded up to 24 is less than one block of 354 -> m_c = 24,
    # n_c = 32; 5000 = 19 * 256 + 136: 9 panels over 8 cores, 2 per core on 5 cores, the last with 1
    x = cake.init_block_dims_2d(20, 5000, 100, 8, _cx())
    want = dict(m_c=24, k_c=368, n_c=32, m_c1=24, k_c1=100, n_c1=32, m_c1_last_core=24, n_c1_last_core=16,
                mr_rem=4, nr_rem=9, pm_l=1, pn_l=5, pm=1, pn=8, m_pad=1, k_pad=1, n_pad=1, Mb=1, Kb=1, Nb=20,
                M_padded=24, N_padded=5008)
    assert _fields(x, want) == want
    # a caller's tile: m_c and k_c are taken, n_c is still set from m_c (the reference overwrites ncu)
    x = cake.init_block_dims_2d(3000, 3000, 3000, 8, _cx(), mcu=96, kcu=200, ncu=999)
    assert (x.m_c, x.k_c, x.n_c, x.k_c1) == (96, 200, 96, 0)


def test_init_block_dims_2d_small_by_hand():
    """100 x 500 x 200 on 8 cores: pn = sqrt(16) = 4, pm = 2; M -> 102, N -> 208; m_c = 51 + 3 = 54,
    n_c = 52 + 12 = 64; k_c = min(m_c, 368) = 54; the last core's blocks: 102 - 54 = 48 and 208 - 192 = 16."""
    x = cake.init_block_dims_2d_small(100, 200, 500, 8, _cx())
    want = dict(m_c=54, k_c=54, n_c=64, m_c1=48, k_c1=14, n_c1=16, m_pad=1, k_pad=1, n_pad=1, Kb=10, pm=2, pn=4,
                M_padded=102, N_padded=208)
    assert _fields(x, want) == want


def test_init_block_dims_2d_covers_the_product():
    rng = np.random.default_rng(4)
    for _ in range(500):
        M, N, K = (int(rng.integers(1, 4000)) for _ in range(3))
        p = int(rng.integers(1, 33))
        cx = _cx(L1=int(rng.choice([16, 32, 48])) << 10, L2=int(rng.choice([256 << 10, 1 << 20, 2 << 20])))
        x = cake.init_block_dims_2d(M, N, K, p, cx)
        assert x.pm >= 1 and x.pn >= 1 and x.pm * x.pn <= p
        assert x.m_c % 6 == 0 and x.n_c % 16 == 0
        assert x.M_padded >= M and x.M_padded % 6 == 0 and x.M_padded - M < 6
        assert x.N_padded >= N and x.N_padded % 16 == 0 and x.N_padded - N < 16
        assert x.Mb * x.pm * x.m_c >= M and (x.Mb - 1) * x.pm * x.m_c < M
        assert x.Nb * x.pn * x.n_c >= N and (x.Nb - 1) * x.pn * x.n_c < N
        assert x.Kb * x.k_c >= K and (x.Kb - 1) * x.k_c < K
        if x.m_pad:   # the last block's panels are dealt over pm_l cores, the last of which may hold fewer
            assert (x.pm_l - 1) * x.m_c1 + x.m_c1_last_core == 6 * x.mr_rem and 0 < x.m_c1_last_core <= x.m_c1
        if x.n_pad:
            assert (x.pn_l - 1) * x.n_c1 + x.n_c1_last_core == 16 * x.nr_rem and 0 < x.n_c1_last_core <= x.n_c1


def test_bad_arguments_are_refused():
    with pytest.raises(cake.CakeHipError):
        cake.init_block_dims_2d(0, 5, 5, 4, _cx())
    with pytest.raises(cake.CakeHipError):
        cake.init_block_dims_2d_small(5, 5, 5, 0, _cx())
