"""cake_sgemm restatement (planner -> pack -> snake schedule -> micro-kernel -> unpack)
against what the mathematics fixes: fp64 triple loop, identity, all-ones,
single non-zero, on the reference's own edge-shape list (src/util.cpp:11-13)."""
import itertools

import numpy as np
import pytest

import oracle

TOL = 1e-4        # the bar: max |C - C64| / sum_k |a||b|
TIGHT = 2e-6      # what a correct fp32 FMA chain actually achieves at these K
SCHEDS = [oracle.KMN, oracle.MKN, oracle.NKM, oracle.NA]
SMALL = [1, 10, 96, 111, 960]


def _check(M, K, N, p, sch, cx=None):
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    Cm = oracle.cake_sgemm(A, B, p, cx or oracle.make_cntx(), sch=sch)
    C64, S = oracle.gemm_f64(A, B)
    err = oracle.max_rel_err(Cm, C64, S)
    assert err <= TOL and err <= TIGHT, (M, K, N, p, sch, err)


@pytest.mark.parametrize("sch", SCHEDS)
@pytest.mark.parametrize("p", [2, 3])
def test_edge_grid_small(sch, p):
    for M, K, N in itertools.product(SMALL, SMALL, SMALL):
        _check(M, K, N, p, sch)


@pytest.mark.parametrize("sch", [oracle.KMN, oracle.MKN, oracle.NKM])
@pytest.mark.parametrize("shape", [(2111, 2111, 2111), (2111, 96, 111), (111, 2111, 96),
                                   (96, 111, 2111), (1, 2111, 10), (2111, 1, 960), (10, 960, 2111)],
                         ids=lambda s: "x".join(map(str, s)))
def test_edge_shapes_with_2111(shape, sch):
    M, K, N = shape
    _check(M, K, N, 8, sch)


@pytest.mark.parametrize("sch", [oracle.KMN, oracle.MKN, oracle.NKM])
@pytest.mark.parametrize("p", [1, 5, 8])
def test_small_caches_many_blocks(sch, p):
    """Tiny caches force many CB blocks in every dimension, so every snake
    direction and every remainder branch is taken."""
    cx = oracle.make_cntx(L2=16 << 10, L3=256 << 10, ncores=8)
    x = oracle.init_block_dims(333, 517, 419, p, cx, sch)
    assert x.Mb * x.Kb * x.Nb >= 8
    _check(333, 419, 517, p, sch, cx)


@pytest.mark.parametrize("sch", [oracle.KMN, oracle.MKN, oracle.NKM])
def test_identity_all_ones_single_nonzero(sch):
    cx = oracle.make_cntx(L2=32 << 10, L3=512 << 10)
    n = 257
    B = oracle.uniform((n, 300), 5)
    assert np.array_equal(oracle.cake_sgemm(np.eye(n, dtype=np.float32), B, 4, cx, sch=sch), B)
    ones = oracle.cake_sgemm(np.ones((70, 513), np.float32), np.ones((513, 91), np.float32), 3, cx, sch=sch)
    assert np.array_equal(ones, np.full((70, 91), 513.0, np.float32))
    A = np.zeros((40, 50), np.float32)
    A[17, 23] = 2.0
    Bm = oracle.uniform((50, 60), 6)
    want = np.zeros((40, 60), np.float32)
    want[17] = 2.0 * Bm[23]
    assert np.array_equal(oracle.cake_sgemm(A, Bm, 2, cx, sch=sch), want)


def test_transposed_operand_would_fail():
    """The checker itself must see a transposed operand (guards the guard)."""
    A, B = oracle.uniform((64, 64), 1), oracle.uniform((64, 64), 2)
    C64, S = oracle.gemm_f64(A, B)
    wrong = (A.T.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    assert oracle.max_rel_err(wrong, C64, S) > 1e-2
    dropped = (A[:, :-1].astype(np.float64) @ B[:-1].astype(np.float64)).astype(np.float32)
    assert oracle.max_rel_err(dropped, C64, S) > 1e-3


def test_overwrite_vs_accumulate_semantics(cx8):
    """KMN assigns; MKN/NKM add to the existing C only when beta != 0
    (src/cake_sgemm.cpp:114, src/pack_ob.cpp:404); alpha is never read."""
    A, B = oracle.uniform((100, 80), 1), oracle.uniform((80, 120), 2)
    C0 = oracle.uniform((100, 120), 3)
    base = oracle.cake_sgemm(A, B, 4, cx8, sch=oracle.KMN)
    assert np.array_equal(oracle.cake_sgemm(A, B, 4, cx8, Cinit=C0, beta=1.0, sch=oracle.KMN), base)
    for sch in (oracle.MKN, oracle.NKM):
        assert np.allclose(oracle.cake_sgemm(A, B, 4, cx8, Cinit=C0, beta=0.0, sch=sch), base, atol=1e-5)
        acc = oracle.cake_sgemm(A, B, 4, cx8, Cinit=C0, beta=0.5, sch=sch)
        C64, S = oracle.gemm_f64(A, B)
        assert oracle.max_rel_err(acc - C0, C64, S + np.abs(C0)) <= 1e-5


def test_deterministic_for_fixed_p(cx8):
    A, B = oracle.uniform((300, 400), 1), oracle.uniform((400, 200), 2)
    first = oracle.cake_sgemm(A, B, 8, cx8, sch=oracle.KMN)
    for _ in range(3):
        assert np.array_equal(oracle.cake_sgemm(A, B, 8, cx8, sch=oracle.KMN), first)
