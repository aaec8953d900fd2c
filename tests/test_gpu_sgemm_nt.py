"""GPU parity of cake_hip_sgemm_nt (C = A . Bt^T with Bt read as it lies: the product inside the
reference's linear_forward, src/linear.cpp:38, without its transposed copy) against the oracle.

The oracle's cake_sgemm takes B as K x N, so it is given Bt transposed on the host; the bar is the
product's: max |C - C_ref| / sum_k |a||b| <= 1e-4 against the oracle and <= 5e-6 against fp64."""
import itertools

import numpy as np
import pytest

import cake_on_cpu_amd as cake
import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-4
TIGHT = 5e-6
TILES = [(256, 256, 32), (256, 128, 32), (128, 256, 32), (128, 128, 32), (64, 64, 32), (64, 64, 64), (96, 128, 32), (128, 32, 32), (32, 128, 32)]


def _operands(M, K, N, seed=0):
    return oracle.uniform((M, K), 31 + seed), oracle.uniform((N, K), 32 + seed)


def _check(A, Bt, Cm, C0=None, with_oracle=False, what=""):
    B = np.ascontiguousarray(Bt.T)
    C64, S = oracle.gemm_f64(A, B)
    base = 0.0 if C0 is None else C0.astype(np.float64)
    S = S + (0.0 if C0 is None else np.abs(C0))
    err = float(np.max(np.abs(Cm.astype(np.float64) - base - C64) / np.maximum(S, 1e-300))) if Cm.size else 0.0
    assert err <= TIGHT, (what, err)
    if with_oracle:
        ref = oracle.cake_sgemm(A, B, 4, oracle.make_cntx()).astype(np.float64)
        d = float(np.max(np.abs(Cm.astype(np.float64) - base - ref) / np.maximum(S, 1e-300)))
        assert d <= TOL, (what, d)


@pytest.mark.parametrize("tile", TILES, ids=lambda t: "x".join(map(str, t)))
@pytest.mark.parametrize("shape", [(512, 512, 512), (700, 520, 900), (333, 419, 517), (257, 1001, 255), (96, 70, 130)],
                         ids=lambda s: "x".join(map(str, s)))
def test_every_tile_shape(tile, shape):
    """Each macro-tile instantiation of the kernel that reads both operands along k: aligned and
    ragged sizes (K not a multiple of 4 or of the K step, M and N not multiples of the tile),
    without and with split-K, overwriting and accumulating."""
    M, K, N = shape
    A, Bt = _operands(M, K, N)
    for split in (0, 3):
        print(f"sgemm_nt tile={tile} split={split} M={M} K={K} N={N}", flush=True)
        Cm = np.full((M, N), np.nan, np.float32)
        cake.sgemm_nt(A, Bt, Cm, M, N, K, tile=tile + (split,))
        _check(A, Bt, Cm, what=(tile, shape, split))
        C0 = oracle.uniform((M, N), 33)
        acc = C0.copy()
        cake.sgemm_nt(A, Bt, acc, M, N, K, accumulate=True, tile=tile + (split,))
        _check(A, Bt, acc, C0, what=(tile, shape, split, "accumulate"))


def test_reference_shape_grid_against_the_oracle():
    """The reference's own shape list (src/util.cpp:11-13), every combination that keeps the job
    small, on the default routes (matrix-vector, streaming, macro-tile) against the oracle."""
    small = [1, 10, 96, 111, 960]
    for M, K, N in itertools.product(small, small, small):
        print(f"sgemm_nt edge M={M} K={K} N={N}", flush=True)
        A, Bt = _operands(M, K, N)
        Cm = np.full((M, N), np.nan, np.float32)
        cake.sgemm_nt(A, Bt, Cm, M, N, K)
        _check(A, Bt, Cm, with_oracle=True, what=(M, K, N))


@pytest.mark.parametrize("shape", [(1, 4096, 3000), (3000, 4096, 1), (1, 20000, 9), (2, 2048, 1024), (8, 1000, 2048),
                                   (32, 2111, 600), (2048, 1000, 8), (600, 2111, 32), (33, 1024, 2048), (2048, 1024, 33),
                                   (2111, 2111, 2111), (4099, 64, 515), (515, 4100, 4099),
                                   (16, 777, 8200), (8200, 777, 16), (4100, 1003, 13), (13, 1003, 4100), (16400, 300, 20)],
                         ids=lambda s: "x".join(map(str, s)))
def test_default_routes(shape):
    """One row on either side (matrix-vector sweep), two rows (two-vector sweep), up to 32 rows on
    either side (streaming kernel, the result written transposed for few rows of Bt), and larger
    products (macro-tiles), overwriting and accumulating, run-to-run identical."""
    M, K, N = shape
    A, Bt = _operands(M, K, N, 1)
    print(f"sgemm_nt route M={M} K={K} N={N}", flush=True)
    Cm = np.full((M, N), np.nan, np.float32)
    cake.sgemm_nt(A, Bt, Cm, M, N, K)
    _check(A, Bt, Cm, with_oracle=M * N * K < 3e9, what=shape)
    C0 = oracle.uniform((M, N), 34)
    acc = C0.copy()
    cake.sgemm_nt(A, Bt, acc, M, N, K, accumulate=True)
    _check(A, Bt, acc, C0, what=(shape, "accumulate"))
    again = np.full((M, N), np.nan, np.float32)
    cake.sgemm_nt(A, Bt, again, M, N, K)
    assert np.array_equal(again, Cm)


def test_random_shapes_against_fp64():
    rng = np.random.default_rng(77)
    pick = lambda: int(rng.choice([1, 2, 3, 17, 31, 33, 64, 65, 100, 255, 257, 511, 513, 700, 1030]))
    deep = lambda: int(rng.choice([1, 3, 31, 32, 33, 63, 64, 65, 100, 255, 257, 1000, 2050, 4099]))
    for case in range(80):
        M, N, K = pick(), pick(), deep()
        A, Bt = _operands(M, K, N, 100 + case)
        accumulate = case % 3 == 0
        C0 = oracle.uniform((M, N), 500 + case)
        Cm = C0.copy() if accumulate else np.full((M, N), np.nan, np.float32)
        print(f"sgemm_nt random case {case}: M={M} K={K} N={N} accumulate={accumulate}", flush=True)
        cake.sgemm_nt(A, Bt, Cm, M, N, K, accumulate=accumulate)
        _check(A, Bt, Cm, C0 if accumulate else None, what=(case, M, N, K))


def test_empty_and_degenerate():
    A, Bt = _operands(5, 7, 3)
    Cm = np.full((5, 3), 2.0, np.float32)
    cake.sgemm_nt(A, Bt, Cm, 5, 3, 0)                       # empty sum: zeros
    assert np.array_equal(Cm, np.zeros((5, 3), np.float32))
    Cm = np.full((5, 3), 2.0, np.float32)
    cake.sgemm_nt(A, Bt, Cm, 5, 3, 0, accumulate=True)      # ... or C as it was
    assert np.array_equal(Cm, np.full((5, 3), 2.0, np.float32))
    cake.sgemm_nt(A, Bt, Cm, 0, 3, 7)                       # nothing to do
    with pytest.raises(cake.CakeHipError):
        cake.sgemm_nt(A, Bt, Cm, -1, 3, 7)


def test_device_operands_at_odd_addresses():
    """Device operands 4, 8 and 12 bytes off a 16-byte boundary that end exactly at the end of
    their allocations: the 16-byte loads along k need 4-byte alignment only and never read past
    an operand."""
    import torch
    dev = torch.device("cuda:0")
    for (M, K, N) in [(257, 1001, 255), (130, 67, 131), (96, 30, 200)]:
        A, Bt = _operands(M, K, N, 7)
        for shift in (1, 2, 3):
            print(f"sgemm_nt odd address M={M} K={K} N={N} shift={shift}", flush=True)
            ta = torch.empty(M * K + shift, dtype=torch.float32, device=dev)
            tb = torch.empty(N * K + shift, dtype=torch.float32, device=dev)
            tc = torch.full((M * N + shift,), float("nan"), dtype=torch.float32, device=dev)
            ta[shift:].copy_(torch.from_numpy(A).reshape(-1))
            tb[shift:].copy_(torch.from_numpy(Bt).reshape(-1))
            cake.sgemm_nt(ta[shift:], tb[shift:], tc[shift:], M, N, K, tile=(64, 64, 32, 0))
            torch.cuda.synchronize()
            _check(A, Bt, tc[shift:].cpu().numpy().reshape(M, N), what=(M, K, N, shift))
