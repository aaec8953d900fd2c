"""GPU parity of cake_sgemm through the C-ABI against the oracle.

Bar (stated by the task): max |C - C_ref| / sum_k |a||b| <= 1e-4, where C_ref is
the oracle's cake_sgemm on the same seeded inputs; the fp64 product is checked
too, with the tighter bound a correct fp32 accumulation meets at these K."""
import itertools

import numpy as np
import pytest

import cake_on_cpu_amd as cake
import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-4
TIGHT = 5e-6
EDGE = [1, 10, 96, 111, 960, 2111]   # src/util.cpp:11-13
SCHEDS = [cake.KMN, cake.MKN, cake.NKM, cake.NA]


def _run(M, K, N, sch=cake.NA, p=4, tile=None, C0=None, beta=0.0, seedA=1, seedB=2):
    A, B = oracle.uniform((M, K), seedA), oracle.uniform((K, N), seedB)
    Cm = np.zeros((M, N), np.float32) if C0 is None else C0.copy()
    if tile is None:
        cake.cake_sgemm(A, B, Cm, M, N, K, p, None, None, False, False, 1.0, beta, sch)
    else:
        import ctypes as C
        from cake_on_cpu_amd import _lib
        ov = (C.c_int * 4)(*tile)
        acc = int(beta != 0)
        _lib.check(cake.load().cake_hip_sgemm(A.ctypes.data, B.ctypes.data, Cm.ctypes.data, M, N, K, sch, acc,
                                              ov, None, None), "cake_hip_sgemm")
    return A, B, Cm


def _check(A, B, Cm, ref=None, what=""):
    C64, S = oracle.gemm_f64(A, B)
    err = oracle.max_rel_err(Cm, C64, S)
    assert err <= TOL and err <= TIGHT, (what, err)
    if ref is not None:
        d = float(np.max(np.abs(Cm.astype(np.float64) - ref) / np.maximum(S, 1e-300)))
        assert d <= TOL, (what, d)


@pytest.mark.parametrize("sch", SCHEDS)
def test_edge_shape_grid(sch):
    """The reference's own shape list: every combination that keeps the job small,
    against the oracle run with the same schedule."""
    small = [1, 10, 96, 111, 960]
    for M, K, N in itertools.product(small, small, small):
        print(f"sgemm edge M={M} K={K} N={N} sch={sch}", flush=True)
        A, B, Cm = _run(M, K, N, sch)
        ref = oracle.cake_sgemm(A, B, 4, oracle.make_cntx(), sch=sch)
        _check(A, B, Cm, ref, (M, K, N, sch))


@pytest.mark.parametrize("shape", [(2111, 2111, 2111), (2111, 96, 111), (111, 2111, 96), (96, 111, 2111),
                                   (1, 2111, 10), (2111, 1, 960), (10, 960, 2111)],
                         ids=lambda s: "x".join(map(str, s)))
def test_edge_shapes_with_2111(shape):
    M, K, N = shape
    for sch in (cake.KMN, cake.NA):
        print(f"sgemm edge M={M} K={K} N={N} sch={sch}", flush=True)
        A, B, Cm = _run(M, K, N, sch)
        ref = oracle.cake_sgemm(A, B, 8, oracle.make_cntx(), sch=sch)
        _check(A, B, Cm, ref, (shape, sch))


TILES = [(256, 256, 32), (256, 128, 32), (128, 256, 32), (128, 128, 32), (64, 64, 32), (64, 64, 64), (96, 128, 32), (128, 32, 32), (32, 128, 32)]


@pytest.mark.parametrize("tile", TILES, ids=lambda t: "x".join(map(str, t)))
@pytest.mark.parametrize("shape", [(512, 512, 512), (700, 520, 900), (333, 419, 517), (257, 1000, 255)],
                         ids=lambda s: "x".join(map(str, s)))
def test_every_tile_shape(tile, shape):
    """Each macro-tile instantiation, on aligned (16-byte loader) and ragged
    (scalar loader) operands, with the planner's choice of K slices, a single one (on 256 x 128
    tiles with K a multiple of 4 that is the kernel of resident workgroups) and three."""
    M, K, N = shape
    for split in (0, 1, 3):
        print(f"sgemm tile={tile} split={split} M={M} K={K} N={N}", flush=True)
        A, B, Cm = _run(M, K, N, cake.KMN, tile=tile + (split,))
        _check(A, B, Cm, None, (tile, shape, split))


TAIL_CASES = [  # (shape M,K,N; tile) -- every CU gets the same number of tiles and a few are left over, on a K
    # walk long enough for cutting them to pay
    ((1100, 1500, 1100), (64, 64, 64)), ((1100, 1497, 1099), (64, 64, 32)),
    ((2900, 512, 2900), (128, 128, 32)), ((4352, 1024, 2048), (256, 128, 32)),
    ((2048, 1024, 4352), (128, 256, 32)), ((4352, 512, 4096), (256, 256, 32)), ((3168, 512, 2048), (96, 128, 32)),
    ((33000, 1536, 30), (128, 32, 32)),
]


@pytest.mark.parametrize("case", TAIL_CASES, ids=lambda c: "x".join(map(str, c[0])) + "_t" + "x".join(map(str, c[1][:2])))
def test_tail_split_shapes(case):
    """Shapes whose tile count leaves a thin last round: the planner cuts those
    tiles along K and a second kernel sums the slices in order."""
    (M, K, N), tile = case
    tile = tile + (0,)
    pl = cake.plan(M, N, K, cake.NA, tile)
    assert pl.tail_tiles > 0 and pl.tail_split > 1, pl.as_dict()
    print(f"sgemm tail M={M} K={K} N={N} plan={pl.as_dict()}", flush=True)
    A, B, Cm = _run(M, K, N, tile=tile)
    _check(A, B, Cm, None, case)
    C0 = oracle.uniform((M, N), 3)
    _, _, acc = _run(M, K, N, cake.MKN, tile=tile, C0=C0, beta=1.0)
    assert np.allclose(acc - Cm, C0, atol=2e-4)
    again = _run(M, K, N, tile=tile)[2]
    assert np.array_equal(again, Cm)


@pytest.mark.parametrize("shape", [(257, 1001, 255), (130, 67, 131), (512, 30, 512), (1, 5, 3), (300, 4099, 2)],
                         ids=lambda s: "x".join(map(str, s)))
def test_operands_at_odd_addresses(shape):
    """Device operands that start 4, 8 and 12 bytes off a 16-byte boundary, with sizes that are
    not multiples of 4: the 16-byte loader only needs 4-byte alignment, masks the K tail when it
    stores a stage, and must never read past the end of an operand."""
    import torch
    M, K, N = shape
    dev = torch.device("cuda:0")
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    C64, S = oracle.gemm_f64(A, B)
    for shift in (1, 2, 3):
        print(f"sgemm odd address M={M} K={K} N={N} shift={shift}", flush=True)
        # each operand ends exactly at the end of its allocation
        ta = torch.empty(M * K + shift, dtype=torch.float32, device=dev)
        tb = torch.empty(K * N + shift, dtype=torch.float32, device=dev)
        tc = torch.full((M * N + shift,), float("nan"), dtype=torch.float32, device=dev)
        ta[shift:].copy_(torch.from_numpy(A).reshape(-1))
        tb[shift:].copy_(torch.from_numpy(B).reshape(-1))
        assert ta[shift:].data_ptr() % 16 == 4 * shift
        cake.cake_sgemm(ta[shift:], tb[shift:], tc[shift:], M, N, K, 1)
        torch.cuda.synchronize()
        got = tc[shift:].cpu().numpy().reshape(M, N)
        assert oracle.max_rel_err(got, C64, S) <= TIGHT
        assert torch.isnan(tc[:shift]).all()      # nothing written in front of C


def test_very_long_k_takes_the_element_loader():
    """K so long that byte offsets inside a 256-row tile pass 2^31: the 16-byte loader does not
    apply and the per-element loader computes the product."""
    M, K, N = 8, 2_200_000, 8
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    assert cake.plan(M, N, K).vector_loads == 0   # byte offsets inside a 256-row tile would pass 2^31
    Cm = np.zeros((M, N), np.float32)
    print(f"sgemm long K M={M} K={K} N={N}", flush=True)
    cake.cake_sgemm(A, B, Cm, M, N, K, 1)
    C64, S = oracle.gemm_f64(A, B)
    assert oracle.max_rel_err(Cm, C64, S) <= TOL


@pytest.mark.parametrize("shape", [(2, 64, 512), (3, 300, 1000), (5, 1000, 4096), (8, 4096, 4097), (13, 777, 2050),
                                   (16, 2111, 16384), (16, 16384, 1024), (1, 100, 600), (9, 65, 515),
                                   (17, 300, 1000), (32, 1000, 2048), (33, 777, 2050), (48, 2111, 1030),
                                   (64, 4096, 1024), (50, 65, 513), (65, 300, 1000), (40, 300, 1000), (47, 4099, 600),
                                   (48, 16384, 4096), (33, 12000, 4100), (41, 7000, 7001), (49, 1000, 2048),
                                   (64, 8192, 12288), (49, 12301, 8200), (57, 10001, 10003),
                                   (65, 5000, 6100), (80, 4099, 8200), (73, 7001, 4500), (97, 8200, 8000),
                                   (112, 9001, 7300), (105, 4100, 16000)],
                         ids=lambda s: "x".join(map(str, s)))
def test_few_rows_times_wide_matrix(shape):
    """Up to 32 rows of A against a wide B, up to 48 against a large one, up to 64 against 100
    million elements and more, 65 to 80 and 97 to 112 where macro-tiles would pad the rows: the
    streaming kernels (B read once, one to seven groups of 16-row MFMAs; other products with
    more than 32 rows take the tile kernel), with K slices summed in order, ragged N and K,
    accumulation, and run-to-run identical sums."""
    M, K, N = shape
    print(f"sgemm few rows M={M} K={K} N={N}", flush=True)
    A, B, Cm = _run(M, K, N)
    _check(A, B, Cm, oracle.cake_sgemm(A, B, 4, oracle.make_cntx()).astype(np.float64), shape)
    C0 = oracle.uniform((M, N), 3)
    _, _, acc = _run(M, K, N, cake.MKN, C0=C0, beta=1.0)
    assert np.allclose(acc - Cm, C0, atol=2e-4)
    assert np.array_equal(_run(M, K, N)[2], Cm)


@pytest.mark.parametrize("shape", [(512, 64, 2), (1000, 300, 3), (4096, 1000, 5), (4097, 4096, 8), (2050, 777, 13),
                                   (16384, 2111, 16), (1024, 16384, 16), (600, 100, 1), (515, 65, 9),
                                   (1000, 300, 17), (5000, 4099, 4), (4096, 1000, 24), (2050, 777, 32),
                                   (513, 65, 31), (1000, 300, 33), (4096, 1000, 40), (2050, 777, 48), (513, 65, 47),
                                   (1000, 300, 49),
                                   # up to 16 columns against rows of 4096 k and more: B is turned into rows first
                                   (4097, 4100, 13), (8200, 4096, 16), (5000, 8192, 7), (4100, 4101, 16),
                                   # 17 to 32 columns below 100 million elements of A, up to 16 in the mid sizes: the 128 x 32
                                   # tile with its own K-slice rule
                                   (8200, 4096, 32), (5000, 4099, 20), (4097, 2050, 17), (16400, 2048, 31), (3000, 3000, 8),
                                   (33000, 1000, 24), (2049, 8200, 16)],
                         ids=lambda s: "x".join(map(str, s)))
def test_tall_matrix_times_few_columns(shape):
    """Few columns of B against a tall A: A streamed once along its rows, or on the 128 x 32
    macro-tile in its K slices; ragged M and K, K slices summed in order, accumulation, run-to-run
    identical sums."""
    M, K, N = shape
    print(f"sgemm few columns M={M} K={K} N={N}", flush=True)
    A, B, Cm = _run(M, K, N)
    _check(A, B, Cm, oracle.cake_sgemm(A, B, 4, oracle.make_cntx()).astype(np.float64), shape)
    C0 = oracle.uniform((M, N), 3)
    _, _, acc = _run(M, K, N, cake.MKN, C0=C0, beta=1.0)
    assert np.allclose(acc - Cm, C0, atol=2e-4)
    assert np.array_equal(_run(M, K, N)[2], Cm)


@pytest.mark.parametrize("shape", [(4096, 64, 4096), (3000, 33, 5000), (4100, 63, 3300), (5000, 1, 4000), (2000, 7, 9000),
                                   (256, 64, 100352), (9000, 4, 2111), (3584, 64, 3520), (3584, 65, 3520),
                                   # one to four tiles per CU: every workgroup has a single tile, surplus ones leave early
                                   (1024, 64, 1024), (2111, 10, 960), (1100, 33, 1500), (960, 7, 1100),
                                   # K up to 24 under very many tiles
                                   (4096, 16, 8200), (3333, 24, 7777), (8192, 25, 4096),
                                   # more than 16 tile rows against 12288 columns and more: bands of 4 tile rows,
                                   # 18 and 19 tile rows (neither a multiple of 4), ragged everything
                                   (1100, 16, 12300), (1160, 24, 12417),
                                   # K from 65 to 160, a multiple of 4: stages of 32 k straight into LDS (one to five
                                   # stages, the last one partial); other K there stay on the macro-tile kernel
                                   (1030, 68, 1100), (2048, 96, 2048), (1024, 128, 1024), (777, 132, 5000), (3001, 160, 1999),
                                   (4096, 100, 4100), (1100, 101, 1100), (1024, 164, 1024), (1160, 72, 12417)],
                         ids=lambda s: "x".join(map(str, s)))
def test_short_k_many_tiles(shape):
    """K of at most 64 under at least one 64 x 64 tile per CU: workgroups that walk over tiles with
    the next tile's operands in flight (K = 65 and fewer tiles stay on the macro-tile kernel),
    ragged M, N and K, overwriting and accumulating, run-to-run identical."""
    M, K, N = shape
    short = K <= 64 or (K <= 160 and K % 4 == 0)
    want = 4 if short and ((M + 63) // 64) * ((N + 63) // 64) >= cake.device_info().cus else 0
    assert cake.plan(M, N, K).kernel == want
    print(f"sgemm short K M={M} K={K} N={N}", flush=True)
    A, B, Cm = _run(M, K, N)
    _check(A, B, Cm, None, shape)
    C0 = oracle.uniform((M, N), 3)
    _, _, acc = _run(M, K, N, cake.MKN, C0=C0, beta=1.0)
    assert np.allclose(acc - Cm, C0, atol=2e-4)
    assert np.array_equal(_run(M, K, N)[2], Cm)


@pytest.mark.parametrize("shape", [(4096, 256, 4096), (4000, 516, 4092), (6144, 388, 4096), (2048, 32, 8192 * 2), (8192, 1020, 4096),
                                   # K up to 160 in whole stages of 32 under three rounds of tiles or more: taken from the 64 x 64 walks
                                   (8192, 64, 8192), (8192, 32, 8192), (6000, 96, 8192), (4096, 160, 4096),
                                   (4010, 36, 8100), (5000, 300, 4100), (4096, 1024, 4096), (4096, 258, 4096), (4000, 516, 4090)],
                         ids=lambda s: "x".join(map(str, s)))
def test_resident_workgroups_walk_256x128_tiles(shape, monkeypatch):
    """K below 1024 on 256 x 128 tiles, two or more per CU, K and N multiples of 4: one workgroup
    per CU walks over the tiles with both operands loaded straight into LDS and writes a finished
    tile out under the next one's first stage.  Ragged last tile rows and columns, a last stage of
    4 k, a single stage per tile (every unit then starts a tile and writes one out), rows of B and
    C that are not 16-byte aligned; the last four shapes stay on (or may stay on) the macro-tile
    kernel.  Same bits as that kernel: both sum k in order."""
    M, K, N = shape
    pl = cake.plan(M, N, K)
    if shape in [(4096, 256, 4096), (4000, 516, 4092), (6144, 388, 4096), (8192, 1020, 4096), (8192, 64, 8192), (8192, 32, 8192), (6000, 96, 8192), (4096, 160, 4096)]:
        assert pl.kernel == 5, pl.as_dict()
    if shape in [(4096, 1024, 4096), (4096, 258, 4096), (4000, 516, 4090)]:
        assert pl.kernel == 0, pl.as_dict()
    print(f"sgemm resident M={M} K={K} N={N} kernel={pl.kernel}", flush=True)
    import torch
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    tA, tB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()     # on the device: host operands of this size go through in blocks of rows

    def run(beta=0.0, sch=cake.NA, C0=None):
        tC = torch.full((M, N), float("nan"), device="cuda") if C0 is None else torch.from_numpy(C0).cuda()
        cake.cake_sgemm(tA, tB, tC, M, N, K, 4, None, None, False, False, 1.0, beta, sch)
        torch.cuda.synchronize()
        return tC.cpu().numpy()

    Cm = run()
    _check(A, B, Cm, None, shape)
    assert np.array_equal(run(), Cm)
    monkeypatch.setenv("CAKE_HIP_GEMM_ROUTE", "tile")
    assert np.array_equal(run(), Cm)
    monkeypatch.delenv("CAKE_HIP_GEMM_ROUTE")
    C0 = oracle.uniform((M, N), 3)
    acc = run(1.0, cake.MKN, C0)                               # accumulation: the macro-tile kernel
    assert np.allclose(acc - Cm, C0, atol=2e-4)


def test_random_shapes_against_fp64():
    """Seeded random shapes drawn around every dispatch boundary (a single row or column, up to 16
    and just past 16 rows or columns, below and above the 512 columns and 64 k where the streaming
    kernels start, ragged everything), each against the fp64 product with C prefilled."""
    rng = np.random.default_rng(2024)
    small = lambda: int(rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 31, 33]))
    mid = lambda: int(rng.integers(1, 700))
    wide = lambda: int(rng.choice([511, 512, 513, 600, 1023, 1030, 2049, 3001]))
    deep = lambda: int(rng.choice([1, 3, 63, 64, 65, 100, 255, 257, 1000, 2050, 4099]))
    for case in range(120):
        kind = case % 4
        if kind == 0: M, N, K = small(), wide(), deep()
        elif kind == 1: M, N, K = wide(), small(), deep()
        elif kind == 2: M, N, K = mid(), mid(), deep()
        else: M, N, K = small(), small(), int(rng.integers(1, 20000))
        print(f"sgemm random case {case}: M={M} K={K} N={N}", flush=True)
        A, B = oracle.uniform((M, K), 100 + case), oracle.uniform((K, N), 300 + case)
        C0 = oracle.uniform((M, N), 500 + case)
        beta = float(case % 3 == 0)
        Cm = C0.copy()
        # beta only counts under the M- and N-first schedules, as in the reference (K-first overwrites C)
        cake.cake_sgemm(A, B, Cm, M, N, K, 4, None, None, False, False, 1.0, beta, cake.MKN if beta else cake.NA)
        C64, S = oracle.gemm_f64(A, B)
        err = float(np.max(np.abs(Cm.astype(np.float64) - beta * C0 - C64) / (S + beta * np.abs(C0) + 1e-300)))
        assert err <= TIGHT, (case, M, N, K, err)


@pytest.mark.parametrize("shape", [(3000, 1500, 2000), (4096, 1024, 4096), (1100, 9000, 520), (2500, 300, 9000)],
                         ids=lambda s: "x".join(map(str, s)))
def test_large_host_operands_take_the_block_pipeline(shape):
    """A and C in host memory and 32 MB or more between them: blocks of rows are uploaded,
    multiplied and downloaded in a pipeline (ragged last block, K-first overwrite of a prefilled C);
    against fp64 on sampled rows, and twice in a row since buffers and events are reused."""
    M, K, N = shape
    print(f"sgemm host pipeline M={M} K={K} N={N}", flush=True)
    A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    rows = sorted({0, 1, 255, 256, M // 4, M // 2, (3 * M) // 4, M - 257, M - 2, M - 1})
    ref = A[rows].astype(np.float64) @ B.astype(np.float64)
    S = np.abs(A[rows]).astype(np.float64) @ np.abs(B).astype(np.float64)
    first = None
    for _ in range(2):
        Cm = np.full((M, N), np.nan, np.float32)
        cake.cake_sgemm(A, B, Cm, M, N, K, 1)
        assert not np.isnan(Cm).any()
        assert float(np.max(np.abs(Cm[rows] - ref) / S)) <= TIGHT
        if first is None:
            first = Cm
        else:
            assert np.array_equal(first, Cm)


def test_identity_all_ones_single_nonzero():
    n = 300
    B = oracle.uniform((n, 260), 5)
    out = np.zeros_like(B)
    cake.cake_sgemm(np.eye(n, dtype=np.float32), B, out, n, 260, n, 1)
    assert np.array_equal(out, B)
    out = np.zeros((70, 91), np.float32)
    cake.cake_sgemm(np.ones((70, 513), np.float32), np.ones((513, 91), np.float32), out, 70, 91, 513, 1)
    assert np.array_equal(out, np.full((70, 91), 513.0, np.float32))
    A = np.zeros((40, 50), np.float32)
    A[17, 23] = 2.0
    Bm = oracle.uniform((50, 60), 6)
    out = np.full((40, 60), 9.0, np.float32)
    cake.cake_sgemm(A, Bm, out, 40, 60, 50, 1)
    want = np.zeros((40, 60), np.float32)
    want[17] = 2.0 * Bm[23]
    assert np.array_equal(out, want)


def test_overwrite_and_accumulate_semantics():
    """K-first assigns whatever C held; M-/N-first add to C only when beta != 0
    (src/cake_sgemm.cpp:114, src/pack_ob.cpp:404) -- same as the oracle."""
    M, K, N = 200, 160, 240
    C0 = oracle.uniform((M, N), 3)
    cx = oracle.make_cntx()
    for sch in (cake.KMN, cake.MKN, cake.NKM):
        for beta in (0.0, 1.0):
            A, B, Cm = _run(M, K, N, sch, C0=C0, beta=beta)
            ref = oracle.cake_sgemm(A, B, 4, cx, Cinit=C0, beta=beta, sch=sch)
            C64, S = oracle.gemm_f64(A, B)
            d = float(np.max(np.abs(Cm.astype(np.float64) - ref) / (S + np.abs(C0))))
            assert d <= 1e-5, (sch, beta, d)
    # and the difference is exactly the old C where accumulation applies
    A, B, plain = _run(M, K, N, cake.MKN)
    _, _, acc = _run(M, K, N, cake.MKN, C0=C0, beta=1.0)
    assert np.allclose(acc - plain, C0, atol=1e-4)


def _cake_cntx(o):
    """The library's cntx struct with the fields of an oracle cntx."""
    cx = cake.CpuCntx()
    cx.alpha_n, cx.mr, cx.nr, cx.L1, cx.L2, cx.L3, cx.ncores = o.alpha_n, o.mr, o.nr, o.L1, o.L2, o.L3, o.ncores
    return cx


@pytest.mark.parametrize("shape,p", [((1024, 1024, 1024), 8), ((960, 111, 960), 4), ((512, 256, 3000), 4),
                                     ((96, 111, 2111), 8), ((300, 3000, 300), 4), ((64, 512, 4096), 4),
                                     ((4096, 512, 64), 4)],
                         ids=lambda s: "x".join(map(str, s)) if isinstance(s, tuple) else f"p{s}")
def test_default_schedule_decides_accumulation_like_the_reference(shape, p):
    """sch = NA, beta = 1 on a prefilled C: whether C is added to follows the schedule the
    reference resolves from cntx and p (src/cake_sgemm.cpp:34-35,114) -- M-/N-first for the
    first four shapes, K-first (assign) for the next two -- whatever order the GPU planner
    walks its tiles in (it differs from the reference's on six of the seven)."""
    M, K, N = shape
    print(f"sgemm NA beta=1 M={M} K={K} N={N} p={p}", flush=True)
    A, B = oracle.uniform((M, K), 21), oracle.uniform((K, N), 22)
    C0 = oracle.uniform((M, N), 23)
    ocx = oracle.make_cntx()
    ref, _, dims = oracle.cake_sgemm(A, B, p, ocx, Cinit=C0, beta=1.0, sch=cake.NA, return_time=True)
    C64, S = oracle.gemm_f64(A, B)
    for name, dev in (("host", False), ("device", True)):
        if dev:
            import torch
            tA, tB, tC = (torch.from_numpy(x).cuda() for x in (A, B, C0))
            cake.cake_sgemm(tA, tB, tC, M, N, K, p, _cake_cntx(ocx), None, False, False, 1.0, 1.0)
            torch.cuda.synchronize()
            Cm = tC.cpu().numpy()
        else:
            Cm = C0.copy()
            cake.cake_sgemm(A, B, Cm, M, N, K, p, _cake_cntx(ocx), None, False, False, 1.0, 1.0)
        d = float(np.max(np.abs(Cm.astype(np.float64) - ref) / (S + np.abs(C0))))
        assert d <= TOL and d <= 1e-5, (name, shape, dims.sch, d)
        adds = dims.sch != cake.KMN
        err = float(np.max(np.abs(Cm.astype(np.float64) - adds * C0 - C64) / (S + np.abs(C0))))
        assert err <= TIGHT, (name, shape, dims.sch, err)
    # the packed entry decides the same way (it always used the reference's rule)
    cx = _cake_cntx(ocx)
    x = cake.init_block_dims(M, N, K, p, cx)
    assert x.sch == dims.sch


def test_schedules_agree_and_are_deterministic():
    M, K, N = 777, 1030, 515
    outs = [_run(M, K, N, sch)[2] for sch in (cake.KMN, cake.MKN, cake.NKM)]
    # the reuse order only changes which workgroup computes a tile, not the sums
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    again = _run(M, K, N, cake.KMN)[2]
    assert np.array_equal(outs[0], again)
    s1 = _run(M, K, N, cake.KMN, tile=(128, 128, 32, 4))[2]
    s2 = _run(M, K, N, cake.KMN, tile=(128, 128, 32, 4))[2]
    assert np.array_equal(s1, s2)      # split-K reduces in a fixed order


def test_empty_and_degenerate():
    a = np.zeros((0, 5), np.float32)
    cake.cake_sgemm(a, np.zeros((5, 3), np.float32), np.zeros((0, 3), np.float32), 0, 3, 5, 1)
    out = np.full((4, 3), 7.0, np.float32)
    cake.cake_sgemm(np.zeros((4, 0), np.float32), np.zeros((0, 3), np.float32), out, 4, 3, 0, 1)
    assert not out.any()               # empty sum assigns zero in K-first
    # an empty sum under the default schedule is K-first as well: beta = 1 still assigns ...
    out = np.full((4, 3), 7.0, np.float32)
    cake.cake_sgemm(np.zeros((4, 0), np.float32), np.zeros((0, 3), np.float32), out, 4, 3, 0, 1, None, None,
                    False, False, 1.0, 1.0)
    assert not out.any()
    # ... and only an explicit M-first or N-first schedule keeps the C it starts from
    for sch in (cake.MKN, cake.NKM):
        out = np.full((4, 3), 7.0, np.float32)
        cake.cake_sgemm(np.zeros((4, 0), np.float32), np.zeros((0, 3), np.float32), out, 4, 3, 0, 1, None, None,
                        False, False, 1.0, 1.0, sch)
        assert (out == 7.0).all()
    sq = np.zeros((4, 4), np.float32)
    with pytest.raises(cake.CakeHipError):
        cake.cake_sgemm(sq, sq, sq.copy(), -1, 3, 5, 1)
    with pytest.raises(cake.CakeHipError):
        cake.cake_sgemm(np.zeros((4, 4), np.float32), np.zeros((4, 4), np.float32),
                        np.zeros((4, 4), np.float32), 4, 4, 4, 1, None, None, False, False, 1.0, 0.0, 9)


def test_calls_from_several_threads_give_the_single_thread_results():
    """Compute entry points serialise on the library's mutex (they share its workspaces): four
    threads issuing different products at once -- split-K, tail slices, the streaming kernels,
    host operands staged through the same buffers -- get bit for bit what one thread gets."""
    import threading
    shapes = [(777, 1030, 515), (64, 9000, 70), (1100, 1100, 1500), (16, 4096, 2048), (300, 40, 5000), (2048, 64, 3000),
              (1, 3000, 3000), (513, 257, 129)]
    alone = [_run(M, K, N, seedA=10 + i, seedB=20 + i)[2] for i, (M, K, N) in enumerate(shapes)]
    errors = []

    def worker(t):
        try:
            for rep in range(3):
                for j in range(len(shapes)):
                    i = (j + 2 * t + rep) % len(shapes)
                    M, K, N = shapes[i]
                    got = _run(M, K, N, seedA=10 + i, seedB=20 + i)[2]
                    if not np.array_equal(got, alone[i]):
                        errors.append((t, rep, shapes[i]))
        except Exception as e:     # noqa: BLE001 -- reported by the assertion below
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads: th.start()
    for th in threads: th.join()
    assert not errors, errors[:5]


def test_memcpy_helpers_round_trip_large_pageable_arrays():
    """cake_hip_memcpy_h2d / _d2h move large pageable arrays through the pinned staging buffers
    (several chunks, a ragged last one) and small ones with a plain copy: bit for bit either way."""
    import ctypes as C
    lib = cake.load()
    for n in (1000, (8 << 20) // 4 + 3, (70 << 20) // 4 + 12345):
        src = oracle.uniform(n, 77)
        back = np.zeros(n, np.float32)
        dev = C.c_void_p()
        assert lib.cake_hip_malloc(C.byref(dev), src.nbytes) == 0
        try:
            assert lib.cake_hip_memcpy_h2d(dev, C.c_void_p(src.ctypes.data), src.nbytes) == 0
            assert lib.cake_hip_memcpy_d2h(C.c_void_p(back.ctypes.data), dev, src.nbytes) == 0
        finally:
            lib.cake_hip_free(dev)
        assert np.array_equal(src, back), n
