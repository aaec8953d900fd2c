"""Host-side checks of libcake_hip.so that need no GPU: the library loads and
exports every symbol include/cake_hip.h declares, the reference-compatible block
sizing and packed index maps agree with the oracle, and the GPU planner's
decisions are sane."""
import ctypes as C
import itertools
import re
from pathlib import Path

import numpy as np
import pytest

import cake_on_cpu_amd as cake
from cake_on_cpu_amd import _lib
import oracle

ROOT = Path(__file__).resolve().parent.parent
EDGE = [1, 10, 96, 111, 960, 2111]


def _cx(**kw):
    o = oracle.make_cntx(**kw)
    c = cake.CpuCntx(o.alpha_n, o.mr, o.nr, o.L1, o.L2, o.L3, o.ncores)
    return o, c


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "cake_hip.h").read_text()
    declared = set(re.findall(r"\b(cake_hip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 25
    lib = cake.load()
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in cake_hip.h but not exported"
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)


def test_struct_sizes_match_reference_layout():
    assert C.sizeof(cake.BlkDims) == 26 * 4
    assert [n for n, _ in cake.BlkDims._fields_] == oracle.BLK_FIELDS


def test_strerror_and_argument_errors():
    lib = cake.load()
    assert lib.cake_hip_strerror(0) == b"ok"
    assert b"argument" in lib.cake_hip_strerror(_lib.ERR_ARG)
    p = cake.Plan()
    assert lib.cake_hip_plan(0, 4, 4, cake.NA, None, C.byref(p)) == _lib.ERR_ARG
    assert lib.cake_hip_plan(4, 4, 4, 7, None, C.byref(p)) == _lib.ERR_ARG
    bad_tile = (C.c_int * 4)(123, 0, 0, 0)
    assert lib.cake_hip_plan(512, 512, 512, cake.NA, bad_tile, C.byref(p)) == _lib.ERR_ARG
    assert lib.cake_hip_last_error() != b""
    x = cake.BlkDims()
    assert lib.cake_hip_init_block_dims(8, 8, 8, 0, C.byref(cake.CpuCntx(1, 6, 16, 1, 1, 1, 1)), 0, 0, 0, 0, C.byref(x)) == _lib.ERR_ARG


@pytest.mark.parametrize("p", [1, 3, 8])
@pytest.mark.parametrize("sch", [cake.KMN, cake.MKN, cake.NKM, cake.NA])
def test_init_block_dims_equals_oracle(p, sch):
    for M, K, N in itertools.product(EDGE, EDGE, EDGE):
        ocx, ccx = _cx()
        want = oracle.init_block_dims(M, N, K, p, ocx, sch).as_dict()
        got = cake.init_block_dims(M, N, K, p, ccx, sch).as_dict()
        assert got == want, (M, K, N)
        assert ccx.alpha_n == ocx.alpha_n


@pytest.mark.parametrize("shape", [(8192, 8192, 8192), (1024, 1024, 1024), (65536, 1024, 128), (256, 2304, 100352)])
def test_init_block_dims_baseline_shapes(shape):
    M, K, N = shape
    for p in (8, 64):
        ocx, ccx = _cx()
        assert cake.init_block_dims(M, N, K, p, ccx).as_dict() == oracle.init_block_dims(M, N, K, p, ocx).as_dict()
    ocx, ccx = _cx()
    assert (cake.init_block_dims(500, 700, 300, 4, ccx, cake.KMN, None, 4, 48, 64, 160).as_dict()
            == oracle.init_block_dims(500, 700, 300, 4, ocx, oracle.KMN, 48, 64, 160).as_dict())


@pytest.mark.parametrize("p", [1, 3, 8])
@pytest.mark.parametrize("sch", [cake.KMN, cake.MKN, cake.NKM])
@pytest.mark.parametrize("shape", [(1, 1, 1), (10, 96, 111), (111, 10, 96), (96, 111, 10), (200, 150, 170)],
                         ids=lambda s: "x".join(map(str, s)))
def test_packed_index_maps_equal_oracle_layout(shape, sch, p):
    """Pack a matrix of distinct integers with the oracle, then ask the library
    where each element lives: the host evaluation of the index map every pack
    kernel and packed loader uses."""
    M, K, N = shape
    ocx, ccx = _cx(L2=16 << 10, L3=256 << 10)  # small caches: several CB blocks even at these sizes
    xo = oracle.init_block_dims(M, N, K, p, ocx, sch)
    xc = cake.init_block_dims(M, N, K, p, ccx, sch)
    mats = {0: np.arange(1, M * K + 1, dtype=np.float32).reshape(M, K),
            1: np.arange(1, K * N + 1, dtype=np.float32).reshape(K, N),
            2: np.arange(1, M * N + 1, dtype=np.float32).reshape(M, N)}
    packed = {0: oracle.pack_A(mats[0], p, xo, ocx, sch), 1: oracle.pack_B(mats[1], p, xo, ocx, sch),
              2: oracle.pack_C(mats[2], p, xo, ocx, sch)}
    assert cake.cake_sgemm_packed_A_size(M, K, p, xc, ccx, sch) == packed[0].nbytes
    assert cake.cake_sgemm_packed_B_size(K, N, p, xc, ccx) == packed[1].nbytes
    assert cake.cake_sgemm_packed_C_size(M, N, p, xc, ccx, sch) == packed[2].nbytes
    for which, m in mats.items():
        rows, cols = m.shape
        seen = set()
        for r in range(rows):
            for c in range(cols):
                off = cake.packed_offset(which, r, c, M, N, K, p, xc, ccx, sch)
                assert 0 <= off < packed[which].size
                assert packed[which][off] == m[r, c], (which, r, c)
                seen.add(off)
        assert len(seen) == rows * cols
        # padding positions map to zeros of the oracle's buffer
        pr = xc.M_padded if which != 1 else K
        pc = xc.N_padded if which != 0 else K
        for r in range(rows, pr):
            off = cake.packed_offset(which, r, 0, M, N, K, p, xc, ccx, sch)
            assert packed[which][off] == 0
        for c in range(cols, pc):
            off = cake.packed_offset(which, 0, c, M, N, K, p, xc, ccx, sch)
            assert packed[which][off] == 0
        assert cake.packed_offset(which, pr, 0, M, N, K, p, xc, ccx, sch) == -1


# ---------------------------------------------------------------------------
# GPU planner (no device: plans for 256 CUs x 160 KB LDS)
# ---------------------------------------------------------------------------
def test_plan_baseline_shapes():
    big = cake.plan(8192, 8192, 8192)
    assert big.tile_m * big.tile_n >= 256 * 128 and big.split_k == 1 and big.tail_tiles == 0
    assert big.sched == cake.KMN and big.grid == big.tiles_m * big.tiles_n
    assert big.lds_bytes <= 160 * 1024 and big.vector_loads == 1
    assert big.flops == 2.0 * 8192 ** 3 and big.min_bytes == 4.0 * 3 * 8192 ** 2
    # a CB block of resident tiles must cut traffic far below one fetch per tile
    naive = 4.0 * (8192.0 * 8192 * (big.tiles_m + big.tiles_n) + 8192.0 * 8192)
    assert big.min_bytes <= big.model_bytes < naive / 3

    skinny = cake.plan(65536, 128, 1024)
    assert skinny.tile_n == 128 and skinny.tiles_n == 1
    assert skinny.sched == cake.MKN          # one tile column: walk down M, B panel shared

    conv = cake.plan(256, 100352, 2304)
    assert conv.tiles_m <= 2 and conv.tiles_n >= 392      # a thin strip of tiles along N
    assert conv.sched in (cake.NKM, cake.KMN)
    strip = cake.plan(256, 100352, 2304, cake.NA, (256, 256, 32, 0))
    assert strip.tiles_m == 1 and strip.sched == cake.NKM  # one tile row: walk along N, A shared

    small = cake.plan(1024, 1024, 1024)
    assert small.grid >= 128                 # enough workgroups to cover most of the 256 CUs


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (10, 111, 96), (2111, 960, 1), (7, 100000, 3), (300, 300, 100000)])
def test_plan_covers_any_shape(M, N, K):
    for sch in (cake.KMN, cake.MKN, cake.NKM, cake.NA):
        pl = cake.plan(M, N, K, sch)
        assert pl.tiles_m * pl.tile_m >= M and pl.tiles_n * pl.tile_n >= N
        assert (pl.tiles_m - 1) * pl.tile_m < M and (pl.tiles_n - 1) * pl.tile_n < N
        tiles = pl.tiles_m * pl.tiles_n
        assert pl.split_k >= 1 and pl.tail_split >= 1 and 0 <= pl.tail_tiles < tiles
        assert not (pl.split_k > 1 and pl.tail_tiles > 0)
        if pl.kernel == 4:   # short K: resident workgroups, as many as a CU's LDS holds, in whole rows of 8 XCDs
            per_cu = 5 if K <= 32 else 4
            assert pl.grid == (min(tiles, per_cu * pl.cus) + 7) // 8 * 8 and pl.split_k == 1 and pl.tail_tiles == 0
        elif pl.kernel == 5:   # one resident workgroup per CU walks over the 256 x 128 tiles
            assert pl.grid == (min(tiles, pl.cus) + 7) // 8 * 8 and pl.split_k == 1 and pl.tail_tiles == 0
        else:
            assert pl.grid == (tiles - pl.tail_tiles) * pl.split_k + pl.tail_tiles * pl.tail_split
        assert 1 <= pl.group <= max(pl.tiles_m, pl.tiles_n)
        assert pl.sched in (cake.KMN, cake.MKN, cake.NKM)
        if sch != cake.NA:
            assert pl.sched == sch
        assert pl.vector_loads == 1   # the 16-byte loader needs 4-byte alignment only


def test_plan_tail_split():
    """A thin last round (a few tiles left over when every CU has had the same number) is cut
    along K instead, where that saves more than the second kernel costs: the convolution GEMM
    leaves 32 of its 1568 tiles of 128 x 128 and 16 of its 784 tiles of 256 x 128."""
    conv = cake.plan(256, 100352, 2304, cake.NA, (128, 128, 32, 0))
    assert conv.split_k == 1 and conv.tail_tiles == 1568 % 256 and conv.tail_split == 8
    assert conv.grid == 1568 - 32 + 32 * 8
    conv = cake.plan(256, 100352, 2304, cake.NA, (256, 128, 32, 0))
    assert conv.split_k == 1 and conv.tail_tiles == 784 % 256 and conv.tail_split == 15   # 72 K steps in slices of 5
    assert conv.grid == 784 - 16 + 16 * 15
    auto = cake.plan(256, 100352, 2304)
    assert auto.tail_tiles > 0 and auto.grid == auto.tiles_m * auto.tiles_n + auto.tail_tiles * (auto.tail_split - 1)
    assert cake.plan(8192, 8192, 8192).tail_tiles == 0          # whole rounds: nothing to cut
    # 64 x 64 tiles: 784 = 3 x 256 + 16 on a walk of 36 steps are cut, 1568 = 6 x 256 + 32 on a walk of 8 are not
    assert cake.plan(128, 25088, 1152).tail_tiles == 16 and cake.plan(1024, 6272, 256).tail_tiles == 0
    assert cake.plan(256, 100352, 2304, cake.NA, (128, 128, 32, 1)).tail_tiles == 0   # explicit split is literal


def test_plan_tile_override():
    pl = cake.plan(4096, 4096, 4096, cake.KMN, (128, 128, 32, 0))
    assert (pl.tile_m, pl.tile_n, pl.tile_k) == (128, 128, 32)
    pl = cake.plan(4096, 4096, 4096, cake.KMN, (0, 0, 0, 4))
    assert pl.split_k == 4


def test_compute_without_gpu_fails_loudly():
    import torch
    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present")
    a = np.zeros((4, 4), np.float32)
    with pytest.raises(cake.CakeHipError) as e:
        cake.cake_sgemm(a, a, a.copy(), 4, 4, 4, 1)
    assert e.value.status == _lib.ERR_NO_DEVICE


def test_missing_library_fails_loudly(tmp_path):
    """No CPU fallback: without libcake_hip.so the package refuses to load, in a fresh
    interpreter so that this process keeps its own library."""
    import subprocess
    import sys
    code = (
        "import sys, pathlib\n"
        "sys.path.insert(0, %r)\n"
        "from cake_on_cpu_amd import _lib\n"
        "_lib.LIB_PATH = pathlib.Path(%r) / 'libcake_hip.so'\n"
        "import cake_on_cpu_amd as cake\n"
        "try:\n"
        "    cake.plan(8, 8, 8)\n"
        "except ImportError as e:\n"
        "    print('ImportError', 'no CPU fallback' in str(e))\n"
        "else:\n"
        "    print('loaded something')\n" % (str(Path(__file__).resolve().parents[1]), str(tmp_path)))
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert res.stdout.strip() == "ImportError True", (res.stdout, res.stderr[-500:])


def test_entry_points_reject_bad_arguments_before_touching_a_device():
    """Argument and range checks come first, so they read the same with or without a GPU:
    negative sizes, unknown schedules, NULL operands and operands of 2^31 elements or more
    (all index arithmetic of the path is int, like the reference's)."""
    lib = cake.load()
    buf = np.zeros(16, np.float32)
    ptr = buf.ctypes.data
    sgemm = lambda M, N, K, sch=cake.NA, a=ptr: lib.cake_hip_sgemm(a, ptr, ptr, M, N, K, sch, 0, None, None, None)
    assert sgemm(-1, 4, 4) == _lib.ERR_ARG
    assert sgemm(4, 4, 4, sch=9) == _lib.ERR_ARG
    assert sgemm(4, 4, 4, a=None) == _lib.ERR_ARG
    assert sgemm(0, 4, 4) == _lib.OK and sgemm(4, 0, 4) == _lib.OK            # nothing to compute
    assert sgemm(65536, 4, 32768) == _lib.ERR_RANGE                            # A has 2^31 elements
    assert sgemm(46341, 46341, 4) == _lib.ERR_RANGE                            # C has more than 2^31 - 1
    assert lib.cake_hip_sgemv(ptr, ptr, ptr, -1, 4, 1, 1, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_sgemv(ptr, ptr, ptr, 65536, 32768, 1, 1, None, None) == _lib.ERR_RANGE
    assert lib.cake_hip_sgemv(None, ptr, ptr, 4, 4, 1, 1, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_transpose(ptr, ptr, 2, 2, None, None) == _lib.ERR_ARG  # in place
    assert lib.cake_hip_transpose(ptr, None, 2, 2, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_transpose(ptr, ptr, 0, 5, None, None) == _lib.OK
    assert lib.cake_hip_linear_forward(ptr, ptr, None, ptr, -2, 4, 4, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_linear_forward(ptr, ptr, None, None, 2, 4, 4, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_linear_forward(ptr, ptr, None, ptr, 65536, 4, 32768, None, None) == _lib.ERR_RANGE
    assert lib.cake_hip_linear_backward(None, ptr, ptr, ptr, ptr, ptr, 2, 2, 2, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_conv2d(ptr, ptr, ptr, 1, 1, 2, 2, 1, 3, 3, 1, 0, 0, None, None, None) == _lib.ERR_ARG  # filter larger than image
    assert lib.cake_hip_conv2d(ptr, ptr, ptr, 1, 1, 4, 4, 1, 3, 3, 0, 0, 0, None, None, None) == _lib.ERR_ARG  # stride 0
    assert lib.cake_hip_conv2d(ptr, None, ptr, 1, 1, 4, 4, 1, 3, 3, 1, 0, 0, None, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_autotune(0, 4, 4, 1.0, None, None, None) == _lib.ERR_ARG
    assert lib.cake_hip_tune_save(None) == _lib.ERR_ARG
    assert lib.cake_hip_last_error() != b""


# ---------------------------------------------------------------------------
# the table of measured choices (no device needed to load, save or consult it)
# ---------------------------------------------------------------------------
def test_tune_table_load_lookup_save_clear(tmp_path):
    cake.tune_clear()
    try:
        default = cake.plan(4096, 4096, 4096).as_dict()
        src = tmp_path / "tuned.txt"
        src.write_text("# comment\n"
                       "4096 4096 4096 1 128 128 32 2 0 0.001\n"      # taken
                       "4096 4096 4096 0 64 64 64 1 1 0.002\n"        # taken (operands not 16-byte loadable)
                       "this line is not an entry\n"
                       "10 10 10 1 96 96 32 1 0 1.0\n"                # no such tile: skipped
                       "64 64 64 1 64 64 64 9 0 1.0\n")               # more slices than K steps: skipped
        assert cake.tune_load(src) == 2 and cake.tune_count() == 2
        tuned = cake.plan(4096, 4096, 4096).as_dict()
        assert (tuned["tile_m"], tuned["tile_n"], tuned["split_k"], tuned["tail_tiles"]) == (128, 128, 2, 0)
        assert tuned["grid"] == 32 * 32 * 2
        # an explicit override still wins, other products are untouched
        assert cake.plan(4096, 4096, 4096, cake.NA, (256, 128, 32, 0)).tile_m == 256
        assert cake.plan(4096, 4096, 4095).as_dict()["tile_m"] == cake.plan(4096, 4096, 4095, cake.NA, (0, 0, 0, 0)).tile_m
        dst = tmp_path / "saved.txt"
        cake.tune_save(dst)
        rows = [l.split() for l in dst.read_text().splitlines() if not l.startswith("#")]
        assert sorted(r[:9] for r in rows) == [["4096", "4096", "4096", "0", "64", "64", "64", "1", "1"],
                                               ["4096", "4096", "4096", "1", "128", "128", "32", "2", "0"]]
        cake.tune_clear()
        assert cake.tune_count() == 0 and cake.plan(4096, 4096, 4096).as_dict() == default
        assert cake.tune_load(dst) == 2          # a saved table loads back
        with pytest.raises(cake.CakeHipError):
            cake.tune_load(tmp_path / "missing.txt")
    finally:
        cake.tune_clear()


def test_plan_names_the_kernel_family():
    """Single rows or columns go to the matrix-vector kernels, up to 32 rows or columns against a
    wide operand (more rows against a large one, up to 112 where tiles would pad them) to the
    streaming kernels, the rest (and anything with a tile override) to the macro-tile kernel."""
    fam = lambda M, N, K, tile=None: cake.plan(M, N, K, tile=tile).kernel
    assert fam(1, 4096, 4096) == 1 and fam(4096, 1, 4096) == 1
    assert fam(16, 16384, 16384) == 2 and fam(32, 600, 256) == 2 and fam(2, 512, 300) == 2
    assert fam(32, 600, 255) == 0 and fam(17, 4096, 255) == 0   # a short K walk of few rows stays on the tile ...
    assert fam(16, 4096, 128) == 2 and fam(16, 4096, 127) == 0   # ... a single group of 16 rows streams from K = 128
    assert fam(16384, 16, 16384) == 3 and fam(512, 16, 64) == 3 and fam(16384, 32, 16384) == 3
    assert fam(512, 32, 64) == 0 and fam(4096, 17, 4096) == 0   # 17 to 32 columns: only against a large A
    assert fam(16384, 32, 4096) == 0 and fam(16384, 32, 8192) == 3   # (from 100 million elements on)
    # few columns on the macro-tiles get the 128 x 32 tile, with slices of about 1024 k and a workgroup per CU
    p = cake.plan(8192, 32, 4096)
    assert (p.kernel, p.tile_m, p.tile_n, p.split_k) == (0, 128, 32, 4)
    p = cake.plan(8192, 24, 8192)
    assert (p.tile_m, p.tile_n, p.split_k) == (128, 32, 8)       # rows of 8192 floats: two workgroups per CU
    p = cake.plan(32768, 32, 1024)
    assert (p.tile_m, p.tile_n, p.split_k) == (128, 32, 1)
    p = cake.plan(8192, 16, 4096)                                  # up to 16 columns: in the mid sizes only
    assert (p.kernel, p.tile_m, p.tile_n) == (0, 128, 32) and fam(16384, 16, 4096) == 3 and fam(4096, 8, 1024) == 3
    assert cake.plan(8192, 64, 4096).tile_n == 64
    # 17 to 32 rows below 100 million elements of B: the 32 x 128 tile (not against a narrow B)
    p = cake.plan(32, 8192, 8192)
    assert (p.kernel, p.tile_m, p.tile_n, p.split_k) == (0, 32, 128, 8)
    assert fam(24, 4096, 4096) == 0 and fam(32, 16384, 8192) == 2 and fam(16, 4096, 4096) == 2 and fam(32, 640, 20000) == 2
    assert fam(33, 16384, 16384) == 2 and fam(48, 8192, 8192) == 2 and fam(49, 8192, 8192) == 0
    assert fam(49, 16384, 16384) == 2 and fam(64, 10240, 10240) == 2 and fam(64, 9000, 9000) == 0
    # 65 to 80 and 97 to 112 rows, which the macro-tiles would pad to 96 and 128
    assert fam(65, 16384, 16384) == 2 and fam(80, 8192, 4096) == 2 and fam(80, 4096, 4096) == 0
    assert fam(81, 16384, 16384) == 0 and fam(96, 16384, 16384) == 0
    assert fam(97, 8192, 8192) == 2 and fam(112, 16384, 16384) == 2 and fam(112, 8192, 4096) == 0 and fam(113, 16384, 16384) == 0
    assert fam(33, 4096, 4096) == 0 and fam(16384, 33, 16384) == 0
    assert fam(16, 511, 4096) == 0 and fam(16, 4096, 127) == 0 and fam(16, 16, 100000) == 0
    assert fam(1024, 1024, 1024) == 0
    assert fam(4096, 4096, 64) == 4 and fam(4096, 4096, 65) == 0 and fam(1024, 1024, 64) == 4 and fam(960, 960, 64) == 0   # short K, a tile per CU
    assert fam(4096, 4096, 68) == 4 and fam(4096, 4096, 144) == 4 and fam(4096, 4096, 164) == 5 and fam(4096, 4096, 130) == 0
    assert fam(960, 960, 128) == 0
    assert fam(16, 16384, 16384, tile=(64, 64, 64)) == 0
    assert cake.KERNEL_NAMES[fam(8, 2048, 2048)] == "streaming, few rows"
    # the plan of a short-K product describes that launch: 64 x 64 tiles holding the whole K, at most
    # four resident workgroups per CU in whole rows of 8 XCDs, no K slices
    p = cake.plan(250, 100352, 64)
    assert (p.kernel, p.tile_m, p.tile_n, p.tile_k, p.threads, p.split_k, p.tail_tiles) == (4, 64, 64, 64, 256, 1, 0)
    assert (p.tiles_m, p.tiles_n) == (4, 1568) and p.grid == 4 * p.cus and p.grid % 8 == 0
    assert 4 * p.lds_bytes <= 160 * 1024
    # K up to 32: stages of 32 k with B loaded straight into LDS, five workgroups per CU
    q = cake.plan(250, 100352, 32)
    assert (q.kernel, q.tile_m, q.tile_n, q.tile_k, q.threads) == (4, 64, 64, 32, 256)
    assert q.grid == 5 * q.cus and 5 * q.lds_bytes <= 160 * 1024
    # K from 65 to 160 (a multiple of 4): stages of 32 k, both operands straight into LDS, four workgroups per CU
    q = cake.plan(250, 100352, 128)
    assert (q.kernel, q.tile_m, q.tile_n, q.tile_k, q.threads) == (4, 64, 64, 32, 256)
    assert q.grid == 4 * q.cus and 4 * q.lds_bytes <= 160 * 1024
    # a K below 1024 (a multiple of 4) on 256 x 128 tiles, two or more per CU and no thin last round: one
    # workgroup of 8 waves per CU walks over the tiles, 105 KB of LDS
    r = cake.plan(8192, 8192, 256)
    assert (r.kernel, r.tile_m, r.tile_n, r.tile_k, r.threads, r.split_k, r.tail_tiles) == (5, 256, 128, 32, 512, 1, 0)
    assert r.grid == r.cus and r.lds_bytes == (2 * 256 * 32 + 2 * 32 * 128 + 8 * 8 * 36) * 4 <= 160 * 1024
    assert fam(8192, 8192, 1020) == 5 and fam(8192, 8192, 1024) == 0 and fam(8192, 8192, 258) == 0 and fam(8192, 8190, 256) == 0
    assert fam(2048, 2048, 256) == 0                                      # 128 tiles of 256 x 128: nothing to walk to
    # where the 64 x 64 walks apply as well (K up to 160): the large tiles when K is whole stages of 32 and the
    # tiles fill three rounds or more (two from K = 96 on) to 90 %
    assert fam(8192, 8192, 64) == 5 and fam(8192, 8192, 32) == 5 and fam(4096, 4096, 160) == 5 and fam(4096, 4096, 96) == 5
    assert fam(4096, 4096, 64) == 4 and fam(8192, 8192, 48) == 4 and fam(5120, 5120, 64) == 4 and fam(8192, 8192, 16) == 4
    r = cake.plan(8192, 8192, 64)
    assert (r.tile_m, r.tile_n, r.threads, r.grid, r.split_k, r.tail_tiles) == (256, 128, 512, r.cus, 1, 0)
    assert fam(700, 900, 520, tile=(256, 128, 32, 1)) == 5              # the caller named the tile (and no K slices): any tile count
    assert fam(700, 900, 520, tile=(256, 128, 32, 3)) == 0              # K slices: the macro-tile kernel
    # (tiles 128 wide exist but lost every measurement: the choice never takes them)
    assert cake.plan(16384, 16384, 16).tile_n == 64 and cake.plan(2048, 2048, 16).tile_n == 64
    # the tile sequence runs in bands: all tile rows of a product up to 16 of them, else 4, 8 or 16
    # tile rows, lower for wider products
    assert p.group == 4 and cake.plan(1024, 50176, 64).group == 16
    assert cake.plan(16384, 16384, 16).group == 4 and cake.plan(8192, 8192, 24).group == 8
    assert cake.plan(16384, 4096, 16).group == 16


def test_default_schedule_resolves_accumulate_by_the_reference_rule(monkeypatch):
    """cake_sgemm(sch=NA, beta=1): the accumulate flag handed to the C-ABI follows
    init_block_dims on the caller's cntx and p (src/cake_sgemm.cpp:34-35,114), on the unpacked
    path exactly as on the packed one, not the GPU planner's tile order."""
    from cake_on_cpu_amd import api
    real = cake.load()
    seen = {}

    class Recorder:
        def __getattr__(self, name):
            return getattr(real, name)

        def cake_hip_sgemm(self, A, B, Cm, M, N, K, sch, accumulate, ov, stream, secs):
            seen["unpacked"] = (sch, accumulate)
            return 0

        def cake_hip_sgemm_packed(self, A, B, Cm, M, N, K, p, x, cx, pa, pb, accumulate, stream, secs):
            seen["packed"] = accumulate
            return 0

    monkeypatch.setattr(api, "load", lambda: Recorder())
    ocx = oracle.make_cntx()
    for (M, N, K, p) in [(1024, 1024, 1024, 8), (512, 3000, 256, 4), (300, 300, 3000, 4), (64, 4096, 512, 4),
                         (960, 960, 111, 4), (96, 2111, 111, 8)]:
        cx = cake.CpuCntx()
        cx.alpha_n, cx.mr, cx.nr, cx.L1, cx.L2, cx.L3, cx.ncores = 1.0, ocx.mr, ocx.nr, ocx.L1, ocx.L2, ocx.L3, ocx.ncores
        want = oracle.init_block_dims(M, N, K, p, ocx, oracle.NA).sch != oracle.KMN
        big = np.zeros(max(M * K, K * N, M * N) + 4096 * 64, np.float32)
        for beta in (0.0, 1.0):
            api.cake_sgemm(big, big, big, M, N, K, p, cx, None, False, False, 1.0, beta)
            api.cake_sgemm(big, big, big, M, N, K, p, cx, None, True, True, 1.0, beta)
            assert seen["unpacked"] == (cake.NA, int(want and beta != 0)), (M, N, K, p, beta)
            assert seen["packed"] == int(want and beta != 0)
