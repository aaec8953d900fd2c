"""GPU parity of cake_sgemv, im2col / conv2d, pack/unpack and the seeded fill
through the C-ABI against the oracle.  Byte/index work (packing, im2col, fill)
is bit-exact; floating-point results meet max |y - ref| / sum|a||x| <= 1e-4."""
import subprocess
from pathlib import Path

import numpy as np
import pytest

import cake_on_cpu_amd as cake
from cake_on_cpu_amd import _lib
import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-4
TIGHT = 5e-6


# ---------------------------------------------------------------------------
# seeded fill
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("n,seed", [(1, 0), (1000, 1), (65537, 2), (1 << 20, 12345678901234)])
def test_fill_uniform_bit_exact(n, seed):
    out = np.empty(n, np.float32)
    cake.fill_uniform(out, seed)
    assert np.array_equal(out, oracle.uniform(n, seed))
    assert out.min() >= -1.0 and out.max() < 1.0


# ---------------------------------------------------------------------------
# GEMV
# ---------------------------------------------------------------------------
GEMV_SHAPES = [(1, 1), (8, 1), (13, 2111), (64, 7), (1000, 333), (1024, 1024), (4099, 517),
               (2048, 3000), (300, 70000), (70000, 36),
               (70000, 400), (70001, 300),     # more blocks of 256 columns than CUs: one launch or a few K slices
               (6, 200000), (9, 65536),        # few long rows: the row-major path cuts K into slices
               (50000, 8), (4097, 20), (333, 31)]  # very short rows: a thread per row


@pytest.mark.parametrize("M,K", GEMV_SHAPES)
def test_sgemv_column_major_matches_oracle(M, K):
    """The reference's contract: A[k*M + m], y accumulates (examples/cake_gemv.cpp:89-140)."""
    print(f"sgemv col-major M={M} K={K}", flush=True)
    A, x, y0 = oracle.uniform(M * K, 41), oracle.uniform(K, 42), oracle.uniform(M, 43)
    ref = oracle.cake_sgemv(A, x, 4, oracle.make_cntx(mr=8), y0=y0, M=M, K=K)
    y64, S = oracle.gemv_f64(A, x, M, K, col_major=True)
    y = y0.copy()
    cake.cake_sgemv(A, x, y, M, K, 4)
    S1 = S + np.abs(y0)
    assert np.max(np.abs(y - ref) / S1) <= TOL
    assert np.max(np.abs(y - (y64 + y0)) / S1) <= TIGHT
    cake.cake_sgemv(A, x, y, M, K, 4)             # accumulates again
    assert np.max(np.abs(y - (2 * y64 + y0)) / S1) <= 2 * TIGHT
    z = np.full(M, 5.0, np.float32)
    cake.cake_sgemv(A, x, z, M, K, 4, accumulate=False)
    assert np.max(np.abs(z - y64) / np.maximum(S, 1e-30)) <= TIGHT


@pytest.mark.parametrize("M,K", GEMV_SHAPES)
def test_sgemv_row_major(M, K):
    print(f"sgemv row-major M={M} K={K}", flush=True)
    A, x = oracle.uniform(M * K, 44), oracle.uniform(K, 45)
    y64, S = oracle.gemv_f64(A, x, M, K, col_major=False)
    y = np.full(M, 3.0, np.float32)
    cake.cake_sgemv(A, x, y, M, K, 1, row_major=True, accumulate=False)
    assert np.max(np.abs(y - y64) / np.maximum(S, 1e-30)) <= TIGHT
    cake.cake_sgemv(A, x, y, M, K, 1, row_major=True, accumulate=True)
    assert np.max(np.abs(y - 2 * y64) / np.maximum(S, 1e-30)) <= 2 * TIGHT
    # the same buffer read column-major is the transposed problem
    if M == K and M > 1:
        yc = np.zeros(M, np.float32)
        cake.cake_sgemv(A, x, yc, M, K, 1, accumulate=False)
        yT, ST = oracle.gemv_f64(A, x, M, K, col_major=True)
        assert np.max(np.abs(yc - yT) / ST) <= TIGHT
        assert np.max(np.abs(yc - y64)) > 1e-2


def test_sgemv_unaligned_views():
    """Operands that are not 16-byte aligned take the scalar-load kernels."""
    M, K = 516, 1028
    buf = oracle.uniform(M * K + 8, 46)
    xb = oracle.uniform(K + 8, 47)
    for off in (1, 3):
        A, x = buf[off:off + M * K], xb[off:off + K]
        for col in (True, False):
            y64, S = oracle.gemv_f64(np.ascontiguousarray(A), np.ascontiguousarray(x), M, K, col_major=col)
            y = np.zeros(M, np.float32)
            secs = np.zeros(1)
            st = cake.load().cake_hip_sgemv(A.ctypes.data, x.ctypes.data, y.ctypes.data, M, K, int(col), 0, None, None)
            assert st == 0
            assert np.max(np.abs(y - y64) / S) <= TIGHT


def test_sgemv_deterministic():
    M, K = 3000, 5000
    A, x = oracle.uniform(M * K, 48), oracle.uniform(K, 49)
    outs = []
    for _ in range(3):
        y = np.zeros(M, np.float32)
        cake.cake_sgemv(A, x, y, M, K, 1, accumulate=False)
        outs.append(y)
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


# ---------------------------------------------------------------------------
# im2col and convolution
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("geom", [
    (1, 3, 18, 18, 3, 3, 1, 0), (2, 5, 9, 13, 3, 3, 1, 1), (3, 4, 12, 12, 3, 3, 2, 1),
    (1, 2, 6, 7, 1, 1, 1, 0), (2, 4, 8, 8, 5, 3, 1, 2), (4, 16, 14, 14, 3, 3, 1, 1), (1, 1, 7, 30, 3, 3, 3, 0),
    # workgroups of 1024 columns that span many small images, columns that are no multiple of 4,
    # padding beyond the filter's reach, strides with padding, a filter width without an unrolled kernel
    (40, 3, 7, 7, 3, 3, 1, 1), (9, 2, 14, 14, 3, 3, 1, 1), (3, 2, 5, 5, 3, 3, 1, 0), (23, 2, 9, 11, 3, 3, 1, 2),
    (7, 3, 31, 29, 5, 5, 2, 2), (5, 2, 33, 40, 7, 7, 3, 3), (6, 2, 20, 21, 2, 4, 1, 1), (3, 1, 64, 64, 3, 3, 2, 0),
    (2, 3, 224, 224, 7, 7, 2, 3), (300, 1, 3, 3, 3, 3, 1, 1), (1500, 1, 1, 1, 1, 1, 1, 0), (2, 2, 40, 5, 11, 3, 4, 1),
    # rows too wide for the staged kernel's LDS: the kernel that loads every window from memory
    (1, 2, 5, 4100, 3, 3, 1, 1), (2, 1, 9, 2500, 5, 5, 2, 2),
], ids=str)
def test_im2col_bit_exact(geom):
    Bn, Cin, Hin, Win, Hf, Wf, stride, pad = geom
    inp = oracle.uniform((Bn, Cin, Hin, Win), 51)
    want = oracle.im2col(inp, Hf, Wf, stride, pad)
    got = np.full_like(want, np.nan)
    cake.im2col(inp, got, Bn, Cin, Hin, Win, Hf, Wf, stride, pad)
    assert np.array_equal(got, want)


def test_im_2_col_reference_signature():
    Cin, Hin, Win, Hf, Wf = 6, 20, 17, 3, 3
    inp = oracle.uniform((Cin, Hin, Win), 52)
    got = cake.im_2_col(inp, Wf, Hf, Win, Hin, Win - 2, Hin - 2, Cin, 4, 1)
    assert np.array_equal(got, oracle.im_2_col(inp, Hf, Wf, Hin - 2, Win - 2))
    with pytest.raises(ValueError):
        cake.im_2_col(inp, Wf, Hf, Win, Hin, Win, Hin, Cin)


CONV_GEOMS = [
    # batch, Cin, Hin, Win, Cout, Hf, Wf, stride, pad
    (2, 5, 10, 9, 7, 3, 3, 1, 1),        # Wout = 9: two-step path only
    (1, 8, 14, 12, 20, 3, 3, 1, 0),      # Wout = 10
    (3, 16, 12, 12, 32, 3, 3, 2, 1),     # Wout = 6
    (2, 64, 28, 28, 96, 3, 3, 1, 1),     # Wout = 28: gathered inside the GEMM
    (2, 8, 16, 16, 24, 3, 3, 1, 1),      # Wout = 16
    (3, 12, 18, 18, 40, 3, 3, 1, 0),     # Wout = 16, no padding
    (2, 4, 17, 17, 300, 3, 3, 2, 1),     # Wout = 9 ... stride 2
    (2, 4, 15, 16, 300, 3, 3, 2, 1),     # Wout = 8, stride 2, Cout over one tile
    (1, 16, 9, 12, 10, 1, 1, 1, 0),      # 1x1 filter, Wout = 12
    (2, 4, 12, 14, 9, 5, 3, 1, 2),       # 5x3 filter, pad 2, Wout = 16
    (4, 32, 14, 8, 64, 3, 3, 1, 1),      # Wout = 8
    (8, 64, 56, 56, 24, 1, 1, 1, 0),     # few output channels, many pixels: the 32-row tile
    (4, 96, 28, 28, 20, 3, 3, 1, 1),     # the same with a 3x3 filter
    (1, 4, 6, 8, 5, 3, 3, 3, 2),         # stride 3, pad 2, Wout = 4
    (2, 6, 10, 12, 12, 7, 7, 1, 3),      # 7x7, pad 3: the 16-byte row gather shifts by up to 3 either way
    (2, 8, 16, 16, 16, 5, 5, 1, 2),      # 5x5, pad 2, Wout = 16
    (3, 5, 5, 4, 8, 3, 3, 1, 1),         # Win = 4: the row gather's narrowest image
    # whole blocks of 32 channels at stride 1: the input read where it lies, a patch of it in LDS
    (3, 32, 14, 14, 40, 3, 3, 1, 1),     # Wout = 14 (rows of the product padded to 16), tiles across image borders
    (5, 64, 7, 7, 300, 3, 3, 1, 1),      # 7 x 7 maps: a tile spans three images; two row tiles of filters
    (2, 32, 13, 9, 33, 3, 3, 1, 0),      # no padding, Win = 9: the last 16 bytes of a row hang over its end
    (2, 96, 12, 20, 70, 5, 3, 1, 2),     # 5 x 3 filter, pad 2 (the left margin holds 2 zero columns)
    (2, 32, 30, 30, 16, 2, 2, 1, 1),     # 2 x 2 filter: Wout = 31; fewer taps than that kernel's walk takes, so the staged gather runs
    (2, 32, 30, 30, 16, 2, 4, 1, 1),     # 2 x 4 filter (an even number of taps: the block starts with a step on its own): Wout = 29
    (2, 32, 12, 20, 20, 1, 7, 1, 3),     # 1 x 7 and
    (2, 64, 20, 12, 20, 7, 1, 1, 3),     # 7 x 1: the fewest taps that kernel's walk takes
    (1, 32, 56, 56, 24, 3, 3, 1, 1),     # a full-width plane of 56 x 56: every row and column of the patch in use
    (34, 32, 32, 32, 72, 3, 3, 1, 1),    # 272 tiles: the 16 of the thin last round are computed in sub-tiles of 64 x 32 (two of the four row blocks in use)
    (34, 64, 32, 32, 40, 5, 3, 1, 2),    # the same with two channel blocks of 15 taps: two K slices per tile of the last round
    (34, 96, 32, 32, 300, 3, 3, 1, 1),   # 544 tiles in two rows, 32 in the last round: sub-tiles of both tile rows, the second 44 rows high
    (35, 32, 30, 30, 72, 3, 3, 1, 1),    # Wout = 30 in rows of 32, 263 tiles: the last of the 7 sub-tiled ones is half full
    (1, 3, 9, 8, 6, 9, 9, 1, 4),         # pad 4: stride 1 but past the row gather's limit
    (2, 16, 8, 8, 260, 3, 3, 1, 1),      # Cout over one tile with the row gather
    (2, 3, 12, 12, 16, 3, 3, 1, 1),      # RGB first layer: K = 27 is not a multiple of 4
    (3, 5, 8, 8, 7, 1, 1, 1, 0),         # 1x1, K = 5
    (2, 3, 17, 17, 33, 3, 3, 2, 1),      # stride 2, K = 27, Wout = 9 (two-step) ...
    (2, 3, 15, 16, 33, 3, 3, 2, 1),      # ... and Wout = 8 (gathered from the phase-split copy)
    (2, 8, 16, 16, 12, 1, 1, 2, 0),      # 1x1 stride 2: the pixels it reads are copied out densely, then a 1x1 layer at stride 1
    (3, 20, 15, 13, 70, 1, 1, 2, 0),     # ... odd sizes: 8 x 7 outputs a plane, 56 a multiple of 4, planes across tile borders
    (5, 7, 10, 11, 9, 1, 1, 3, 0),       # ... stride 3, 4 x 4 outputs, K = 7
    (4, 96, 28, 28, 128, 1, 1, 2, 0),    # ... 14 x 14 outputs on 96 channels: the kernels with a short K
    (2, 6, 9, 9, 5, 1, 1, 2, 1),         # 1x1 stride 2 with padding: staged like any other filter
    (2, 3, 32, 32, 16, 7, 7, 2, 3),      # 7x7 stride 2 pad 3 (a first layer), Wout = 16
    (1, 4, 33, 29, 6, 3, 3, 4, 1),       # stride 4 over a 3x3 filter: rows and phases skipped, Wout = 8
    (2, 2, 21, 27, 5, 2, 5, 3, 0),       # 2x5 filter, stride 3: Hf below and Wf above the stride, Wout = 8
    (2, 5, 19, 35, 9, 4, 4, 2, 1),       # even filter, stride 2, Wout = 17 -> two-step
    (1, 6, 18, 34, 9, 4, 4, 2, 1),       # even filter, stride 2, Wout = 17 ... and
    (1, 6, 18, 32, 9, 4, 4, 2, 1),       # ... Wout = 16: gathered
]


def test_conv2d_random_geometries():
    """Seeded random geometries (filters 1..7 square or not, stride 1..4, padding up to the filter,
    widths around multiples of 4) through the gather path, NCHW and matrix output, against the
    naive fp64 convolution."""
    rng = np.random.default_rng(77)
    done = 0
    while done < 60:
        Hf, Wf = int(rng.integers(1, 8)), int(rng.integers(1, 8))
        stride, pad = int(rng.integers(1, 5)), int(rng.integers(0, 4))
        Hin, Win = int(rng.integers(Hf, 40)), int(rng.integers(Wf, 40))
        Bn, Cin, Cout = int(rng.integers(1, 4)), int(rng.integers(1, 20)), int(rng.integers(1, 70))
        if Hin + 2 * pad < Hf or Win + 2 * pad < Wf:
            continue
        nchw = bool(done % 2)
        print(f"conv2d random {done}: b={Bn} Cin={Cin} {Hin}x{Win} Cout={Cout} {Hf}x{Wf} s={stride} p={pad} nchw={nchw}",
              flush=True)
        inp = oracle.uniform((Bn, Cin, Hin, Win), 700 + done)
        wt = oracle.uniform((Cout, Cin, Hf, Wf), 900 + done)
        ref64, S = oracle.conv_naive_f64(inp, wt, stride, pad)
        _, _, Hout, Wout = ref64.shape
        out = np.full((Bn, Cout, Hout, Wout) if nchw else (Cout, Bn * Hout * Wout), np.nan, np.float32)
        cake.conv2d(inp, wt, out, Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, out_nchw=nchw)
        got = out if nchw else out.reshape(Cout, Bn, Hout, Wout).transpose(1, 0, 2, 3)
        err = float(np.max(np.abs(got.astype(np.float64) - ref64) / np.maximum(S, 1e-300)))
        assert err <= TIGHT, (done, err)
        done += 1


def test_conv2d_random_geometries_whole_channel_blocks(monkeypatch):
    """Seeded random stride-1 geometries with 32, 64 or 96 input channels on the kernel that reads
    the input where it lies, a patch per channel block in LDS (CAKE_HIP_CONV_ROUTE=patch takes it
    wherever the geometry allows; by default only large layers do): filters of 8 to 25 taps, square or not, padding 0 to 4
    (also wider than the filter needs), maps from the filter's size to 60 pixels wide, tiles that
    straddle image rows and images, against the naive fp64 convolution; NCHW and matrix output,
    and the same result twice."""
    monkeypatch.setenv("CAKE_HIP_CONV_ROUTE", "patch")
    rng = np.random.default_rng(1234)
    done = refused = 0
    while done < 40:
        Hf, Wf = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        if Hf * Wf < 7:
            continue
        pad = int(rng.integers(0, 5))
        Hin, Win = int(rng.integers(max(1, Hf - 2 * pad), 40)), int(rng.integers(max(1, Wf - 2 * pad), 61))
        Bn, Cin, Cout = int(rng.integers(1, 5)), 32 * int(rng.integers(1, 4)), int(rng.integers(1, 300))
        if Hin * Win * Cin * Bn > 2_000_000:
            continue
        nchw = bool(done % 2)
        print(f"conv2d patch random {done}: b={Bn} Cin={Cin} {Hin}x{Win} Cout={Cout} {Hf}x{Wf} p={pad} nchw={nchw}", flush=True)
        inp = oracle.uniform((Bn, Cin, Hin, Win), 1700 + done)
        wt = oracle.uniform((Cout, Cin, Hf, Wf), 1900 + done)
        ref64, S = oracle.conv_naive_f64(inp, wt, 1, pad)
        _, _, Hout, Wout = ref64.shape
        shape = (Bn, Cout, Hout, Wout) if nchw else (Cout, Bn * Hout * Wout)
        out, again = np.full(shape, np.nan, np.float32), np.full(shape, np.nan, np.float32)
        cake.conv2d(inp, wt, out, Bn, Cin, Hin, Win, Cout, Hf, Wf, 1, pad, out_nchw=nchw)
        route = cake.last_conv_route()
        cake.conv2d(inp, wt, again, Bn, Cin, Hin, Win, Cout, Hf, Wf, 1, pad, out_nchw=nchw)
        got = out if nchw else out.reshape(Cout, Bn, Hout, Wout).transpose(1, 0, 2, 3)
        err = float(np.max(np.abs(got.astype(np.float64) - ref64) / np.maximum(S, 1e-300)))
        assert err <= TIGHT, (done, err)
        assert np.array_equal(out, again), done
        if route != cake.CONV_PATCH:      # a patch too large for that kernel: right all the same, but not counted
            refused += 1
            assert route == cake.CONV_GATHER and refused <= 40
            continue
        done += 1


@pytest.mark.parametrize("geom", CONV_GEOMS, ids=str)
@pytest.mark.parametrize("nchw", [False, True])
@pytest.mark.parametrize("route", ["two steps", "gather", "gather, input where it lies"])
def test_conv2d_matches_oracle(geom, nchw, route, monkeypatch):
    """The convolution routes (column matrix materialised first, as the reference does; gathered
    inside the GEMM by the library's own choice of kernel; gathered from the input where it lies
    wherever that kernel's geometry allows) against the naive fp64 convolution and against the
    oracle's own im2col -> cake_sgemm pipeline."""
    Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad = geom
    explicit = route == "two steps"
    if route == "gather, input where it lies":
        if Cin % 32 or stride != 1:
            pytest.skip("that kernel takes whole blocks of 32 channels at stride 1")
        monkeypatch.setenv("CAKE_HIP_CONV_ROUTE", "patch")
    print(f"conv2d geom={geom} nchw={nchw} route={route}", flush=True)
    inp = oracle.uniform((Bn, Cin, Hin, Win), 54)
    wt = oracle.uniform((Cout, Cin, Hf, Wf), 55)
    ref64, S = oracle.conv_naive_f64(inp, wt, stride, pad)
    _, _, Hout, Wout = ref64.shape
    out = np.full((Bn, Cout, Hout, Wout) if nchw else (Cout, Bn * Hout * Wout), np.nan, np.float32)
    cake.conv2d(inp, wt, out, Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, out_nchw=nchw,
                explicit_im2col=explicit)
    took = cake.last_conv_route()
    got = out if nchw else out.reshape(Cout, Bn, Hout, Wout).transpose(1, 0, 2, 3)
    assert np.max(np.abs(got - ref64) / np.maximum(S, 1e-30)) <= TIGHT
    if explicit:
        assert took == cake.CONV_TWO_STEP
    elif route == "gather, input where it lies" and took != cake.CONV_PATCH:
        pytest.skip(f"this geometry is outside that kernel's (route {took} ran, and was right)")
    cols = oracle.im2col(inp, Hf, Wf, stride, pad)
    cpu = oracle.cake_sgemm(wt.reshape(Cout, -1), cols, 4, oracle.make_cntx(), sch=oracle.KMN)
    cpu = cpu.reshape(Cout, Bn, Hout, Wout).transpose(1, 0, 2, 3)
    assert np.max(np.abs(got - cpu) / np.maximum(S, 1e-30)) <= TOL


@pytest.mark.parametrize("geom", [(8, 14, 12, 20, 3, 3, 1), (64, 34, 34, 96, 3, 3, 1), (3, 37, 29, 10, 5, 3, 1),
                                  (16, 33, 33, 24, 3, 3, 2), (40, 19, 23, 33, 1, 1, 1), (5, 30, 31, 7, 7, 7, 3)], ids=str)
def test_cake_sconv_accumulates_the_direct_convolution(geom):
    """cake_sconv (examples/cake_conv.cpp:765-848): one CHW image, no padding, the result added
    to what C holds (its micro-kernel starts from C, :36-47) -- against the naive fp64 convolution,
    against the oracle's im_2_col -> cake_sgemm sequence (the reference's own cross-check,
    conv_gemm_checker :1216-1234), on host and on device memory, and twice to see it add."""
    Cin, Hin, Win, Cout, Hf, Wf, s = geom
    Hout, Wout = (Hin - Hf) // s + 1, (Win - Wf) // s + 1
    print(f"cake_sconv geom={geom}", flush=True)
    inp = oracle.uniform((Cin, Hin, Win), 61)
    wt = oracle.uniform((Cout, Cin, Hf, Wf), 62)
    C0 = oracle.uniform((Cout, Hout, Wout), 63)
    ref64, S = oracle.conv_naive_f64(inp[None], wt, s, 0)
    ref64, S = ref64[0], S[0]
    out = C0.copy()
    cake.cake_sconv(wt, inp, out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, 4)
    assert np.max(np.abs(out.astype(np.float64) - C0 - ref64) / (S + np.abs(C0))) <= TIGHT
    cake.cake_sconv(wt, inp, out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, 4)
    assert np.max(np.abs(out.astype(np.float64) - C0 - 2 * ref64) / (2 * S + np.abs(C0))) <= TIGHT
    import torch
    tw, ti, to = (torch.from_numpy(x).cuda() for x in (wt, inp, C0))
    cake.cake_sconv(tw, ti, to, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, 4)
    torch.cuda.synchronize()
    dev = to.cpu().numpy()
    assert np.max(np.abs(dev.astype(np.float64) - C0 - ref64) / (S + np.abs(C0))) <= TIGHT
    if s == 1:
        cols = oracle.im_2_col(inp, Hf, Wf, Hout, Wout)
        cpu = oracle.cake_sgemm(wt.reshape(Cout, -1), cols, 4, oracle.make_cntx(), sch=oracle.KMN).reshape(Cout, Hout, Wout)
        assert np.max(np.abs(dev - C0 - cpu) / (S + np.abs(C0))) <= TOL
    with pytest.raises(cake.CakeHipError):
        cake.cake_sconv(wt, inp, out, Wf, Hf, Win, Hin, Wout - 1, Hout, Cin, Cout, s, 4)


@pytest.mark.parametrize("filt", [(3, 3), (5, 3)], ids=str)
def test_cake_sconv_accumulates_through_the_last_round_of_the_patch_kernel(filt, monkeypatch):
    """cake_sconv on one tall image (32 channels, 700 x 50, no padding) through the kernel that
    reads the input where it lies: 262 tiles of 256 x 128, so the last 6 -- the last of them half
    full, 72 of the tile's 256 rows in use -- run as sub-tiles of 64 x 32 under the 3 x 3 filter
    and as K slices under the 5 x 3 one (two channel blocks), and both add to what C holds."""
    Hf, Wf = filt
    Cin, Hin, Win, Cout = 32 if filt == (3, 3) else 64, 700, 50, 72
    Hout, Wout = Hin - Hf + 1, Win - Wf + 1
    monkeypatch.setenv("CAKE_HIP_CONV_ROUTE", "patch")
    print(f"cake_sconv on the patch kernel: {Cin} x {Hin} x {Win} -> {Cout}, {Hf} x {Wf}", flush=True)
    inp = oracle.uniform((Cin, Hin, Win), 71)
    wt = oracle.uniform((Cout, Cin, Hf, Wf), 72)
    C0 = oracle.uniform((Cout, Hout, Wout), 73)
    ref64, S = oracle.conv_naive_f64(inp[None], wt, 1, 0)
    ref64, S = ref64[0], S[0]
    out = C0.copy()
    cake.cake_sconv(wt, inp, out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, 1, 4)
    assert cake.last_conv_route() == cake.CONV_PATCH
    assert np.max(np.abs(out.astype(np.float64) - C0 - ref64) / (S + np.abs(C0))) <= TIGHT
    cake.cake_sconv(wt, inp, out, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, 1, 4)
    assert np.max(np.abs(out.astype(np.float64) - C0 - 2 * ref64) / (2 * S + np.abs(C0))) <= TIGHT
    if filt == (3, 3):
        # the same last round cut along K instead: the same sums in another order
        monkeypatch.setenv("CAKE_HIP_CONV_TAIL", "slices")
        sliced = C0.copy()
        cake.cake_sconv(wt, inp, sliced, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, 1, 4)
        assert np.max(np.abs(sliced.astype(np.float64) - C0 - ref64) / (S + np.abs(C0))) <= TIGHT


@pytest.mark.parametrize("geom", [(16, 16, 56, 56, 256, 1, 1), (70, 7, 30, 30, 130, 1, 1), (256, 5, 21, 21, 100, 1, 1),
                                  (16, 64, 56, 56, 256, 1, 1), (16, 65, 56, 56, 256, 1, 1),
                                  # 65 to 256 channels, a multiple of 4: the batch runs in stages of 32 channels
                                  (16, 128, 28, 28, 200, 1, 1), (13, 100, 30, 30, 130, 1, 1), (40, 68, 21, 21, 100, 1, 1),
                                  (6, 256, 56, 56, 70, 1, 1), (32, 160, 14, 14, 512, 1, 1), (32, 192, 14, 14, 256, 1, 1),
                                  # planes that do not fill their last tile of 64 columns: tiles across image borders
                                  (32, 256, 14, 14, 1024, 1, 1), (37, 192, 14, 14, 300, 1, 1), (150, 72, 10, 6, 200, 1, 1),
                                  (13, 128, 26, 26, 640, 1, 1)],
                         ids=str)
@pytest.mark.parametrize("nchw", [False, True])
def test_conv2d_1x1_many_images(geom, nchw):
    """1 x 1 filters at stride 1 without padding and many tiles: every image is a plain product on
    the input as it lies, and the images are walked as a batch by the short-K kernels -- up to 64
    channels of any count, 65 to 256 when a multiple of 4 (65 stay on the gather path; so do 192
    channels on 32 maps of 14 x 14, fewer than two tiles per CU) -- HW a multiple of 64, of 4 only
    (beyond 64 channels the column tiles then run across image borders), and odd."""
    Bn, Cin, Hin, Win, Cout, Hf, Wf = geom
    print(f"conv2d 1x1 geom={geom} nchw={nchw}", flush=True)
    inp = oracle.uniform((Bn, Cin, Hin, Win), 58)
    wt = oracle.uniform((Cout, Cin, 1, 1), 59)
    HW = Hin * Win
    w64 = wt.reshape(Cout, Cin).astype(np.float64)
    x64 = inp.reshape(Bn, Cin, HW).astype(np.float64)
    ref64 = np.einsum("ok,bkp->bop", w64, x64)
    S = np.einsum("ok,bkp->bop", np.abs(w64), np.abs(x64))
    out = np.full((Bn, Cout, HW) if nchw else (Cout, Bn * HW), np.nan, np.float32)
    cake.conv2d(inp, wt, out, Bn, Cin, Hin, Win, Cout, 1, 1, 1, 0, out_nchw=nchw)
    batch_route = Cin != 65 and not (Cin == 192 and HW == 196 and Bn == 32)
    assert cake.last_conv_route() == (cake.CONV_SHORTK_BATCH if batch_route else cake.CONV_GATHER)
    got = out if nchw else out.reshape(Cout, Bn, HW).transpose(1, 0, 2)
    assert np.max(np.abs(got - ref64) / np.maximum(S, 1e-30)) <= TIGHT
    two_step = np.full_like(out, np.nan)
    cake.conv2d(inp, wt, two_step, Bn, Cin, Hin, Win, Cout, 1, 1, 1, 0, out_nchw=nchw, explicit_im2col=True)
    assert np.max(np.abs(two_step - out) / np.maximum(S.max(), 1e-30)) <= TIGHT


def test_conv2d_paths_agree_bitwise_layouts(monkeypatch):
    """The gather from a staged copy sums in the order of the column matrix: same bits as the two
    steps.  The kernel that reads the input where it lies sums channel block by channel block
    (another order, within the bar), the same on every run."""
    Bn, Cin, Hin, Win, Cout = 2, 24, 20, 20, 48
    inp, wt = oracle.uniform((Bn, Cin, Hin, Win), 56), oracle.uniform((Cout, Cin, 3, 3), 57)
    a = np.empty((Cout, Bn * 400), np.float32)
    b = np.empty_like(a)
    cake.conv2d(inp, wt, a, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1)
    cake.conv2d(inp, wt, b, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1, explicit_im2col=True)
    assert np.array_equal(a, b)
    Cin = 32
    inp, wt = oracle.uniform((Bn, Cin, Hin, Win), 56), oracle.uniform((Cout, Cin, 3, 3), 57)
    cake.conv2d(inp, wt, a, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1)
    cake.conv2d(inp, wt, b, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1, explicit_im2col=True)
    assert np.array_equal(a, b)          # by default a layer this small is gathered from the staged copy
    assert cake.last_conv_route() == cake.CONV_TWO_STEP
    monkeypatch.setenv("CAKE_HIP_CONV_ROUTE", "patch")
    cake.conv2d(inp, wt, a, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1)
    assert cake.last_conv_route() == cake.CONV_PATCH
    cake.conv2d(inp, wt, b, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1, explicit_im2col=True)
    _, S = oracle.conv_naive_f64(inp, wt, 1, 1)
    S = S.transpose(1, 0, 2, 3).reshape(Cout, -1)
    assert np.max(np.abs(a - b) / S) <= TIGHT
    again = np.empty_like(a)
    cake.conv2d(inp, wt, again, Bn, Cin, Hin, Win, Cout, 3, 3, 1, 1)
    assert np.array_equal(a, again)


@pytest.mark.parametrize("geom", [(3, 12, 18, 20, 40, 3, 3, 1, 1), (2, 8, 17, 22, 24, 3, 3, 2, 1),
                                  (2, 8, 16, 16, 12, 1, 1, 2, 0), (1, 6, 20, 13, 9, 5, 5, 1, 0)], ids=str)
def test_conv2d_with_a_caller_workspace_on_device_tensors(geom):
    """Device operands and a caller-owned workspace of cake_hip_conv2d_workspace bytes, offset so it
    is not 256-byte aligned: both paths must give what they give with the library's own buffer
    (stride 1 with padding, stride 2 with the phase-split staged input and an output width of 11,
    a 1x1 stride-2 layer, and an unpadded layer that reads the input as it lies)."""
    import torch
    dev = torch.device("cuda:0")
    Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad = geom
    Hout, Wout = (Hin + 2 * pad - Hf) // stride + 1, (Win + 2 * pad - Wf) // stride + 1
    inp, wt = oracle.uniform((Bn, Cin, Hin, Win), 58), oracle.uniform((Cout, Cin, Hf, Wf), 59)
    want = np.empty((Bn, Cout, Hout, Wout), np.float32)
    cake.conv2d(inp, wt, want, Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, out_nchw=True)
    need = cake.load().cake_hip_conv2d_workspace(Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad)
    assert need >= 4 * Cin * Hf * Wf * Bn * Hout * Wout
    ws = torch.empty((need + 3) // 4 + 1, dtype=torch.float32, device=dev)[1:]
    ti, tw = torch.from_numpy(inp).to(dev), torch.from_numpy(wt).to(dev)
    for explicit in (False, True):
        out = torch.full((Bn, Cout, Hout, Wout), float("nan"), dtype=torch.float32, device=dev)
        cake.conv2d(ti, tw, out, Bn, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, out_nchw=True,
                    workspace=ws, explicit_im2col=explicit)
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), want)


# ---------------------------------------------------------------------------
# packed layouts
# ---------------------------------------------------------------------------
def _cx(**kw):
    o = oracle.make_cntx(**kw)
    return o, cake.CpuCntx(o.alpha_n, o.mr, o.nr, o.L1, o.L2, o.L3, o.ncores)


PACK_SHAPES = [(1, 1, 1), (10, 96, 111), (111, 10, 96), (96, 111, 10), (960, 111, 96), (111, 960, 2111),
               (2111, 96, 111), (500, 700, 300), (1030, 1500, 1000)]


@pytest.mark.parametrize("p", [1, 3, 8])
@pytest.mark.parametrize("sch", [cake.KMN, cake.MKN, cake.NKM])
@pytest.mark.parametrize("shape", PACK_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_pack_unpack_bit_exact(shape, sch, p):
    M, K, N = shape
    print(f"pack M={M} K={K} N={N} sch={sch} p={p}", flush=True)
    small = M * K * N < 10 ** 7
    ocx, ccx = _cx(**({"L2": 32 << 10, "L3": 512 << 10} if small else {}))
    xo = oracle.init_block_dims(M, N, K, p, ocx, sch)
    xc = cake.init_block_dims(M, N, K, p, ccx, sch)
    A, B, Cm = oracle.uniform((M, K), 11), oracle.uniform((K, N), 12), oracle.uniform((M, N), 13)

    Ap = np.full(cake.cake_sgemm_packed_A_size(M, K, p, xc, ccx, sch) // 4, np.nan, np.float32)
    cake.pack_A(A, Ap, M, K, p, xc, ccx, sch)
    assert np.array_equal(Ap, oracle.pack_A(A, p, xo, ocx, sch))

    Bp = np.full(cake.cake_sgemm_packed_B_size(K, N, p, xc, ccx) // 4, np.nan, np.float32)
    cake.pack_B(B, Bp, K, N, p, xc, ccx, sch)
    assert np.array_equal(Bp, oracle.pack_B(B, p, xo, ocx, sch))

    Cp = np.full(cake.cake_sgemm_packed_C_size(M, N, p, xc, ccx, sch) // 4, np.nan, np.float32)
    cake.pack_C(Cm, Cp, M, N, p, xc, ccx, sch)
    assert np.array_equal(Cp, oracle.pack_C(Cm, p, xo, ocx, sch))

    back = np.full((M, N), np.nan, np.float32)
    cake.unpack_C(back, Cp, M, N, p, xc, ccx, sch)
    assert np.array_equal(back, Cm)

    # product straight from the packed operands, in every packed/plain combination
    C64, S = oracle.gemm_f64(A, B)
    for pa, pb in ((True, True), (True, False), (False, True)):
        out = np.full((M, N), np.nan, np.float32)
        st = cake.load().cake_hip_sgemm_packed((Ap if pa else A).ctypes.data, (Bp if pb else B).ctypes.data,
                                               out.ctypes.data, M, N, K, p, xc, ccx, int(pa), int(pb), 0, None, None)
        assert st == 0, cake.load().cake_hip_last_error()
        assert oracle.max_rel_err(out, C64, S) <= TIGHT, (pa, pb)


def _pack_round_trip(M, K, N, p, sch, ocx, ccx, device=False):
    """pack_A, pack_B, pack_C against the oracle bit for bit, unpack_C back to the values packed."""
    xo = oracle.init_block_dims(M, N, K, p, ocx, sch)
    xc = cake.init_block_dims(M, N, K, p, ccx, sch)
    A, B, Cm = oracle.uniform((M, K), 21), oracle.uniform((K, N), 22), oracle.uniform((M, N), 23)
    sizes = (cake.cake_sgemm_packed_A_size(M, K, p, xc, ccx, sch) // 4, cake.cake_sgemm_packed_B_size(K, N, p, xc, ccx) // 4,
             cake.cake_sgemm_packed_C_size(M, N, p, xc, ccx, sch) // 4)
    if device:
        import torch
        dev = torch.device("cuda:0")
        up = lambda a: torch.from_numpy(a).to(dev)
        dn = lambda t: t.cpu().numpy()
        new = lambda shape: torch.full(shape, float("nan"), dtype=torch.float32, device=dev)
    else:
        up = dn = lambda a: a
        new = lambda shape: np.full(shape, np.nan, np.float32)
    Ap, Bp, Cp, back = new((sizes[0],)), new((sizes[1],)), new((sizes[2],)), new((M, N))
    cake.pack_A(up(A), Ap, M, K, p, xc, ccx, sch)
    assert np.array_equal(dn(Ap), oracle.pack_A(A, p, xo, ocx, sch))
    cake.pack_B(up(B), Bp, K, N, p, xc, ccx, sch)
    assert np.array_equal(dn(Bp), oracle.pack_B(B, p, xo, ocx, sch))
    cake.pack_C(up(Cm), Cp, M, N, p, xc, ccx, sch)
    assert np.array_equal(dn(Cp), oracle.pack_C(Cm, p, xo, ocx, sch))
    cake.unpack_C(back, Cp, M, N, p, xc, ccx, sch)
    assert np.array_equal(dn(back), Cm)


# micro-panels of every tile height of the copy kernels (16, 24, 32 and 64 rows), panels wider than a
# tile row is long (one thread per element instead), sizes that are no multiple of 4
@pytest.mark.parametrize("sch", [cake.KMN, cake.MKN, cake.NKM])
@pytest.mark.parametrize("mr,nr", [(8, 12), (4, 48), (14, 24), (30, 8), (12, 64), (40, 100), (64, 128), (6, 160), (70, 16),
                                   (5, 7), (1, 1)])
def test_pack_unpack_other_micro_panels(mr, nr, sch):
    print(f"pack mr={mr} nr={nr} sch={sch}", flush=True)
    ocx, ccx = _cx(mr=mr, nr=nr, L2=256 << 10, L3=2 << 20)
    for (M, K, N), p in (((333, 270, 401), 3), ((130, 515, 259), 8)):
        _pack_round_trip(M, K, N, p, sch, ocx, ccx)


def test_pack_unpack_operands_past_the_streaming_threshold():
    """From 100 MB per operand on the copy kernels read and write past the caches; device operands."""
    ocx, ccx = _cx()
    _pack_round_trip(5200, 5200, 5200, 8, cake.KMN, ocx, ccx, device=True)


def test_packed_sgemm_through_reference_call_sequence():
    """examples/cake_conv.cpp:1028-1055: init_block_dims -> pack_A, pack_B -> cake_sgemm(..., 1, 1, 1, 0, KMN)."""
    M, K, N, p = 96, 8 * 9, 30 * 28, 10
    ocx, ccx = _cx()
    A, B = oracle.uniform((M, K), 61), oracle.uniform((K, N), 62)
    x = cake.init_block_dims(M, N, K, p, ccx, cake.KMN)
    Ap = np.empty(cake.cake_sgemm_packed_A_size(M, K, p, x, ccx, cake.KMN) // 4, np.float32)
    Bp = np.empty(cake.cake_sgemm_packed_B_size(K, N, p, x, ccx) // 4, np.float32)
    cake.pack_A(A, Ap, M, K, p, x, ccx, cake.KMN)
    cake.pack_B(B, Bp, K, N, p, x, ccx, cake.KMN)
    out = np.zeros((M, N), np.float32)
    cake.cake_sgemm(Ap, Bp, out, M, N, K, p, ccx, None, True, True, 1.0, 0.0, cake.KMN)
    ref = oracle.cake_sgemm(A, B, p, ocx, sch=oracle.KMN)
    C64, S = oracle.gemm_f64(A, B)
    assert np.max(np.abs(out - ref) / S) <= TOL
    assert oracle.max_rel_err(out, C64, S) <= TIGHT


# ---------------------------------------------------------------------------
# the C++ drop-in library, driven the way the reference's example mains drive it
# ---------------------------------------------------------------------------
def test_cpp_dropin_program():
    exe = _lib.LIB_DIR / "dropin_test"
    assert exe.exists(), "build it with make -C cake_on_cpu_amd/csrc"
    res = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600)
    print(res.stdout[-3000:], res.stderr[-2000:])
    assert res.returncode == 0 and "ALL PASS" in res.stdout


# ---------------------------------------------------------------------------
# committed outputs of the reference's own compiled code (tests/golden/reference_vectors.npz)
# ---------------------------------------------------------------------------
def test_device_kernels_against_reference_golden_vectors():
    """pack_A/B/C, unpack_C, im_2_col bit for bit and cake_sgemv within tolerance against what
    the reference's own pack_*.cpp, unpack_*.cpp, im_2_col and schedule_mvm produced."""
    from tests import golden_vectors
    meta, Z = golden_vectors.load()
    seed = meta["seeds"]
    ocx, ccx = _cx()
    for i, (M, K, N, p, sch) in enumerate(meta["pack"]):
        print(f"golden pack M={M} K={K} N={N} p={p} sch={sch}", flush=True)
        xc = cake.init_block_dims(M, N, K, p, ccx, sch)
        assert [getattr(xc, n) for n in oracle.BLK_FIELDS] == Z[f"pack{i}_dims"].tolist()
        xo = golden_vectors.blk_dims(Z[f"pack{i}_dims"])
        A, B, Cm = oracle.uniform((M, K), seed["A"]), oracle.uniform((K, N), seed["B"]), oracle.uniform((M, N), seed["C"])
        Ap = np.full(cake.cake_sgemm_packed_A_size(M, K, p, xc, ccx, sch) // 4, np.nan, np.float32)
        cake.pack_A(A, Ap, M, K, p, xc, ccx, sch)
        assert np.array_equal(Ap, Z[f"pack{i}_A"])
        Bp = np.full(cake.cake_sgemm_packed_B_size(K, N, p, xc, ccx) // 4, np.nan, np.float32)
        cake.pack_B(B, Bp, K, N, p, xc, ccx, sch)
        real = oracle.pack_B(np.ones((K, N), np.float32), p, xo, ocx, sch) != 0
        assert np.array_equal(Bp[real], Z[f"pack{i}_B"][real]) and not Bp[~real].any()
        Cp = oracle.uniform(cake.cake_sgemm_packed_C_size(M, N, p, xc, ccx, sch) // 4, seed["Cp"])
        back = np.full((M, N), 7.0, np.float32)
        cake.unpack_C(back, Cp, M, N, p, xc, ccx, sch)
        assert np.array_equal(back, Z[f"pack{i}_Cunpacked"])
        if not (sch == cake.NKM and xc.m_pad):
            Cpk = np.full(Cp.size, np.nan, np.float32)
            cake.pack_C(Cm, Cpk, M, N, p, xc, ccx, sch)
            assert np.array_equal(Cpk, Z[f"pack{i}_Cpacked"])
    for (M, K, p) in meta["gemv"]:
        print(f"golden gemv M={M} K={K}", flush=True)
        A, xv, y = oracle.uniform(M * K, seed["gemv_A"]), oracle.uniform(K, seed["gemv_x"]), oracle.uniform(M, seed["gemv_y"]).copy()
        cake.cake_sgemv(A, xv, y, M, K, p)
        ref = Z[f"gemv_{M}_{K}_{p}"]
        _, S = oracle.gemv_f64(A, xv, M, K, True)
        assert np.max(np.abs(y - ref) / np.maximum(S + 1.0, 1e-30)) <= 1e-6
    for (Cin, Hin, Win, Hf, Wf) in meta["im2col"]:
        print(f"golden im_2_col Cin={Cin} {Hin}x{Win} filter {Hf}x{Wf}", flush=True)
        inp = oracle.uniform((Cin, Hin, Win), seed["image"])
        cols = cake.im_2_col(inp, Wf, Hf, Win, Hin, Win - Wf + 1, Hin - Hf + 1, Cin)
        assert np.array_equal(cols, Z[f"im2col_{Cin}_{Hin}_{Win}_{Hf}_{Wf}"])


def test_pack_filters_is_the_references_layout():
    """pack_filters (examples/cake_conv.cpp:536-610) on the device against what the reference's own
    compiled function returned (tests/golden/conv_filter_vectors.npz) and against the oracle, bit for
    bit, with the blocks from the library's init_block_dims_conv; host and device operands."""
    import json
    import torch
    from pathlib import Path
    z = np.load(Path(__file__).resolve().parent / "golden" / "conv_filter_vectors.npz", allow_pickle=False)
    meta = json.loads(bytes(z["meta"]).decode())
    for i, (Cin, Cout, Hin, Win, p, L2) in enumerate(meta["cases"]):
        print(f"pack_filters case {i}: Cin={Cin} Cout={Cout} {Hin}x{Win} p={p} L2={L2}", flush=True)
        cx = cake.CpuCntx(alpha_n=1.0, mr=6, nr=16, L1=48 << 10, L2=L2, L3=32 << 20, ncores=8)
        x = cake.init_block_dims_conv(3, 3, Win, Hin, Win - 2, Hin - 2, Cin, Cout, 1, p, cx)
        assert [getattr(x, n) for n in oracle.BLK_FIELDS] == [int(v) for v in z[f"case{i}_dims"]]
        F = oracle.uniform((Cout, Cin * 9), meta["filter_seed"])
        Fp = np.full(x.M_padded * Cin * 9, np.nan, np.float32)
        cake.pack_filters(F, Fp, Cout, Cin * 9, p, x, cx)
        assert np.array_equal(Fp, z[f"case{i}_packed"]), i
        tF = torch.from_numpy(F).cuda()
        tFp = torch.full((x.M_padded * Cin * 9,), float("nan"), dtype=torch.float32, device="cuda")
        cake.pack_filters(tF, tFp, Cout, Cin * 9, p, x, cx)
        assert np.array_equal(tFp.cpu().numpy(), Fp), i
    # other filter sizes than the reference's 3 x 3, against the oracle's restatement
    for (Cin, Cout, Hf, Wf, p, L2) in [(20, 50, 5, 3, 3, 8 << 10), (7, 200, 1, 1, 8, 1 << 20), (33, 9, 2, 4, 2, 16 << 10)]:
        cx = cake.CpuCntx(alpha_n=1.0, mr=6, nr=16, L1=48 << 10, L2=L2, L3=32 << 20, ncores=8)
        ocx = oracle.make_cntx(mr=6, nr=16, L2=L2)
        ocx.alpha_n = 1.0
        x = cake.init_block_dims_conv(Wf, Hf, 30, 30, 31 - Wf, 31 - Hf, Cin, Cout, 1, p, cx)
        ox = oracle.init_block_dims_conv(Wf, Hf, 30, 30, 31 - Wf, 31 - Hf, Cin, Cout, 1, p, ocx)
        taps = Hf * Wf
        F = oracle.uniform((Cout, Cin * taps), 77)
        Fp = np.full(x.M_padded * Cin * taps, np.nan, np.float32)
        cake.pack_filters(F, Fp, Cout, Cin * taps, p, x, cx, taps=taps)
        assert np.array_equal(Fp, oracle.pack_filters(F, Cin, taps, p, ox, ocx)), (Cin, Cout, Hf, Wf)


@pytest.mark.parametrize("geom", [(64, 34, 34, 100, 3, 3, 1, 4), (5, 21, 37, 130, 3, 3, 1, 3), (20, 19, 23, 50, 5, 3, 2, 3)], ids=str)
def test_cake_sconv_takes_packed_filters(geom):
    """cake_sconv with packedA (examples/cake_conv.cpp:791-799): filters from pack_filters give the
    very bits the plain filters give, host and device memory, and add to C like the plain call."""
    import torch
    Cin, Hin, Win, Cout, Hf, Wf, s, p = geom
    Hout, Wout = (Hin - Hf) // s + 1, (Win - Wf) // s + 1
    taps = Hf * Wf
    cx = cake.cake_query_cntx()
    F, In = oracle.uniform((Cout, Cin * taps), 81), oracle.uniform((Cin, Hin, Win), 82)
    C0 = oracle.uniform((Cout, Hout * Wout), 83)
    want = C0.copy()
    cake.cake_sconv(F, In, want, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cx)
    x = cake.init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cx)
    Fp = np.empty(x.M_padded * Cin * taps, np.float32)
    cake.pack_filters(F, Fp, Cout, Cin * taps, p, x, cx, taps=taps)
    got = C0.copy()
    cake.cake_sconv(Fp, In, got, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cx, packedA=True)
    assert np.array_equal(got, want)
    ref64, S = oracle.conv_naive_f64(In[None], F.reshape(Cout, Cin, Hf, Wf), s, 0)
    err = np.max(np.abs(got.reshape(Cout, Hout, Wout) - C0.reshape(Cout, Hout, Wout) - ref64[0]) / np.maximum(S[0], 1e-30))
    assert err <= TIGHT
    tFp, tIn, tC = torch.from_numpy(Fp).cuda(), torch.from_numpy(In).cuda(), torch.from_numpy(C0).cuda()
    cake.cake_sconv(tFp, tIn, tC, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cx, packedA=True)
    assert np.array_equal(tC.cpu().numpy(), want)
    # blocks that belong to another geometry are refused, nothing is computed
    other = cake.init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout + 40, s, p, cx)
    import ctypes
    assert cake.load().cake_hip_packed_filters_size(Cout, Cin, taps, p, ctypes.byref(other), ctypes.byref(cx)) == 0
