"""GPU parity of the transpose and of the linear layer (src/linear.cpp,
python/cake.py) through the C-ABI, against the oracle's restatement, plus the
reference's own run_tests sweep through libcake.so.

Bar: transpose bit-exact; products max |C - C_ref| / sum_k |a||b| <= 1e-4
against the oracle (and <= 5e-6 against fp64); bias sums within the bound any
fp32 summation order meets."""
import subprocess

import numpy as np
import pytest

import cake_on_cpu_amd as cake
import oracle
from cake_on_cpu_amd import _lib

pytestmark = pytest.mark.gpu

TOL = 1e-4
TIGHT = 5e-6


def _rel(got, ref64, S):
    return float(np.max(np.abs(got.astype(np.float64) - ref64) / np.maximum(S, 1e-300))) if got.size else 0.0


@pytest.mark.parametrize("shape", [(1, 1), (1, 1000), (1000, 1), (64, 64), (130, 77), (333, 1025), (2048, 4096)],
                         ids=lambda s: "x".join(map(str, s)))
def test_transpose_bit_exact(shape):
    K, N = shape
    A = oracle.uniform((K, N), 21)
    At = np.full((N, K), np.nan, np.float32)
    print(f"transpose K={K} N={N}", flush=True)
    cake.transpose_mat(A, At, K, N, 8, 8)
    assert np.array_equal(At, A.T)


# M (batch), K (in features), N (out features): aligned, ragged, thin, split-K and tail-split plans
LINEAR_SHAPES = [(1, 1, 1), (7, 5, 3), (64, 96, 48), (33, 130, 257), (128, 10, 960), (512, 512, 512),
                 (300, 2111, 96), (96, 4096, 100), (1100, 520, 1100), (16, 8192, 32),
                 # small batches: w streamed once as it lies (forward), grad_y . w by the few-rows kernel
                 (8, 1024, 4096), (3, 333, 1030), (16, 4099, 2048), (1, 64, 512), (13, 16390, 600), (16, 70, 5000),
                 (32, 1024, 2048), (20, 333, 1030), (17, 4099, 513), (33, 1024, 2048), (48, 2048, 1000), (40, 513, 600),
                 (49, 1024, 2048), (200, 1000, 4099), (64, 4096, 1000), (130, 77, 260), (131, 77, 260),
                 # the streaming kernel's three shapes: 16, 32 and 64 rows of w per workgroup, ragged everywhere
                 (16, 1003, 4100), (16, 777, 8200), (30, 1000, 8190), (9, 300, 16400), (24, 2050, 4097),
                 # 2 samples on long rows: one matrix-vector sweep over w for both
                 (2, 2048, 1024), (2, 4096, 2050), (2, 2052, 4097), (2, 16384, 2051), (2, 2048, 1023),
                 # a single sample: the row-major matrix-vector kernels (long rows, K slices, short rows, odd K)
                 (1, 8192, 300), (1, 20000, 8), (1, 24, 5000), (1, 2111, 777)]


@pytest.mark.parametrize("shape", LINEAR_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("with_bias", [True, False], ids=["bias", "nobias"])
def test_linear_forward(shape, with_bias):
    M, K, N = shape
    x, w = oracle.uniform((M, K), 11), oracle.uniform((N, K), 12)
    b = oracle.uniform((N,), 13) if with_bias else None
    y = np.full((M, N), np.nan, np.float32)
    print(f"linear forward M={M} K={K} N={N} bias={with_bias} plan={cake.plan(M, N, K).as_dict()}", flush=True)
    cake.linear_forward(x, w, b, y, M, N, K)
    ref = oracle.linear_forward(x, w, b)
    y64 = x.astype(np.float64) @ w.astype(np.float64).T + (b.astype(np.float64)[None, :] if with_bias else 0)
    S = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T + (np.abs(b)[None, :] if with_bias else 0)
    assert _rel(y, y64, S) <= TIGHT
    assert _rel(y, ref.astype(np.float64), S) <= TOL
    # the bias is added to the finished fp32 product, as the reference does: removing it
    # again gives the bias-free product to within one rounding of the sum
    if with_bias:
        y0 = np.empty_like(y)
        cake.linear_forward(x, w, None, y0, M, N, K)
        assert np.array_equal(y, y0 + b[None, :])


@pytest.mark.parametrize("shape", LINEAR_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_linear_backward(shape):
    M, K, N = shape
    x, w, g = oracle.uniform((M, K), 11), oracle.uniform((N, K), 12), oracle.uniform((M, N), 14)
    gx = np.full((M, K), np.nan, np.float32)
    gw = np.full((N, K), np.nan, np.float32)
    gb = np.full((N,), np.nan, np.float32)
    print(f"linear backward M={M} K={K} N={N}", flush=True)
    cake.linear_backward(g, x, w, gx, gw, gb, M, N, K)
    rx, rw, rb = oracle.linear_backward(g, x, w, np.zeros(N, np.float32))
    g64, x64, w64 = g.astype(np.float64), x.astype(np.float64), w.astype(np.float64)
    assert _rel(gx, g64 @ w64, np.abs(g64) @ np.abs(w64)) <= TIGHT
    assert _rel(gw, g64.T @ x64, np.abs(g64).T @ np.abs(x64)) <= TIGHT
    assert _rel(gx, rx.astype(np.float64), np.abs(g64) @ np.abs(w64)) <= TOL
    assert _rel(gw, rw.astype(np.float64), np.abs(g64).T @ np.abs(x64)) <= TOL
    assert _rel(gb, rb, np.abs(g64).sum(axis=0)) <= TIGHT
    # skipping outputs leaves the others bit-identical; the sums are run-to-run deterministic
    gx2 = np.empty_like(gx)
    cake.linear_backward(g, None, w, gx2, None, None, M, N, K)
    assert np.array_equal(gx2, gx)
    gw2, gb2 = np.empty_like(gw), np.empty_like(gb)
    cake.linear_backward(g, x, None, None, gw2, gb2, M, N, K)
    assert np.array_equal(gw2, gw) and np.array_equal(gb2, gb)


def test_linear_empty_dimensions():
    x, w, b = np.zeros((4, 0), np.float32), np.zeros((3, 0), np.float32), oracle.uniform((3,), 5)
    y = np.full((4, 3), np.nan, np.float32)
    cake.linear_forward(np.zeros(1, np.float32), np.zeros(1, np.float32), b, y, 4, 3, 0)   # K = 0: y = bias
    assert np.array_equal(y, np.broadcast_to(b, (4, 3)))
    gb = np.full((3,), np.nan, np.float32)
    cake.linear_backward(np.zeros(1, np.float32), None, None, None, None, gb, 0, 3, 5)     # M = 0: sums are 0
    assert np.array_equal(gb, np.zeros(3, np.float32))
    del x, w


def test_torch_module_matches_nn_linear():
    """cake_linear on ROCm tensors: device pointers go straight into the C-ABI on torch's
    stream; forward and all three gradients against torch's own layer in fp64."""
    import torch
    from cake_on_cpu_amd.torch_linear import cake_linear
    torch.manual_seed(0)
    dev = torch.device("cuda:0")
    for (batch, fin, fout, bias) in [((5, 7), 130, 77, True), ((256,), 512, 384, True), ((64,), 96, 200, False)]:
        print(f"cake_linear batch={batch} in={fin} out={fout} bias={bias}", flush=True)
        layer = cake_linear(fin, fout, bias=bias).to(dev)
        ref = torch.nn.Linear(fin, fout, bias=bias).to(dev).double()
        with torch.no_grad():
            ref.weight.copy_(layer.weight.double())
            if bias:
                ref.bias.copy_(layer.bias.double())
        x = torch.rand(*batch, fin, device=dev) * 2 - 1
        x1 = x.clone().requires_grad_()
        x2 = x.double().requires_grad_()
        y1, y2 = layer(x1), ref(x2)
        assert y1.shape == y2.shape and y1.is_cuda
        g = torch.rand_like(y1) * 2 - 1
        y1.backward(g)
        y2.backward(g.double())
        torch.cuda.synchronize()
        scale_y = fin * 1.0
        assert (y1.double() - y2).abs().max().item() <= TIGHT * scale_y
        assert (x1.grad.double() - x2.grad).abs().max().item() <= TIGHT * fout
        rows = int(np.prod(batch))
        assert (layer.weight.grad.double() - ref.weight.grad).abs().max().item() <= TIGHT * rows
        if bias:
            assert (layer.bias.grad.double() - ref.bias.grad).abs().max().item() <= TIGHT * rows
    # CPU tensors take the staged path and give the same numbers
    layer_cpu = cake_linear(40, 24)
    xc = torch.rand(9, 40) * 2 - 1
    yc = layer_cpu(xc)
    assert torch.allclose(yc, torch.nn.functional.linear(xc, layer_cpu.weight, layer_cpu.bias), atol=1e-5)


@pytest.mark.parametrize("shape", [(64, 96, 48), (33, 130, 257), (300, 2111, 96), (7, 5, 3)],
                         ids=lambda s: "x".join(map(str, s)))
def test_linear_forward_with_pretransposed_weights(shape):
    """cake_hip_linear_forward_wt on a transposed copy of the weights gives what
    cake_hip_linear_forward gives on the weights themselves (same product, same bias rounding)."""
    M, K, N = shape
    x, w, b = oracle.uniform((M, K), 11), oracle.uniform((N, K), 12), oracle.uniform((N,), 13)
    wt = np.empty((K, N), np.float32)
    cake.transpose_mat(w, wt, N, K)
    assert np.array_equal(wt, w.T)
    y1 = np.full((M, N), np.nan, np.float32)
    y2 = np.full((M, N), np.nan, np.float32)
    cake.linear_forward(x, w, b, y1, M, N, K)
    cake.linear_forward_wt(x, wt, b, y2, M, N, K)
    y64 = x.astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64)[None, :]
    S = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T + np.abs(b)[None, :]
    assert _rel(y2, y64, S) <= TIGHT
    # (not bit-identical: one reads w along k, the other the copy along n, in different macro-tile plans)
    y3 = np.full((M, N), np.nan, np.float32)
    cake.linear_forward_wt(x, wt, None, y3, M, N, K, timed=False)
    assert _rel(y3, x.astype(np.float64) @ w.astype(np.float64).T, S) <= TIGHT


def test_torch_module_follows_weight_updates_without_a_copy():
    """The module hands its weights to the library as they lie at every call (no transposed copy
    is kept, so nothing can go stale): outputs match torch's layer before and after in-place
    updates, for batches on every route (a single sample, two, a small batch, a large one), and
    training steps through autograd and an optimizer work."""
    import torch
    from cake_on_cpu_amd.torch_linear import cake_linear
    torch.manual_seed(1)
    dev = torch.device("cuda:0")
    layer = cake_linear(2048, 1024).to(dev)
    x = torch.rand(300, 2048, device=dev) * 2 - 1
    want = lambda t: torch.nn.functional.linear(t.double(), layer.weight.double(), layer.bias.double())
    with torch.no_grad():
        for rows in (300, 40, 8, 2, 1):
            y = layer(x[:rows])
            assert (y.double() - want(x[:rows])).abs().max().item() <= TIGHT * 2048
        layer.weight.mul_(0.5)                          # what an optimizer step does: in place
        for rows in (300, 40, 8, 2, 1):
            y = layer(x[:rows])
            assert (y.double() - want(x[:rows])).abs().max().item() <= TIGHT * 2048
    assert not [k for k in vars(layer) if "wt" in k]     # only parameters, no cached copies
    opt = torch.optim.SGD(layer.parameters(), lr=0.01)
    for _ in range(2):
        opt.zero_grad()
        out = layer(x)
        assert (out.double() - want(x)).abs().max().item() <= TIGHT * 2048
        out.sum().backward()
        opt.step()
    torch.cuda.synchronize()


def test_reference_run_tests_sweep():
    """run_tests of src/util.cpp:3-136 through libcake.so: 216 shapes x five entry points."""
    exe = _lib.LIB_DIR / "dropin_test"
    assert exe.exists(), "build it with make -C cake_on_cpu_amd/csrc"
    res = subprocess.run([str(exe), "run_tests"], capture_output=True, text=True, timeout=900)
    tail = res.stdout[-400:]
    print(tail, res.stderr[-2000:])
    assert res.returncode == 0 and "ALL TESTS PASSED!" in res.stdout and "TESTS FAILED" not in res.stdout
    assert res.stdout.count("CORRECT!") >= 216 * 5


@pytest.mark.parametrize("rows,cols", [(4100, 4099), (2048, 1024), (1449, 1448), (8193, 1025)],
                         ids=lambda v: str(v))
def test_large_host_operands_survive_the_staging_pipeline(rows, cols):
    """Host arrays of 8 MB and more travel through pinned buffers in 32 MB chunks (below that a
    plain copy): a transpose moves every byte both ways, so the result must be bit-exact, also when
    the last chunk is ragged and when the size sits just under and over the threshold."""
    src = oracle.uniform((rows, cols), 21)
    dst = np.full((cols, rows), np.nan, np.float32)
    print(f"host staging {rows}x{cols}: {src.nbytes / 2**20:.1f} MiB", flush=True)
    cake.transpose_mat(src, dst, rows, cols)
    assert np.array_equal(dst, src.T)
    # twice in a row: the buffers and events are reused
    dst2 = np.full((cols, rows), np.nan, np.float32)
    cake.transpose_mat(src, dst2, rows, cols)
    assert np.array_equal(dst2, src.T)


def test_zz_shutdown_releases_and_the_next_call_starts_over():
    """cake_hip_shutdown frees the workspaces, pinned buffers, streams and events; the next
    call initialises again and computes the same product (host operands large enough to use the
    pinned staging on both sides of the shutdown)."""
    import ctypes as C
    lib = cake.load()
    M, K, N = 1536, 1500, 1400
    A, B = oracle.uniform((M, K), 31), oracle.uniform((K, N), 32)
    before = np.zeros((M, N), np.float32)
    cake.cake_sgemm(A, B, before, M, N, K, 1)
    assert lib.cake_hip_shutdown() == 0
    assert lib.cake_hip_shutdown() == 0          # idempotent
    after = np.zeros((M, N), np.float32)
    cake.cake_sgemm(A, B, after, M, N, K, 1)
    assert np.array_equal(before, after)
    C64, S = oracle.gemm_f64(A, B)
    assert oracle.max_rel_err(after, C64, S) <= 5e-6
