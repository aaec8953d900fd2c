"""The five BASELINE configurations at full size, operands resident on the GPU.

Where the oracle finishes in seconds the whole result is compared; at 8192^3
and for the 32-image convolution the check is on sampled rows/columns against
fp64 plus size-independent properties (linearity, schedule independence)."""
import numpy as np
import pytest

import cake_on_cpu_amd as cake
import oracle

pytestmark = pytest.mark.gpu
TOL = 1e-4
TIGHT = 5e-6

torch = pytest.importorskip("torch")


def _dev(shape, seed):
    t = torch.empty(shape, dtype=torch.float32, device="cuda:0")
    cake.fill_uniform(t, seed)
    return t


def test_c1_sgemm_1024_matches_oracle_every_schedule():
    M = K = N = 1024
    A, B = _dev((M, K), 1), _dev((K, N), 2)
    Ah, Bh = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    assert np.array_equal(A.cpu().numpy(), Ah)
    C64, S = oracle.gemm_f64(Ah, Bh)
    cx = oracle.make_cntx()
    for sch in (cake.NA, cake.KMN, cake.MKN, cake.NKM):
        Cm = torch.zeros((M, N), dtype=torch.float32, device="cuda:0")
        cake.cake_sgemm(A, B, Cm, M, N, K, 8, None, None, False, False, 1.0, 0.0, sch)
        got = Cm.cpu().numpy()
        ref = oracle.cake_sgemm(Ah, Bh, 8, cx, sch=sch)
        assert np.max(np.abs(got - ref) / S) <= TOL
        assert oracle.max_rel_err(got, C64, S) <= TIGHT


def test_c2_sgemm_8192_sampled_rows_and_linearity():
    n = 8192
    A, B = _dev((n, n), 1), _dev((n, n), 2)
    Cm = torch.zeros((n, n), dtype=torch.float32, device="cuda:0")
    cake.cake_sgemm(A, B, Cm, n, n, n, 8)
    torch.cuda.synchronize()
    rng = np.random.default_rng(7)
    rows = np.unique(np.concatenate([[0, 1, 255, 256, n - 1], rng.integers(0, n, 40)]))
    Ah = A[torch.as_tensor(rows, device="cuda:0")].cpu().numpy()
    Bh = B.cpu().numpy()
    C64, S = oracle.gemm_f64(np.ascontiguousarray(Ah), Bh)
    got = Cm[torch.as_tensor(rows, device="cuda:0")].cpu().numpy()
    assert oracle.max_rel_err(np.ascontiguousarray(got), C64, S) <= TIGHT
    # linearity in B: (A.B1 + A.B2) == A.(B1+B2) to rounding, on the whole matrix
    B2 = _dev((n, n), 9)
    C2 = torch.zeros_like(Cm)
    cake.cake_sgemm(A, B2, C2, n, n, n, 8)
    Csum = torch.zeros_like(Cm)
    cake.cake_sgemm(A, B + B2, Csum, n, n, n, 8)
    scale = float(n) * 0.25 * 2      # E|a||b| * K for uniform[-1,1) inputs, B+B2 doubles it at most
    assert float((Csum - (Cm + C2)).abs().max()) / scale <= 1e-5
    # every schedule computes the same sums
    Ck = torch.zeros_like(Cm)
    cake.cake_sgemm(A, B, Ck, n, n, n, 8, None, None, False, False, 1.0, 0.0, cake.MKN)
    assert torch.equal(Ck, Cm)


def test_c3_tall_skinny_full_check():
    M, K, N = 65536, 1024, 128
    A, B = _dev((M, K), 1), _dev((K, N), 2)
    Cm = torch.zeros((M, N), dtype=torch.float32, device="cuda:0")
    cake.cake_sgemm(A, B, Cm, M, N, K, 8)
    Ah, Bh = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
    C64, S = oracle.gemm_f64(Ah, Bh)
    got = Cm.cpu().numpy()
    assert oracle.max_rel_err(got, C64, S) <= TIGHT
    ref = oracle.cake_sgemm(Ah, Bh, 8, oracle.make_cntx())
    assert np.max(np.abs(got - ref) / S) <= TOL


@pytest.mark.parametrize("col_major", [False, True])
def test_c4_gemv_16384(col_major):
    n = 16384
    A, x = _dev((n * n,), 1), _dev((n,), 3)
    y = torch.zeros((n,), dtype=torch.float32, device="cuda:0")
    cake.cake_sgemv(A, x, y, n, n, 8, row_major=not col_major, accumulate=False)
    Ah, xh = oracle.uniform(n * n, 1), oracle.uniform(n, 3)
    y64, S = oracle.gemv_f64(Ah, xh, n, n, col_major=col_major)
    got = y.cpu().numpy()
    assert np.max(np.abs(got - y64) / S) <= TIGHT
    if col_major:
        ref = oracle.cake_sgemv(Ah, xh, 8, oracle.make_cntx(mr=8), M=n, K=n)
        assert np.max(np.abs(got - ref) / S) <= TOL


def test_c5_conv_256x256x56x56_batch32_sampled():
    Bn, Cin, Cout, H = 32, 256, 256, 56
    inp, wt = _dev((Bn, Cin, H, H), 5), _dev((Cout, Cin, 3, 3), 4)
    out = torch.empty((Cout, Bn * H * H), dtype=torch.float32, device="cuda:0")
    cake.conv2d(inp, wt, out, Bn, Cin, H, H, Cout, 3, 3, 1, 1)
    torch.cuda.synchronize()
    # the reference's own two steps (column matrix first) give the same numbers up to the order of
    # the sums (the direct path walks K channel block by channel block): 5e-6 of sum |a||b| <= 2304 / 4
    two_step = torch.empty_like(out)
    cake.conv2d(inp, wt, two_step, Bn, Cin, H, H, Cout, 3, 3, 1, 1, explicit_im2col=True)
    assert float((two_step - out).abs().max()) <= 5e-6 * 576
    # two whole images (first and last) against the naive fp64 convolution
    wh = wt.cpu().numpy()
    for b in (0, Bn - 1):
        img = inp[b:b + 1].cpu().numpy()
        ref64, S = oracle.conv_naive_f64(img, wh, 1, 1)
        got = out[:, b * H * H:(b + 1) * H * H].cpu().numpy().reshape(Cout, H, H)
        assert np.max(np.abs(got - ref64[0]) / S[0]) <= TIGHT
    # NCHW output is the same numbers, permuted
    nchw = torch.empty((Bn, Cout, H, H), dtype=torch.float32, device="cuda:0")
    cake.conv2d(inp, wt, nchw, Bn, Cin, H, H, Cout, 3, 3, 1, 1, out_nchw=True)
    assert torch.equal(nchw, out.view(Cout, Bn, H, H).permute(1, 0, 2, 3).contiguous())
