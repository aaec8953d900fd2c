"""Operands beyond 2^32 bytes (the reference indexes with int, so 2^31 - 1 elements per matrix is
its limit and the library's): every kernel family is run once on a matrix of 34000 x 34000 floats
(4.6 GB) in each of its roles, and the convolution on batches whose staged input passes 2 GiB and
is therefore cut into chunks of images.

The oracle cannot finish such sizes, so the check is what the mathematics fixes: sampled rows and
columns of each result, including the last ones (whose sources lie past byte 2^32), against fp64
dot products of the same device data; max |C - C64| / sum_k |a||b| <= 5e-6.  Copies are bit-exact."""
import pytest

torch = pytest.importorskip("torch")

import cake_on_cpu_amd as cake

pytestmark = pytest.mark.gpu

R = 34000            # R * R = 1.156e9 elements, 4.62e9 bytes
TIGHT = 5e-6


def _dev():
    return torch.device("cuda:0")


def _sample(n, count=48):
    """First, last and evenly spread indices of range(n)."""
    idx = set(range(min(8, n))) | set(range(max(0, n - 8), n)) | {(i * 2654435761) % n for i in range(count)}
    return torch.tensor(sorted(idx), device=_dev(), dtype=torch.long)


def _filled(shape, seed):
    t = torch.empty(shape, dtype=torch.float32, device=_dev())
    cake.fill_uniform(t, seed)
    return t


def _check(got, a64, b64, what):
    """got ~ a64 @ b64 (fp64 operands on the device)."""
    ref = a64 @ b64
    S = a64.abs() @ b64.abs()
    err = float(((got.double() - ref).abs() / S.clamp_min(1e-300)).max())
    assert err <= TIGHT, f"{what}: {err}"


@pytest.fixture(scope="module")
def big():
    t = _filled((R, R), 901)
    yield t
    del t
    torch.cuda.empty_cache()


def test_fill_reaches_the_end(big):
    # the generator is a function of (seed, index): the tail of the large fill equals a small
    # fill's values only if indices are not truncated, which the statistics of the tail show
    tail = big[-1]
    assert torch.isfinite(tail).all() and float(tail.std()) > 0.1
    assert not torch.equal(big[-1], big[0])


def test_matrix_vector_products(big):
    x = _filled((R,), 902)
    rows = _sample(R)
    for accumulate in (False, True):
        y = torch.full((R,), 0.5, dtype=torch.float32, device=_dev())
        print(f"row-major gemv {R}x{R} accumulate={accumulate}", flush=True)
        cake.cake_sgemv(big, x, y, R, R, 1, row_major=True, accumulate=accumulate)
        got = y[rows] - (0.5 if accumulate else 0.0)
        _check(got[:, None], big[rows].double(), x.double()[:, None], "row-major gemv")
    y = torch.zeros((R,), dtype=torch.float32, device=_dev())
    print(f"column-major gemv {R}x{R}", flush=True)
    cake.cake_sgemv(big, x, y, R, R, 1)       # big read as A[k*M + m]
    _check(y[rows][:, None], big[:, rows].double().t().contiguous(), x.double()[:, None], "column-major gemv")


@pytest.mark.parametrize("N", [9, 16, 48, 200], ids=lambda n: f"N{n}")
def test_large_a(big, N):
    """C = big . B: few columns (streaming kernel for N <= 32) and macro-tiles."""
    B = _filled((R, N), 903)
    Cm = torch.full((R, N), float("nan"), dtype=torch.float32, device=_dev())
    print(f"sgemm {R}x{N}x{R} plan={cake.plan(R, N, R).as_dict()}", flush=True)
    cake.cake_sgemm(big, B, Cm, R, N, R, 1)
    assert torch.isfinite(Cm).all()
    rows = _sample(R)
    _check(Cm[rows], big[rows].double(), B.double(), f"large A, N={N}")


@pytest.mark.parametrize("M", [16, 300], ids=lambda m: f"M{m}")
def test_large_b(big, M):
    """C = A . big: few rows (streaming kernel) and macro-tiles."""
    A = _filled((M, R), 904)
    Cm = torch.full((M, R), float("nan"), dtype=torch.float32, device=_dev())
    print(f"sgemm {M}x{R}x{R} plan={cake.plan(M, R, R).as_dict()}", flush=True)
    cake.cake_sgemm(A, big, Cm, M, R, R, 1)
    assert torch.isfinite(Cm).all()
    cols = _sample(R)
    _check(Cm[:, cols], A.double(), big[:, cols].double(), f"large B, M={M}")


@pytest.mark.parametrize("K", [24, 48, 100])
def test_large_c(K):
    """C of 4.6 GB from a short K: the epilogue's addressing in each of the three kernels that walk
    over tiles (K up to 32, up to 64, beyond)."""
    A, B = _filled((R, K), 905), _filled((K, R), 906)
    Cm = torch.empty((R, R), dtype=torch.float32, device=_dev())
    Cm.fill_(float("nan"))
    print(f"sgemm {R}x{R}x{K} plan={cake.plan(R, R, K).as_dict()}", flush=True)
    cake.cake_sgemm(A, B, Cm, R, R, K, 1)
    rows = _sample(R)
    assert torch.isfinite(Cm[rows]).all() and torch.isfinite(Cm[:, rows]).all()
    _check(Cm[rows], A[rows].double(), B.double(), "large C")
    # and added to what C holds (M-first schedule, beta != 0)
    before = Cm[rows].clone()
    cake.cake_sgemm(A, B, Cm, R, R, K, 1, beta=1.0, sch=cake.MKN)
    _check(Cm[rows] - before, A[rows].double(), B.double(), "large C, accumulated")
    del Cm
    torch.cuda.empty_cache()


def test_transpose(big):
    out = torch.empty((R, R), dtype=torch.float32, device=_dev())
    print(f"transpose {R}x{R}", flush=True)
    cake.transpose_mat(big, out, R, R)
    rows = _sample(R)
    assert torch.equal(out[rows], big[:, rows].t())
    del out
    torch.cuda.empty_cache()


def test_store_bound_product_with_rows_off_cache_lines():
    """K = 12 into a C of 324 MB whose rows are 36004 bytes apart: the planner leaves the short-K
    kernel for the 96 x 128 macro-tile; the whole result against fp64 on the device."""
    M, K, N = 9000, 12, 9001
    plan = cake.plan(M, N, K)
    assert (plan.tile_m, plan.tile_n, plan.tile_k, plan.split_k) == (96, 128, 32, 1)
    assert (cake.plan(M, 9024, K).tile_m, cake.plan(M, 9024, K).tile_n) == (64, 64)   # rows of whole lines: the short-K kernel
    A, B = _filled((M, K), 961), _filled((K, N), 962)
    C = torch.full((M, N), float("nan"), dtype=torch.float32, device=_dev())
    lib = cake.load()
    stream = torch.cuda.current_stream().cuda_stream
    print(f"sgemm {M}x{K}x{N}", flush=True)
    assert lib.cake_hip_sgemm(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, cake.NA, 0, None, stream, None) == 0
    _check(C, A.double(), B.double(), "store-bound product")
    first = C.clone()
    assert lib.cake_hip_sgemm(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, cake.NA, 1, None, stream, None) == 0
    assert torch.equal(C, first + first)       # accumulating once more doubles every element exactly
    del A, B, C, first
    torch.cuda.empty_cache()


def test_im2col_columns_past_4_gb():
    """A column matrix of 576 x 2 000 000 floats (4.6 GB): sampled rows, the last ones among them,
    equal the shifted planes they are copies of, bit for bit."""
    Bn, Cin, H, W, Hf, Wf, pad = 32, 64, 250, 250, 3, 3, 1
    K, N = Cin * Hf * Wf, Bn * H * W
    inp = _filled((Bn, Cin, H, W), 977)
    cols = torch.full((K, N), float("nan"), dtype=torch.float32, device=_dev())
    print(f"im2col {K}x{N}: {K * N * 4 / 1e9:.2f} GB", flush=True)
    cake.im2col(inp, cols, Bn, Cin, H, W, Hf, Wf, 1, pad)
    for k in (0, 1, 4, 8, 9, K // 2, K - 10, K - 9, K - 2, K - 1):
        c, h, w = k // (Hf * Wf), (k % (Hf * Wf)) // Wf, k % Wf
        padded = torch.nn.functional.pad(inp[:, c], (pad, pad, pad, pad))
        assert torch.equal(cols[k], padded[:, h:h + H, w:w + W].reshape(-1)), k
    del cols, inp
    torch.cuda.empty_cache()


def test_pack_and_unpack(big):
    """pack_A and pack_C of the large matrix: sampled elements, the last rows among them, sit at the
    offsets of the packed index map (evaluated on the host), and unpack_C brings every bit back."""
    p = 8
    ccx = cake.CpuCntx(1.0, 6, 16, 48 << 10, 2 << 20, 105 << 20, 8)
    x = cake.init_block_dims(R, R, R, p, ccx, cake.KMN)
    picks = [(0, 0), (5, 17), (R // 2 + 1, R // 3), (R - 7, 11), (R - 1, R - 1), (R - 2, 3), (12345, R - 1)]
    for which, size, pack in ((0, cake.cake_sgemm_packed_A_size(R, R, p, x, ccx, cake.KMN), cake.pack_A),
                              (2, cake.cake_sgemm_packed_C_size(R, R, p, x, ccx, cake.KMN), cake.pack_C)):
        print(f"pack {'AC'[which // 2]} {R}x{R}: {size / 1e9:.2f} GB packed", flush=True)
        packed = torch.full((size // 4,), float("nan"), dtype=torch.float32, device=_dev())
        pack(big, packed, R, R, p, x, ccx, cake.KMN)
        for r, c in picks:
            off = cake.packed_offset(which, r, c, R, R, R, p, x, ccx, cake.KMN)
            assert 0 <= off < size // 4
            assert float(packed[off]) == float(big[r, c]), (which, r, c, off)
        if which == 2:
            back = torch.full((R, R), float("nan"), dtype=torch.float32, device=_dev())
            cake.unpack_C(back, packed, R, R, p, x, ccx, cake.KMN)
            assert torch.equal(back, big)
            del back
        del packed
        torch.cuda.empty_cache()


@pytest.mark.parametrize("batch", [1, 2, 16, 40], ids=lambda b: f"batch{b}")
def test_linear_forward(big, batch):
    """y = x . big^T + b: matrix-vector sweep, its two-vector form, the streaming kernel, and the
    macro-tiles that read the weights along k."""
    x, b = _filled((batch, R), 907), _filled((R,), 908)
    y = torch.full((batch, R), float("nan"), dtype=torch.float32, device=_dev())
    print(f"linear forward batch={batch} {R}->{R}", flush=True)
    cake.linear_forward(x, big, b, y, batch, R, R)
    assert torch.isfinite(y).all()
    cols = _sample(R)
    ref = x.double() @ big[cols].double().t() + b[cols].double()
    S = x.double().abs() @ big[cols].double().abs().t() + b[cols].double().abs()
    err = float(((y[:, cols].double() - ref).abs() / S).max())
    assert err <= TIGHT, err


def test_linear_backward_small_batch(big):
    batch = 16
    g, x = _filled((batch, R), 909), _filled((batch, R), 910)
    gx = torch.full((batch, R), float("nan"), dtype=torch.float32, device=_dev())
    gw = torch.empty((R, R), dtype=torch.float32, device=_dev())
    gb = torch.empty((R,), dtype=torch.float32, device=_dev())
    print(f"linear backward batch={batch} {R}->{R}", flush=True)
    cake.linear_backward(g, x, big, gx, gw, gb, batch, R, R)
    cols = _sample(R)
    _check(gx[:, cols], g.double(), big[:, cols].double(), "grad_x")
    _check(gw[cols], g[:, cols].double().t().contiguous(), x.double(), "grad_w")
    _check(gb[cols][None, :], torch.ones((1, batch), dtype=torch.float64, device=_dev()), g[:, cols].double(), "grad_bias")
    del gw
    torch.cuda.empty_cache()


def test_host_operands(big):
    """The same matrix in host memory: staged through the pinned chunks (matrix-vector product,
    bit-identical to the device-operand call) and through the row-block pipeline of a product
    whose A and C are host arrays."""
    import numpy as np
    host = big.cpu().numpy()
    x = _filled((R,), 913)
    y_dev = torch.zeros((R,), dtype=torch.float32, device=_dev())
    cake.cake_sgemv(big, x, y_dev, R, R, 1, row_major=True, accumulate=False)
    y = np.full((R,), np.nan, np.float32)
    print(f"host row-major gemv {R}x{R}", flush=True)
    cake.cake_sgemv(host, x.cpu().numpy(), y, R, R, 1, row_major=True, accumulate=False)
    assert np.array_equal(y, y_dev.cpu().numpy())
    N = 48
    B = _filled((R, N), 914)
    Cm = np.full((R, N), np.nan, np.float32)
    print(f"host sgemm {R}x{N}x{R}", flush=True)
    cake.cake_sgemm(host, B.cpu().numpy(), Cm, R, N, R, 1)
    assert np.isfinite(Cm).all()
    rows = _sample(R)
    _check(torch.from_numpy(Cm).to(_dev())[rows], big[rows].double(), B.double(), "host A and C")


# batch, Cin, H, W, Cout, filter, stride, pad: the staged input of the whole batch is 3.3, 2.7 and 2.2 GB
BIG_CONVS = [(49, 64, 512, 512, 8, 3, 1, 1), (40, 64, 512, 512, 8, 3, 1, 0), (33, 64, 514, 514, 12, 3, 2, 1)]


@pytest.mark.parametrize("geom", BIG_CONVS, ids=str)
@pytest.mark.parametrize("nchw", [False, True], ids=["cn", "nchw"])
def test_conv_in_chunks_of_images(geom, nchw):
    batch, Cin, H, W, Cout, F, stride, pad = geom
    Hout, Wout = (H + 2 * pad - F) // stride + 1, (W + 2 * pad - F) // stride + 1
    HW = Hout * Wout
    inp, wt = _filled((batch, Cin, H, W), 911), _filled((Cout, Cin * F * F), 912)
    out = torch.full((batch * Cout * HW,), float("nan"), dtype=torch.float32, device=_dev())
    print(f"conv {geom} nchw={nchw}", flush=True)
    cake.conv2d(inp, wt, out, batch, Cin, H, W, Cout, F, F, stride, pad, out_nchw=nchw)
    assert torch.isfinite(out).all()
    w64 = wt.double()
    for b in sorted({0, batch // 2 - 1, batch // 2, batch // 2 + 1, batch - 1}):
        cols = torch.nn.functional.unfold(inp[b:b + 1].double(), F, padding=pad, stride=stride)[0]   # [Cin*F*F][HW]
        ref = w64 @ cols
        S = w64.abs() @ cols.abs()
        got = out.view(batch, Cout, HW)[b] if nchw else out.view(Cout, batch, HW)[:, b]
        err = float(((got.double() - ref).abs() / S.clamp_min(1e-300)).max())
        assert err <= TIGHT, f"image {b}: {err}"
    del inp, out
    torch.cuda.empty_cache()
