"""The library's launches can be captured into a HIP graph once its workspaces are warm: device
operands, no timing, nothing but kernels on the caller's stream (zero fills are kernels, not
memset nodes).  Every replay is checked against the eager result for the inputs of that moment."""
import pytest

torch = pytest.importorskip("torch")

import ctypes

import cake_on_cpu_amd as cake

pytestmark = pytest.mark.gpu


def test_captured_sequence_replays_like_eager_calls():
    dev = torch.device("cuda:0")
    lib = cake.load()
    M, N, K = 520, 300, 4096           # split-K product: main kernel + slice reduction
    gm = 2048                          # column-major matrix-vector product with K slices
    bm, bn, bk = 8, 1024, 768          # small-batch linear layer: streaming kernel + reduction
    A = torch.empty((M, K), dtype=torch.float32, device=dev)
    B = torch.empty((K, N), dtype=torch.float32, device=dev)
    G = torch.empty((gm * gm,), dtype=torch.float32, device=dev)
    x = torch.empty((gm,), dtype=torch.float32, device=dev)
    lx = torch.empty((bm, bk), dtype=torch.float32, device=dev)
    lw = torch.empty((bn, bk), dtype=torch.float32, device=dev)
    lb = torch.empty((bn,), dtype=torch.float32, device=dev)
    for i, t in enumerate((A, B, G, x, lx, lw, lb)):
        cake.fill_uniform(t, 40 + i)

    def outputs():
        return (torch.zeros((M, N), dtype=torch.float32, device=dev), torch.zeros((gm,), dtype=torch.float32, device=dev),
                torch.zeros((bm, bn), dtype=torch.float32, device=dev))

    def run(out, stream):
        c, y, ly = out
        assert lib.cake_hip_sgemm(A.data_ptr(), B.data_ptr(), c.data_ptr(), M, N, K, cake.NA, 0, None, stream, None) == 0
        assert lib.cake_hip_sgemv(G.data_ptr(), x.data_ptr(), y.data_ptr(), gm, gm, 1, 0, stream, None) == 0
        assert lib.cake_hip_linear_forward(lx.data_ptr(), lw.data_ptr(), lb.data_ptr(), ly.data_ptr(), bm, bn, bk,
                                           stream, None) == 0

    side = torch.cuda.Stream()
    captured = outputs()
    with torch.cuda.stream(side):
        run(captured, side.cuda_stream)          # warm: every workspace is allocated before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(captured, torch.cuda.current_stream().cuda_stream)

    def grow_every_workspace():
        """Eager calls whose partial sums need several times the memory the captured ones did: the
        library's workspaces grow, and the graph must keep working on the addresses it recorded
        (an outgrown workspace is kept, not freed)."""
        bigA = torch.empty((1500, 8192), dtype=torch.float32, device=dev)
        bigB = torch.empty((8192, 1300), dtype=torch.float32, device=dev)
        bigC = torch.empty((1500, 1300), dtype=torch.float32, device=dev)
        ov = (ctypes.c_int * 4)(128, 128, 32, 8)
        assert lib.cake_hip_sgemm(bigA.data_ptr(), bigB.data_ptr(), bigC.data_ptr(), 1500, 1300, 8192, cake.NA, 0, ov,
                                  None, None) == 0
        bg = 6144
        bigG = torch.empty((bg * bg,), dtype=torch.float32, device=dev)
        by = torch.empty((bg,), dtype=torch.float32, device=dev)
        assert lib.cake_hip_sgemv(bigG.data_ptr(), bigG.data_ptr(), by.data_ptr(), bg, bg, 1, 0, None, None) == 0
        bx = torch.empty((24, 4096), dtype=torch.float32, device=dev)
        bw = torch.empty((8192, 4096), dtype=torch.float32, device=dev)
        bo = torch.empty((24, 8192), dtype=torch.float32, device=dev)
        assert lib.cake_hip_linear_forward(bx.data_ptr(), bw.data_ptr(), None, bo.data_ptr(), 24, 8192, 4096, None, None) == 0
        torch.cuda.synchronize()

    for replay in range(5):
        if replay == 2:
            grow_every_workspace()
        for i, t in enumerate((A, x, lx)):       # new inputs, written by eager work between the replays
            cake.fill_uniform(t, 100 + 10 * replay + i)
        for t in captured:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = outputs()
        run(eager, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {replay}"


def test_captured_convolutions_replay_like_eager_calls(monkeypatch):
    """The convolution routes under capture: the input read where it lies (under a 3 x 3 filter one
    kernel with the last round in sub-tiles; under a 5 x 3 one re-laid filters and tail slices
    summed by a second kernel), the gather from a staged copy (stride 2: staging kernel, tap
    table), a 1 x 1 layer at stride 2 (dense copy first) and the reference's two steps (column
    matrix in a workspace).  A larger eager
    convolution between the replays grows every one of those workspaces."""
    monkeypatch.setenv("CAKE_HIP_CONV_ROUTE", "patch")   # layers this small would take the staged copy by themselves
    dev = torch.device("cuda:0")
    lib = cake.load()
    geoms = [(34, 32, 32, 32, 72, 3, 3, 1, 1, lib.cake_hip_conv2d),        # 272 tiles: the 16 of the last round as sub-tiles
             (34, 64, 32, 32, 40, 5, 3, 1, 2, lib.cake_hip_conv2d),        # the same under 15 taps: re-laid filters, K slices
             (3, 16, 12, 12, 32, 3, 3, 2, 1, lib.cake_hip_conv2d),         # staged copy
             (4, 32, 16, 16, 48, 1, 1, 2, 0, lib.cake_hip_conv2d),         # 1 x 1 at stride 2: dense copy of the pixels it reads
             (2, 8, 16, 16, 24, 3, 3, 1, 1, lib.cake_hip_conv2d_im2col)]   # column matrix first
    ins, wts = [], []
    for i, (b, cin, h, w, cout, hf, wf, s, p, _) in enumerate(geoms):
        ins.append(torch.empty((b, cin, h, w), dtype=torch.float32, device=dev))
        wts.append(torch.empty((cout, cin, hf, wf), dtype=torch.float32, device=dev))
        cake.fill_uniform(ins[-1], 300 + i)
        cake.fill_uniform(wts[-1], 310 + i)

    def outputs():
        outs = []
        for b, cin, h, w, cout, hf, wf, s, p, _ in geoms:
            ho, wo = (h + 2 * p - hf) // s + 1, (w + 2 * p - wf) // s + 1
            outs.append(torch.zeros((b, cout, ho, wo), dtype=torch.float32, device=dev))
        return outs

    def run(outs, stream):
        for (b, cin, h, w, cout, hf, wf, s, p, fn), x, f, o in zip(geoms, ins, wts, outs):
            assert fn(x.data_ptr(), f.data_ptr(), o.data_ptr(), b, cin, h, w, cout, hf, wf, s, p, 1, None, stream, None) == 0

    side = torch.cuda.Stream()
    captured = outputs()
    with torch.cuda.stream(side):
        run(captured, side.cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(captured, torch.cuda.current_stream().cuda_stream)

    def grow_every_workspace():
        # (the first one under 15 taps: more re-laid filters and more K slices of a last round than captured)
        for b, cin, h, w, cout, hf, wf, s, p, fn in ((70, 96, 32, 32, 300, 5, 3, 1, 2, lib.cake_hip_conv2d),
                                                     (8, 32, 40, 40, 64, 3, 3, 2, 1, lib.cake_hip_conv2d),
                                                     (8, 16, 32, 32, 48, 3, 3, 1, 1, lib.cake_hip_conv2d_im2col)):
            x = torch.empty((b, cin, h, w), dtype=torch.float32, device=dev)
            f = torch.empty((cout, cin, hf, wf), dtype=torch.float32, device=dev)
            ho, wo = (h + 2 * p - hf) // s + 1, (w + 2 * p - wf) // s + 1
            o = torch.empty((b, cout, ho, wo), dtype=torch.float32, device=dev)
            assert fn(x.data_ptr(), f.data_ptr(), o.data_ptr(), b, cin, h, w, cout, hf, wf, s, p, 1, None, None, None) == 0
        torch.cuda.synchronize()

    for replay in range(4):
        if replay == 2:
            grow_every_workspace()
        for i, t in enumerate(ins):
            cake.fill_uniform(t, 400 + 10 * replay + i)
        for t in captured:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = outputs()
        run(eager, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {replay}"


def test_captured_packing_and_im2col_replay_like_eager_calls():
    """pack_A, pack_B, pack_C, unpack_C (index tables in a workspace, then the copy kernels) and im2col."""
    dev = torch.device("cuda:0")
    lib = cake.load()
    M, K, N, p = 333, 270, 401, 3
    ccx = cake.CpuCntx(1.0, 6, 16, 48 << 10, 256 << 10, 2 << 20, 8)
    x = cake.init_block_dims(M, N, K, p, ccx, cake.KMN)
    A = torch.empty((M, K), dtype=torch.float32, device=dev)
    B = torch.empty((K, N), dtype=torch.float32, device=dev)
    Cm = torch.empty((M, N), dtype=torch.float32, device=dev)
    img = torch.empty((5, 6, 13, 14), dtype=torch.float32, device=dev)
    sizes = (cake.cake_sgemm_packed_A_size(M, K, p, x, ccx, cake.KMN) // 4, cake.cake_sgemm_packed_B_size(K, N, p, x, ccx) // 4,
             cake.cake_sgemm_packed_C_size(M, N, p, x, ccx, cake.KMN) // 4)
    bx, bc = ctypes.byref(x), ctypes.byref(ccx)

    def outputs():
        return tuple(torch.zeros(shape, dtype=torch.float32, device=dev)
                     for shape in ((sizes[0],), (sizes[1],), (sizes[2],), (M, N), (6 * 9, 5 * 13 * 14)))

    def run(out, stream):
        ap, bp, cp, back, cols = out
        assert lib.cake_hip_pack_a(A.data_ptr(), ap.data_ptr(), M, K, p, bx, bc, cake.KMN, stream, None) == 0
        assert lib.cake_hip_pack_b(B.data_ptr(), bp.data_ptr(), K, N, p, bx, bc, cake.KMN, stream, None) == 0
        assert lib.cake_hip_pack_c(Cm.data_ptr(), cp.data_ptr(), M, N, p, bx, bc, cake.KMN, stream, None) == 0
        assert lib.cake_hip_unpack_c(back.data_ptr(), cp.data_ptr(), M, N, p, bx, bc, cake.KMN, stream, None) == 0
        assert lib.cake_hip_im2col(img.data_ptr(), cols.data_ptr(), 5, 6, 13, 14, 3, 3, 1, 1, stream, None) == 0

    side = torch.cuda.Stream()
    captured = outputs()
    with torch.cuda.stream(side):
        run(captured, side.cuda_stream)          # warm: the index tables' workspace is allocated before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(captured, torch.cuda.current_stream().cuda_stream)

    for replay in range(4):
        if replay == 2:   # larger index tables between the replays: the workspace grows, the graph keeps its addresses
            big = torch.empty((3000, 2000), dtype=torch.float32, device=dev)
            bx2 = cake.init_block_dims(3000, 2000, 2000, p, ccx, cake.KMN)
            bp2 = torch.empty((cake.cake_sgemm_packed_A_size(3000, 2000, p, bx2, ccx, cake.KMN) // 4,), dtype=torch.float32, device=dev)
            cake.pack_A(big, bp2, 3000, 2000, p, bx2, ccx, cake.KMN)
            torch.cuda.synchronize()
        for i, t in enumerate((A, B, Cm, img)):
            cake.fill_uniform(t, 500 + 10 * replay + i)
        for t in captured:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = outputs()
        run(eager, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {replay}"
        assert torch.equal(captured[3], Cm)
