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
