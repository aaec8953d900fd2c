"""Device contexts (cake_hip_ctx_create): each has workspaces, events and a stream of its own, so
two host threads on two contexts run different products at the same time -- split-K slices, tail
slices, the streaming kernels' partial sums all in flight at once -- and each result is bit for bit
what the same product gives alone on the default context."""
import threading

import numpy as np
import pytest

import cake_on_cpu_amd as cake
from cake_on_cpu_amd import _lib
import oracle

pytestmark = pytest.mark.gpu

# every one of these uses a workspace (K slices, tail slices, streaming or matrix-vector partial sums)
SHAPES_A = [(256, 8192, 256), (1100, 512, 1100), (16, 4096, 4096), (1, 5000, 3000), (64, 50000, 64)]
SHAPES_B = [(192, 4096, 192), (700, 300, 650), (4096, 4096, 24), (3000, 9000, 1), (60, 7000, 50)]


def _operands(shapes, base):
    import torch
    out = []
    for i, (M, K, N) in enumerate(shapes):
        A = torch.from_numpy(oracle.uniform((M, K), base + i)).cuda()
        B = torch.from_numpy(oracle.uniform((K, N), base + 50 + i)).cuda()
        out.append((A, B, M, K, N))
    return out


def _product(A, B, M, K, N, stream):
    import torch
    # (no fill: a fill kernel would run on torch's stream, which a context's own stream does not wait for)
    Cm = torch.empty((M, N), dtype=torch.float32, device="cuda")
    st = cake.load().cake_hip_sgemm(A.data_ptr(), B.data_ptr(), Cm.data_ptr(), M, N, K, cake.NA, 0, None, stream, None)
    _lib.check(st, "cake_hip_sgemm")
    return Cm


def test_two_contexts_on_two_streams_run_side_by_side():
    import torch
    ops = {"a": _operands(SHAPES_A, 100), "b": _operands(SHAPES_B, 300)}
    torch.cuda.synchronize()
    alone = {k: [_product(*o, 0).cpu().numpy() for o in v] for k, v in ops.items()}
    torch.cuda.synchronize()
    for (A, B, M, K, N), got in zip(ops["a"], alone["a"]):   # the bar itself, once
        C64, S = oracle.gemm_f64(A.cpu().numpy(), B.cpu().numpy())
        assert oracle.max_rel_err(got, C64, S) <= 5e-6

    ctxs = {"a": cake.Context(), "b": cake.Context()}
    assert ctxs["a"].stream and ctxs["b"].stream and ctxs["a"].stream != ctxs["b"].stream
    results, errors = {"a": [], "b": []}, []
    start = threading.Barrier(2)

    def worker(name):
        try:
            with ctxs[name] as ctx:
                assert cake.load().cake_hip_ctx_get_current() == ctx.handle
                start.wait()
                for rep in range(6):
                    # stream = NULL: the context's own stream; nothing waits for the host in between
                    outs = [_product(*o, None) for o in ops[name]]
                    _lib.check(cake.load().cake_hip_synchronize(), "sync")
                    results[name].append([t.cpu().numpy() for t in outs])
        except Exception as e:     # noqa: BLE001 -- reported below
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=worker, args=(n,)) for n in ("a", "b")]
    for t in threads: t.start()
    for t in threads: t.join()
    assert not errors, errors
    for name in ("a", "b"):
        for rep, outs in enumerate(results[name]):
            for i, got in enumerate(outs):
                assert np.array_equal(got, alone[name][i]), (name, rep, i)
    assert cake.load().cake_hip_ctx_get_current() is None     # the main thread never left the default context
    for c in ctxs.values():
        c.destroy()


def test_context_lifetime_and_errors():
    lib = cake.load()
    ctx = cake.Context()
    h = ctx.handle
    with ctx:
        M, K, N = 300, 200, 100
        A, B = oracle.uniform((M, K), 1), oracle.uniform((K, N), 2)
        Cm = np.zeros((M, N), np.float32)
        cake.cake_sgemm(A, B, Cm, M, N, K, 4)       # host operands staged through the context's own buffers
        C64, S = oracle.gemm_f64(A, B)
        assert oracle.max_rel_err(Cm, C64, S) <= 5e-6
    assert lib.cake_hip_ctx_get_current() is None
    ctx.destroy()
    assert lib.cake_hip_ctx_set_current(h) == _lib.ERR_ARG     # gone
    assert lib.cake_hip_ctx_destroy(h) == _lib.ERR_ARG
    assert lib.cake_hip_ctx_destroy(None) == _lib.OK
    assert lib.cake_hip_ctx_stream(h) is None
