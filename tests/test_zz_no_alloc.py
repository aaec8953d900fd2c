"""cake_hip_sgemm_noalloc: the entry point for callers that cannot allocate device memory.

It runs the kernels of cake_hip_sgemm with their partial sums in a fixed array of the library's
device image, so its result must be the very bits cake_hip_sgemm gives (the bar for the product
itself -- 1e-4 of sum |a||b| against the oracle -- is checked on top).  Every shape is run twice
in a row, the second time on a smaller product, since all calls share the one array and it keeps
the previous call's contents."""
import ctypes as C

import numpy as np
import pytest

import cake_on_cpu_amd as cake
from cake_on_cpu_amd import _lib
import oracle

pytestmark = pytest.mark.gpu

# (M, K, N) pairs: first call, then a smaller product of the same kind right after it
CASES = {
    "split_k": [(256, 8192, 256), (192, 4096, 192)],
    "split_k_many_slices": [(64, 50000, 64), (60, 7000, 50)],
    "tail_split": [(1100, 512, 1100), (700, 300, 650)],
    "stream_rows": [(16, 4096, 4096), (9, 2048, 1500)],
    "stream_cols": [(4096, 4096, 24), (3000, 1024, 7)],
    # up to 16 columns of B that are turned into rows first: the turned copy comes from the same array
    "stream_cols_turned": [(8200, 4096, 16), (4100, 4096, 9)],
    "single_row": [(1, 5000, 3000), (1, 700, 900)],
    "single_column": [(3000, 9000, 1), (1200, 8200, 1)],
    "no_partial_sums": [(2111, 300, 960), (96, 111, 10)],
}


def _noalloc(tA, tB, tC, M, N, K, sch, acc):
    import torch
    st = cake.load().cake_hip_sgemm_noalloc(tA.data_ptr(), tB.data_ptr(), tC.data_ptr(), M, N, K, sch, acc,
                                            torch.cuda.current_stream().cuda_stream)
    _lib.check(st, "cake_hip_sgemm_noalloc")


def _plain(tA, tB, tC, M, N, K, sch, acc):
    import torch
    st = cake.load().cake_hip_sgemm(tA.data_ptr(), tB.data_ptr(), tC.data_ptr(), M, N, K, sch, acc, None,
                                    torch.cuda.current_stream().cuda_stream, None)
    _lib.check(st, "cake_hip_sgemm")


@pytest.mark.parametrize("kind", list(CASES))
def test_noalloc_equals_cake_hip_sgemm_twice_in_a_row(kind):
    import torch
    _lib.check(cake.load().cake_hip_init(0), "cake_hip_init")
    for acc in (0, 1):
        for call, (M, K, N) in enumerate(CASES[kind]):
            print(f"noalloc {kind} call {call} M={M} K={K} N={N} accumulate={acc}", flush=True)
            A, B = oracle.uniform((M, K), 31 + call), oracle.uniform((K, N), 41 + call)
            C0 = oracle.uniform((M, N), 51 + call)
            tA, tB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
            want, got = torch.from_numpy(C0).cuda(), torch.from_numpy(C0).cuda()
            _plain(tA, tB, want, M, N, K, cake.NA, acc)
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            _noalloc(tA, tB, got, M, N, K, cake.NA, acc)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the device's free memory"
            got_h, want_h = got.cpu().numpy(), want.cpu().numpy()
            assert np.array_equal(got_h, want_h), (kind, call, acc)
            C64, S = oracle.gemm_f64(A, B)
            err = float(np.max(np.abs(got_h.astype(np.float64) - acc * C0 - C64) / (S + acc * np.abs(C0))))
            assert err <= 1e-4 and err <= 5e-6, (kind, call, acc, err)
            if call == 0 and acc == 0 and M * N * K <= 2.2e8:
                ref = oracle.cake_sgemm(A, B, 4, oracle.make_cntx())
                assert float(np.max(np.abs(got_h - ref) / S)) <= 1e-4


def test_noalloc_rejects_what_does_not_fit_and_host_memory():
    import torch
    _lib.check(cake.load().cake_hip_init(0), "cake_hip_init")
    # 640 x 16384 x 4096 runs in 8 K slices of 640 x 4096 floats: 80 MiB of partial sums
    M, K, N = 640, 16384, 4096
    pl = cake.plan(M, N, K)
    assert pl.split_k * M * N * 4 > 64 << 20, (pl.split_k, "the shape no longer needs more than the array holds")
    tA = torch.zeros((M, K), dtype=torch.float32, device="cuda")
    tB = torch.zeros((K, N), dtype=torch.float32, device="cuda")
    tC = torch.full((M, N), 7.0, dtype=torch.float32, device="cuda")
    st = cake.load().cake_hip_sgemm_noalloc(tA.data_ptr(), tB.data_ptr(), tC.data_ptr(), M, N, K, cake.NA, 0, None)
    assert st == _lib.ERR_RANGE
    assert b"partial sums" in cake.load().cake_hip_last_error()
    torch.cuda.synchronize()
    assert float(tC.min()) == 7.0 and float(tC.max()) == 7.0      # nothing was launched
    _plain(tA, tB, tC, M, N, K, cake.NA, 0)                          # the allocating entry point takes it
    torch.cuda.synchronize()
    assert float(tC.abs().max()) == 0.0
    # host operands would need staging buffers
    a = np.zeros((8, 8), np.float32)
    st = cake.load().cake_hip_sgemm_noalloc(a.ctypes.data, a.ctypes.data, a.ctypes.data, 8, 8, 8, cake.NA, 0, None)
    assert st == _lib.ERR_ARG
