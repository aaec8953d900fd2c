"""cake_sgemv and im_2_col restatements."""
import ctypes as C

import numpy as np
import pytest

import oracle
from tests import refparts


@pytest.mark.parametrize("M,K,p", [(1024, 1024, 8), (4096, 2048, 8), (64, 7, 3), (8, 1, 1), (2048, 3000, 5)])
def test_sgemv_matches_reference_sources(M, K, p):
    """schedule_mvm + the 8-row AVX2 kernel compiled from examples/cake_gemv.cpp,
    driven with the same block dims (M a multiple of 8: the reference kernel
    over-runs y otherwise)."""
    L = refparts.lib()
    cx = oracle.make_cntx(mr=8)
    x = oracle.BlkDims()
    oracle.lib().orc_init_block_dims_mvm(M, K, p, C.byref(x), C.byref(cx))
    A = oracle.uniform(M * K, 41)  # column-major: A[k*M + m]
    xv = oracle.uniform(K, 42)
    y0 = oracle.uniform(M, 43)
    mine = oracle.cake_sgemv(A, xv, p, cx, y0=y0, M=M, K=K)
    def slack(a):  # the reference's 8-row kernel may touch a little past its arrays
        buf = np.zeros(a.size + 256, np.float32)
        buf[:a.size] = a
        return buf
    ref = slack(y0)
    L.ref_schedule_mvm(refparts.f(slack(A)), refparts.f(slack(xv)), refparts.f(ref), M, K, p, refparts.dims_array(x), 8)
    assert np.array_equal(mine, ref[:M])


@pytest.mark.parametrize("M,K,p", [(1024, 1024, 8), (1000, 333, 3), (13, 2111, 2), (1, 1, 1), (4099, 517, 8)])
def test_sgemv_against_fp64_and_accumulates(M, K, p):
    cx = oracle.make_cntx(mr=8)
    A = oracle.uniform(M * K, 41)
    xv = oracle.uniform(K, 42)
    y64, S = oracle.gemv_f64(A, xv, M, K, col_major=True)
    y = oracle.cake_sgemv(A, xv, p, cx, M=M, K=K)
    assert np.max(np.abs(y - y64) / np.maximum(S, 1e-30)) <= 2e-6
    # column-major contract: a row-major reading of the same buffer is a different answer
    if M > 1 and K > 1:
        yr, _ = oracle.gemv_f64(A, xv, M, K, col_major=False) if M == K else (None, None)
        if yr is not None:
            assert np.max(np.abs(y - yr)) > 1e-2
    # second call adds to y (examples/cake_gemv.cpp:94,139)
    y2 = oracle.cake_sgemv(A, xv, p, cx, y0=y, M=M, K=K)
    assert np.max(np.abs(y2 - 2 * y64) / np.maximum(S, 1e-30)) <= 4e-6


def test_mvm_block_dims_closed_form():
    """get_cache_dims_mvm (examples/cake_gemv.cpp:273-340): positive root of
    x^2 + 2x = L2/4, rounded up to the next multiple of 64."""
    cx = oracle.make_cntx(mr=8, L2=2 << 20)
    x = oracle.BlkDims()
    oracle.lib().orc_init_block_dims_mvm(16384, 16384, 8, C.byref(x), C.byref(cx))
    root = int((-2 + (4 + 4 * (2 << 20) / 4) ** 0.5) / 2)
    assert root == 723
    assert x.m_c == x.k_c == 768
    assert (x.Mb, x.Kb) == (-(-16384 // (8 * 768)), -(-16384 // 768))


@pytest.mark.parametrize("Cin,Hin,Win,Hf,Wf", [(3, 18, 18, 3, 3), (5, 9, 13, 3, 3), (2, 6, 7, 1, 1), (4, 8, 8, 5, 3)])
def test_im_2_col_matches_reference_sources(Cin, Hin, Win, Hf, Wf):
    L = refparts.lib()
    Hout, Wout = Hin - Hf + 1, Win - Wf + 1
    inp = oracle.uniform((Cin, Hin, Win), 51)
    mine = oracle.im_2_col(inp, Hf, Wf, Hout, Wout)
    ref = np.empty_like(mine)
    L.ref_im_2_col(refparts.f(inp), refparts.f(ref), Wf, Hf, Win, Hin, Wout, Hout, Cin)
    assert np.array_equal(mine, ref)


@pytest.mark.parametrize("stride,pad", [(1, 0), (1, 1), (2, 1), (2, 0), (3, 2)])
def test_im2col_brute_force_definition(stride, pad):
    Bn, Cin, Hin, Win, Hf, Wf = 2, 3, 9, 8, 3, 3
    inp = oracle.uniform((Bn, Cin, Hin, Win), 52)
    got = oracle.im2col(inp, Hf, Wf, stride, pad)
    Hout = (Hin + 2 * pad - Hf) // stride + 1
    Wout = (Win + 2 * pad - Wf) // stride + 1
    padded = np.zeros((Bn, Cin, Hin + 2 * pad, Win + 2 * pad), np.float32)
    padded[:, :, pad:pad + Hin, pad:pad + Win] = inp
    for c in range(Cin):
        for h in range(Hf):
            for w in range(Wf):
                k = c * Hf * Wf + h * Wf + w
                for b in range(Bn):
                    for ho in range(Hout):
                        for wo in range(Wout):
                            n = (b * Hout + ho) * Wout + wo
                            assert got[k, n] == padded[b, c, ho * stride + h, wo * stride + w]


def test_pad1_equals_prepadded_input():
    inp = oracle.uniform((2, 4, 7, 6), 53)
    pre = np.zeros((2, 4, 9, 8), np.float32)
    pre[:, :, 1:-1, 1:-1] = inp
    assert np.array_equal(oracle.im2col(inp, 3, 3, 1, 1), oracle.im2col(pre, 3, 3, 1, 0))


@pytest.mark.parametrize("stride,pad", [(1, 1), (2, 0)])
def test_conv_as_im2col_gemm_equals_naive_conv(stride, pad, cx8):
    Bn, Cin, Cout, Hin, Win = 2, 5, 7, 10, 9
    inp = oracle.uniform((Bn, Cin, Hin, Win), 54)
    wt = oracle.uniform((Cout, Cin, 3, 3), 55)
    ref, S = oracle.conv_naive_f64(inp, wt, stride, pad)
    cols = oracle.im2col(inp, 3, 3, stride, pad)
    out = oracle.cake_sgemm(wt.reshape(Cout, -1), cols, 4, cx8, sch=oracle.KMN)
    _, _, Hout, Wout = ref.shape
    out = out.reshape(Cout, Bn, Hout, Wout).transpose(1, 0, 2, 3)
    assert np.max(np.abs(out - ref) / S) <= 2e-6
