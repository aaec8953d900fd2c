"""The oracle against committed outputs of the reference's own code (tests/golden/
reference_vectors.npz: the reference's pack_*.cpp, unpack_*.cpp, 6x16 kernel, schedule_mvm and
im_2_col compiled from its sources and run on seeded inputs).  Unlike the comparisons in
test_oracle_packing.py / test_oracle_gemv_conv.py these need no reference checkout, so they also
run where only the repository travels."""
import ctypes as C

import numpy as np
import pytest

import oracle
from tests import golden_vectors

META, Z = golden_vectors.load()
SEED = META["seeds"]


@pytest.mark.parametrize("i", range(len(META["pack"])), ids=lambda i: "x".join(map(str, META["pack"][i])))
def test_packing_equals_reference_output(i):
    M, K, N, p, sch = META["pack"][i]
    cx = oracle.make_cntx()
    x = oracle.init_block_dims(M, N, K, p, cx, sch)
    # the block dimensions handed to the reference are the oracle planner's
    assert [getattr(x, n) for n in oracle.BLK_FIELDS] == Z[f"pack{i}_dims"].tolist()
    A, B, Cm = oracle.uniform((M, K), SEED["A"]), oracle.uniform((K, N), SEED["B"]), oracle.uniform((M, N), SEED["C"])
    assert np.array_equal(oracle.pack_A(A, p, x, cx, sch), Z[f"pack{i}_A"])
    # M-first / N-first pack_B of the reference leaves part of the N padding unzeroed (wrapped reads
    # of B that never reach C): compare where elements of B belong, and the padding only for K-first
    Bp, Bref = oracle.pack_B(B, p, x, cx, sch), Z[f"pack{i}_B"]
    real = oracle.pack_B(np.ones((K, N), np.float32), p, x, cx, sch) != 0
    assert real.sum() == K * N and np.array_equal(Bp[real], Bref[real]) and not Bp[~real].any()
    if sch == oracle.KMN:
        assert np.array_equal(Bp, Bref)
    Cp = oracle.uniform(oracle.packed_C_size(M, N, p, x, cx, sch) // 4, SEED["Cp"])
    got = oracle.unpack_C(Cp, M, N, p, x, cx, sch, into=np.full((M, N), 7.0, np.float32))
    assert np.array_equal(got, Z[f"pack{i}_Cunpacked"])
    if not (sch == oracle.NKM and x.m_pad):  # the reference's n-first pack_C offset disagrees with its own unpack there
        assert np.array_equal(oracle.pack_C(Cm, p, x, cx, sch), Z[f"pack{i}_Cpacked"])


@pytest.mark.parametrize("k", META["ukernel"])
def test_micro_kernel_equals_reference_output(k):
    Ap, Bp, C0 = oracle.uniform(6 * k, SEED["uk_A"]), oracle.uniform(16 * k, SEED["uk_B"]), oracle.uniform(96, SEED["uk_C"])
    assert np.array_equal(oracle.ukernel(Ap, Bp, C0.copy(), 6, 16, k), Z[f"ukernel_k{k}"])


@pytest.mark.parametrize("case", META["gemv"], ids=lambda c: "x".join(map(str, c)))
def test_sgemv_equals_reference_output(case):
    M, K, p = case
    cx = oracle.make_cntx(mr=8)
    A, xv, y0 = oracle.uniform(M * K, SEED["gemv_A"]), oracle.uniform(K, SEED["gemv_x"]), oracle.uniform(M, SEED["gemv_y"])
    assert np.array_equal(oracle.cake_sgemv(A, xv, p, cx, y0=y0, M=M, K=K), Z[f"gemv_{M}_{K}_{p}"])


@pytest.mark.parametrize("case", META["im2col"], ids=lambda c: "x".join(map(str, c)))
def test_im_2_col_equals_reference_output(case):
    Cin, Hin, Win, Hf, Wf = case
    inp = oracle.uniform((Cin, Hin, Win), SEED["image"])
    got = oracle.im_2_col(inp, Hf, Wf, Hin - Hf + 1, Win - Wf + 1)
    assert np.array_equal(got, Z[f"im2col_{Cin}_{Hin}_{Win}_{Hf}_{Wf}"])
