"""Packing / unpacking / micro-kernel restatement.

Pinned (a) bit for bit against the reference's own pack_*.cpp, unpack_*.cpp and
6x16 kernel compiled from /root/reference (oracle/_ref), and (b) by properties
that do not need the reference: packing is a permutation of the source plus
zero padding, and unpack(pack(C)) == C."""
import numpy as np
import pytest

import oracle
from tests import refparts

SHAPES = [(1, 1, 1), (10, 96, 111), (111, 10, 96), (96, 111, 10), (960, 111, 96),
          (111, 960, 2111), (2111, 96, 111), (500, 700, 300), (1030, 1500, 1000)]
SCHEDS = [oracle.KMN, oracle.MKN, oracle.NKM]


def _mats(M, K, N):
    return oracle.uniform((M, K), 11), oracle.uniform((K, N), 12), oracle.uniform((M, N), 13)


def _slack(a, fill=0.0, extra=256):
    """A copy of `a` with room behind it: the reference's packing loops read (and for partial
    panels write) a little past the arrays they are given."""
    buf = np.full(a.size + extra, fill, np.float32)
    buf[:a.size] = a.ravel()
    return buf


@pytest.mark.parametrize("p", [1, 3, 8])
@pytest.mark.parametrize("sch", SCHEDS)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_pack_matches_reference_sources(shape, sch, p):
    L = refparts.lib()
    M, K, N = shape
    cx = oracle.make_cntx()
    x = oracle.init_block_dims(M, N, K, p, cx, sch)
    dims = refparts.dims_array(x)
    A, B, Cm = _mats(M, K, N)

    assert L.ref_packed_A_size(M, K, p, dims, cx.mr, cx.nr, sch) == oracle.packed_A_size(M, K, p, x, cx, sch)
    assert L.ref_packed_B_size(K, N, p, dims, cx.mr, cx.nr) == oracle.packed_B_size(K, N, p, x, cx)
    assert L.ref_packed_C_size(M, N, p, dims, cx.mr, cx.nr, sch) == oracle.packed_C_size(M, N, p, x, cx, sch)

    Ap = oracle.pack_A(A, p, x, cx, sch)
    Ar = _slack(Ap, np.nan)
    Ar[:Ap.size] = np.nan
    L.ref_pack_A(refparts.f(_slack(A)), refparts.f(Ar), M, K, p, dims, cx.mr, cx.nr, sch)
    assert np.array_equal(Ap, Ar[:Ap.size])

    # MKN/NKM pack_B in the reference bounds-checks the N padding only in the
    # last core of the last K block (pack_m_first.cpp:128-139 passes a K-derived
    # flag as pad_n), so elsewhere its padding columns hold wrapped reads of B
    # instead of zeros.  Those columns never reach C.  Compare real data
    # everywhere and the padding only for KMN; give the reference slack to read.
    Bp = oracle.pack_B(B, p, x, cx, sch)
    Br = _slack(Bp, np.nan)
    Br[:Bp.size] = np.nan
    L.ref_pack_B(refparts.f(_slack(B)), refparts.f(Br), K, N, p, dims, cx.mr, cx.nr, sch)
    Br = Br[:Bp.size]
    if sch == oracle.KMN:
        assert np.array_equal(Bp, Br)
    else:
        real = oracle.pack_B(np.ones((K, N), np.float32), p, x, cx, sch) != 0
        assert real.sum() == K * N
        assert np.array_equal(Bp[real], Br[real])
        assert not Bp[~real].any()

    # unpack: the reference writes only the in-range part of C
    Cp = oracle.uniform(oracle.packed_C_size(M, N, p, x, cx, sch) // 4, 14)
    Cu = oracle.unpack_C(Cp, M, N, p, x, cx, sch, into=np.full((M, N), 7.0, np.float32))
    Cr = _slack(np.full((M, N), 7.0, np.float32))
    L.ref_unpack_C(refparts.f(Cr), refparts.f(_slack(Cp)), M, N, p, dims, cx.mr, cx.nr, sch)
    assert np.array_equal(Cu, Cr[:M * N].reshape(M, N))

    # pack_C: identical to the reference except NKM with a partial last M block,
    # where the reference's own offset disagrees with its unpack and schedule
    Cpk = oracle.pack_C(Cm, p, x, cx, sch)
    if not (sch == oracle.NKM and x.m_pad):
        Cpr = _slack(Cpk, np.nan)
        Cpr[:Cpk.size] = np.nan
        L.ref_pack_C(refparts.f(_slack(Cm)), refparts.f(Cpr), M, N, p, dims, cx.mr, cx.nr, sch)
        assert np.array_equal(Cpk, Cpr[:Cpk.size])


@pytest.mark.parametrize("p", [2, 8])
@pytest.mark.parametrize("sch", SCHEDS)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_pack_is_permutation_plus_zero_padding(shape, sch, p):
    M, K, N = shape
    cx = oracle.make_cntx()
    x = oracle.init_block_dims(M, N, K, p, cx, sch)
    # distinct positive integers make "same multiset" a strong statement
    A = np.arange(1, M * K + 1, dtype=np.float32).reshape(M, K)
    B = np.arange(1, K * N + 1, dtype=np.float32).reshape(K, N)
    Cm = np.arange(1, M * N + 1, dtype=np.float32).reshape(M, N)
    for src, packed in ((A, oracle.pack_A(A, p, x, cx, sch)), (B, oracle.pack_B(B, p, x, cx, sch)),
                        (Cm, oracle.pack_C(Cm, p, x, cx, sch))):
        assert not np.isnan(packed).any()
        nz = packed[packed != 0]
        assert nz.size == src.size
        assert np.array_equal(np.sort(nz), src.ravel())
    assert np.array_equal(oracle.unpack_C(oracle.pack_C(Cm, p, x, cx, sch), M, N, p, x, cx, sch), Cm)


def test_packed_panel_layout_explicit():
    """KMN layouts written out by hand for a shape small enough to reason about:
    A_p = [m_r-panel][k][j<m_r], B_p = [n_r-panel][k][j<n_r] inside one block."""
    cx = oracle.make_cntx(mr=2, nr=4)
    M, K, N, p = 4, 3, 8, 1
    x = oracle.init_block_dims(M, N, K, p, cx, oracle.KMN, 4, 3, 8)
    A = np.arange(M * K, dtype=np.float32).reshape(M, K)
    B = np.arange(K * N, dtype=np.float32).reshape(K, N)
    Ap = oracle.pack_A(A, p, x, cx, oracle.KMN)
    Bp = oracle.pack_B(B, p, x, cx, oracle.KMN)
    wantA = [A[pnl * 2 + j, k] for pnl in range(2) for k in range(K) for j in range(2)]
    wantB = [B[k, pnl * 4 + j] for pnl in range(2) for k in range(K) for j in range(4)]
    assert Ap.tolist() == wantA
    assert Bp.tolist() == wantB


@pytest.mark.parametrize("k", [1, 3, 4, 7, 36, 492])
def test_ukernel_matches_reference_6x16(k):
    L = refparts.lib()
    Ap = oracle.uniform(6 * k, 21)
    # the reference kernel uses aligned 32-byte loads of B
    raw = np.empty(16 * k + 16, dtype=np.float32)
    off = (-raw.ctypes.data % 32) // 4
    Bp = raw[off:off + 16 * k]
    Bp[:] = oracle.uniform(16 * k, 22)
    C0 = oracle.uniform(96, 23)
    mine = oracle.ukernel(Ap, np.ascontiguousarray(Bp), C0.copy(), 6, 16, k)
    ref = C0.copy()
    L.ref_ukernel_6x16(refparts.f(Ap), Bp.ctypes.data_as(refparts._fp), refparts.f(ref), k)
    assert np.array_equal(mine, ref)


@pytest.mark.parametrize("mr,nr,k", [(6, 16, 9), (8, 12, 5), (2, 4, 3)])
def test_ukernel_is_fma_chain(mr, nr, k):
    """Each element is one fused-multiply-add chain in ascending k: compare with
    an exactly rounded emulation (fp64 product of two fp32 is exact; one rounding per step)."""
    Ap, Bp, C0 = oracle.uniform(mr * k, 31), oracle.uniform(nr * k, 32), oracle.uniform(mr * nr, 33)
    got = oracle.ukernel(Ap, Bp, C0.copy(), mr, nr, k).reshape(mr, nr)
    acc = C0.reshape(mr, nr).astype(np.float64)
    for kk in range(k):
        a = Ap[kk * mr:(kk + 1) * mr].astype(np.float64)[:, None]
        b = Bp[kk * nr:(kk + 1) * nr].astype(np.float64)[None, :]
        acc = (a * b + acc).astype(np.float32).astype(np.float64)  # 24+24+... fits: one rounding
    assert np.array_equal(got, acc.astype(np.float32))
