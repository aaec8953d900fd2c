"""Blocks of the reference's direct convolution and its packed filters (examples/cake_conv.cpp:
get_cache_dims_conv + init_block_dims_conv :262-425, pack_filters :536-610): the oracle's restatement
and the library's host arithmetic against (1) what the reference's own compiled functions returned
(tests/golden/conv_filter_vectors.npz; and oracle/_ref itself where it is built), (2) a block table
computed by hand from the reference's formulas, (3) the layout's definition, element by element."""
import ctypes as C
import json
from pathlib import Path

import numpy as np
import pytest

import oracle

GOLDEN = Path(__file__).resolve().parent / "golden" / "conv_filter_vectors.npz"


def _golden():
    z = np.load(GOLDEN, allow_pickle=False)
    return json.loads(bytes(z["meta"]).decode()), z


def _cx(L2):
    cx = oracle.make_cntx(mr=6, nr=16, L2=L2)
    cx.alpha_n = 1.0
    return cx


def _dims_list(x):
    return [getattr(x, n) for n in oracle.BLK_FIELDS]


def test_conv_blocks_by_hand():
    """Cout = 100 over p = 4 cores, m_r = 6: ceil(100 / 4) = 25 -> 24 channels per core; n_c =
    floor(4 * 24 / 32) = 3 rows; k_c = ceil((2^18 - 3 * 32 * 24) / (24 * 9 + 3 * 34)) = 818 -> Cin = 64.
    100 = 96 + 4: one panel of 6 is left for a single core.  With L2 = 64 KiB k_c = ceil(14080 / 318) = 45."""
    x = oracle.init_block_dims_conv(3, 3, 34, 34, 32, 32, 64, 100, 1, 4, _cx(1 << 20))
    got = {n: getattr(x, n) for n in oracle.BLK_FIELDS}
    want = dict(m_c=24, k_c=64, n_c=3, m_c1=6, k_c1=0, n_c1=2, m_c1_last_core=6, mr_rem=1, p_l=1, m_pad=1, k_pad=0,
                n_pad=1, Mb=2, Kb=1, Nb=11, M_padded=102, N_padded=32, sch=oracle.KMN)
    assert {k: got[k] for k in want} == want
    x = oracle.init_block_dims_conv(3, 3, 34, 34, 32, 32, 64, 100, 1, 4, _cx(64 << 10))
    assert (x.k_c, x.k_c1, x.Kb, x.k_pad) == (45, 19, 2, 1)


def test_oracle_equals_reference_outputs():
    meta, z = _golden()
    for i, (Cin, Cout, Hin, Win, p, L2) in enumerate(meta["cases"]):
        cx = _cx(L2)
        x = oracle.init_block_dims_conv(3, 3, Win, Hin, Win - 2, Hin - 2, Cin, Cout, 1, p, cx)
        assert _dims_list(x) == [int(v) for v in z[f"case{i}_dims"]], (i, "block dims")
        F = oracle.uniform((Cout, Cin * 9), meta["filter_seed"])
        got = oracle.pack_filters(F, Cin, 9, p, x, cx)
        assert np.array_equal(got, z[f"case{i}_packed"]), (i, "packed filters")


def test_oracle_equals_reference_build():
    """The same comparison against the reference's functions themselves, on more geometries."""
    from tests import refparts
    L = refparts.lib()
    rng = np.random.default_rng(5)
    for case in range(40):
        Cin, Cout = int(rng.integers(1, 90)), int(rng.integers(1, 200))
        Hin, Win = int(rng.integers(3, 40)), int(rng.integers(3, 70))
        p, L2 = int(rng.integers(1, 9)), int(rng.choice([8 << 10, 64 << 10, 1 << 20]))
        cx = _cx(L2)
        probe = oracle.init_block_dims_conv(3, 3, Win, Hin, Win - 2, Hin - 2, Cin, Cout, 1, p, cx)
        raw = (L2 / 4.0 - probe.n_c * (Win - 2) * probe.m_c) / (probe.m_c * 9 + probe.n_c * Win)
        if int(np.ceil(raw)) == 0:
            continue          # the reference divides by this k_c (a floating point exception, not a result)
        out = (C.c_int * 26)()
        L.ref_init_block_dims_conv(3, 3, Win, Hin, Win - 2, Hin - 2, Cin, Cout, 1, p, 6, 16, L2, 1.0, out)
        x = oracle.init_block_dims_conv(3, 3, Win, Hin, Win - 2, Hin - 2, Cin, Cout, 1, p, cx)
        assert _dims_list(x) == list(out), (case, Cin, Cout, Hin, Win, p, L2)
        F = oracle.uniform((Cout, Cin * 9), 70 + case)
        src = np.zeros(F.size + 4096, np.float32)
        src[:F.size] = F.ravel()
        ref = np.full(x.M_padded * Cin * 9 + 256, np.nan, np.float32)
        L.ref_pack_filters(refparts.f(src), refparts.f(ref), Cout, Cin * 9, p, out, 6, 16)
        assert np.array_equal(oracle.pack_filters(F, Cin, 9, p, x, cx), ref[:x.M_padded * Cin * 9]), case


def test_packed_filters_are_a_permutation_with_zero_rows():
    """Every filter value lands exactly once, rows past Cout are zero, and inside an m_r panel the
    order is [tap][channel][m_r] (checked from the definition on the first panel of the first block)."""
    Cin, Cout, p, taps = 20, 50, 3, 9
    cx = _cx(8 << 10)
    x = oracle.init_block_dims_conv(3, 3, 30, 30, 28, 28, Cin, Cout, 1, p, cx)
    assert x.Kb > 1 and x.m_pad
    F = np.arange(1, Cout * Cin * taps + 1, dtype=np.float32).reshape(Cout, Cin * taps)
    P = oracle.pack_filters(F, Cin, taps, p, x, cx)
    assert P.size == x.M_padded * Cin * taps
    nz = P[P != 0]
    assert nz.size == F.size and np.array_equal(np.sort(nz), F.ravel())
    assert np.count_nonzero(P == 0) == (x.M_padded - Cout) * Cin * taps
    kc = x.k_c
    first = P[:6 * kc * taps].reshape(taps, kc, 6)
    want = F[:6].reshape(6, Cin, taps)[:, :kc, :].transpose(2, 1, 0)
    assert np.array_equal(first, want)


def test_library_host_arithmetic_equals_oracle():
    """cake_hip_init_block_dims_conv and the packed-size query (host code of the shipped library)."""
    import cake_on_cpu_amd as cake
    lib = cake.load()
    rng = np.random.default_rng(9)
    for case in range(200):
        Cin, Cout = int(rng.integers(1, 300)), int(rng.integers(1, 600))
        Hin, Win = int(rng.integers(3, 80)), int(rng.integers(3, 80))
        Hf, Wf = int(rng.integers(1, min(Hin, 6) + 1)), int(rng.integers(1, min(Win, 6) + 1))
        p, L2 = int(rng.integers(1, 17)), int(rng.choice([8 << 10, 64 << 10, 1 << 20, 4 << 20]))
        cx = oracle.make_cntx(mr=6, nr=16, L2=L2)
        cx.alpha_n = float(rng.choice([1.0, 0.5, 2.25]))
        want = oracle.init_block_dims_conv(Wf, Hf, Win, Hin, Win - Wf + 1, Hin - Hf + 1, Cin, Cout, 1, p, cx)
        hcx = cake.CpuCntx(alpha_n=cx.alpha_n, mr=6, nr=16, L1=48 << 10, L2=L2, L3=32 << 20, ncores=8)
        got = cake.BlkDims()
        st = lib.cake_hip_init_block_dims_conv(Wf, Hf, Win, Hin, Win - Wf + 1, Hin - Hf + 1, Cin, Cout, 1, p,
                                               C.byref(hcx), C.byref(got))
        assert st == 0
        assert [getattr(got, n) for n in oracle.BLK_FIELDS] == _dims_list(want), (case, Cin, Cout, Hin, Win, Hf, Wf, p, L2)
        size = lib.cake_hip_packed_filters_size(Cout, Cin, Hf * Wf, p, C.byref(got), C.byref(hcx))
        assert size == want.M_padded * Cin * Hf * Wf * 4
