"""Writes tests/golden/reference_vectors.npz: outputs of the reference's OWN code
for the parts of the path that compile straight from its sources
(oracle/_ref/libcake_ref_parts.so, built by oracle/build_ref.sh from
src/pack_*.cpp, src/unpack_*.cpp, src/kernels/haswell/dense.cpp,
examples/cake_gemv.cpp and examples/cake_conv.cpp where they lie under
/root/reference).  The file holds data only -- seeds and shapes of the inputs,
the block dimensions handed to the reference, and what the reference returned --
so the checks built on it also run where the reference is absent.

Run from the repository root, where /root/reference exists:
    bash oracle/build_ref.sh && python -m tests.golden.make_reference_vectors
Inputs are oracle.uniform(shape, seed) streams (counter-based, reproducible)."""
import ctypes as C
import json
from pathlib import Path

import numpy as np

import oracle
from tests import refparts

OUT = Path(__file__).resolve().parent / "reference_vectors.npz"

PACK_CASES = [  # M, K, N, p, sch
    (10, 7, 5, 1, oracle.KMN), (10, 7, 5, 3, oracle.MKN), (10, 7, 5, 2, oracle.NKM),
    (50, 33, 70, 3, oracle.KMN), (50, 33, 70, 1, oracle.MKN), (50, 33, 70, 3, oracle.NKM),
    (111, 96, 60, 3, oracle.KMN), (111, 96, 60, 8, oracle.MKN), (96, 60, 111, 2, oracle.NKM),
]
UKERNEL_K = [1, 7, 64]
GEMV_CASES = [(64, 7, 3), (200, 130, 4), (1024, 96, 8)]   # M (multiple of 8), K, p
IM2COL_CASES = [(3, 8, 9, 3, 3), (4, 6, 6, 1, 1), (2, 9, 7, 5, 3)]  # Cin, Hin, Win, Hf, Wf


def slack(a, extra=256):
    """The reference's packing loops read (and for partial panels write) a little past the
    arrays they are given; give every array it touches room behind the data."""
    buf = np.zeros(a.size + extra, np.float32)
    buf[:a.size] = a.ravel()
    return buf


def main():
    L = refparts.lib()
    out, meta = {}, {"pack": [], "ukernel": UKERNEL_K, "gemv": GEMV_CASES, "im2col": IM2COL_CASES,
                     "seeds": {"A": 11, "B": 12, "C": 13, "Cp": 14, "uk_A": 21, "uk_B": 22, "uk_C": 23,
                               "gemv_A": 41, "gemv_x": 42, "gemv_y": 43, "image": 51}}
    cx = oracle.make_cntx()
    for i, (M, K, N, p, sch) in enumerate(PACK_CASES):
        x = oracle.init_block_dims(M, N, K, p, cx, sch)
        dims = refparts.dims_array(x)
        A, B, Cm = oracle.uniform((M, K), 11), oracle.uniform((K, N), 12), oracle.uniform((M, N), 13)
        asize = L.ref_packed_A_size(M, K, p, dims, cx.mr, cx.nr, sch) // 4
        Ar = slack(np.zeros(asize, np.float32))
        L.ref_pack_A(refparts.f(slack(A)), refparts.f(Ar), M, K, p, dims, cx.mr, cx.nr, sch)
        Ar = Ar[:asize].copy()
        bsize = L.ref_packed_B_size(K, N, p, dims, cx.mr, cx.nr) // 4
        Br = slack(np.zeros(bsize, np.float32))
        L.ref_pack_B(refparts.f(slack(B)), refparts.f(Br), K, N, p, dims, cx.mr, cx.nr, sch)
        Br = Br[:bsize].copy()
        csize = L.ref_packed_C_size(M, N, p, dims, cx.mr, cx.nr, sch) // 4
        Cp = oracle.uniform(csize, 14)
        Cu = slack(np.full((M, N), 7.0, np.float32))
        L.ref_unpack_C(refparts.f(Cu), refparts.f(slack(Cp)), M, N, p, dims, cx.mr, cx.nr, sch)
        Cu = Cu[:M * N].reshape(M, N).copy()
        Cpk = slack(np.zeros(csize, np.float32))
        L.ref_pack_C(refparts.f(slack(Cm)), refparts.f(Cpk), M, N, p, dims, cx.mr, cx.nr, sch)
        Cpk = Cpk[:csize].copy()
        out[f"pack{i}_dims"] = np.array([getattr(x, n) for n in oracle.BLK_FIELDS], np.int32)
        out[f"pack{i}_A"], out[f"pack{i}_B"] = Ar, Br
        out[f"pack{i}_Cunpacked"], out[f"pack{i}_Cpacked"] = Cu, Cpk
        meta["pack"].append([M, K, N, p, sch])
    for k in UKERNEL_K:
        Ap = oracle.uniform(6 * k, 21)
        raw = np.empty(16 * k + 16, np.float32)
        off = (-raw.ctypes.data % 32) // 4          # the reference kernel uses aligned 32-byte loads of B
        Bp = raw[off:off + 16 * k]
        Bp[:] = oracle.uniform(16 * k, 22)
        Ct = oracle.uniform(96, 23).copy()
        L.ref_ukernel_6x16(refparts.f(Ap), Bp.ctypes.data_as(refparts._fp), refparts.f(Ct), k)
        out[f"ukernel_k{k}"] = Ct
    cx8 = oracle.make_cntx(mr=8)
    for (M, K, p) in GEMV_CASES:
        x = oracle.BlkDims()
        oracle.lib().orc_init_block_dims_mvm(M, K, p, C.byref(x), C.byref(cx8))
        A, xv, y = oracle.uniform(M * K, 41), oracle.uniform(K, 42), slack(oracle.uniform(M, 43))
        L.ref_schedule_mvm(refparts.f(slack(A)), refparts.f(slack(xv)), refparts.f(y), M, K, p, refparts.dims_array(x), 8)
        out[f"gemv_{M}_{K}_{p}"] = y[:M].copy()
    for (Cin, Hin, Win, Hf, Wf) in IM2COL_CASES:
        Hout, Wout = Hin - Hf + 1, Win - Wf + 1
        inp = oracle.uniform((Cin, Hin, Win), 51)
        cols = slack(np.zeros(Cin * Hf * Wf * Hout * Wout, np.float32))
        L.ref_im_2_col(refparts.f(slack(inp)), refparts.f(cols), Wf, Hf, Win, Hin, Wout, Hout, Cin)
        out[f"im2col_{Cin}_{Hin}_{Win}_{Hf}_{Wf}"] = cols[:Cin * Hf * Wf * Hout * Wout].reshape(Cin * Hf * Wf, Hout * Wout).copy()
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
