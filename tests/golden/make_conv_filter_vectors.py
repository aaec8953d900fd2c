"""Writes tests/golden/conv_filter_vectors.npz: what the reference's OWN init_block_dims_conv and
pack_filters (examples/cake_conv.cpp:262-425,536-610, compiled where it lies into
oracle/_ref/libcake_ref_parts.so by oracle/build_ref.sh) return for seeded 3 x 3 filters.  Data
only: geometry, the 26 block dimensions and the packed filters.

Run from the repository root, where /root/reference exists:
    bash oracle/build_ref.sh && python -m tests.golden.make_conv_filter_vectors"""
import ctypes as C
import json
from pathlib import Path

import numpy as np

import oracle
from tests import refparts

OUT = Path(__file__).resolve().parent / "conv_filter_vectors.npz"

# Cin, Cout, Hin, Win, p, L2 bytes (3 x 3 filters, stride 1; mr = 6, nr = 16, alpha_n = 1)
CASES = [(64, 100, 34, 34, 4, 1 << 20), (64, 100, 34, 34, 4, 64 << 10), (5, 130, 21, 37, 3, 256 << 10),
         (16, 24, 34, 34, 4, 2 << 20), (40, 7, 12, 50, 8, 32 << 10), (33, 61, 9, 9, 2, 16 << 10),
         (32, 150, 18, 18, 8, 2 << 20)]
FILTER_SEED = 61


def ref_dims(L, Cin, Cout, Hin, Win, p, L2):
    out = (C.c_int * 26)()
    L.ref_init_block_dims_conv(3, 3, Win, Hin, Win - 2, Hin - 2, Cin, Cout, 1, p, 6, 16, L2, 1.0, out)
    return np.array(list(out), np.int32)


def main():
    L = refparts.lib()
    out = {}
    for i, (Cin, Cout, Hin, Win, p, L2) in enumerate(CASES):
        dims = ref_dims(L, Cin, Cout, Hin, Win, p, L2)
        F = oracle.uniform((Cout, Cin * 9), FILTER_SEED)
        m_padded = int(dims[oracle.BLK_FIELDS.index("M_padded")])
        Fp = np.full(m_padded * Cin * 9 + 256, np.nan, np.float32)
        src = np.zeros(F.size + 4096, np.float32)      # the reference reads a little past the last row when it pads
        src[:F.size] = F.ravel()
        L.ref_pack_filters(refparts.f(src), refparts.f(Fp), Cout, Cin * 9, p, (C.c_int * 26)(*[int(v) for v in dims]), 6, 16)
        out[f"case{i}_dims"] = dims
        out[f"case{i}_packed"] = Fp[:m_padded * Cin * 9].copy()
    meta = {"cases": CASES, "filter_seed": FILTER_SEED, "mr": 6, "nr": 16, "alpha_n": 1.0}
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
