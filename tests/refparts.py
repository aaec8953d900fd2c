"""Loader for oracle/_ref/libcake_ref_parts.so (reference sources compiled where they lie).

Only present where /root/reference was available at build time; tests that
need it skip otherwise."""
import ctypes as C
from pathlib import Path

import numpy as np
import pytest

import oracle

PATH = Path(oracle.HERE) / "_ref" / "libcake_ref_parts.so"
_fp = C.POINTER(C.c_float)
_ip = C.POINTER(C.c_int)
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not PATH.exists():
            pytest.skip("oracle/_ref not built (reference sources absent)")
        L = C.CDLL(str(PATH))
        i = C.c_int
        L.ref_packed_A_size.restype = C.c_size_t
        L.ref_packed_A_size.argtypes = [i, i, i, _ip, i, i, i]
        L.ref_packed_B_size.restype = C.c_size_t
        L.ref_packed_B_size.argtypes = [i, i, i, _ip, i, i]
        L.ref_packed_C_size.restype = C.c_size_t
        L.ref_packed_C_size.argtypes = [i, i, i, _ip, i, i, i]
        for name in ("ref_pack_A", "ref_pack_B", "ref_pack_C", "ref_unpack_C"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [_fp, _fp, i, i, i, _ip, i, i, i]
        L.ref_ukernel_6x16.restype = None
        L.ref_ukernel_6x16.argtypes = [_fp, _fp, _fp, i]
        L.ref_schedule_mvm.restype = None
        L.ref_schedule_mvm.argtypes = [_fp, _fp, _fp, i, i, i, _ip, i]
        L.ref_im_2_col.restype = None
        L.ref_im_2_col.argtypes = [_fp, _fp, i, i, i, i, i, i, i]
        L.ref_init_block_dims_conv.restype = None
        L.ref_init_block_dims_conv.argtypes = [i] * 13 + [C.c_double, _ip]
        L.ref_pack_filters.restype = None
        L.ref_pack_filters.argtypes = [_fp, _fp, i, i, i, _ip, i, i]
        assert L.ref_sizeof_blk_dims() == C.sizeof(oracle.BlkDims)
        _lib = L
    return _lib


def dims_array(x: oracle.BlkDims):
    vals = [getattr(x, n) for n in oracle.BLK_FIELDS]
    return (C.c_int * 26)(*vals)


def f(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)
