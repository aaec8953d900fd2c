"""CPU oracle for the CAKE fp32 GEMM hot path -- TEST INFRASTRUCTURE ONLY.

ctypes bindings over ``oracle/cake_oracle.c`` (a from-scratch C restatement of
the reference algorithm: planner -> pack -> K/M/N-first snake schedule ->
6x16 outer-product micro-kernel -> unpack, plus cake_sgemv, im_2_col and the
linear layer that calls cake_sgemm) and
over the fp64 closed-form checkers that live in the same file.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped library never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "libcake_oracle.so"
SRC_PATH = HERE / "cake_oracle.c"

KMN, MKN, NKM, NA = 0, 1, 2, 3
SCHED_NAMES = {KMN: "KMN", MKN: "MKN", NKM: "NKM", NA: "NA"}

BLK_FIELDS = [
    "m_c", "k_c", "n_c", "m_c1", "k_c1", "n_c1",
    "m_c1_last_core", "n_c1_last_core", "k_c1_last_core",
    "mr_rem", "nr_rem", "k_rem", "p_l", "pm_l", "pn_l", "pm", "pn",
    "m_pad", "k_pad", "n_pad", "Mb", "Kb", "Nb", "M_padded", "N_padded", "sch",
]


class BlkDims(C.Structure):
    _fields_ = [(n, C.c_int) for n in BLK_FIELDS]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n in BLK_FIELDS}


class Cntx(C.Structure):
    _fields_ = [("alpha_n", C.c_double), ("mr", C.c_int), ("nr", C.c_int),
                ("L1", C.c_int), ("L2", C.c_int), ("L3", C.c_int), ("ncores", C.c_int)]


def make_cntx(mr=6, nr=16, L1=48 << 10, L2=2 << 20, L3=105 << 20, ncores=8) -> Cntx:
    """A fixed machine description (defaults: the 8-core host the reference was probed on)."""
    return Cntx(1.0, mr, nr, L1, L2, L3, ncores)


def build(force: bool = False) -> Path:
    """Compile the C restatement with the reference's own optimisation flags
    (Makefile:129: -O2 -mavx -mfma -fopenmp; -mavx2 added for the 256-bit FMA kernel)."""
    if LIB_PATH.exists() and not force and LIB_PATH.stat().st_mtime >= SRC_PATH.stat().st_mtime:
        return LIB_PATH
    cmd = ["gcc", "-O2", "-mavx2", "-mfma", "-fopenmp", "-fPIC", "-shared", "-std=gnu11",
           "-Wall", "-Wextra", "-o", str(LIB_PATH), str(SRC_PATH), "-lm"]
    subprocess.run(cmd, check=True)
    return LIB_PATH


_lib = None
_fp = C.POINTER(C.c_float)
_dp = C.POINTER(C.c_double)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        build()
    L = C.CDLL(str(LIB_PATH))
    bp, cp = C.POINTER(BlkDims), C.POINTER(Cntx)
    i = C.c_int
    sig = {
        "orc_fill_uniform": (None, [_fp, C.c_size_t, C.c_uint64]),
        "orc_physical_cores": (i, []),
        "orc_query_cntx": (None, [cp]),
        "orc_derive_schedule": (i, [i, i, i, i, i, cp]),
        "orc_get_cache_dims": (None, [i, i, i, i, cp, i, i, i, i, C.POINTER(i), C.POINTER(i), C.POINTER(i), C.POINTER(i)]),
        "orc_init_block_dims": (None, [i, i, i, i, bp, cp, i, i, i, i]),
        "orc_packed_A_size": (C.c_size_t, [i, i, i, bp, cp, i]),
        "orc_packed_B_size": (C.c_size_t, [i, i, i, bp, cp]),
        "orc_packed_C_size": (C.c_size_t, [i, i, i, bp, cp, i]),
        "orc_pack_A": (C.c_double, [_fp, _fp, i, i, i, bp, cp, i]),
        "orc_pack_B": (None, [_fp, _fp, i, i, i, bp, cp, i]),
        "orc_pack_C": (None, [_fp, _fp, i, i, i, bp, cp, i]),
        "orc_unpack_C": (None, [_fp, _fp, i, i, i, bp, cp, i]),
        "orc_ukernel": (None, [_fp, _fp, _fp, i, i, i]),
        "orc_schedule_KMN": (None, [_fp, _fp, _fp, i, i, i, i, cp, bp]),
        "orc_schedule_MKN": (None, [_fp, _fp, _fp, i, i, i, i, cp, bp]),
        "orc_schedule_NKM": (None, [_fp, _fp, _fp, i, i, i, i, cp, bp]),
        "orc_cake_sgemm": (C.c_double, [_fp, _fp, _fp, i, i, i, i, cp, i, i, C.c_float, C.c_float, i, i, i, i, bp]),
        "orc_init_block_dims_mvm": (None, [i, i, i, bp, cp]),
        "orc_cake_sgemv": (C.c_double, [_fp, _fp, _fp, i, i, i, cp]),
        "orc_im2col": (None, [_fp, _fp, i, i, i, i, i, i, i, i, i, i]),
        "orc_im_2_col": (None, [_fp, _fp, i, i, i, i, i, i, i]),
        "orc_gemm_f64": (None, [_fp, _fp, i, i, i, _dp, _dp]),
        "orc_max_rel_err": (C.c_double, [_fp, _dp, _dp, C.c_size_t]),
        "orc_gemv_f64": (None, [_fp, _fp, i, i, i, _dp, _dp]),
        "orc_conv_naive_f64": (None, [_fp, _fp, _dp, _dp] + [i] * 11),
        "orc_init_block_dims_conv": (None, [i] * 10 + [bp, cp]),
        "orc_pack_filters": (None, [_fp, _fp, i, i, i, i, bp, cp]),
        "orc_sizeof_blk_dims": (i, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    assert L.orc_sizeof_blk_dims() == C.sizeof(BlkDims)
    _lib = L
    return L


def _f(a: np.ndarray):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def _d(a: np.ndarray):
    assert a.dtype == np.float64 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_dp)


# ----------------------------------------------------------------------------
# seeded inputs
# ----------------------------------------------------------------------------
def uniform(shape, seed: int) -> np.ndarray:
    """fp32 uniform[-1, 1) from the counter-based splitmix64 stream `seed`."""
    out = np.empty(shape, dtype=np.float32)
    lib().orc_fill_uniform(_f(out), out.size, seed)
    return out


def uniform_numpy(n: int, seed: int) -> np.ndarray:
    """The same stream in pure numpy (an independent statement of the generator)."""
    with np.errstate(over="ignore"):
        i = np.arange(1, n + 1, dtype=np.uint64)
        z = np.uint64(seed) + i * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    bits = (z >> np.uint64(40)).astype(np.float32)
    return bits * np.float32(2.0 ** -23) - np.float32(1.0)


# ----------------------------------------------------------------------------
# planner
# ----------------------------------------------------------------------------
def init_block_dims(M, N, K, p, cx: Cntx, sch=NA, mcu=0, kcu=0, ncu=0) -> BlkDims:
    x = BlkDims()
    lib().orc_init_block_dims(M, N, K, p, C.byref(x), C.byref(cx), sch, mcu, kcu, ncu)
    return x


def derive_schedule(M, N, K, p, mc, cx: Cntx) -> int:
    return lib().orc_derive_schedule(M, N, K, p, mc, C.byref(cx))


def packed_A_size(M, K, p, x, cx, sch):
    return lib().orc_packed_A_size(M, K, p, C.byref(x), C.byref(cx), sch)


def packed_B_size(K, N, p, x, cx):
    return lib().orc_packed_B_size(K, N, p, C.byref(x), C.byref(cx))


def packed_C_size(M, N, p, x, cx, sch):
    return lib().orc_packed_C_size(M, N, p, C.byref(x), C.byref(cx), sch)


# ----------------------------------------------------------------------------
# packing
# ----------------------------------------------------------------------------
def pack_A(A, p, x, cx, sch) -> np.ndarray:
    M, K = A.shape
    out = np.full(packed_A_size(M, K, p, x, cx, sch) // 4, np.nan, dtype=np.float32)
    lib().orc_pack_A(_f(A), _f(out), M, K, p, C.byref(x), C.byref(cx), sch)
    return out


def pack_B(B, p, x, cx, sch) -> np.ndarray:
    K, N = B.shape
    out = np.full(packed_B_size(K, N, p, x, cx) // 4, np.nan, dtype=np.float32)
    lib().orc_pack_B(_f(B), _f(out), K, N, p, C.byref(x), C.byref(cx), sch)
    return out


def pack_C(Cm, p, x, cx, sch) -> np.ndarray:
    M, N = Cm.shape
    out = np.full(packed_C_size(M, N, p, x, cx, sch) // 4, np.nan, dtype=np.float32)
    lib().orc_pack_C(_f(Cm), _f(out), M, N, p, C.byref(x), C.byref(cx), sch)
    return out


def unpack_C(Cp, M, N, p, x, cx, sch, into=None) -> np.ndarray:
    out = np.zeros((M, N), dtype=np.float32) if into is None else into
    lib().orc_unpack_C(_f(out), _f(Cp), M, N, p, C.byref(x), C.byref(cx), sch)
    return out


def init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cx: Cntx) -> BlkDims:
    """Blocks of the reference's direct convolution (examples/cake_conv.cpp:262-425), K-first."""
    x = BlkDims()
    lib().orc_init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, C.byref(x), C.byref(cx))
    return x


def pack_filters(F, Cin, taps, p, x, cx) -> np.ndarray:
    """F[Cout][Cin*taps] in the layout of the reference's pack_filters (examples/cake_conv.cpp:536-610)."""
    Cout = F.shape[0]
    assert F.size == Cout * Cin * taps
    out = np.full(x.M_padded * Cin * taps, np.nan, dtype=np.float32)
    lib().orc_pack_filters(_f(np.ascontiguousarray(F.reshape(Cout, -1))), _f(out), Cout, Cin, taps, p, C.byref(x), C.byref(cx))
    return out


def ukernel(Ap, Bp, Ct, mr, nr, k):
    lib().orc_ukernel(_f(Ap), _f(Bp), _f(Ct), mr, nr, k)
    return Ct


# ----------------------------------------------------------------------------
# entry points
# ----------------------------------------------------------------------------
def cake_sgemm(A, B, p, cx=None, Cinit=None, beta=0.0, sch=NA, mcu=0, kcu=0, ncu=0,
               return_time=False):
    """C = A.B through the restated CAKE pipeline.  Returns C (and seconds, dims)."""
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    Cm = np.zeros((M, N), dtype=np.float32) if Cinit is None else np.ascontiguousarray(Cinit, dtype=np.float32).copy()
    x = BlkDims()
    cxp = C.byref(cx) if cx is not None else None
    t = lib().orc_cake_sgemm(_f(A), _f(B), _f(Cm), M, N, K, p, cxp, 0, 0, 1.0, beta, sch,
                             mcu, kcu, ncu, C.byref(x))
    if return_time:
        return Cm, t, x
    return Cm


def cake_sgemv(A_colmajor, x, p, cx=None, y0=None, M=None, K=None, return_time=False):
    """y (+)= A.x with A given column-major as a flat or (K, M) array."""
    if M is None:
        K, M = A_colmajor.shape
    y = np.zeros(M, dtype=np.float32) if y0 is None else np.ascontiguousarray(y0, dtype=np.float32).copy()
    cxp = C.byref(cx) if cx is not None else None
    t = lib().orc_cake_sgemv(_f(A_colmajor), _f(x), _f(y), M, K, p, cxp)
    return (y, t) if return_time else y


def im2col(inp, Hf, Wf, stride=1, pad=0) -> np.ndarray:
    """NCHW input -> [Cin*Hf*Wf, B*Hout*Wout]."""
    Bn, Cin, Hin, Win = inp.shape
    Hout = (Hin + 2 * pad - Hf) // stride + 1
    Wout = (Win + 2 * pad - Wf) // stride + 1
    out = np.empty((Cin * Hf * Wf, Bn * Hout * Wout), dtype=np.float32)
    lib().orc_im2col(_f(inp), _f(out), Bn, Cin, Hin, Win, Hf, Wf, Hout, Wout, stride, pad)
    return out


def im_2_col(inp_chw, Hf, Wf, Hout, Wout) -> np.ndarray:
    Cin, Hin, Win = inp_chw.shape
    out = np.empty((Cin * Hf * Wf, Hout * Wout), dtype=np.float32)
    lib().orc_im_2_col(_f(inp_chw), _f(out), Wf, Hf, Win, Hin, Wout, Hout, Cin)
    return out


# ----------------------------------------------------------------------------
# the linear layer of src/linear.cpp (caller of cake_sgemm; p = 10 there)
# ----------------------------------------------------------------------------
def linear_forward(x, w, bias=None, p=10, cx=None) -> np.ndarray:
    """src/linear.cpp:12-50: weight.t() made contiguous (K x N), cake_sgemm with
    default arguments, then the bias added to every row."""
    wt = np.ascontiguousarray(w.T)
    out = cake_sgemm(np.ascontiguousarray(x), wt, p, cx)
    if bias is not None:
        out = out + bias.astype(np.float32)[None, :]
    return out


def linear_backward(grad_y, x, w, bias=None, p=10, cx=None):
    """src/linear.cpp:53-102: grad_input = cake_sgemm(grad_output, weight),
    grad_weight = cake_sgemm(grad_output.t() contiguous, input), grad_bias =
    grad_output.sum(0).  The bias sum is returned in fp64 (torch's summation order
    is its own; callers compare within the bound any fp32 order meets)."""
    gx = cake_sgemm(np.ascontiguousarray(grad_y), np.ascontiguousarray(w), p, cx)
    gw = cake_sgemm(np.ascontiguousarray(grad_y.T), np.ascontiguousarray(x), p, cx)
    gb = None if bias is None else grad_y.astype(np.float64).sum(axis=0)
    return gx, gw, gb


# ----------------------------------------------------------------------------
# closed-form checkers
# ----------------------------------------------------------------------------
def gemm_f64(A, B):
    M, K = A.shape
    _, N = B.shape
    C64 = np.empty((M, N), dtype=np.float64)
    S = np.empty((M, N), dtype=np.float64)
    lib().orc_gemm_f64(_f(A), _f(B), M, N, K, _d(C64), _d(S))
    return C64, S


def max_rel_err(Cm, C64, S) -> float:
    Cm = np.ascontiguousarray(Cm, dtype=np.float32)
    return float(lib().orc_max_rel_err(_f(Cm), _d(C64), _d(S), Cm.size))


def gemv_f64(A, x, M, K, col_major):
    y = np.empty(M, dtype=np.float64)
    S = np.empty(M, dtype=np.float64)
    lib().orc_gemv_f64(_f(A), _f(x), M, K, int(col_major), _d(y), _d(S))
    return y, S


def conv_naive_f64(inp, wt, stride=1, pad=0):
    Bn, Cin, Hin, Win = inp.shape
    Cout, Cin2, Hf, Wf = wt.shape
    assert Cin == Cin2
    Hout = (Hin + 2 * pad - Hf) // stride + 1
    Wout = (Win + 2 * pad - Wf) // stride + 1
    out = np.empty((Bn, Cout, Hout, Wout), dtype=np.float64)
    S = np.empty_like(out)
    lib().orc_conv_naive_f64(_f(inp), _f(wt), _d(out), _d(S), Bn, Cin, Hin, Win, Cout, Hf, Wf,
                             Hout, Wout, stride, pad)
    return out, S


def physical_cores() -> int:
    return int(lib().orc_physical_cores())


def query_cntx() -> Cntx:
    cx = Cntx()
    lib().orc_query_cntx(C.byref(cx))
    return cx
