"""Host-side mirror of the reference's operator interface for the fp32 GEMM path.

Names, argument order and meaning follow include/cake.h, include/tiling.h,
include/packing.h, examples/cake_gemv.cpp and examples/cake_conv.cpp of
vnatesh/CAKE_on_CPU, so code (and tests) written against the reference read the
same here.  Matrices are float32, C-contiguous numpy arrays (host memory, staged
by the library) or torch ROCm tensors (used in place through their device
pointer, on torch's current stream)."""
from __future__ import annotations

import ctypes as C
import os
import re
import subprocess

import numpy as np

from . import _lib
from ._lib import KMN, MKN, NKM, NA, BlkDims, CpuCntx, DeviceInfo, Plan, check, load


# ----------------------------------------------------------------------------
# array plumbing
# ----------------------------------------------------------------------------
def _is_torch(a) -> bool:
    return hasattr(a, "data_ptr") and hasattr(a, "is_contiguous")


def _ptr(a, what: str) -> int:
    if a is None:
        raise ValueError(f"{what} is None")
    if _is_torch(a):
        import torch
        if a.dtype != torch.float32 or not a.is_contiguous():
            raise TypeError(f"{what} must be a contiguous float32 tensor")
        return a.data_ptr()
    if not isinstance(a, np.ndarray) or a.dtype != np.float32 or not a.flags["C_CONTIGUOUS"]:
        raise TypeError(f"{what} must be a C-contiguous float32 numpy array or torch tensor")
    return a.ctypes.data


def _stream(*arrays) -> int:
    """torch's current HIP stream when any operand lives on the GPU, else the default stream."""
    for a in arrays:
        if _is_torch(a) and a.is_cuda:
            import torch
            return torch.cuda.current_stream(a.device).cuda_stream
    return 0


def _numel(a) -> int:
    return a.numel() if _is_torch(a) else a.size


def _empty_like_kind(ref, shape):
    if _is_torch(ref):
        import torch
        return torch.empty(shape, dtype=torch.float32, device=ref.device)
    return np.empty(shape, dtype=np.float32)


def _need(a, n: int, what: str):
    if _numel(a) < n:
        raise ValueError(f"{what} holds {_numel(a)} elements, {n} needed")


# ----------------------------------------------------------------------------
# machine description and block sizing (include/tiling.h:15-41)
# ----------------------------------------------------------------------------
def _lscpu_cache(level: int) -> int:
    try:
        col = "ONE-SIZE" if level < 3 else "ALL-SIZE"
        out = subprocess.run(["lscpu", f"--caches=NAME,{col}"], capture_output=True, text=True, timeout=10).stdout
        for line in out.splitlines():
            if line.strip().startswith(f"L{level}"):
                m = re.search(r"(\d+)([KMG])", line)
                if m:
                    return int(m.group(1)) << {"K": 10, "M": 20, "G": 30}[m.group(2)]
    except Exception:
        pass
    return 0


def _physical_cores() -> int:
    logical = os.cpu_count() or 1
    try:
        out = subprocess.run(["lscpu"], capture_output=True, text=True, timeout=10).stdout
        tpc = int(re.search(r"Thread\(s\) per core:\s*(\d+)", out).group(1))
        sockets = int(re.search(r"Socket\(s\):\s*(\d+)", out).group(1))
        return max(1, logical // (tpc * sockets))
    except Exception:
        return logical


def cake_query_cntx() -> CpuCntx:
    """cake_query_cntx (src/block_sizing.cpp:40-75): host cache sizes and physical core
    count, m_r x n_r = 6 x 16.  On the GPU these only shape the reference-compatible
    blk_dims_t / packed layouts; the kernels are planned from the device instead."""
    cx = CpuCntx()
    cx.alpha_n = 1.0
    cx.mr, cx.nr = 6, 16
    cx.L1 = _lscpu_cache(1) or (32 << 10)
    cx.L2 = _lscpu_cache(2) or (1 << 20)
    cx.L3 = _lscpu_cache(3) or (32 << 20)
    cx.ncores = _physical_cores()
    return cx


_DEFAULT_CNTX = None


def _default_cntx() -> CpuCntx:
    """What a NULL cake_cntx stands for (src/cake_sgemm.cpp:14-16): the host's own description,
    queried once per process here instead of on every call."""
    global _DEFAULT_CNTX
    if _DEFAULT_CNTX is None:
        _DEFAULT_CNTX = cake_query_cntx()
    cx = CpuCntx()
    C.memmove(C.byref(cx), C.byref(_DEFAULT_CNTX), C.sizeof(CpuCntx))
    return cx


def update_mr_nr(cake_cntx: CpuCntx, m_r: int, n_r: int) -> None:
    """update_mr_nr (src/block_sizing.cpp:78-83)."""
    cake_cntx.mr, cake_cntx.nr = m_r, n_r


def init_block_dims(M, N, K, p, cake_cntx: CpuCntx, sch=NA, argv=None, type_size=4,
                    mcu=0, kcu=0, ncu=0, x: BlkDims | None = None) -> BlkDims:
    """init_block_dims (src/block_sizing.cpp:465-595).  Returns (and fills) blk_dims_t."""
    x = BlkDims() if x is None else x
    check(load().cake_hip_init_block_dims(M, N, K, p, C.byref(cake_cntx), sch, mcu, kcu, ncu, C.byref(x)),
          "init_block_dims")
    return x


def grid_dims_2d(M, N, K, p, ncores=0) -> int:
    """pn of the reference's pm x pn grid of cores (src/block_sizing.cpp:596-634): the factor of p
    closest to sqrt(p N / M).  Host arithmetic."""
    return load().cake_hip_grid_dims_2d(M, N, K, p, ncores)


def init_block_dims_2d(M, N, K, p, cake_cntx: CpuCntx, sch=NA, argv=None, type_size=4,
                       mcu=0, kcu=0, ncu=0) -> BlkDims:
    """init_block_dims_2d (include/tiling.h:43-45, src/block_sizing.cpp:639-779)."""
    x = BlkDims()
    check(load().cake_hip_init_block_dims_2d(M, N, K, p, C.byref(cake_cntx), sch, float(type_size), mcu, kcu, ncu,
                                             C.byref(x)), "init_block_dims_2d")
    return x


def init_block_dims_2d_small(M, N, K, p, cake_cntx: CpuCntx, sch=NA, argv=None, type_size=4) -> BlkDims:
    """init_block_dims_2d_small (include/tiling.h:47-49, src/block_sizing.cpp:785-841)."""
    x = BlkDims()
    check(load().cake_hip_init_block_dims_2d_small(M, N, K, p, C.byref(cake_cntx), sch, float(type_size), C.byref(x)),
          "init_block_dims_2d_small")
    return x


def init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cake_cntx: CpuCntx, sch=KMN,
                         argv=None, density=0.0, type_size=4) -> BlkDims:
    """init_block_dims_conv (examples/cake_conv.cpp:333-425): blocks of the direct convolution, K-first."""
    x = BlkDims()
    check(load().cake_hip_init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, C.byref(cake_cntx),
                                               C.byref(x)), "init_block_dims_conv")
    return x


def plan(M, N, K, sch=NA, tile=None) -> Plan:
    """The GPU planner's decision for one product (tile, wave layout, reuse order, split-K)."""
    out = Plan()
    ov = (C.c_int * 4)(*tile) if tile is not None else None
    check(load().cake_hip_plan(M, N, K, sch, ov, C.byref(out)), "plan")
    return out


def _tile_override(M, N, K, sch, mcu, kcu, ncu):
    """mcu,kcu,ncu ask for a block of m x k x n; honoured when a macro-tile of that shape exists."""
    if not (mcu and kcu and ncu):
        return None
    ov = (C.c_int * 4)(mcu, ncu, kcu, 0)
    if load().cake_hip_plan(M, N, K, sch, ov, C.byref(Plan())) != _lib.OK:
        return None
    return ov


# ----------------------------------------------------------------------------
# cake_sgemm (include/cake.h:12-14)
# ----------------------------------------------------------------------------
def cake_sgemm(A, B, Cm, M, N, K, p, cake_cntx: CpuCntx | None = None, argv=None,
               packedA=False, packedB=False, alpha=1.0, beta=0.0, sch=NA,
               mcu=0, kcu=0, ncu=0) -> float:
    """C = A.B in place, returns seconds (device time of the kernels).

    Semantics follow src/cake_sgemm.cpp:9-175: alpha is ignored; K-first assigns
    C; for M-/N-first beta != 0 means "start from the existing C".  With
    packedA/packedB the operand is a buffer written by pack_A/pack_B for the same
    (M,N,K,p,cake_cntx,sch)."""
    lib = load()
    _need(Cm, M * N, "C")
    secs = C.c_double(0.0)
    stream = _stream(A, B, Cm)
    if packedA or packedB:
        cx = cake_cntx if cake_cntx is not None else _default_cntx()
        x = init_block_dims(M, N, K, p, cx, sch, argv, 4, mcu, kcu, ncu)
        accumulate = int(x.sch != KMN and beta != 0)
        check(lib.cake_hip_sgemm_packed(_ptr(A, "A"), _ptr(B, "B"), _ptr(Cm, "C"), M, N, K, p,
                                        C.byref(x), C.byref(cx), int(packedA), int(packedB),
                                        accumulate, stream, C.byref(secs)), "cake_sgemm")
        return secs.value
    _need(A, M * K, "A")
    _need(B, K * N, "B")
    # beta != 0 means "start from C" only under the schedule the reference resolves from the
    # caller's cntx and p (src/cake_sgemm.cpp:34-35,114); the GPU's tile order stays the planner's.
    resolved = sch
    if M > 0 and N > 0 and K > 0:
        cx = cake_cntx if cake_cntx is not None else _default_cntx()
        resolved = init_block_dims(M, N, K, p, cx, sch, argv, 4, mcu, kcu, ncu).sch
    elif sch == NA:
        resolved = KMN
    accumulate = int(resolved != KMN and beta != 0)
    ov = _tile_override(M, N, K, sch, mcu, kcu, ncu)
    check(lib.cake_hip_sgemm(_ptr(A, "A"), _ptr(B, "B"), _ptr(Cm, "C"), M, N, K, sch, accumulate, ov,
                             stream, C.byref(secs)), "cake_sgemm")
    return secs.value


# ----------------------------------------------------------------------------
# packing (include/packing.h:6-13,70-72)
# ----------------------------------------------------------------------------
def cake_sgemm_packed_A_size(M, K, p, x, cake_cntx, sch) -> int:
    return load().cake_hip_packed_a_size(M, K, p, C.byref(x), C.byref(cake_cntx), sch)


def cake_sgemm_packed_B_size(K, N, p, x, cake_cntx) -> int:
    return load().cake_hip_packed_b_size(K, N, p, C.byref(x), C.byref(cake_cntx))


def cake_sgemm_packed_C_size(M, N, p, x, cake_cntx, sch) -> int:
    return load().cake_hip_packed_c_size(M, N, p, C.byref(x), C.byref(cake_cntx), sch)


def pack_A(A, A_p, M, K, p, x, cake_cntx, sch) -> float:
    _need(A, M * K, "A")
    _need(A_p, cake_sgemm_packed_A_size(M, K, p, x, cake_cntx, sch) // 4, "A_p")
    secs = C.c_double(0.0)
    check(load().cake_hip_pack_a(_ptr(A, "A"), _ptr(A_p, "A_p"), M, K, p, C.byref(x), C.byref(cake_cntx),
                                 sch, _stream(A, A_p), C.byref(secs)), "pack_A")
    return secs.value


def pack_B(B, B_p, K, N, p, x, cake_cntx, sch) -> float:
    _need(B, K * N, "B")
    _need(B_p, cake_sgemm_packed_B_size(K, N, p, x, cake_cntx) // 4, "B_p")
    secs = C.c_double(0.0)
    check(load().cake_hip_pack_b(_ptr(B, "B"), _ptr(B_p, "B_p"), K, N, p, C.byref(x), C.byref(cake_cntx),
                                 sch, _stream(B, B_p), C.byref(secs)), "pack_B")
    return secs.value


def pack_C(Cm, C_p, M, N, p, x, cake_cntx, sch) -> float:
    _need(Cm, M * N, "C")
    _need(C_p, cake_sgemm_packed_C_size(M, N, p, x, cake_cntx, sch) // 4, "C_p")
    secs = C.c_double(0.0)
    check(load().cake_hip_pack_c(_ptr(Cm, "C"), _ptr(C_p, "C_p"), M, N, p, C.byref(x), C.byref(cake_cntx),
                                 sch, _stream(Cm, C_p), C.byref(secs)), "pack_C")
    return secs.value


def unpack_C(Cm, C_p, M, N, p, x, cake_cntx, sch) -> float:
    _need(Cm, M * N, "C")
    _need(C_p, cake_sgemm_packed_C_size(M, N, p, x, cake_cntx, sch) // 4, "C_p")
    secs = C.c_double(0.0)
    check(load().cake_hip_unpack_c(_ptr(Cm, "C"), _ptr(C_p, "C_p"), M, N, p, C.byref(x), C.byref(cake_cntx),
                                   sch, _stream(Cm, C_p), C.byref(secs)), "unpack_C")
    return secs.value


def packed_offset(which, row, col, M, N, K, p, x, cake_cntx, sch) -> int:
    """Host evaluation of the packed index map (which: 0 A, 1 B, 2 C); -1 when out of range."""
    return load().cake_hip_packed_offset(which, row, col, M, N, K, p, C.byref(x), C.byref(cake_cntx), sch)


# ----------------------------------------------------------------------------
# cake_sgemv (examples/cake_gemv.cpp:7-9)
# ----------------------------------------------------------------------------
def cake_sgemv(A, B, Cv, M, K, p, cake_cntx=None, argv=None, packedA=False, alpha=1.0, beta=0.0,
               sch=NA, *, row_major=False, accumulate=True) -> float:
    """y += A.x with A column-major (A[k*M + m]), as examples/cake_gemv.cpp:716-767 does.
    row_major=True reads A[m*K + k]; accumulate=False overwrites y.  Returns seconds."""
    _need(A, M * K, "A")
    _need(B, K, "x")
    _need(Cv, M, "y")
    secs = C.c_double(0.0)
    check(load().cake_hip_sgemv(_ptr(A, "A"), _ptr(B, "x"), _ptr(Cv, "y"), M, K, int(not row_major),
                                int(accumulate), _stream(A, B, Cv), C.byref(secs)), "cake_sgemv")
    return secs.value


# ----------------------------------------------------------------------------
# convolution through im2col (examples/cake_conv.cpp:24-25,1007-1066)
# ----------------------------------------------------------------------------
def im2col(inp, cols, batch, Cin, Hin, Win, Hf, Wf, stride=1, pad=0) -> float:
    Hout = (Hin + 2 * pad - Hf) // stride + 1
    Wout = (Win + 2 * pad - Wf) // stride + 1
    _need(inp, batch * Cin * Hin * Win, "input")
    _need(cols, Cin * Hf * Wf * batch * Hout * Wout, "cols")
    secs = C.c_double(0.0)
    check(load().cake_hip_im2col(_ptr(inp, "input"), _ptr(cols, "cols"), batch, Cin, Hin, Win, Hf, Wf,
                                 stride, pad, _stream(inp, cols), C.byref(secs)), "im2col")
    return secs.value


def im_2_col(In, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout=0, s=1):
    """im_2_col (examples/cake_conv.cpp:1178-1213): one CHW image, no padding; the
    stride argument is accepted and unused, as in the reference.  Returns the new
    [Cin*Hf*Wf, Hout*Wout] matrix."""
    if Hout != Hin - Hf + 1 or Wout != Win - Wf + 1:
        raise ValueError("im_2_col needs Hout = Hin - Hf + 1 and Wout = Win - Wf + 1")
    cols = _empty_like_kind(In, (Cin * Hf * Wf, Hout * Wout))
    im2col(In, cols, 1, Cin, Hin, Win, Hf, Wf, 1, 0)
    return cols


def conv2d(inp, weights, out, batch, Cin, Hin, Win, Cout, Hf, Wf, stride=1, pad=0,
           out_nchw=False, workspace=None, explicit_im2col=False) -> float:
    """weights[Cout x Cin*Hf*Wf] . im2col(inp): the im2col path of
    examples/cake_conv.cpp:1007-1066.  out is [Cout][batch*Hout*Wout] or NCHW.
    By default the column matrix is gathered inside the GEMM when the geometry
    allows; explicit_im2col=True always materialises it first, as the reference does."""
    Hout = (Hin + 2 * pad - Hf) // stride + 1
    Wout = (Win + 2 * pad - Wf) // stride + 1
    _need(inp, batch * Cin * Hin * Win, "input")
    _need(weights, Cout * Cin * Hf * Wf, "weights")
    _need(out, Cout * batch * Hout * Wout, "out")
    ws = 0
    if workspace is not None:
        need = load().cake_hip_conv2d_workspace(batch, Cin, Hin, Win, Cout, Hf, Wf, stride, pad)
        _need(workspace, (need + 3) // 4, "workspace")
        ws = _ptr(workspace, "workspace")
    secs = C.c_double(0.0)
    fn = load().cake_hip_conv2d_im2col if explicit_im2col else load().cake_hip_conv2d
    check(fn(_ptr(inp, "input"), _ptr(weights, "weights"), _ptr(out, "out"),
                                 batch, Cin, Hin, Win, Cout, Hf, Wf, stride, pad, int(out_nchw), ws,
                                 _stream(inp, weights, out), C.byref(secs)), "conv2d")
    return secs.value


def pack_filters(A, A_p, M, K, p, x, cake_cntx, taps=9) -> float:
    """pack_filters (examples/cake_conv.cpp:536-610): filters A[M = Cout][K = Cin * taps] into the K-first
    blocks of init_block_dims_conv; A_p holds x.M_padded * K floats.  The reference is written for
    3 x 3 filters (taps = 9)."""
    _need(A, M * K, "filters")
    _need(A_p, x.M_padded * K, "packed filters")
    secs = C.c_double(0.0)
    check(load().cake_hip_pack_filters(_ptr(A, "filters"), _ptr(A_p, "packed filters"), M, K // taps, taps, p,
                                       C.byref(x), C.byref(cake_cntx), _stream(A, A_p), C.byref(secs)), "pack_filters")
    return secs.value


def cake_sconv(A, B, Cm, Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cake_cntx=None, argv=None,
               packedA=False, sch=NA) -> float:
    """cake_sconv (examples/cake_conv.cpp:5-8,765-848): C[Cout][Hout][Wout] += A[Cout][Cin][Hf][Wf] * B[Cin][Hin][Win],
    one CHW image, no padding; sch is accepted and unused (the reference always runs it K-first).
    With packedA the filters are in the layout of pack_filters for the blocks that
    init_block_dims_conv derives from the same geometry, p and cake_cntx (:791-799).  Returns seconds."""
    _need(B, Cin * Hin * Win, "input")
    _need(Cm, Cout * Hout * Wout, "output")
    secs = C.c_double(0.0)
    if packedA:
        cx = cake_cntx if cake_cntx is not None else _default_cntx()
        x = init_block_dims_conv(Wf, Hf, Win, Hin, Wout, Hout, Cin, Cout, s, p, cx)
        _need(A, x.M_padded * Cin * Hf * Wf, "packed filters")
        check(load().cake_hip_sconv_packed(_ptr(A, "filters"), _ptr(B, "input"), _ptr(Cm, "output"), Wf, Hf, Win, Hin,
                                           Wout, Hout, Cin, Cout, s, p, C.byref(x), C.byref(cx), _stream(A, B, Cm),
                                           C.byref(secs)), "cake_sconv")
        return secs.value
    _need(A, Cout * Cin * Hf * Wf, "filters")
    check(load().cake_hip_sconv(_ptr(A, "filters"), _ptr(B, "input"), _ptr(Cm, "output"), Wf, Hf, Win, Hin, Wout, Hout,
                                Cin, Cout, s, _stream(A, B, Cm), C.byref(secs)), "cake_sconv")
    return secs.value


def last_conv_route() -> int:
    """Which route this thread's last convolution call took (_lib.CONV_*)."""
    return load().cake_hip_last_conv_route()


# ----------------------------------------------------------------------------
# device contexts
# ----------------------------------------------------------------------------
class Context:
    """A device context of its own (cake_hip_ctx_create): workspaces, events and a stream that calls
    made while it is current do not share with the default context or with other contexts.

        with cake.Context() as ctx:          # current on this thread inside the block
            cake.cake_sgemm(...)             # device operands: enqueued on ctx.stream unless torch's
                                             # current stream is passed by the operands
    """

    def __init__(self):
        h = C.c_void_p()
        check(load().cake_hip_ctx_create(C.byref(h)), "cake_hip_ctx_create")
        self.handle = h.value
        self._before = []

    @property
    def stream(self) -> int:
        return load().cake_hip_ctx_stream(self.handle) or 0

    def make_current(self) -> None:
        check(load().cake_hip_ctx_set_current(self.handle), "cake_hip_ctx_set_current")

    def __enter__(self):
        self._before.append(load().cake_hip_ctx_get_current())
        self.make_current()
        return self

    def __exit__(self, *exc):
        check(load().cake_hip_ctx_set_current(self._before.pop()), "cake_hip_ctx_set_current")
        return False

    def destroy(self) -> None:
        if self.handle:
            check(load().cake_hip_ctx_destroy(self.handle), "cake_hip_ctx_destroy")
            self.handle = None


def transpose_mat(A_old, At, K, N, Kt=0, Nt=0) -> float:
    """At[n][k] = A_old[k][n] for a K x N matrix (src/transpose.cpp:5-29; the
    blocking arguments Kt, Nt are accepted and unused).  Returns seconds."""
    _need(A_old, K * N, "A_old")
    _need(At, K * N, "At")
    secs = C.c_double(0.0)
    check(load().cake_hip_transpose(_ptr(A_old, "A_old"), _ptr(At, "At"), K, N, _stream(A_old, At),
                                    C.byref(secs)), "transpose_mat")
    return secs.value


def _opt_ptr(a, what):
    return None if a is None else _ptr(a, what)


def linear_forward(x, w, bias, y, M, N, K, timed=True) -> float:
    """y[M][N] = x[M][K] . w[N][K]^T + bias[N] (bias may be None): linear_forward of
    src/linear.cpp:12-50.  Returns seconds; timed=False skips the event timing, which makes
    the call asynchronous on device operands (it then returns 0)."""
    _need(x, M * K, "x")
    _need(w, N * K, "w")
    _need(y, M * N, "y")
    if bias is not None:
        _need(bias, N, "bias")
    secs = C.c_double(0.0)
    check(load().cake_hip_linear_forward(_ptr(x, "x"), _ptr(w, "w"), _opt_ptr(bias, "bias"), _ptr(y, "y"),
                                         M, N, K, _stream(x, w, y), C.byref(secs) if timed else None), "linear_forward")
    return secs.value


def sgemm_nt(A, Bt, Cm, M, N, K, accumulate=False, tile=None, timed=True) -> float:
    """C[M][N] = (C if accumulate else 0) + A[M][K] . Bt[N][K]^T with Bt read as it lies (the
    product of linear_forward, src/linear.cpp:38, without its transposed copy and bias).
    tile = (tile_m, tile_n, tile_k, split_k) forces the macro-tile kernel.  Returns seconds."""
    _need(A, M * K, "A")
    _need(Bt, N * K, "Bt")
    _need(Cm, M * N, "C")
    secs = C.c_double(0.0)
    ov = (C.c_int * 4)(*tile) if tile is not None else None
    check(load().cake_hip_sgemm_nt(_ptr(A, "A"), _ptr(Bt, "Bt"), _ptr(Cm, "C"), M, N, K, int(accumulate), ov,
                                   _stream(A, Bt, Cm), C.byref(secs) if timed else None), "sgemm_nt")
    return secs.value


def linear_forward_wt(x, wt, bias, y, M, N, K, timed=True) -> float:
    """The same with the weights already transposed: wt is [K][N] (transpose_mat of w), for callers
    that keep the transposed copy while the weights stay the same."""
    _need(x, M * K, "x")
    _need(wt, N * K, "wt")
    _need(y, M * N, "y")
    if bias is not None:
        _need(bias, N, "bias")
    secs = C.c_double(0.0)
    check(load().cake_hip_linear_forward_wt(_ptr(x, "x"), _ptr(wt, "wt"), _opt_ptr(bias, "bias"), _ptr(y, "y"),
                                            M, N, K, _stream(x, wt, y), C.byref(secs) if timed else None), "linear_forward_wt")
    return secs.value


def linear_backward(grad_y, x, w, grad_x, grad_w, grad_bias, M, N, K, timed=True) -> float:
    """grad_x = grad_y . w, grad_w = grad_y^T . x, grad_bias = column sums of grad_y
    (src/linear.cpp:53-102).  Outputs passed as None are skipped.  Returns seconds (0 with timed=False)."""
    _need(grad_y, M * N, "grad_y")
    for a, n, what in ((x, M * K, "x"), (w, N * K, "w"), (grad_x, M * K, "grad_x"),
                       (grad_w, N * K, "grad_w"), (grad_bias, N, "grad_bias")):
        if a is not None:
            _need(a, n, what)
    secs = C.c_double(0.0)
    check(load().cake_hip_linear_backward(_ptr(grad_y, "grad_y"), _opt_ptr(x, "x"), _opt_ptr(w, "w"),
                                          _opt_ptr(grad_x, "grad_x"), _opt_ptr(grad_w, "grad_w"),
                                          _opt_ptr(grad_bias, "grad_bias"), M, N, K,
                                          _stream(grad_y, x, w), C.byref(secs) if timed else None), "linear_backward")
    return secs.value


# ----------------------------------------------------------------------------
# autotuner (successor of mcu,kcu,ncu + src/autotune_sa.cpp)
# ----------------------------------------------------------------------------
def autotune(M, N, K, budget_seconds=2.0):
    """Measure the macro-tile / split-K candidates for an M x N x K product and keep the
    fastest for later calls.  Returns (plan, best_seconds, default_seconds)."""
    out = Plan()
    best, base = C.c_double(0.0), C.c_double(0.0)
    check(load().cake_hip_autotune(M, N, K, float(budget_seconds), C.byref(out), C.byref(best), C.byref(base)),
          "autotune")
    return out, best.value, base.value


def tune_save(path) -> None:
    check(load().cake_hip_tune_save(os.fsencode(path)), "tune_save")


def tune_load(path) -> int:
    n = C.c_int(0)
    check(load().cake_hip_tune_load(os.fsencode(path), C.byref(n)), "tune_load")
    return n.value


def tune_clear() -> None:
    check(load().cake_hip_tune_clear(), "tune_clear")


def tune_count() -> int:
    return load().cake_hip_tune_count()


# ----------------------------------------------------------------------------
# utilities
# ----------------------------------------------------------------------------
def fill_uniform(dst, seed: int) -> None:
    """dst[i] = uniform[-1,1) value i of stream `seed` (replaces rand_init, src/util.cpp:259-267)."""
    check(load().cake_hip_fill_uniform(_ptr(dst, "dst"), _numel(dst), seed, _stream(dst)), "fill_uniform")


def device_info() -> DeviceInfo:
    info = DeviceInfo()
    check(load().cake_hip_device_info(C.byref(info)), "device_info")
    return info


def last_kernel_seconds() -> dict:
    arr = (C.c_double * 5)()
    check(load().cake_hip_last_kernel_seconds(C.byref(arr)), "last_kernel_seconds")
    return dict(zip(("gemm", "splitk_reduce", "gemv", "im2col", "pack"), arr))
