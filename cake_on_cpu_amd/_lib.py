"""ctypes binding of libcake_hip.so (the C-ABI declared in include/cake_hip.h).

The library is built in-tree by ``cake_on_cpu_amd/csrc/Makefile`` into
``cake_on_cpu_amd/lib/``.  Loading fails loudly when it is missing: there is no
fallback path."""
from __future__ import annotations

import ctypes as C
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libcake_hip.so"
CXX_LIB_PATH = LIB_DIR / "libcake.so"

KMN, MKN, NKM, NA = 0, 1, 2, 3
SCHED_NAMES = {KMN: "KMN", MKN: "MKN", NKM: "NKM", NA: "NA"}
# Plan.kernel: which kernel family cake_hip_sgemm runs for a shape
CONV_NONE, CONV_SHORTK_BATCH, CONV_PATCH, CONV_GATHER, CONV_TWO_STEP = range(5)   # cake_hip_last_conv_route
KERNEL_NAMES = {0: "macro-tile", 1: "matrix-vector", 2: "streaming, few rows", 3: "streaming, few columns",
                4: "short K, tiles walked by resident workgroups",
                5: "256 x 128 tiles walked by one resident workgroup per CU"}

OK, ERR_ARG, ERR_NO_DEVICE, ERR_HIP, ERR_ALLOC, ERR_RANGE, ERR_ARCH = range(7)

BLK_FIELDS = [
    "m_c", "k_c", "n_c", "m_c1", "k_c1", "n_c1",
    "m_c1_last_core", "n_c1_last_core", "k_c1_last_core",
    "mr_rem", "nr_rem", "k_rem", "p_l", "pm_l", "pn_l", "pm", "pn",
    "m_pad", "k_pad", "n_pad", "Mb", "Kb", "Nb", "M_padded", "N_padded", "sch",
]


class BlkDims(C.Structure):
    """cake_hip_blk_dims_t == blk_dims_t of the reference (include/common.h:108-135)."""
    _fields_ = [(n, C.c_int) for n in BLK_FIELDS]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n in BLK_FIELDS}


class CpuCntx(C.Structure):
    """cake_hip_cpu_cntx_t: the block-sizing inputs of cake_cntx_t (include/common.h:138-151)."""
    _fields_ = [("alpha_n", C.c_double), ("mr", C.c_int), ("nr", C.c_int),
                ("L1", C.c_int), ("L2", C.c_int), ("L3", C.c_int), ("ncores", C.c_int)]


class Plan(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("sched", "tile_m", "tile_n", "tile_k", "wave_m", "wave_n", "threads", "split_k",
                 "tail_tiles", "tail_split", "tiles_m", "tiles_n", "group", "grid", "lds_bytes", "vector_loads", "cus",
                 "kernel")] + \
               [("flops", C.c_double), ("min_bytes", C.c_double), ("model_bytes", C.c_double)]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


class DeviceInfo(C.Structure):
    _fields_ = [("device", C.c_int), ("cus", C.c_int), ("xcds", C.c_int),
                ("lds_bytes_per_cu", C.c_int), ("l2_bytes", C.c_int), ("wavefront", C.c_int),
                ("clock_khz", C.c_int), ("hbm_bytes", C.c_size_t), ("arch", C.c_char * 32)]


class CakeHipError(RuntimeError):
    def __init__(self, status: int, where: str, detail: str):
        self.status = status
        super().__init__(f"{where}: status {status} ({detail})")


_fp = C.c_void_p  # float* as an address: host numpy buffers and device pointers alike
_i = C.c_int
_dp = C.POINTER(C.c_double)
_bd = C.POINTER(BlkDims)
_cx = C.POINTER(CpuCntx)

# name -> (restype, argtypes); every symbol include/cake_hip.h declares
SIGNATURES = {
    "cake_hip_init": (_i, [_i]),
    "cake_hip_shutdown": (_i, []),
    "cake_hip_device_info": (_i, [C.POINTER(DeviceInfo)]),
    "cake_hip_strerror": (C.c_char_p, [_i]),
    "cake_hip_last_error": (C.c_char_p, []),
    "cake_hip_malloc": (_i, [C.POINTER(C.c_void_p), C.c_size_t]),
    "cake_hip_free": (_i, [C.c_void_p]),
    "cake_hip_memcpy_h2d": (_i, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "cake_hip_memcpy_d2h": (_i, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "cake_hip_memset": (_i, [C.c_void_p, _i, C.c_size_t]),
    "cake_hip_synchronize": (_i, []),
    "cake_hip_plan": (_i, [_i, _i, _i, _i, C.POINTER(_i), C.POINTER(Plan)]),
    "cake_hip_init_block_dims": (_i, [_i, _i, _i, _i, _cx, _i, _i, _i, _i, _bd]),
    "cake_hip_derive_schedule": (_i, [_i, _i, _i, _i, _i, _cx]),
    "cake_hip_grid_dims_2d": (_i, [_i] * 5),
    "cake_hip_init_block_dims_2d": (_i, [_i, _i, _i, _i, _cx, _i, C.c_float, _i, _i, _i, _bd]),
    "cake_hip_init_block_dims_2d_small": (_i, [_i, _i, _i, _i, _cx, _i, C.c_float, _bd]),
    "cake_hip_init_block_dims_conv": (_i, [_i] * 10 + [_cx, _bd]),
    "cake_hip_packed_filters_size": (C.c_size_t, [_i, _i, _i, _i, _bd, _cx]),
    "cake_hip_pack_filters": (_i, [_fp, _fp, _i, _i, _i, _i, _bd, _cx, C.c_void_p, _dp]),
    "cake_hip_sconv_packed": (_i, [_fp, _fp, _fp] + [_i] * 10 + [_bd, _cx, C.c_void_p, _dp]),
    "cake_hip_sgemm": (_i, [_fp, _fp, _fp, _i, _i, _i, _i, _i, C.POINTER(_i), C.c_void_p, _dp]),
    "cake_hip_sgemm_noalloc": (_i, [_fp, _fp, _fp, _i, _i, _i, _i, _i, C.c_void_p]),
    "cake_hip_sgemm_packed": (_i, [_fp, _fp, _fp, _i, _i, _i, _i, _bd, _cx, _i, _i, _i, C.c_void_p, _dp]),
    "cake_hip_packed_a_size": (C.c_size_t, [_i, _i, _i, _bd, _cx, _i]),
    "cake_hip_packed_b_size": (C.c_size_t, [_i, _i, _i, _bd, _cx]),
    "cake_hip_packed_c_size": (C.c_size_t, [_i, _i, _i, _bd, _cx, _i]),
    "cake_hip_pack_a": (_i, [_fp, _fp, _i, _i, _i, _bd, _cx, _i, C.c_void_p, _dp]),
    "cake_hip_pack_b": (_i, [_fp, _fp, _i, _i, _i, _bd, _cx, _i, C.c_void_p, _dp]),
    "cake_hip_pack_c": (_i, [_fp, _fp, _i, _i, _i, _bd, _cx, _i, C.c_void_p, _dp]),
    "cake_hip_unpack_c": (_i, [_fp, _fp, _i, _i, _i, _bd, _cx, _i, C.c_void_p, _dp]),
    "cake_hip_packed_offset": (C.c_int64, [_i, _i, _i, _i, _i, _i, _i, _bd, _cx, _i]),
    "cake_hip_sgemv": (_i, [_fp, _fp, _fp, _i, _i, _i, _i, C.c_void_p, _dp]),
    "cake_hip_im2col": (_i, [_fp, _fp, _i, _i, _i, _i, _i, _i, _i, _i, C.c_void_p, _dp]),
    "cake_hip_conv2d_workspace": (C.c_size_t, [_i] * 9),
    "cake_hip_conv2d": (_i, [_fp, _fp, _fp] + [_i] * 10 + [C.c_void_p, C.c_void_p, _dp]),
    "cake_hip_conv2d_im2col": (_i, [_fp, _fp, _fp] + [_i] * 10 + [C.c_void_p, C.c_void_p, _dp]),
    "cake_hip_sconv": (_i, [_fp, _fp, _fp] + [_i] * 9 + [C.c_void_p, _dp]),
    "cake_hip_transpose": (_i, [_fp, _fp, _i, _i, C.c_void_p, _dp]),
    "cake_hip_linear_forward": (_i, [_fp, _fp, _fp, _fp, _i, _i, _i, C.c_void_p, _dp]),
    "cake_hip_linear_forward_wt": (_i, [_fp, _fp, _fp, _fp, _i, _i, _i, C.c_void_p, _dp]),
    "cake_hip_sgemm_nt": (_i, [_fp, _fp, _fp, _i, _i, _i, _i, C.POINTER(_i), C.c_void_p, _dp]),
    "cake_hip_linear_backward": (_i, [_fp] * 6 + [_i, _i, _i, C.c_void_p, _dp]),
    "cake_hip_autotune": (_i, [_i, _i, _i, C.c_double, C.POINTER(Plan), _dp, _dp]),
    "cake_hip_tune_save": (_i, [C.c_char_p]),
    "cake_hip_tune_load": (_i, [C.c_char_p, C.POINTER(_i)]),
    "cake_hip_tune_clear": (_i, []),
    "cake_hip_tune_count": (_i, []),
    "cake_hip_fill_uniform": (_i, [_fp, C.c_size_t, C.c_uint64, C.c_void_p]),
    "cake_hip_last_conv_route": (_i, []),
    "cake_hip_ctx_create": (_i, [C.POINTER(C.c_void_p)]),
    "cake_hip_ctx_destroy": (_i, [C.c_void_p]),
    "cake_hip_ctx_set_current": (_i, [C.c_void_p]),
    "cake_hip_ctx_get_current": (C.c_void_p, []),
    "cake_hip_ctx_stream": (C.c_void_p, [C.c_void_p]),
    "cake_hip_last_kernel_seconds": (_i, [C.POINTER(C.c_double * 5)]),
}

_lib = None


def _share_torch_hip_runtime() -> None:
    """A process can hold one HIP runtime.  PyTorch-ROCm wheels bundle their own
    libamdhip64.so (soname libamdhip64.so.7) and look it up by file name, so if
    the system copy is already loaded under its soname torch loads a second
    runtime, which then finds no GPU.  When such a wheel is installed, load its
    copy first: libcake_hip.so's libamdhip64.so.7 dependency then resolves to it
    whichever of the two packages is used first.  torch itself is not imported."""
    import importlib.util
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        return
    if spec is None or not spec.origin:
        return
    bundled = Path(spec.origin).parent / "lib" / "libamdhip64.so"
    if bundled.exists():
        try:
            C.CDLL(str(bundled), mode=C.RTLD_GLOBAL)
        except OSError:
            pass  # fall back to the system runtime


def load() -> C.CDLL:
    """dlopen libcake_hip.so and type every entry point.  No GPU is touched."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C cake_on_cpu_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback")
        _share_torch_hip_runtime()
        lib = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(status: int, where: str) -> None:
    if status != OK:
        lib = load()
        detail = lib.cake_hip_last_error().decode() or lib.cake_hip_strerror(status).decode()
        raise CakeHipError(status, where, detail)
