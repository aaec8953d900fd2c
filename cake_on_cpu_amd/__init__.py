"""MI355X-native implementation of CAKE's fp32 GEMM hot path.

Host-side mirror of the reference's interface for this path (cake_sgemm,
cake_sgemv, init_block_dims, pack_A/pack_B/unpack_C, im_2_col, the linear layer) over the
C-ABI of libcake_hip.so.  PyTorch is not required; torch ROCm tensors and numpy
arrays are both accepted wherever a matrix is."""
from ._lib import (CONV_GATHER, CONV_NONE, CONV_PATCH, CONV_SHORTK_BATCH, CONV_TWO_STEP, KMN, MKN, NKM, NA, SCHED_NAMES, KERNEL_NAMES, BlkDims, CakeHipError, CpuCntx, DeviceInfo,
                   Plan, load)
from .api import (Context, autotune, cake_query_cntx, cake_sgemm, cake_sgemm_packed_A_size, cake_sgemm_packed_B_size,
                  cake_sgemm_packed_C_size, cake_sconv, cake_sgemv, conv2d, device_info, fill_uniform, im2col,
                  im_2_col, init_block_dims, init_block_dims_2d, init_block_dims_2d_small, init_block_dims_conv, grid_dims_2d,
                  last_conv_route, last_kernel_seconds, pack_filters, linear_backward, linear_forward, linear_forward_wt, sgemm_nt, pack_A, pack_B, pack_C,
                  packed_offset, plan, transpose_mat, tune_clear, tune_count, tune_load, tune_save, unpack_C,
                  update_mr_nr)

__all__ = [
    "KMN", "MKN", "NKM", "NA", "SCHED_NAMES", "KERNEL_NAMES", "BlkDims", "CpuCntx", "Plan", "DeviceInfo",
    "CakeHipError", "load", "cake_query_cntx", "update_mr_nr", "init_block_dims", "plan",
    "cake_sgemm", "cake_sgemv", "cake_sconv", "pack_A", "pack_B", "pack_C", "unpack_C",
    "cake_sgemm_packed_A_size", "cake_sgemm_packed_B_size", "cake_sgemm_packed_C_size",
    "packed_offset", "im2col", "im_2_col", "conv2d", "fill_uniform", "device_info",
    "last_kernel_seconds", "transpose_mat", "linear_forward", "linear_forward_wt", "linear_backward", "sgemm_nt",
    "Context", "grid_dims_2d", "init_block_dims_2d", "init_block_dims_2d_small", "init_block_dims_conv", "pack_filters",
    "last_conv_route", "CONV_NONE", "CONV_SHORTK_BATCH", "CONV_PATCH", "CONV_GATHER", "CONV_TWO_STEP",
    "autotune", "tune_save", "tune_load", "tune_clear", "tune_count",
]
