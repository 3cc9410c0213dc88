"""MI355X-native implementation of CAM's MoE hot path (dispatch -> w8a8 grouped GEMM -> combine).

The product is the shared library `lib/libcam_mi355x.so` (HIP kernels for gfx950 behind the C ABI of
include/cam_mi355x.h); this package is the thin Python host side that mirrors the reference's
`umdk_cam_op_lib` operators.
"""
from . import _lib
from .ops import (CamError, fused_deep_moe, fused_deep_moe_fp8, get_dispatch_layout, grouped_matmul_dequant,
                  grouped_matmul_fp8, grouped_matmul_int32, quant_rows_fp8,
                  grouped_matmul_swiglu_quant, moe_combine_gather, moe_combine_index, moe_combine_normal,
                  moe_combine_prefill, moe_dispatch_fused, moe_dispatch_normal,
                  moe_dispatch_plan, moe_dispatch_prefill, moe_dispatch_shmem, moe_combine_shmem, notify_dispatch,
                  prepack_weight, register_torch_ops)

__version__ = "0.1.0"

try:
    register_torch_ops()
except RuntimeError:  # the library name is already defined in this process
    pass
