"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares, and
phase 1 rejects bad arguments without touching a GPU (the reference's op_host validation,
e.g. src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_host/fused_deep_moe_tiling.cpp:278-316)."""
import ctypes
import os
import re

import pytest
import torch

from umdk_original_amd import _lib
from umdk_original_amd._lib import (CAM_ERR_DTYPE, CAM_ERR_NULL, CAM_ERR_RANGE, CAM_ERR_SHAPE, CAM_ERR_UNSUPPORTED,
                                    CAM_ERR_ALIGN, CAM_ERR_EXECUTOR, CAM_ERR_WORKSPACE, CAM_OK, CAM_FORMAT_MFMA_B)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "cam_mi355x.h")).read()
    return sorted(set(re.findall(r"CAM_API\s+[\w\s\*]*?\b(cam\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _header_symbols()
    assert len(names) == len(_lib.EXPORTS) >= 29, names
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), n
    assert sorted(_lib.EXPORTS) == names


def test_calibration_library_loads_and_exports_its_entry_points():
    from umdk_original_amd import build
    handle = ctypes.CDLL(build.CALIB_LIB_PATH)
    for n in ("camCalibMfmaInt8", "camCalibRowStores", "camCalibStreamRead", "camCalibDestinationOrder"):
        assert hasattr(handle, n), n


def test_plain_c_caller_validates_without_a_gpu():
    """csrc/abi_consumer.c is compiled as C11 with -Wall -Wextra -Werror against include/cam_mi355x.h and linked with
    nothing but the library and the HIP runtime: phase 1 (validation, workspace size, error strings) from plain C."""
    import subprocess
    from umdk_original_amd import build
    p = subprocess.run([build.ABI_CONSUMER_PATH, "check"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=120)
    assert p.returncode == 0 and "check ok" in p.stdout, p.stdout


def test_version_and_error_string():
    assert b"gfx950" in _lib.lib().camGetVersion()
    st, _, msg = _lib.phase1("DispatchLayout", [None, 1, 1, 1, 1, None, None, None])
    assert st == CAM_ERR_NULL and "topkIdx" in msg


def _t(shape, dtype):
    return torch.zeros(shape, dtype=dtype)


def _layout_args(T=8, K=2, E=4, R=2, idx_dtype=torch.int64):
    return [_t((T, K), idx_dtype), T, R, E, K, _t((R,), torch.int32), _t((E,), torch.int32), _t((T, R), torch.int32)]


def test_dispatch_layout_validation():
    assert _lib.phase1("DispatchLayout", _layout_args())[0] == CAM_OK
    assert _lib.phase1("DispatchLayout", _layout_args(R=385, E=385))[0] == CAM_ERR_RANGE
    assert _lib.phase1("DispatchLayout", _layout_args(E=513, R=1))[0] == CAM_ERR_RANGE
    assert _lib.phase1("DispatchLayout", _layout_args(K=17))[0] == CAM_ERR_RANGE
    assert _lib.phase1("DispatchLayout", _layout_args(E=5, R=2))[0] == CAM_ERR_RANGE  # E % R
    assert _lib.phase1("DispatchLayout", _layout_args(idx_dtype=torch.float32))[0] == CAM_ERR_DTYPE
    a = _layout_args()
    a[0] = _t((8, 2, 1), torch.int64)
    assert _lib.phase1("DispatchLayout", a)[0] == CAM_ERR_SHAPE
    a = _layout_args()
    a[0] = _t((8, 4), torch.int64)[:, ::2]  # not contiguous
    assert _lib.phase1("DispatchLayout", a)[0] == CAM_ERR_SHAPE
    a = _layout_args()
    a[6] = _t((3,), torch.int32)
    assert _lib.phase1("DispatchLayout", a)[0] == CAM_ERR_SHAPE


def _dispatch_args(T=4, K=2, E=8, H=1024, quant=0, R=1, x_dtype=torch.bfloat16, A=None):
    A = T * K if A is None else A
    return [_t((T, H), x_dtype), _t((T, K), torch.int32), _t((E,), torch.int32), _t((T, K), torch.int32),
            _t((E,), torch.int32), _t((E,), torch.int32), "g", R, 0, "g", 1, 0, E, quant, 0,
            _t((A, H), torch.int8 if quant else x_dtype), _t((A,), torch.float32), _t((3 * A,), torch.int32)]


def test_moe_dispatch_normal_validation():
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args())[0] == CAM_OK
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(quant=2))[0] == CAM_OK
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(H=512))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(H=7184))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(H=1028))[0] == CAM_ERR_ALIGN
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(K=17, E=32))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(E=513))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(quant=4))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchNormal", _dispatch_args(quant=1))[0] == CAM_ERR_UNSUPPORTED
    st, _, msg = _lib.phase1("MoeDispatchNormal", _dispatch_args(R=2))
    assert st == CAM_ERR_UNSUPPORTED and "single-GPU" in msg
    a = _dispatch_args(quant=2)
    a[15] = _t((8, 1024), torch.bfloat16)  # quantised output must be int8
    assert _lib.phase1("MoeDispatchNormal", a)[0] == CAM_ERR_DTYPE
    a = _dispatch_args()
    a[1] = _t((5, 2), torch.int32)  # ids disagree with x on dim 0
    assert _lib.phase1("MoeDispatchNormal", a)[0] == CAM_ERR_SHAPE
    a = _dispatch_args()
    a[1] = _t((4, 2), torch.int64)  # kernels take int32 ids
    assert _lib.phase1("MoeDispatchNormal", a)[0] == CAM_ERR_DTYPE
    a = _dispatch_args()
    a[17] = _t((5,), torch.int32)
    assert _lib.phase1("MoeDispatchNormal", a)[0] == CAM_ERR_SHAPE


def _combine_args(T=4, K=2, E=8, H=1024, R=1, gbs=0):
    A = T * K
    return [_t((A, H), torch.bfloat16), _t((3 * A,), torch.int32), _t((E,), torch.int32), _t((T, K), torch.float32),
            None, "g", R, 0, "g", 1, 0, E, gbs, _t((T, H), torch.bfloat16)]


def test_moe_combine_normal_validation():
    st, ws, _ = _lib.phase1("MoeCombineNormal", _combine_args())
    assert st == CAM_OK and ws >= 4 * 2 * 4
    assert _lib.phase1("MoeCombineNormal", _combine_args(H=1000))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeCombineNormal", _combine_args(K=17))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeCombineNormal", _combine_args(R=4))[0] == CAM_ERR_UNSUPPORTED
    assert _lib.phase1("MoeCombineNormal", _combine_args(gbs=3))[0] == CAM_ERR_RANGE
    a = _combine_args()
    a[3] = _t((4, 2), torch.float16)
    assert _lib.phase1("MoeCombineNormal", a)[0] == CAM_ERR_DTYPE
    a = _combine_args()
    a[13] = _t((4, 2048), torch.bfloat16)
    assert _lib.phase1("MoeCombineNormal", a)[0] == CAM_ERR_SHAPE
    a = _combine_args()
    a[0] = _t((8, 1024), torch.float32)
    assert _lib.phase1("MoeCombineNormal", a)[0] == CAM_ERR_DTYPE


def _prefill_args(T=4, K=2, E=8, H=1024, quant=0, R=1, x_dtype=torch.bfloat16, idx_dtype=torch.int64):
    A = T * K
    i32 = torch.int32
    return [_t((T, H), x_dtype), _t((T, K), idx_dtype), E, R, 0, quant,
            _t((A, H), torch.int8 if quant else x_dtype), _t((A,), torch.float32), _t((3 * A,), i32), _t((T, K), i32),
            _t((T, K), i32), _t((E,), i32), _t((E,), i32), _t((E,), i32), _t((E,), torch.int64), _t((1,), torch.int64)]


def test_moe_dispatch_prefill_validation():
    st, ws, _ = _lib.phase1("MoeDispatchPrefill", _prefill_args())
    assert st == CAM_OK and ws > 0
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(quant=2, x_dtype=torch.float16))[0] == CAM_OK
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(idx_dtype=torch.int32, quant=3))[0] == CAM_OK
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(quant=1))[0] == CAM_ERR_UNSUPPORTED
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(quant=5))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(R=2))[0] == CAM_ERR_UNSUPPORTED
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(H=512))[0] == CAM_ERR_RANGE
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(K=17, E=32))[0] == CAM_ERR_RANGE
    a = _prefill_args(quant=2)
    a[7] = None  # scales are required when quantising
    assert _lib.phase1("MoeDispatchPrefill", a)[0] == CAM_ERR_NULL
    a = _prefill_args()
    a[9] = _t((4, 3), torch.int32)
    assert _lib.phase1("MoeDispatchPrefill", a)[0] == CAM_ERR_SHAPE
    a = _prefill_args()
    for i in (10, 11, 12, 13, 14, 15):  # every optional output may be absent
        a[i] = None
    assert _lib.phase1("MoeDispatchPrefill", a)[0] == CAM_OK
    # a long id sequence (many ranking chunks) validates like a short one
    assert _lib.phase1("MoeDispatchPrefill", _prefill_args(T=40000, K=16, E=32))[0] == CAM_OK


def test_combine_gather_validation():
    T, K, H, A, E = 4, 2, 1024, 8, 8
    ok = [_t((A, H), torch.bfloat16), None, _t((T, K), torch.int32), None, _t((T, K), torch.float32), None,
          _t((T, H), torch.bfloat16)]
    assert _lib.phase1("MoeCombineGather", ok)[0] == CAM_OK
    # the shared expert's rows: [T,H] of the output's type
    a = list(ok)
    a[5] = _t((T, H), torch.bfloat16)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_OK
    a[5] = _t((T + 1, H), torch.bfloat16)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_ERR_SHAPE
    a[5] = _t((T, H), torch.float16)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_ERR_DTYPE
    a = list(ok)
    a[1], a[3] = _t((3 * A,), torch.int32), _t((E,), torch.int32)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_OK
    a[1] = _t((3 * A - 1,), torch.int32)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_ERR_SHAPE
    a = list(ok)
    a[2] = _t((T, K + 1), torch.int32)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_ERR_SHAPE
    # rows quantised for the wire: int8 [A, H + H/4]
    a = list(ok)
    a[0] = _t((A, H + H // 4), torch.int8)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_OK
    a[0] = _t((A, H), torch.int8)
    assert _lib.phase1("MoeCombineGather", a)[0] == CAM_ERR_SHAPE


def _dispatch_shmem_args(T=4, K=2, H=1024, E=8, quant=2, dtype=torch.bfloat16):
    A = T * K
    return [_t((T, H), dtype), _t((T, K), torch.int32), None, None, 1, 0, E, 1, 0, 0, 1, 0, quant, 0, 1, 0,
            _t((A, H), torch.int8 if quant == 2 else dtype), _t((A,), torch.float32), _t((T * K,), torch.int32),
            _t((E,), torch.int64), _t((E,), torch.int32), _t((1,), torch.int32)]


def test_dispatch_shmem_validation():
    """Attribute and shape checks of AK/moe_dispatch_shmem/op_host/moe_dispatch_shmem_tiling.cpp:365-535 that
    have a meaning on one rank; the transport's limits (epWorldSize list, H == 7168) are lifted."""
    assert _lib.phase1("MoeDispatchShmem", _dispatch_shmem_args())[0] == CAM_OK
    assert _lib.phase1("MoeDispatchShmem", _dispatch_shmem_args(quant=0))[0] == CAM_OK
    assert _lib.phase1("MoeDispatchShmem", _dispatch_shmem_args(dtype=torch.float16))[0] == CAM_OK
    a = _dispatch_shmem_args()
    a[2] = _t((8, 1024), torch.float32)            # smooth scales [moeExpertNum, H]
    assert _lib.phase1("MoeDispatchShmem", a)[0] == CAM_OK
    a[2] = _t((9, 1024), torch.float32)
    assert _lib.phase1("MoeDispatchShmem", a)[0] == CAM_ERR_SHAPE
    a = _dispatch_shmem_args()
    a[3] = _t((4,), torch.bool)                    # xActiveMask is reserved
    assert _lib.phase1("MoeDispatchShmem", a)[0] == CAM_ERR_UNSUPPORTED
    for pos, bad, want in ((4, 8, CAM_ERR_UNSUPPORTED),     # more than one rank needs peers
                           (4, 0, CAM_ERR_RANGE), (5, 1, CAM_ERR_RANGE), (9, 1, CAM_ERR_RANGE),
                           (12, 1, CAM_ERR_UNSUPPORTED),    # static quantisation
                           (12, 3, CAM_ERR_RANGE), (14, 2, CAM_ERR_RANGE), (7, 2, CAM_ERR_UNSUPPORTED),
                           (13, 3, CAM_ERR_RANGE)):         # globalBs below bs * ranks
        a = _dispatch_shmem_args()
        a[pos] = bad
        assert _lib.phase1("MoeDispatchShmem", a)[0] == want, (pos, bad, _lib.recent_error())
    a = _dispatch_shmem_args()
    a[18] = _t((7,), torch.int32)                  # expandIdx holds bs * K values
    assert _lib.phase1("MoeDispatchShmem", a)[0] == CAM_ERR_SHAPE
    a = _dispatch_shmem_args()
    a[16] = _t((8, 1024), torch.bfloat16)          # int8 rows when quantising
    assert _lib.phase1("MoeDispatchShmem", a)[0] == CAM_ERR_DTYPE
    a = _dispatch_shmem_args()
    a[19] = _t((7,), torch.int64)
    assert _lib.phase1("MoeDispatchShmem", a)[0] == CAM_ERR_SHAPE


def _combine_shmem_args(T=4, K=2, H=1024, E=8, A=8, comm=0, dtype=torch.bfloat16):
    return [_t((A, H), dtype), _t((T, K), torch.int32), _t((T * K,), torch.int32), _t((E,), torch.int32),
            _t((T, K), torch.float32), None, None, None, None, None, None, 1, 0, E, 1, 0, 0, 1, 0, 0, comm, 0, 0, 0,
            _t((T, H), dtype)]


def test_combine_shmem_validation():
    """AK/moe_combine_shmem/op_host/moe_combine_shmem_tiling.cpp:120-200 on one rank."""
    st, ws0, _ = _lib.phase1("MoeCombineShmem", _combine_shmem_args())
    assert st == CAM_OK and ws0 >= 4 * 2 * 4
    st, ws2, _ = _lib.phase1("MoeCombineShmem", _combine_shmem_args(comm=2))
    assert st == CAM_OK and ws2 >= ws0 + 8 * (1024 + 256)  # the wire rows live in the workspace
    assert _lib.phase1("MoeCombineShmem", _combine_shmem_args(dtype=torch.float16))[0] == CAM_OK
    assert _lib.phase1("MoeCombineShmem", _combine_shmem_args(comm=2, dtype=torch.float16))[0] == CAM_OK
    assert _lib.phase1("MoeCombineShmem", _combine_shmem_args(comm=1))[0] == CAM_ERR_RANGE
    for pos in (6, 7, 8, 9, 10):  # reserved inputs
        a = _combine_shmem_args()
        a[pos] = _t((4,), torch.float32)
        assert _lib.phase1("MoeCombineShmem", a)[0] == CAM_ERR_UNSUPPORTED
    for pos, bad, want in ((11, 8, CAM_ERR_UNSUPPORTED), (12, 1, CAM_ERR_RANGE), (16, 1, CAM_ERR_RANGE),
                           (18, 1, CAM_ERR_RANGE), (14, 2, CAM_ERR_UNSUPPORTED)):
        a = _combine_shmem_args()
        a[pos] = bad
        assert _lib.phase1("MoeCombineShmem", a)[0] == want, (pos, bad, _lib.recent_error())
    a = _combine_shmem_args()
    a[2] = _t((7,), torch.int32)
    assert _lib.phase1("MoeCombineShmem", a)[0] == CAM_ERR_SHAPE
    a = _combine_shmem_args()
    a[24] = _t((4, 1024), torch.float16)
    assert _lib.phase1("MoeCombineShmem", a)[0] == CAM_ERR_DTYPE


def _packed(shape):
    w = _t(shape, torch.int8)
    w._cam_format = CAM_FORMAT_MFMA_B
    return w


def _fused_args(bs=4, K=2, E=4, H=1024, I=512, R=1, packed=True, smooth=None, mask=None):
    mk = _packed if packed else (lambda s: _t(s, torch.int8))
    return [_t((bs, H), torch.bfloat16), _t((bs, K), torch.int32), [mk((E, H, 2 * I))], [_t((E, 2 * I), torch.float32)],
            [mk((E, I, H))], [_t((E, H), torch.float32)], _t((bs, K), torch.float32), smooth, mask, "g", R, 0, E, 1, 0,
            0, 0, _t((bs, H), torch.bfloat16), _t((E,), torch.int64)]


def test_fused_deep_moe_validation():
    st, ws, _ = _lib.phase1("FusedDeepMoe", _fused_args())
    assert st == CAM_OK and ws > 0
    assert _lib.phase1("FusedDeepMoe", _fused_args(H=384))[0] == CAM_ERR_RANGE
    assert _lib.phase1("FusedDeepMoe", _fused_args(I=256))[0] == CAM_ERR_RANGE     # 2I < 1024
    assert _lib.phase1("FusedDeepMoe", _fused_args(I=3200))[0] == CAM_ERR_RANGE    # 2I > 6144
    assert _lib.phase1("FusedDeepMoe", _fused_args(K=13, E=16))[0] == CAM_ERR_RANGE
    assert _lib.phase1("FusedDeepMoe", _fused_args(E=513))[0] == CAM_ERR_RANGE
    assert _lib.phase1("FusedDeepMoe", _fused_args(R=2))[0] == CAM_ERR_UNSUPPORTED
    st, _, msg = _lib.phase1("FusedDeepMoe", _fused_args(packed=False))
    assert st == CAM_ERR_UNSUPPORTED and "camPrepackWeight" in msg
    assert _lib.phase1("FusedDeepMoe", _fused_args(smooth=_t((4, 1024), torch.float32)))[0] == CAM_ERR_UNSUPPORTED
    assert _lib.phase1("FusedDeepMoe", _fused_args(mask=_t((5,), torch.bool)))[0] == CAM_ERR_SHAPE
    assert _lib.phase1("FusedDeepMoe", _fused_args(mask=_t((4,), torch.bool)))[0] == CAM_OK
    a = _fused_args()
    a[1] = _t((5, 2), torch.int32)
    assert _lib.phase1("FusedDeepMoe", a)[0] == CAM_ERR_SHAPE
    a = _fused_args()
    a[15] = 7  # quantMode
    assert _lib.phase1("FusedDeepMoe", a)[0] == CAM_ERR_RANGE
    a = _fused_args()
    a[2] = [_packed((4, 1024, 512))]  # wrong 2I
    assert _lib.phase1("FusedDeepMoe", a)[0] == CAM_ERR_SHAPE
    a = _fused_args()
    a[18] = _t((4,), torch.int32)
    assert _lib.phase1("FusedDeepMoe", a)[0] == CAM_ERR_DTYPE
    a = _fused_args()
    a[2] = [_packed((1024, 1024)), _packed((1024, 1024))]  # list length neither 1 nor E
    a[3] = [_t((1024,), torch.float32)] * 2
    assert _lib.phase1("FusedDeepMoe", a)[0] == CAM_ERR_SHAPE


def test_gemm_and_prepack_validation():
    ok = [_t((2, 128, 128), torch.int8), 0, _t((2, 128, 128), torch.int8)]
    assert _lib.phase1("PrepackWeight", ok)[0] == CAM_OK
    assert _lib.phase1("PrepackWeight", [_t((2, 100, 128), torch.int8), 0, _t((2, 100, 128), torch.int8)])[0] == \
        CAM_ERR_UNSUPPORTED
    assert _lib.phase1("PrepackWeight", [_t((2, 128, 64), torch.int8), 1, _t((2, 128, 64), torch.int8)])[0] == \
        CAM_ERR_UNSUPPORTED
    assert _lib.phase1("PrepackWeight", [_t((2, 128, 128), torch.int8), 0, _t((2, 128, 256), torch.int8)])[0] == \
        CAM_ERR_SHAPE
    x = _t((10, 128), torch.int8)
    gl = _t((2,), torch.int64)
    out = _t((10, 128), torch.int32)
    assert _lib.phase1("GroupedMatmulInt32", [x, [_packed((2, 128, 128))], 0, gl, 0, out])[0] == CAM_OK
    assert _lib.phase1("GroupedMatmulInt32", [x, [_t((2, 128, 128), torch.int8)], 0, gl, 0, out])[0] == \
        CAM_ERR_UNSUPPORTED
    assert _lib.phase1("GroupedMatmulInt32", [x, [_packed((2, 128, 128))], 0, gl, 2, out])[0] == CAM_ERR_RANGE
    assert _lib.phase1("GroupedMatmulInt32", [x, [_packed((2, 128, 128))], 0, _t((2,), torch.int32), 0, out])[0] == \
        CAM_ERR_DTYPE
    # outputs and weight scales are written and read 16 bytes at a time
    skewed = _t((10 * 128 + 1,), torch.int32)[1:].view(10, 128)
    assert _lib.phase1("GroupedMatmulInt32", [x, [_packed((2, 128, 128))], 0, gl, 0, skewed])[0] == CAM_ERR_ALIGN
    xs, bf = _t((10,), torch.float32), _t((10, 128), torch.bfloat16)
    deq = [x, xs, [_packed((2, 128, 128))], [_t((2, 128), torch.float32)], gl, 0, bf]
    assert _lib.phase1("GroupedMatmulDequant", deq)[0] == CAM_OK
    deq[3] = [_t((2 * 128 + 1,), torch.float32)[1:].view(2, 128)]
    assert _lib.phase1("GroupedMatmulDequant", deq)[0] == CAM_ERR_ALIGN
    deq[3] = [_t((2, 128), torch.float32)]
    deq[6] = _t((10 * 128 + 1,), torch.bfloat16)[1:].view(10, 128)
    assert _lib.phase1("GroupedMatmulDequant", deq)[0] == CAM_ERR_ALIGN
    deq[6] = _t((10, 160), torch.int8)  # wire rows: N + N/4 columns of int8
    st, ws_wire, _ = _lib.phase1("GroupedMatmulDequant", deq)
    assert st == CAM_OK and ws_wire >= 10 * 128 * 2
    deq[6] = _t((10, 128), torch.int8)
    assert _lib.phase1("GroupedMatmulDequant", deq)[0] == CAM_ERR_SHAPE


def test_phase2_rejects_wrong_executor_and_small_workspace():
    handle = _lib.lib()
    assert handle.camDispatchLayout(None, 0, None, None) == CAM_ERR_EXECUTOR
    # a combine executor handed to the layout op
    args = _combine_args()
    keep = [_lib.as_cam_tensor(a) if isinstance(a, torch.Tensor) else a for a in args]
    cargs = [ctypes.byref(k) if isinstance(k, _lib.camTensor) else (k.encode() if isinstance(k, str) else k)
             for k in keep]
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    assert handle.camMoeCombineNormalGetWorkspaceSize(*cargs, ctypes.byref(ws), ctypes.byref(ex)) == CAM_OK
    assert handle.camDispatchLayout(None, 0, ex, None) == CAM_ERR_EXECUTOR  # consumed and freed
    ex = ctypes.c_void_p(None)
    assert handle.camMoeCombineNormalGetWorkspaceSize(*cargs, ctypes.byref(ws), ctypes.byref(ex)) == CAM_OK
    assert handle.camMoeCombineNormal(None, 0, ex, None) == CAM_ERR_WORKSPACE  # no launch attempted
    assert "workspace" in _lib.recent_error()


def test_ops_refuse_cpu_tensors_and_unpacked_weights():
    import umdk_original_amd as cam
    with pytest.raises(RuntimeError, match="ROCm device"):
        cam.get_dispatch_layout(torch.zeros(4, 2, dtype=torch.int64), 4, 1)
    with pytest.raises(RuntimeError, match="Assertion failed"):
        cam.get_dispatch_layout(torch.zeros(4, dtype=torch.int64), 4, 1)
    with pytest.raises(cam.CamError):
        cam.grouped_matmul_int32(torch.zeros(4, 128, dtype=torch.int8), torch.zeros(1, 128, 128, dtype=torch.int8),
                                 torch.zeros(1, dtype=torch.int64))


def test_torch_ops_registered_with_reference_schemas():
    import umdk_original_amd  # noqa: F401
    s = str(torch.ops.umdk_cam_op_lib.fused_deep_moe.default._schema)
    assert "Tensor[] gmm1PermutedWeight" in s and "Tensor? xActiveMask" in s and "-> Tensor[]" in s
    s = str(torch.ops.umdk_cam_op_lib.moe_dispatch_prefill.default._schema)
    assert "int num_worst_tokens" in s and "str group_ep" in s
    out = torch.ops.umdk_cam_op_lib.fused_deep_moe(
        torch.empty(4, 1024, device="meta", dtype=torch.bfloat16), torch.empty(4, 2, device="meta", dtype=torch.int32),
        [], [], [], [], torch.empty(4, 2, device="meta"), None, None, "g", 1, 0, 8, 1, 0, 0, 0)
    assert out[0].shape == (4, 1024) and out[1].shape == (8,) and out[1].dtype == torch.int64


def test_fp8_operator_validation():
    f8, u8 = torch.float8_e4m3fn, torch.uint8

    def packed8(shape):
        w = _t(shape, f8)
        w._cam_format = CAM_FORMAT_MFMA_B
        return w

    gl = _t((2,), torch.int64)
    ok = [_t((10, 256), f8), _t((10, 2), u8), packed8((2, 256, 512)), _t((2, 2, 4), u8), 0, gl, 0,
          _t((10, 512), torch.float32), None]
    assert _lib.phase1("GroupedMatmulFp8", ok)[0] == CAM_OK
    a = list(ok)
    a[7] = _t((10, 512), torch.bfloat16)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_OK
    a = list(ok)
    a[4], a[7] = 1, _t((10, 256), torch.float32)      # SwiGLU product: N/2 columns
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_OK
    a[7] = _t((10, 256), torch.bfloat16)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_DTYPE
    a[7], a[8] = _t((10, 256), f8), _t((10, 2), u8)    # product quantised in the epilogue
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_OK
    a[8] = None
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_NULL
    a[8] = _t((10, 1), u8)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_SHAPE
    a[4], a[7], a[8] = 0, _t((10, 512), f8), _t((10, 4), u8)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_DTYPE   # FP8 out needs the gate/up pairing
    a[7] = _t((10, 512), torch.float32)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_DTYPE   # outScale without an FP8 out
    a = list(ok)
    a[1] = _t((10, 3), u8)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_SHAPE
    a = list(ok)
    a[2] = _t((2, 256, 512), f8)                       # not prepacked
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_UNSUPPORTED
    a = list(ok)
    a[0], a[1], a[2], a[3] = _t((10, 192), f8), _t((10, 1), u8), packed8((2, 192, 512)), _t((2, 1, 4), u8)
    assert _lib.phase1("GroupedMatmulFp8", a)[0] == CAM_ERR_RANGE   # K not a multiple of 128
    assert _lib.phase1("QuantRowsFp8", [_t((4, 256), torch.float32), _t((4, 256), f8), _t((4, 2), u8)])[0] == CAM_OK
    assert _lib.phase1("QuantRowsFp8", [_t((4, 200), torch.float32), _t((4, 200), f8), _t((4, 1), u8)])[0] == \
        CAM_ERR_ALIGN
    T, K, E, H, I = 4, 2, 4, 1024, 512
    fused = [_t((T, H), torch.bfloat16), _t((T, K), torch.int32), packed8((E, H, 2 * I)), _t((E, H // 128, 2 * I // 128), u8),
             packed8((E, I, H)), _t((E, I // 128, H // 128), u8), _t((T, K), torch.float32), None, E,
             _t((T, H), torch.bfloat16), _t((E,), torch.int64)]
    st, ws, _ = _lib.phase1("FusedDeepMoeFp8", fused)
    assert st == CAM_OK and ws > 0
    a = list(fused)
    a[3] = _t((E, H // 128, 2 * I // 128 + 1), u8)
    assert _lib.phase1("FusedDeepMoeFp8", a)[0] == CAM_ERR_SHAPE
    a = list(fused)
    a[8] = 513
    assert _lib.phase1("FusedDeepMoeFp8", a)[0] == CAM_ERR_RANGE
    a = list(fused)
    a[0] = _t((T, H), torch.float16)                   # the block-scaled layer takes bf16 activations only
    assert _lib.phase1("FusedDeepMoeFp8", a)[0] == CAM_ERR_DTYPE
    # quantMode 4 of MoeDispatchPrefill: FP8 rows with uint8 block scales
    pre = _prefill_args()
    pre[5] = 4
    assert _lib.phase1("MoeDispatchPrefill", pre)[0] != CAM_OK          # int8 rows / fp32 scales do not fit


def test_torch_operator_library_is_built_and_registers_the_reference_schemas():
    import os
    from umdk_original_amd import ops
    path = os.path.join(os.path.dirname(_lib.LIB_PATH), "libcam_torch_ops.so")
    assert os.path.exists(path), "python -m umdk_original_amd.build builds it"
    assert ops._torch_lib == "cpp"
    for name in ("fused_deep_moe", "get_dispatch_layout", "moe_dispatch_prefill", "moe_combine_prefill",
                 "moe_dispatch_shmem", "moe_combine_shmem", "prepack_weight"):
        assert hasattr(torch.ops.umdk_cam_op_lib, name)
    s = str(torch.ops.umdk_cam_op_lib.moe_combine_prefill.default._schema)
    assert "Tensor send_head, str group_ep, int rank, int num_ranks" in s
    s = str(torch.ops.umdk_cam_op_lib.moe_dispatch_shmem.default._schema)
    assert "Tensor? scales, Tensor? xActiveMask, int epWorldSize, int epRankId, int moeExpertNum" in s
    s = str(torch.ops.umdk_cam_op_lib.moe_combine_shmem.default._schema)
    assert "int globalBS, int commQuantMode, int extInfo, int outDtype, int groupListType) -> Tensor" in s


def test_torch_operators_have_autograd_and_meta_registrations():
    """As in the reference: every operator sits on the autograd key too (backward returns no gradients,
    src/cam/comm_operator/pybind/fused_deep_moe.cpp:152-229), and the operators whose shapes follow from their
    arguments have Meta implementations (…/moe_dispatch_shmem.cpp:153-190, …/moe_combine_shmem.cpp:88-123)."""
    for name in ("fused_deep_moe", "get_dispatch_layout", "moe_dispatch_prefill", "moe_combine_prefill",
                 "moe_dispatch_shmem", "moe_combine_shmem"):
        assert torch._C._dispatch_has_kernel_for_dispatch_key("umdk_cam_op_lib::" + name, "AutogradCUDA"), name
        assert torch._C._dispatch_has_kernel_for_dispatch_key("umdk_cam_op_lib::" + name, "CUDA"), name
    ops = torch.ops.umdk_cam_op_lib
    x = torch.empty((6, 2048), dtype=torch.bfloat16, device="meta")
    ids = torch.empty((6, 4), dtype=torch.int32, device="meta")
    d = ops.moe_dispatch_shmem(x, ids, None, None, 1, 0, 16, 1, 0, 0, 1, 0, 2, 0, 1, 0)
    assert [tuple(t.shape) for t in d] == [(24, 2048), (24,), (24,), (16,), (16,), (1,)]
    assert d[0].dtype == torch.int8 and d[1].dtype == torch.float32 and d[3].dtype == torch.int64
    d0 = ops.moe_dispatch_shmem(x, ids, None, None, 1, 0, 2, 1, 0, 0, 1, 0, 0, 0, 1, 0)
    assert tuple(d0[0].shape) == (12, 2048) and d0[0].dtype == torch.bfloat16   # bs * min(K, experts) rows
    w = torch.empty((6, 4), dtype=torch.float32, device="meta")
    out = ops.moe_combine_shmem(torch.empty((24, 2048), dtype=torch.bfloat16, device="meta"), ids, d[2], d[4], w, None,
                                None, None, None, None, None, 1, 0, 16, 1, 0, 0, 1, 0, 0, 0, 0, 0, 0)
    assert tuple(out.shape) == (6, 2048) and out.dtype == torch.bfloat16
