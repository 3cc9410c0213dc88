"""ctypes binding of libcam_mi355x.so (the C ABI of include/cam_mi355x.h).

This is the stub a maintainer of the reference's binding would write in place of the dlsym trampoline
EXEC_NPU_CMD (src/cam/comm_operator/pybind/pytorch_extension/pytorch_npu_helper.hpp:533-582):
tensors become camTensor structs, phase 1 returns the workspace size and an executor, the caller
allocates the workspace, phase 2 enqueues on the current stream.

There is no fallback: if the shared library is missing or a call fails, an exception is raised.
"""
import contextlib
import ctypes
import os

import torch

_PKG = os.path.dirname(os.path.abspath(__file__))
# CAM_MI355X_LIB names another build of the same library (the clock-stamping profiling build); the default is the
# product library beside this file.
LIB_PATH = os.environ.get("CAM_MI355X_LIB") or os.path.join(_PKG, "lib", "libcam_mi355x.so")

CAM_MAX_DIMS = 8

CAM_OK = 0
CAM_ERR_NULL = 1
CAM_ERR_DTYPE = 2
CAM_ERR_SHAPE = 3
CAM_ERR_RANGE = 4
CAM_ERR_ALIGN = 5
CAM_ERR_UNSUPPORTED = 6
CAM_ERR_WORKSPACE = 7
CAM_ERR_EXECUTOR = 8
CAM_ERR_LAUNCH = 9

CAM_DT_FLOAT = 0
CAM_DT_FLOAT16 = 1
CAM_DT_INT8 = 2
CAM_DT_INT32 = 3
CAM_DT_UINT8 = 4
CAM_DT_INT64 = 9
CAM_DT_BOOL = 12
CAM_DT_BF16 = 27
CAM_DT_FLOAT8_E4M3FN = 36

CAM_FORMAT_ND = 2
CAM_FORMAT_MFMA_B = 100

_DTYPES = {
    torch.float32: CAM_DT_FLOAT,
    torch.float16: CAM_DT_FLOAT16,
    torch.int8: CAM_DT_INT8,
    torch.int32: CAM_DT_INT32,
    torch.uint8: CAM_DT_UINT8,
    torch.int64: CAM_DT_INT64,
    torch.bool: CAM_DT_BOOL,
    torch.bfloat16: CAM_DT_BF16,
    torch.float8_e4m3fn: CAM_DT_FLOAT8_E4M3FN,
}


class CamError(RuntimeError):
    """A non-zero status from the C ABI; `.status` holds the CAM_ERR_* code."""

    def __init__(self, status, message):
        super().__init__("cam status %d: %s" % (status, message))
        self.status = status
        self.message = message


class camTensor(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("ndim", ctypes.c_int32),
        ("sizes", ctypes.c_int64 * CAM_MAX_DIMS),
        ("strides", ctypes.c_int64 * CAM_MAX_DIMS),
        ("format", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class camTensorList(ctypes.Structure):
    _fields_ = [
        ("tensors", ctypes.POINTER(ctypes.POINTER(camTensor))),
        ("count", ctypes.c_uint64),
    ]


_TP = ctypes.POINTER(camTensor)
_LP = ctypes.POINTER(camTensorList)
_I64 = ctypes.c_int64
_STR = ctypes.c_char_p
_PHASE1_TAIL = [ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_void_p)]

# Operator name -> argument types of cam<Op>GetWorkspaceSize before (workspaceSize, executor).
SIGNATURES = {
    "DispatchLayout": [_TP, _I64, _I64, _I64, _I64, _TP, _TP, _TP],
    "NotifyDispatch": [_TP, _TP, _I64, _I64, _STR, _I64, _I64, _I64, _I64, _TP, _TP],
    "MoeDispatchPlan": [_TP, _I64, _I64, _I64, _TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP],
    "MoeDispatchPrefill": [_TP, _TP, _I64, _I64, _I64, _I64, _TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP],
    "MoeDispatchNormal": [_TP, _TP, _TP, _TP, _TP, _TP, _STR, _I64, _I64, _STR, _I64, _I64, _I64, _I64, _I64,
                          _TP, _TP, _TP],
    "MoeCombineNormal": [_TP, _TP, _TP, _TP, _TP, _STR, _I64, _I64, _STR, _I64, _I64, _I64, _I64, _TP],
    "MoeCombineIndex": [_TP, _I64, _TP],
    "MoeCombineGather": [_TP, _TP, _TP, _TP, _TP, _TP, _TP],
    "MoeDispatchShmem": [_TP, _TP, _TP, _TP] + [_I64] * 12 + [_TP] * 6,
    "MoeCombineShmem": [_TP] * 11 + [_I64] * 13 + [_TP],
    "PrepackWeight": [_TP, _I64, _TP],
    "GroupedMatmulSwigluQuant": [_TP, _TP, _LP, _LP, _TP, _I64, _TP, _TP],
    "GroupedMatmulDequant": [_TP, _TP, _LP, _LP, _TP, _I64, _TP],
    "GroupedMatmulInt32": [_TP, _LP, _I64, _TP, _I64, _TP],
    "FusedDeepMoe": [_TP, _TP, _LP, _LP, _LP, _LP, _TP, _TP, _TP, _STR, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                     _TP, _TP],
    "GroupedMatmulFp8": [_TP, _TP, _TP, _TP, _I64, _TP, _I64, _TP, _TP],
    "QuantRowsFp8": [_TP, _TP, _TP],
    "FusedDeepMoeFp8": [_TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP, _I64, _TP, _TP],
}

# Single-call entry points (no executor, no workspace): name -> argument types before the stream.
DIRECT_SIGNATURES = {
    "MoeDispatchPlanNoAlloc": [_TP, _I64, _I64, _I64, _TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP],
}

EXPORTS = ["camGetRecentErrMsg", "camDestroyExecutor", "camGetVersion", "camGemmTimelineInfo"] + [
    "cam%s" % op for op in DIRECT_SIGNATURES] + [
    "cam%s%s" % (op, suffix) for op in SIGNATURES for suffix in ("GetWorkspaceSize", "")
]

_lib = None


def lib():
    """Load the shared library (once). Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m umdk_original_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        handle.camGetRecentErrMsg.restype = ctypes.c_char_p
        handle.camGetVersion.restype = ctypes.c_char_p
        handle.camDestroyExecutor.argtypes = [ctypes.c_void_p]
        for op, argtypes in SIGNATURES.items():
            f1 = getattr(handle, "cam%sGetWorkspaceSize" % op)
            f1.argtypes = argtypes + _PHASE1_TAIL
            f1.restype = ctypes.c_int32
            f2 = getattr(handle, "cam%s" % op)
            f2.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_void_p]
            f2.restype = ctypes.c_int32
        for op, argtypes in DIRECT_SIGNATURES.items():
            f = getattr(handle, "cam%s" % op)
            f.argtypes = argtypes + [ctypes.c_void_p]
            f.restype = ctypes.c_int32
        _lib = handle
    return _lib


def recent_error():
    return lib().camGetRecentErrMsg().decode("utf-8", "replace")


def gemm_timeline_info():
    """camGemmTimelineInfo: (stamps compiled in, words before the first tile record, words per record, byte
    offset of the schedule in a grouped-GEMM operator's workspace)."""
    info = (ctypes.c_int32 * 4)()
    st = lib().camGemmTimelineInfo(info)
    if st != CAM_OK:
        raise CamError(st, recent_error())
    return tuple(int(v) for v in info)


def as_cam_tensor(t, fmt=CAM_FORMAT_ND):
    """camTensor view of a torch tensor (no copy; the caller keeps `t` alive)."""
    if t is None:
        return None
    if t.dtype not in _DTYPES:
        raise CamError(CAM_ERR_DTYPE, "torch dtype %s has no CAM code" % t.dtype)
    if t.dim() > CAM_MAX_DIMS:
        raise CamError(CAM_ERR_SHAPE, "too many dimensions")
    ct = camTensor()
    ct.data = t.data_ptr() if t.numel() > 0 else (t.data_ptr() or 0)
    ct.dtype = _DTYPES[t.dtype]
    ct.ndim = t.dim()
    for d in range(t.dim()):
        ct.sizes[d] = t.size(d)
        ct.strides[d] = t.stride(d)
    ct.format = getattr(t, "_cam_format", fmt)
    return ct


def _ptr(ct):
    return ctypes.byref(ct) if ct is not None else None


class _ListHolder:
    """Keeps the ctypes arrays behind a camTensorList alive."""

    def __init__(self, tensors):
        self.cts = [as_cam_tensor(t) for t in tensors]
        arr_t = ctypes.POINTER(camTensor) * len(self.cts)
        self.arr = arr_t(*[ctypes.pointer(c) for c in self.cts])
        self.lst = camTensorList()
        self.lst.tensors = ctypes.cast(self.arr, ctypes.POINTER(ctypes.POINTER(camTensor)))
        self.lst.count = len(self.cts)


def call(op, args, device=None, stream=None, workspace=None):
    """Run cam<op>GetWorkspaceSize then cam<op>.

    `args` follows the C argument order; entries may be torch tensors (or None), lists of tensors
    (tensor lists), ints, or str/bytes/None for group names.  Returns the workspace tensor used (or
    None) so that a caller may keep it alive or reuse it.
    """
    handle = lib()
    argtypes = SIGNATURES[op]
    if len(args) != len(argtypes):
        raise TypeError("%s expects %d arguments, got %d" % (op, len(argtypes), len(args)))
    keep = []
    cargs = []
    for a, ty in zip(args, argtypes):
        if ty is _TP:
            ct = as_cam_tensor(a) if isinstance(a, torch.Tensor) else a
            keep.append(ct)
            if device is None and isinstance(a, torch.Tensor) and a.is_cuda:
                device = a.device
            cargs.append(_ptr(ct))
        elif ty is _LP:
            if a is None:
                cargs.append(None)
            else:
                h = _ListHolder(list(a))
                keep.append(h)
                cargs.append(ctypes.byref(h.lst))
        elif ty is _STR:
            if isinstance(a, str):
                a = a.encode()
            cargs.append(a)
        else:
            cargs.append(int(a))
    ws_size = ctypes.c_uint64(0)
    executor = ctypes.c_void_p(None)
    st = getattr(handle, "cam%sGetWorkspaceSize" % op)(*cargs, ctypes.byref(ws_size), ctypes.byref(executor))
    if st != CAM_OK:
        raise CamError(st, recent_error())
    try:
        ws = workspace
        if ws_size.value > 0:
            if ws is None or ws.numel() * ws.element_size() < ws_size.value:
                if device is None:
                    raise CamError(CAM_ERR_WORKSPACE, "no device to allocate the workspace on")
                ws = torch.empty(ws_size.value, dtype=torch.uint8, device=device)
        if stream is None:
            if device is not None and device.type == "cuda":
                stream = torch.cuda.current_stream(device).cuda_stream
            else:
                stream = 0
        ws_ptr = ws.data_ptr() if ws is not None else None
        ws_bytes = ws.numel() * ws.element_size() if ws is not None else 0
    except Exception:
        handle.camDestroyExecutor(executor)
        raise
    st = getattr(handle, "cam%s" % op)(ws_ptr, ws_bytes, executor, ctypes.c_void_p(stream))
    if st != CAM_OK:
        raise CamError(st, recent_error())
    return ws


def call_direct(op, args, stream=None):
    """Run a single-call entry point (DIRECT_SIGNATURES) on `stream` (default: torch's current stream)."""
    handle = lib()
    argtypes = DIRECT_SIGNATURES[op]
    if len(args) != len(argtypes):
        raise TypeError("%s expects %d arguments, got %d" % (op, len(argtypes), len(args)))
    keep = []
    cargs = []
    device = None
    for a, ty in zip(args, argtypes):
        if ty is _TP:
            ct = as_cam_tensor(a) if isinstance(a, torch.Tensor) else a
            keep.append(ct)
            if device is None and isinstance(a, torch.Tensor) and a.is_cuda:
                device = a.device
            cargs.append(_ptr(ct))
        else:
            cargs.append(int(a))
    if stream is None:
        stream = torch.cuda.current_stream(device).cuda_stream if device is not None else 0
    # a single-call entry point resolves library-owned device memory for the CURRENT device
    with torch.cuda.device(device) if device is not None else contextlib.nullcontext():
        st = getattr(handle, "cam%s" % op)(*cargs, ctypes.c_void_p(stream))
    if st != CAM_OK:
        raise CamError(st, recent_error())


def phase1(op, args):
    """Phase 1 only (validation): returns (status, workspace size, message); frees the executor."""
    handle = lib()
    argtypes = SIGNATURES[op]
    keep = []
    cargs = []
    for a, ty in zip(args, argtypes):
        if ty is _TP:
            ct = as_cam_tensor(a) if isinstance(a, torch.Tensor) else a
            keep.append(ct)
            cargs.append(_ptr(ct))
        elif ty is _LP:
            if a is None:
                cargs.append(None)
            else:
                h = _ListHolder(list(a))
                keep.append(h)
                cargs.append(ctypes.byref(h.lst))
        elif ty is _STR:
            cargs.append(a.encode() if isinstance(a, str) else a)
        else:
            cargs.append(int(a))
    ws_size = ctypes.c_uint64(0)
    executor = ctypes.c_void_p(None)
    st = getattr(handle, "cam%sGetWorkspaceSize" % op)(*cargs, ctypes.byref(ws_size), ctypes.byref(executor))
    msg = recent_error() if st != CAM_OK else ""
    if st == CAM_OK:
        handle.camDestroyExecutor(executor)
    return st, int(ws_size.value), msg
