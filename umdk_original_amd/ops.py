"""Host-side mirror of CAM's Python operator surface, on top of the C ABI.

Same names, argument meaning, return shapes/dtypes and error behaviour as the reference's
`umdk_cam_op_lib` module (src/cam/comm_operator/pybind/pybind.cpp:13-41):

    get_dispatch_layout   src/cam/comm_operator/pybind/get_dispatch_layout.cpp:26-56
    moe_dispatch_prefill  src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:26-192
    moe_combine_prefill   src/cam/comm_operator/pybind/moe_combine_prefill.cpp:26-74
    fused_deep_moe        src/cam/comm_operator/pybind/fused_deep_moe.cpp:23-79

The same four operators are registered as torch custom ops under the library name
`umdk_cam_op_lib` with the reference's schemas, so `torch.ops.umdk_cam_op_lib.fused_deep_moe(...)`
works on a ROCm device exactly as it does on the reference's device.

Differences a caller can observe, all stated where they occur: one rank only; weights must be
prepacked with `prepack_weight` (the reference needs `npu_format_cast(..., FRACTAL_NZ)` at the same
place); `moe_dispatch_prefill` takes an optional `quant_mode` keyword (the reference binding
hard-codes 0 although its kernel supports dynamic quantisation).
"""
import os
import weakref

import torch

from . import _lib
from ._lib import CamError, CAM_FORMAT_MFMA_B

__all__ = [
    "CamError", "get_dispatch_layout", "moe_dispatch_plan", "moe_dispatch_fused", "moe_dispatch_prefill", "moe_dispatch_normal",
    "moe_dispatch_shmem", "moe_combine_shmem",
    "moe_combine_prefill", "moe_combine_normal", "moe_combine_index", "moe_combine_gather", "notify_dispatch", "prepack_weight",
    "grouped_matmul_swiglu_quant", "grouped_matmul_dequant", "grouped_matmul_int32", "fused_deep_moe",
]


def _bind_assert(cond, what):
    # Counterpart of TORCH_BIND_ASSERT (src/cam/comm_operator/pybind/utils.h:15-38): throws.
    if not cond:
        raise RuntimeError("Assertion failed: " + what)


def _require_gpu(t, name):
    if not t.is_cuda:
        raise RuntimeError("%s must live on a ROCm device (the CAM kernels have no CPU path)" % name)


# --------------------------------------------------------------------------------------------------
def get_dispatch_layout(topk_idx, num_experts, num_ranks):
    """-> (num_tokens_per_rank int32 [R], num_tokens_per_expert int32 [E], is_token_in_rank bool [T,R])."""
    _bind_assert(topk_idx.dim() == 2, "topkIdx.dim() == 2")
    _bind_assert(topk_idx.is_contiguous(), "topkIdx.is_contiguous()")
    _bind_assert(num_experts > 0, "numExperts > 0")
    _require_gpu(topk_idx, "topk_idx")
    T, K = topk_idx.shape
    dev = topk_idx.device
    per_expert = torch.empty(num_experts, dtype=torch.int32, device=dev)
    per_rank = torch.empty(num_ranks, dtype=torch.int32, device=dev)
    in_rank = torch.empty((T, num_ranks), dtype=torch.bool, device=dev)
    _lib.call("DispatchLayout", [topk_idx, T, num_ranks, num_experts, K, per_rank, per_expert, in_rank])
    return per_rank, per_expert, in_rank


def notify_dispatch(num_tokens_per_expert, num_tokens, group_ep="", rank=0, num_ranks=1):
    """Exclusive offsets and (count, offset, numTokens) triplets -> (send_data, send_data_offset, recv_data)."""
    _require_gpu(num_tokens_per_expert, "num_tokens_per_expert")
    E = num_tokens_per_expert.numel()
    dev = num_tokens_per_expert.device
    send_data = torch.empty(3 * E, dtype=torch.int32, device=dev)
    offset = torch.empty(E, dtype=torch.int32, device=dev)
    recv_data = torch.empty(3 * E, dtype=torch.int32, device=dev)
    _lib.call("NotifyDispatch", [send_data, num_tokens_per_expert, 3 * E, num_tokens, group_ep, num_ranks, rank,
                                 num_ranks, rank % max(num_ranks, 1), offset, recv_data])
    return send_data, offset, recv_data


def moe_dispatch_plan(topk_idx, num_experts, num_ranks=1, rank=0):
    """Device-side replacement of the binding's two CPU loops.

    -> dict(send_token_idx [T,K] i32, num_tokens_per_expert [E] i32, send_offset [E] i32,
            recv_offset [E] i32, recv_count [E] i32, num_recv_tokens_per_expert [E/R] i64, total [1] i64,
            slot_row [T,K] i32: output row of every (token, k), -1 where the entry is skipped)
    """
    _require_gpu(topk_idx, "topk_idx")
    T, K = topk_idx.shape
    dev = topk_idx.device
    i32 = dict(dtype=torch.int32, device=dev)
    out = dict(
        send_token_idx=torch.empty((T, K), **i32),
        num_tokens_per_expert=torch.empty(num_experts, **i32),
        send_offset=torch.empty(num_experts, **i32),
        recv_offset=torch.empty(num_experts, **i32),
        recv_count=torch.empty(num_experts, **i32),
        num_recv_tokens_per_expert=torch.empty(num_experts // max(num_ranks, 1), dtype=torch.int64, device=dev),
        total=torch.empty(1, dtype=torch.int64, device=dev),
        slot_row=torch.empty((T, K), **i32),
    )
    _lib.call("MoeDispatchPlan", [topk_idx, num_experts, num_ranks, rank, out["send_token_idx"],
                                  out["num_tokens_per_expert"], out["send_offset"], out["recv_offset"],
                                  out["recv_count"], out["num_recv_tokens_per_expert"], out["total"],
                                  out["slot_row"]])
    return out


def moe_dispatch_fused(x, topk_idx, num_experts, quant_mode=0, num_rows=None, rank=0, num_ranks=1):
    """Plan + permute (+ quantisation) as one operator (MoeDispatchPrefill of the C ABI).

    Outputs are sized for `num_rows` rows (default: the worst case T*K); rows at or past total[0] are
    left unwritten.  -> dict(recv_x, recv_x_scales, expand_idx, send_token_idx, slot_row,
    num_tokens_per_expert, send_offset, recv_count, num_recv_tokens_per_expert, total)
    """
    _require_gpu(x, "x")
    T, H = x.shape
    K = topk_idx.size(1)
    A = max(int(T * K if num_rows is None else num_rows), 1)
    dev = x.device
    i32 = dict(dtype=torch.int32, device=dev)
    if quant_mode == 4:   # block-scaled FP8: E4M3 rows, one E8M0 scale per row and 128 columns
        rx = torch.empty((A, H), dtype=torch.float8_e4m3fn, device=dev)
        rs = torch.empty((A, H // 128), dtype=torch.uint8, device=dev)
    else:
        rx = torch.empty((A, H), dtype=torch.int8 if quant_mode != 0 else x.dtype, device=dev)
        rs = torch.empty(A, dtype=torch.float32, device=dev)
    out = dict(
        recv_x=rx,
        recv_x_scales=rs,
        expand_idx=torch.empty(3 * A, **i32),
        send_token_idx=torch.empty((T, K), **i32),
        slot_row=torch.empty((T, K), **i32),
        num_tokens_per_expert=torch.empty(num_experts, **i32),
        send_offset=torch.empty(num_experts, **i32),
        recv_count=torch.empty(num_experts, **i32),
        num_recv_tokens_per_expert=torch.empty(num_experts // max(num_ranks, 1), dtype=torch.int64, device=dev),
        total=torch.empty(1, dtype=torch.int64, device=dev),
    )
    _lib.call("MoeDispatchPrefill", [x, topk_idx, num_experts, num_ranks, rank, quant_mode, out["recv_x"],
                                     out["recv_x_scales"], out["expand_idx"], out["send_token_idx"], out["slot_row"],
                                     out["num_tokens_per_expert"], out["send_offset"], out["recv_count"],
                                     out["num_recv_tokens_per_expert"], out["total"]])
    return out


def moe_dispatch_normal(x, topk_idx, send_offset, send_token_idx, recv_offset, recv_count, total_rows,
                        num_experts, quant_mode=0, group_ep="", rank=0, num_ranks=1, global_bs=0):
    """aclnnMoeDispatchNormal: -> (recv_x [A,H], recv_x_scales fp32 [A], assist_info int32 [3A])."""
    _require_gpu(x, "x")
    H = x.size(1)
    A = max(int(total_rows), 1)
    dev = x.device
    recv_x = torch.empty((A, H), dtype=torch.int8 if quant_mode != 0 else x.dtype, device=dev)
    scales = torch.empty(A, dtype=torch.float32, device=dev)
    assist = torch.empty(3 * A, dtype=torch.int32, device=dev)
    ids = topk_idx if topk_idx.dtype == torch.int32 else topk_idx.to(torch.int32)
    _lib.call("MoeDispatchNormal", [x, ids, send_offset, send_token_idx, recv_offset, recv_count, group_ep,
                                    num_ranks, rank, group_ep, 1, 0, num_experts, quant_mode, global_bs,
                                    recv_x, scales, assist])
    return recv_x, scales, assist


def moe_dispatch_prefill(x, topk_idx, topk_weights, num_tokens_per_rank, is_token_in_rank, num_tokens_per_expert,
                         num_worst_tokens, group_ep, rank, num_ranks, quant_mode=0, return_scales=False):
    """-> (expand_x [total,H], expand_idx int32 [3*total], recv_count int32 [E],
           num_recv_tokens_per_expert int64 [E/R] on the CPU).

    One launch (MoeDispatchPrefill) ranks, places and copies/quantises the rows.  The total row count
    decides the output shapes, so one 8-byte device-to-host copy is made afterwards (the reference makes
    two larger ones and runs the index arithmetic on the CPU).  With `num_worst_tokens` > 0 the outputs keep
    that many rows instead, nothing is copied until the fourth return value is produced, and rows beyond the
    true total are left unwritten (moe_combine_prefill ignores them: it stops at recv_count[-1]).
    """
    _bind_assert(is_token_in_rank.dtype == torch.bool, "isTokenInRank.scalar_type() == at::kBool")
    _bind_assert(num_tokens_per_expert.dtype == torch.int32, "numTokensPerExpert.scalar_type() == at::kInt")
    _bind_assert(num_tokens_per_rank.dtype == torch.int32, "numTokensPerRank.scalar_type() == at::kInt")
    _bind_assert(x.dim() == 2 and x.is_contiguous(), "newX.dim() == 2 and newX.is_contiguous()")
    _bind_assert(is_token_in_rank.dim() == 2 and is_token_in_rank.is_contiguous(),
                 "isTokenInRank.dim() == 2 and isTokenInRank.is_contiguous()")
    _bind_assert(is_token_in_rank.size(0) == x.size(0) and is_token_in_rank.size(1) == num_ranks,
                 "isTokenInRank.size(0) == newX.size(0) and isTokenInRank.size(1) == numRanks")
    _bind_assert(num_tokens_per_expert.dim() == 1 and num_tokens_per_expert.is_contiguous(),
                 "numTokensPerExpert.dim() == 1 and numTokensPerExpert.is_contiguous()")
    _bind_assert(num_tokens_per_expert.size(0) % num_ranks == 0, "numTokensPerExpert.size(0) % numRanks == 0")
    _bind_assert(num_tokens_per_rank.dim() == 1 and num_tokens_per_rank.is_contiguous(),
                 "numTokensPerRank.dim() == 1 and numTokensPerRank.is_contiguous()")
    _bind_assert(num_tokens_per_rank.size(0) == num_ranks, "numTokensPerRank.size(0) == numRanks")
    num_experts = num_tokens_per_expert.size(0)
    _bind_assert(num_experts > 0, "numExperts > 0")
    _bind_assert(topk_idx.dim() == 2 and topk_idx.is_contiguous(), "topkIdx.dim() == 2 and topkIdx.is_contiguous()")
    _bind_assert(topk_weights.dim() == 2 and topk_weights.is_contiguous(),
                 "topkWeights.dim() == 2 and topkWeights.is_contiguous()")
    _bind_assert(x.size(0) == topk_idx.size(0), "numTokens == topkIdx.size(0)")
    _bind_assert(topk_idx.size(1) == topk_weights.size(1), "numTopk == topkWeights.size(1)")
    _bind_assert(topk_weights.dtype == torch.float32, "topkWeights.scalar_type() == at::kFloat")
    _require_gpu(x, "x")

    worst = bool(num_worst_tokens and num_worst_tokens > 0)
    d = moe_dispatch_fused(x, topk_idx, num_experts, quant_mode=quant_mode,
                           num_rows=int(num_worst_tokens) if worst else None, rank=rank, num_ranks=num_ranks)
    recv_x, scales, expand_idx = d["recv_x"], d["recv_x_scales"], d["expand_idx"]
    if not worst:
        # The reference sizes expand_x by the true total (moe_dispatch_prefill.cpp:156-162); the rows were written
        # into worst-case buffers, so the results are prefix views of those and nothing is copied.
        total = int(d["total"].item())
        recv_x, scales, expand_idx = recv_x[:total], scales[:total], expand_idx[:3 * total]
    per_expert_cpu = d["num_recv_tokens_per_expert"].cpu()
    if return_scales:
        return recv_x, expand_idx, d["recv_count"], per_expert_cpu, scales
    return recv_x, expand_idx, d["recv_count"], per_expert_cpu


def moe_combine_normal(recv_x, token_src_info, ep_recv_counts, topk_weights, group_ep="", rank=0, num_ranks=1,
                       global_bs=0):
    """aclnnMoeCombineNormal: -> combined bf16 [T,H]."""
    _require_gpu(recv_x, "recv_x")
    T = topk_weights.size(0)
    out = torch.empty((T, recv_x.size(1)), dtype=recv_x.dtype, device=recv_x.device)
    _lib.call("MoeCombineNormal", [recv_x, token_src_info, ep_recv_counts, topk_weights, None, group_ep, num_ranks,
                                   rank, group_ep, 1, 0, ep_recv_counts.size(0), global_bs, out])
    return out


def moe_combine_index(token_src_info, num_rows, num_tokens, top_k):
    """(token, k) -> row map from the (srcRank, token, k) triples; build once, reuse for several gathers."""
    _require_gpu(token_src_info, "token_src_info")
    slot_row = torch.empty((num_tokens, top_k), dtype=torch.int32, device=token_src_info.device)
    _lib.call("MoeCombineIndex", [token_src_info, num_rows, slot_row])
    return slot_row


def moe_combine_gather(recv_x, token_src_info, slot_row, topk_weights, out=None, ep_recv_counts=None,
                       shared_x=None):
    """Weighted gather-reduce with a prebuilt map: -> combined bf16 [T,H].

    token_src_info=None trusts slot_row as it stands (the dispatch operators' slot_row output); with the
    triples given, entries whose row does not point back at the slot are skipped (a map from moe_combine_index).
    shared_x [T,H]: the shared expert's rows, added un-weighted after the routed rows, before the rounding.
    """
    _require_gpu(recv_x, "recv_x")
    if out is None:
        # int8 rows are wire rows [A, H + H/4] (grouped_matmul_dequant(..., wire_rows=True))
        h = recv_x.size(1) // 5 * 4 if recv_x.dtype == torch.int8 else recv_x.size(1)
        out = torch.empty((topk_weights.size(0), h),
                          dtype=torch.bfloat16 if recv_x.dtype == torch.int8 else recv_x.dtype, device=recv_x.device)
    _lib.call("MoeCombineGather", [recv_x, token_src_info, slot_row, ep_recv_counts, topk_weights, shared_x, out])
    return out


def moe_dispatch_shmem(x, expertIds, scales=None, xActiveMask=None, epWorldSize=1, epRankId=0, moeExpertNum=0,
                       tpWorldSize=1, tpRankId=0, expertShardType=0, sharedExpertNum=1, sharedExpertRankNum=0,
                       quantMode=0, globalBS=0, expertTokenNumsType=1, extInfo=0):
    """The reference's moe_dispatch_shmem on one rank (src/cam/comm_operator/pybind/moe_dispatch_shmem.cpp:27-153).
    -> [expandX [bs*min(K, experts), H], dynamicScales fp32, expandIdx int32 [bs*K], expertTokenNums int64,
        epRecvCount int32, tpRecvCount int32 [tpWorldSize]]"""
    _require_gpu(x, "x")
    bs, h = x.shape
    k = expertIds.size(1)
    _bind_assert(epWorldSize != sharedExpertRankNum, "epWorldSize != sharedExpertRankNum")
    per_rank = moeExpertNum // (epWorldSize - sharedExpertRankNum)
    rows = bs * epWorldSize * min(per_rank, k)
    dev = x.device
    expand_x = torch.empty((rows, h), dtype=torch.int8 if quantMode == 2 else x.dtype, device=dev)
    dyn = torch.empty(rows, dtype=torch.float32, device=dev)
    expand_idx = torch.empty(bs * k, dtype=torch.int32, device=dev)
    etn = torch.empty(per_rank, dtype=torch.int64, device=dev)
    ep_cnt = torch.empty(epWorldSize * per_rank, dtype=torch.int32, device=dev)
    tp_cnt = torch.empty(tpWorldSize, dtype=torch.int32, device=dev)
    _lib.call("MoeDispatchShmem", [x, expertIds, scales, xActiveMask, epWorldSize, epRankId, moeExpertNum, tpWorldSize,
                                   tpRankId, expertShardType, sharedExpertNum, sharedExpertRankNum, quantMode,
                                   globalBS, expertTokenNumsType, extInfo, expand_x, dyn, expand_idx, etn, ep_cnt,
                                   tp_cnt])
    return [expand_x, dyn, expand_idx, etn, ep_cnt, tp_cnt]


def moe_combine_shmem(expandX, expertIds, expandIdx, epSendCounts, expertScales, tpSendCounts=None,
                      xActiveMask=None, activationScale=None, weightScale=None, groupList=None, expandScales=None,
                      epWorldSize=1, epRankId=0, moeExpertNum=0, tpWorldSize=1, tpRankId=0, expertShardType=0,
                      sharedExpertNum=1, sharedExpertRankNum=0, globalBS=0, commQuantMode=0, extInfo=0, outDtype=0,
                      groupListType=0):
    """The reference's moe_combine_shmem on one rank (src/cam/comm_operator/pybind/moe_combine_shmem.cpp:27-86).
    -> out [bs,H], dtype of expandX."""
    _require_gpu(expandX, "expandX")
    out = torch.empty((expertIds.size(0), expandX.size(1)), dtype=expandX.dtype, device=expandX.device)
    _lib.call("MoeCombineShmem", [expandX, expertIds, expandIdx, epSendCounts, expertScales, tpSendCounts, xActiveMask,
                                  activationScale, weightScale, groupList, expandScales, epWorldSize, epRankId,
                                  moeExpertNum, tpWorldSize, tpRankId, expertShardType, sharedExpertNum,
                                  sharedExpertRankNum, globalBS, commQuantMode, extInfo, outDtype, groupListType, out])
    return out


def moe_combine_prefill(x, topk_idx, topk_weights, src_idx, send_head, group_ep, rank, num_ranks):
    """-> combined_x [T,H], dtype of x."""
    _bind_assert(x.dim() == 2 and x.is_contiguous(), "x.dim() == 2 and x.is_contiguous()")
    global_bs = topk_idx.size(0) * num_ranks
    return moe_combine_normal(x, src_idx, send_head, topk_weights, group_ep, rank, num_ranks, global_bs)


# --------------------------------------------------------------------------------------------------
def prepack_weight(w, gate_up):
    """One-time conversion of int8 weights [G,Kd,N] / [Kd,N] to the MFMA operand layout.

    gate_up=True for the fused gate/up projection (GMM1), False for the down projection (GMM2).
    The result carries the format tag the GEMM operators insist on.
    """
    _require_gpu(w, "w")
    w = w.contiguous()
    if _torch_lib == "cpp":
        # the C++ operator library remembers the storage of its packed results; fused_deep_moe checks it
        out = torch.ops.umdk_cam_op_lib.prepack_weight(w, bool(gate_up))
    else:
        out = torch.empty_like(w)
        _lib.call("PrepackWeight", [w, 1 if gate_up else 0, out])
    out._cam_format = CAM_FORMAT_MFMA_B
    out._cam_gate_up = bool(gate_up)
    _PACKED[out.data_ptr()] = (weakref.ref(out), bool(gate_up))
    return out


def _tag_list(ws):
    for w in ws:
        if getattr(w, "_cam_format", None) != CAM_FORMAT_MFMA_B:
            raise CamError(_lib.CAM_ERR_UNSUPPORTED,
                           "weights must be converted once with prepack_weight() before the call")
    return list(ws)


def grouped_matmul_swiglu_quant(x, x_scale, weight, weight_scale, group_list, group_list_type=0):
    """GMM1 stage: int8 [A,H] -> (int8 [A,I], fp32 [A])."""
    weight = _tag_list(weight if isinstance(weight, (list, tuple)) else [weight])
    weight_scale = list(weight_scale) if isinstance(weight_scale, (list, tuple)) else [weight_scale]
    A = x.size(0)
    I = weight[0].size(-1) // 2
    y = torch.empty((A, I), dtype=torch.int8, device=x.device)
    ys = torch.empty(A, dtype=torch.float32, device=x.device)
    _lib.call("GroupedMatmulSwigluQuant", [x, x_scale, weight, weight_scale, group_list, group_list_type, y, ys])
    return y, ys


def grouped_matmul_dequant(x, x_scale, weight, weight_scale, group_list, group_list_type=0, wire_rows=False,
                           out_dtype=torch.bfloat16):
    """GMM2 stage: int8 [A,I] -> bf16 [A,H]; wire_rows=True: -> int8 [A, H + H/4], the bf16 rows quantised for
    the wire (8-column blocks: int8 values, then bf16 block scales), which moe_combine_gather reads back."""
    weight = _tag_list(weight if isinstance(weight, (list, tuple)) else [weight])
    weight_scale = list(weight_scale) if isinstance(weight_scale, (list, tuple)) else [weight_scale]
    n = weight[0].size(-1)
    if wire_rows:
        out = torch.empty((x.size(0), n + n // 4), dtype=torch.int8, device=x.device)
    else:
        out = torch.empty((x.size(0), n), dtype=out_dtype, device=x.device)
    _lib.call("GroupedMatmulDequant", [x, x_scale, weight, weight_scale, group_list, group_list_type, out])
    return out


def grouped_matmul_int32(x, weight, group_list, group_list_type=0):
    """Raw int32 accumulators [A,N] in logical column order."""
    weight = _tag_list(weight if isinstance(weight, (list, tuple)) else [weight])
    gate_up = bool(getattr(weight[0], "_cam_gate_up", False))
    out = torch.zeros((x.size(0), weight[0].size(-1)), dtype=torch.int32, device=x.device)
    _lib.call("GroupedMatmulInt32", [x, weight, 1 if gate_up else 0, group_list, group_list_type, out])
    return out


# --------------------------------------------------------------------------------------------------
# Block-scaled FP8 (a definition of this library: include/cam_fp8_spec.h; the reference is W8A8 only)
def grouped_matmul_fp8(x, x_scale, weight, weight_scale, group_list, group_list_type=0, out_dtype=torch.float32):
    """x E4M3 [A,K], x_scale uint8 [A,K/128], weight E4M3 [G,K,N] prepacked, weight_scale uint8 [G,K/128,N/128].
    Prepacked with gate_up=True: -> fp32 [A,N/2] = silu(gate) * up, or, with out_dtype=torch.float8_e4m3fn, that
    product quantised in the epilogue -> (E4M3 [A,N/2], uint8 E8M0 scales [A,N/256]);
    else -> out_dtype [A,N] (fp32 sums or bf16)."""
    _tag_list([weight])
    gate_up = bool(getattr(weight, "_cam_gate_up", False))
    n = weight.size(-1)
    out_scale = None
    if gate_up and out_dtype == torch.float8_e4m3fn:
        out = torch.empty((x.size(0), n // 2), dtype=torch.float8_e4m3fn, device=x.device)
        out_scale = torch.empty((x.size(0), n // 256), dtype=torch.uint8, device=x.device)
    elif gate_up:
        out = torch.empty((x.size(0), n // 2), dtype=torch.float32, device=x.device)
    else:
        out = torch.empty((x.size(0), n), dtype=out_dtype, device=x.device)
    _lib.call("GroupedMatmulFp8", [x, x_scale, weight, weight_scale, 1 if gate_up else 0, group_list,
                                   group_list_type, out, out_scale])
    return out if out_scale is None else (out, out_scale)


def quant_rows_fp8(x):
    """fp32 [A,I] -> (E4M3 [A,I], uint8 E8M0 scales [A,I/128])."""
    _require_gpu(x, "x")
    q = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    sc = torch.empty((x.size(0), x.size(1) // 128), dtype=torch.uint8, device=x.device)
    _lib.call("QuantRowsFp8", [x, q, sc])
    return q, sc


def fused_deep_moe_fp8(x, expert_ids, gmm1_weight, gmm1_weight_scale, gmm2_weight, gmm2_weight_scale, expert_scales,
                       x_active_mask=None, moe_expert_num=0):
    """-> [output bf16 [bs,H], expertTokenNums int64 [experts]]."""
    _require_gpu(x, "x")
    _tag_list([gmm1_weight, gmm2_weight])
    bs, h = x.shape
    e = moe_expert_num or gmm1_weight.size(0)
    output = torch.empty((bs, h), dtype=torch.bfloat16, device=x.device)
    etn = torch.empty(e, dtype=torch.int64, device=x.device)
    _lib.call("FusedDeepMoeFp8", [x, expert_ids, gmm1_weight, gmm1_weight_scale, gmm2_weight, gmm2_weight_scale,
                                  expert_scales, x_active_mask, e, output, etn])
    return [output, etn]


def fused_deep_moe(x, expertIds, gmm1PermutedWeight, gmm1PermutedWeightScale, gmm2Weight, gmm2WeightScale,
                   expertScales, expertSmoothScales=None, xActiveMask=None, groupEp="", epRankSize=1, epRankId=0,
                   moeExpertNum=0, sharedExpertNum=1, sharedExpertRankNum=0, quantMode=0, globalBs=0):
    """-> [output bf16 [bs,H], expertTokenNums int64 [local experts]]."""
    _require_gpu(x, "x")
    bs, h = x.shape
    output = torch.empty((bs, h), dtype=x.dtype, device=x.device)
    is_shared = epRankId < sharedExpertRankNum
    local_experts = 1 if is_shared else moeExpertNum // max(epRankSize - sharedExpertRankNum, 1)
    expert_token_nums = torch.empty(local_experts, dtype=torch.int64, device=x.device)
    w1 = _tag_list(gmm1PermutedWeight)
    w2 = _tag_list(gmm2Weight)
    _lib.call("FusedDeepMoe", [x, expertIds, w1, list(gmm1PermutedWeightScale), w2, list(gmm2WeightScale),
                               expertScales, expertSmoothScales, xActiveMask, groupEp, epRankSize, epRankId,
                               moeExpertNum, sharedExpertNum, sharedExpertRankNum, quantMode, globalBs, output,
                               expert_token_nums])
    return [output, expert_token_nums]


# --------------------------------------------------------------------------------------------------
# torch.ops.umdk_cam_op_lib.* with the reference's schemas (pybind.cpp:23-41).
_torch_lib = None


def register_torch_ops():
    """Define `umdk_cam_op_lib` and attach the ROCm implementations (idempotent)."""
    global _torch_lib
    if _torch_lib is not None:
        return _torch_lib
    # The C++ registration (csrc/torch_binding.cpp, built next to the kernel library) when it is there; the
    # Python one below otherwise.  Both define the same schemas and call the same C ABI.
    cpp = os.path.join(os.path.dirname(_lib.LIB_PATH), "libcam_torch_ops.so")
    if os.path.exists(cpp) and os.environ.get("CAM_TORCH_OPS", "cpp") != "python":
        _lib.lib()  # the kernel library first: the operator library links against it
        torch.ops.load_library(cpp)
        _torch_lib = "cpp"
        return _torch_lib
    lib = torch.library.Library("umdk_cam_op_lib", "DEF")
    lib.define("fused_deep_moe(Tensor x, Tensor expertIds, Tensor[] gmm1PermutedWeight, "
               "Tensor[] gmm1PermutedWeightScale, Tensor[] gmm2Weight, Tensor[] gmm2WeightScale, "
               "Tensor expertScales, Tensor? expertSmoothScales, Tensor? xActiveMask, str groupEp, "
               "int epRankSize, int epRankId, int moeExpertNum, int sharedExpertNum, int sharedExpertRankNum, "
               "int quantMode, int globalBs) -> Tensor[]")
    lib.define("get_dispatch_layout(Tensor topk_idx, int num_experts, int num_ranks) -> (Tensor, Tensor, Tensor)")
    lib.define("moe_dispatch_prefill(Tensor x, Tensor topk_idx, Tensor topk_weights, Tensor num_tokens_per_rank, "
               "Tensor is_token_in_rank, Tensor num_tokens_per_expert, int num_worst_tokens, str group_ep, "
               "int rank, int num_ranks) -> (Tensor, Tensor, Tensor, Tensor)")
    lib.define("moe_combine_prefill(Tensor x, Tensor topk_idx, Tensor topk_weights, Tensor src_idx, "
               "Tensor send_head, str group_ep, int rank, int num_ranks) -> Tensor")
    lib.define("moe_dispatch_shmem(Tensor x, Tensor expertIds, Tensor? scales, Tensor? xActiveMask, "
               "int epWorldSize, int epRankId, int moeExpertNum, int tpWorldSize, int tpRankId, "
               "int expertShardType, int sharedExpertNum, int sharedExpertRankNum, int quantMode, int globalBS, "
               "int expertTokenNumsType, int extInfo) -> Tensor[]")
    lib.define("moe_combine_shmem(Tensor expandX, Tensor expertIds, Tensor expandIdx, Tensor epSendCounts, "
               "Tensor expertScales, Tensor? tpSendCounts, Tensor? xActiveMask, Tensor? activationScale, "
               "Tensor? weightScale, Tensor? groupList, Tensor? expandScales, int epWorldSize, int epRankId, "
               "int moeExpertNum, int tpWorldSize, int tpRankId, int expertShardType, int sharedExpertNum, "
               "int sharedExpertRankNum, int globalBS, int commQuantMode, int extInfo, int outDtype, "
               "int groupListType) -> Tensor")

    def _fused(x, expertIds, w1, w1s, w2, w2s, expertScales, smooth, mask, groupEp, epRankSize, epRankId,
               moeExpertNum, sharedExpertNum, sharedExpertRankNum, quantMode, globalBs):
        # The dispatcher hands over fresh tensor objects; the format tag travels in a registry keyed by storage.
        for w in list(w1) + list(w2):
            ref, gate_up = _PACKED.get(w.data_ptr(), (None, False))
            if ref is not None and ref() is not None and getattr(w, "_cam_format", None) is None:
                w._cam_format, w._cam_gate_up = CAM_FORMAT_MFMA_B, gate_up
        return fused_deep_moe(x, expertIds, w1, w1s, w2, w2s, expertScales, smooth, mask, groupEp, epRankSize,
                              epRankId, moeExpertNum, sharedExpertNum, sharedExpertRankNum, quantMode, globalBs)

    def _fused_meta(x, expertIds, w1, w1s, w2, w2s, expertScales, smooth, mask, groupEp, epRankSize, epRankId,
                    moeExpertNum, sharedExpertNum, sharedExpertRankNum, quantMode, globalBs):
        local = 1 if epRankId < sharedExpertRankNum else moeExpertNum // max(epRankSize - sharedExpertRankNum, 1)
        return [x.new_empty(x.shape), expertIds.new_empty((local,), dtype=torch.int64)]

    lib.impl("fused_deep_moe", _fused, "CUDA")
    lib.impl("fused_deep_moe", _fused_meta, "Meta")
    lib.impl("get_dispatch_layout", get_dispatch_layout, "CUDA")
    lib.impl("moe_dispatch_prefill",
             lambda *a: tuple(moe_dispatch_prefill(*a)), "CUDA")
    lib.impl("moe_combine_prefill", moe_combine_prefill, "CUDA")
    lib.impl("moe_dispatch_shmem", moe_dispatch_shmem, "CUDA")
    lib.impl("moe_combine_shmem", moe_combine_shmem, "CUDA")
    _torch_lib = lib
    return lib


# data_ptr -> (weak reference, gate_up) of live tensors produced by prepack_weight, for calls that
# reach this module through the torch dispatcher with fresh tensor objects.
_PACKED = {}
