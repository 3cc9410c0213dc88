/*
 * cam_mi355x.h -- C ABI of the MI355X (gfx950) implementation of CAM's MoE hot path.
 *
 * Drop-in boundary.  The reference's PyTorch binding reaches its kernels through CANN's two-phase
 * "aclnn" C ABI: EXEC_NPU_CMD resolves "aclnn<Op>GetWorkspaceSize" and "aclnn<Op>" with dlsym and
 * calls them with tensors, attributes, then outputs (src/cam/comm_operator/pybind/pytorch_extension/
 * pytorch_npu_helper.hpp:136-151,533-582).  This library exports the same pairs under the prefix
 * "cam" with the same argument order.  Differences, all forced by the platform:
 *   - aclTensor / aclTensorList (opaque CANN handles) become the plain structs camTensor /
 *     camTensorList below; the library never allocates, frees or retains device memory;
 *   - aclrtStream becomes camStream_t, which is a hipStream_t passed as void*;
 *   - aclOpExecutor becomes camOpExecutor: created by phase 1, consumed and freed by phase 2
 *     (single use, any thread).  camDestroyExecutor() frees one that will not be run.
 * Phase 1 validates everything on the host and never touches the GPU.  Phase 2 only enqueues kernels
 * on the given stream: no allocation, no synchronisation, no host read of device data.
 * Every function returns 0 on success and a CAM_ERR_* code otherwise; camGetRecentErrMsg() returns
 * the calling thread's last message (the counterpart of aclGetRecentErrMsg).
 *
 * One GPU: epWorldSize / numRanks > 1 is accepted where the arithmetic is rank-local
 * (camDispatchLayout) and refused with CAM_ERR_UNSUPPORTED where peers would be needed.
 * Limits kept from the reference: hidden size, top-k and expert-count ranges, dtypes and ranks.
 * Limits lifted: tokens per call (reference: 256 fused / 8000 normal), local experts per rank
 * (reference: 24), and epWorldSize >= 2 for the normal ops (1 is allowed here).
 *
 * Paths in comments are relative to the reference tree; AUTOGEN =
 * src/cam/comm_operator/ascend_kernels/pregen/build_out/autogen.
 */
#ifndef CAM_MI355X_H_
#define CAM_MI355X_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CAM_API __attribute__((visibility("default")))

typedef int32_t camStatus;

enum {
    CAM_OK = 0,
    CAM_ERR_NULL = 1,        /* a required pointer is NULL */
    CAM_ERR_DTYPE = 2,       /* wrong element type */
    CAM_ERR_SHAPE = 3,       /* wrong rank / extent / contiguity */
    CAM_ERR_RANGE = 4,       /* attribute outside the supported range */
    CAM_ERR_ALIGN = 5,       /* pointer or extent not aligned as the kernels need */
    CAM_ERR_UNSUPPORTED = 6, /* valid in the reference, not built here (e.g. more than one rank) */
    CAM_ERR_WORKSPACE = 7,   /* workspace NULL or smaller than phase 1 asked for */
    CAM_ERR_EXECUTOR = 8,    /* executor NULL or not produced by the matching phase 1 */
    CAM_ERR_LAUNCH = 9       /* the HIP runtime refused a launch */
};

/* Element types; numbering follows aclDataType so a binding can pass its codes through. */
enum {
    CAM_DT_FLOAT = 0,
    CAM_DT_FLOAT16 = 1,
    CAM_DT_INT8 = 2,
    CAM_DT_INT32 = 3,
    CAM_DT_UINT8 = 4,
    CAM_DT_INT64 = 9,
    CAM_DT_BOOL = 12,
    CAM_DT_BF16 = 27,
    CAM_DT_FLOAT8_E4M3FN = 36      /* OCP FP8 E4M3 (block-scaled FP8 operators only) */
};

/* Storage formats.  CAM_FORMAT_ND is plain row-major.  CAM_FORMAT_MFMA_B is the weight layout
 * produced by camPrepackWeight (this build's counterpart of the reference's FRACTAL_NZ cast,
 * test/cam/ut/fused_deep_moe/test_fused_deep_moe.py:243-246). */
enum {
    CAM_FORMAT_ND = 2,
    CAM_FORMAT_MFMA_B = 100
};

#define CAM_MAX_DIMS 8

typedef struct camTensor {
    void *data;                    /* device pointer */
    int32_t dtype;                 /* CAM_DT_* */
    int32_t ndim;
    int64_t sizes[CAM_MAX_DIMS];
    int64_t strides[CAM_MAX_DIMS]; /* in elements */
    int32_t format;                /* CAM_FORMAT_* */
    int32_t reserved;
} camTensor;

typedef struct camTensorList {
    const camTensor *const *tensors;
    uint64_t count;
} camTensorList;

typedef struct camOpExecutor camOpExecutor;
typedef void *camStream_t; /* hipStream_t */

CAM_API const char *camGetRecentErrMsg(void);
CAM_API camStatus camDestroyExecutor(camOpExecutor *executor);
CAM_API const char *camGetVersion(void);

/* Profiling aid with no counterpart in the reference.  A library built with -DCAM_GEMM_TIMELINE makes the
 * grouped-GEMM kernel stamp every tile of its schedule with the device's wall clock (100 MHz): begin and end in
 * words 6 and 7 of the tile's 8-word record, the workgroup that ran it in the upper 16 bits of word 3, and the ticks
 * from its begin to its first multiply and to the end of its K loop in the upper 16 bits of words 4 and 5.  The
 * schedule is the first region of the workspace of every camGroupedMatmul* operator, so a caller that owns the
 * workspace can read the stamps back after a call.  info[0] = 1 when the stamps are compiled in (0 in a normal
 * build, whose kernel writes nothing to the schedule), info[1] = 32-bit words before the first tile record,
 * info[2] = words per record, info[3] = byte offset of the schedule in those workspaces. */
CAM_API camStatus camGemmTimelineInfo(int32_t info[4]);

/* ------------------------------------------------------------------------------------------------
 * DispatchLayout -- replaces aclnnDispatchLayout (AUTOGEN/aclnn_dispatch_layout.h:32-54).
 * topkIdx int64 [T,K] (int32 also accepted) -> numTokensPerRank int32 [R], numTokensPerExpert
 * int32 [E], isTokenInRank int32 [T,R] (bool/uint8 also accepted).  Ids < 0 are skipped
 * (src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:106); ids >= E, which the reference kernel does not
 * guard against (AK/dispatch_layout/op_kernel/dispatch_layout.h:113-118) and which would index past its
 * count table, are skipped the same way and counted nowhere.  Outputs need not be zeroed by the caller.
 * Limits (AK/dispatch_layout/op_host/dispatch_layout_tiling.cc:43-50): 0 < R <= 384, 0 < K <= 16;
 * E <= 512 here (reference: 384). */
CAM_API camStatus camDispatchLayoutGetWorkspaceSize(const camTensor *topkIdx, int64_t numTokens,
                                                    int64_t numRanks, int64_t numExperts, int64_t numTopk,
                                                    const camTensor *numTokensPerRank,
                                                    const camTensor *numTokensPerExpert,
                                                    const camTensor *isTokenInRank, uint64_t *workspaceSize,
                                                    camOpExecutor **executor);
CAM_API camStatus camDispatchLayout(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                    camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * NotifyDispatch -- replaces aclnnNotifyDispatch (AUTOGEN/aclnn_notify_dispatch.h:35-63).
 * tokenPerExpertData int32 [E] -> sendDataOffset int32 [E] (exclusive prefix sum), sendData int32 [3E]
 * ((count, offset, numTokens) per expert; AK/notify_dispatch/op_kernel/notify_dispatch.h:121-152) and
 * recvData int32 [3E].  With rankSize == 1 the all-to-all is the identity, so recvData == sendData.
 * rankSize > 1 -> CAM_ERR_UNSUPPORTED. */
CAM_API camStatus camNotifyDispatchGetWorkspaceSize(const camTensor *sendData,
                                                    const camTensor *tokenPerExpertData, int64_t sendCount,
                                                    int64_t numTokens, char *commGroup, int64_t rankSize,
                                                    int64_t rankId, int64_t localRankSize,
                                                    int64_t localRankId, const camTensor *sendDataOffset,
                                                    const camTensor *recvData, uint64_t *workspaceSize,
                                                    camOpExecutor **executor);
CAM_API camStatus camNotifyDispatch(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                    camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeDispatchPlan -- replaces the two host loops of the reference binding, which copy the ids and
 * the exchanged counts to the CPU and synchronise twice (src/cam/comm_operator/pybind/
 * moe_dispatch_prefill.cpp:96-112 and :114-149), by one device kernel.
 * topkIdx int64/int32 [T,K] ->
 *   sendTokenIdx int32 [T,K]   rank of (t,k) among earlier flat entries with the same id (-1 if id<0)
 *   numTokensPerExpert int32 [E], sendOffset int32 [E] (exclusive scan), recvOffset int32 [E],
 *   recvCount int32 [E] (inclusive cumsum in (local expert, source rank) order),
 *   numRecvTokensPerExpert int64 [E/R], totalRecvTokens int64 [1],
 *   slotRowOptional int32 [T,K]  output row of (t,k) = offset of its expert + its rank, -1 if the entry is
 *                                skipped: the (token, k) -> row map MoeCombineGather consumes.
 *   Any output except sendTokenIdx may be NULL.  numRanks must be 1.  Ids outside [0, E) are skipped:
 *   negative ones are the reference's marker for a dropped entry (moe_dispatch_prefill.cpp:106); ids >= E,
 *   which the reference does not guard against, would index past every per-expert table. */
CAM_API camStatus camMoeDispatchPlanGetWorkspaceSize(const camTensor *topkIdx, int64_t numExperts,
                                                     int64_t numRanks, int64_t rankId,
                                                     const camTensor *sendTokenIdx,
                                                     const camTensor *numTokensPerExpert,
                                                     const camTensor *sendOffset, const camTensor *recvOffset,
                                                     const camTensor *recvCount,
                                                     const camTensor *numRecvTokensPerExpert,
                                                     const camTensor *totalRecvTokens,
                                                     const camTensor *slotRowOptional,
                                                     uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camMoeDispatchPlan(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                     camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeDispatchPlanNoAlloc -- MoeDispatchPlan in one call that allocates nothing.  It has no counterpart in
 * the reference; it is for callers that cannot allocate device memory at the call site (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): there is no workspace to size and pass and
 * no executor object.  Same arguments, outputs and validation as MoeDispatchPlan, followed by the stream.
 * The plan's scratch (one histogram row per ranking workgroup) lives in a 129 KiB array inside the library's
 * device image; every GPU the library runs on holds its own copy until the process ends.  Limit: at most
 * 131072 (token, k) entries (T*K); more returns CAM_ERR_RANGE.  Every call on a GPU uses that GPU's one
 * array, so calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
 * Nothing in the array has to start at zero.  The call must be made with the target device current.  The first
 * call on a device looks up the array's address in the library's device image (hipGetSymbolAddress): make it
 * once outside any stream capture; every later call on that device only enqueues kernels and may be captured. */
CAM_API camStatus camMoeDispatchPlanNoAlloc(const camTensor *topkIdx, int64_t numExperts, int64_t numRanks,
                                            int64_t rankId, const camTensor *sendTokenIdx,
                                            const camTensor *numTokensPerExpert, const camTensor *sendOffset,
                                            const camTensor *recvOffset, const camTensor *recvCount,
                                            const camTensor *numRecvTokensPerExpert,
                                            const camTensor *totalRecvTokens, const camTensor *slotRowOptional,
                                            camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeDispatchNormal -- replaces aclnnMoeDispatchNormal (AUTOGEN/aclnn_moe_dispatch_normal.h:17-25).
 * x bf16 or fp16 [T,H]; topkIdx int32 [T,K]; sendOffset, recvOffset, recvCount int32 [E]; sendTokenIdx
 * int32 [T,K] -> recvX [A,H] (int8 when quantMode == 2, else x's dtype), recvXScales fp32 [A],
 * assistInfoForCombine int32 [3A] = (srcRank, token, k) per row.
 * Row of (t,k) with e = topkIdx[t,k] >= 0 (AK/moe_dispatch_normal/op_kernel/moe_dispatch_normal.h:
 * 366-372 send side, :501-532 receive side): window row w = sendOffset[e] + sendTokenIdx[t,k];
 * output row = (e ? recvCount[e-1] : 0) + (w - recvOffset[e]).  Rows outside [0,A) are dropped.
 * quantMode 0: copy; 2: per-token dynamic int8, scale = 127/(max|x| + 1e-12), recvXScales = 1/scale
 * (moe_dispatch_normal.h:278-316); 3 (extension): the fused kernel's variant without the epsilon
 * (…/grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:780-818).
 * quantMode 1 (static) -> CAM_ERR_UNSUPPORTED.  epWorldSize must be 1 (reference: >= 2).
 * Limits (AK/moe_dispatch_normal/op_host/moe_dispatch_normal_tiling.cc:87-100): 1024 <= H <= 7168,
 * 0 < K <= 16, 0 < E <= 512.  H must be a multiple of 8. */
CAM_API camStatus camMoeDispatchNormalGetWorkspaceSize(
    const camTensor *x, const camTensor *topkIdx, const camTensor *sendOffset, const camTensor *sendTokenIdx,
    const camTensor *recvOffset, const camTensor *recvCount, char *groupEp, int64_t epWorldSize,
    int64_t epRankId, char *groupTpOptional, int64_t tpWorldSize, int64_t tpRankId, int64_t moeExpertNum,
    int64_t quantMode, int64_t globalBs, const camTensor *recvX, const camTensor *recvXScales,
    const camTensor *assistInfoForCombine, uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camMoeDispatchNormal(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                       camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeDispatchPrefill -- the whole body of the reference's binding-level operator moe_dispatch_prefill
 * (src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:96-192: the CPU ranking loop, the CPU loop over the
 * exchanged counts, two device-to-host copies and the aclnnMoeDispatchNormal call) as one operator with no host
 * round trip for one rank: MoeDispatchPlan's launches and MoeDispatchNormal's back to back on the stream.
 * x bf16/fp16 [T,H]; topkIdx int64/int32 [T,K] -> recvX [A,H] (int8 when quantMode is 2 or 3, else
 * x's dtype), recvXScalesOptional fp32 [A] (required when quantising); quantMode 4, which the reference does
 * not have, gives block-scaled FP8 rows instead (recvX E4M3 [A,H], recvXScales uint8 [A,H/128], cam_fp8_spec.h);
 * expandIdx int32 [3A] = (srcRank,
 * token, k) per row, sendTokenIdx int32 [T,K]; optional slotRow int32 [T,K], numTokensPerExpert int32 [E],
 * sendOffset int32 [E], recvCount int32 [E], numRecvTokensPerExpert int64 [E], totalRecvTokens int64 [1],
 * all exactly as MoeDispatchPlan / MoeDispatchNormal produce them.  Rows outside [0,A) are dropped, so A
 * may be a worst-case bound (T*K) and the true total read later from totalRecvTokens.
 * The workspace may hold anything on first use.  Launches that share a workspace must not overlap. */
CAM_API camStatus camMoeDispatchPrefillGetWorkspaceSize(
    const camTensor *x, const camTensor *topkIdx, int64_t numExperts, int64_t numRanks, int64_t rankId,
    int64_t quantMode, const camTensor *recvX, const camTensor *recvXScalesOptional, const camTensor *expandIdx,
    const camTensor *sendTokenIdx, const camTensor *slotRowOptional, const camTensor *numTokensPerExpertOptional,
    const camTensor *sendOffsetOptional, const camTensor *recvCountOptional,
    const camTensor *numRecvTokensPerExpertOptional, const camTensor *totalRecvTokensOptional,
    uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camMoeDispatchPrefill(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                        camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeCombineNormal -- replaces aclnnMoeCombineNormal (AUTOGEN/aclnn_moe_combine_normal.h:37-65).
 * recvX bf16 or fp16 [A,H]; tokenSrcInfo int32 [3A]; epRecvCounts int32 [E]; recvTopkWeights fp32 [T,K]
 * -> out [T,H] of recvX's type (op_host/moe_combine_normal.cpp:18,49 lists both 16-bit types).
 * out[t] = round(sum over k ascending of float(recvX[row(t,k)]) * w[t,k]), multiply
 * and add rounded separately (AK/moe_combine_normal/op_kernel/moe_combine_normal.h:303-338); row(t,k) is
 * the row whose triple names (t,k) (:232-238).  Slots no row names contribute nothing.  Only the first
 * epRecvCounts[E-1] rows are looked at (:206-207): rows past the receive total were never written.
 * Workspace: T*K int32 (the inverse map). */
CAM_API camStatus camMoeCombineNormalGetWorkspaceSize(
    const camTensor *recvX, const camTensor *tokenSrcInfo, const camTensor *epRecvCounts,
    const camTensor *recvTopkWeights, const camTensor *tpRecvCountsOptional, char *epGroupName,
    int64_t epWorldSize, int64_t epRankId, char *tpGroupNameOptional, int64_t tpWorldSize, int64_t tpRankId,
    int64_t moeExpertNum, int64_t globalBs, const camTensor *out, uint64_t *workspaceSize,
    camOpExecutor **executor);
CAM_API camStatus camMoeCombineNormal(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                      camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeCombineIndex / MoeCombineGather -- the two halves of MoeCombineNormal as operators of their own, for
 * callers that already hold the (token, k) -> row map (slotRow of MoeDispatchPlan / MoeDispatchPrefill) or
 * that combine more than one tensor with the same routing.  No counterpart in the reference, which scatters
 * rows instead of gathering them (AK/moe_combine_normal/op_kernel/moe_combine_normal.h:210-275).
 * MoeCombineIndex:  tokenSrcInfo int32 [3A] -> slotRow int32 [T,K] (entries no row names are left untouched).
 * MoeCombineGather: recvX bf16 [A,H], slotRow int32 [T,K], recvTopkWeights fp32 [T,K] -> out bf16 [T,H].
 *   tokenSrcInfoOptional int32 [3A]: when given, a slotRow entry counts only if the triple of the row it
 *   names points back at that slot, so a slotRow built by MoeCombineIndex needs no initialisation; when NULL,
 *   slotRow is trusted (entries < 0 are skipped), which is what the dispatch operators' slotRow output is for.
 *   epRecvCountsOptional int32 [E]: when given, rows at or past its last element are never read.
 *   Same arithmetic and limits as MoeCombineNormal.
 *   recvX may instead hold rows quantised for the wire, int8 [A, H + H/4] (H = out's columns): H int8 values,
 *   then one 16-bit scale per block of 8 columns -- the int8 communication quantisation of
 *   AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:564-592.  The scales have the type of the rows the wire
 *   rows were made from, and out's type says which that is (bf16, or IEEE fp16).  Each value is rebuilt as
 *   round_to_that_type(float(q) * float(scale)) (:755-773) before it is weighted and summed.
 *   GroupedMatmulDequant writes such rows (from bf16) when its out tensor is int8.
 *   sharedXOptional [T,H] of out's type: the shared expert's output row of every token, added un-weighted to
 *   the fp32 accumulator after the K routed rows and before the one rounding
 *   (FDM/raw_distributed/cam_moe_distribute_combine.h:757-774; AK/moe_combine_shmem/op_kernel/
 *   moe_combine_shmem.h:873-907).  Where that row lives on which rank is the caller's business here. */
CAM_API camStatus camMoeCombineIndexGetWorkspaceSize(const camTensor *tokenSrcInfo, int64_t numRows,
                                                     const camTensor *slotRow, uint64_t *workspaceSize,
                                                     camOpExecutor **executor);
CAM_API camStatus camMoeCombineIndex(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                     camStream_t stream);
CAM_API camStatus camMoeCombineGatherGetWorkspaceSize(const camTensor *recvX, const camTensor *tokenSrcInfoOptional,
                                                      const camTensor *slotRow, const camTensor *epRecvCountsOptional,
                                                      const camTensor *recvTopkWeights,
                                                      const camTensor *sharedXOptional, const camTensor *out,
                                                      uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camMoeCombineGather(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                      camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeDispatchShmem -- replaces aclnnMoeDispatchShmem (AUTOGEN/aclnn_moe_dispatch_shmem.h:46-53), one rank.
 * x bf16/fp16 [bs,H]; expertIds int32 [bs,K]; scalesOptional fp32 [moeExpertNum,H] (per-expert smooth scales);
 * xActiveMaskOptional must be NULL (reserved in the reference) -> expandXOut [A,H] (int8 when quantMode == 2, else
 * x's dtype), dynamicScalesOut fp32 [A] (written when quantising), expandIdxOut int32 [bs*K] = the place of
 * entry (t,k) among the entries of its expert (AK/moe_dispatch_shmem/op_kernel/moe_dispatch_shmem.h:541-548),
 * expertTokenNumsOut int64 [moeExpertNum]: running totals when expertTokenNumsType == 0, per-expert counts when 1
 * (:1022-1051), epRecvCountOut int32 [moeExpertNum]: inclusive running totals in (local expert, source rank)
 * order (:853-856,:927-931); tpRecvCountOut is left untouched (tpWorldSize <= 1).
 * Row of (t,k) with e = expertIds[t,k]: (e ? epRecvCountOut[e-1] : 0) + expandIdxOut[t*K+k]; rows outside [0,A)
 * are dropped, so A may be the worst case bs*K.  Ids outside [0, moeExpertNum) name no expert (expandIdx -1).
 * quantMode 2: every COPY is quantised on its own, xf = float(x) * scales[e][h] when scales are given, then
 * s = 127 / max|xf| (no epsilon, :720), q = int8(rint(xf * s)), dynamicScalesOut = 1/s (:693-733); an all-zero row
 * gives zeros and scale 0.  quantMode 0 copies (scales ignored); 1 (static) -> CAM_ERR_UNSUPPORTED.
 * Limits lifted: the reference accepts only epWorldSize in {8,16,32,64,128,144,256,288} and H == 7168
 * (AK/moe_dispatch_shmem/op_host/moe_dispatch_shmem_tiling.cpp:493-501,548); here epWorldSize must be 1
 * (sharedExpertRankNum 0, tpWorldSize <= 1) and H is a multiple of 8 in [1024, 7168].  extInfo is ignored. */
CAM_API camStatus camMoeDispatchShmemGetWorkspaceSize(
    const camTensor *x, const camTensor *expertIds, const camTensor *scalesOptional,
    const camTensor *xActiveMaskOptional, int64_t epWorldSize, int64_t epRankId, int64_t moeExpertNum,
    int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType, int64_t sharedExpertNum,
    int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs, int64_t expertTokenNumsType, int64_t extInfo,
    const camTensor *expandXOut, const camTensor *dynamicScalesOut, const camTensor *expandIdxOut,
    const camTensor *expertTokenNumsOut, const camTensor *epRecvCountOut, const camTensor *tpRecvCountOut,
    uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camMoeDispatchShmem(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                      camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * MoeCombineShmem -- replaces aclnnMoeCombineShmem (AUTOGEN/aclnn_moe_combine_shmem.h:49-56), one rank.
 * expandX bf16/fp16 [A,H] (the expert outputs, in MoeDispatchShmem's row order); expertIds int32 [bs,K];
 * expandIdx int32 [bs*K] and epSendCounts int32 [moeExpertNum] as MoeDispatchShmem wrote them; expertScales
 * fp32 [bs,K]; the six optional tensors are reserved in the reference and must be NULL -> out [bs,H] of
 * expandX's type: out[t] = round(sum over k ascending of float(row(t,k)) * expertScales[t,k]), multiply and add
 * rounded separately (AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:819-912), row(t,k) located as above
 * (:514-556,:833-837).  commQuantMode 2: every row first takes the int8 wire format of :567-592 (blocks of 8
 * columns, scales of expandX's type) and is rebuilt as :755-773 before it is weighted -- the rounding a row
 * suffers when it crosses ranks; 0: rows are used as they are.  Ids outside [0, moeExpertNum) are skipped.
 * epWorldSize must be 1 (sharedExpertRankNum 0, tpWorldSize <= 1); the shared expert's add-back, which needs a
 * shared-expert rank there, is available as MoeCombineGather's sharedXOptional.
 * Workspace: bs*K int32, plus the wire rows when commQuantMode is 2. */
CAM_API camStatus camMoeCombineShmemGetWorkspaceSize(
    const camTensor *expandX, const camTensor *expertIds, const camTensor *expandIdx, const camTensor *epSendCounts,
    const camTensor *expertScales, const camTensor *tpSendCountsOptional, const camTensor *xActiveMaskOptional,
    const camTensor *activationScaleOptional, const camTensor *weightScaleOptional,
    const camTensor *groupListOptional, const camTensor *expandScalesOptional, int64_t epWorldSize,
    int64_t epRankId, int64_t moeExpertNum, int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType,
    int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int64_t commQuantMode, int64_t extInfo,
    int64_t outDtype, int64_t groupListType, const camTensor *out, uint64_t *workspaceSize,
    camOpExecutor **executor);
CAM_API camStatus camMoeCombineShmem(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                     camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * PrepackWeight -- one-time weight layout conversion, off the timed path; the counterpart of
 * torch_npu.npu_format_cast(w, FRACTAL_NZ) (test/cam/ut/fused_deep_moe/test_fused_deep_moe.py:243-246).
 * src int8 [G,Kd,N] or [Kd,N], row-major -> dst int8, same extents, CAM_FORMAT_MFMA_B.
 * gateUp != 0 pairs column c of the gate half [0,N/2) with column N/2 + c of the up half so that the
 * SwiGLU product can be formed in registers (GMM1); 0 keeps column order (GMM2).
 * Requires Kd % 128 == 0 and N % 64 == 0 (gateUp: N % 128 == 0). */
CAM_API camStatus camPrepackWeightGetWorkspaceSize(const camTensor *src, int64_t gateUp, const camTensor *dst,
                                                   uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camPrepackWeight(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                   camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * GroupedMatmulSwigluQuant -- the GMM1 stage of the fused kernel as an operator of its own
 * (GroupedMatmulSliceMPerTokenDequantSwigluQuantMultiStageWorkspace, FDM/gemm/kernel/
 * grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:355-1718; epilogue
 * FDM/epilogue/block/block_epilogue_per_token_dequant_swiglu.h:164-275; re-quant :160-277).
 * x int8 [A,H]; xScale fp32 [A]; weight list: one [G,H,2I] or G tensors [H,2I], CAM_FORMAT_MFMA_B with
 * gateUp=1; weightScale list fp32 [G,2I] / G x [2I]; groupList int64 [G], cumulative row counts when
 * groupListType == 0, per-expert counts when 1 -> y int8 [A,I], yScale fp32 [A].
 * Workspace holds the fp32 SwiGLU product [A,I] and the tile table. */
CAM_API camStatus camGroupedMatmulSwigluQuantGetWorkspaceSize(
    const camTensor *x, const camTensor *xScale, const camTensorList *weight, const camTensorList *weightScale,
    const camTensor *groupList, int64_t groupListType, const camTensor *y, const camTensor *yScale,
    uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camGroupedMatmulSwigluQuant(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                              camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * GroupedMatmulDequant -- the GMM2 stage (GroupedMatmulSliceMPerTokenDequantMultiStageWorkspace,
 * FDM/gemm/kernel/grouped_matmul_slice_m_per_token_dequant_multistage_workspace.h:24-378; epilogue
 * FDM/epilogue/block/block_epilogue_per_token_dequant.hpp:572-703).
 * x int8 [A,I]; xScale fp32 [A]; weight list [G,I,H] / G x [I,H], CAM_FORMAT_MFMA_B with gateUp=0;
 * weightScale fp32 [G,H] -> out bf16 (or fp16) [A,H] = round((float(acc) * weightScale[g][h]) * xScale[m]).
 * out int8 [A, H + H/4] selects wire rows instead: every bf16 row above is quantised in blocks of 8 columns as
 * AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:567-592 does before a row leaves the rank:
 *   m = max |x| over the block; s = m * (1/127); q = int8(half(x / s)) (both casts round to nearest even);
 *   the row is the H values q followed by the H/8 scales bf16(s); an all-zero block gives q = 0, scale 0
 *   (0/0 in the reference).  The workspace then also holds the bf16 rows. */
CAM_API camStatus camGroupedMatmulDequantGetWorkspaceSize(
    const camTensor *x, const camTensor *xScale, const camTensorList *weight, const camTensorList *weightScale,
    const camTensor *groupList, int64_t groupListType, const camTensor *out, uint64_t *workspaceSize,
    camOpExecutor **executor);
CAM_API camStatus camGroupedMatmulDequant(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                          camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * GroupedMatmulInt32 -- the raw int32 accumulators of either GEMM, before any epilogue; the tile the
 * reference's cube cores hand to its vector cores (…swiglu_quant_multistage_workspace.h:558-632).
 * Exists so that accumulation can be checked bit-for-bit.  gateUp says how `weight` was prepacked;
 * out int32 [A,N] is in logical column order either way. */
CAM_API camStatus camGroupedMatmulInt32GetWorkspaceSize(const camTensor *x, const camTensorList *weight,
                                                        int64_t gateUp, const camTensor *groupList,
                                                        int64_t groupListType, const camTensor *out,
                                                        uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camGroupedMatmulInt32(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                        camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * FusedDeepMoe -- replaces aclnnFusedDeepMoe (AUTOGEN/aclnn_fused_deep_moe.h:19-46).
 * x bf16 or fp16 [bs,H]; expertIds int32 [bs,K]; gmm1PermutedWeight int8 [Epr,H,2I] (or Epr x [H,2I]),
 * CAM_FORMAT_MFMA_B gateUp=1; gmm1PermutedWeightScale fp32 [Epr,2I]; gmm2Weight int8 [Epr,I,H],
 * CAM_FORMAT_MFMA_B gateUp=0; gmm2WeightScale fp32 [Epr,H]; expertScales fp32 [bs,K];
 * expertSmoothScalesOptional must be NULL (the reference stores and never uses it,
 * AK/fused_deep_moe/op_kernel/fused_deep_moe.h:307); xActiveMaskOptional bool [bs], prefix semantics
 * (…swiglu_quant_multistage_workspace.h:647-678) -> output [bs,H] of x's type (the expert rows GMM2 writes
 * and the combined rows take it too), expertTokenNums int64 [Epr].
 * quantMode in [0, 3] is accepted and has no effect, as in the reference (fused_deep_moe.h:148,326).
 * sharedExpertNum must be 1 (AK/fused_deep_moe/op_host/fused_deep_moe_tiling.cpp:345).
 * epRankSize must be 1 and sharedExpertRankNum 0.  Output rows of masked tokens are zero.
 * Limits kept (AK/fused_deep_moe/op_host/fused_deep_moe_tiling.cpp:49-61): 512 <= H <= 7168,
 * 1024 <= 2I <= 6144, K <= 12, moeExpertNum <= 512; H and I multiples of 128. */
CAM_API camStatus camFusedDeepMoeGetWorkspaceSize(
    const camTensor *x, const camTensor *expertIds, const camTensorList *gmm1PermutedWeight,
    const camTensorList *gmm1PermutedWeightScale, const camTensorList *gmm2Weight,
    const camTensorList *gmm2WeightScale, const camTensor *expertScales,
    const camTensor *expertSmoothScalesOptional, const camTensor *xActiveMaskOptional, char *groupEp,
    int64_t epRankSize, int64_t epRankId, int64_t moeExpertNum, int64_t sharedExpertNum,
    int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs, const camTensor *output,
    const camTensor *expertTokenNums, uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camFusedDeepMoe(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                  camStream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Block-scaled FP8 variant of the layer.  No counterpart in the reference, whose fused operator is W8A8 int8
 * only (src/cam/README.md:20-21); the arithmetic is defined in cam_fp8_spec.h: OCP E4M3 values, one E8M0
 * (power-of-two) scale per activation row and 128 columns of K and per 128 x 128 block of a weight, fp32
 * accumulation.  Results are compared with a tolerance (bf16 outputs within 1e-2 relative), not bit for bit;
 * the quantised activations themselves are exact.
 *
 * MoeDispatchPrefill with quantMode 4 produces the quantised rows (recvX E4M3 [A,H], recvXScales uint8 [A,H/128]).
 *
 * GroupedMatmulFp8: x E4M3 [A,K]; xScale uint8 [A,K/128]; weight E4M3 [G,K,N], CAM_FORMAT_MFMA_B (PrepackWeight
 *   with the same gateUp); weightScale uint8 [G,K/128,N/128]; groupList int64 [G] as for the int8 operators.
 *   gateUp == 0: out fp32 [A,N] (the sums) or bf16 [A,N];  gateUp != 0: out fp32 [A,N/2] = silu(gate) * up with
 *   gate = columns [0,N/2) and up = [N/2,N) of the logical weight, as in the int8 layer; or out E4M3 [A,N/2]
 *   with outScaleOptional uint8 [A,N/256]: that product quantised in the GEMM's epilogue, bit-identical to
 *   QuantRowsFp8 applied to the fp32 form (outScaleOptional is NULL for the other outputs).
 * QuantRowsFp8: x fp32 [A,I] -> q E4M3 [A,I], scale uint8 [A,I/128] (the re-quantisation between the two GEMMs).
 * FusedDeepMoeFp8: x bf16 [bs,H]; expertIds int32 [bs,K]; gmm1Weight E4M3 [E,H,2I] (MFMA_B, gateUp=1) with
 *   gmm1WeightScale uint8 [E,H/128,2I/128]; gmm2Weight E4M3 [E,I,H] (MFMA_B, gateUp=0) with gmm2WeightScale
 *   uint8 [E,I/128,H/128]; expertScales fp32 [bs,K]; xActiveMaskOptional as FusedDeepMoe
 *   -> output bf16 [bs,H], expertTokenNums int64 [E].  One rank; 1024 <= H <= 7168, H and I multiples of 128,
 *   K <= 16. */
CAM_API camStatus camGroupedMatmulFp8GetWorkspaceSize(const camTensor *x, const camTensor *xScale,
                                                      const camTensor *weight, const camTensor *weightScale,
                                                      int64_t gateUp, const camTensor *groupList,
                                                      int64_t groupListType, const camTensor *out,
                                                      const camTensor *outScaleOptional,
                                                      uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camGroupedMatmulFp8(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                      camStream_t stream);
CAM_API camStatus camQuantRowsFp8GetWorkspaceSize(const camTensor *x, const camTensor *q, const camTensor *scale,
                                                  uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camQuantRowsFp8(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                  camStream_t stream);
CAM_API camStatus camFusedDeepMoeFp8GetWorkspaceSize(
    const camTensor *x, const camTensor *expertIds, const camTensor *gmm1Weight, const camTensor *gmm1WeightScale,
    const camTensor *gmm2Weight, const camTensor *gmm2WeightScale, const camTensor *expertScales,
    const camTensor *xActiveMaskOptional, int64_t moeExpertNum, const camTensor *output,
    const camTensor *expertTokenNums, uint64_t *workspaceSize, camOpExecutor **executor);
CAM_API camStatus camFusedDeepMoeFp8(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                     camStream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* CAM_MI355X_H_ */
