// Host side of the C ABI declared in include/cam_mi355x.h: argument validation (the counterpart of
// the reference's op_host tiling functions), workspace layout, and the kernel launch sequence of
// every operator.  Phase 1 never touches the GPU; phase 2 only enqueues kernels.
//
// Validation follows (paths relative to the reference tree, AK = src/cam/comm_operator/ascend_kernels):
//   AK/dispatch_layout/op_host/dispatch_layout_tiling.cc:43-50,79-144
//   AK/moe_dispatch_normal/op_host/moe_dispatch_normal_tiling.cc:87-100,129-466
//   AK/moe_combine_normal/op_host/moe_combine_normal_tiling.cc:144-400
//   AK/fused_deep_moe/op_host/fused_deep_moe_tiling.cpp:49-61,83-348
//   src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:44-70
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <functional>
#include <mutex>
#include <new>
#include <string>

#include <hip/hip_runtime.h>

#include "../../include/cam_mi355x.h"
#include "cam_kernels.h"

namespace {

thread_local std::string g_err;

camStatus fail(camStatus code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_err = buf;
    return code;
}

enum OpTag {
    kOpLayout = 0x4c41594f,
    kOpNotify = 0x4e4f5449,
    kOpPlan = 0x504c414e,
    kOpDispatch = 0x44495350,
    kOpPrefill = 0x50524546,
    kOpCombine = 0x434f4d42,
    kOpCombIndex = 0x43494458,
    kOpCombGather = 0x43475448,
    kOpPrepack = 0x5052454b,
    kOpGmm1 = 0x474d4d31,
    kOpGmm2 = 0x474d4d32,
    kOpGmmI32 = 0x474d4d49,
    kOpFused = 0x46555345,
    kOpGmmFp8 = 0x474d4638,
    kOpQuantFp8 = 0x51544638,
    kOpFusedFp8 = 0x46554638,
    kOpDispShmem = 0x4453484d,
    kOpCombShmem = 0x4353484d
};

constexpr uint64_t kAlign = 256;
uint64_t align_up(uint64_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

// Carves consecutive 256-byte aligned regions out of a workspace.
struct Carver {
    uint64_t off = 0;
    uint64_t take(uint64_t bytes)
    {
        uint64_t o = off;
        off += align_up(bytes == 0 ? 1 : bytes);
        return o;
    }
};

bool is_contiguous(const camTensor *t)
{
    int64_t expect = 1;
    for (int d = t->ndim - 1; d >= 0; --d) {
        if (t->sizes[d] != 1 && t->strides[d] != expect) {
            return false;
        }
        expect *= t->sizes[d];
    }
    return true;
}

int64_t numel(const camTensor *t)
{
    int64_t n = 1;
    for (int d = 0; d < t->ndim; ++d) {
        n *= t->sizes[d];
    }
    return n;
}

// Common checks on a tensor argument: present, rank, dtype (any of up to 3), contiguous, data non-null
// unless it is empty.
camStatus check_tensor(const camTensor *t, const char *name, int ndim, int dt0, int dt1 = -1, int dt2 = -1)
{
    if (t == nullptr) {
        return fail(CAM_ERR_NULL, "%s is NULL", name);
    }
    if (t->ndim != ndim) {
        return fail(CAM_ERR_SHAPE, "%s must have %d dimension(s), has %d", name, ndim, t->ndim);
    }
    if (t->dtype != dt0 && t->dtype != dt1 && t->dtype != dt2) {
        return fail(CAM_ERR_DTYPE, "%s has unsupported dtype code %d", name, t->dtype);
    }
    for (int d = 0; d < ndim; ++d) {
        if (t->sizes[d] < 0) {
            return fail(CAM_ERR_SHAPE, "%s has a negative extent", name);
        }
    }
    if (!is_contiguous(t)) {
        return fail(CAM_ERR_SHAPE, "%s must be contiguous", name);
    }
    if (numel(t) > 0 && t->data == nullptr) {
        return fail(CAM_ERR_NULL, "%s has a NULL data pointer", name);
    }
    return CAM_OK;
}

camStatus check_aligned(const camTensor *t, const char *name, uintptr_t a)
{
    if (((uintptr_t)t->data) % a != 0) {
        return fail(CAM_ERR_ALIGN, "%s data pointer must be %zu-byte aligned", name, (size_t)a);
    }
    return CAM_OK;
}

#define CAM_TRY(expr)            \
    do {                         \
        camStatus st_ = (expr);  \
        if (st_ != CAM_OK) {     \
            return st_;          \
        }                        \
    } while (0)

}  // namespace

struct camOpExecutor {
    int tag;
    uint64_t workspace_size;
    std::function<hipError_t(void *, hipStream_t)> run;
};

namespace {

camStatus finish_phase1(int tag, uint64_t ws, std::function<hipError_t(void *, hipStream_t)> run,
                        uint64_t *workspaceSize, camOpExecutor **executor)
{
    if (workspaceSize == nullptr || executor == nullptr) {
        return fail(CAM_ERR_NULL, "workspaceSize / executor output pointer is NULL");
    }
    camOpExecutor *ex = new (std::nothrow) camOpExecutor();
    if (ex == nullptr) {
        return fail(CAM_ERR_EXECUTOR, "out of host memory");
    }
    ex->tag = tag;
    ex->workspace_size = ws;
    ex->run = std::move(run);
    *workspaceSize = ws;
    *executor = ex;
    return CAM_OK;
}

camStatus run_phase2(int tag, const char *op, void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                     camStream_t stream)
{
    if (executor == nullptr) {
        return fail(CAM_ERR_EXECUTOR, "%s: executor is NULL", op);
    }
    if (executor->tag != tag) {
        return fail(CAM_ERR_EXECUTOR, "%s: executor belongs to another operator", op);
    }
    camStatus st = CAM_OK;
    if (executor->workspace_size > 0 && (workspace == nullptr || workspaceSize < executor->workspace_size)) {
        st = fail(CAM_ERR_WORKSPACE, "%s: workspace of %llu bytes required, %llu given", op,
                  (unsigned long long)executor->workspace_size, (unsigned long long)(workspace ? workspaceSize : 0));
    } else if (executor->workspace_size > 0 && ((uintptr_t)workspace) % kAlign != 0) {
        st = fail(CAM_ERR_ALIGN, "%s: workspace must be %llu-byte aligned", op, (unsigned long long)kAlign);
    } else {
        hipError_t e = executor->run(workspace, (hipStream_t)stream);
        if (e != hipSuccess) {
            st = fail(CAM_ERR_LAUNCH, "%s: %s", op, hipGetErrorString(e));
        }
    }
    delete executor;
    return st;
}

// Resolves a weight / scale tensor-list pair against (G, Kd, N).
struct WeightSet {
    int per_expert = 0;
    const int8_t *w = nullptr;
    const float *s = nullptr;
    cam::WeightPtrs list;
};

camStatus resolve_weights(const camTensorList *wl, const camTensorList *sl, const char *wname, int64_t G,
                          int64_t Kd, int64_t N, bool need_scale, WeightSet *out)
{
    if (wl == nullptr || wl->tensors == nullptr || wl->count == 0) {
        return fail(CAM_ERR_NULL, "%s list is NULL or empty", wname);
    }
    if (need_scale && (sl == nullptr || sl->tensors == nullptr || sl->count != wl->count)) {
        return fail(CAM_ERR_SHAPE, "%s scale list must match the weight list length", wname);
    }
    if (wl->count != 1 && (int64_t)wl->count != G) {
        return fail(CAM_ERR_SHAPE, "%s list length must be 1 or the number of local experts (%lld), is %llu",
                    wname, (long long)G, (unsigned long long)wl->count);
    }
    std::memset(&out->list, 0, sizeof(out->list));
    for (uint64_t i = 0; i < wl->count; ++i) {
        const camTensor *w = wl->tensors[i];
        if (w == nullptr) {
            return fail(CAM_ERR_NULL, "%s[%llu] is NULL", wname, (unsigned long long)i);
        }
        if (w->dtype != CAM_DT_INT8) {
            return fail(CAM_ERR_DTYPE, "%s must be int8", wname);
        }
        if (w->format != CAM_FORMAT_MFMA_B) {
            return fail(CAM_ERR_UNSUPPORTED,
                        "%s must be converted once with camPrepackWeight (format CAM_FORMAT_MFMA_B)", wname);
        }
        bool stacked = wl->count == 1 && w->ndim == 3;
        bool single = w->ndim == 2 && (wl->count == (uint64_t)G);
        if (stacked) {
            if (w->sizes[0] != G || w->sizes[1] != Kd || w->sizes[2] != N) {
                return fail(CAM_ERR_SHAPE, "%s must be [%lld,%lld,%lld]", wname, (long long)G, (long long)Kd,
                            (long long)N);
            }
        } else if (single) {
            if (w->sizes[0] != Kd || w->sizes[1] != N) {
                return fail(CAM_ERR_SHAPE, "%s[%llu] must be [%lld,%lld]", wname, (unsigned long long)i,
                            (long long)Kd, (long long)N);
            }
        } else {
            return fail(CAM_ERR_SHAPE, "%s: expected one 3-D tensor or one 2-D tensor per local expert", wname);
        }
        if (w->data == nullptr || ((uintptr_t)w->data) % 16 != 0) {
            return fail(CAM_ERR_ALIGN, "%s data must be non-NULL and 16-byte aligned", wname);
        }
        const camTensor *s = need_scale ? sl->tensors[i] : nullptr;
        if (need_scale) {
            if (s == nullptr || s->data == nullptr) {
                return fail(CAM_ERR_NULL, "%s scale[%llu] is NULL", wname, (unsigned long long)i);
            }
            if (s->dtype != CAM_DT_FLOAT) {
                return fail(CAM_ERR_DTYPE, "%s scale must be float32", wname);
            }
            if (((uintptr_t)s->data) % 16 != 0) {
                return fail(CAM_ERR_ALIGN, "%s scale[%llu] data must be 16-byte aligned", wname,
                            (unsigned long long)i);
            }
            int64_t want = stacked ? G * N : N;
            if (numel(s) != want || !is_contiguous(s)) {
                return fail(CAM_ERR_SHAPE, "%s scale[%llu] must hold %lld contiguous values", wname,
                            (unsigned long long)i, (long long)want);
            }
        }
        if (stacked) {
            out->per_expert = 0;
            out->w = (const int8_t *)w->data;
            out->s = need_scale ? (const float *)s->data : nullptr;
        } else {
            if (G > cam::kMaxListExperts) {
                return fail(CAM_ERR_UNSUPPORTED, "%s: at most %d per-expert tensors; stack them instead", wname,
                            cam::kMaxListExperts);
            }
            out->per_expert = G > 1 || w->ndim == 2;
            out->list.w[i] = (const int8_t *)w->data;
            out->list.s[i] = need_scale ? (const float *)s->data : nullptr;
        }
    }
    return CAM_OK;
}

camStatus check_gemm_dims(const char *op, int64_t Kd, int64_t N, bool gate_up)
{
    if (Kd <= 0 || Kd % 128 != 0) {
        return fail(CAM_ERR_UNSUPPORTED, "%s: reduction length %lld must be a positive multiple of 128", op,
                    (long long)Kd);
    }
    if (N <= 0 || N % (gate_up ? 128 : 64) != 0) {
        return fail(CAM_ERR_UNSUPPORTED, "%s: %lld output columns must be a positive multiple of %d", op,
                    (long long)N, gate_up ? 128 : 64);
    }
    return CAM_OK;
}

// One schedule for a GEMM of N packed columns over `rows` rows of G experts, carved out of a workspace.
cam::SchedSpec sched_spec(int64_t rows, int64_t G, int64_t N, int64_t Kd, bool swiglu)
{
    cam::SchedSpec sp{};
    sp.N = (int)N;
    sp.Kd = (int)Kd;
    sp.swiglu = swiglu ? 1 : 0;
    sp.max_items = cam::sched_max_items(rows, (int)G, (int)N);
    return sp;
}

}  // namespace

extern "C" {

const char *camGetRecentErrMsg(void) { return g_err.c_str(); }

const char *camGetVersion(void) { return "cam-mi355x 0.1 (gfx950)"; }

camStatus camGemmTimelineInfo(int32_t info[4])
{
    if (info == nullptr) {
        return fail(CAM_ERR_NULL, "info is NULL");
    }
#ifdef CAM_GEMM_TIMELINE
    info[0] = 1;
#else
    info[0] = 0;
#endif
    info[1] = cam::kSchedHeader;
    info[2] = (int32_t)(sizeof(cam::SchedItem) / sizeof(int32_t));
    info[3] = 0;  // every camGroupedMatmul* phase 1 carves its schedule first
    return CAM_OK;
}

camStatus camDestroyExecutor(camOpExecutor *executor)
{
    delete executor;
    return CAM_OK;
}

// ------------------------------------------------------------------------------------------------
camStatus camDispatchLayoutGetWorkspaceSize(const camTensor *topkIdx, int64_t numTokens, int64_t numRanks,
                                            int64_t numExperts, int64_t numTopk,
                                            const camTensor *numTokensPerRank,
                                            const camTensor *numTokensPerExpert, const camTensor *isTokenInRank,
                                            uint64_t *workspaceSize, camOpExecutor **executor)
{
    CAM_TRY(check_tensor(topkIdx, "topkIdx", 2, CAM_DT_INT64, CAM_DT_INT32));
    if (numRanks <= 0 || numRanks > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "numRanks %lld outside (0, %d]", (long long)numRanks, cam::kMaxRanks);
    }
    if (numExperts <= 0 || numExperts > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "numExperts %lld outside (0, %d]", (long long)numExperts, cam::kMaxExperts);
    }
    if (numTopk <= 0 || numTopk > cam::kMaxTopk) {
        return fail(CAM_ERR_RANGE, "numTopk %lld outside (0, %d]", (long long)numTopk, cam::kMaxTopk);
    }
    if (numExperts % numRanks != 0) {
        return fail(CAM_ERR_RANGE, "numExperts %lld is not divisible by numRanks %lld", (long long)numExperts,
                    (long long)numRanks);
    }
    if (topkIdx->sizes[0] != numTokens || topkIdx->sizes[1] != numTopk) {
        return fail(CAM_ERR_SHAPE, "topkIdx must be [numTokens, numTopk]");
    }
    if (numTokens < 0 || numTokens * numTopk > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "numTokens * numTopk does not fit 32 bits");
    }
    CAM_TRY(check_tensor(numTokensPerRank, "numTokensPerRank", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(numTokensPerExpert, "numTokensPerExpert", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(isTokenInRank, "isTokenInRank", 2, CAM_DT_INT32, CAM_DT_BOOL, CAM_DT_UINT8));
    if (numTokensPerRank->sizes[0] != numRanks || numTokensPerExpert->sizes[0] != numExperts ||
        isTokenInRank->sizes[0] != numTokens || isTokenInRank->sizes[1] != numRanks) {
        return fail(CAM_ERR_SHAPE, "DispatchLayout outputs must be [R], [E] and [T,R]");
    }
    Carver c;
    const uint64_t o_pos = c.take((uint64_t)numTokens * numTopk * 4);
    const uint64_t o_hist = c.take(cam::plan_workspace_bytes(numTokens, numTopk, (int)numExperts));
    cam::PlanArgs p{};
    p.idx = topkIdx->data;
    p.idx_is64 = topkIdx->dtype == CAM_DT_INT64;
    p.T = (int)numTokens;
    p.K = (int)numTopk;
    p.E = (int)numExperts;
    p.R = (int)numRanks;
    p.cnt = (int32_t *)numTokensPerExpert->data;
    p.per_rank_zero = (int32_t *)numTokensPerRank->data;
    cam::InRankArgs r{};
    r.idx = p.idx;
    r.idx_is64 = p.idx_is64;
    r.T = p.T;
    r.K = p.K;
    r.E = p.E;
    r.R = p.R;
    r.in_rank = isTokenInRank->data;
    r.in_rank_bytes = isTokenInRank->dtype == CAM_DT_INT32 ? 4 : 1;
    r.per_rank = (int32_t *)numTokensPerRank->data;
    auto run = [p, r, o_pos, o_hist](void *ws, hipStream_t s) mutable -> hipError_t {
        p.pos = (int32_t *)((char *)ws + o_pos);
        p.hist_ws = (int32_t *)((char *)ws + o_hist);
        hipError_t e = cam::launch_plan(p, s);
        if (e != hipSuccess) {
            return e;
        }
        return cam::launch_in_rank(r, s);
    };
    return finish_phase1(kOpLayout, c.off, run, workspaceSize, executor);
}

camStatus camDispatchLayout(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpLayout, "camDispatchLayout", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
camStatus camNotifyDispatchGetWorkspaceSize(const camTensor *sendData, const camTensor *tokenPerExpertData,
                                            int64_t sendCount, int64_t numTokens, char *commGroup,
                                            int64_t rankSize, int64_t rankId, int64_t localRankSize,
                                            int64_t localRankId, const camTensor *sendDataOffset,
                                            const camTensor *recvData, uint64_t *workspaceSize,
                                            camOpExecutor **executor)
{
    (void)commGroup;
    (void)localRankSize;
    (void)localRankId;
    CAM_TRY(check_tensor(tokenPerExpertData, "tokenPerExpertData", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(sendData, "sendData", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(sendDataOffset, "sendDataOffset", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(recvData, "recvData", 1, CAM_DT_INT32));
    if (rankSize <= 0 || rankSize > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "rankSize %lld outside (0, %d]", (long long)rankSize, cam::kMaxRanks);
    }
    if (rankId < 0 || rankId >= rankSize) {
        return fail(CAM_ERR_RANGE, "rankId %lld outside [0, rankSize)", (long long)rankId);
    }
    if (rankSize != 1) {
        return fail(CAM_ERR_UNSUPPORTED, "NotifyDispatch: the count exchange across %lld ranks is not built "
                                         "(single-GPU library)", (long long)rankSize);
    }
    const int64_t E = tokenPerExpertData->sizes[0];
    if (E <= 0 || E > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "expert count %lld outside (0, %d]", (long long)E, cam::kMaxExperts);
    }
    if (sendCount != 3 * E) {
        return fail(CAM_ERR_SHAPE, "sendCount must be 3 * experts (%lld), is %lld", (long long)(3 * E),
                    (long long)sendCount);
    }
    if (sendData->sizes[0] < 3 * E || recvData->sizes[0] < 3 * E || sendDataOffset->sizes[0] < E) {
        return fail(CAM_ERR_SHAPE, "sendData/recvData need 3*E and sendDataOffset E int32 elements");
    }
    if (numTokens < 0 || numTokens > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "numTokens out of range");
    }
    const int32_t *cnt = (const int32_t *)tokenPerExpertData->data;
    int32_t *off = (int32_t *)sendDataOffset->data;
    int32_t *sd = (int32_t *)sendData->data;
    int32_t *rd = (int32_t *)recvData->data;
    int e = (int)E;
    int nt = (int)numTokens;
    auto run = [=](void *, hipStream_t s) -> hipError_t { return cam::launch_notify_scan(cnt, e, nt, off, sd, rd, s); };
    return finish_phase1(kOpNotify, 0, run, workspaceSize, executor);
}

camStatus camNotifyDispatch(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpNotify, "camNotifyDispatch", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
namespace {

// Validation shared by the two plan entry points; fills every PlanArgs field except the scratch pointer.
camStatus validate_plan(const camTensor *topkIdx, int64_t numExperts, int64_t numRanks, int64_t rankId,
                        const camTensor *sendTokenIdx, const camTensor *numTokensPerExpert,
                        const camTensor *sendOffset, const camTensor *recvOffset, const camTensor *recvCount,
                        const camTensor *numRecvTokensPerExpert, const camTensor *totalRecvTokens,
                        const camTensor *slotRowOptional, cam::PlanArgs *out)
{
    CAM_TRY(check_tensor(topkIdx, "topkIdx", 2, CAM_DT_INT64, CAM_DT_INT32));
    if (numExperts <= 0 || numExperts > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "numExperts %lld outside (0, %d]", (long long)numExperts, cam::kMaxExperts);
    }
    if (numRanks <= 0 || rankId < 0 || rankId >= numRanks) {
        return fail(CAM_ERR_RANGE, "rank %lld / numRanks %lld invalid", (long long)rankId, (long long)numRanks);
    }
    if (numRanks != 1) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeDispatchPlan: numRanks must be 1 (single-GPU library)");
    }
    const int64_t T = topkIdx->sizes[0], K = topkIdx->sizes[1];
    if (K <= 0 || K > cam::kMaxTopk) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, %d]", (long long)K, cam::kMaxTopk);
    }
    if (T * K > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "numTokens * numTopk does not fit 32 bits");
    }
    CAM_TRY(check_tensor(sendTokenIdx, "sendTokenIdx", 2, CAM_DT_INT32));
    if (sendTokenIdx->sizes[0] != T || sendTokenIdx->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "sendTokenIdx must be [T,K]");
    }
    const camTensor *opt_e[4] = {numTokensPerExpert, sendOffset, recvOffset, recvCount};
    const char *opt_n[4] = {"numTokensPerExpert", "sendOffset", "recvOffset", "recvCount"};
    for (int i = 0; i < 4; ++i) {
        if (opt_e[i] != nullptr) {
            CAM_TRY(check_tensor(opt_e[i], opt_n[i], 1, CAM_DT_INT32));
            if (opt_e[i]->sizes[0] != numExperts) {
                return fail(CAM_ERR_SHAPE, "%s must hold numExperts elements", opt_n[i]);
            }
        }
    }
    if (numRecvTokensPerExpert != nullptr) {
        CAM_TRY(check_tensor(numRecvTokensPerExpert, "numRecvTokensPerExpert", 1, CAM_DT_INT64));
        if (numRecvTokensPerExpert->sizes[0] != numExperts / numRanks) {
            return fail(CAM_ERR_SHAPE, "numRecvTokensPerExpert must hold numExperts / numRanks elements");
        }
    }
    if (totalRecvTokens != nullptr) {
        CAM_TRY(check_tensor(totalRecvTokens, "totalRecvTokens", 1, CAM_DT_INT64));
        if (totalRecvTokens->sizes[0] < 1) {
            return fail(CAM_ERR_SHAPE, "totalRecvTokens must hold one element");
        }
    }
    if (slotRowOptional != nullptr) {
        CAM_TRY(check_tensor(slotRowOptional, "slotRow", 2, CAM_DT_INT32));
        if (slotRowOptional->sizes[0] != T || slotRowOptional->sizes[1] != K) {
            return fail(CAM_ERR_SHAPE, "slotRow must be [T,K]");
        }
    }
    cam::PlanArgs p{};
    p.idx = topkIdx->data;
    p.idx_is64 = topkIdx->dtype == CAM_DT_INT64;
    p.T = (int)T;
    p.K = (int)K;
    p.E = (int)numExperts;
    p.R = 1;
    p.pos = (int32_t *)sendTokenIdx->data;
    p.dst_row = slotRowOptional ? (int32_t *)slotRowOptional->data : nullptr;
    p.cnt = numTokensPerExpert ? (int32_t *)numTokensPerExpert->data : nullptr;
    p.off = sendOffset ? (int32_t *)sendOffset->data : nullptr;
    p.recv_off = recvOffset ? (int32_t *)recvOffset->data : nullptr;
    p.recv_count = recvCount ? (int32_t *)recvCount->data : nullptr;
    p.tokens_per_expert = numRecvTokensPerExpert ? (int64_t *)numRecvTokensPerExpert->data : nullptr;
    p.total = totalRecvTokens ? (int64_t *)totalRecvTokens->data : nullptr;
    *out = p;
    return CAM_OK;
}

}  // namespace

camStatus camMoeDispatchPlanGetWorkspaceSize(const camTensor *topkIdx, int64_t numExperts, int64_t numRanks,
                                             int64_t rankId, const camTensor *sendTokenIdx,
                                             const camTensor *numTokensPerExpert, const camTensor *sendOffset,
                                             const camTensor *recvOffset, const camTensor *recvCount,
                                             const camTensor *numRecvTokensPerExpert,
                                             const camTensor *totalRecvTokens, const camTensor *slotRowOptional,
                                             uint64_t *workspaceSize, camOpExecutor **executor)
{
    cam::PlanArgs p{};
    CAM_TRY(validate_plan(topkIdx, numExperts, numRanks, rankId, sendTokenIdx, numTokensPerExpert, sendOffset,
                          recvOffset, recvCount, numRecvTokensPerExpert, totalRecvTokens, slotRowOptional, &p));
    const uint64_t ws_bytes = align_up(cam::plan_workspace_bytes(p.T, p.K, p.E));
    auto run = [p](void *ws, hipStream_t s) mutable -> hipError_t {
        p.hist_ws = (int32_t *)ws;
        return cam::launch_plan(p, s);
    };
    return finish_phase1(kOpPlan, ws_bytes, run, workspaceSize, executor);
}

camStatus camMoeDispatchPlan(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpPlan, "camMoeDispatchPlan", workspace, workspaceSize, executor, stream);
}

// The plan's scratch (one histogram row per ranking workgroup) as library-owned device memory, for the
// entry point below.  Host code must not use this name as an address: the per-device address comes from
// hipGetSymbolAddress (scratch_on_current_device).
constexpr int64_t kNoAllocMaxEntries = 131072;  // T*K: 64 ranking workgroups of 2048 ids
constexpr size_t kNoAllocScratchBytes = (64 * (size_t)cam::kMaxExperts + 64) * sizeof(int32_t);
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device, resolved once per device.
hipError_t scratch_on_current_device(void **out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        return e;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            return e;
        }
        if (ptr == nullptr) {
            return hipErrorInvalidSymbol;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return hipSuccess;
}

}  // namespace

camStatus camMoeDispatchPlanNoAlloc(const camTensor *topkIdx, int64_t numExperts, int64_t numRanks, int64_t rankId,
                                    const camTensor *sendTokenIdx, const camTensor *numTokensPerExpert,
                                    const camTensor *sendOffset, const camTensor *recvOffset,
                                    const camTensor *recvCount, const camTensor *numRecvTokensPerExpert,
                                    const camTensor *totalRecvTokens, const camTensor *slotRowOptional,
                                    camStream_t stream)
{
    cam::PlanArgs p{};
    CAM_TRY(validate_plan(topkIdx, numExperts, numRanks, rankId, sendTokenIdx, numTokensPerExpert, sendOffset,
                          recvOffset, recvCount, numRecvTokensPerExpert, totalRecvTokens, slotRowOptional, &p));
    const int64_t entries = (int64_t)p.T * p.K;
    if (entries > kNoAllocMaxEntries) {
        return fail(CAM_ERR_RANGE,
                    "MoeDispatchPlanNoAlloc: %lld (token, k) entries exceed the %lld the built-in scratch holds; "
                    "use MoeDispatchPlan with a workspace",
                    (long long)entries, (long long)kNoAllocMaxEntries);
    }
    const uint64_t need = cam::plan_workspace_bytes(p.T, p.K, p.E);
    if (need > kNoAllocScratchBytes) {  // cannot happen within the entry limit; guards a change of the plan's chunking
        return fail(CAM_ERR_RANGE,
                    "MoeDispatchPlanNoAlloc: the plan needs %llu bytes of scratch, the built-in array holds %llu; "
                    "use MoeDispatchPlan with a workspace",
                    (unsigned long long)need, (unsigned long long)kNoAllocScratchBytes);
    }
    void *ptr = nullptr;
    hipError_t e = scratch_on_current_device(&ptr);
    if (e != hipSuccess) {
        return fail(CAM_ERR_LAUNCH, "MoeDispatchPlanNoAlloc: cannot resolve the scratch array: %s",
                    hipGetErrorString(e));
    }
    p.hist_ws = (int32_t *)ptr;
    e = cam::launch_plan(p, (hipStream_t)stream);
    if (e != hipSuccess) {
        return fail(CAM_ERR_LAUNCH, "MoeDispatchPlanNoAlloc: %s", hipGetErrorString(e));
    }
    return CAM_OK;
}

// ------------------------------------------------------------------------------------------------
camStatus camMoeDispatchNormalGetWorkspaceSize(const camTensor *x, const camTensor *topkIdx,
                                               const camTensor *sendOffset, const camTensor *sendTokenIdx,
                                               const camTensor *recvOffset, const camTensor *recvCount,
                                               char *groupEp, int64_t epWorldSize, int64_t epRankId,
                                               char *groupTpOptional, int64_t tpWorldSize, int64_t tpRankId,
                                               int64_t moeExpertNum, int64_t quantMode, int64_t globalBs,
                                               const camTensor *recvX, const camTensor *recvXScales,
                                               const camTensor *assistInfoForCombine, uint64_t *workspaceSize,
                                               camOpExecutor **executor)
{
    (void)groupEp;
    (void)groupTpOptional;
    (void)tpRankId;
    (void)globalBs;
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_BF16, CAM_DT_FLOAT16));
    CAM_TRY(check_tensor(topkIdx, "topkIdx", 2, CAM_DT_INT32));
    if (epWorldSize <= 0 || epWorldSize > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "epWorldSize %lld outside (0, %d]", (long long)epWorldSize, cam::kMaxRanks);
    }
    if (epRankId < 0 || epRankId >= epWorldSize) {
        return fail(CAM_ERR_RANGE, "epRankId %lld outside [0, epWorldSize)", (long long)epRankId);
    }
    if (tpWorldSize < 0 || tpWorldSize > 2) {
        return fail(CAM_ERR_RANGE, "tpWorldSize %lld outside [0, 2]", (long long)tpWorldSize);
    }
    if (moeExpertNum <= 0 || moeExpertNum > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "moeExpertNum %lld outside (0, %d]", (long long)moeExpertNum, cam::kMaxExperts);
    }
    if (moeExpertNum % epWorldSize != 0) {
        return fail(CAM_ERR_RANGE, "moeExpertNum must be divisible by epWorldSize");
    }
    if (quantMode < 0 || quantMode > 3) {
        return fail(CAM_ERR_RANGE, "quantMode %lld outside [0, 3]", (long long)quantMode);
    }
    if (quantMode == 1) {
        return fail(CAM_ERR_UNSUPPORTED, "quantMode 1 (static quantisation) is not built");
    }
    if (epWorldSize != 1) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeDispatchNormal: epWorldSize must be 1 (single-GPU library)");
    }
    const int64_t T = x->sizes[0], H = x->sizes[1], K = topkIdx->sizes[1];
    if (T < 1) {
        return fail(CAM_ERR_RANGE, "batch size must be at least 1");
    }
    if (H < 1024 || H > 7168) {
        return fail(CAM_ERR_RANGE, "hidden size %lld outside [1024, 7168]", (long long)H);
    }
    if (H % 8 != 0) {
        return fail(CAM_ERR_ALIGN, "hidden size %lld must be a multiple of 8", (long long)H);
    }
    if (topkIdx->sizes[0] != T) {
        return fail(CAM_ERR_SHAPE, "x and topkIdx must agree on dimension 0");
    }
    if (K <= 0 || K > cam::kMaxTopk || K > moeExpertNum) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, min(%d, moeExpertNum)]", (long long)K, cam::kMaxTopk);
    }
    if (T * K > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "tokens * top-k does not fit 32 bits");
    }
    CAM_TRY(check_tensor(sendOffset, "sendOffset", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(recvOffset, "recvOffset", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(recvCount, "recvCount", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(sendTokenIdx, "sendTokenIdx", 2, CAM_DT_INT32));
    if (sendOffset->sizes[0] != moeExpertNum || recvOffset->sizes[0] != moeExpertNum ||
        recvCount->sizes[0] != moeExpertNum) {
        return fail(CAM_ERR_SHAPE, "sendOffset, recvOffset and recvCount must hold moeExpertNum elements");
    }
    if (sendTokenIdx->sizes[0] != T || sendTokenIdx->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "sendTokenIdx must be [T,K]");
    }
    const bool quant = quantMode != 0;
    CAM_TRY(check_tensor(recvX, "recvX", 2, quant ? CAM_DT_INT8 : x->dtype));
    if (recvX->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "recvX dimension 1 must equal the hidden size");
    }
    const int64_t A = recvX->sizes[0];
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_aligned(recvX, "recvX", 16));
    if (quant) {
        CAM_TRY(check_tensor(recvXScales, "recvXScales", 1, CAM_DT_FLOAT));
        if (recvXScales->sizes[0] < A) {
            return fail(CAM_ERR_SHAPE, "recvXScales must hold one value per recvX row");
        }
    }
    CAM_TRY(check_tensor(assistInfoForCombine, "assistInfoForCombine", 1, CAM_DT_INT32));
    if (assistInfoForCombine->sizes[0] < 3 * A) {
        return fail(CAM_ERR_SHAPE, "assistInfoForCombine must hold 3 values per recvX row");
    }
    cam::DispatchArgs d{};
    d.x = (const uint16_t *)x->data;
    d.idx = (const int32_t *)topkIdx->data;
    d.send_offset = (const int32_t *)sendOffset->data;
    d.send_token_idx = (const int32_t *)sendTokenIdx->data;
    d.recv_offset = (const int32_t *)recvOffset->data;
    d.recv_count = (const int32_t *)recvCount->data;
    d.T = (int)T;
    d.K = (int)K;
    d.H = (int)H;
    d.E = (int)moeExpertNum;
    d.A = A;
    d.quant = quantMode == 0 ? 0 : (quantMode == 2 ? 1 : 2);
    d.x_is_fp16 = x->dtype == CAM_DT_FLOAT16;
    d.out = recvX->data;
    d.scales = quant ? (float *)recvXScales->data : nullptr;
    d.src_info = (int32_t *)assistInfoForCombine->data;
    d.src_rank = (int)epRankId;
    auto run = [d](void *, hipStream_t s) -> hipError_t { return cam::launch_dispatch(d, s); };
    return finish_phase1(kOpDispatch, 0, run, workspaceSize, executor);
}

camStatus camMoeDispatchNormal(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                               camStream_t stream)
{
    return run_phase2(kOpDispatch, "camMoeDispatchNormal", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
camStatus camMoeDispatchPrefillGetWorkspaceSize(const camTensor *x, const camTensor *topkIdx, int64_t numExperts,
                                                int64_t numRanks, int64_t rankId, int64_t quantMode,
                                                const camTensor *recvX, const camTensor *recvXScalesOptional,
                                                const camTensor *expandIdx, const camTensor *sendTokenIdx,
                                                const camTensor *slotRowOptional,
                                                const camTensor *numTokensPerExpertOptional,
                                                const camTensor *sendOffsetOptional,
                                                const camTensor *recvCountOptional,
                                                const camTensor *numRecvTokensPerExpertOptional,
                                                const camTensor *totalRecvTokensOptional, uint64_t *workspaceSize,
                                                camOpExecutor **executor)
{
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_BF16, CAM_DT_FLOAT16));
    CAM_TRY(check_tensor(topkIdx, "topkIdx", 2, CAM_DT_INT64, CAM_DT_INT32));
    if (numExperts <= 0 || numExperts > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "numExperts %lld outside (0, %d]", (long long)numExperts, cam::kMaxExperts);
    }
    if (numRanks <= 0 || rankId < 0 || rankId >= numRanks) {
        return fail(CAM_ERR_RANGE, "rank %lld / numRanks %lld invalid", (long long)rankId, (long long)numRanks);
    }
    if (numRanks != 1) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeDispatchPrefill: numRanks must be 1 (single-GPU library)");
    }
    // quantMode 4 is this library's block-scaled FP8 (include/cam_fp8_spec.h); 0..3 are the reference's values
    if (quantMode < 0 || quantMode > 4) {
        return fail(CAM_ERR_RANGE, "quantMode %lld outside [0, 4]", (long long)quantMode);
    }
    if (quantMode == 1) {
        return fail(CAM_ERR_UNSUPPORTED, "quantMode 1 (static quantisation) is not built");
    }
    const int64_t T = x->sizes[0], H = x->sizes[1], K = topkIdx->sizes[1];
    if (T < 1) {
        return fail(CAM_ERR_RANGE, "batch size must be at least 1");
    }
    if (H < 1024 || H > 7168) {
        return fail(CAM_ERR_RANGE, "hidden size %lld outside [1024, 7168]", (long long)H);
    }
    if (H % 8 != 0) {
        return fail(CAM_ERR_ALIGN, "hidden size %lld must be a multiple of 8", (long long)H);
    }
    if (topkIdx->sizes[0] != T) {
        return fail(CAM_ERR_SHAPE, "x and topkIdx must agree on dimension 0");
    }
    if (K <= 0 || K > cam::kMaxTopk || K > numExperts) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, min(%d, numExperts)]", (long long)K, cam::kMaxTopk);
    }
    if (T * K > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "tokens * top-k does not fit 32 bits");
    }
    const bool quant = quantMode != 0;
    const bool fp8 = quantMode == 4;
    if (fp8 && H % 128 != 0) {
        return fail(CAM_ERR_ALIGN, "FP8 block scales need a hidden size that is a multiple of 128");
    }
    if (fp8) {
        CAM_TRY(check_tensor(recvX, "recvX", 2, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    } else {
        CAM_TRY(check_tensor(recvX, "recvX", 2, quant ? CAM_DT_INT8 : x->dtype));
    }
    if (recvX->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "recvX dimension 1 must equal the hidden size");
    }
    const int64_t A = recvX->sizes[0];
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_aligned(recvX, "recvX", 16));
    if (fp8) {
        CAM_TRY(check_tensor(recvXScalesOptional, "recvXScales", 2, CAM_DT_UINT8));
        if (recvXScalesOptional->sizes[0] < A || recvXScalesOptional->sizes[1] != H / 128) {
            return fail(CAM_ERR_SHAPE, "recvXScales must be uint8 [rows, H/128] (E8M0)");
        }
    } else if (quant) {
        CAM_TRY(check_tensor(recvXScalesOptional, "recvXScales", 1, CAM_DT_FLOAT));
        if (recvXScalesOptional->sizes[0] < A) {
            return fail(CAM_ERR_SHAPE, "recvXScales must hold one value per recvX row");
        }
    }
    CAM_TRY(check_tensor(expandIdx, "expandIdx", 1, CAM_DT_INT32));
    if (expandIdx->sizes[0] < 3 * A) {
        return fail(CAM_ERR_SHAPE, "expandIdx must hold 3 values per recvX row");
    }
    CAM_TRY(check_tensor(sendTokenIdx, "sendTokenIdx", 2, CAM_DT_INT32));
    if (sendTokenIdx->sizes[0] != T || sendTokenIdx->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "sendTokenIdx must be [T,K]");
    }
    if (slotRowOptional != nullptr) {
        CAM_TRY(check_tensor(slotRowOptional, "slotRow", 2, CAM_DT_INT32));
        if (slotRowOptional->sizes[0] != T || slotRowOptional->sizes[1] != K) {
            return fail(CAM_ERR_SHAPE, "slotRow must be [T,K]");
        }
    }
    const camTensor *opt_e[3] = {numTokensPerExpertOptional, sendOffsetOptional, recvCountOptional};
    const char *opt_n[3] = {"numTokensPerExpert", "sendOffset", "recvCount"};
    for (int i = 0; i < 3; ++i) {
        if (opt_e[i] != nullptr) {
            CAM_TRY(check_tensor(opt_e[i], opt_n[i], 1, CAM_DT_INT32));
            if (opt_e[i]->sizes[0] != numExperts) {
                return fail(CAM_ERR_SHAPE, "%s must hold numExperts elements", opt_n[i]);
            }
        }
    }
    if (numRecvTokensPerExpertOptional != nullptr) {
        CAM_TRY(check_tensor(numRecvTokensPerExpertOptional, "numRecvTokensPerExpert", 1, CAM_DT_INT64));
        if (numRecvTokensPerExpertOptional->sizes[0] != numExperts / numRanks) {
            return fail(CAM_ERR_SHAPE, "numRecvTokensPerExpert must hold numExperts / numRanks elements");
        }
    }
    if (totalRecvTokensOptional != nullptr) {
        CAM_TRY(check_tensor(totalRecvTokensOptional, "totalRecvTokens", 1, CAM_DT_INT64));
        if (totalRecvTokensOptional->sizes[0] < 1) {
            return fail(CAM_ERR_SHAPE, "totalRecvTokens must hold one element");
        }
    }
    cam::PlanArgs p{};
    p.idx = topkIdx->data;
    p.idx_is64 = topkIdx->dtype == CAM_DT_INT64;
    p.T = (int)T;
    p.K = (int)K;
    p.E = (int)numExperts;
    p.R = 1;
    p.pos = (int32_t *)sendTokenIdx->data;
    p.dst_row = slotRowOptional ? (int32_t *)slotRowOptional->data : nullptr;
    p.cnt = numTokensPerExpertOptional ? (int32_t *)numTokensPerExpertOptional->data : nullptr;
    p.off = sendOffsetOptional ? (int32_t *)sendOffsetOptional->data : nullptr;
    p.recv_count = recvCountOptional ? (int32_t *)recvCountOptional->data : nullptr;
    p.tokens_per_expert =
        numRecvTokensPerExpertOptional ? (int64_t *)numRecvTokensPerExpertOptional->data : nullptr;
    p.total = totalRecvTokensOptional ? (int64_t *)totalRecvTokensOptional->data : nullptr;
    cam::DispatchArgs d{};
    d.x = (const uint16_t *)x->data;
    d.x_is_fp16 = x->dtype == CAM_DT_FLOAT16;
    d.T = (int)T;
    d.K = (int)K;
    d.H = (int)H;
    d.E = (int)numExperts;
    d.A = A;
    d.quant = quantMode == 0 ? 0 : (quantMode == 2 ? 1 : (quantMode == 4 ? 3 : 2));
    d.out = recvX->data;
    d.scales = quant ? (float *)recvXScalesOptional->data : nullptr;
    d.src_info = (int32_t *)expandIdx->data;
    d.src_rank = (int)rankId;
    // The plan's launches, then the permute's.
    Carver c;
    const uint64_t o_hist = c.take(cam::plan_workspace_bytes(T, K, (int)numExperts));
    const uint64_t o_row = c.take((uint64_t)T * K * 4);
    auto run = [p, d, o_hist, o_row](void *ws, hipStream_t s) mutable -> hipError_t {
        p.hist_ws = (int32_t *)((char *)ws + o_hist);
        if (p.dst_row == nullptr) {
            p.dst_row = (int32_t *)((char *)ws + o_row);
        }
        hipError_t e = cam::launch_plan(p, s);
        if (e != hipSuccess) {
            return e;
        }
        d.dst_row = p.dst_row;
        return cam::launch_dispatch(d, s);
    };
    return finish_phase1(kOpPrefill, c.off, run, workspaceSize, executor);
}

camStatus camMoeDispatchPrefill(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                camStream_t stream)
{
    return run_phase2(kOpPrefill, "camMoeDispatchPrefill", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
camStatus camMoeCombineNormalGetWorkspaceSize(const camTensor *recvX, const camTensor *tokenSrcInfo,
                                              const camTensor *epRecvCounts, const camTensor *recvTopkWeights,
                                              const camTensor *tpRecvCountsOptional, char *epGroupName,
                                              int64_t epWorldSize, int64_t epRankId, char *tpGroupNameOptional,
                                              int64_t tpWorldSize, int64_t tpRankId, int64_t moeExpertNum,
                                              int64_t globalBs, const camTensor *out, uint64_t *workspaceSize,
                                              camOpExecutor **executor)
{
    (void)tpRecvCountsOptional;
    (void)epGroupName;
    (void)tpGroupNameOptional;
    (void)tpRankId;
    // bf16 or fp16 rows (AK/moe_combine_normal/op_host/moe_combine_normal.cpp:18,49); out has the same type
    CAM_TRY(check_tensor(recvX, "recvX", 2, CAM_DT_BF16, CAM_DT_FLOAT16));
    CAM_TRY(check_tensor(tokenSrcInfo, "tokenSrcInfo", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(epRecvCounts, "epRecvCounts", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(recvTopkWeights, "recvTopkWeights", 2, CAM_DT_FLOAT));
    CAM_TRY(check_tensor(out, "out", 2, recvX->dtype));
    if (epWorldSize <= 0 || epWorldSize > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "epWorldSize %lld outside (0, %d]", (long long)epWorldSize, cam::kMaxRanks);
    }
    if (epRankId < 0 || epRankId >= epWorldSize) {
        return fail(CAM_ERR_RANGE, "epRankId %lld outside [0, epWorldSize)", (long long)epRankId);
    }
    if (tpWorldSize < 0 || tpWorldSize > 2) {
        return fail(CAM_ERR_RANGE, "tpWorldSize %lld outside [0, 2]", (long long)tpWorldSize);
    }
    if (moeExpertNum <= 0 || moeExpertNum > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "moeExpertNum %lld outside (0, %d]", (long long)moeExpertNum, cam::kMaxExperts);
    }
    if (epWorldSize != 1) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeCombineNormal: epWorldSize must be 1 (single-GPU library)");
    }
    const int64_t A = recvX->sizes[0], H = recvX->sizes[1];
    const int64_t T = recvTopkWeights->sizes[0], K = recvTopkWeights->sizes[1];
    if (H < 1024 || H > 7168) {
        return fail(CAM_ERR_RANGE, "hidden size %lld outside [1024, 7168]", (long long)H);
    }
    if (H % 8 != 0) {
        return fail(CAM_ERR_ALIGN, "hidden size %lld must be a multiple of 8", (long long)H);
    }
    if (K <= 0 || K > cam::kMaxTopk) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, %d]", (long long)K, cam::kMaxTopk);
    }
    if (T < 1) {
        return fail(CAM_ERR_RANGE, "batch size must be at least 1");
    }
    if (globalBs != 0 && (globalBs < epWorldSize * T || globalBs % epWorldSize != 0)) {
        return fail(CAM_ERR_RANGE, "globalBs must be 0 or a multiple of epWorldSize that is >= epWorldSize * bs");
    }
    if (out->sizes[0] != T || out->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "out must be [bs, H]");
    }
    if (tokenSrcInfo->sizes[0] < 3 * A) {
        return fail(CAM_ERR_SHAPE, "tokenSrcInfo must hold 3 values per recvX row");
    }
    if (epRecvCounts->sizes[0] != moeExpertNum) {
        return fail(CAM_ERR_SHAPE, "epRecvCounts must hold moeExpertNum elements");
    }
    if (T * K > 0x7fffffffll || A > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "row counts do not fit 32 bits");
    }
    CAM_TRY(check_aligned(recvX, "recvX", 16));
    CAM_TRY(check_aligned(out, "out", 16));
    Carver c;
    const uint64_t o_slot = c.take((uint64_t)T * K * 4);
    cam::CombineArgs g{};
    g.y = (const uint16_t *)recvX->data;
    g.src_info = (const int32_t *)tokenSrcInfo->data;
    g.w = (const float *)recvTopkWeights->data;
    g.T = (int)T;
    g.K = (int)K;
    g.H = (int)H;
    g.A = A;
    g.act_fp16 = recvX->dtype == CAM_DT_FLOAT16;
    // Rows at or past the receive total were never written (moe_combine_normal.h:206-207 bounds its loop the same way).
    g.row_limit = (const int32_t *)epRecvCounts->data + (moeExpertNum - 1);
    g.out = (uint16_t *)out->data;
    auto run = [g, o_slot](void *ws, hipStream_t s) mutable -> hipError_t {
        int32_t *slot = (int32_t *)((char *)ws + o_slot);
        hipError_t e = cam::launch_invert_src_info(g.src_info, g.A, g.row_limit, g.T, g.K, slot, s);
        if (e != hipSuccess) {
            return e;
        }
        g.slot_row = slot;
        return cam::launch_combine(g, s);
    };
    return finish_phase1(kOpCombine, c.off, run, workspaceSize, executor);
}

camStatus camMoeCombineNormal(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpCombine, "camMoeCombineNormal", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
camStatus camMoeCombineIndexGetWorkspaceSize(const camTensor *tokenSrcInfo, int64_t numRows, const camTensor *slotRow,
                                             uint64_t *workspaceSize, camOpExecutor **executor)
{
    CAM_TRY(check_tensor(tokenSrcInfo, "tokenSrcInfo", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(slotRow, "slotRow", 2, CAM_DT_INT32));
    if (numRows < 0 || numRows > 0x7fffffffll || tokenSrcInfo->sizes[0] < 3 * numRows) {
        return fail(CAM_ERR_SHAPE, "tokenSrcInfo must hold 3 values for each of the %lld rows", (long long)numRows);
    }
    const int64_t T = slotRow->sizes[0], K = slotRow->sizes[1];
    if (K <= 0 || K > cam::kMaxTopk || T * K > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "slotRow must be [T,K] with 0 < K <= %d", cam::kMaxTopk);
    }
    const int32_t *src = (const int32_t *)tokenSrcInfo->data;
    int32_t *slot = (int32_t *)slotRow->data;
    const int iT = (int)T, iK = (int)K;
    auto run = [=](void *, hipStream_t s) -> hipError_t {
        return cam::launch_invert_src_info(src, numRows, nullptr, iT, iK, slot, s);
    };
    return finish_phase1(kOpCombIndex, 0, run, workspaceSize, executor);
}

camStatus camMoeCombineIndex(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpCombIndex, "camMoeCombineIndex", workspace, workspaceSize, executor, stream);
}

camStatus camMoeCombineGatherGetWorkspaceSize(const camTensor *recvX, const camTensor *tokenSrcInfoOptional,
                                              const camTensor *slotRow, const camTensor *epRecvCountsOptional,
                                              const camTensor *recvTopkWeights, const camTensor *sharedXOptional,
                                              const camTensor *out, uint64_t *workspaceSize,
                                              camOpExecutor **executor)
{
    // recvX: bf16 rows [A,H], or rows quantised for the wire, int8 [A, H + H/4] (the int8 communication
    // quantisation of AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:564-592, dequantised as :755-773).
    CAM_TRY(check_tensor(recvX, "recvX", 2, CAM_DT_BF16, CAM_DT_FLOAT16, CAM_DT_INT8));
    CAM_TRY(check_tensor(slotRow, "slotRow", 2, CAM_DT_INT32));
    CAM_TRY(check_tensor(recvTopkWeights, "recvTopkWeights", 2, CAM_DT_FLOAT));
    const bool wire = recvX->dtype == CAM_DT_INT8;
    // (wire rows carry block scales of the type they were quantised from, which is the type they come back as)
    CAM_TRY(check_tensor(out, "out", 2, wire ? (out->dtype == CAM_DT_FLOAT16 ? CAM_DT_FLOAT16 : CAM_DT_BF16) : recvX->dtype));
    const int64_t A = recvX->sizes[0], H = out->sizes[1];
    const int64_t T = recvTopkWeights->sizes[0], K = recvTopkWeights->sizes[1];
    if (recvX->sizes[1] != (wire ? H + H / 4 : H)) {
        return fail(CAM_ERR_SHAPE, "recvX must be [A,H] bf16 or [A, H + H/4] int8 wire rows, H = out's columns");
    }
    if (H < 1024 || H > 7168) {
        return fail(CAM_ERR_RANGE, "hidden size %lld outside [1024, 7168]", (long long)H);
    }
    if (H % 8 != 0) {
        return fail(CAM_ERR_ALIGN, "hidden size %lld must be a multiple of 8", (long long)H);
    }
    if (K <= 0 || K > cam::kMaxTopk || T < 1) {
        return fail(CAM_ERR_RANGE, "recvTopkWeights must be [T,K] with T >= 1 and 0 < K <= %d", cam::kMaxTopk);
    }
    if (slotRow->sizes[0] != T || slotRow->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "slotRow must be [T,K]");
    }
    if (out->sizes[0] != T || out->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "out must be [T,H]");
    }
    if (tokenSrcInfoOptional != nullptr) {
        CAM_TRY(check_tensor(tokenSrcInfoOptional, "tokenSrcInfo", 1, CAM_DT_INT32));
        if (tokenSrcInfoOptional->sizes[0] < 3 * A) {
            return fail(CAM_ERR_SHAPE, "tokenSrcInfo must hold 3 values per recvX row");
        }
    }
    if (epRecvCountsOptional != nullptr) {
        CAM_TRY(check_tensor(epRecvCountsOptional, "epRecvCounts", 1, CAM_DT_INT32));
        if (epRecvCountsOptional->sizes[0] < 1) {
            return fail(CAM_ERR_SHAPE, "epRecvCounts must hold at least one element");
        }
    }
    if (T * K > 0x7fffffffll || A > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "row counts do not fit 32 bits");
    }
    CAM_TRY(check_aligned(recvX, "recvX", 16));
    CAM_TRY(check_aligned(out, "out", 16));
    if (sharedXOptional != nullptr) {
        // the shared expert's output rows, one per token, in the output's type; added un-weighted after the routed
        // rows (FDM/raw_distributed/cam_moe_distribute_combine.h:757-774)
        CAM_TRY(check_tensor(sharedXOptional, "sharedX", 2, out->dtype));
        if (sharedXOptional->sizes[0] != T || sharedXOptional->sizes[1] != H) {
            return fail(CAM_ERR_SHAPE, "sharedX must be [T,H] like out");
        }
        CAM_TRY(check_aligned(sharedXOptional, "sharedX", 16));
    }
    cam::CombineArgs g{};
    g.shared = sharedXOptional ? (const uint16_t *)sharedXOptional->data : nullptr;
    g.y = (const uint16_t *)recvX->data;
    g.slot_row = (const int32_t *)slotRow->data;
    g.src_info = tokenSrcInfoOptional ? (const int32_t *)tokenSrcInfoOptional->data : nullptr;
    g.row_limit = epRecvCountsOptional
                      ? (const int32_t *)epRecvCountsOptional->data + (epRecvCountsOptional->sizes[0] - 1)
                      : nullptr;
    g.w = (const float *)recvTopkWeights->data;
    g.T = (int)T;
    g.K = (int)K;
    g.H = (int)H;
    g.A = A;
    g.wire_rows = wire ? 1 : 0;
    g.act_fp16 = (wire ? out->dtype : recvX->dtype) == CAM_DT_FLOAT16;
    g.out = (uint16_t *)out->data;
    auto run = [g](void *, hipStream_t s) -> hipError_t { return cam::launch_combine(g, s); };
    return finish_phase1(kOpCombGather, 0, run, workspaceSize, executor);
}

camStatus camMoeCombineGather(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpCombGather, "camMoeCombineGather", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
// The SHMEM operator pair on one rank.  Validation follows AK/moe_dispatch_shmem/op_host/
// moe_dispatch_shmem_tiling.cpp:123-215,365-535 and AK/moe_combine_shmem/op_host/moe_combine_shmem_tiling.cpp:
// 120-200; the limits tied to the transport (epWorldSize in {8,...,288}, H == 7168) are lifted, epWorldSize > 1 is
// refused.
camStatus camMoeDispatchShmemGetWorkspaceSize(const camTensor *x, const camTensor *expertIds,
                                              const camTensor *scalesOptional,
                                              const camTensor *xActiveMaskOptional, int64_t epWorldSize,
                                              int64_t epRankId, int64_t moeExpertNum, int64_t tpWorldSize,
                                              int64_t tpRankId, int64_t expertShardType, int64_t sharedExpertNum,
                                              int64_t sharedExpertRankNum, int64_t quantMode, int64_t globalBs,
                                              int64_t expertTokenNumsType, int64_t extInfo,
                                              const camTensor *expandXOut, const camTensor *dynamicScalesOut,
                                              const camTensor *expandIdxOut, const camTensor *expertTokenNumsOut,
                                              const camTensor *epRecvCountOut, const camTensor *tpRecvCountOut,
                                              uint64_t *workspaceSize, camOpExecutor **executor)
{
    (void)tpRankId;
    (void)sharedExpertNum;
    (void)extInfo;         // the reference's handle of its symmetric heap
    (void)tpRecvCountOut;  // written only when tpWorldSize == 2 (moe_dispatch_shmem.h:1078-1086)
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_BF16, CAM_DT_FLOAT16));
    CAM_TRY(check_tensor(expertIds, "expertIds", 2, CAM_DT_INT32));
    if (epWorldSize <= 0 || epWorldSize > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "epWorldSize %lld outside (0, %d]", (long long)epWorldSize, cam::kMaxRanks);
    }
    if (epRankId < 0 || epRankId >= epWorldSize) {
        return fail(CAM_ERR_RANGE, "epRankId %lld outside [0, epWorldSize)", (long long)epRankId);
    }
    if (moeExpertNum <= 0 || moeExpertNum > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "moeExpertNum %lld outside (0, %d]", (long long)moeExpertNum, cam::kMaxExperts);
    }
    if (tpWorldSize < 0 || tpWorldSize > 2) {
        return fail(CAM_ERR_RANGE, "tpWorldSize %lld outside [0, 2]", (long long)tpWorldSize);
    }
    if (expertShardType != 0) {
        return fail(CAM_ERR_RANGE, "expertShardType must be 0");
    }
    if (sharedExpertRankNum < 0 || sharedExpertRankNum >= epWorldSize) {
        return fail(CAM_ERR_RANGE, "sharedExpertRankNum %lld outside [0, epWorldSize)", (long long)sharedExpertRankNum);
    }
    if (quantMode < 0 || quantMode > 2) {
        return fail(CAM_ERR_RANGE, "quantMode %lld outside [0, 2]", (long long)quantMode);
    }
    if (expertTokenNumsType != 0 && expertTokenNumsType != 1) {
        return fail(CAM_ERR_RANGE, "expertTokenNumsType must be 0 (running totals) or 1 (counts)");
    }
    if (quantMode == 1) {
        return fail(CAM_ERR_UNSUPPORTED, "quantMode 1 (static quantisation) is not built");
    }
    if (epWorldSize != 1 || sharedExpertRankNum != 0 || tpWorldSize > 1) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeDispatchShmem: epWorldSize must be 1, sharedExpertRankNum 0 and "
                                         "tpWorldSize at most 1 (single-GPU library)");
    }
    if (xActiveMaskOptional != nullptr) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeDispatchShmem: xActiveMask is reserved in the reference; pass NULL");
    }
    const int64_t T = x->sizes[0], H = x->sizes[1], K = expertIds->sizes[1];
    if (T < 1) {
        return fail(CAM_ERR_RANGE, "batch size must be at least 1");
    }
    if (H < 1024 || H > 7168 || H % 8 != 0) {
        return fail(CAM_ERR_RANGE, "hidden size %lld must be a multiple of 8 in [1024, 7168]", (long long)H);
    }
    if (expertIds->sizes[0] != T) {
        return fail(CAM_ERR_SHAPE, "x and expertIds must agree on dimension 0");
    }
    if (K <= 0 || K > cam::kMaxTopk || K > moeExpertNum) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, min(%d, moeExpertNum)]", (long long)K, cam::kMaxTopk);
    }
    if (globalBs != 0 && (globalBs < T * epWorldSize || globalBs % epWorldSize != 0)) {
        return fail(CAM_ERR_RANGE, "globalBs must be 0 or a multiple of epWorldSize that is >= epWorldSize * bs");
    }
    if (T * K > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "tokens * top-k does not fit 32 bits");
    }
    const bool quant = quantMode == 2;
    if (scalesOptional != nullptr) {
        CAM_TRY(check_tensor(scalesOptional, "scales", 2, CAM_DT_FLOAT));
        if (scalesOptional->sizes[0] != moeExpertNum || scalesOptional->sizes[1] != H) {
            return fail(CAM_ERR_SHAPE, "scales must be fp32 [moeExpertNum, H]");
        }
        CAM_TRY(check_aligned(scalesOptional, "scales", 16));
    }
    CAM_TRY(check_tensor(expandXOut, "expandXOut", 2, quant ? CAM_DT_INT8 : x->dtype));
    if (expandXOut->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "expandXOut dimension 1 must equal the hidden size");
    }
    const int64_t A = expandXOut->sizes[0];
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_aligned(expandXOut, "expandXOut", 16));
    CAM_TRY(check_tensor(dynamicScalesOut, "dynamicScalesOut", 1, CAM_DT_FLOAT));
    if (quant && dynamicScalesOut->sizes[0] < A) {
        return fail(CAM_ERR_SHAPE, "dynamicScalesOut must hold one value per expandXOut row");
    }
    CAM_TRY(check_tensor(expandIdxOut, "expandIdxOut", 1, CAM_DT_INT32));
    if (expandIdxOut->sizes[0] != T * K) {
        return fail(CAM_ERR_SHAPE, "expandIdxOut must hold bs * K elements");
    }
    CAM_TRY(check_tensor(expertTokenNumsOut, "expertTokenNumsOut", 1, CAM_DT_INT64));
    CAM_TRY(check_tensor(epRecvCountOut, "epRecvCountOut", 1, CAM_DT_INT32));
    if (expertTokenNumsOut->sizes[0] != moeExpertNum || epRecvCountOut->sizes[0] != moeExpertNum) {
        return fail(CAM_ERR_SHAPE, "expertTokenNumsOut and epRecvCountOut must hold one value per local expert");
    }
    cam::PlanArgs p{};
    p.idx = expertIds->data;
    p.idx_is64 = 0;
    p.T = (int)T;
    p.K = (int)K;
    p.E = (int)moeExpertNum;
    p.R = 1;
    p.pos = (int32_t *)expandIdxOut->data;
    p.recv_count = (int32_t *)epRecvCountOut->data;
    if (expertTokenNumsType == 0) {
        p.group_list = (int64_t *)expertTokenNumsOut->data;
    } else {
        p.tokens_per_expert = (int64_t *)expertTokenNumsOut->data;
    }
    cam::DispatchArgs d{};
    d.x = (const uint16_t *)x->data;
    d.x_is_fp16 = x->dtype == CAM_DT_FLOAT16;
    d.idx = (const int32_t *)expertIds->data;
    d.T = (int)T;
    d.K = (int)K;
    d.H = (int)H;
    d.E = (int)moeExpertNum;
    d.A = A;
    d.quant = quant ? 2 : 0;  // the variant without the epsilon (moe_dispatch_shmem.h:720)
    d.out = expandXOut->data;
    d.scales = quant ? (float *)dynamicScalesOut->data : nullptr;
    d.src_rank = (int)epRankId;
    d.smooth = quant && scalesOptional ? (const float *)scalesOptional->data : nullptr;
    Carver c;
    const uint64_t o_hist = c.take(cam::plan_workspace_bytes(T, K, (int)moeExpertNum));
    const uint64_t o_row = c.take((uint64_t)T * K * 4);
    auto run = [p, d, o_hist, o_row](void *ws, hipStream_t s) mutable -> hipError_t {
        p.hist_ws = (int32_t *)((char *)ws + o_hist);
        p.dst_row = (int32_t *)((char *)ws + o_row);
        hipError_t e = cam::launch_plan(p, s);
        if (e != hipSuccess) {
            return e;
        }
        d.dst_row = p.dst_row;
        return cam::launch_dispatch(d, s);
    };
    return finish_phase1(kOpDispShmem, c.off, run, workspaceSize, executor);
}

camStatus camMoeDispatchShmem(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpDispShmem, "camMoeDispatchShmem", workspace, workspaceSize, executor, stream);
}

camStatus camMoeCombineShmemGetWorkspaceSize(
    const camTensor *expandX, const camTensor *expertIds, const camTensor *expandIdx, const camTensor *epSendCounts,
    const camTensor *expertScales, const camTensor *tpSendCountsOptional, const camTensor *xActiveMaskOptional,
    const camTensor *activationScaleOptional, const camTensor *weightScaleOptional,
    const camTensor *groupListOptional, const camTensor *expandScalesOptional, int64_t epWorldSize,
    int64_t epRankId, int64_t moeExpertNum, int64_t tpWorldSize, int64_t tpRankId, int64_t expertShardType,
    int64_t sharedExpertNum, int64_t sharedExpertRankNum, int64_t globalBs, int64_t commQuantMode, int64_t extInfo,
    int64_t outDtype, int64_t groupListType, const camTensor *out, uint64_t *workspaceSize,
    camOpExecutor **executor)
{
    (void)tpSendCountsOptional;
    (void)tpRankId;
    (void)sharedExpertNum;
    (void)extInfo;
    (void)outDtype;
    (void)groupListType;
    if (xActiveMaskOptional != nullptr || activationScaleOptional != nullptr || weightScaleOptional != nullptr ||
        groupListOptional != nullptr || expandScalesOptional != nullptr) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeCombineShmem: xActiveMask, activationScale, weightScale, groupList and "
                                         "expandScales are reserved in the reference; pass NULL");
    }
    CAM_TRY(check_tensor(expandX, "expandX", 2, CAM_DT_BF16, CAM_DT_FLOAT16));
    CAM_TRY(check_tensor(expertIds, "expertIds", 2, CAM_DT_INT32));
    CAM_TRY(check_tensor(expandIdx, "expandIdx", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(epSendCounts, "epSendCounts", 1, CAM_DT_INT32));
    CAM_TRY(check_tensor(expertScales, "expertScales", 2, CAM_DT_FLOAT));
    CAM_TRY(check_tensor(out, "out", 2, expandX->dtype));
    if (epWorldSize <= 0 || epWorldSize > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "epWorldSize %lld outside (0, %d]", (long long)epWorldSize, cam::kMaxRanks);
    }
    if (epRankId < 0 || epRankId >= epWorldSize) {
        return fail(CAM_ERR_RANGE, "epRankId %lld outside [0, epWorldSize)", (long long)epRankId);
    }
    if (moeExpertNum <= 0 || moeExpertNum > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "moeExpertNum %lld outside (0, %d]", (long long)moeExpertNum, cam::kMaxExperts);
    }
    if (tpWorldSize < 0 || tpWorldSize > 2) {
        return fail(CAM_ERR_RANGE, "tpWorldSize %lld outside [0, 2]", (long long)tpWorldSize);
    }
    if (expertShardType != 0) {  // moe_combine_shmem_tiling.cpp:174
        return fail(CAM_ERR_RANGE, "expertShardType must be 0");
    }
    if (sharedExpertRankNum < 0 || sharedExpertRankNum >= epWorldSize) {
        return fail(CAM_ERR_RANGE, "sharedExpertRankNum %lld outside [0, epWorldSize)", (long long)sharedExpertRankNum);
    }
    if (commQuantMode != 0 && commQuantMode != 2) {  // moe_combine_shmem_tiling.cpp:190-191
        return fail(CAM_ERR_RANGE, "commQuantMode must be 0 or 2, is %lld", (long long)commQuantMode);
    }
    if (epWorldSize != 1 || sharedExpertRankNum != 0 || tpWorldSize > 1) {
        return fail(CAM_ERR_UNSUPPORTED, "MoeCombineShmem: epWorldSize must be 1, sharedExpertRankNum 0 and "
                                         "tpWorldSize at most 1 (single-GPU library)");
    }
    const int64_t A = expandX->sizes[0], H = expandX->sizes[1];
    const int64_t T = expertIds->sizes[0], K = expertIds->sizes[1];
    if (T < 1) {
        return fail(CAM_ERR_RANGE, "batch size must be at least 1");
    }
    if (H < 1024 || H > 7168 || H % 8 != 0) {
        return fail(CAM_ERR_RANGE, "hidden size %lld must be a multiple of 8 in [1024, 7168]", (long long)H);
    }
    if (K <= 0 || K > cam::kMaxTopk) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, %d]", (long long)K, cam::kMaxTopk);
    }
    if (expandIdx->sizes[0] != T * K) {
        return fail(CAM_ERR_SHAPE, "expandIdx must hold bs * K elements");
    }
    if (expertScales->sizes[0] != T || expertScales->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "expertScales must be [bs, K]");
    }
    if (epSendCounts->sizes[0] != moeExpertNum) {
        return fail(CAM_ERR_SHAPE, "epSendCounts must hold one value per local expert");
    }
    if (out->sizes[0] != T || out->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "out must be [bs, H]");
    }
    if (globalBs != 0 && (globalBs < T * epWorldSize || globalBs % epWorldSize != 0)) {
        return fail(CAM_ERR_RANGE, "globalBs must be 0 or a multiple of epWorldSize that is >= epWorldSize * bs");
    }
    if (T * K > 0x7fffffffll || A > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "row counts do not fit 32 bits");
    }
    const bool wire = commQuantMode == 2;
    CAM_TRY(check_aligned(expandX, "expandX", 16));
    CAM_TRY(check_aligned(out, "out", 16));
    Carver c;
    const uint64_t o_slot = c.take((uint64_t)T * K * 4);
    const uint64_t o_wire = wire ? c.take((uint64_t)A * (uint64_t)(H + H / 4)) : 0;
    cam::CombineArgs g{};
    g.y = (const uint16_t *)expandX->data;
    g.w = (const float *)expertScales->data;
    g.T = (int)T;
    g.K = (int)K;
    g.H = (int)H;
    g.A = A;
    g.act_fp16 = expandX->dtype == CAM_DT_FLOAT16;
    g.out = (uint16_t *)out->data;
    const int32_t *ids = (const int32_t *)expertIds->data;
    const int32_t *eidx = (const int32_t *)expandIdx->data;
    const int32_t *counts = (const int32_t *)epSendCounts->data;
    const int iE = (int)moeExpertNum;
    auto run = [=](void *ws, hipStream_t s) mutable -> hipError_t {
        int32_t *slot = (int32_t *)((char *)ws + o_slot);
        hipError_t e = cam::launch_rows_from_counts(ids, eidx, counts, (int64_t)g.T * g.K, iE, g.A, slot, s);
        if (e != hipSuccess) {
            return e;
        }
        g.slot_row = slot;
        if (wire) {  // every row takes the int8 wire format on its way (moe_combine_shmem.h:567-592,755-773)
            uint8_t *rows = (uint8_t *)ws + o_wire;
            e = cam::launch_comm_quant(g.y, g.act_fp16, g.A, g.H, counts + (iE - 1), rows, s);
            if (e != hipSuccess) {
                return e;
            }
            g.y = (const uint16_t *)rows;
            g.wire_rows = 1;
            g.row_limit = counts + (iE - 1);
        }
        return cam::launch_combine(g, s);
    };
    return finish_phase1(kOpCombShmem, c.off, run, workspaceSize, executor);
}

camStatus camMoeCombineShmem(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpCombShmem, "camMoeCombineShmem", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
camStatus camPrepackWeightGetWorkspaceSize(const camTensor *src, int64_t gateUp, const camTensor *dst,
                                           uint64_t *workspaceSize, camOpExecutor **executor)
{
    if (src == nullptr || dst == nullptr) {
        return fail(CAM_ERR_NULL, "src / dst is NULL");
    }
    if (src->ndim != 2 && src->ndim != 3) {
        return fail(CAM_ERR_SHAPE, "src must be [Kd,N] or [G,Kd,N]");
    }
    // the layout moves bytes: int8 weights, or FP8 E4M3 weights of the block-scaled operators
    CAM_TRY(check_tensor(src, "src", src->ndim, CAM_DT_INT8, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    CAM_TRY(check_tensor(dst, "dst", src->ndim, CAM_DT_INT8, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    if (src->dtype != dst->dtype) {
        return fail(CAM_ERR_DTYPE, "src and dst must have the same dtype");
    }
    for (int d = 0; d < src->ndim; ++d) {
        if (src->sizes[d] != dst->sizes[d]) {
            return fail(CAM_ERR_SHAPE, "src and dst must have the same extents");
        }
    }
    if (src->format != CAM_FORMAT_ND) {
        return fail(CAM_ERR_SHAPE, "src must be in row-major format");
    }
    if (src->data == dst->data) {
        return fail(CAM_ERR_SHAPE, "prepack cannot run in place");
    }
    const int64_t G = src->ndim == 3 ? src->sizes[0] : 1;
    const int64_t Kd = src->sizes[src->ndim - 2], N = src->sizes[src->ndim - 1];
    CAM_TRY(check_gemm_dims("PrepackWeight", Kd, N, gateUp != 0));
    if (G <= 0 || G > 65535) {
        return fail(CAM_ERR_RANGE, "expert count %lld outside (0, 65535]", (long long)G);
    }
    CAM_TRY(check_aligned(dst, "dst", 16));
    const int8_t *s = (const int8_t *)src->data;
    int8_t *d = (int8_t *)dst->data;
    int g = (int)G, kd = (int)Kd, n = (int)N, gu = gateUp != 0;
    auto run = [=](void *, hipStream_t st) -> hipError_t { return cam::launch_prepack(s, d, g, kd, n, gu, st); };
    return finish_phase1(kOpPrepack, 0, run, workspaceSize, executor);
}

camStatus camPrepackWeight(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpPrepack, "camPrepackWeight", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
namespace {

struct GemmCommon {
    int64_t A, Kd, G;
    const int64_t *group_list;
    int cumulative;
};

camStatus check_gemm_inputs(const char *op, const camTensor *x, const camTensor *xScale, bool need_scale,
                            const camTensor *groupList, int64_t groupListType, GemmCommon *gc)
{
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_INT8));
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_tensor(groupList, "groupList", 1, CAM_DT_INT64));
    if (groupListType != 0 && groupListType != 1) {
        return fail(CAM_ERR_RANGE, "%s: groupListType must be 0 (cumulative) or 1 (counts)", op);
    }
    gc->A = x->sizes[0];
    gc->Kd = x->sizes[1];
    gc->G = groupList->sizes[0];
    if (gc->G <= 0 || gc->G > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "%s: %lld local experts outside (0, %d]", op, (long long)gc->G,
                    cam::kMaxExperts);
    }
    if (gc->A > 0x3fffffffll) {
        return fail(CAM_ERR_RANGE, "%s: too many rows", op);
    }
    if (need_scale) {
        CAM_TRY(check_tensor(xScale, "xScale", 1, CAM_DT_FLOAT));
        if (xScale->sizes[0] < gc->A) {
            return fail(CAM_ERR_SHAPE, "%s: xScale must hold one value per row of x", op);
        }
    }
    gc->group_list = (const int64_t *)groupList->data;
    gc->cumulative = groupListType == 0;
    return CAM_OK;
}

}  // namespace

camStatus camGroupedMatmulSwigluQuantGetWorkspaceSize(const camTensor *x, const camTensor *xScale,
                                                      const camTensorList *weight,
                                                      const camTensorList *weightScale,
                                                      const camTensor *groupList, int64_t groupListType,
                                                      const camTensor *y, const camTensor *yScale,
                                                      uint64_t *workspaceSize, camOpExecutor **executor)
{
    GemmCommon gc{};
    CAM_TRY(check_gemm_inputs("GroupedMatmulSwigluQuant", x, xScale, true, groupList, groupListType, &gc));
    CAM_TRY(check_tensor(y, "y", 2, CAM_DT_INT8));
    CAM_TRY(check_tensor(yScale, "yScale", 1, CAM_DT_FLOAT));
    const int64_t I = y->sizes[1];
    if (y->sizes[0] != gc.A || yScale->sizes[0] < gc.A) {
        return fail(CAM_ERR_SHAPE, "y must be [A,I] and yScale hold A values");
    }
    CAM_TRY(check_gemm_dims("GroupedMatmulSwigluQuant", gc.Kd, 2 * I, true));
    if (I > 4096) {
        return fail(CAM_ERR_RANGE, "intermediate size %lld above 4096", (long long)I);
    }
    WeightSet ws{};
    CAM_TRY(resolve_weights(weight, weightScale, "weight", gc.G, gc.Kd, 2 * I, true, &ws));
    CAM_TRY(check_aligned(y, "y", 16));
    cam::SchedSpec sp = sched_spec(gc.A, gc.G, 2 * I, gc.Kd, true);
    Carver c;
    const uint64_t o_sched = c.take(cam::sched_bytes(gc.A, (int)gc.G, (int)(2 * I)));
    const uint64_t o_prod = c.take((uint64_t)gc.A * I * 4);
    cam::GemmArgs g{};
    g.a = (const int8_t *)x->data;
    g.a_scale = (const float *)xScale->data;
    g.w = ws.w;
    g.w_scale = ws.s;
    g.per_expert = ws.per_expert;
    g.list = ws.list;
    g.Kd = (int)gc.Kd;
    g.N = (int)(2 * I);
    g.gate_up = 1;
    g.epilogue = cam::kEpiSwiglu;
    int8_t *yq = (int8_t *)y->data;
    float *ys = (float *)yScale->data;
    auto run = [=](void *wsp, hipStream_t s) mutable -> hipError_t {
        sp.sched = (int32_t *)((char *)wsp + o_sched);
        float *prod = (float *)((char *)wsp + o_prod);
        hipError_t e = cam::launch_build_sched(gc.group_list, gc.cumulative, (int)gc.G, gc.A, 1, &sp, s);
        if (e != hipSuccess) {
            return e;
        }
        g.sched = sp.sched;
        g.out = prod;
        e = cam::launch_gemm(g, s);
        if (e != hipSuccess) {
            return e;
        }
        return cam::launch_requant(prod, gc.A, (int)I, sp.sched, yq, ys, s);
    };
    return finish_phase1(kOpGmm1, c.off, run, workspaceSize, executor);
}

camStatus camGroupedMatmulSwigluQuant(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                      camStream_t stream)
{
    return run_phase2(kOpGmm1, "camGroupedMatmulSwigluQuant", workspace, workspaceSize, executor, stream);
}

camStatus camGroupedMatmulDequantGetWorkspaceSize(const camTensor *x, const camTensor *xScale,
                                                  const camTensorList *weight, const camTensorList *weightScale,
                                                  const camTensor *groupList, int64_t groupListType,
                                                  const camTensor *out, uint64_t *workspaceSize,
                                                  camOpExecutor **executor)
{
    GemmCommon gc{};
    CAM_TRY(check_gemm_inputs("GroupedMatmulDequant", x, xScale, true, groupList, groupListType, &gc));
    // out: bf16 [A,N], or int8 [A, N + N/4]: the bf16 rows quantised for the wire on their way out (blocks of 8
    // columns, AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:564-592), which MoeCombineGather reads back.
    CAM_TRY(check_tensor(out, "out", 2, CAM_DT_BF16, CAM_DT_FLOAT16, CAM_DT_INT8));
    const bool wire = out->dtype == CAM_DT_INT8;
    if (wire && out->sizes[1] % 10 != 0) {
        return fail(CAM_ERR_SHAPE, "int8 out must be [A, N + N/4] with N a multiple of 8");
    }
    const int64_t N = wire ? out->sizes[1] / 5 * 4 : out->sizes[1];
    if (out->sizes[0] != gc.A) {
        return fail(CAM_ERR_SHAPE, "out must have one row per row of x");
    }
    CAM_TRY(check_gemm_dims("GroupedMatmulDequant", gc.Kd, N, false));
    CAM_TRY(check_aligned(out, "out", 16));
    WeightSet ws{};
    CAM_TRY(resolve_weights(weight, weightScale, "weight", gc.G, gc.Kd, N, true, &ws));
    cam::SchedSpec sp = sched_spec(gc.A, gc.G, N, gc.Kd, false);
    Carver c;
    const uint64_t o_sched = c.take(cam::sched_bytes(gc.A, (int)gc.G, (int)N));
    const uint64_t o_rows = wire ? c.take((uint64_t)gc.A * N * 2) : 0;  // the bf16 rows before quantisation
    cam::GemmArgs g{};
    g.a = (const int8_t *)x->data;
    g.a_scale = (const float *)xScale->data;
    g.w = ws.w;
    g.w_scale = ws.s;
    g.per_expert = ws.per_expert;
    g.list = ws.list;
    g.Kd = (int)gc.Kd;
    g.N = (int)N;
    g.gate_up = 0;
    g.epilogue = cam::kEpiDequantBf16;
    g.out = out->data;
    g.out_fp16 = out->dtype == CAM_DT_FLOAT16;
    uint8_t *wire_out = (uint8_t *)out->data;
    auto run = [=](void *wsp, hipStream_t s) mutable -> hipError_t {
        sp.sched = (int32_t *)((char *)wsp + o_sched);
        hipError_t e = cam::launch_build_sched(gc.group_list, gc.cumulative, (int)gc.G, gc.A, 1, &sp, s);
        if (e != hipSuccess) {
            return e;
        }
        g.sched = sp.sched;
        if (!wire) {
            return cam::launch_gemm(g, s);
        }
        uint16_t *rows = (uint16_t *)((char *)wsp + o_rows);
        g.out = rows;
        e = cam::launch_gemm(g, s);
        if (e != hipSuccess) {
            return e;
        }
        return cam::launch_comm_quant(rows, 0, gc.A, g.N, sp.sched + 1, wire_out, s);  // sched[1]: rows that exist
    };
    return finish_phase1(kOpGmm2, c.off, run, workspaceSize, executor);
}

camStatus camGroupedMatmulDequant(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                  camStream_t stream)
{
    return run_phase2(kOpGmm2, "camGroupedMatmulDequant", workspace, workspaceSize, executor, stream);
}

camStatus camGroupedMatmulInt32GetWorkspaceSize(const camTensor *x, const camTensorList *weight, int64_t gateUp,
                                                const camTensor *groupList, int64_t groupListType,
                                                const camTensor *out, uint64_t *workspaceSize,
                                                camOpExecutor **executor)
{
    GemmCommon gc{};
    CAM_TRY(check_gemm_inputs("GroupedMatmulInt32", x, nullptr, false, groupList, groupListType, &gc));
    CAM_TRY(check_tensor(out, "out", 2, CAM_DT_INT32));
    const int64_t N = out->sizes[1];
    if (out->sizes[0] != gc.A) {
        return fail(CAM_ERR_SHAPE, "out must have one row per row of x");
    }
    CAM_TRY(check_gemm_dims("GroupedMatmulInt32", gc.Kd, N, gateUp != 0));
    CAM_TRY(check_aligned(out, "out", 16));
    WeightSet ws{};
    CAM_TRY(resolve_weights(weight, nullptr, "weight", gc.G, gc.Kd, N, false, &ws));
    cam::SchedSpec sp = sched_spec(gc.A, gc.G, N, gc.Kd, false);
    Carver c;
    const uint64_t o_sched = c.take(cam::sched_bytes(gc.A, (int)gc.G, (int)N));
    cam::GemmArgs g{};
    g.a = (const int8_t *)x->data;
    g.w = ws.w;
    g.per_expert = ws.per_expert;
    g.list = ws.list;
    g.Kd = (int)gc.Kd;
    g.N = (int)N;
    g.gate_up = gateUp != 0;
    g.epilogue = cam::kEpiInt32;
    g.out = out->data;
    auto run = [=](void *wsp, hipStream_t s) mutable -> hipError_t {
        sp.sched = (int32_t *)((char *)wsp + o_sched);
        hipError_t e = cam::launch_build_sched(gc.group_list, gc.cumulative, (int)gc.G, gc.A, 1, &sp, s);
        if (e != hipSuccess) {
            return e;
        }
        g.sched = sp.sched;
        return cam::launch_gemm(g, s);
    };
    return finish_phase1(kOpGmmI32, c.off, run, workspaceSize, executor);
}

camStatus camGroupedMatmulInt32(void *workspace, uint64_t workspaceSize, camOpExecutor *executor,
                                camStream_t stream)
{
    return run_phase2(kOpGmmI32, "camGroupedMatmulInt32", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
camStatus camFusedDeepMoeGetWorkspaceSize(const camTensor *x, const camTensor *expertIds,
                                          const camTensorList *gmm1PermutedWeight,
                                          const camTensorList *gmm1PermutedWeightScale,
                                          const camTensorList *gmm2Weight, const camTensorList *gmm2WeightScale,
                                          const camTensor *expertScales,
                                          const camTensor *expertSmoothScalesOptional,
                                          const camTensor *xActiveMaskOptional, char *groupEp,
                                          int64_t epRankSize, int64_t epRankId, int64_t moeExpertNum,
                                          int64_t sharedExpertNum, int64_t sharedExpertRankNum,
                                          int64_t quantMode, int64_t globalBs, const camTensor *output,
                                          const camTensor *expertTokenNums, uint64_t *workspaceSize,
                                          camOpExecutor **executor)
{
    (void)groupEp;
    // The fused operator always quantises per token (the only path the reference kernel has); quantMode is
    // carried into the tiling data unchecked there (AK/fused_deep_moe/op_host/fused_deep_moe_tiling.cpp:356).
    // Values no dispatch operator knows are rejected here instead of being ignored.
    if (quantMode < 0 || quantMode > 3) {
        return fail(CAM_ERR_RANGE, "quantMode %lld outside [0, 3]", (long long)quantMode);
    }
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_BF16, CAM_DT_FLOAT16));
    CAM_TRY(check_tensor(expertIds, "expertIds", 2, CAM_DT_INT32));
    CAM_TRY(check_tensor(expertScales, "expertScales", 2, CAM_DT_FLOAT));
    if (epRankSize <= 0 || epRankSize > cam::kMaxRanks) {
        return fail(CAM_ERR_RANGE, "epRankSize %lld outside (0, %d]", (long long)epRankSize, cam::kMaxRanks);
    }
    if (epRankId < 0 || epRankId >= epRankSize) {
        return fail(CAM_ERR_RANGE, "epRankId %lld outside [0, epRankSize)", (long long)epRankId);
    }
    if (moeExpertNum <= 0 || moeExpertNum > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "moeExpertNum %lld outside (0, %d]", (long long)moeExpertNum, cam::kMaxExperts);
    }
    if (sharedExpertNum != 1) {  // AK/fused_deep_moe/op_host/fused_deep_moe_tiling.cpp:345
        return fail(CAM_ERR_RANGE, "sharedExpertNum must be 1, is %lld", (long long)sharedExpertNum);
    }
    if (sharedExpertRankNum < 0 || sharedExpertRankNum >= epRankSize) {
        return fail(CAM_ERR_RANGE, "sharedExpertRankNum %lld outside [0, epRankSize)", (long long)sharedExpertRankNum);
    }
    if (moeExpertNum % (epRankSize - sharedExpertRankNum) != 0) {
        return fail(CAM_ERR_RANGE, "moeExpertNum must be divisible by epRankSize - sharedExpertRankNum");
    }
    if (epRankSize != 1 || sharedExpertRankNum != 0) {
        return fail(CAM_ERR_UNSUPPORTED, "FusedDeepMoe: epRankSize must be 1 and sharedExpertRankNum 0 "
                                         "(single-GPU library)");
    }
    if (expertSmoothScalesOptional != nullptr) {
        return fail(CAM_ERR_UNSUPPORTED, "expertSmoothScales is accepted by the reference but never used; pass NULL");
    }
    const int64_t T = x->sizes[0], H = x->sizes[1], K = expertIds->sizes[1];
    if (expertIds->sizes[0] != T) {
        return fail(CAM_ERR_SHAPE, "expertIds dimension 0 must equal the batch size");
    }
    if (expertScales->sizes[0] != T || expertScales->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "expertScales must be [bs, K]");
    }
    if (T < 1) {
        return fail(CAM_ERR_RANGE, "batch size must be at least 1");
    }
    if (H < 512 || H > 7168) {
        return fail(CAM_ERR_RANGE, "hidden size %lld outside [512, 7168]", (long long)H);
    }
    if (K <= 0 || K > 12) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, 12]", (long long)K);
    }
    if (globalBs != 0 && globalBs % epRankSize != 0) {
        return fail(CAM_ERR_RANGE, "globalBs must be divisible by epRankSize");
    }
    if (T * K > 0x3fffffffll) {
        return fail(CAM_ERR_RANGE, "tokens * top-k too large");
    }
    const int64_t Epr = moeExpertNum;
    // intermediate size from the GMM2 weight
    if (gmm2Weight == nullptr || gmm2Weight->tensors == nullptr || gmm2Weight->count == 0 ||
        gmm2Weight->tensors[0] == nullptr) {
        return fail(CAM_ERR_NULL, "gmm2Weight list is NULL or empty");
    }
    const camTensor *w2_0 = gmm2Weight->tensors[0];
    if (w2_0->ndim != 2 && w2_0->ndim != 3) {
        return fail(CAM_ERR_SHAPE, "gmm2Weight must be [Epr,I,H] or a list of [I,H]");
    }
    const int64_t I = w2_0->sizes[w2_0->ndim - 2];
    if (2 * I < 1024 || 2 * I > 6144) {
        return fail(CAM_ERR_RANGE, "2 * intermediate size %lld outside [1024, 6144]", (long long)(2 * I));
    }
    CAM_TRY(check_gemm_dims("FusedDeepMoe GMM1", H, 2 * I, true));
    CAM_TRY(check_gemm_dims("FusedDeepMoe GMM2", I, H, false));
    WeightSet w1{}, w2{};
    CAM_TRY(resolve_weights(gmm1PermutedWeight, gmm1PermutedWeightScale, "gmm1PermutedWeight", Epr, H, 2 * I, true,
                            &w1));
    CAM_TRY(resolve_weights(gmm2Weight, gmm2WeightScale, "gmm2Weight", Epr, I, H, true, &w2));
    if (xActiveMaskOptional != nullptr) {
        CAM_TRY(check_tensor(xActiveMaskOptional, "xActiveMask", 1, CAM_DT_BOOL, CAM_DT_UINT8));
        if (xActiveMaskOptional->sizes[0] != T) {
            return fail(CAM_ERR_SHAPE, "xActiveMask must be [bs]");
        }
    }
    CAM_TRY(check_tensor(output, "output", 2, x->dtype));  // the layer's output has the type of its input
    if (output->sizes[0] != T || output->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "output must be [bs, H]");
    }
    CAM_TRY(check_tensor(expertTokenNums, "expertTokenNums", 1, CAM_DT_INT64));
    if (expertTokenNums->sizes[0] != Epr) {
        return fail(CAM_ERR_SHAPE, "expertTokenNums must hold one value per local expert");
    }
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_aligned(output, "output", 16));

    const int64_t A = T * K;  // maxTokenNum of AK/fused_deep_moe/op_kernel/fused_deep_moe.h:336 for one rank
    cam::SchedSpec sp1 = sched_spec(A, Epr, 2 * I, H, true);
    cam::SchedSpec sp2 = sched_spec(A, Epr, H, I, false);
    Carver c;
    const uint64_t o_pos = c.take((uint64_t)A * 4);
    const uint64_t o_row = c.take((uint64_t)A * 4);
    const uint64_t o_meta = c.take(cam::kPlanMeta * 4);
    const uint64_t o_sched1 = c.take(cam::sched_bytes(A, (int)Epr, (int)(2 * I)));
    const uint64_t o_sched2 = c.take(cam::sched_bytes(A, (int)Epr, (int)H));
    const uint64_t o_hist = c.take(cam::plan_workspace_bytes(T, K, (int)Epr));
    // The bf16 rows GMM2 writes (2*A*H bytes) live where the quantised rows (A*H) and the fp32 SwiGLU products
    // (4*A*I) lived: both are dead once the re-quantisation has run (the reference overlays its stages the same
    // way, AK/fused_deep_moe/op_kernel/fused_deep_moe.h:362-391).  GMM2's own input stays apart.
    const uint64_t x1_bytes = align_up((uint64_t)A * H);
    const uint64_t shared_bytes = std::max<uint64_t>((uint64_t)A * H * 2, x1_bytes + (uint64_t)A * I * 4);
    const uint64_t o_x1 = c.take(shared_bytes);
    const uint64_t o_prod = o_x1 + x1_bytes;
    const uint64_t o_y = o_x1;
    const uint64_t o_x1s = c.take((uint64_t)A * 4);
    const uint64_t o_x2 = c.take((uint64_t)A * I);
    const uint64_t o_x2s = c.take((uint64_t)A * 4);

    const uint16_t *xp = (const uint16_t *)x->data;
    const int x_is_fp16 = x->dtype == CAM_DT_FLOAT16;
    const int32_t *ids = (const int32_t *)expertIds->data;
    const float *gates = (const float *)expertScales->data;
    const uint8_t *mask = xActiveMaskOptional ? (const uint8_t *)xActiveMaskOptional->data : nullptr;
    uint16_t *outp = (uint16_t *)output->data;
    int64_t *etn = (int64_t *)expertTokenNums->data;
    const int iT = (int)T, iK = (int)K, iH = (int)H, iI = (int)I, iE = (int)Epr;

    auto run = [=](void *wsp, hipStream_t s) -> hipError_t {
        char *w = (char *)wsp;
        int32_t *pos = (int32_t *)(w + o_pos);
        int32_t *row = (int32_t *)(w + o_row);
        int32_t *meta = (int32_t *)(w + o_meta);
        int8_t *x1 = (int8_t *)(w + o_x1);
        float *x1s = (float *)(w + o_x1s);
        float *prod = (float *)(w + o_prod);
        int8_t *x2 = (int8_t *)(w + o_x2);
        float *x2s = (float *)(w + o_x2s);
        uint16_t *y = (uint16_t *)(w + o_y);

        cam::PlanArgs p{};
        p.idx = ids;
        p.idx_is64 = 0;
        p.mask = mask;
        p.T = iT;
        p.K = iK;
        p.E = iE;
        p.R = 1;
        p.pos = pos;
        p.dst_row = row;
        p.tokens_per_expert = etn;
        p.meta = meta;
        p.hist_ws = (int32_t *)(w + o_hist);
        hipError_t e;
        cam::SchedSpec specs[2] = {sp1, sp2};  // both GEMM schedules come from the per-expert counts of the plan
        specs[0].sched = (int32_t *)(w + o_sched1);
        specs[1].sched = (int32_t *)(w + o_sched2);
        e = cam::launch_plan(p, s);
        if (e != hipSuccess) return e;
        cam::DispatchArgs d{};
        d.x = xp;
        d.x_is_fp16 = x_is_fp16;
        d.idx = ids;
        d.dst_row = row;
        d.T = iT;
        d.K = iK;
        d.H = iH;
        d.E = iE;
        d.A = A;
        d.quant = 2;
        d.out = x1;
        d.scales = x1s;
        // the plan has written the per-expert counts: spare workgroups of the permute build both schedules
        d.sched.group_list = etn;
        d.sched.cumulative = 0;
        d.sched.G = iE;
        d.sched.nspec = 2;
        d.sched.max_rows = A;
        d.sched.spec[0] = specs[0];
        d.sched.spec[1] = specs[1];
        e = cam::launch_dispatch(d, s);
        if (e != hipSuccess) return e;

        cam::GemmArgs g1{};
        g1.a = x1;
        g1.a_scale = x1s;
        g1.w = w1.w;
        g1.w_scale = w1.s;
        g1.per_expert = w1.per_expert;
        g1.list = w1.list;
        g1.sched = specs[0].sched;
        g1.Kd = iH;
        g1.N = 2 * iI;
        g1.gate_up = 1;
        g1.epilogue = cam::kEpiSwiglu;
        g1.out = prod;
        e = cam::launch_gemm(g1, s);
        if (e != hipSuccess) return e;
        e = cam::launch_requant(prod, A, iI, specs[0].sched, x2, x2s, s);
        if (e != hipSuccess) return e;

        cam::GemmArgs g2{};
        g2.a = x2;
        g2.a_scale = x2s;
        g2.w = w2.w;
        g2.w_scale = w2.s;
        g2.per_expert = w2.per_expert;
        g2.list = w2.list;
        g2.sched = specs[1].sched;
        g2.Kd = iI;
        g2.N = iH;
        g2.gate_up = 0;
        g2.epilogue = cam::kEpiDequantBf16;
        g2.out = y;
        g2.out_fp16 = x_is_fp16;
        e = cam::launch_gemm(g2, s);
        if (e != hipSuccess) return e;

        cam::CombineArgs cb{};
        cb.y = y;
        cb.slot_row = row;
        cb.w = gates;
        cb.T = iT;
        cb.K = iK;
        cb.H = iH;
        cb.A = A;
        cb.t_active = meta + 2;
        cb.act_fp16 = x_is_fp16;
        cb.out = outp;
        return cam::launch_combine(cb, s);
    };
    return finish_phase1(kOpFused, c.off, run, workspaceSize, executor);
}

camStatus camFusedDeepMoe(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpFused, "camFusedDeepMoe", workspace, workspaceSize, executor, stream);
}

// ------------------------------------------------------------------------------------------------
// Block-scaled FP8 operators (include/cam_fp8_spec.h).  No counterpart in the reference, whose fused operator
// is W8A8 only (src/cam/README.md:20-21).
namespace {

struct Fp8Weight {
    const int8_t *w;
    const uint8_t *s;
};

camStatus check_fp8_weight(const camTensor *w, const camTensor *ws, const char *name, int64_t G, int64_t Kd,
                           int64_t N, Fp8Weight *out)
{
    CAM_TRY(check_tensor(w, name, 3, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    if (w->format != CAM_FORMAT_MFMA_B) {
        return fail(CAM_ERR_UNSUPPORTED, "%s must be converted once with camPrepackWeight (format CAM_FORMAT_MFMA_B)",
                    name);
    }
    if (w->sizes[0] != G || w->sizes[1] != Kd || w->sizes[2] != N) {
        return fail(CAM_ERR_SHAPE, "%s must be [%lld,%lld,%lld]", name, (long long)G, (long long)Kd, (long long)N);
    }
    CAM_TRY(check_tensor(ws, "weight scale", 3, CAM_DT_UINT8));
    if (ws->sizes[0] != G || ws->sizes[1] != Kd / 128 || ws->sizes[2] != N / 128) {
        return fail(CAM_ERR_SHAPE, "%s scale must be uint8 [%lld,%lld,%lld] (E8M0 per 128 x 128 block)", name,
                    (long long)G, (long long)(Kd / 128), (long long)(N / 128));
    }
    CAM_TRY(check_aligned(w, name, 16));
    out->w = (const int8_t *)w->data;
    out->s = (const uint8_t *)ws->data;
    return CAM_OK;
}

camStatus check_fp8_dims(const char *op, int64_t Kd, int64_t N, bool gate_up)
{
    if (Kd < 128 || Kd % 128 != 0 || Kd > 8192) {
        return fail(CAM_ERR_RANGE, "%s: K %lld must be a multiple of 128 in [128, 8192]", op, (long long)Kd);
    }
    if (N < 128 || N % (gate_up ? 256 : 128) != 0) {
        return fail(CAM_ERR_RANGE, "%s: N %lld must be a multiple of %d", op, (long long)N, gate_up ? 256 : 128);
    }
    return CAM_OK;
}

}  // namespace

camStatus camGroupedMatmulFp8GetWorkspaceSize(const camTensor *x, const camTensor *xScale, const camTensor *weight,
                                              const camTensor *weightScale, int64_t gateUp,
                                              const camTensor *groupList, int64_t groupListType,
                                              const camTensor *out, const camTensor *outScaleOptional,
                                              uint64_t *workspaceSize, camOpExecutor **executor)
{
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_tensor(groupList, "groupList", 1, CAM_DT_INT64));
    if (groupListType != 0 && groupListType != 1) {
        return fail(CAM_ERR_RANGE, "GroupedMatmulFp8: groupListType must be 0 (cumulative) or 1 (counts)");
    }
    const int64_t A = x->sizes[0], Kd = x->sizes[1], G = groupList->sizes[0];
    if (G <= 0 || G > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "GroupedMatmulFp8: %lld experts outside (0, %d]", (long long)G, cam::kMaxExperts);
    }
    if (A > 0x3fffffffll) {
        return fail(CAM_ERR_RANGE, "GroupedMatmulFp8: too many rows");
    }
    CAM_TRY(check_tensor(xScale, "xScale", 2, CAM_DT_UINT8));
    if (xScale->sizes[0] < A || xScale->sizes[1] != Kd / 128) {
        return fail(CAM_ERR_SHAPE, "xScale must be uint8 [rows, K/128] (E8M0)");
    }
    if (out == nullptr) {
        return fail(CAM_ERR_NULL, "out is NULL");
    }
    const bool gate_up = gateUp != 0;
    const bool quant_out = out->dtype == CAM_DT_FLOAT8_E4M3FN || out->dtype == CAM_DT_UINT8;
    if (quant_out) {
        CAM_TRY(check_tensor(out, "out", 2, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
        if (!gate_up) {
            return fail(CAM_ERR_DTYPE, "an FP8 out is the quantised SwiGLU product: it needs gateUp != 0");
        }
        CAM_TRY(check_tensor(outScaleOptional, "outScale", 2, CAM_DT_UINT8));
        if (outScaleOptional->sizes[0] != A || outScaleOptional->sizes[1] * 128 != out->sizes[1]) {
            return fail(CAM_ERR_SHAPE, "outScale must be uint8 [rows, I/128] (E8M0)");
        }
    } else {
        CAM_TRY(check_tensor(out, "out", 2, CAM_DT_FLOAT, CAM_DT_BF16));
        if (outScaleOptional != nullptr) {
            return fail(CAM_ERR_DTYPE, "outScale goes with an FP8 out only");
        }
    }
    if (out->sizes[0] != A) {
        return fail(CAM_ERR_SHAPE, "out must have one row per row of x");
    }
    if (gate_up && !quant_out && out->dtype != CAM_DT_FLOAT) {
        return fail(CAM_ERR_DTYPE, "the SwiGLU product (gateUp != 0) is written as float32 or as FP8 with outScale");
    }
    const int64_t N = gate_up ? 2 * out->sizes[1] : out->sizes[1];
    CAM_TRY(check_fp8_dims("GroupedMatmulFp8", Kd, N, gate_up));
    CAM_TRY(check_aligned(out, "out", 16));
    CAM_TRY(check_aligned(xScale, "xScale", 4));  // a row's block scales are fetched as words
    Fp8Weight fw{};
    CAM_TRY(check_fp8_weight(weight, weightScale, "weight", G, Kd, N, &fw));
    cam::SchedSpec sp = sched_spec(A, G, N, Kd, gate_up);
    Carver c;
    const uint64_t o_sched = c.take(cam::sched_bytes(A, (int)G, (int)N));
    cam::GemmArgs g{};
    g.a = (const int8_t *)x->data;
    g.w = fw.w;
    g.fp8 = 1;
    g.a_scale8 = (const uint8_t *)xScale->data;
    g.w_scale8 = fw.s;
    g.Kd = (int)Kd;
    g.N = (int)N;
    g.gate_up = gate_up;
    g.epilogue = quant_out ? cam::kEpiSwigluFp8
                           : (gate_up ? cam::kEpiSwiglu
                                      : (out->dtype == CAM_DT_BF16 ? cam::kEpiDequantBf16 : cam::kEpiInt32));
    g.out = out->data;
    g.out_scale8 = quant_out ? (uint8_t *)outScaleOptional->data : nullptr;
    const int64_t *gl = (const int64_t *)groupList->data;
    const int cumulative = groupListType == 0;
    auto run = [=](void *wsp, hipStream_t s) mutable -> hipError_t {
        sp.sched = (int32_t *)((char *)wsp + o_sched);
        hipError_t e = cam::launch_build_sched(gl, cumulative, (int)G, A, 1, &sp, s);
        if (e != hipSuccess) {
            return e;
        }
        g.sched = sp.sched;
        return cam::launch_gemm(g, s);
    };
    return finish_phase1(kOpGmmFp8, c.off, run, workspaceSize, executor);
}

camStatus camGroupedMatmulFp8(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpGmmFp8, "camGroupedMatmulFp8", workspace, workspaceSize, executor, stream);
}

camStatus camQuantRowsFp8GetWorkspaceSize(const camTensor *x, const camTensor *q, const camTensor *scale,
                                          uint64_t *workspaceSize, camOpExecutor **executor)
{
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_FLOAT));
    CAM_TRY(check_tensor(q, "q", 2, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    CAM_TRY(check_tensor(scale, "scale", 2, CAM_DT_UINT8));
    const int64_t A = x->sizes[0], I = x->sizes[1];
    if (I < 128 || I % 128 != 0) {
        return fail(CAM_ERR_ALIGN, "the row length %lld must be a multiple of 128", (long long)I);
    }
    if (q->sizes[0] != A || q->sizes[1] != I || scale->sizes[0] != A || scale->sizes[1] != I / 128) {
        return fail(CAM_ERR_SHAPE, "q must be [rows, I] and scale uint8 [rows, I/128]");
    }
    if (A > 0x7fffffffll) {
        return fail(CAM_ERR_RANGE, "too many rows");
    }
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_aligned(q, "q", 16));
    const float *xp = (const float *)x->data;
    uint8_t *qp = (uint8_t *)q->data;
    uint8_t *sp = (uint8_t *)scale->data;
    const int iI = (int)I;
    auto run = [=](void *, hipStream_t s) -> hipError_t {
        return cam::launch_requant_fp8(xp, A, iI, nullptr, qp, sp, s);
    };
    return finish_phase1(kOpQuantFp8, 0, run, workspaceSize, executor);
}

camStatus camQuantRowsFp8(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpQuantFp8, "camQuantRowsFp8", workspace, workspaceSize, executor, stream);
}

camStatus camFusedDeepMoeFp8GetWorkspaceSize(const camTensor *x, const camTensor *expertIds,
                                             const camTensor *gmm1Weight, const camTensor *gmm1WeightScale,
                                             const camTensor *gmm2Weight, const camTensor *gmm2WeightScale,
                                             const camTensor *expertScales, const camTensor *xActiveMaskOptional,
                                             int64_t moeExpertNum, const camTensor *output,
                                             const camTensor *expertTokenNums, uint64_t *workspaceSize,
                                             camOpExecutor **executor)
{
    CAM_TRY(check_tensor(x, "x", 2, CAM_DT_BF16));  // the block-scaled layer is specified for bf16 activations only
    CAM_TRY(check_tensor(expertIds, "expertIds", 2, CAM_DT_INT32));
    CAM_TRY(check_tensor(expertScales, "expertScales", 2, CAM_DT_FLOAT));
    if (moeExpertNum <= 0 || moeExpertNum > cam::kMaxExperts) {
        return fail(CAM_ERR_RANGE, "moeExpertNum %lld outside (0, %d]", (long long)moeExpertNum, cam::kMaxExperts);
    }
    const int64_t T = x->sizes[0], H = x->sizes[1], K = expertIds->sizes[1], E = moeExpertNum;
    if (T < 1 || expertIds->sizes[0] != T || expertScales->sizes[0] != T || expertScales->sizes[1] != K) {
        return fail(CAM_ERR_SHAPE, "x, expertIds and expertScales must agree on [bs] and [bs,K]");
    }
    if (H < 1024 || H > 7168) {
        return fail(CAM_ERR_RANGE, "hidden size %lld outside [1024, 7168]", (long long)H);
    }
    if (K <= 0 || K > cam::kMaxTopk) {
        return fail(CAM_ERR_RANGE, "top-k %lld outside (0, %d]", (long long)K, cam::kMaxTopk);
    }
    if (T * K > 0x3fffffffll) {
        return fail(CAM_ERR_RANGE, "tokens * top-k too large");
    }
    CAM_TRY(check_tensor(gmm2Weight, "gmm2Weight", 3, CAM_DT_FLOAT8_E4M3FN, CAM_DT_UINT8));
    const int64_t I = gmm2Weight->sizes[1];
    CAM_TRY(check_fp8_dims("FusedDeepMoeFp8 GMM1", H, 2 * I, true));
    CAM_TRY(check_fp8_dims("FusedDeepMoeFp8 GMM2", I, H, false));
    Fp8Weight w1{}, w2{};
    CAM_TRY(check_fp8_weight(gmm1Weight, gmm1WeightScale, "gmm1Weight", E, H, 2 * I, &w1));
    CAM_TRY(check_fp8_weight(gmm2Weight, gmm2WeightScale, "gmm2Weight", E, I, H, &w2));
    if (xActiveMaskOptional != nullptr) {
        CAM_TRY(check_tensor(xActiveMaskOptional, "xActiveMask", 1, CAM_DT_BOOL, CAM_DT_UINT8));
        if (xActiveMaskOptional->sizes[0] != T) {
            return fail(CAM_ERR_SHAPE, "xActiveMask must be [bs]");
        }
    }
    CAM_TRY(check_tensor(output, "output", 2, CAM_DT_BF16));
    if (output->sizes[0] != T || output->sizes[1] != H) {
        return fail(CAM_ERR_SHAPE, "output must be [bs, H]");
    }
    CAM_TRY(check_tensor(expertTokenNums, "expertTokenNums", 1, CAM_DT_INT64));
    if (expertTokenNums->sizes[0] != E) {
        return fail(CAM_ERR_SHAPE, "expertTokenNums must hold one value per expert");
    }
    CAM_TRY(check_aligned(x, "x", 16));
    CAM_TRY(check_aligned(output, "output", 16));

    const int64_t A = T * K;
    cam::SchedSpec sp1 = sched_spec(A, E, 2 * I, H, true);
    cam::SchedSpec sp2 = sched_spec(A, E, H, I, false);
    Carver c;
    const uint64_t o_pos = c.take((uint64_t)A * 4);
    const uint64_t o_row = c.take((uint64_t)A * 4);
    const uint64_t o_meta = c.take(cam::kPlanMeta * 4);
    const uint64_t o_sched1 = c.take(cam::sched_bytes(A, (int)E, (int)(2 * I)));
    const uint64_t o_sched2 = c.take(cam::sched_bytes(A, (int)E, (int)H));
    const uint64_t o_hist = c.take(cam::plan_workspace_bytes(T, K, (int)E));
    // as in the int8 layer, the bf16 rows of GMM2 overlay the quantised input rows and the fp32 products
    const uint64_t x1_bytes = align_up((uint64_t)A * H);
    const uint64_t shared_bytes = std::max<uint64_t>((uint64_t)A * H * 2, x1_bytes + (uint64_t)A * I * 4);
    const uint64_t o_x1 = c.take(shared_bytes);
    const uint64_t o_prod = o_x1 + x1_bytes;
    const uint64_t o_y = o_x1;
    const uint64_t o_x1s = c.take((uint64_t)A * (H / 128));
    const uint64_t o_x2 = c.take((uint64_t)A * I);
    const uint64_t o_x2s = c.take((uint64_t)A * (I / 128));

    const uint16_t *xp = (const uint16_t *)x->data;
    const int x_is_fp16 = 0;
    const int32_t *ids = (const int32_t *)expertIds->data;
    const float *gates = (const float *)expertScales->data;
    const uint8_t *mask = xActiveMaskOptional ? (const uint8_t *)xActiveMaskOptional->data : nullptr;
    uint16_t *outp = (uint16_t *)output->data;
    int64_t *etn = (int64_t *)expertTokenNums->data;
    const int iT = (int)T, iK = (int)K, iE = (int)E, iH = (int)H, iI = (int)I;

    auto run = [=](void *wsp, hipStream_t s) -> hipError_t {
        char *w = (char *)wsp;
        int32_t *pos = (int32_t *)(w + o_pos);
        int32_t *row = (int32_t *)(w + o_row);
        int32_t *meta = (int32_t *)(w + o_meta);
        uint8_t *x1 = (uint8_t *)(w + o_x1);
        uint8_t *x1s = (uint8_t *)(w + o_x1s);
        float *prod = (float *)(w + o_prod);
        uint8_t *x2 = (uint8_t *)(w + o_x2);
        uint8_t *x2s = (uint8_t *)(w + o_x2s);
        uint16_t *y = (uint16_t *)(w + o_y);

        cam::PlanArgs p{};
        p.idx = ids;
        p.idx_is64 = 0;
        p.mask = mask;
        p.T = iT;
        p.K = iK;
        p.E = iE;
        p.R = 1;
        p.pos = pos;
        p.dst_row = row;
        p.tokens_per_expert = etn;
        p.meta = meta;
        p.hist_ws = (int32_t *)(w + o_hist);
        hipError_t e;
        cam::SchedSpec specs[2] = {sp1, sp2};
        specs[0].sched = (int32_t *)(w + o_sched1);
        specs[1].sched = (int32_t *)(w + o_sched2);
        e = cam::launch_plan(p, s);
        if (e != hipSuccess) return e;
        cam::DispatchArgs d{};
        d.x = xp;
        d.x_is_fp16 = x_is_fp16;
        d.idx = ids;
        d.dst_row = row;
        d.T = iT;
        d.K = iK;
        d.H = iH;
        d.E = iE;
        d.A = A;
        d.quant = 3;
        d.out = x1;
        d.scales = (float *)x1s;
        d.sched.group_list = etn;  // spare workgroups of the permute build both schedules
        d.sched.cumulative = 0;
        d.sched.G = iE;
        d.sched.nspec = 2;
        d.sched.max_rows = A;
        d.sched.spec[0] = specs[0];
        d.sched.spec[1] = specs[1];
        e = cam::launch_dispatch(d, s);
        if (e != hipSuccess) return e;

        cam::GemmArgs g1{};
        g1.a = (const int8_t *)x1;
        g1.w = w1.w;
        g1.fp8 = 1;
        g1.a_scale8 = x1s;
        g1.w_scale8 = w1.s;
        g1.sched = specs[0].sched;
        g1.Kd = iH;
        g1.N = 2 * iI;
        g1.gate_up = 1;
        g1.epilogue = cam::kEpiSwigluFp8;  // the SwiGLU product leaves GMM1 quantised for GMM2
        g1.out = x2;
        g1.out_scale8 = x2s;
        e = cam::launch_gemm(g1, s);
        if (e != hipSuccess) return e;

        cam::GemmArgs g2{};
        g2.a = (const int8_t *)x2;
        g2.w = w2.w;
        g2.fp8 = 1;
        g2.a_scale8 = x2s;
        g2.w_scale8 = w2.s;
        g2.sched = specs[1].sched;
        g2.Kd = iI;
        g2.N = iH;
        g2.gate_up = 0;
        g2.epilogue = cam::kEpiDequantBf16;
        g2.out = y;
        e = cam::launch_gemm(g2, s);
        if (e != hipSuccess) return e;

        cam::CombineArgs cb{};
        cb.y = y;
        cb.slot_row = row;
        cb.w = gates;
        cb.T = iT;
        cb.K = iK;
        cb.H = iH;
        cb.A = A;
        cb.t_active = meta + 2;
        cb.out = outp;
        return cam::launch_combine(cb, s);
    };
    return finish_phase1(kOpFusedFp8, c.off, run, workspaceSize, executor);
}

camStatus camFusedDeepMoeFp8(void *workspace, uint64_t workspaceSize, camOpExecutor *executor, camStream_t stream)
{
    return run_phase2(kOpFusedFp8, "camFusedDeepMoeFp8", workspace, workspaceSize, executor, stream);
}

}  // extern "C"
