// torch.ops.umdk_cam_op_lib.* implemented in C++ on top of the C ABI (include/cam_mi355x.h).
//
// The reference registers the same six schemas from C++ (paths relative to the reference tree):
//   src/cam/comm_operator/pybind/pybind.cpp:13-41                    schemas and TORCH_LIBRARY_IMPL
//   src/cam/comm_operator/pybind/fused_deep_moe.cpp:46-79,152-235    output allocation, EXEC_NPU_CMD, autograd
//   src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:96-192     host loops replaced here by one operator
//   src/cam/comm_operator/pybind/moe_dispatch_shmem.cpp:27-153       output shapes of the SHMEM dispatch
//   src/cam/comm_operator/pybind/moe_combine_shmem.cpp:27-86         output shape of the SHMEM combine
//   src/cam/comm_operator/pybind/pytorch_npu_helper.hpp:533-582      phase 1, workspace, phase 2 on the stream
// Each implementation allocates the outputs, asks phase 1 for the workspace size, takes the workspace from the
// caching allocator and queues phase 2 on the current stream of the tensors' device; nothing synchronises except
// where the reference's operator returns a host tensor or a data-dependent shape.
//
// Autograd.  The reference registers every operator on the autograd key as well, as a function whose backward
// returns undefined gradients (fused_deep_moe.cpp:152-229, get_dispatch_layout.cpp:113, moe_combine_prefill.cpp:
// 146): inputs that require grad are accepted, the outputs take part in a graph, nothing flows back.  The
// AutogradCUDA registrations at the end of this file do the same.
//
// Packed weights.  The reference marks converted weights inside the tensor (npu_format_cast to FRACTAL_NZ,
// test/cam/ut/fused_deep_moe/test_fused_deep_moe.py:243-246).  A torch tensor on ROCm has no such field, so
// prepack_weight (an operator of this library beyond the reference's four) remembers the storage of its result
// and fused_deep_moe accepts only weights that live in such a storage: views of a packed tensor pass, a copy
// made by clone() or to() does not (its bytes would still be packed, but nothing says so) and is refused with a
// message instead of being multiplied as if it were row-major.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/cam_mi355x.h"

namespace {

int32_t cam_dtype(const at::Tensor &t)
{
    switch (t.scalar_type()) {
        case at::kFloat: return CAM_DT_FLOAT;
        case at::kHalf: return CAM_DT_FLOAT16;
        case at::kChar: return CAM_DT_INT8;
        case at::kInt: return CAM_DT_INT32;
        case at::kByte: return CAM_DT_UINT8;
        case at::kLong: return CAM_DT_INT64;
        case at::kBool: return CAM_DT_BOOL;
        case at::kBFloat16: return CAM_DT_BF16;
        case at::kFloat8_e4m3fn: return CAM_DT_FLOAT8_E4M3FN;
        default: TORCH_CHECK(false, "umdk_cam_op_lib: unsupported dtype ", t.scalar_type());
    }
}

camTensor to_cam(const at::Tensor &t, int32_t format = CAM_FORMAT_ND)
{
    TORCH_CHECK(t.is_cuda(), "umdk_cam_op_lib: tensors must live on a ROCm device (the CAM kernels have no CPU path)");
    TORCH_CHECK(t.dim() <= CAM_MAX_DIMS, "umdk_cam_op_lib: too many dimensions");
    camTensor c{};
    c.data = t.data_ptr();
    c.dtype = cam_dtype(t);
    c.ndim = (int32_t)t.dim();
    for (int64_t d = 0; d < t.dim(); ++d) {
        c.sizes[d] = t.size(d);
        c.strides[d] = t.stride(d);
    }
    c.format = format;
    return c;
}

// Views of a TensorList for the C ABI; keeps the camTensor structs alive.
struct CamList {
    std::vector<camTensor> items;
    std::vector<const camTensor *> ptrs;
    camTensorList list{};
    CamList(at::TensorList ts, int32_t format)
    {
        items.reserve(ts.size());
        for (const at::Tensor &t : ts) {
            items.push_back(to_cam(t, format));
        }
        for (const camTensor &c : items) {
            ptrs.push_back(&c);
        }
        list.tensors = ptrs.data();
        list.count = ptrs.size();
    }
};

void check(camStatus st, const char *op)
{
    TORCH_CHECK(st == CAM_OK, op, " failed with cam status ", (int)st, ": ", camGetRecentErrMsg());
}

typedef camStatus (*Phase2)(void *, uint64_t, camOpExecutor *, camStream_t);

// Phase 2 of an operator whose phase 1 has produced (bytes, executor).
void run_phase2(Phase2 fn, const char *op, uint64_t bytes, camOpExecutor *executor, const at::Tensor &like)
{
    // the workspace, the stream and the launches belong to the device the tensors live on
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(like.device());
    at::Tensor ws = at::empty({(int64_t)(bytes > 0 ? bytes : 1)}, like.options().dtype(at::kByte));
    const camStatus st = fn(ws.data_ptr(), bytes, executor,
                            (camStream_t)c10::hip::getCurrentHIPStream(like.device().index()).stream());
    check(st, op);
}

// ---- storages that hold packed weights: StorageImpl -> (weak reference, gate/up pairing)
struct PackedEntry {
    c10::weak_intrusive_ptr<c10::StorageImpl> storage;
    bool gate_up;
};
std::mutex g_packed_mutex;
std::unordered_map<const c10::StorageImpl *, PackedEntry> g_packed;

void remember_packed(const at::Tensor &t, bool gate_up)
{
    std::lock_guard<std::mutex> lock(g_packed_mutex);
    for (auto it = g_packed.begin(); it != g_packed.end();) {  // drop the entries of storages that are gone
        it = it->second.storage.expired() ? g_packed.erase(it) : std::next(it);
    }
    c10::StorageImpl *impl = t.storage().unsafeGetStorageImpl();
    g_packed.erase(impl);
    g_packed.emplace(impl, PackedEntry{t.storage().getWeakStorageImpl(), gate_up});
}

void require_packed(at::TensorList ws, bool gate_up, const char *name)
{
    std::lock_guard<std::mutex> lock(g_packed_mutex);
    for (const at::Tensor &w : ws) {
        auto it = g_packed.find(w.storage().unsafeGetStorageImpl());
        const bool ok = it != g_packed.end() && !it->second.storage.expired() && it->second.gate_up == gate_up;
        TORCH_CHECK(ok, name, " must be the result of umdk_cam_op_lib::prepack_weight(w, ", gate_up ? "True" : "False",
                    ") or a view of it (the counterpart of npu_format_cast(w, FRACTAL_NZ)); a clone()/to() copy "
                    "loses that mark");
    }
}

// ---- operators
at::Tensor prepack_weight(const at::Tensor &w, bool gate_up)
{
    at::Tensor src = w.contiguous();
    at::Tensor dst = at::empty_like(src);
    camTensor cs = to_cam(src), cd = to_cam(dst);
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camPrepackWeightGetWorkspaceSize(&cs, gate_up ? 1 : 0, &cd, &bytes, &ex), "camPrepackWeight");
    run_phase2(camPrepackWeight, "camPrepackWeight", bytes, ex, src);
    remember_packed(dst, gate_up);
    return dst;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> get_dispatch_layout(const at::Tensor &topk_idx, int64_t num_experts,
                                                                   int64_t num_ranks)
{
    TORCH_CHECK(topk_idx.dim() == 2, "Assertion failed: topkIdx.dim() == 2");
    TORCH_CHECK(topk_idx.is_contiguous(), "Assertion failed: topkIdx.is_contiguous()");
    TORCH_CHECK(num_experts > 0, "Assertion failed: numExperts > 0");
    const int64_t T = topk_idx.size(0), K = topk_idx.size(1);
    at::Tensor per_expert = at::empty({num_experts}, topk_idx.options().dtype(at::kInt));
    at::Tensor per_rank = at::empty({num_ranks}, topk_idx.options().dtype(at::kInt));
    at::Tensor in_rank = at::empty({T, num_ranks}, topk_idx.options().dtype(at::kBool));
    camTensor ci = to_cam(topk_idx), cr = to_cam(per_rank), ce = to_cam(per_expert), cb = to_cam(in_rank);
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camDispatchLayoutGetWorkspaceSize(&ci, T, num_ranks, num_experts, K, &cr, &ce, &cb, &bytes, &ex),
          "camDispatchLayout");
    run_phase2(camDispatchLayout, "camDispatchLayout", bytes, ex, topk_idx);
    return {per_rank, per_expert, in_rank};
}

// -> (expand_x [total,H], expand_idx int32 [3*total], recv_count int32 [E], num_recv_tokens_per_expert int64 on
// the CPU), total = max(rows received, 1) as in the reference (moe_dispatch_prefill.cpp:161-167).  The row total
// decides the output shapes, so 8 bytes come back to the host first (the reference brings two whole tensors back and
// loops over them).  num_worst_tokens only enters the reference's globalBs (:154-155), which one rank does not need.
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> moe_dispatch_prefill(
    const at::Tensor &x, const at::Tensor &topk_idx, const at::Tensor &topk_weights,
    const at::Tensor &num_tokens_per_rank, const at::Tensor &is_token_in_rank, const at::Tensor &num_tokens_per_expert,
    int64_t num_worst_tokens, c10::string_view group_ep, int64_t rank, int64_t num_ranks)
{
    (void)group_ep;
    TORCH_CHECK(is_token_in_rank.scalar_type() == at::kBool, "Assertion failed: isTokenInRank.scalar_type() == at::kBool");
    TORCH_CHECK(num_tokens_per_expert.scalar_type() == at::kInt,
                "Assertion failed: numTokensPerExpert.scalar_type() == at::kInt");
    TORCH_CHECK(num_tokens_per_rank.scalar_type() == at::kInt, "Assertion failed: numTokensPerRank.scalar_type() == at::kInt");
    TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "Assertion failed: newX.dim() == 2 and newX.is_contiguous()");
    TORCH_CHECK(is_token_in_rank.dim() == 2 && is_token_in_rank.is_contiguous(),
                "Assertion failed: isTokenInRank.dim() == 2 and isTokenInRank.is_contiguous()");
    TORCH_CHECK(is_token_in_rank.size(0) == x.size(0) && is_token_in_rank.size(1) == num_ranks,
                "Assertion failed: isTokenInRank.size(0) == newX.size(0) and isTokenInRank.size(1) == numRanks");
    TORCH_CHECK(num_tokens_per_expert.dim() == 1 && num_tokens_per_expert.is_contiguous(),
                "Assertion failed: numTokensPerExpert.dim() == 1 and numTokensPerExpert.is_contiguous()");
    TORCH_CHECK(num_ranks > 0 && num_tokens_per_expert.size(0) % num_ranks == 0,
                "Assertion failed: numTokensPerExpert.size(0) % numRanks == 0");
    TORCH_CHECK(num_tokens_per_rank.dim() == 1 && num_tokens_per_rank.size(0) == num_ranks,
                "Assertion failed: numTokensPerRank.size(0) == numRanks");
    const int64_t E = num_tokens_per_expert.size(0);
    TORCH_CHECK(E > 0, "Assertion failed: numExperts > 0");
    TORCH_CHECK(topk_idx.dim() == 2 && topk_idx.is_contiguous(),
                "Assertion failed: topkIdx.dim() == 2 and topkIdx.is_contiguous()");
    TORCH_CHECK(topk_weights.dim() == 2 && topk_weights.is_contiguous(),
                "Assertion failed: topkWeights.dim() == 2 and topkWeights.is_contiguous()");
    TORCH_CHECK(x.size(0) == topk_idx.size(0), "Assertion failed: numTokens == topkIdx.size(0)");
    TORCH_CHECK(topk_idx.size(1) == topk_weights.size(1), "Assertion failed: numTopk == topkWeights.size(1)");
    TORCH_CHECK(topk_weights.scalar_type() == at::kFloat, "Assertion failed: topkWeights.scalar_type() == at::kFloat");

    (void)num_worst_tokens;
    const int64_t T = x.size(0), H = x.size(1), K = topk_idx.size(1);
    const int64_t A = std::max<int64_t>(T * K, 1);
    auto i32 = x.options().dtype(at::kInt);
    at::Tensor recv_x = at::empty({A, H}, x.options());
    at::Tensor expand_idx = at::empty({3 * A}, i32);
    at::Tensor pos = at::empty({T, K}, i32);
    at::Tensor recv_count = at::empty({E}, i32);
    at::Tensor per_expert = at::empty({E / num_ranks}, x.options().dtype(at::kLong));
    at::Tensor total = at::empty({1}, x.options().dtype(at::kLong));
    camTensor cx = to_cam(x), ci = to_cam(topk_idx), crx = to_cam(recv_x), cidx = to_cam(expand_idx), cpos = to_cam(pos),
              crc = to_cam(recv_count), cpe = to_cam(per_expert), ct = to_cam(total);
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camMoeDispatchPrefillGetWorkspaceSize(&cx, &ci, E, num_ranks, rank, 0, &crx, nullptr, &cidx, &cpos, nullptr,
                                                nullptr, nullptr, &crc, &cpe, &ct, &bytes, &ex),
          "camMoeDispatchPrefill");
    run_phase2(camMoeDispatchPrefill, "camMoeDispatchPrefill", bytes, ex, x);
    const int64_t n = std::max<int64_t>(total.item<int64_t>(), 1);  // the one host round trip: the shapes need it
    recv_x = recv_x.narrow(0, 0, n);
    expand_idx = expand_idx.narrow(0, 0, 3 * n);
    return {recv_x, expand_idx, recv_count, per_expert.cpu()};
}

at::Tensor moe_combine_prefill(const at::Tensor &x, const at::Tensor &topk_idx, const at::Tensor &topk_weights,
                               const at::Tensor &src_idx, const at::Tensor &send_head, c10::string_view group_ep,
                               int64_t rank, int64_t num_ranks)
{
    TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "Assertion failed: x.dim() == 2 and x.is_contiguous()");
    const int64_t T = topk_weights.size(0);
    at::Tensor out = at::empty({T, x.size(1)}, x.options());
    camTensor cx = to_cam(x), cs = to_cam(src_idx), ch = to_cam(send_head), cw = to_cam(topk_weights), co = to_cam(out);
    std::string group(group_ep);
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camMoeCombineNormalGetWorkspaceSize(&cx, &cs, &ch, &cw, nullptr, group.data(), num_ranks, rank, group.data(), 1,
                                              0, send_head.size(0), topk_idx.size(0) * num_ranks, &co, &bytes, &ex),
          "camMoeCombineNormal");
    run_phase2(camMoeCombineNormal, "camMoeCombineNormal", bytes, ex, x);
    return out;
}

std::vector<at::Tensor> fused_deep_moe(const at::Tensor &x, const at::Tensor &expert_ids, at::TensorList w1,
                                       at::TensorList w1s, at::TensorList w2, at::TensorList w2s,
                                       const at::Tensor &expert_scales, const c10::optional<at::Tensor> &smooth,
                                       const c10::optional<at::Tensor> &mask, c10::string_view group_ep,
                                       int64_t ep_rank_size, int64_t ep_rank_id, int64_t moe_expert_num,
                                       int64_t shared_expert_num, int64_t shared_expert_rank_num, int64_t quant_mode,
                                       int64_t global_bs)
{
    TORCH_CHECK(x.dim() == 2, "x must be [bs, H]");
    require_packed(w1, true, "gmm1PermutedWeight");
    require_packed(w2, false, "gmm2Weight");
    at::Tensor output = at::empty({x.size(0), x.size(1)}, x.options());
    const bool shared = ep_rank_id < shared_expert_rank_num;
    const int64_t local = shared ? 1 : moe_expert_num / std::max<int64_t>(ep_rank_size - shared_expert_rank_num, 1);
    at::Tensor expert_token_nums = at::empty({local}, x.options().dtype(at::kLong));
    camTensor cx = to_cam(x), ci = to_cam(expert_ids), cs = to_cam(expert_scales), co = to_cam(output),
              cn = to_cam(expert_token_nums);
    CamList l1(w1, CAM_FORMAT_MFMA_B), l1s(w1s, CAM_FORMAT_ND), l2(w2, CAM_FORMAT_MFMA_B), l2s(w2s, CAM_FORMAT_ND);
    camTensor csm{}, cm{};
    const camTensor *psm = nullptr, *pm = nullptr;
    if (smooth.has_value() && smooth->defined()) {
        csm = to_cam(*smooth);
        psm = &csm;
    }
    if (mask.has_value() && mask->defined()) {
        cm = to_cam(*mask);
        pm = &cm;
    }
    std::string group(group_ep);
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camFusedDeepMoeGetWorkspaceSize(&cx, &ci, &l1.list, &l1s.list, &l2.list, &l2s.list, &cs, psm, pm, group.data(),
                                          ep_rank_size, ep_rank_id, moe_expert_num, shared_expert_num,
                                          shared_expert_rank_num, quant_mode, global_bs, &co, &cn, &bytes, &ex),
          "camFusedDeepMoe");
    run_phase2(camFusedDeepMoe, "camFusedDeepMoe", bytes, ex, x);
    return {output, expert_token_nums};
}

std::vector<at::Tensor> fused_deep_moe_meta(const at::Tensor &x, const at::Tensor &expert_ids, at::TensorList,
                                            at::TensorList, at::TensorList, at::TensorList, const at::Tensor &,
                                            const c10::optional<at::Tensor> &, const c10::optional<at::Tensor> &,
                                            c10::string_view, int64_t ep_rank_size, int64_t ep_rank_id,
                                            int64_t moe_expert_num, int64_t, int64_t shared_expert_rank_num, int64_t,
                                            int64_t)
{
    const bool shared = ep_rank_id < shared_expert_rank_num;
    const int64_t local = shared ? 1 : moe_expert_num / std::max<int64_t>(ep_rank_size - shared_expert_rank_num, 1);
    return {at::empty_like(x), at::empty({local}, expert_ids.options().dtype(at::kLong))};
}

const camTensor *opt_cam(const c10::optional<at::Tensor> &t, camTensor *slot)
{
    if (t.has_value() && t->defined()) {
        *slot = to_cam(*t);
        return slot;
    }
    return nullptr;
}

// Output shapes of src/cam/comm_operator/pybind/moe_dispatch_shmem.cpp:27-107.
std::vector<at::Tensor> dispatch_shmem_outputs(const at::Tensor &x, const at::Tensor &expert_ids, int64_t ep_world_size,
                                               int64_t ep_rank_id, int64_t moe_expert_num, int64_t tp_world_size,
                                               int64_t shared_expert_rank_num, int64_t quant_mode)
{
    TORCH_CHECK(x.dim() == 2 && expert_ids.dim() == 2, "x must be [bs, H] and expertIds [bs, K]");
    TORCH_CHECK(ep_world_size != shared_expert_rank_num, "Wrong parameters! Check the validation of sharedExpertRankNum");
    const bool shared = ep_rank_id < shared_expert_rank_num;
    const int64_t per_rank = moe_expert_num / (ep_world_size - shared_expert_rank_num);
    const int64_t bs = x.size(0), h = x.size(1), k = expert_ids.size(1);
    const int64_t rows = shared ? bs * ep_world_size / shared_expert_rank_num
                                : bs * ep_world_size * std::min<int64_t>(per_rank, k);
    auto ids = expert_ids.options();
    return {at::empty({rows, h}, quant_mode == 2 ? x.options().dtype(at::kChar) : x.options()),
            at::empty({rows}, x.options().dtype(at::kFloat)),
            at::empty({bs * k}, ids),
            at::empty({shared ? 1 : per_rank}, ids.dtype(at::kLong)),
            at::empty({shared ? ep_world_size : ep_world_size * per_rank}, ids),
            at::empty({tp_world_size}, ids)};
}

std::vector<at::Tensor> moe_dispatch_shmem(const at::Tensor &x, const at::Tensor &expert_ids,
                                           const c10::optional<at::Tensor> &scales,
                                           const c10::optional<at::Tensor> &mask, int64_t ep_world_size,
                                           int64_t ep_rank_id, int64_t moe_expert_num, int64_t tp_world_size,
                                           int64_t tp_rank_id, int64_t expert_shard_type, int64_t shared_expert_num,
                                           int64_t shared_expert_rank_num, int64_t quant_mode, int64_t global_bs,
                                           int64_t expert_token_nums_type, int64_t ext_info)
{
    std::vector<at::Tensor> out = dispatch_shmem_outputs(x, expert_ids, ep_world_size, ep_rank_id, moe_expert_num,
                                                         tp_world_size, shared_expert_rank_num, quant_mode);
    camTensor cx = to_cam(x), ci = to_cam(expert_ids), c0 = to_cam(out[0]), c1 = to_cam(out[1]), c2 = to_cam(out[2]),
              c3 = to_cam(out[3]), c4 = to_cam(out[4]), c5 = to_cam(out[5]);
    camTensor cs{}, cm{};
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camMoeDispatchShmemGetWorkspaceSize(&cx, &ci, opt_cam(scales, &cs), opt_cam(mask, &cm), ep_world_size,
                                              ep_rank_id, moe_expert_num, tp_world_size, tp_rank_id,
                                              expert_shard_type, shared_expert_num, shared_expert_rank_num, quant_mode,
                                              global_bs, expert_token_nums_type, ext_info, &c0, &c1, &c2, &c3, &c4, &c5,
                                              &bytes, &ex),
          "camMoeDispatchShmem");
    run_phase2(camMoeDispatchShmem, "camMoeDispatchShmem", bytes, ex, x);
    return out;
}

std::vector<at::Tensor> moe_dispatch_shmem_meta(const at::Tensor &x, const at::Tensor &expert_ids,
                                                const c10::optional<at::Tensor> &, const c10::optional<at::Tensor> &,
                                                int64_t ep_world_size, int64_t ep_rank_id, int64_t moe_expert_num,
                                                int64_t tp_world_size, int64_t, int64_t, int64_t,
                                                int64_t shared_expert_rank_num, int64_t quant_mode, int64_t, int64_t,
                                                int64_t)
{
    return dispatch_shmem_outputs(x, expert_ids, ep_world_size, ep_rank_id, moe_expert_num, tp_world_size,
                                  shared_expert_rank_num, quant_mode);
}

at::Tensor moe_combine_shmem(const at::Tensor &expand_x, const at::Tensor &expert_ids, const at::Tensor &expand_idx,
                             const at::Tensor &ep_send_counts, const at::Tensor &expert_scales,
                             const c10::optional<at::Tensor> &tp_send_counts, const c10::optional<at::Tensor> &mask,
                             const c10::optional<at::Tensor> &activation_scale,
                             const c10::optional<at::Tensor> &weight_scale, const c10::optional<at::Tensor> &group_list,
                             const c10::optional<at::Tensor> &expand_scales, int64_t ep_world_size, int64_t ep_rank_id,
                             int64_t moe_expert_num, int64_t tp_world_size, int64_t tp_rank_id,
                             int64_t expert_shard_type, int64_t shared_expert_num, int64_t shared_expert_rank_num,
                             int64_t global_bs, int64_t comm_quant_mode, int64_t ext_info, int64_t out_dtype,
                             int64_t group_list_type)
{
    TORCH_CHECK(expand_x.dim() == 2 && expert_ids.dim() == 2, "expandX must be [A, H] and expertIds [bs, K]");
    at::Tensor out = at::empty({expert_ids.size(0), expand_x.size(1)}, expand_x.options());
    camTensor cx = to_cam(expand_x), ci = to_cam(expert_ids), ce = to_cam(expand_idx), cc = to_cam(ep_send_counts),
              cw = to_cam(expert_scales), co = to_cam(out);
    camTensor t0{}, t1{}, t2{}, t3{}, t4{}, t5{};
    uint64_t bytes = 0;
    camOpExecutor *ex = nullptr;
    check(camMoeCombineShmemGetWorkspaceSize(&cx, &ci, &ce, &cc, &cw, opt_cam(tp_send_counts, &t0), opt_cam(mask, &t1),
                                             opt_cam(activation_scale, &t2), opt_cam(weight_scale, &t3),
                                             opt_cam(group_list, &t4), opt_cam(expand_scales, &t5), ep_world_size,
                                             ep_rank_id, moe_expert_num, tp_world_size, tp_rank_id, expert_shard_type,
                                             shared_expert_num, shared_expert_rank_num, global_bs, comm_quant_mode,
                                             ext_info, out_dtype, group_list_type, &co, &bytes, &ex),
          "camMoeCombineShmem");
    run_phase2(camMoeCombineShmem, "camMoeCombineShmem", bytes, ex, expand_x);
    return out;
}

at::Tensor moe_combine_shmem_meta(const at::Tensor &expand_x, const at::Tensor &expert_ids, const at::Tensor &,
                                  const at::Tensor &, const at::Tensor &, const c10::optional<at::Tensor> &,
                                  const c10::optional<at::Tensor> &, const c10::optional<at::Tensor> &,
                                  const c10::optional<at::Tensor> &, const c10::optional<at::Tensor> &,
                                  const c10::optional<at::Tensor> &, int64_t, int64_t, int64_t, int64_t, int64_t,
                                  int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t)
{
    return at::empty({expert_ids.size(0), expand_x.size(1)}, expand_x.options());
}

// ---- autograd: forward = the operator below the autograd key, backward = one undefined gradient per input.
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

template <int NumInputs>
variable_list no_gradients()
{
    return variable_list((size_t)NumInputs);
}

struct FusedDeepMoeFn : torch::autograd::Function<FusedDeepMoeFn> {
    static variable_list forward(AutogradContext *, const at::Tensor &x, const at::Tensor &ids, at::TensorList w1,
                                 at::TensorList w1s, at::TensorList w2, at::TensorList w2s, const at::Tensor &es,
                                 const c10::optional<at::Tensor> &smooth, const c10::optional<at::Tensor> &mask,
                                 c10::string_view group, int64_t a, int64_t b, int64_t c, int64_t d, int64_t e, int64_t f,
                                 int64_t g)
    {
        at::AutoDispatchBelowADInplaceOrView below;
        return fused_deep_moe(x, ids, w1, w1s, w2, w2s, es, smooth, mask, group, a, b, c, d, e, f, g);
    }
    static variable_list backward(AutogradContext *, variable_list) { return no_gradients<17>(); }
};

struct DispatchLayoutFn : torch::autograd::Function<DispatchLayoutFn> {
    static variable_list forward(AutogradContext *, const at::Tensor &idx, int64_t e, int64_t r)
    {
        at::AutoDispatchBelowADInplaceOrView below;
        auto t = get_dispatch_layout(idx, e, r);
        return {std::get<0>(t), std::get<1>(t), std::get<2>(t)};
    }
    static variable_list backward(AutogradContext *, variable_list) { return no_gradients<3>(); }
};

struct DispatchPrefillFn : torch::autograd::Function<DispatchPrefillFn> {
    static variable_list forward(AutogradContext *, const at::Tensor &x, const at::Tensor &idx, const at::Tensor &w,
                                 const at::Tensor &per_rank, const at::Tensor &in_rank, const at::Tensor &per_expert,
                                 int64_t worst, c10::string_view group, int64_t rank, int64_t ranks)
    {
        at::AutoDispatchBelowADInplaceOrView below;
        auto t = moe_dispatch_prefill(x, idx, w, per_rank, in_rank, per_expert, worst, group, rank, ranks);
        return {std::get<0>(t), std::get<1>(t), std::get<2>(t), std::get<3>(t)};
    }
    static variable_list backward(AutogradContext *, variable_list) { return no_gradients<10>(); }
};

struct CombinePrefillFn : torch::autograd::Function<CombinePrefillFn> {
    static at::Tensor forward(AutogradContext *, const at::Tensor &x, const at::Tensor &idx, const at::Tensor &w,
                              const at::Tensor &src, const at::Tensor &head, c10::string_view group, int64_t rank,
                              int64_t ranks)
    {
        at::AutoDispatchBelowADInplaceOrView below;
        return moe_combine_prefill(x, idx, w, src, head, group, rank, ranks);
    }
    static variable_list backward(AutogradContext *, variable_list) { return no_gradients<8>(); }
};

struct DispatchShmemFn : torch::autograd::Function<DispatchShmemFn> {
    static variable_list forward(AutogradContext *, const at::Tensor &x, const at::Tensor &ids,
                                 const c10::optional<at::Tensor> &scales, const c10::optional<at::Tensor> &mask,
                                 int64_t a, int64_t b, int64_t c, int64_t d, int64_t e, int64_t f, int64_t g, int64_t h,
                                 int64_t i, int64_t j, int64_t k, int64_t l)
    {
        at::AutoDispatchBelowADInplaceOrView below;
        return moe_dispatch_shmem(x, ids, scales, mask, a, b, c, d, e, f, g, h, i, j, k, l);
    }
    static variable_list backward(AutogradContext *, variable_list) { return no_gradients<16>(); }
};

struct CombineShmemFn : torch::autograd::Function<CombineShmemFn> {
    static at::Tensor forward(AutogradContext *, const at::Tensor &x, const at::Tensor &ids, const at::Tensor &eidx,
                              const at::Tensor &counts, const at::Tensor &w, const c10::optional<at::Tensor> &o0,
                              const c10::optional<at::Tensor> &o1, const c10::optional<at::Tensor> &o2,
                              const c10::optional<at::Tensor> &o3, const c10::optional<at::Tensor> &o4,
                              const c10::optional<at::Tensor> &o5, int64_t a, int64_t b, int64_t c, int64_t d,
                              int64_t e, int64_t f, int64_t g, int64_t h, int64_t i, int64_t j, int64_t k, int64_t l,
                              int64_t m)
    {
        at::AutoDispatchBelowADInplaceOrView below;
        return moe_combine_shmem(x, ids, eidx, counts, w, o0, o1, o2, o3, o4, o5, a, b, c, d, e, f, g, h, i, j, k, l, m);
    }
    static variable_list backward(AutogradContext *, variable_list) { return no_gradients<24>(); }
};

std::vector<at::Tensor> fused_deep_moe_autograd(const at::Tensor &x, const at::Tensor &ids, at::TensorList w1,
                                                at::TensorList w1s, at::TensorList w2, at::TensorList w2s,
                                                const at::Tensor &es, const c10::optional<at::Tensor> &smooth,
                                                const c10::optional<at::Tensor> &mask, c10::string_view group,
                                                int64_t a, int64_t b, int64_t c, int64_t d, int64_t e, int64_t f,
                                                int64_t g)
{
    return FusedDeepMoeFn::apply(x, ids, w1, w1s, w2, w2s, es, smooth, mask, group, a, b, c, d, e, f, g);
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> get_dispatch_layout_autograd(const at::Tensor &idx, int64_t e, int64_t r)
{
    variable_list v = DispatchLayoutFn::apply(idx, e, r);
    return {v[0], v[1], v[2]};
}

std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor> moe_dispatch_prefill_autograd(
    const at::Tensor &x, const at::Tensor &idx, const at::Tensor &w, const at::Tensor &per_rank,
    const at::Tensor &in_rank, const at::Tensor &per_expert, int64_t worst, c10::string_view group, int64_t rank,
    int64_t ranks)
{
    variable_list v = DispatchPrefillFn::apply(x, idx, w, per_rank, in_rank, per_expert, worst, group, rank, ranks);
    return {v[0], v[1], v[2], v[3]};
}

at::Tensor moe_combine_prefill_autograd(const at::Tensor &x, const at::Tensor &idx, const at::Tensor &w,
                                        const at::Tensor &src, const at::Tensor &head, c10::string_view group,
                                        int64_t rank, int64_t ranks)
{
    return CombinePrefillFn::apply(x, idx, w, src, head, group, rank, ranks);
}

std::vector<at::Tensor> moe_dispatch_shmem_autograd(const at::Tensor &x, const at::Tensor &ids,
                                                    const c10::optional<at::Tensor> &scales,
                                                    const c10::optional<at::Tensor> &mask, int64_t a, int64_t b,
                                                    int64_t c, int64_t d, int64_t e, int64_t f, int64_t g, int64_t h,
                                                    int64_t i, int64_t j, int64_t k, int64_t l)
{
    return DispatchShmemFn::apply(x, ids, scales, mask, a, b, c, d, e, f, g, h, i, j, k, l);
}

at::Tensor moe_combine_shmem_autograd(const at::Tensor &x, const at::Tensor &ids, const at::Tensor &eidx,
                                      const at::Tensor &counts, const at::Tensor &w,
                                      const c10::optional<at::Tensor> &o0, const c10::optional<at::Tensor> &o1,
                                      const c10::optional<at::Tensor> &o2, const c10::optional<at::Tensor> &o3,
                                      const c10::optional<at::Tensor> &o4, const c10::optional<at::Tensor> &o5,
                                      int64_t a, int64_t b, int64_t c, int64_t d, int64_t e, int64_t f, int64_t g,
                                      int64_t h, int64_t i, int64_t j, int64_t k, int64_t l, int64_t m)
{
    return CombineShmemFn::apply(x, ids, eidx, counts, w, o0, o1, o2, o3, o4, o5, a, b, c, d, e, f, g, h, i, j, k, l, m);
}

}  // namespace

TORCH_LIBRARY(umdk_cam_op_lib, m)
{
    m.def("fused_deep_moe(Tensor x, Tensor expertIds, Tensor[] gmm1PermutedWeight, "
          "Tensor[] gmm1PermutedWeightScale, Tensor[] gmm2Weight, Tensor[] gmm2WeightScale, "
          "Tensor expertScales, Tensor? expertSmoothScales, Tensor? xActiveMask, str groupEp, "
          "int epRankSize, int epRankId, int moeExpertNum, int sharedExpertNum, int sharedExpertRankNum, "
          "int quantMode, int globalBs) -> Tensor[]");
    m.def("get_dispatch_layout(Tensor topk_idx, int num_experts, int num_ranks) -> (Tensor, Tensor, Tensor)");
    m.def("moe_dispatch_prefill(Tensor x, Tensor topk_idx, Tensor topk_weights, Tensor num_tokens_per_rank, "
          "Tensor is_token_in_rank, Tensor num_tokens_per_expert, int num_worst_tokens, str group_ep, "
          "int rank, int num_ranks) -> (Tensor, Tensor, Tensor, Tensor)");
    m.def("moe_combine_prefill(Tensor x, Tensor topk_idx, Tensor topk_weights, Tensor src_idx, "
          "Tensor send_head, str group_ep, int rank, int num_ranks) -> Tensor");
    m.def("moe_dispatch_shmem(Tensor x, Tensor expertIds, Tensor? scales, Tensor? xActiveMask, "
          "int epWorldSize, int epRankId, int moeExpertNum, int tpWorldSize, int tpRankId, "
          "int expertShardType, int sharedExpertNum, int sharedExpertRankNum, int quantMode, int globalBS, "
          "int expertTokenNumsType, int extInfo) -> Tensor[]");
    m.def("moe_combine_shmem(Tensor expandX, Tensor expertIds, Tensor expandIdx, Tensor epSendCounts, "
          "Tensor expertScales, Tensor? tpSendCounts, Tensor? xActiveMask, Tensor? activationScale, "
          "Tensor? weightScale, Tensor? groupList, Tensor? expandScales, int epWorldSize, int epRankId, "
          "int moeExpertNum, int tpWorldSize, int tpRankId, int expertShardType, int sharedExpertNum, "
          "int sharedExpertRankNum, int globalBS, int commQuantMode, int extInfo, int outDtype, "
          "int groupListType) -> Tensor");
    m.def("prepack_weight(Tensor w, bool gate_up) -> Tensor");
}

TORCH_LIBRARY_IMPL(umdk_cam_op_lib, CUDA, m)
{
    m.impl("fused_deep_moe", &fused_deep_moe);
    m.impl("get_dispatch_layout", &get_dispatch_layout);
    m.impl("moe_dispatch_prefill", &moe_dispatch_prefill);
    m.impl("moe_combine_prefill", &moe_combine_prefill);
    m.impl("moe_dispatch_shmem", &moe_dispatch_shmem);
    m.impl("moe_combine_shmem", &moe_combine_shmem);
    m.impl("prepack_weight", &prepack_weight);
}

TORCH_LIBRARY_IMPL(umdk_cam_op_lib, AutogradCUDA, m)
{
    m.impl("fused_deep_moe", &fused_deep_moe_autograd);
    m.impl("get_dispatch_layout", &get_dispatch_layout_autograd);
    m.impl("moe_dispatch_prefill", &moe_dispatch_prefill_autograd);
    m.impl("moe_combine_prefill", &moe_combine_prefill_autograd);
    m.impl("moe_dispatch_shmem", &moe_dispatch_shmem_autograd);
    m.impl("moe_combine_shmem", &moe_combine_shmem_autograd);
}

// The fused and the SHMEM operators have shapes that follow from their arguments; the "normal" pair does not
// (src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:200).
TORCH_LIBRARY_IMPL(umdk_cam_op_lib, Meta, m)
{
    m.impl("fused_deep_moe", &fused_deep_moe_meta);
    m.impl("moe_dispatch_shmem", &moe_dispatch_shmem_meta);
    m.impl("moe_combine_shmem", &moe_combine_shmem_meta);
}
