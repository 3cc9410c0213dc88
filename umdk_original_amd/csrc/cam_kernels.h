// Host-callable launchers of the CAM HIP kernels.  Pointers are device pointers unless noted.
// Each launcher only enqueues work on `stream`; it never allocates or synchronises.
#ifndef CAM_KERNELS_H_
#define CAM_KERNELS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cam {

constexpr int kMaxExperts = 512;   // E <= 512 on every CAM operator
constexpr int kMaxRanks = 384;
constexpr int kMaxTopk = 16;
constexpr int kMaxListExperts = 64;  // per-expert weight tensors that fit in the kernel arguments
// GEMM schedule (device-built, one per GEMM launch): kSchedHeader ints, then the work items.
//   [0] item count  [1] total rows  [2] queues in use
//   [3] bit 0: no queue holds more than one item; bit 1: one queue per XCD, shared by its workgroups, instead
//       of one queue per workgroup
//   [kSchedQueueStart + w]     first item of queue w (w = 0 .. queues in use; the last entry is the end of the
//                              last queue)
//   [kSchedQueueCount + 32 w]  items already handed out from queue w (a workgroup's own queue starts at 1: the
//                              first item is its workgroup's without asking; a shared queue at 0; advanced by
//                              the GEMM); one counter per 128-byte line, so that the queues do not share a line
constexpr int kNumXcd = 8;       // workgroup i of a launch runs on XCD i % 8
constexpr int kMaxQueues = 512;  // one queue per workgroup of the persistent GEMM (one workgroup per CU)
constexpr int kSchedQueueStart = 4;
constexpr int kSchedQueueCount = 544;
constexpr int kSchedQueueStride = 32;
constexpr int kSchedHeader = kSchedQueueCount + kMaxQueues * kSchedQueueStride;
// One work item: rows [m0, m0 + rows) of expert g times column block nb.  flat != 0: at most 128 rows x 512
// packed columns, the two wave teams split the columns; flat == 0: at most 256 rows x 256 packed columns, team
// 0 takes tile rows [0, split), team 1 the rest.
struct SchedItem {
    int32_t g, m0, rows, split, nb, flat, pad0, pad1;
};
// Run metadata the plan kernels leave for the kernels after them: {0, total rows, active tokens, 0}.
constexpr int kPlanMeta = 4;

// ---------------------------------------------------------------------------------------------
// Routing plan: counts, offsets, within-expert ranks, receive bookkeeping, GEMM tile table.
struct PlanArgs {
    const void *idx;          // [T,K] int32 or int64
    int idx_is64;
    const uint8_t *mask;      // optional [T] bool; the number of set entries is the active prefix
    int T, K, E;
    int32_t *pos;             // [T,K]  required: rank within expert, -1 where skipped
    int32_t *dst_row;         // [T,K]  optional: off[e] + pos, -1 where skipped
    int32_t *cnt;             // [E]    optional
    int32_t *off;             // [E]    optional exclusive scan of cnt
    int32_t *recv_off;        // [E]    optional (== off on one rank)
    int32_t *recv_count;      // [E]    optional inclusive scan
    int64_t *tokens_per_expert;  // [E] optional
    int64_t *group_list;      // [E]    optional cumulative rows, int64
    int64_t *total;           // [1]    optional
    int32_t *per_rank_zero;   // [R]    optional: zeroed here so a later kernel can accumulate into it
    int R;
    int32_t *meta;            // optional run metadata, kPlanMeta ints (see above)
    int32_t *hist_ws;         // required scratch of plan_workspace_bytes(T, K, E) bytes
};
uint64_t plan_workspace_bytes(int64_t T, int64_t K, int E);
// Chunking of the flat id sequence: `it` ids per thread (1, 2, 4 or 8) and `nb` workgroups of 256 threads.
void plan_geometry(long long n_all, int *it_out, int *nb_out);
hipError_t launch_plan(const PlanArgs &a, hipStream_t stream);

// isTokenInRank / numTokensPerRank (per_rank must have been zeroed on the same stream).
struct InRankArgs {
    const void *idx;
    int idx_is64;
    int T, K, E, R;
    void *in_rank;     // [T,R] int32 or 1-byte
    int in_rank_bytes; // 4 or 1
    int32_t *per_rank; // [R]
};
hipError_t launch_in_rank(const InRankArgs &a, hipStream_t stream);

// NotifyDispatch on one rank: exclusive scan + triplets.
hipError_t launch_notify_scan(const int32_t *cnt, int E, int num_tokens, int32_t *off, int32_t *send_data,
                              int32_t *recv_data, hipStream_t stream);

// GEMM schedules from a group list (cumulative or per-expert counts, int64): one launch builds the schedule of
// one or two GEMMs over the same rows (they differ in the number of weight columns).
struct SchedSpec {
    int N;             // packed weight columns of the GEMM
    int Kd;            // its reduction length (the cost model of the builder needs it)
    int swiglu;        // its epilogue forms SiLU(gate) * up (costlier per row than a plain dequantisation)
    int max_items;     // capacity of the item table (sched_max_items)
    int32_t *sched;    // sched_bytes() of device memory
};
int sched_max_items(int64_t max_rows, int G, int N);
uint64_t sched_bytes(int64_t max_rows, int G, int N);
hipError_t launch_build_sched(const int64_t *group_list, int cumulative, int G, int64_t max_rows, int nspec,
                              const SchedSpec *specs, hipStream_t stream);
// The same job as kernel arguments: nspec == 0 means "nothing to build".
struct SchedBuild {
    const int64_t *group_list;
    int cumulative, G, nspec;
    int queues;        // workgroups of the GEMM launch the schedule is for (set by the launchers: CUs of the device)
    int parts;         // workgroups that share the building of one schedule (set by the launchers, 1..8)
    long long max_rows;
    SchedSpec spec[2];
};
// CUs of the current device = workgroups of a GEMM launch = queues of its schedule.
hipError_t gemm_workgroups(int *out);

// ---------------------------------------------------------------------------------------------
// Permute (+ per-token int8 quantisation).
struct DispatchArgs {
    const uint16_t *x;   // [T,H] bf16 bits
    const int32_t *idx;  // [T,K]
    const int32_t *send_offset, *send_token_idx, *recv_offset, *recv_count;  // row = see cam_mi355x.h
    const int32_t *dst_row;  // if non-null, used instead of the four arrays above
    int T, K, H, E;
    int64_t A;           // rows in the outputs
    int quant;           // 0 copy, 1 = epsilon variant, 2 = no-epsilon variant (int8, one fp32 scale per row),
                         // 3 = FP8 E4M3 with one E8M0 scale per row and 128 columns (scales: uint8 [A, H/128])
    int x_is_fp16;       // activations are IEEE fp16 instead of bf16 (matters only when quantising)
    void *out;           // [A,H] bf16 bits or int8
    float *scales;       // [A]   (quant only)
    int32_t *src_info;   // [3A]  optional
    int src_rank;
    // quant == 2 only: optional per-expert smooth scales fp32 [E,H].  Copy (t,k) is then quantised on its own,
    // from float(x[t]) * smooth[idx[t,k]] (moe_dispatch_shmem.h:693-733); idx must be set.
    const float *smooth;
    // GEMM schedules to build in the same launch (sched.nspec > 0): sched.nspec extra workgroups do what
    // launch_build_sched would, beside the ones that move rows.  The group list must be complete before the
    // launch (it is when it comes from launch_plan on the same stream).  sched.queues is set by the launcher.
    SchedBuild sched;
};
hipError_t launch_dispatch(const DispatchArgs &a, hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Combine.
// row_limit: optional device scalar; rows >= *row_limit are ignored (they were never written).
hipError_t launch_invert_src_info(const int32_t *src_info, int64_t A, const int32_t *row_limit, int T, int K,
                                  int32_t *slot_row, hipStream_t stream);
struct CombineArgs {
    const uint16_t *y;        // [A,H] bf16 bits, or wire rows [A, H + H/4] bytes (wire_rows != 0)
    int wire_rows;            // rows are H int8 values + H/8 block scales of the activation type (launch_comm_quant's output)
    int act_fp16;             // rows and output are IEEE fp16 instead of bf16 (not with wire_rows)
    const int32_t *slot_row;  // [T,K] row of slot (t,k) (<0: skip)
    const int32_t *src_info;  // optional: when set, slot_row entries are verified against the triples
    const float *w;           // [T,K]
    int T, K, H;
    int64_t A;
    const int32_t *row_limit; // optional device scalar: rows >= *row_limit are never read
    const int32_t *t_active;  // optional device scalar: tokens >= *t_active produce zero rows
    const uint16_t *shared;   // optional [T,H] rows of the output's type, added un-weighted after the routed rows
    uint16_t *out;            // [T,H]
};
hipError_t launch_combine(const CombineArgs &a, hipStream_t stream);
// slot_row[i] = (e ? ep_send_counts[e-1] : 0) + expand_idx[i] for e = ids[i] in [0,E) and a row below A, else -1
// (how the SHMEM combine finds the row of slot i: moe_combine_shmem.h:514-556,833-837).
hipError_t launch_rows_from_counts(const int32_t *ids, const int32_t *expand_idx, const int32_t *ep_send_counts,
                                   int64_t n, int E, int64_t A, int32_t *slot_row, hipStream_t stream);
// bf16 rows [A,H] -> wire rows [A, H + H/4] bytes: per block of 8 columns int8 values and one bf16 scale.
// row_limit: optional device scalar; rows >= *row_limit are left untouched.
hipError_t launch_comm_quant(const uint16_t *y, int act_fp16, int64_t A, int H, const int32_t *row_limit, uint8_t *out,
                             hipStream_t stream);

// ---------------------------------------------------------------------------------------------
// Grouped int8 GEMM.
struct WeightPtrs {
    const int8_t *w[kMaxListExperts];   // used when per_expert != 0
    const float *s[kMaxListExperts];
};
enum GemmEpilogue { kEpiInt32 = 0, kEpiSwiglu = 1, kEpiDequantBf16 = 2, kEpiSwigluFp8 = 3 };
struct GemmArgs {
    const int8_t *a;       // [A,Kd] int8
    const float *a_scale;  // [A]
    const int8_t *w;       // stacked packed weights [G,Kd,N] (per_expert == 0)
    const float *w_scale;  // stacked [G,N]
    int per_expert;        // weights given per expert through `list`
    WeightPtrs list;
    int32_t *sched;        // schedule built for this launch (its queue counters are consumed by the launch)
    // Block-scaled FP8 (fp8 != 0; include/cam_fp8_spec.h): a and w hold E4M3 bytes, the fp32 scales above are
    // unused, and every 128 bytes of K carry a power-of-two scale (E8M0 byte) per activation row and per 128
    // weight columns.  Stacked weights only.  Epilogues: kEpiInt32 stores the fp32 sums, kEpiSwiglu stores
    // silu(gate) * up as fp32, kEpiDequantBf16 stores bf16(sum), kEpiSwigluFp8 (FP8 only) stores that product
    // already quantised for the next GEMM: E4M3 bytes in out [A,N/2] and one E8M0 byte per row and 128 columns
    // in out_scale8 [A,N/256], bit-identical to kEpiSwiglu followed by launch_requant_fp8.
    int fp8;
    const uint8_t *a_scale8;  // [A, Kd/128]
    const uint8_t *w_scale8;  // [G, Kd/128, N/128]
    int Kd, N;             // N = logical columns of the weight
    int gate_up;           // weight prepacked with gate/up pairing
    int epilogue;
    void *out;             // int32 [A,N] | fp32 [A,N/2] | bf16 bits [A,N]
    int out_fp16;          // kEpiDequantBf16 writes IEEE fp16 instead of bf16
    uint8_t *out_scale8;   // kEpiSwigluFp8: [A, N/256]
};
hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream);

// fp32 SwiGLU products [rows,I] -> int8 + per-row scale.  sched_for_rows: optional schedule whose header holds
// the number of valid rows.
hipError_t launch_requant(const float *y, int64_t max_rows, int I, const int32_t *sched_for_rows, int8_t *q,
                          float *scale, hipStream_t stream);

hipError_t launch_prepack(const int8_t *src, int8_t *dst, int G, int Kd, int N, int gate_up, hipStream_t stream);

// fp32 rows [rows, I] -> E4M3 bytes + one E8M0 scale per row and 128 columns (I % 128 == 0).  sched_for_rows as
// for launch_requant.
hipError_t launch_requant_fp8(const float *y, int64_t max_rows, int I, const int32_t *sched_for_rows, uint8_t *q,
                              uint8_t *scale, hipStream_t stream);

}  // namespace cam

#endif  // CAM_KERNELS_H_
