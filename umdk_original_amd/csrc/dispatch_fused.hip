// Routing plan and token permutation (+ per-token int8 quantisation) in ONE launch.
//
// Reference semantics (paths relative to the reference tree): the whole body of the binding-level
// operator src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:96-192 -- the CPU loop that ranks every
// (token, k) entry inside its expert (:96-112), the CPU loop over the exchanged counts (:126-145) and the
// dispatch kernel call (:164-190, src/cam/comm_operator/ascend_kernels/moe_dispatch_normal/op_kernel/
// moe_dispatch_normal.h:278-396,486-535) -- for one rank.
//
// Design.  A destination row depends on every id before it, so the plan has to be complete before the
// first row can be placed; run as separate launches, the plan's few microseconds of latency-bound work
// sit in front of the bandwidth-bound permute.  Here the grid has three kinds of workgroups:
//   * workgroups [0, nb) first rank one chunk of 2048 flat ids each (rank_chunk), publish the chunk's
//     per-expert histogram and the chunk-local ranks, then raise their tag;
//   * workgroup nb, the finisher, first waits for the nb tags, turns the histograms into per-(chunk,
//     expert) bases and per-expert offsets, writes the plan's per-expert outputs, then raises the flag;
//   * every workgroup (those above once their plan duty is done) then handles four tokens, one wavefront
//     each: load the token row and quantise it in registers -- none of which needs the plan -- and only
//     then wait for the flag, compute the K destination rows (offset + chunk base + chunk-local rank)
//     and store.
// The plan therefore runs underneath the first row loads.  Waiting is safe because workgroups are
// started in index order: the ones being waited for never wait themselves and are resident before any
// waiter.  Every wait is bounded; a wave that gives up raises an error word and stores nothing.
// Everything one workgroup hands to another (histograms, chunk-local ranks, bases, offsets, tags, flag) is
// written with device-scope write-through stores and read with device-scope loads, and a tag or flag is
// raised only after the stores before it have completed.  A release or acquire FENCE at device scope is
// deliberately not used: on this part it writes back, or invalidates, a whole L2, which costs several
// microseconds per fence while the row traffic is in flight.
// The tags and the flag live in the caller's workspace.  A launch leaves them cleared (the last token
// workgroup to finish does it), and "raised" means "equal to a 64-bit magic number", so a workspace
// that has never been used, whatever it holds, reads as "not raised".
#include "cam_device.h"
#include "cam_kernels.h"
#include "permute_device.h"
#include "rank_device.h"

namespace cam {

namespace {

constexpr int kFusedIT = 8;                              // ids per thread of a ranking workgroup
constexpr int kFusedChunk = kFusedIT * kLocalThreads;    // 2048 flat ids per chunk
constexpr unsigned long long kRaised = 0x43414d5f504c414eull;
constexpr int kSpinLimit = 1 << 21;                      // polls (about a second) before a waiter gives up

__device__ __forceinline__ unsigned long long peek(const unsigned long long *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ int peek_i32(const int32_t *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bool wait_raised(const unsigned long long *p)
{
    for (int i = 0; i < kSpinLimit; ++i) {
        if (peek(p) == kRaised) {
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // orders the loads that follow; no cache action
            return true;
        }
        __builtin_amdgcn_s_sleep(16);
    }
    return false;
}

__device__ __forceinline__ void poke_i32(int32_t *p, int v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// All threads: wait until this thread's write-through stores have completed, then meet at the barrier.
__device__ __forceinline__ void stores_done_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0) on gfx9
    __syncthreads();
}

__device__ __forceinline__ void raise(unsigned long long *p)
{
    __hip_atomic_store(p, kRaised, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Workspace words used by one launch (64-bit each): tags[kFusedMaxChunks], flag, finished-workgroup counter,
// error counter.
constexpr int kCtrlFlag = kFusedMaxChunks;
constexpr int kCtrlDone = kFusedMaxChunks + 1;
constexpr int kCtrlErr = kFusedMaxChunks + 2;

template <typename IdT, int QUANT, int ACT>
__global__ __launch_bounds__(kLocalThreads) void dispatch_fused_kernel(FusedDispatchArgs a)
{
    __shared__ int hist[kLocalWaves * kMaxExperts];
    __shared__ int scan_s[kLocalWaves];
    __shared__ int total_s;
    __shared__ int ok_s;
    const int tid = threadIdx.x;
    const int b = blockIdx.x;
    const int nb = a.nb;
    const int E = a.p.E;
    const int K = a.p.K;
    int32_t *table = a.p.hist_ws;                        // [nb][E] chunk histograms, then chunk bases
    int32_t *off_ws = table + (long long)nb * E + 4;     // [E] exclusive offsets
    unsigned long long *ctrl = a.ctrl;

    if (b < nb) {
        // ---- ranking workgroup
        const int t_active = count_active(a.p.mask, a.p.T, tid, kLocalThreads, &total_s);
        rank_chunk<IdT, kFusedIT, true>((const IdT *)a.p.idx, b, (long long)t_active * K, (long long)a.p.T * K, E,
                                        hist, a.p.pos, table + (long long)b * E);
        if (b == 0 && tid == 0) {
            poke_i32(&table[(long long)nb * E], t_active);
        }
        stores_done_barrier();
        if (tid == 0) {
            raise(&ctrl[b]);
        }
    } else if (b == nb) {
        // ---- finisher
        bool ok = true;
        for (int j = tid; j < nb; j += kLocalThreads) {
            ok = wait_raised(&ctrl[j]) && ok;
        }
        if (tid == 0) {
            ok_s = 1;
        }
        __syncthreads();
        if (!ok) {
            ok_s = 0;
        }
        __syncthreads();
        if (ok_s == 0) {
            if (tid == 0) {
                atomicAdd(&ctrl[kCtrlErr], 1ull);
            }
            return;  // the flag stays down: every token workgroup gives up as well
        }
        const int t_active = peek_i32(&table[(long long)nb * E]);
        // Thread i owns experts 2i and 2i+1: chunk histograms -> exclusive prefix over the chunks (in place).
        int cnt2[2] = {0, 0};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int e = 2 * tid + h;
            if (e < E) {
                int32_t *col = table + e;
                int run = 0;
                int bb = 0;
                for (; bb + 16 <= nb; bb += 16) {  // 16 independent loads in flight
                    int v[16];
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        v[j] = peek_i32(&col[(long long)(bb + j) * E]);
                    }
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        poke_i32(&col[(long long)(bb + j) * E], run);
                        run += v[j];
                    }
                }
                for (; bb < nb; ++bb) {
                    const int v = peek_i32(&col[(long long)bb * E]);
                    poke_i32(&col[(long long)bb * E], run);
                    run += v;
                }
                cnt2[h] = run;
            }
        }
        const int pair_off = block_exclusive_scan<kLocalWaves>(cnt2[0] + cnt2[1], tid, scan_s, &total_s);
        const int total = total_s;
        const int off2[2] = {pair_off, pair_off + cnt2[0]};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int e = 2 * tid + h;
            if (e < E) {
                poke_i32(&off_ws[e], off2[h]);
                if (a.p.cnt) a.p.cnt[e] = cnt2[h];
                if (a.p.off) a.p.off[e] = off2[h];
                if (a.p.recv_off) a.p.recv_off[e] = off2[h];
                if (a.p.recv_count) a.p.recv_count[e] = off2[h] + cnt2[h];
                if (a.p.tokens_per_expert) a.p.tokens_per_expert[e] = cnt2[h];
                if (a.p.group_list) a.p.group_list[e] = (int64_t)off2[h] + cnt2[h];
            }
        }
        if (tid == 0 && a.p.total) {
            a.p.total[0] = total;
        }
        if (tid == 0 && a.p.meta != nullptr) {
            a.p.meta[0] = 0;
            a.p.meta[1] = total;
            a.p.meta[2] = t_active;
            a.p.meta[3] = 0;
        }
        if (tid == 0) {
            __hip_atomic_store(&ctrl[kCtrlDone], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        stores_done_barrier();
        if (tid == 0) {
            raise(&ctrl[kCtrlFlag]);
        }
    }

    // ---- every workgroup, the first nb + 1 after their plan duty: one wavefront per token
    const int lane = tid & (kWave - 1);
    const int t = b * kDispWaves + (tid >> 6);
    const bool have_token = t < a.p.T;
    TokenRow r;
    if (have_token) {
        load_token_row(a.x, t, a.H, lane, r);
        if (QUANT != 0) {
            quant_token_row<QUANT, ACT>(r);
        }
    }
    if (tid == 0) {
        ok_s = wait_raised(&ctrl[kCtrlFlag]) ? 1 : 0;
    }
    __syncthreads();
    if (ok_s == 0) {
        if (tid == 0) {
            atomicAdd(&ctrl[kCtrlErr], 1ull);
        }
        return;
    }
    if (have_token) {
        // Lane k resolves entry (t, k); the rows are then handed round with readlane.
        int my_row = -1;
        if (lane < K) {
            const long long i = (long long)t * K + lane;
            const int t_active = peek_i32(&table[(long long)nb * E]);
            const int e = t < t_active ? load_id((const IdT *)a.p.idx, i, E) : -1;
            int pos = -1;
            if (e >= 0) {
                const int chunk = (int)(i / kFusedChunk);
                pos = peek_i32(&table[(long long)chunk * E + e]) + peek_i32(&a.p.pos[i]);
                my_row = peek_i32(&off_ws[e]) + pos;
            }
            a.p.pos[i] = pos;
            if (a.p.dst_row != nullptr) {
                a.p.dst_row[i] = my_row;
            }
        }
        for (int k = 0; k < K; ++k) {
            const long long row = __shfl(my_row, k, kWave);
            if (row < 0 || row >= a.A) {
                continue;
            }
            store_token_row<QUANT>(r, a.out, a.scales, a.src_info, a.src_rank, row, t, k, a.H, lane);
        }
    }
    __syncthreads();
    if (tid == 0) {
        const unsigned long long token_blocks = gridDim.x;
        if (atomicAdd(&ctrl[kCtrlDone], 1ull) == token_blocks - 1) {
            // Last one out: leave the workspace as "not raised" for the next launch that uses it.
            for (int j = 0; j < nb; ++j) {
                ctrl[j] = 0ull;
            }
            ctrl[kCtrlFlag] = 0ull;
        }
    }
}

template <typename IdT>
hipError_t launch_t(const FusedDispatchArgs &a, dim3 grid, hipStream_t stream)
{
    const dim3 blk(kLocalThreads);
    if (a.quant == 0) {
        hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 0, 0>), grid, blk, 0, stream, a);
    } else if (a.quant == 1) {
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 1, 1>), grid, blk, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 1, 0>), grid, blk, 0, stream, a);
        }
    } else if (a.quant == 3) {
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 3, 1>), grid, blk, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 3, 0>), grid, blk, 0, stream, a);
        }
    } else {
        if (a.x_is_fp16) {
            hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 2, 1>), grid, blk, 0, stream, a);
        } else {
            hipLaunchKernelGGL((dispatch_fused_kernel<IdT, 2, 0>), grid, blk, 0, stream, a);
        }
    }
    return hipGetLastError();
}

}  // namespace

bool fused_dispatch_fits(int64_t T, int64_t K)
{
    return T >= 1 && (T * K + kFusedChunk - 1) / kFusedChunk <= kFusedMaxChunks;
}

uint64_t fused_dispatch_table_bytes(int64_t T, int64_t K, int E)
{
    const uint64_t nb = (uint64_t)((T * K + kFusedChunk - 1) / kFusedChunk);
    return ((nb < 1 ? 1 : nb) * (uint64_t)E + 4 + (uint64_t)E) * sizeof(int32_t);
}

uint64_t fused_dispatch_ctrl_bytes() { return (uint64_t)kFusedCtrlWords * sizeof(unsigned long long); }

hipError_t launch_dispatch_fused(FusedDispatchArgs a, hipStream_t stream)
{
    if (!fused_dispatch_fits(a.p.T, a.p.K) || a.p.hist_ws == nullptr || a.ctrl == nullptr || a.p.pos == nullptr) {
        return hipErrorInvalidValue;
    }
    if (a.H % 8 != 0 || a.H / 8 > kDispMaxChunks * kWave || (a.quant == 3 && a.H % 128 != 0)) {
        return hipErrorInvalidValue;
    }
    const long long n_all = (long long)a.p.T * a.p.K;
    a.nb = (int)((n_all + kFusedChunk - 1) / kFusedChunk);
    const long long token_blocks = (a.p.T + kDispWaves - 1) / kDispWaves;
    const long long blocks = token_blocks > a.nb + 1 ? token_blocks : a.nb + 1;
    if (blocks > 0x7fffffffll) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((unsigned)blocks);
    return a.p.idx_is64 ? launch_t<int64_t>(a, grid, stream) : launch_t<int32_t>(a, grid, stream);
}

}  // namespace cam
