// Routing plan kernels: per-expert counts, prefix offsets, the stable within-expert rank of every
// (token, k) entry and receive bookkeeping.
//
// Reference semantics restated here (paths relative to the reference tree):
//   counts        src/cam/comm_operator/ascend_kernels/dispatch_layout/op_kernel/dispatch_layout.h:83-134
//   offsets       src/cam/comm_operator/ascend_kernels/notify_dispatch/op_kernel/notify_dispatch.h:121-152
//   ranks         src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:96-112 (a CPU loop there)
//   recv cumsum   src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:126-145
//
// Design.  The rank of an entry is its position among earlier flat (t,k) entries with the same
// expert id, i.e. a stable counting sort; atomics would make the order depend on scheduling.  Two
// short launches, no atomics on results, no spinning, fully deterministic:
//   1. every workgroup ranks its own contiguous chunk of the flat id sequence (wave ballots + per-wave
//      LDS histograms) and publishes the chunk's per-expert histogram;
//   2. every workgroup sums the histograms of the chunks before it (its base), scans the per-expert
//      totals into offsets, and finishes its chunk.  The reference does this part on the CPU after a
//      device-to-host copy.
#include "cam_device.h"
#include "cam_kernels.h"
#include "rank_device.h"

namespace cam {

namespace {

constexpr int kScanThreads = 1024;  // single-workgroup scan kernel (notify)
constexpr int kGlobalThreads = 512; // phase 2: one thread per expert column

// Phase 1.  Workgroup b ranks the flat entries [b*chunk, (b+1)*chunk), chunk = IT*256 (rank_chunk), and
// publishes the chunk's per-expert histogram in hist_out[b][*].
template <typename IdT, int IT>
__global__ __launch_bounds__(kLocalThreads) void plan_local_kernel(PlanArgs a, int32_t *hist_out)
{
    __shared__ int hist[kLocalWaves * kMaxExperts];
    __shared__ int active_s;
    const int tid = threadIdx.x;
    const int b = blockIdx.x;
    const int t_active = count_active(a.mask, a.T, tid, kLocalThreads, &active_s);
    rank_chunk<IdT, IT>((const IdT *)a.idx, b, (long long)t_active * a.K, (long long)a.T * a.K, a.E, hist, a.pos,
                        hist_out + (long long)b * a.E);
    if (b == 0 && tid == 0) {
        hist_out[(long long)gridDim.x * a.E] = t_active;
    }
}

// Phase 2.  Every workgroup sums the histogram columns (all rows for the per-expert count, the rows
// before its own for its base), scans the counts into offsets, and finishes its own chunk:
// pos += base[e], dst_row = off[e] + pos.  Workgroup 0 also writes the per-expert outputs (counts, offsets,
// cumulative group list, receive bookkeeping), the total row count, the zeroed per-rank counters and the
// four words of the receive metadata.
template <typename IdT>
__global__ __launch_bounds__(kGlobalThreads) void plan_global_kernel(PlanArgs a, int chunk, const int32_t *hist_in)
{
    constexpr int NW = kGlobalThreads / kWave;
    __shared__ int base_s[kMaxExperts];
    __shared__ int off_s[kMaxExperts];
    __shared__ int scan_s[NW];
    __shared__ int total_s;
    const int tid = threadIdx.x;
    const int b = blockIdx.x;
    const int nb = gridDim.x;
    const int E = a.E;
    const IdT *__restrict__ idx = (const IdT *)a.idx;

    // This thread's first entry of the chunk is requested before the histogram columns, so that its round trip
    // to memory runs beside theirs instead of after the scan.
    const long long n_all = (long long)a.T * a.K;
    const long long lo = (long long)b * chunk;
    const long long hi = min(n_all, lo + chunk);
    const long long i0 = lo + tid;
    long long raw0 = -1;
    int pos0 = 0;
    if (i0 < hi) {
        raw0 = (long long)idx[i0];
        pos0 = a.pos[i0];
    }

    int cnt = 0, base = 0;
    if (tid < E) {
        const int32_t *col = hist_in + tid;
        int bb = 0;
        for (; bb + 64 <= nb; bb += 64) {  // 64 independent loads in flight per thread: one round trip at C2
            int v[64];
#pragma unroll
            for (int j = 0; j < 64; ++j) {
                v[j] = col[(long long)(bb + j) * E];
            }
#pragma unroll
            for (int j = 0; j < 64; ++j) {
                cnt += v[j];
                base += (bb + j) < b ? v[j] : 0;
            }
        }
        for (; bb + 8 <= nb; bb += 8) {
            int v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                v[j] = col[(long long)(bb + j) * E];
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                cnt += v[j];
                base += (bb + j) < b ? v[j] : 0;
            }
        }
        for (; bb < nb; ++bb) {
            const int v = col[(long long)bb * E];
            cnt += v;
            base += bb < b ? v : 0;
        }
    }
    const int off = block_exclusive_scan<NW>(cnt, tid, scan_s, &total_s);
    const int total = total_s;
    base_s[tid] = base;
    off_s[tid] = off;
    __syncthreads();

    const int t_active = hist_in[(long long)nb * E];
    const long long n = (long long)t_active * a.K;
    for (long long i = i0; i < hi; i += kGlobalThreads) {
        int e, p0;
        if (i == i0) {
            e = (i < n && raw0 >= 0 && raw0 < (long long)E) ? (int)raw0 : -1;
            p0 = pos0;
        } else {
            e = i < n ? load_id(idx, i, E) : -1;
            p0 = e >= 0 ? a.pos[i] : 0;
        }
        int row = -1;
        if (e >= 0) {
            const int p = p0 + base_s[e];
            a.pos[i] = p;
            row = off_s[e] + p;
        }
        if (a.dst_row != nullptr) {
            a.dst_row[i] = row;
        }
    }
    if (b != 0) {
        return;
    }
    if (tid < E) {
        if (a.cnt) a.cnt[tid] = cnt;
        if (a.off) a.off[tid] = off;
        if (a.recv_off) a.recv_off[tid] = off;
        if (a.recv_count) a.recv_count[tid] = off + cnt;
        if (a.tokens_per_expert) a.tokens_per_expert[tid] = cnt;
        if (a.group_list) a.group_list[tid] = (int64_t)off + cnt;
    }
    if (tid == 0 && a.total) {
        a.total[0] = total;
    }
    if (a.per_rank_zero != nullptr) {
        for (int r = tid; r < a.R; r += kGlobalThreads) {
            a.per_rank_zero[r] = 0;
        }
    }
    if (tid == 0 && a.meta != nullptr) {
        a.meta[0] = 0;
        a.meta[1] = total;
        a.meta[2] = t_active;
        a.meta[3] = 0;
    }
}

// Both phases in one workgroup, for id sequences that fit one chunk (at most 8 * 256 entries): the chunk's
// histogram is the per-expert count and every base is zero, so nothing has to pass between workgroups and the
// plan costs one launch instead of two.
template <typename IdT, int IT>
__global__ __launch_bounds__(kLocalThreads) void plan_single_kernel(PlanArgs a)
{
    __shared__ int hist[kLocalWaves * kMaxExperts];
    __shared__ int cnt_s[kMaxExperts];
    __shared__ int off_s[kMaxExperts];
    __shared__ int scan_s[kLocalWaves];
    __shared__ int total_s;
    __shared__ int active_s;
    const int tid = threadIdx.x;
    const int E = a.E;
    const IdT *__restrict__ idx = (const IdT *)a.idx;
    const int t_active = count_active(a.mask, a.T, tid, kLocalThreads, &active_s);
    const long long n = (long long)t_active * a.K;
    const long long n_all = (long long)a.T * a.K;
    rank_chunk<IdT, IT>(idx, 0, n, n_all, E, hist, a.pos, cnt_s);
    __syncthreads();  // cnt_s complete; the ranks in a.pos are visible to the whole workgroup
    // thread i owns experts 2i and 2i+1
    int c2[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        c2[h] = 2 * tid + h < E ? cnt_s[2 * tid + h] : 0;
    }
    const int pair_off = block_exclusive_scan<kLocalWaves>(c2[0] + c2[1], tid, scan_s, &total_s);
    const int total = total_s;
    const int o2[2] = {pair_off, pair_off + c2[0]};
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int e = 2 * tid + h;
        if (e < E) {
            off_s[e] = o2[h];
            if (a.cnt) a.cnt[e] = c2[h];
            if (a.off) a.off[e] = o2[h];
            if (a.recv_off) a.recv_off[e] = o2[h];
            if (a.recv_count) a.recv_count[e] = o2[h] + c2[h];
            if (a.tokens_per_expert) a.tokens_per_expert[e] = c2[h];
            if (a.group_list) a.group_list[e] = (int64_t)o2[h] + c2[h];
        }
    }
    __syncthreads();
    if (a.dst_row != nullptr) {
        for (long long i = tid; i < n_all; i += kLocalThreads) {
            const int e = i < n ? load_id(idx, i, E) : -1;
            a.dst_row[i] = e >= 0 ? off_s[e] + a.pos[i] : -1;
        }
    }
    if (tid == 0 && a.total) {
        a.total[0] = total;
    }
    if (a.per_rank_zero != nullptr) {
        for (int r = tid; r < a.R; r += kLocalThreads) {
            a.per_rank_zero[r] = 0;
        }
    }
    if (tid == 0 && a.meta != nullptr) {
        a.meta[0] = 0;
        a.meta[1] = total;
        a.meta[2] = t_active;
        a.meta[3] = 0;
    }
}

// isTokenInRank[t,r] and numTokensPerRank[r] (dispatch_layout.h:106-123): a token counts once per rank.
template <typename IdT, typename OutT>
__global__ __launch_bounds__(256) void in_rank_kernel(InRankArgs a)
{
    __shared__ int per_rank_s[kMaxRanks];
    const int tid = threadIdx.x;
    const int t0 = blockIdx.x * 256;
    const int nt = min(256, a.T - t0);
    const int R = a.R;
    const int epr = a.E / R;
    OutT *out = (OutT *)a.in_rank;
    for (int r = tid; r < R; r += 256) {
        per_rank_s[r] = 0;
    }
    for (long long i = tid; i < (long long)nt * R; i += 256) {
        out[(long long)t0 * R + i] = (OutT)0;
    }
    __syncthreads();
    if (tid < nt) {
        const IdT *ids = (const IdT *)a.idx + (long long)(t0 + tid) * a.K;
        int ranks[kMaxTopk];
        for (int k = 0; k < a.K; ++k) {
            int e = load_id(ids, k, a.E);
            int r = e < 0 ? -1 : e / epr;
            bool seen = false;
            for (int j = 0; j < k; ++j) {
                seen = seen || (ranks[j] == r);
            }
            ranks[k] = r;
            if (r >= 0 && r < R && !seen) {
                out[(long long)(t0 + tid) * R + r] = (OutT)1;
                atomicAdd(&per_rank_s[r], 1);
            }
        }
    }
    __syncthreads();
    for (int r = tid; r < R; r += 256) {
        if (per_rank_s[r] != 0) {
            atomicAdd(&a.per_rank[r], per_rank_s[r]);
        }
    }
}

__global__ __launch_bounds__(kScanThreads) void notify_scan_kernel(const int32_t *cnt, int E, int num_tokens,
                                                                  int32_t *off, int32_t *send_data,
                                                                  int32_t *recv_data)
{
    __shared__ int scan_s[kScanThreads / kWave];
    __shared__ int total_s;
    const int tid = threadIdx.x;
    int c = tid < E ? cnt[tid] : 0;
    int o = block_exclusive_scan<kScanThreads / kWave>(c, tid, scan_s, &total_s);
    if (tid < E) {
        if (off) off[tid] = o;
        if (send_data) {
            send_data[3 * tid + 0] = c;
            send_data[3 * tid + 1] = o;
            send_data[3 * tid + 2] = num_tokens;
        }
        if (recv_data) {
            recv_data[3 * tid + 0] = c;
            recv_data[3 * tid + 1] = o;
            recv_data[3 * tid + 2] = num_tokens;
        }
    }
}

template <typename IdT>
hipError_t launch_plan_t(const PlanArgs &a, int it, int nb, int32_t *hist, hipStream_t stream)
{
    dim3 grid(nb), blk(kLocalThreads);
    if (nb == 1) {
        switch (it) {
            case 1: hipLaunchKernelGGL((plan_single_kernel<IdT, 1>), grid, blk, 0, stream, a); break;
            case 2: hipLaunchKernelGGL((plan_single_kernel<IdT, 2>), grid, blk, 0, stream, a); break;
            case 4: hipLaunchKernelGGL((plan_single_kernel<IdT, 4>), grid, blk, 0, stream, a); break;
            default: hipLaunchKernelGGL((plan_single_kernel<IdT, 8>), grid, blk, 0, stream, a); break;
        }
        return hipGetLastError();
    }
    switch (it) {
        case 1: hipLaunchKernelGGL((plan_local_kernel<IdT, 1>), grid, blk, 0, stream, a, hist); break;
        case 2: hipLaunchKernelGGL((plan_local_kernel<IdT, 2>), grid, blk, 0, stream, a, hist); break;
        case 4: hipLaunchKernelGGL((plan_local_kernel<IdT, 4>), grid, blk, 0, stream, a, hist); break;
        default: hipLaunchKernelGGL((plan_local_kernel<IdT, 8>), grid, blk, 0, stream, a, hist); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        return e;
    }
    hipLaunchKernelGGL(plan_global_kernel<IdT>, grid, dim3(kGlobalThreads), 0, stream, a, it * kLocalThreads,
                       (const int32_t *)hist);
    return hipGetLastError();
}

}  // namespace

void plan_geometry(long long n_all, int *it_out, int *nb_out)
{
    int it = 1;
    if (n_all <= 8 * kLocalThreads) {  // one chunk: the single-workgroup plan
        while ((long long)it * kLocalThreads < n_all) {
            it *= 2;
        }
    } else {
        while (it < 8 && (n_all + (long long)it * kLocalThreads - 1) / ((long long)it * kLocalThreads) > 64) {
            it *= 2;
        }
    }
    long long nb = (n_all + (long long)it * kLocalThreads - 1) / ((long long)it * kLocalThreads);
    *it_out = it;
    *nb_out = (int)(nb < 1 ? 1 : nb);
}

uint64_t plan_workspace_bytes(int64_t T, int64_t K, int E)
{
    int it, nb;
    plan_geometry(T * K, &it, &nb);
    return ((uint64_t)nb * (uint64_t)E + 4) * sizeof(int32_t);
}

hipError_t launch_plan(const PlanArgs &a, hipStream_t stream)
{
    if (a.hist_ws == nullptr) {
        return hipErrorInvalidValue;
    }
    int it, nb;
    plan_geometry((long long)a.T * a.K, &it, &nb);
    if (a.idx_is64) {
        return launch_plan_t<int64_t>(a, it, nb, a.hist_ws, stream);
    }
    return launch_plan_t<int32_t>(a, it, nb, a.hist_ws, stream);
}

hipError_t launch_in_rank(const InRankArgs &a, hipStream_t stream)
{
    if (a.T <= 0) {
        return hipSuccess;
    }
    dim3 grid((a.T + 255) / 256);
    if (a.idx_is64) {
        if (a.in_rank_bytes == 4) {
            hipLaunchKernelGGL((in_rank_kernel<int64_t, int32_t>), grid, dim3(256), 0, stream, a);
        } else {
            hipLaunchKernelGGL((in_rank_kernel<int64_t, uint8_t>), grid, dim3(256), 0, stream, a);
        }
    } else {
        if (a.in_rank_bytes == 4) {
            hipLaunchKernelGGL((in_rank_kernel<int32_t, int32_t>), grid, dim3(256), 0, stream, a);
        } else {
            hipLaunchKernelGGL((in_rank_kernel<int32_t, uint8_t>), grid, dim3(256), 0, stream, a);
        }
    }
    return hipGetLastError();
}

hipError_t launch_notify_scan(const int32_t *cnt, int E, int num_tokens, int32_t *off, int32_t *send_data,
                              int32_t *recv_data, hipStream_t stream)
{
    hipLaunchKernelGGL(notify_scan_kernel, dim3(1), dim3(kScanThreads), 0, stream, cnt, E, num_tokens, off,
                       send_data, recv_data);
    return hipGetLastError();
}

}  // namespace cam
