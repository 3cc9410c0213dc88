// Routing plan kernels: per-expert counts, prefix offsets, the stable within-expert rank of every
// (token, k) entry, receive bookkeeping and the GEMM tile table.
//
// Reference semantics restated here (paths relative to the reference tree):
//   counts        src/cam/comm_operator/ascend_kernels/dispatch_layout/op_kernel/dispatch_layout.h:83-134
//   offsets       src/cam/comm_operator/ascend_kernels/notify_dispatch/op_kernel/notify_dispatch.h:121-152
//   ranks         src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:96-112 (a CPU loop there)
//   recv cumsum   src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:126-145
//
// Design.  The rank of an entry is its position among earlier flat (t,k) entries with the same
// expert id, i.e. a stable counting sort; atomics would make the order depend on scheduling.  All
// integer work of one call is a few hundred KB, so one 1024-thread workgroup does it in a single
// launch: each of the 16 waves owns a contiguous slice of the flat id sequence and ranks 64 ids at a
// time with wave ballots (lanes holding the same id find each other bit by bit), keeping a private
// running histogram in LDS; a scan across the 16 histograms then turns wave-local ranks into global
// ones.  No inter-workgroup synchronisation, no atomics, fully deterministic.
#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

namespace {

constexpr int kPlanThreads = 1024;
constexpr int kPlanWaves = kPlanThreads / kWave;
constexpr int kUnroll = 4;

template <typename IdT>
__device__ __forceinline__ int load_id(const IdT *p, int i, int E)
{
    long long v = (long long)p[i];
    return (v < 0 || v >= (long long)E) ? -1 : (int)v;
}

// Exclusive scan of one value per thread for tid < 512 (others pass 0); returns the exclusive prefix
// and leaves the grand total in *total_out (LDS).  Uses `scratch` (>= 16 ints of LDS).
__device__ __forceinline__ int block_exclusive_scan(int v, int tid, int *scratch, int *total_out)
{
    int lane = tid & (kWave - 1);
    int w = tid >> 6;
    int inc = wave_inclusive_scan(v, lane);
    if (lane == kWave - 1) {
        scratch[w] = inc;
    }
    __syncthreads();
    if (w == 0) {
        int t = lane < kPlanWaves ? scratch[lane] : 0;
        int ti = wave_inclusive_scan(t, lane);
        if (lane < kPlanWaves) {
            scratch[lane] = ti - t;
        }
        if (lane == kPlanWaves - 1) {
            *total_out = ti;
        }
    }
    __syncthreads();
    int r = inc - v + scratch[w];
    __syncthreads();
    return r;
}

template <typename IdT>
__global__ __launch_bounds__(kPlanThreads) void plan_kernel(PlanArgs a)
{
    __shared__ int hist[kPlanWaves * kMaxExperts];  // 32 KB: running per-wave histograms
    __shared__ int off_s[kMaxExperts];
    __shared__ int scan_s[kPlanWaves];
    __shared__ int total_s;
    __shared__ int active_s;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = tid >> 6;
    const int E = a.E;
    const IdT *__restrict__ idx = (const IdT *)a.idx;
    int32_t *__restrict__ pos = a.pos;

    for (int i = tid; i < kPlanWaves * kMaxExperts; i += kPlanThreads) {
        hist[i] = 0;
    }
    // Active prefix length: number of set mask entries (all tokens when there is no mask).
    int t_active = a.T;
    if (a.mask != nullptr) {
        int c = 0;
        for (int t = tid; t < a.T; t += kPlanThreads) {
            c += a.mask[t] != 0 ? 1 : 0;
        }
        c = wave_sum(c);
        if (tid == 0) {
            active_s = 0;
        }
        __syncthreads();
        if (lane == 0) {
            atomicAdd(&active_s, c);
        }
        __syncthreads();
        t_active = active_s;
    }
    __syncthreads();

    const int n = t_active * a.K;
    const int n_all = a.T * a.K;
    int per_wave = (n + kPlanWaves - 1) / kPlanWaves;
    per_wave = (per_wave + kWave - 1) & ~(kWave - 1);
    const int beg = min(n, w * per_wave);
    const int end = min(n, beg + per_wave);
    int nbits = 0;
    while ((1 << nbits) < E) {
        ++nbits;
    }
    int *my_hist = hist + w * kMaxExperts;
    const unsigned long long lt_mask = (1ull << lane) - 1ull;

    // Pass 1: wave-local stable ranks.
    for (int base = beg; base < end; base += kWave * kUnroll) {
        int e[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int i = base + u * kWave + lane;
            e[u] = i < end ? load_id(idx, i, E) : -1;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int i = base + u * kWave + lane;
            bool act = e[u] >= 0;
            unsigned long long peers = __ballot(act);
            for (int b = 0; b < nbits; ++b) {
                bool bit = act && ((e[u] >> b) & 1);
                unsigned long long bal = __ballot(bit);
                peers &= bit ? bal : ~bal;
            }
            int r = -1;
            int prior = 0;
            if (act) {
                prior = my_hist[e[u]];
                r = prior + __popcll(peers & lt_mask);
            }
            __builtin_amdgcn_wave_barrier();
            if (act && (peers >> lane) == 1ull) {  // highest lane of the group publishes the new count
                my_hist[e[u]] = prior + __popcll(peers);
            }
            __builtin_amdgcn_wave_barrier();
            if (i < end) {
                pos[i] = r;
            }
        }
    }
    __syncthreads();

    // Per expert: exclusive scan across the waves' histograms, total count.
    int cnt = 0;
    if (tid < E) {
        int run = 0;
#pragma unroll
        for (int ww = 0; ww < kPlanWaves; ++ww) {
            int t = hist[ww * kMaxExperts + tid];
            hist[ww * kMaxExperts + tid] = run;
            run += t;
        }
        cnt = run;
    }
    int off = block_exclusive_scan(tid < E ? cnt : 0, tid, scan_s, &total_s);
    if (tid < E) {
        off_s[tid] = off;
    }
    __syncthreads();
    const int total = total_s;

    // Pass 2: global ranks and destination rows.
    for (int i = beg + lane; i < end; i += kWave) {
        int e = load_id(idx, i, E);
        int r = pos[i];
        int row = -1;
        if (e >= 0) {
            r += my_hist[e];
            row = off_s[e] + r;
            pos[i] = r;
        }
        if (a.dst_row != nullptr) {
            a.dst_row[i] = row;
        }
    }
    for (int i = n + tid; i < n_all; i += kPlanThreads) {  // masked-out tokens
        pos[i] = -1;
        if (a.dst_row != nullptr) {
            a.dst_row[i] = -1;
        }
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
    if (a.per_rank_zero != nullptr && tid < a.R) {
        a.per_rank_zero[tid] = 0;
    }

    // GEMM tile table: expert e owns ceil(cnt/kGemmTileM) tiles, in expert order.
    if (a.tiles != nullptr) {
        int nt = tid < E ? (cnt + kGemmTileM - 1) / kGemmTileM : 0;
        int tbase = block_exclusive_scan(nt, tid, scan_s, &total_s);
        if (tid < E) {
            for (int j = 0; j < nt; ++j) {
                int32_t *t = a.tiles + 4 + 4 * (tbase + j);
                t[0] = tid;
                t[1] = off + j * kGemmTileM;
                t[2] = min(kGemmTileM, cnt - j * kGemmTileM);
                t[3] = 0;
            }
        }
        if (tid == 0) {
            a.tiles[0] = total_s;
            a.tiles[1] = total;
            a.tiles[2] = t_active;
            a.tiles[3] = 0;
        }
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

__global__ __launch_bounds__(kPlanThreads) void notify_scan_kernel(const int32_t *cnt, int E, int num_tokens,
                                                                  int32_t *off, int32_t *send_data,
                                                                  int32_t *recv_data)
{
    __shared__ int scan_s[kPlanWaves];
    __shared__ int total_s;
    const int tid = threadIdx.x;
    int c = tid < E ? cnt[tid] : 0;
    int o = block_exclusive_scan(c, tid, scan_s, &total_s);
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

__global__ __launch_bounds__(kPlanThreads) void build_tiles_kernel(const int64_t *group_list, int cumulative,
                                                                  int G, long long max_rows, int max_tiles,
                                                                  int32_t *tiles)
{
    __shared__ int scan_s[kPlanWaves];
    __shared__ int total_s;
    const int tid = threadIdx.x;
    long long m0 = 0, m1 = 0;
    if (tid < G) {
        if (cumulative) {
            m0 = tid == 0 ? 0 : group_list[tid - 1];
            m1 = group_list[tid];
        } else {
            m1 = group_list[tid];  // converted to a cumulative value below
        }
    }
    if (!cumulative) {
        int c = tid < G ? (int)min(max(m1, 0ll), max_rows) : 0;
        int o = block_exclusive_scan(c, tid, scan_s, &total_s);
        m0 = o;
        m1 = (long long)o + c;
    }
    // Clamp to the rows that exist so that a corrupt group list cannot index past the tensors.
    m0 = min(max(m0, 0ll), max_rows);
    m1 = min(max(m1, m0), max_rows);
    int cnt = tid < G ? (int)(m1 - m0) : 0;
    int nt = (cnt + kGemmTileM - 1) / kGemmTileM;
    int tbase = block_exclusive_scan(nt, tid, scan_s, &total_s);
    int num_tiles = min(total_s, max_tiles);
    if (tid < G) {
        for (int j = 0; j < nt && tbase + j < max_tiles; ++j) {  // a corrupt list cannot overrun the table
            int32_t *t = tiles + 4 + 4 * (tbase + j);
            t[0] = tid;
            t[1] = (int)m0 + j * kGemmTileM;
            t[2] = min(kGemmTileM, cnt - j * kGemmTileM);
            t[3] = 0;
        }
    }
    __syncthreads();
    int rows_total = block_exclusive_scan(cnt, tid, scan_s, &total_s);
    (void)rows_total;
    if (tid == 0) {
        tiles[0] = num_tiles;
        tiles[1] = total_s;
        tiles[2] = 0;
        tiles[3] = 0;
    }
}

__global__ void cast_i64_to_i32_kernel(const int64_t *src, int32_t *dst, long long n)
{
    long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        long long v = src[i];
        dst[i] = v < -2147483647ll ? -1 : (v > 2147483647ll ? 2147483647 : (int32_t)v);
    }
}

}  // namespace

hipError_t launch_plan(const PlanArgs &a, hipStream_t stream)
{
    if (a.idx_is64) {
        hipLaunchKernelGGL(plan_kernel<int64_t>, dim3(1), dim3(kPlanThreads), 0, stream, a);
    } else {
        hipLaunchKernelGGL(plan_kernel<int32_t>, dim3(1), dim3(kPlanThreads), 0, stream, a);
    }
    return hipGetLastError();
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
    hipLaunchKernelGGL(notify_scan_kernel, dim3(1), dim3(kPlanThreads), 0, stream, cnt, E, num_tokens, off,
                       send_data, recv_data);
    return hipGetLastError();
}

hipError_t launch_build_tiles(const int64_t *group_list, int cumulative, int G, int64_t max_rows, int max_tiles,
                              int32_t *tiles, hipStream_t stream)
{
    hipLaunchKernelGGL(build_tiles_kernel, dim3(1), dim3(kPlanThreads), 0, stream, group_list, cumulative, G,
                       (long long)max_rows, max_tiles, tiles);
    return hipGetLastError();
}

hipError_t launch_cast_i64_to_i32(const int64_t *src, int32_t *dst, int64_t n, hipStream_t stream)
{
    if (n <= 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(cast_i64_to_i32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, src, dst,
                       (long long)n);
    return hipGetLastError();
}

}  // namespace cam
