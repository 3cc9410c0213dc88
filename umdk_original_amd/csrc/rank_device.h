// Device code shared by the routing-plan kernels: id loading, workgroup
// scans and the stable ranking of one chunk of the flat (token, k) id sequence.
#ifndef CAM_RANK_DEVICE_H_
#define CAM_RANK_DEVICE_H_

#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

constexpr int kLocalThreads = 256;  // ranking workgroup: 4 waves
constexpr int kLocalWaves = kLocalThreads / kWave;

// Ids outside [0, E) name no expert: negative ones are the reference's "dropped" marker
// (src/cam/comm_operator/pybind/moe_dispatch_prefill.cpp:106), ids >= E would index past every
// per-expert table and are treated the same way.
template <typename IdT>
__device__ __forceinline__ int load_id(const IdT *p, long long i, int E)
{
    long long v = (long long)p[i];
    return (v < 0 || v >= (long long)E) ? -1 : (int)v;
}

// Exclusive scan of one value per thread across a workgroup of NWAVES waves; returns the exclusive
// prefix and leaves the grand total in *total_out (LDS).  Uses `scratch` (>= NWAVES ints of LDS).
template <int NWAVES>
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
        int t = lane < NWAVES ? scratch[lane] : 0;
        int ti = wave_inclusive_scan(t, lane);
        if (lane < NWAVES) {
            scratch[lane] = ti - t;
        }
        if (lane == NWAVES - 1) {
            *total_out = ti;
        }
    }
    __syncthreads();
    int r = inc - v + scratch[w];
    __syncthreads();
    return r;
}

// Number of set mask entries (the active prefix of the batch); T when there is no mask.
__device__ __forceinline__ int count_active(const uint8_t *mask, int T, int tid, int nthreads, int *slot)
{
    if (mask == nullptr) {
        return T;
    }
    int c = 0;
    for (int t = tid; t < T; t += nthreads) {
        c += mask[t] != 0 ? 1 : 0;
    }
    c = wave_sum(c);
    if (tid == 0) {
        *slot = 0;
    }
    __syncthreads();
    if ((tid & (kWave - 1)) == 0 && c != 0) {
        atomicAdd(slot, c);
    }
    __syncthreads();
    return *slot;
}

// Ranks the chunk of flat entries [b*IT*256, (b+1)*IT*256) of one workgroup of 256 threads.
// Wave w owns the IT*64 entries from b*chunk + w*IT*64 and each lane keeps its IT ids in registers.
// 64 ids at a time, lanes holding the same id find each other with one ballot per id bit; the rank
// inside the wave is the wave's running count of that id (LDS) plus the number of lower lanes in the
// group, and the group's highest lane publishes the new count.  A scan over the 4 waves' histograms
// turns wave-local ranks into chunk-local ones.  Writes the chunk-local rank of every entry below
// n_all to pos_out (-1 for skipped entries and entries at or beyond n) and the chunk's per-expert
// histogram to hist_row[0..E).  `hist` is LDS, kLocalWaves * kMaxExperts ints.
template <typename IdT, int IT>
__device__ __forceinline__ void rank_chunk(const IdT *__restrict__ idx, int b, long long n, long long n_all, int E,
                                           int *hist, int32_t *pos_out, int32_t *hist_row)
{
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = tid >> 6;
    // the ids are requested first: their trip to memory runs while the histograms are cleared
    const long long base = (long long)b * (IT * kLocalThreads) + (long long)w * (IT * kWave);
    int e[IT], r[IT];
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const long long i = base + it * kWave + lane;
        e[it] = i < n ? load_id(idx, i, E) : -1;
    }
    for (int i = tid; i < kLocalWaves * kMaxExperts; i += kLocalThreads) {
        hist[i] = 0;
    }
    __syncthreads();
    int nbits = 0;
    while ((1 << nbits) < E) {
        ++nbits;
    }
    int *my_hist = hist + w * kMaxExperts;
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const bool act = e[it] >= 0;
        unsigned long long peers = __ballot(act);
        for (int bit_i = 0; bit_i < nbits; ++bit_i) {
            const bool bit = act && ((e[it] >> bit_i) & 1);
            const unsigned long long bal = __ballot(bit);
            peers &= bit ? bal : ~bal;
        }
        int prior = 0;
        r[it] = -1;
        if (act) {
            prior = my_hist[e[it]];
            r[it] = prior + __popcll(peers & lt_mask);
        }
        __builtin_amdgcn_wave_barrier();
        if (act && (peers >> lane) == 1ull) {
            my_hist[e[it]] = prior + __popcll(peers);
        }
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    for (int ee = tid; ee < E; ee += kLocalThreads) {
        int run = 0;
#pragma unroll
        for (int ww = 0; ww < kLocalWaves; ++ww) {
            const int t = hist[ww * kMaxExperts + ee];
            hist[ww * kMaxExperts + ee] = run;
            run += t;
        }
        hist_row[ee] = run;
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const long long i = base + it * kWave + lane;
        if (i < n_all) {
            const int v = e[it] >= 0 ? r[it] + my_hist[e[it]] : -1;
            pos_out[i] = v;
        }
    }
}

}  // namespace cam

#endif  // CAM_RANK_DEVICE_H_
