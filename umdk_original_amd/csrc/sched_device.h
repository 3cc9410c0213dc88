// Device code that builds the work-item schedule of the grouped GEMM: used by the stand-alone builder kernel and
// by the permute kernel of the dispatch, whose spare workgroups build the schedules of the GEMMs that follow while
// the others move rows.
#ifndef CAM_SCHED_DEVICE_H_
#define CAM_SCHED_DEVICE_H_

#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

// A schedule is built by `parts` workgroups: every one derives the per-expert tables and then writes every
// parts-th batch of 256 items; the item arithmetic (divisions, a binary search) is what takes the time, so it is
// what is spread over workgroups.
// Expert g with r rows: r == 0 owns nothing; r <= 128 is "flat": one tile and ceil(N/512) column blocks;
// otherwise "tall": ceil(r/256) tiles of (nearly) equal height, a multiple of 32, and ceil(N/256) column
// blocks.  Experts are ranked by rows, largest first.
//   * Tall experts: the (expert, column block) groups, in rank order, are cut into eight consecutive runs of
//     equal work (rows x column blocks), one per queue.  A queue therefore holds few experts, each with
//     neighbouring column blocks: the CUs of an XCD that work side by side share the weight panels (row tiles
//     of one group) and the activation tiles (column blocks of one expert) through their L2, and an expert's
//     activations are fetched by as few XCDs as its size requires.
//   * Flat experts are dealt to the queues whole, in rank order, so that the column blocks of one expert,
//     which all read the same few activation rows, run on one XCD.
// A queue lists its tall items big experts first, with its flat items spread evenly among them except for the
// last kTallTail places.  A flat item streams its weights at the pace one CU can pull them from memory and takes
// longer than a tall one although it computes less: spread out, flat items run beside tall ones, which need
// the matrix cores rather than the memory, and the queues end with items of even length.
// The work is laid out so that it needs few workgroup barriers: every prefix sum over the experts is the job
// of one wave, which walks the ranks 64 at a time.
constexpr int kTallTail = 24;  // tall items a queue ends with (three quarters of a round of its 32 workgroups)

struct ExpertShape {
    int rows, tiles, blocks, units;
    bool tall, flat;
};

__device__ __forceinline__ ExpertShape expert_shape(int rows, int nb_tall, int nb_flat)
{
    ExpertShape e;
    e.rows = rows;
    e.tall = rows > 128;
    e.flat = rows > 0 && !e.tall;
    e.tiles = e.tall ? (rows + 255) / 256 : (e.flat ? 1 : 0);
    e.blocks = e.tall ? nb_tall : (e.flat ? nb_flat : 0);
    e.units = (rows + 31) / 32;
    return e;
}

// Queue of the tall group whose work (in units) starts at `before` and is `units` long: the queue its middle
// falls into when the total work is cut into eight equal runs.
__device__ __forceinline__ int queue_of_group(long long before, int units, long long wtotal)
{
    const long long mid16 = (2 * before + units) * kNumXcd;  // 2 * middle * 8
    int x = 0;
#pragma unroll
    for (int k = 1; k < kNumXcd; ++k) {
        x += mid16 >= 2 * wtotal * k ? 1 : 0;
    }
    return x;
}

// LDS of one building workgroup.
struct SchedShared {
    int rows[kMaxExperts], off[kMaxExperts], order[kMaxExperts];
    int first_item[kMaxExperts + 1];      // by rank: items of the experts ranked before
    int work_before[kMaxExperts];         // by rank: work of the tall experts ranked before
    int flat_rank[kMaxExperts];           // by rank: flat experts ranked before
    short ngroups[kNumXcd][kMaxExperts];  // by rank: the expert's groups in queue x (tall)
    int qbase[kNumXcd][kMaxExperts];      // by rank: items of earlier experts of its kind in queue x
    int qtall[kNumXcd], qflat[kNumXcd];
    int wtotal, total_rows;
};

// Part `part` of `parts` of schedule sb.spec[which]; called by all NT threads of a workgroup (NT a multiple of 256).
template <int NT>
__device__ __forceinline__ void build_sched_part(SchedShared &sh, const SchedBuild &sb, int which, int part, int parts)
{
    const int G = sb.G;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;

    // the group list, clamped to the rows that exist so that a corrupt list cannot index past the tensors
    // (sh.order is free until the ranking below)
    for (int g = tid; g < G; g += NT) {
        sh.order[g] = (int)min(max(sb.group_list[g], (int64_t)0), (int64_t)sb.max_rows);
    }
    __syncthreads();
    // rows and first row of every expert (wave 0)
    if (wave == 0) {
        int run = 0;  // rows before this chunk (counts)
        for (int base = 0; base < G; base += kWave) {
            const int g = base + lane;
            int m0 = 0, m1 = 0;
            if (sb.cumulative) {
                if (g < G) {
                    m0 = g == 0 ? 0 : sh.order[g - 1];
                    m1 = max(sh.order[g], m0);
                }
            } else {
                const int c = g < G ? sh.order[g] : 0;
                const int inc = wave_inclusive_scan(c, lane);
                m0 = (int)min(max((long long)run + inc - c, 0ll), sb.max_rows);
                m1 = (int)min(max((long long)m0 + c, (long long)m0), sb.max_rows);
                run = (int)min(max((long long)run + __shfl(inc, kWave - 1, kWave), 0ll), sb.max_rows);
            }
            if (g < G) {
                sh.rows[g] = m1 - m0;
                sh.off[g] = m0;
            }
            const int chunk_rows = wave_sum(g < G ? m1 - m0 : 0);
            if (lane == 0) {
                sh.total_rows = (base == 0 ? 0 : sh.total_rows) + chunk_rows;
            }
        }
    }
    __syncthreads();
    // rank by rows, largest first (ties: lower index first)
    for (int g = tid; g < G; g += NT) {
        const int cnt = sh.rows[g];
        int rank = 0;
        for (int j = 0; j < G; ++j) {
            const int rj = sh.rows[j];
            rank += (rj > cnt || (rj == cnt && j < g)) ? 1 : 0;
        }
        sh.order[rank] = g;
    }
    __syncthreads();
    const int total_rows = sh.total_rows;

    {
        const SchedSpec spec = sb.spec[which];
        int32_t *sched = spec.sched;
        SchedItem *items = (SchedItem *)(sched + kSchedHeader);
        const int nb_tall = (spec.N + 255) / 256;
        const int nb_flat = (spec.N + 511) / 512;

        // by rank: items, tall work and flat experts before (wave 0)
        if (wave == 0) {
            int items_run = 0, work_run = 0, flat_run = 0;
            for (int base = 0; base < G; base += kWave) {
                const int rank = base + lane;
                const ExpertShape e = expert_shape(rank < G ? sh.rows[sh.order[rank]] : 0, nb_tall, nb_flat);
                const int vi = e.blocks * e.tiles, vw = e.tall ? e.blocks * e.units : 0, vf = e.flat ? 1 : 0;
                const int ii = wave_inclusive_scan(vi, lane);
                const int iw = wave_inclusive_scan(vw, lane);
                const int jf = wave_inclusive_scan(vf, lane);
                if (rank < G) {
                    sh.first_item[rank] = items_run + ii - vi;
                    sh.work_before[rank] = work_run + iw - vw;
                    sh.flat_rank[rank] = flat_run + jf - vf;
                }
                items_run += __shfl(ii, kWave - 1, kWave);
                work_run += __shfl(iw, kWave - 1, kWave);
                flat_run += __shfl(jf, kWave - 1, kWave);
            }
            if (lane == 0) {
                sh.first_item[G] = items_run;
                sh.wtotal = max(work_run, 1);
            }
        }
        __syncthreads();
        const int n_items = sh.first_item[G];
        const long long wtotal = sh.wtotal;

        // by rank and queue: items of earlier experts.  Role x (0..7) counts the tall items of queue x, role 8 + x
        // its flat items; the waves share the sixteen roles.
        for (int role = wave; role < 2 * kNumXcd; role += NT / kWave) {
            const int x = role & (kNumXcd - 1);
            const bool flat_wave = role >= kNumXcd;
            int run = 0;
            for (int base = 0; base < G; base += kWave) {
                const int rank = base + lane;
                const ExpertShape e = expert_shape(rank < G ? sh.rows[sh.order[rank]] : 0, nb_tall, nb_flat);
                int v = 0;
                if (flat_wave) {
                    v = (e.flat && sh.flat_rank[rank] % kNumXcd == x) ? e.blocks : 0;
                } else if (e.tall) {
                    int mine = 0;
                    const long long before = sh.work_before[rank];
                    for (int c = 0; c < e.blocks; ++c) {
                        mine += queue_of_group(before + (long long)c * e.units, e.units, wtotal) == x ? 1 : 0;
                    }
                    sh.ngroups[x][rank] = (short)mine;
                    v = mine * e.tiles;
                }
                const int inc = wave_inclusive_scan(v, lane);
                if (rank < G && (flat_wave ? e.flat : e.tall)) {
                    sh.qbase[x][rank] = run + inc - v;
                }
                run += __shfl(inc, kWave - 1, kWave);
            }
            if (lane == 0) {
                (flat_wave ? sh.qflat : sh.qtall)[x] = run;
            }
        }
        __syncthreads();
        if (tid == 0 && part == 0) {
            int run = 0;
            for (int x = 0; x < kNumXcd; ++x) {
                sched[kSchedQueueStart + x] = run;
                sched[kSchedQueueCount + x * kSchedQueueStride] = 0;
                run += sh.qflat[x] + sh.qtall[x];
            }
            sched[kSchedQueueStart + kNumXcd] = run;
            sched[0] = min(n_items, spec.max_items);
            sched[1] = total_rows;
            sched[2] = 0;
            sched[3] = 0;
        }
        // one thread per item, in rank-major order; the workgroups of a schedule share the items
        // (256 items per workgroup and pass: four waves, one per SIMD, so that the arithmetic is not queued four deep)
        for (int i = part * 256 + tid; tid < 256 && i < n_items; i += parts * 256) {
            int lo = 0, hi = G;  // largest rank with first_item <= i
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (sh.first_item[mid] <= i) {
                    lo = mid;
                } else {
                    hi = mid;
                }
            }
            const int rank = lo;
            const int eg = sh.order[rank];
            const ExpertShape e = expert_shape(sh.rows[eg], nb_tall, nb_flat);
            const int local = i - sh.first_item[rank];
            const int c = local / e.tiles;
            const int j = local - c * e.tiles;
            int x, qpos;
            if (e.flat) {
                x = sh.flat_rank[rank] % kNumXcd;
                qpos = sh.qbase[x][rank] + c;
            } else {
                x = queue_of_group(sh.work_before[rank] + (long long)c * e.units, e.units, wtotal);
                int cfirst = 0;  // the expert's groups in earlier queues
                for (int xx = 0; xx < x; ++xx) {
                    cfirst += sh.ngroups[xx][rank];
                }
                qpos = sh.qbase[x][rank] + (c - cfirst) * e.tiles + j;
            }
            {
                // Queue order: the flat items spread evenly among the tall ones (flat item j has key (2j+1)/(2F),
                // tall item i key (2i+1)/(2T), smaller keys first, a tall item first on a tie), except that the
                // last kTallTail tall items follow the last flat one.
                const long long F = sh.qflat[x];
                const long long T = max(sh.qtall[x] - kTallTail, 0);
                if (e.flat) {
                    const long long num = (2ll * qpos + 1) * T - F;
                    qpos += (int)(num < 0 ? 0 : min(T, num / (2 * F) + 1));
                } else if (qpos < T) {
                    const long long num = (2ll * qpos + 1) * F - T;
                    qpos += (int)(num <= 0 ? 0 : min(F, (num + 2 * T - 1) / (2 * T)));
                } else {
                    qpos += (int)F;
                }
            }
            int pos = qpos;
            for (int xx = 0; xx < x; ++xx) {
                pos += sh.qflat[xx] + sh.qtall[xx];
            }
            if (pos >= spec.max_items) {
                continue;  // cannot happen with a table sized by sched_bytes(); guards a corrupt list
            }
            // tile j of e.tiles: heights are multiples of 32 that differ by at most 32
            const int base_u = e.units / e.tiles, extra = e.units % e.tiles;
            const int u0 = j * base_u + min(j, extra);
            const int uj = base_u + (j < extra ? 1 : 0);
            SchedItem it;
            it.g = eg;
            it.m0 = sh.off[eg] + u0 * 32;
            it.rows = min(uj * 32, e.rows - u0 * 32);
            it.split = e.flat ? 0 : 32 * ((it.rows + 63) / 64);
            it.nb = c;
            it.flat = e.flat ? 1 : 0;
            it.pad0 = 0;
            it.pad1 = 0;
            items[pos] = it;
        }
    }
}


}  // namespace cam

#endif  // CAM_SCHED_DEVICE_H_
