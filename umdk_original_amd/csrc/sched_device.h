// Device code that builds the work-item schedule of the grouped GEMM: used by the stand-alone builder kernel and
// by the permute kernel of the dispatch, one of whose spare workgroups builds each schedule of the GEMMs that
// follow while the others move rows.
#ifndef CAM_SCHED_DEVICE_H_
#define CAM_SCHED_DEVICE_H_

#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

// Work items.  Expert g with r rows: r == 0 owns nothing; r <= 128 is "flat": one row tile and ceil(N/512) column
// blocks, each an item that streams its weight panel at the pace one CU pulls bytes from memory; otherwise "tall":
// ceil(r/256) row tiles of (nearly) equal height, a multiple of 32 rows (tiles of one expert differ by at most 32),
// times ceil(N/256) column blocks.  Shorter tall tiles are no cheaper per row: below 256 rows the K loop is bound
// by the loads of its 256-column weight panel, not by the matrix cores.
//
// The schedule gives every workgroup of the persistent GEMM (one per CU) a queue of its own.  The items are put in
// one line, costliest first by the model below and otherwise in the order in which they share operands (experts
// largest first; per expert column block by column block; the row tiles of a column block side by side), and the
// line is dealt row by row into a matrix with one column per workgroup:
//   * with n items and m workgroups, R = n / m: the first m - b columns take R items each from the costly end of
//     the line, the last b = n - R m columns take R + 1 from the cheap end, so that no column holds one item more
//     than another of the same kind and the columns with more items hold the cheaper ones;
//   * a row runs over its columns in alternating direction, so the costliest item of one row meets the cheapest of
//     the next;
//   * 32 neighbouring columns are the workgroups of one XCD (workgroup w runs on XCD w % 8), so the items an XCD
//     works on at one time are neighbours in the line: the row tiles of one (expert, column block) share the
//     weight panel through that XCD's L2, the column blocks of one expert its activation rows.  Measured on the
//     Zipf-skewed shape this matters more than balance: the same items dealt for balance alone run a third slower.
// A queue is run front to back by its workgroup; one that runs out takes the next item of the queue with the most
// items left (gemm.hip), which covers what the cost model gets wrong.
//
// Long schedules (kSharedFrom items per workgroup or more) get eight shared queues instead, one per XCD, from which
// the workgroups of that XCD take item by item: with many short items per workgroup the sums of fixed queues
// drift apart by more than an item, and what counts is that an XCD works through neighbouring items one after the
// other as well as side by side.
//   * Tall experts: the (expert, column block) groups, largest expert first, are cut into eight consecutive runs
//     of equal work (rows x column blocks), one per queue.  A queue therefore holds few experts, each with
//     neighbouring column blocks: the CUs of an XCD share the weight panels (row tiles of one group) and the
//     activation tiles (column blocks of one expert) through their L2, now and a moment later.
//   * Flat experts are dealt to the queues whole, in rank order, and a queue spreads its flat items evenly among
//     its tall ones except for the last kTallTail places: a flat item streams its weights and needs the memory,
//     a tall one the matrix cores, so they run well side by side, and the queues end with items of even length.
//
// Cost model, nanoseconds; it only ranks the item kinds.  A tall tile of u row units (32 rows) over KT sub-steps
// of 64 K bytes: fixed + KT * max(load-bound step, u * matrix step); a flat item: fixed + KT * streaming step.
constexpr float kTallFixedSwiglu = 15000.0f;
constexpr float kTallFixedPlain = 10000.0f;
constexpr float kTallLoadStep = 550.0f;
constexpr float kTallUnitStep = 92.0f;
constexpr float kFlatFixed = 22400.0f;
constexpr float kFlatStep = 862.0f;
constexpr int kClasses = 9;  // item kinds: 0 = flat, h = 1..8 = tall tile of h row units
constexpr int kSharedFrom = 12;                       // items per workgroup from which the queues are shared
constexpr int kTallTail = 24;                        // tall items a shared queue ends with

struct ExpertShape {
    int rows, units, tiles, base, extra;  // tall: `extra` tiles of base + 1 units, then tiles - extra of base units
    bool tall, flat;
};

__device__ __forceinline__ ExpertShape expert_shape(int rows)
{
    ExpertShape e;
    e.rows = rows;
    e.tall = rows > 128;
    e.flat = rows > 0 && !e.tall;
    e.units = (rows + 31) / 32;
    e.tiles = e.tall ? (rows + 255) / 256 : (e.flat ? 1 : 0);
    e.base = e.tall ? e.units / e.tiles : 0;
    e.extra = e.tall ? e.units % e.tiles : 0;
    return e;
}

// Items of class c one column block of the expert holds.
__device__ __forceinline__ int class_count(const ExpertShape &e, int c)
{
    if (e.flat) {
        return c == 0 ? 1 : 0;
    }
    if (!e.tall) {
        return 0;
    }
    return (c == e.base + 1 ? e.extra : 0) + (c == e.base ? e.tiles - e.extra : 0);
}

// LDS of the building workgroup.  The two forms of schedule need different tables; they share the space.
struct SchedOwnTables {
    int class_before[kClasses][kMaxExperts];  // by class and rank: items of that class the experts ranked before hold
    int class_total[kClasses];
    int class_start[kClasses];                // where the class starts in the line
};
struct SchedSharedTables {
    int work_before[kMaxExperts];         // by rank: work of the tall experts ranked before
    int flat_rank[kMaxExperts];           // by rank: flat experts ranked before
    short ngroups[kNumXcd][kMaxExperts];  // by rank: the expert's groups in queue x (tall)
    int qbase[kNumXcd][kMaxExperts];      // by rank: items of earlier experts of its kind in queue x
    int qtall[kNumXcd], qflat[kNumXcd];
    int wtotal;
};
struct SchedShared {
    int rows[kMaxExperts], off[kMaxExperts], order[kMaxExperts];
    int first_item[kMaxExperts + 1];       // by rank: items of the experts ranked before
    union {
        SchedOwnTables own;
        SchedSharedTables shr;
    };
    int qstart[kMaxQueues + 1];
    int total_rows;
};

// Shared queues: the queue of the tall group whose work (in row units) starts at `before` and is `units` long is
// the one its middle falls into when the total work is cut into eight equal runs.
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

// Workgroup of column j when the columns are numbered XCD by XCD, and the inverse.
__device__ __forceinline__ int workgroup_of_column(int j, int m)
{
    int x = 0;
    for (; x < kNumXcd - 1; ++x) {
        const int here = (m - x + kNumXcd - 1) / kNumXcd;  // workgroups of XCD x
        if (j < here) {
            break;
        }
        j -= here;
    }
    return x + kNumXcd * j;
}

__device__ __forceinline__ int column_of_workgroup(int w, int m)
{
    const int x = w % kNumXcd;
    int before = 0;
    for (int xx = 0; xx < x; ++xx) {
        before += (m - xx + kNumXcd - 1) / kNumXcd;
    }
    return before + w / kNumXcd;
}

// One item of a schedule from its expert's shape: column block c, row tile j.
__device__ __forceinline__ SchedItem make_item(const ExpertShape &e, int expert, int first_row, int c, int j)
{
    // row tile j: heights are multiples of 32 rows that differ by at most 32
    const int u0 = j * e.base + min(j, e.extra);
    const int uj = e.base + (j < e.extra ? 1 : 0);
    SchedItem it;
    it.g = expert;
    it.m0 = first_row + u0 * 32;
    it.rows = e.flat ? e.rows : min(uj * 32, e.rows - u0 * 32);
    it.split = e.flat ? 0 : 32 * ((it.rows + 63) / 64);
    it.nb = c;
    it.flat = e.flat ? 1 : 0;
    it.pad0 = 0;
    it.pad1 = 0;
    return it;
}

// The shared-queue form of a schedule (long schedules); sh.rows / off / order / first_item are complete.
template <int NT>
__device__ __forceinline__ void build_shared_queues(SchedShared &sh, const SchedSpec &spec, int G, int n_items,
                                                    int part, int parts)
{
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    int32_t *sched = spec.sched;
    SchedItem *items = (SchedItem *)(sched + kSchedHeader);
    const int nb_tall = (spec.N + 255) / 256;
    const int nb_flat = (spec.N + 511) / 512;
    SchedSharedTables &t = sh.shr;

    // by rank: tall work and flat experts before (wave 0)
    if (wave == 0) {
        int work_run = 0, flat_run = 0;
        for (int base = 0; base < G; base += kWave) {
            const int rank = base + lane;
            const ExpertShape e = expert_shape(rank < G ? sh.rows[sh.order[rank]] : 0);
            const int vw = e.tall ? nb_tall * e.units : 0, vf = e.flat ? 1 : 0;
            const int iw = wave_inclusive_scan(vw, lane);
            const int jf = wave_inclusive_scan(vf, lane);
            if (rank < G) {
                t.work_before[rank] = work_run + iw - vw;
                t.flat_rank[rank] = flat_run + jf - vf;
            }
            work_run += __shfl(iw, kWave - 1, kWave);
            flat_run += __shfl(jf, kWave - 1, kWave);
        }
        if (lane == 0) {
            t.wtotal = max(work_run, 1);
        }
    }
    __syncthreads();
    const long long wtotal = t.wtotal;

    // by rank and queue: items of earlier experts.  Role x (0..7) counts the tall items of queue x, role 8 + x its
    // flat items; the waves share the sixteen roles.
    for (int role = wave; role < 2 * kNumXcd; role += NT / kWave) {
        const int x = role & (kNumXcd - 1);
        const bool flat_wave = role >= kNumXcd;
        int run = 0;
        for (int base = 0; base < G; base += kWave) {
            const int rank = base + lane;
            const ExpertShape e = expert_shape(rank < G ? sh.rows[sh.order[rank]] : 0);
            int v = 0;
            if (flat_wave) {
                v = (e.flat && t.flat_rank[rank] % kNumXcd == x) ? nb_flat : 0;
            } else if (e.tall) {
                int mine = 0;
                const long long before = t.work_before[rank];
                for (int c = 0; c < nb_tall; ++c) {
                    mine += queue_of_group(before + (long long)c * e.units, e.units, wtotal) == x ? 1 : 0;
                }
                t.ngroups[x][rank] = (short)mine;
                v = mine * e.tiles;
            }
            const int inc = wave_inclusive_scan(v, lane);
            if (rank < G && (flat_wave ? e.flat : e.tall)) {
                t.qbase[x][rank] = run + inc - v;
            }
            run += __shfl(inc, kWave - 1, kWave);
        }
        if (lane == 0) {
            (flat_wave ? t.qflat : t.qtall)[x] = run;
        }
    }
    __syncthreads();
    if (tid == 0 && part == 0) {
        int run = 0;
        for (int x = 0; x < kNumXcd; ++x) {
            sched[kSchedQueueStart + x] = min(run, spec.max_items);
            sched[kSchedQueueCount + x * kSchedQueueStride] = 0;  // every item of a shared queue is asked for
            run += t.qflat[x] + t.qtall[x];
        }
        sched[kSchedQueueStart + kNumXcd] = min(run, spec.max_items);
        sched[0] = min(n_items, spec.max_items);
        sched[1] = sh.total_rows;
        sched[2] = kNumXcd;
        sched[3] = 2;  // bit 1: shared queues
    }
    // one thread per item; the parts take turns of NT items
    for (int i = part * NT + tid; i < n_items; i += parts * NT) {
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
        const ExpertShape e = expert_shape(sh.rows[eg]);
        const int local = i - sh.first_item[rank];
        const int c = local / e.tiles;
        const int j = local - c * e.tiles;
        int x, qpos;
        if (e.flat) {
            x = t.flat_rank[rank] % kNumXcd;
            qpos = t.qbase[x][rank] + c;
        } else {
            x = queue_of_group(t.work_before[rank] + (long long)c * e.units, e.units, wtotal);
            int cfirst = 0;  // the expert's groups in earlier queues
            for (int xx = 0; xx < x; ++xx) {
                cfirst += t.ngroups[xx][rank];
            }
            qpos = t.qbase[x][rank] + (c - cfirst) * e.tiles + j;
        }
        {
            // Queue order: the flat items spread evenly among the tall ones (flat item j has key (2j+1)/(2F), tall
            // item i key (2i+1)/(2T), smaller keys first, a tall item first on a tie), except that the last
            // kTallTail tall items follow the last flat one.
            const long long F = t.qflat[x];
            const long long T = max(t.qtall[x] - kTallTail, 0);
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
            pos += t.qflat[xx] + t.qtall[xx];
        }
        if (pos >= spec.max_items) {
            continue;  // cannot happen with a table sized by sched_bytes(); guards a corrupt list
        }
        items[pos] = make_item(e, eg, sh.off[eg], c, j);
    }
}

// Schedule sb.spec[which]; called by all NT threads of a workgroup (NT a multiple of 64, at least 256).  `parts`
// workgroups share a schedule: each works out the same tables in its own LDS, part 0 writes the header and the queue
// tables, and the items go round the parts in turns of NT (placing an item costs about a microsecond of dependent
// lookups and divisions, and a long schedule has several thousand).
template <int NT>
__device__ __forceinline__ void build_sched_part(SchedShared &sh, const SchedBuild &sb, int which, int part, int parts)
{
    const int G = sb.G;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;
    const int m = min(max(sb.queues, 1), kMaxQueues);

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

    const SchedSpec spec = sb.spec[which];
    int32_t *sched = spec.sched;
    SchedItem *items = (SchedItem *)(sched + kSchedHeader);
    const int nb_tall = (spec.N + 255) / 256;
    const int nb_flat = (spec.N + 511) / 512;

    // by rank: items before, in all and per class.  One wave per prefix sum (class c, or the total for c == kClasses).
    for (int c = wave; c <= kClasses; c += NT / kWave) {
        int run = 0;
        for (int base = 0; base < G; base += kWave) {
            const int rank = base + lane;
            const ExpertShape e = expert_shape(rank < G ? sh.rows[sh.order[rank]] : 0);
            const int blocks = e.tall ? nb_tall : (e.flat ? nb_flat : 0);
            const int v = (c == kClasses ? e.tiles : class_count(e, c)) * blocks;
            const int inc = wave_inclusive_scan(v, lane);
            if (rank < G) {
                if (c == kClasses) {
                    sh.first_item[rank] = run + inc - v;
                } else {
                    sh.own.class_before[c][rank] = run + inc - v;
                }
            }
            run += __shfl(inc, kWave - 1, kWave);
        }
        if (lane == 0) {
            if (c == kClasses) {
                sh.first_item[G] = run;
            } else {
                sh.own.class_total[c] = run;
            }
        }
    }
    __syncthreads();
    const int n_items = sh.first_item[G];

    // long schedules: eight shared queues
    if (n_items / m >= kSharedFrom && m >= kNumXcd) {
        build_shared_queues<NT>(sh, spec, G, n_items, part, parts);
        return;
    }

    // the classes in the order of the line: costliest first (ties: flat, then the taller tile)
    if (tid < kClasses) {
        const float KT = (float)(spec.Kd / 64);
        auto cost = [&](int c) {
            return c == 0 ? kFlatFixed + KT * kFlatStep
                          : (spec.swiglu ? kTallFixedSwiglu : kTallFixedPlain) +
                                KT * fmaxf(kTallLoadStep, (float)c * kTallUnitStep);
        };
        const float mine = cost(tid);
        int start = 0;
        for (int c = 0; c < kClasses; ++c) {
            const float other = cost(c);
            const bool ahead = other > mine || (other == mine && c != tid && (c == 0 || (tid != 0 && c > tid)));
            start += ahead ? sh.own.class_total[c] : 0;
        }
        sh.own.class_start[tid] = start;
    }
    // the matrix: R items in each of the first m - b columns, R + 1 in the last b
    const int R = n_items / m, b = n_items - R * m;
    const int n_big = (m - b) * R;
    if (wave == 0) {  // first item of every workgroup's queue: prefix sum of the column heights in workgroup order
        constexpr int PER = kMaxQueues / kWave;
        int v[PER], run = 0;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int w = lane * PER + i;
            v[i] = w < m ? R + (column_of_workgroup(w, m) >= m - b ? 1 : 0) : 0;
            run += v[i];
        }
        const int inc = wave_inclusive_scan(run, lane);
        int before = inc - run;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            sh.qstart[lane * PER + i] = before;
            before += v[i];
        }
        if (lane == kWave - 1) {
            sh.qstart[kMaxQueues] = inc;
        }
    }
    __syncthreads();
    if (tid == 0 && part == 0) {
        sched[0] = min(n_items, spec.max_items);
        sched[1] = sh.total_rows;
        sched[2] = m;
        sched[3] = R + (b > 0 ? 1 : 0) <= 1 ? 1 : 0;  // bit 0: no queue holds a second item, nothing can be taken over
    }
    for (int w = tid; w <= m && part == 0; w += NT) {  // m workgroups: the entries beyond are never read
        sched[kSchedQueueStart + w] = min(sh.qstart[w], spec.max_items);
        if (w < m) {
            // the first item of a queue belongs to its workgroup without asking; the counter starts behind it
            sched[kSchedQueueCount + w * kSchedQueueStride] = 1;
        }
    }

    // one thread per item; the parts take turns of NT items
    for (int i = part * NT + tid; i < n_items; i += parts * NT) {
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
        const ExpertShape e = expert_shape(sh.rows[eg]);
        const int local = i - sh.first_item[rank];
        int c, j, cls, pos;  // column block, row tile, class, place among the expert's items of that class
        if (e.flat) {
            c = local;
            j = 0;
            cls = 0;
            pos = local;
        } else {
            c = local / e.tiles;
            j = local - c * e.tiles;
            const bool taller = j < e.extra;
            cls = taller ? e.base + 1 : e.base;
            pos = c * (taller ? e.extra : e.tiles - e.extra) + (taller ? j : j - e.extra);
        }
        const int s = sh.own.class_start[cls] + sh.own.class_before[cls][rank] + pos;  // place in the line
        int col, row;
        {
            const bool small = s >= n_big;
            const int cols = small ? b : m - b, t = small ? s - n_big : s;
            row = t / cols;
            const int k = t - row * cols;
            col = (small ? m - b : 0) + ((row & 1) ? cols - 1 - k : k);
        }
        const int at = sh.qstart[workgroup_of_column(col, m)] + row;
        if (at >= spec.max_items) {
            continue;  // cannot happen with a table sized by sched_bytes(); guards a corrupt list
        }
        items[at] = make_item(e, eg, sh.off[eg], c, j);
    }
}

}  // namespace cam

#endif  // CAM_SCHED_DEVICE_H_
