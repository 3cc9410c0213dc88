// Grouped w8a8 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8), with the CAM epilogues.
//
// Reference semantics (paths relative to the reference tree; FDM =
// src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe):
//   GMM1 main loop  FDM/gemm/kernel/grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:490-645
//   GMM1 epilogue   FDM/epilogue/block/block_epilogue_per_token_dequant_swiglu.h:236-264
//   re-quant        the GMM1 kernel file :160-277
//   GMM2 main loop  FDM/gemm/kernel/grouped_matmul_slice_m_per_token_dequant_multistage_workspace.h:115-215
//   GMM2 epilogue   FDM/epilogue/block/block_epilogue_per_token_dequant.hpp:665-684
//
// Design (not a translation of the cube/vector split above).
//   * Persistent kernel, one workgroup of 8 waves per CU.  Work items (one row tile of ONE expert x one
//     block of packed weight columns) come from a device-built schedule (sched_device.h).  Short schedules
//     give every workgroup a queue of its own, dealt so that the queues last equally long and that the
//     workgroups of an XCD work on tiles which share operands; a workgroup whose queue runs out takes from
//     the fullest one.  Long schedules use one queue per XCD, shared by its workgroups, in which the row
//     tiles of an expert that read the same weight columns sit next to each other and big experts come
//     first, which leaves the small items for the end, where they even out the finishing times.
//   * Two tile shapes.  Tall tiles (129..256 rows) x 256 columns: the two teams of four waves split the
//     rows, every wave owns 64 columns.  Flat tiles (<= 128 rows) x 512 columns: the teams split the
//     columns, so that the weights, which is all such an expert streams from HBM, feed every wave and
//     twice as many weight bytes are in flight per CU.  A wave always owns up to 128 rows x 64 columns
//     (up to 128 int32 accumulators per lane), in 32-row fragments; the fragment count is a template
//     parameter, so the main loop has no control flow.
//   * Both operands travel global -> LDS with direct-to-LDS loads (16 bytes per lane, no registers),
//     four (tall) or three (flat) stages of 64 K-bytes each, up to a whole ring ahead of the MFMAs: the
//     fragments of a stage are read into registers one phase before they are multiplied, which frees the
//     stage for the next load at once.  Weights were laid out once by the prepack kernel in the lane
//     order the MFMA wants; activation rows are placed with an XOR swizzle of their 16-byte chunks
//     (chosen on the global side, since a direct-to-LDS load writes lane i at base + 16*i), which makes
//     the ds_read_b128 fragment reads bank-conflict free.
//   * Ping-pong.  Every sub-step has two phases separated by workgroup barriers.  In the first, team 0
//     issues nothing but its 16 MFMAs while team 1 reads its fragments and issues its loads; in the
//     second they swap.  A SIMD holds one wave of each team, so its matrix pipe always has a wave that
//     does nothing else.  Loads are addressed by a scalar base plus a per-lane 32-bit offset computed
//     once per item: vector ALU work in the load path would queue behind the other wave's MFMAs (64-bit
//     vector address arithmetic per load made the issue of eight loads take 2.3x as long).
//   * The loads are issued from inline assembly and the waits are written out by hand: left to itself
//     the compiler drains every outstanding load at each barrier and before LDS reads it cannot prove
//     independent, which serialises the pipeline.
//   * The int32 accumulators stay in registers through the epilogue: dequantisation, SiLU and the
//     gate*up product are applied in place; the int32 tile never goes to memory.  The MFMAs take the
//     weights as their first operand, so a lane ends up with ONE activation row and runs of four
//     consecutive weight columns: one row scale per lane, column scales as 16-byte vectors, and each
//     32-row fragment passes through a small LDS staging slice from which whole 128-byte lines are
//     stored.  For GMM1 the prepack pairs gate column c with up column I+c inside one wave.
//   * The K order inside a 32-deep MFMA step is whatever the two operands agree on (an integer dot
//     product does not care), which is what lets both be loaded as plain 16-byte pieces.
//   * Flat items are bound by the memory, and three things in this file exist for them alone: their weight
//     panels are fetched with non-temporal loads (nobody else reads them); they stop requesting stages in
//     their last sub-steps, where tall items keep a branch-free loop body and fetch the last sub-step again;
//     and between the K loop and the epilogue of a flat item the workgroup takes its next item and, if that
//     is flat too, touches the lines of its first stages so that they travel to L2 under the epilogue.
#include <algorithm>
#include <atomic>

#include "cam_device.h"
#include "cam_kernels.h"
#include "rank_device.h"
#include "permute_device.h"
#include "sched_device.h"
#include "../../include/cam_expf_spec.h"

namespace cam {

namespace {

constexpr int kBK = 64;                         // K bytes per sub-step
constexpr int kThreads = 512;                   // two teams of four waves
constexpr int kMaxStages = 4;
constexpr int kStageTall = 256 * kBK + 256 * kBK;   // 16 KB of activations + 16 KB of weights
constexpr int kStageFlat = 128 * kBK + 512 * kBK;   //  8 KB of activations + 32 KB of weights
constexpr int kLdsBytes = kMaxStages * kStageTall;  // 128 KB (flat: 3 x 40 KB = 120 KB)
constexpr int kScaleKb = 64;                    // FP8: K-blocks of 128 bytes an item may span (Kd <= 8192)
constexpr int kEpiRowBytes = 144;               // epilogue staging: 128 data bytes + 16 of padding per row
constexpr int kEpiSlice = 32 * kEpiRowBytes;    // one 32-row fragment per wave

// LDS offset (bytes) inside a stage of the 16-byte chunk `c` (0..3) of activation row `r`.
__device__ __forceinline__ int a_lds_offset(int r, int c)
{
    return r * kBK + ((c ^ ((r >> 2) & 3)) << 4);
}

// One direct-to-LDS load: lane i of the wave fetches 16 bytes at base + voff(i) and the data lands at LDS byte
// address lds_addr + 16*i.  The base is a scalar register pair, so issuing the load needs no vector ALU work.
__device__ __forceinline__ void dma16(const void *base, unsigned voff, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"((unsigned long long)base)
                 : "memory", "m0");
}

// The same load marked non-temporal, for bytes that are read once: a stream of them moves at 6.6-7.1 TB/s from
// HBM where the plain form stays at 5.8-6.0 (measured with a bare ring of these loads, 256 workgroups).
__device__ __forceinline__ void dma16_stream(const void *base, unsigned voff, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(lds_addr), "v"(voff), "s"((unsigned long long)base)
                 : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_loads_outstanding()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ void wait_lds_reads()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

// Workgroup barrier without the memory fence of __syncthreads(); the waits are explicit (above).
__device__ __forceinline__ void barrier_no_fence()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// What a wave needs to know about the item it works on (all wave-uniform).
struct ItemCtx {
    const int8_t *a_tile;   // first activation row of the tile
    const int8_t *wg;       // the expert's packed weights
    const float *sg;        // the expert's per-channel scales
    int m0, rows;           // first row and rows of the tile
    int a_row0, my_rows;    // first tile row of this wave's fragments, rows of them that exist
    int bslot;              // this wave's 64-column group inside the stage
    int nw;                 // this wave's packed 64-column group of the weight (clamped to a valid one)
    bool wave_live;         // the group exists (ragged last column block)
    int stage_a, stage_bytes;
    int Kd, N;
#ifdef CAM_GEMM_TIMELINE
    int *phase_s;           // LDS: wall clock at the first multiply and after the K loop (written by thread 0)
#endif
};

// One wave's part of one item.  TEAM 0 multiplies in the first phase of every sub-step, TEAM 1 in the second.
// FLAT selects the tile shape (it fixes the loads per wave and sub-step); MF is the wave's fragment count.
__device__ __forceinline__ int acc_bits(int v) { return v; }
__device__ __forceinline__ int acc_bits(float v) { return __float_as_int(v); }

template <bool FP8>
struct AccType {
    typedef v16i type;
};
template <>
struct AccType<true> {
    typedef v16f type;
};

// FP8 items (FP8 = true) run the same pipeline with v_mfma_scale_f32_32x32x64_f8f6f4: one instruction covers
// the 64 K bytes of a sub-step (the two 16-byte pieces a lane holds), takes the E8M0 scale of the lane's weight
// column block and of its activation row for the current 128-byte K block, and accumulates in fp32.  The
// scales of the item wait in LDS (a_scale8_s[kb * 256 + tile row], w_scale8_s[column group * kScaleKb + kb]) and
// are read with the fragments.
template <int MF, int TEAM, bool FLAT, bool FP8, typename Hook, typename Stage>
__device__ __forceinline__ void run_item(const GemmArgs &a, const ItemCtx &t, int nb, int8_t *lds,
                                         const float *row_scale_s, const uint8_t *a_scale8_s,
                                         const uint8_t *w_scale8_s, Hook &between, Stage &stage_scales)
{
    constexpr int NS = FLAT ? 3 : 4;                       // ring of stages
    constexpr int LPS = FLAT ? (TEAM == 0 ? 6 : 4) : 4;    // loads per wave and sub-step
    constexpr int MFR = MF > 0 ? MF : 1;
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wn = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);
    const int KT = t.Kd / kBK;
    const int last = KT - 1;
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) int8_t *)lds;

    typename AccType<FP8>::type acc[MFR][2];
#pragma unroll
    for (int mf = 0; mf < MFR; ++mf) {
#pragma unroll
        for (int nf = 0; nf < 2; ++nf) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                acc[mf][nf][i] = 0;
            }
        }
    }

    // ---- loads.  Tall: team 0 brings the activations (wave wn: tile rows 64wn .. 64wn+63, four loads of 16
    // rows), team 1 the weights (wave wn: the 4 KB of column group wn).  Flat: team 0 brings the activations
    // (wave wn: rows 32wn .. 32wn+31) and column groups 0..3, team 1 column groups 4..7.  Lane i of an
    // activation load brings row (i / 4) of its 16 and the chunk whose swizzled slot is i % 4; rows beyond the
    // tile repeat its last row (their results are dropped in the epilogue).
    constexpr int NA = FLAT ? (TEAM == 0 ? 2 : 0) : (TEAM == 0 ? 4 : 0);
    constexpr int NB = LPS - NA;
    unsigned a_voff[NA > 0 ? NA : 1];
    unsigned a_dst[NA > 0 ? NA : 1];
#pragma unroll
    for (int j = 0; j < NA; ++j) {
        const int r0 = (FLAT ? 32 : 64) * wn + 16 * j;
        const int r = r0 + (lane >> 2);
        const int c = (lane & 3) ^ ((r >> 2) & 3);
        a_voff[j] = (unsigned)(min(r, t.rows - 1) * t.Kd + c * 16);
        a_dst[j] = (unsigned)(r0 * kBK);
    }
    const int ngroups = t.N / 64;
    const int bgroup = FLAT ? TEAM * 4 + wn : wn;  // the column group of the stage this wave loads
    const int nw_load = min(nb * (FLAT ? 8 : 4) + bgroup, ngroups - 1);
    // Packed weights: column groups in blocks of eight; inside a block the 4 KB of a K step of its groups lie
    // side by side, so the loads of one step of a workgroup cover one contiguous stretch of memory.
    const int b_block = nw_load >> 3;
    const int b_step = min(8, ngroups - 8 * b_block) * 4096;
    const int8_t *b_base = t.wg + (long long)b_block * 8 * t.Kd * 64 + (nw_load & 7) * 4096;
    const unsigned b_voff = (unsigned)(lane * 16);
    const unsigned b_dst = (unsigned)(t.stage_a + bgroup * 4096);

    auto issue = [&](int s_idx, int slot) {
        const int s = min(s_idx, last);
        const unsigned sbase = lds0 + (unsigned)(slot * t.stage_bytes);
        if (NA > 0) {
            const int8_t *ab = t.a_tile + (long long)s * kBK;
#pragma unroll
            for (int j = 0; j < NA; ++j) {
                dma16(ab, a_voff[j], sbase + a_dst[j]);
            }
        }
        if (NB > 0) {
            const int8_t *bb = b_base + (long long)s * b_step;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                if (FLAT) {  // a flat item is the only reader of its weight panel
                    dma16_stream(bb + j * 1024, b_voff, sbase + b_dst + j * 1024);
                } else {
                    dma16(bb + j * 1024, b_voff, sbase + b_dst + j * 1024);
                }
            }
        }
    };

    // ---- fragments: read from LDS one phase before they are multiplied.
    v8i af[MFR];  // .lo: the K bytes of the first 32-byte half of the sub-step, .hi: of the second
    v8i bf[2];
    int sa[MFR];  // FP8: E8M0 scales of this lane's activation rows, and of its two weight column fragments
    int sw[2] = {0, 0};
    const int a_row = lane & 31;
    const int a_half = lane >> 5;
    auto read_frags = [&](int slot, int s_idx) {
        const int8_t *st = lds + slot * t.stage_bytes;
        const int8_t *sb = st + t.stage_a + t.bslot * 4096 + lane * 16;
#pragma unroll
        for (int nf = 0; nf < 2; ++nf) {
            bf[nf].lo = *(const v4i *)(sb + nf * 1024);
            bf[nf].hi = *(const v4i *)(sb + (2 + nf) * 1024);
        }
#pragma unroll
        for (int mf = 0; mf < MF; ++mf) {
            af[mf].lo = *(const v4i *)(st + a_lds_offset(t.a_row0 + mf * 32 + a_row, a_half));
            af[mf].hi = *(const v4i *)(st + a_lds_offset(t.a_row0 + mf * 32 + a_row, 2 + a_half));
        }
        if (FP8) {
            const int kb = min(s_idx, last) >> 1;
            sw[0] = w_scale8_s[(t.bslot * 2 + 0) * kScaleKb + kb];
            sw[1] = w_scale8_s[(t.bslot * 2 + 1) * kScaleKb + kb];
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
                sa[mf] = a_scale8_s[kb * 256 + t.a_row0 + mf * 32 + a_row];
            }
        }
    };
    auto multiply = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(2);
        // Weights as the first operand: the result tile comes out transposed, i.e. a lane holds ONE
        // activation row and 4 consecutive weight columns per register quad.
        if constexpr (FP8) {
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                for (int nf = 0; nf < 2; ++nf) {
                    acc[mf][nf] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[nf], af[mf], acc[mf][nf], 0, 0, 0,
                                                                                 sw[nf], 0, sa[mf]);
                }
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                    for (int nf = 0; nf < 2; ++nf) {
                        acc[mf][nf] = __builtin_amdgcn_mfma_i32_32x32x32_i8(kk == 0 ? bf[nf].lo : bf[nf].hi,
                                                                            kk == 0 ? af[mf].lo : af[mf].hi,
                                                                            acc[mf][nf], 0, 0, 0);
                    }
                }
            }
        }
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- pipeline.  Loads retire in order and every sub-step that requests a stage issues exactly LPS loads per
    // wave, so "at most n * LPS outstanding" says which sub-steps of this wave's loads have landed; the barrier
    // after the wait makes that true for the whole workgroup.  In the last NS sub-steps nothing is left to request
    // and the wait is for what remains: with `rem` stages after the current one, stage s+1 has landed once at most
    // rem - 1 stages are outstanding.
    //   barrier A(s): every load of stage s+1 has landed; team 1 is done reading stage s
    //   barrier B(s): team 0 is done reading stage s+1
    // Stage s is free once both teams have its fragments in registers, i.e. after barrier A(s): team 0 refills
    // it in the phase that follows, team 1 at the end of its own reading phase.
    auto wait_stages = [&](int n) {  // at most n stages of this wave's loads outstanding (n wave-uniform)
        if (n <= 0) {
            wait_loads_outstanding<0>();
        } else if (n == 1) {
            wait_loads_outstanding<LPS>();
        } else if (n == 2) {
            wait_loads_outstanding<2 * LPS>();
        } else {
            wait_loads_outstanding<3 * LPS>();
        }
    };
    // Tall tiles keep a loop body without control flow instead (their long bodies schedule worse with it: +2-4 %):
    // sub-step indices past the end are clamped, i.e. the last sub-step is fetched again into a stage nobody
    // reads, and every sub-step requests a stage.
#pragma unroll
    for (int p = 0; p < NS; ++p) {
        if (!FLAT || p <= last) {
            issue(p, p);
        }
    }
    // The item's scales go to LDS now, behind the requests for the first stages, so that their round trip to
    // memory runs beside that of the weights instead of ahead of it.  (Their loads are younger than the stage
    // loads and complete after them: the wait below is then met at once.)
    stage_scales();
    wait_lds_reads();
    if (FLAT) {
        wait_stages(min(NS - 1, last));
    } else {
        wait_loads_outstanding<(NS - 1) * LPS>();
    }
    barrier_no_fence();  // stage 0 has landed and every wave's share of the scales is in LDS
#ifdef CAM_GEMM_TIMELINE
    if (tid == 0) {
        t.phase_s[0] = (int)wall_clock64();
    }
#endif
    int slot = 0;        // slot of stage s
    const int steady = FLAT ? KT - NS : KT;  // sub-steps that request the stage NS ahead
    if (TEAM == 0) {
        read_frags(0, 0);
        wait_lds_reads();
        for (int s = 0; s < KT; ++s) {
            const int next = slot + 1 == NS ? 0 : slot + 1;
            multiply();                                   // phase 1: stage s, from registers
            if (!FLAT || s < steady) {
                wait_loads_outstanding<(NS - 2) * LPS>(); // my part of stage s+1 has landed
            } else if (s < last) {
                wait_stages(last - s - 1);
            }
            barrier_no_fence();                           // A(s)
            if (!FLAT || s < steady) {
                issue(s + NS, slot);                      // phase 2: refill stage s's slot ...
            }
            read_frags(next, s + 1);                      // ... and fetch the fragments of stage s+1
            wait_lds_reads();
            barrier_no_fence();                           // B(s)
            slot = next;
        }
    } else {
        for (int s = 0; s < KT; ++s) {
            const int next = slot + 1 == NS ? 0 : slot + 1;
            read_frags(slot, s);                          // phase 1: fragments of stage s ...
            wait_lds_reads();
            if (!FLAT || s < steady) {
                issue(s + NS, slot);                      // ... then refill its slot
                wait_loads_outstanding<(NS - 1) * LPS>(); // my part of stage s+1 has landed
            } else if (s < last) {
                wait_stages(last - s - 1);
            }
            barrier_no_fence();                           // A(s)
            multiply();                                   // phase 2: stage s
            barrier_no_fence();                           // B(s)
            slot = next;
        }
    }
    if (!FLAT) {
        wait_loads_outstanding<0>();
    }
    barrier_no_fence();  // nobody reads or fills the stages any more: the epilogue may stage through them
#ifdef CAM_GEMM_TIMELINE
    if (tid == 0) {
        t.phase_s[1] = (int)wall_clock64();
    }
#endif

    // ---- epilogue, accumulators in registers.
    // Lane l holds activation row (l & 31) of each 32x32 fragment; registers 4j .. 4j+3 hold the four
    // consecutive weight columns 8j + 4*(l/32) + 0..3.  Dequantisation runs on that layout with one row scale
    // per lane and fragment and the column scales fetched as 16-byte vectors.  To store whole 128-byte lines,
    // every wave passes one fragment at a time through its own slice of LDS: 128 staged bytes per row, then
    // 16 bytes per lane and 8 rows per store instruction.
    // `between` is the workgroup's business between two items (taking the next one and asking for its first
    // bytes, see gemm_kernel).  It runs after this wave has requested its column scales and before it uses them,
    // so that its memory traffic travels under the arithmetic of the epilogue; it returns a value that depends on
    // what it loaded, consumed at the very end so that nothing waits for those loads earlier.
    int between_sink = 0;
    auto epilogue = [&]() {
    const bool work = MF > 0 && t.wave_live;
    v4f csc[2][4];  // column scales: [0] gate / [1] up of a paired group, or the two fragments of a plain one
    if (FLAT && !FP8 && work && a.epilogue != kEpiInt32) {
        const int col_half = (lane >> 5) * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (a.epilogue == kEpiSwiglu) {
                csc[0][j] = *(const v4f *)(t.sg + t.nw * 32 + 8 * j + col_half);
                csc[1][j] = *(const v4f *)(t.sg + t.N / 2 + t.nw * 32 + 8 * j + col_half);
            } else {
                csc[0][j] = *(const v4f *)(t.sg + t.nw * 64 + 8 * j + col_half);
                csc[1][j] = *(const v4f *)(t.sg + t.nw * 64 + 32 + 8 * j + col_half);
            }
        }
    }
    if (FLAT) {
        between_sink = between();
    }
    if (work) {
        const int wave = tid >> 6;
        const int row_in = lane & 31;
        const int col_half = (lane >> 5) * 4;
        int8_t *slice = lds + wave * kEpiSlice;
        const int N = t.N;
        const int nw = t.nw;

        // Copies rows [0, 32) of the slice (128 bytes each) to dst + (first + row) * row_pitch_bytes.
        auto flush_fragment = [&](int8_t *dst, long long row_pitch_bytes, int mf) {
            const int sub = lane >> 3;    // row inside a group of 8
            const int piece = lane & 7;   // 16-byte piece of the 128-byte row
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int row = it * 8 + sub;
                const v4u v = *(const v4u *)(slice + row * kEpiRowBytes + piece * 16);
                const int trow = mf * 32 + row;
                if (trow < t.my_rows) {
                    // the next kernel reads these rows once; stored non-temporally they do not push weight panels
                    // and activation tiles out of the L2 (C3 both operators 519 -> 506 us, decode layer 427 -> 420 us)
                    __builtin_nontemporal_store(v, (v4u *)(dst + (long long)(t.m0 + t.a_row0 + trow) * row_pitch_bytes + piece * 16));
                }
            }
        };

        if (a.epilogue == kEpiInt32) {
#pragma unroll
            for (int nf = 0; nf < 2; ++nf) {
                const int col0 = a.gate_up ? (nf * (N / 2) + nw * 32) : (nw * 64 + nf * 32);
#pragma unroll
                for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // int32 sums, or the bits of the fp32 sums of an FP8 item
                        const v4i v = {acc_bits(acc[mf][nf][4 * j]), acc_bits(acc[mf][nf][4 * j + 1]),
                                       acc_bits(acc[mf][nf][4 * j + 2]), acc_bits(acc[mf][nf][4 * j + 3])};
                        *(v4i *)(slice + row_in * kEpiRowBytes + (8 * j + col_half) * 4) = v;
                    }
                    flush_fragment((int8_t *)a.out + (long long)col0 * 4, (long long)N * 4, mf);
                }
            }
        } else if (a.epilogue == kEpiSwiglu) {
            // t = (float(C) * w_scale[n]) * x_scale[m]; y = silu(t_gate) * t_up
            const int I = N / 2;
            v4f sg_gate[4], sg_up[4];
            if (!FP8) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (FLAT) {
                        sg_gate[j] = csc[0][j];
                        sg_up[j] = csc[1][j];
                    } else {
                        sg_gate[j] = *(const v4f *)(t.sg + nw * 32 + 8 * j + col_half);
                        sg_up[j] = *(const v4f *)(t.sg + I + nw * 32 + 8 * j + col_half);
                    }
                }
            }
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
                const float xs = FP8 ? 1.0f : row_scale_s[t.a_row0 + mf * 32 + row_in];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    v4f y;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float tg, tu;
                        if constexpr (FP8) {  // the sums carry their scales already
                            tg = acc[mf][0][4 * j + e];
                            tu = acc[mf][1][4 * j + e];
                        } else {
                            tg = __fmul_rn(__fmul_rn((float)acc[mf][0][4 * j + e], sg_gate[j][e]), xs);
                            tu = __fmul_rn(__fmul_rn((float)acc[mf][1][4 * j + e], sg_up[j][e]), xs);
                        }
                        y[e] = __fmul_rn(cam_silu_spec(tg), tu);
                    }
                    *(v4f *)(slice + row_in * kEpiRowBytes + (8 * j + col_half) * 4) = y;
                }
                flush_fragment((int8_t *)a.out + (long long)(nw * 32) * 4, (long long)I * 4, mf);
            }
        } else {
            v4f ws[2][4];
            if (!FP8) {
#pragma unroll
                for (int nf = 0; nf < 2; ++nf) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        ws[nf][j] = FLAT ? csc[nf][j] : *(const v4f *)(t.sg + nw * 64 + nf * 32 + 8 * j + col_half);
                    }
                }
            }
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
                const float xs = FP8 ? 1.0f : row_scale_s[t.a_row0 + mf * 32 + row_in];
#pragma unroll
                for (int nf = 0; nf < 2; ++nf) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float f[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if constexpr (FP8) {
                                f[e] = acc[mf][nf][4 * j + e];
                            } else {
                                f[e] = __fmul_rn(__fmul_rn((float)acc[mf][nf][4 * j + e], ws[nf][j][e]), xs);
                            }
                        }
                        // two values per conversion instruction: with the rounding spelled out in integer
                        // arithmetic this epilogue took a quarter of a short-K tile's time in the vector ALU
                        v2u v;
                        if (a.out_fp16) {
                            v = v2u{f32_to_fp16_bits(f[0]) | (f32_to_fp16_bits(f[1]) << 16),
                                    f32_to_fp16_bits(f[2]) | (f32_to_fp16_bits(f[3]) << 16)};
                        } else {
                            v = v2u{f32x2_to_bf16x2_bits(f[0], f[1]), f32x2_to_bf16x2_bits(f[2], f[3])};
                        }
                        *(v2u *)(slice + row_in * kEpiRowBytes + (nf * 32 + 8 * j + col_half) * 2) = v;
                    }
                }
                flush_fragment((int8_t *)a.out + (long long)(nw * 64) * 2, (long long)N * 2, mf);
            }
        }
    }
    };

    // ---- FP8 gate/up GEMM whose output feeds the next FP8 GEMM: quantise the SwiGLU product here.  A block of
    // 128 product columns is exactly what the four waves of a team hold for their rows (32 columns each), so the
    // block maximum needs one exchange through LDS; every wave of the workgroup takes part in its barrier.
    auto epilogue_quant = [&]() {
        if (FLAT) {
            between_sink = between();
        }
        const bool work = MF > 0 && t.wave_live;
        const int wave = tid >> 6;
        const int row_in = lane & 31;
        const int col_half = (lane >> 5) * 4;
        float *rowmax = (float *)(lds + 8 * kEpiSlice);  // [wave][tile row of the wave's fragments]
        if constexpr (FP8) {
            if (work) {
#pragma unroll
                for (int mf = 0; mf < MF; ++mf) {
                    float m = 0.0f;
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const float y = __fmul_rn(cam_silu_spec(acc[mf][0][i]), acc[mf][1][i]);
                        acc[mf][0][i] = y;
                        m = fmaxf(m, fabsf(y));
                    }
                    m = fmaxf(m, __shfl_xor(m, 32, kWave));
                    if (lane < 32) {
                        rowmax[wave * 128 + mf * 32 + lane] = m;
                    }
                }
            }
            wait_lds_reads();
            barrier_no_fence();
            if (work) {
                const int I = t.N / 2;
                int8_t *slice = lds + wave * kEpiSlice;
                uint8_t *q = (uint8_t *)a.out;
#pragma unroll
                for (int mf = 0; mf < MF; ++mf) {
                    const float *pm = rowmax + (wave & 4) * 128 + mf * 32 + row_in;  // the team's four waves
                    const float m = fmaxf(fmaxf(pm[0], pm[128]), fmaxf(pm[256], pm[384]));
                    const int ex = fp8_block_scale_exp(m);
                    const float f1 = exp2_int(-(ex / 2)), f2 = exp2_int(-(ex - ex / 2));
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        int w = 0;
                        w = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(acc[mf][0][4 * j], f1), f2),
                                                            __fmul_rn(__fmul_rn(acc[mf][0][4 * j + 1], f1), f2), w, false);
                        w = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(acc[mf][0][4 * j + 2], f1), f2),
                                                            __fmul_rn(__fmul_rn(acc[mf][0][4 * j + 3], f1), f2), w, true);
                        *(int *)(slice + row_in * 48 + 8 * j + col_half) = w;
                    }
                    // 32 rows x 32 bytes staged (48-byte pitch): two lanes per row write its two 16-byte halves
                    const int row = lane >> 1, piece = lane & 1;
                    const v4u v = *(const v4u *)(slice + row * 48 + piece * 16);
                    if (mf * 32 + row < t.my_rows) {
                        const long long grow = t.m0 + t.a_row0 + mf * 32 + row;
                        *(v4u *)(q + grow * I + t.nw * 32 + piece * 16) = v;
                    }
                    if ((wave & 3) == 0 && lane < 32 && mf * 32 + lane < t.my_rows) {
                        const long long grow = t.m0 + t.a_row0 + mf * 32 + lane;
                        a.out_scale8[grow * (I >> 7) + (t.nw >> 2)] = (uint8_t)(ex + 127);
                    }
                }
            }
        }
    };

    if (FP8 && a.epilogue == kEpiSwigluFp8) {
        epilogue_quant();
    } else {
        epilogue();
    }
    barrier_no_fence();  // the staging slices are free again before the next item's loads land
    asm volatile("" ::"v"(between_sink));
}

template <int TEAM, bool FLAT, bool FP8, typename Hook, typename Stage>
__device__ __forceinline__ void run_item_mf(int mf, const GemmArgs &a, const ItemCtx &t, int nb, int8_t *lds,
                                            const float *row_scale_s, const uint8_t *a_scale8_s,
                                            const uint8_t *w_scale8_s, Hook &between, Stage &stage_scales)
{
    switch (mf) {
        case 0: run_item<0, TEAM, FLAT, FP8>(a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales); break;
        case 1: run_item<1, TEAM, FLAT, FP8>(a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales); break;
        case 2: run_item<2, TEAM, FLAT, FP8>(a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales); break;
        case 3: run_item<3, TEAM, FLAT, FP8>(a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales); break;
        default: run_item<4, TEAM, FLAT, FP8>(a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales); break;
    }
}

template <bool FP8>
__global__ __launch_bounds__(kThreads, 1) void gemm_kernel(GemmArgs a)
{
    __shared__ __attribute__((aligned(1024))) int8_t lds[kLdsBytes];
    __shared__ float row_scale_s[256];
    __shared__ __attribute__((aligned(16))) uint8_t a_scale8_s[FP8 ? kScaleKb * 256 : 4];
    __shared__ uint8_t w_scale8_s[FP8 ? 16 * kScaleKb : 4];
    __shared__ int item_s;
    __shared__ int next_s;
#ifdef CAM_GEMM_TIMELINE
    __shared__ int phase_s[2];
#endif

    const int tid = threadIdx.x;
    const int team = __builtin_amdgcn_readfirstlane(tid >> 8);
    const int wn = __builtin_amdgcn_readfirstlane((tid >> 6) & 3);
    int32_t *sched = a.sched;
    const int32_t *qstart = sched + kSchedQueueStart;
    int32_t *qcount = sched + kSchedQueueCount;
    const SchedItem *items = (const SchedItem *)(sched + kSchedHeader);
    const bool shared = (sched[3] & 2) != 0;   // long schedules: one queue per XCD, every item asked for
    const int me = shared ? (int)blockIdx.x % max(min(sched[2], kMaxQueues), 1) : (int)blockIdx.x;  // this workgroup's queue
    const int q0 = qstart[min(me, kMaxQueues)];
    const int qlen = me < kMaxQueues ? qstart[me + 1] - q0 : 0;
    bool own_empty = qlen <= (shared ? 0 : 1);  // an own queue's first item needs no asking; there may be nothing after it

    // Work items.  Short schedules: every workgroup has a queue of its own, built to last as long as the others
    // (sched_device.h).  Its first item is its own without asking; for the following ones it advances its queue's
    // counter with a device-scope atomic, a round trip to the memory side that is issued at the START of an item
    // and looked at only when the item is done (take_begin / take_end).  Long schedules: the workgroups of an XCD
    // share one queue and ask for every item, the first included.  Every counter has a cache line of its own.  A
    // workgroup whose queue has run out helps the queue with the most items left (its own XCD's first, so that
    // what it fetches is likely to be in its L2): wave 0 looks at every counter at once, one round trip, and its
    // first lane then advances the chosen one.  A counter only ever grows and every queue is finite, so every
    // workgroup leaves.
    auto take_begin = [&]() -> int {  // thread 0
        return own_empty ? 0 : atomicAdd(&qcount[me * kSchedQueueStride], 1);
    };
    auto steal = [&]() -> int {  // all lanes of wave 0; the result is valid in every lane
        const int lane = tid & (kWave - 1);
        const int nq = min(sched[2], kMaxQueues);
        if ((sched[3] & 1) != 0) {  // every queue's only item is its workgroup's own: there is nothing to take over
            return -1;
        }
        for (int attempt = 0; attempt < 4; ++attempt) {
            int best = -1;  // (items left, same XCD, queue) packed so that the maximum is the choice
            for (int v = lane; v < nq; v += kWave) {
                const int len = qstart[v + 1] - qstart[v];
                const int seen = __hip_atomic_load(&qcount[v * kSchedQueueStride], __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
                const int left = len - seen;
                if (left > 0 && v != me) {
                    best = max(best, (min(left, 1023) << 11) | ((v % kNumXcd == me % kNumXcd ? 1 : 0) << 10) | v);
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                best = max(best, __shfl_xor(best, off, kWave));
            }
            if (best < 0) {
                return -1;
            }
            // the queue number fits ten bits only below 1024 queues, which kMaxQueues guarantees
            const int v = best & 1023;
            int got = -1;
            if (lane == 0) {
                const int i = atomicAdd(&qcount[v * kSchedQueueStride], 1);
                got = i < qstart[v + 1] - qstart[v] ? qstart[v] + i : -1;
            }
            got = __shfl(got, 0, kWave);
            if (got >= 0) {
                return got;
            }
        }
        return -1;
    };
    // The item after the one whose take was `taken`; called by all threads of wave 0 (the answer is for thread 0).
    auto take_end = [&](int taken) -> int {
        taken = __shfl(taken, 0, kWave);
        if (!own_empty) {
            if (taken < qlen) {
                return q0 + taken;
            }
            own_empty = true;
        }
        return steal();
    };

    int next = -1;
    if (tid < kWave) {
        if (shared) {
            int taken = 0;
            if (tid == 0) {
                taken = take_begin();
            }
            next = take_end(taken);
        } else {
            next = qlen > 0 ? q0 : steal();
        }
    }
    for (;;) {
        if (tid == 0) {
            item_s = next;
        }
        __syncthreads();
        const int idx = item_s;
        if (idx < 0) {
            return;
        }
        int taken = 0;
        if (tid == 0) {
            taken = take_begin();  // in flight while this item runs
        }
        SchedItem it = items[idx];
#ifdef CAM_GEMM_TIMELINE
        // Build option for profiling only: thread 0 leaves the item's start and end times (wall_clock64, 100 MHz)
        // and the workgroup that ran it in the item's two spare words.
        const long long timeline_t0 = wall_clock64();
#endif
        const int g = __builtin_amdgcn_readfirstlane(it.g);
        const int m0 = __builtin_amdgcn_readfirstlane(it.m0);
        const int rows = __builtin_amdgcn_readfirstlane(it.rows);
        const int split = __builtin_amdgcn_readfirstlane(it.split);
        const int nb = __builtin_amdgcn_readfirstlane(it.nb);
        const bool flat = __builtin_amdgcn_readfirstlane(it.flat) != 0;

        ItemCtx t;
#ifdef CAM_GEMM_TIMELINE
        t.phase_s = phase_s;
#endif
        t.Kd = a.Kd;
        t.N = a.N;
        t.m0 = m0;
        t.rows = rows;
        t.a_tile = a.a + (long long)m0 * a.Kd;
        t.wg = a.per_expert ? a.list.w[g] : a.w + (long long)g * a.Kd * a.N;
        t.sg = a.per_expert ? a.list.s[g] : a.w_scale + (long long)g * a.N;
        if (flat) {
            t.a_row0 = 0;
            t.my_rows = rows;
            t.bslot = team * 4 + wn;
            t.stage_a = 128 * kBK;
            t.stage_bytes = kStageFlat;
        } else {
            t.a_row0 = team == 0 ? 0 : split;
            t.my_rows = team == 0 ? min(split, rows) : rows - split;
            t.bslot = wn;
            t.stage_a = 256 * kBK;
            t.stage_bytes = kStageTall;
        }
        const int group = nb * (flat ? 8 : 4) + t.bslot;
        t.wave_live = group < a.N / 64;
        t.nw = min(group, a.N / 64 - 1);
        auto stage_scales = [&]() {
            if (FP8) {
                // the item's scales: activation rows x K blocks (transposed, so that the lanes of a fragment read
                // neighbouring bytes), and one row of K blocks per 64-column group of the item
                // Only the rows the fragments read (the tile's rows, to the next multiple of 32), and, where a row's
                // scales are whole words, four K blocks per load and four loads in flight per thread: fetched a byte
                // at a time for all 256 rows, with a wait per byte, this took 3-4 us of every item.
                const int KB = a.Kd >> 7;
                const int rpad = min(256, (rows + 31) & ~31);
                if ((KB & 3) == 0) {
                    // a thread takes four K blocks of four consecutive rows: four word loads, a 4x4 byte transpose,
                    // four word stores (neighbouring lanes write neighbouring words)
                    const int wpr = KB >> 2;    // words per row
                    const int rgs = rpad >> 2;  // groups of four rows
                    for (int i = tid; i < rgs * wpr; i += kThreads) {
                        const int q = i / rgs, rg = i - q * rgs;
                        uint32_t v[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            v[u] = *(const uint32_t *)(a.a_scale8 + (long long)(m0 + min(4 * rg + u, rows - 1)) * KB + 4 * q);
                        }
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const uint32_t w = ((v[0] >> (8 * j)) & 0xffu) | (((v[1] >> (8 * j)) & 0xffu) << 8) |
                                               (((v[2] >> (8 * j)) & 0xffu) << 16) | (((v[3] >> (8 * j)) & 0xffu) << 24);
                            *(uint32_t *)(a_scale8_s + (4 * q + j) * 256 + 4 * rg) = w;
                        }
                    }
                } else {
                    for (int i = tid; i < rpad * KB; i += kThreads) {
                        const int r = i / KB, kb = i - r * KB;
                        a_scale8_s[kb * 256 + r] = a.a_scale8[(long long)(m0 + min(r, rows - 1)) * KB + kb];
                    }
                }
                const int ngr = flat ? 8 : 4;
                const int nblk = a.N >> 7;
                for (int i = tid; i < ngr * 2 * KB; i += kThreads) {
                    const int gf = i / KB, kb = i - gf * KB;  // gf = column group of the item * 2 + fragment
                    const int grp = min(nb * ngr + (gf >> 1), a.N / 64 - 1);  // packed 64-column group of the weight
                    const int nf = gf & 1;
                    // first logical column of the fragment (a paired group holds 32 gate and 32 up columns)
                    const int col = a.gate_up ? nf * (a.N / 2) + grp * 32 : grp * 64 + nf * 32;
                    w_scale8_s[gf * kScaleKb + kb] = a.w_scale8[((long long)g * KB + kb) * nblk + (col >> 7)];
                }
            } else if (a.epilogue != kEpiInt32 && tid < 256) {
                row_scale_s[tid] = a.a_scale[m0 + min(tid, rows - 1)];
            }
        };

        // Between the K loop and the epilogue of this item: thread 0 learns which item comes next (its take has
        // been in flight since this item began), and every wave asks for the first bytes that item will load --
        // one word of every 128-byte line of its first stages -- so that they are on their way to this XCD's L2
        // while the epilogue computes, and the next item's first direct-to-LDS loads find them there.
        auto between = [&]() -> int {
            if (tid < kWave) {
                next = take_end(taken);
                if (tid == 0) {
                    next_s = next;
                }
            }
            __syncthreads();
            const int nidx = next_s;
            int sink = 0;
            if (nidx >= 0 && items[nidx].flat != 0) {  // tall items find their panels in L2 (sibling tiles)
                const SchedItem nx = items[nidx];
                const int ng = __builtin_amdgcn_readfirstlane(nx.g);
                const int nm0 = __builtin_amdgcn_readfirstlane(nx.m0);
                const int nrows = __builtin_amdgcn_readfirstlane(nx.rows);
                const int nnb = __builtin_amdgcn_readfirstlane(nx.nb);
                const bool nflat = __builtin_amdgcn_readfirstlane(nx.flat) != 0;
                const int stages = nflat ? 3 : 4;
                const int lane = tid & (kWave - 1);
                if (nflat || team == 1) {  // the waves that load weights: 4 KB per stage and wave
                    const int8_t *wgn = a.per_expert ? a.list.w[ng] : a.w + (long long)ng * a.Kd * a.N;
                    const int ngroups = a.N / 64;
                    const int grp = min(nnb * (nflat ? 8 : 4) + (nflat ? team * 4 + wn : wn), ngroups - 1);
                    const int blk = grp >> 3;
                    const long long step = (long long)min(8, ngroups - 8 * blk) * 4096;
                    const int8_t *base = wgn + (long long)blk * 8 * a.Kd * 64 + (grp & 7) * 4096;
                    const int steps = min(stages, a.Kd / kBK);
                    for (int i = lane; i < steps * 32; i += kWave) {  // 32 lines per stage
                        sink ^= *(const int *)(base + (long long)(i >> 5) * step + (i & 31) * 128);
                    }
                }
                if (team == 0) {  // the waves that load activations: rows of 64 bytes per stage
                    const int per_wave = nflat ? 32 : 64;
                    const int span = min(stages * kBK, a.Kd);          // bytes of a row the first stages cover
                    const int lines = (span + 127) / 128;
                    for (int i = lane; i < per_wave * lines; i += kWave) {
                        const int r = min(per_wave * wn + i / lines, nrows - 1);
                        sink ^= *(const int *)(a.a + (long long)(nm0 + r) * a.Kd + (i % lines) * 128);
                    }
                }
            }
            return sink;
        };

        const int mf = t.my_rows <= 0 ? 0 : (t.my_rows + 31) >> 5;
        if (flat) {
            if (team == 0) {
                run_item_mf<0, true, FP8>(mf, a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales);
            } else {
                run_item_mf<1, true, FP8>(mf, a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales);
            }
        } else {
            if (team == 0) {
                run_item_mf<0, false, FP8>(mf, a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales);
            } else {
                run_item_mf<1, false, FP8>(mf, a, t, nb, lds, row_scale_s, a_scale8_s, w_scale8_s, between, stage_scales);
            }
        }
#ifdef CAM_GEMM_TIMELINE
        if (tid == 0) {
            int32_t *stamp = (int32_t *)&items[idx];
            stamp[6] = (int32_t)timeline_t0;
            stamp[7] = (int32_t)wall_clock64();
            stamp[3] = (stamp[3] & 0xffff) | ((int)blockIdx.x << 16);  // split is read at the start of the item only
            // ticks from the start of the item to its first multiply and to the end of its K loop, in the upper
            // halves of the column-block and shape words (both below 2^16 and read before an item starts)
            const int d1 = min(max(phase_s[0] - (int32_t)timeline_t0, 0), 0xffff);
            const int d2 = min(max(phase_s[1] - (int32_t)timeline_t0, 0), 0x7fff);
            stamp[4] = (stamp[4] & 0xffff) | (d1 << 16);
            stamp[5] = (stamp[5] & 0xffff) | (d2 << 16);
        }
#endif
        if (!flat && tid < kWave) {  // a flat item has taken its successor between its K loop and its epilogue
            next = take_end(taken);
        }
    }
}

__global__ __launch_bounds__(1024) void build_sched_kernel(SchedBuild sb)
{
    __shared__ SchedShared sh;
    build_sched_part<1024>(sh, sb, (int)blockIdx.y, (int)blockIdx.x, (int)gridDim.x);
}

// SwiGLU product rows (fp32) -> int8 rows + per-row scale:
//   m = max|y|; y_scale = m * (1/127); q = rint((y * 127) * (1/m)).   One wave per row (four rows per workgroup):
// the row waits in registers between the maximum and the scaling, the maximum needs wave shuffles only, and no
// wave waits for another.
__global__ __launch_bounds__(256) void requant_kernel(const float *__restrict__ y, int I,
                                                      const int32_t *__restrict__ sched, long long max_rows,
                                                      int8_t *__restrict__ q, float *__restrict__ scale)
{
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long valid = sched != nullptr ? min((long long)sched[1], max_rows) : max_rows;
    if (row >= valid) {
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const int n4 = I >> 2;
    constexpr int kMaxPer = 16;  // I <= 4096
    v4f v[kMaxPer];
    float m = 0.0f;
    const v4f *src = (const v4f *)(y + row * I);
#pragma unroll
    for (int j = 0; j < kMaxPer; ++j) {
        const int c = lane + j * kWave;
        v[j] = v4f{0.f, 0.f, 0.f, 0.f};
        if (c < n4) {
            v[j] = __builtin_nontemporal_load(src + c);
        }
    }
#pragma unroll
    for (int j = 0; j < kMaxPer; ++j) {
        m = fmaxf(m, fmaxf(fmaxf(fabsf(v[j][0]), fabsf(v[j][1])), fmaxf(fabsf(v[j][2]), fabsf(v[j][3]))));
    }
    m = wave_max(m);
    const bool zero_row = m == 0.0f;
    const float rcp = zero_row ? 0.0f : __fdiv_rn(1.0f, m);
    if (lane == 0) {
        scale[row] = zero_row ? 0.0f : __fmul_rn(m, 1.0f / 127.0f);
    }
    uint32_t *dst = (uint32_t *)(q + row * I);
#pragma unroll
    for (int j = 0; j < kMaxPer; ++j) {
        const int c = lane + j * kWave;
        if (c < n4) {
            int b[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                b[e] = (int)rintf(__fmul_rn(__fmul_rn(v[j][e], 127.0f), rcp));
            }
            dst[c] = (uint32_t)(b[0] & 0xff) | ((uint32_t)(b[1] & 0xff) << 8) | ((uint32_t)(b[2] & 0xff) << 16) |
                     ((uint32_t)(b[3] & 0xff) << 24);
        }
    }
}

// fp32 rows -> FP8 E4M3 with one E8M0 scale per row and 128 columns (include/cam_fp8_spec.h).  A wave takes 512
// columns of a row: lane l the 8 columns from 8 l, so a block of 128 columns is a quarter of the wave.
__global__ __launch_bounds__(256) void requant_fp8_kernel(const float *__restrict__ y, int I,
                                                          const int32_t *__restrict__ sched, long long max_rows,
                                                          uint8_t *__restrict__ q, uint8_t *__restrict__ scale)
{
    const long long row = blockIdx.x;
    const long long valid = sched != nullptr ? min((long long)sched[1], max_rows) : max_rows;
    if (row >= valid) {
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    for (int c0 = wave * 512; c0 < I; c0 += 4 * 512) {
        const int col = c0 + lane * 8;
        const bool live = col < I;
        float x[8];
        float m = 0.0f;
        if (live) {
            const v4f lo = __builtin_nontemporal_load((const v4f *)(y + row * I + col));
            const v4f hi = __builtin_nontemporal_load((const v4f *)(y + row * I + col + 4));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                x[e] = lo[e];
                x[4 + e] = hi[e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                m = fmaxf(m, fabsf(x[e]));
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[e] = 0.0f;
            }
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            m = fmaxf(m, __shfl_xor(m, off, kWave));
        }
        const int ex = fp8_block_scale_exp(m);
        const float f1 = exp2_int(-(ex / 2)), f2 = exp2_int(-(ex - ex / 2));
        int lo = 0, hi = 0;
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[0], f1), f2), __fmul_rn(__fmul_rn(x[1], f1), f2), lo,
                                             false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[2], f1), f2), __fmul_rn(__fmul_rn(x[3], f1), f2), lo,
                                             true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[4], f1), f2), __fmul_rn(__fmul_rn(x[5], f1), f2), hi,
                                             false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[6], f1), f2), __fmul_rn(__fmul_rn(x[7], f1), f2), hi,
                                             true);
        if (live) {
            *(v2u *)(q + row * I + col) = v2u{(uint32_t)lo, (uint32_t)hi};
            if ((lane & 15) == 0) {
                scale[row * (I >> 7) + (col >> 7)] = (uint8_t)(ex + 127);
            }
        }
    }
}

// Row-major [G,Kd,N] int8 -> MFMA operand order.  One thread writes one 16-byte piece: piece (nw, ks, nf, lane)
// holds K rows ks*32 + (lane/32)*16 + 0..15 of logical column
//   gate_up ? nf*(N/2) + nw*32 + lane%32 : nw*64 + nf*32 + lane%32.
// The NW = N/64 column groups are stored in blocks of eight (the last block may hold fewer, gw of them); a block
// starts at piece 8*(nw/8)*KS*128 of the expert and orders its pieces as [ks/2][nw%8][ks%2][nf][lane], i.e. the
// gw * 4 KB that one 64-byte K step of the block's groups needs are contiguous.
__global__ __launch_bounds__(256) void prepack_kernel(const int8_t *__restrict__ src, int8_t *__restrict__ dst,
                                                      int Kd, int N, int gate_up, long long pieces_per_expert)
{
    const long long p = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const int g = blockIdx.y;
    if (p >= pieces_per_expert) {
        return;
    }
    const int KS = Kd / 32;
    const int lane = (int)(p & 63);
    long long r = p >> 6;
    const int nf = (int)(r & 1);
    r >>= 1;
    const int ks = (int)(r % KS);
    const int nw = (int)(r / KS);
    const int col = gate_up ? nf * (N / 2) + nw * 32 + (lane & 31) : nw * 64 + nf * 32 + (lane & 31);
    const int k0 = ks * 32 + (lane >> 5) * 16;
    const int8_t *s = src + (long long)g * Kd * N + (long long)k0 * N + col;
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t b0 = (uint8_t)s[(long long)(4 * j + 0) * N];
        uint32_t b1 = (uint8_t)s[(long long)(4 * j + 1) * N];
        uint32_t b2 = (uint8_t)s[(long long)(4 * j + 2) * N];
        uint32_t b3 = (uint8_t)s[(long long)(4 * j + 3) * N];
        w[j] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
    }
    v4u o = {w[0], w[1], w[2], w[3]};
    const int NW = N / 64;
    const int block = nw >> 3;
    const int gw = min(8, NW - 8 * block);
    const long long q = (long long)block * 8 * KS * 128 + (long long)(ks >> 1) * (gw * 256) + (nw & 7) * 256 +
                        (ks & 1) * 128 + nf * 64 + lane;
    *((v4u *)(dst + (long long)g * Kd * N) + q) = o;
}

// Workgroups of the persistent kernel: one per CU of the device the launch goes to (looked up once per device).
constexpr int kMaxDevices = 64;
std::atomic<int> g_num_cus[kMaxDevices];

hipError_t cus_of_current_device(int *out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        return e;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    int n = g_num_cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) {
            return e;
        }
        n = n > 0 ? n : 256;
        g_num_cus[dev].store(n, std::memory_order_relaxed);
    }
    *out = n;
    return hipSuccess;
}

}  // namespace

int sched_max_items(int64_t max_rows, int G, int N)
{
    // tall experts own at most max_rows / 129 + G row tiles between them, flat experts one each
    const int64_t tiles = max_rows / 129 + G;
    return (int)(tiles * ((N + 255) / 256));
}

uint64_t sched_bytes(int64_t max_rows, int G, int N)
{
    return (uint64_t)(kSchedHeader + (int64_t)sched_max_items(max_rows, G, N) * (int)(sizeof(SchedItem) / 4)) * 4;
}

hipError_t gemm_workgroups(int *out)
{
    int n = 0;
    const hipError_t e = cus_of_current_device(&n);
    if (e == hipSuccess) {
        *out = n < kMaxQueues ? n : kMaxQueues;
    }
    return e;
}

hipError_t launch_build_sched(const int64_t *group_list, int cumulative, int G, int64_t max_rows, int nspec,
                              const SchedSpec *specs, hipStream_t stream)
{
    if (G <= 0 || G > kMaxExperts || nspec < 1 || nspec > 2) {
        return hipErrorInvalidValue;
    }
    SchedBuild sb{};
    sb.group_list = group_list;
    sb.cumulative = cumulative;
    sb.G = G;
    sb.nspec = nspec;
    sb.max_rows = (long long)max_rows;
    sb.spec[0] = specs[0];
    sb.spec[1] = nspec > 1 ? specs[1] : specs[0];
    const hipError_t qe = gemm_workgroups(&sb.queues);
    if (qe != hipSuccess) {
        return qe;
    }
    const int cap = max(sb.spec[0].max_items, sb.spec[1].max_items);
    sb.parts = min(max(cap / 2048, 1), 4);  // long tables only: two turns of a thousand items cost no more than a second workgroup
    hipLaunchKernelGGL(build_sched_kernel, dim3((unsigned)sb.parts, (unsigned)nspec), dim3(1024), 0, stream, sb);
    return hipGetLastError();
}

hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream)
{
    if (a.sched == nullptr) {
        return hipErrorInvalidValue;
    }
    if (a.Kd % kBK != 0 || a.Kd < kBK || a.N % 64 != 0 || (a.gate_up && a.N % 128 != 0)) {
        return hipErrorInvalidValue;
    }
    int num_cus = 0;
    const hipError_t ce = gemm_workgroups(&num_cus);
    if (ce != hipSuccess) {
        return ce;
    }
    if (a.fp8) {
        if (a.Kd % 128 != 0 || a.N % 128 != 0 || (a.gate_up && a.N % 256 != 0) || a.Kd / 128 > kScaleKb ||
            a.per_expert || a.a_scale8 == nullptr || a.w_scale8 == nullptr) {
            return hipErrorInvalidValue;
        }
        if (a.epilogue == kEpiSwigluFp8 && (!a.gate_up || a.out_scale8 == nullptr)) {
            return hipErrorInvalidValue;
        }
        hipLaunchKernelGGL(gemm_kernel<true>, dim3((unsigned)num_cus), dim3(kThreads), 0, stream, a);
    } else {
        if (a.epilogue == kEpiSwigluFp8) {
            return hipErrorInvalidValue;
        }
        hipLaunchKernelGGL(gemm_kernel<false>, dim3((unsigned)num_cus), dim3(kThreads), 0, stream, a);
    }
    return hipGetLastError();
}

hipError_t launch_requant(const float *y, int64_t max_rows, int I, const int32_t *sched_for_rows, int8_t *q,
                          float *scale, hipStream_t stream)
{
    if (max_rows <= 0) {
        return hipSuccess;
    }
    if (I % 4 != 0 || I > 4096) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(requant_kernel, dim3((unsigned)((max_rows + 3) / 4)), dim3(256), 0, stream, y, I, sched_for_rows,
                       (long long)max_rows, q, scale);
    return hipGetLastError();
}

hipError_t launch_requant_fp8(const float *y, int64_t max_rows, int I, const int32_t *sched_for_rows, uint8_t *q,
                              uint8_t *scale, hipStream_t stream)
{
    if (max_rows <= 0) {
        return hipSuccess;
    }
    if (I % 128 != 0) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(requant_fp8_kernel, dim3((unsigned)max_rows), dim3(256), 0, stream, y, I, sched_for_rows,
                       (long long)max_rows, q, scale);
    return hipGetLastError();
}

hipError_t launch_prepack(const int8_t *src, int8_t *dst, int G, int Kd, int N, int gate_up, hipStream_t stream)
{
    if (Kd % kBK != 0 || N % 64 != 0 || (gate_up && N % 128 != 0)) {
        return hipErrorInvalidValue;
    }
    const long long pieces = (long long)Kd * N / 16;
    dim3 grid((unsigned)((pieces + 255) / 256), (unsigned)G);
    hipLaunchKernelGGL(prepack_kernel, grid, dim3(256), 0, stream, src, dst, Kd, N, gate_up, pieces);
    return hipGetLastError();
}

}  // namespace cam
