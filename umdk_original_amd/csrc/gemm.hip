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
//   * One workgroup = 4 waves = a tile of up to 128 rows of ONE expert x 256 packed weight columns.
//     Every wave covers all rows of the tile and its own 64 columns (128 int32 accumulators per lane),
//     and two workgroups share a CU so that one runs MFMAs while the other waits on memory or
//     writes its epilogue.  The grouped shape is bound by streaming the weights: a tall tile makes
//     every weight byte fetched feed up to 128 rows, and sibling tiles of one expert are scheduled
//     next to each other so that they find the same weight panel in L2.
//   * Both operands travel global -> LDS with direct-to-LDS loads (16 bytes per lane, no registers),
//     three stages deep, two 64-deep K steps ahead of the MFMAs.  Weights were laid out once by the
//     prepack kernel in the lane order the MFMA wants, so a wave's weight load is 1 KB of contiguous
//     memory that lands in LDS already in fragment order.  Activation rows are placed with an XOR
//     swizzle of their 16-byte chunks (chosen on the global side, since a direct-to-LDS load writes
//     lane i at base + 16*i), which makes the ds_read_b128 fragment reads bank-conflict free.
//   * The loads are issued from inline assembly and the pipeline's waits are written out by hand.
//     Left to itself the compiler drains every outstanding load at each workgroup barrier and before
//     LDS reads it cannot prove independent, which serialises the pipeline.
//   * The int32 accumulators stay in registers through the epilogue: dequantisation, SiLU and the
//     gate*up product are applied in place; the int32 tile never goes to memory.  The MFMAs take the
//     weights as their first operand, so a lane ends up with ONE activation row and runs of four
//     consecutive weight columns: one row scale per lane, column scales as 16-byte vectors, 8- or
//     16-byte pieces into the LDS staging from which whole 128-byte lines are stored.
//     For GMM1 the prepack pairs gate column c with up column I+c inside one wave.
//   * Variable rows per expert: a device-built tile table lists, per tile, (expert, first row, rows,
//     first tile of the expert, tiles of the expert); an expert's rows are split evenly over its
//     tiles and empty experts own no tile.  The grid is sized for the worst case and surplus
//     workgroups exit at once.  Work ids are dealt to the 8 XCDs in contiguous runs, tile index
//     fastest inside an expert, so that the workgroups reading one weight panel run together on one
//     XCD and share its L2; all workgroups of an expert start their K loop at the same step (which
//     differs from expert to expert), so that they also find each other's activation rows there.
//   * The K order inside a 32-deep MFMA step is whatever the two operands agree on (an integer dot
//     product does not care), which is what lets both be loaded as plain 16-byte pieces.
#include "cam_device.h"
#include "cam_kernels.h"
#include "../../include/cam_expf_spec.h"

namespace cam {

namespace {

constexpr int kBM = kGemmTileM;  // rows per tile
constexpr int kNF = 2;           // 2 column fragments per wave (64 columns)
constexpr int kBK = 64;          // K bytes per pipeline step
constexpr int kKK = kBK / 32;    // MFMA sub-steps per step
constexpr int kThreads = 256;
constexpr int kWaveCols = 64;
constexpr int kBlockCols = 4 * kWaveCols;
constexpr int kNumXcd = 8;
constexpr int kStages = 3;
constexpr int kStageA = kBM * kBK;                    // 8 KB of activations per stage
constexpr int kStageB = 4 * kWaveCols * kBK;          // 16 KB of weights per stage (4 KB per wave)
constexpr int kStageBytes = kStageA + kStageB;
constexpr int kBLoads = kKK * kNF;                    // weight loads per wave and step
constexpr int kEpiRowBytes = 144;                     // epilogue staging: 128 data bytes + 16 of padding per row
constexpr int kLdsBytes = kStages * kStageBytes > 4 * kBM * kEpiRowBytes ? kStages * kStageBytes
                                                                         : 4 * kBM * kEpiRowBytes;

// LDS offset (bytes) inside a stage of the 16-byte chunk `c` (0..3) of activation row `r`.
__device__ __forceinline__ int a_lds_offset(int r, int c)
{
    return r * kBK + ((c ^ ((r >> 2) & 3)) << 4);
}

// One direct-to-LDS load: lane i of the wave fetches 16 bytes at its own global address `g` and the
// data lands at LDS byte address lds_base + 16*i.
__device__ __forceinline__ void dma16(const void *g, unsigned lds_base)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g)
                 : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_loads_outstanding()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Workgroup barrier without the memory fence of __syncthreads(); the waits are explicit (above).
__device__ __forceinline__ void barrier_no_fence()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

struct TileCtx {
    const int8_t *a_tile;   // first activation row of the tile
    const int8_t *wp;       // this wave's weight stream (+ 16 * lane)
    const float *sg;        // this expert's per-channel scales
    int m0, rows, nw, Kd, N;
    int k_start;            // first K step of this workgroup (the K loop wraps around)
    bool wave_live;
};

// The whole tile for a compile-time number of 32-row fragments, so that the main loop is branch-free.
template <int EPI, int MF>
__device__ __forceinline__ void gemm_tile(const GemmArgs &a, const TileCtx &t, int8_t *lds, const float *row_scale_s)
{
    constexpr int AI = (MF + 1) / 2;           // activation loads per wave and step (1 KB each)
    constexpr int PER_STEP = AI + kBLoads;     // loads per wave and step
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KT = t.Kd / kBK;
    const int last = KT - 1;
    const unsigned lds0 = (unsigned)(unsigned long long)(__attribute__((address_space(3))) int8_t *)lds;

    v16i acc[MF][kNF];
#pragma unroll
    for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
        for (int nf = 0; nf < kNF; ++nf) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                acc[mf][nf][i] = 0;
            }
        }
    }

    // Per-lane source addresses of the activation loads (they advance by kBK per step).
    // Load j of wave w fills the 64-byte LDS rows 16q .. 16q+15 with q = 4j + w (q = w & 1 for a
    // single-fragment tile, where waves 2 and 3 repeat the loads of waves 0 and 1); lane i brings row
    // 16q + i/4, and the chunk whose swizzled slot is i%4.  Rows inside the last fragment but beyond
    // the tile repeat its last row (their results are dropped in the epilogue).
    const int8_t *a_src[AI];
    unsigned a_dst[AI];
#pragma unroll
    for (int j = 0; j < AI; ++j) {
        const int q = MF >= 2 ? j * 4 + wave : (wave & 1);  // MF == 3: loads 6, 7 bring rows of a fourth, unused fragment
        const int r = 16 * q + (lane >> 2);
        const int c = (lane & 3) ^ ((r >> 2) & 3);
        a_src[j] = t.a_tile + (long long)min(r, t.rows - 1) * t.Kd + c * 16;
        a_dst[j] = (unsigned)(q * 1024);
    }
    const unsigned b_dst = (unsigned)(kStageA + wave * (kWaveCols * kBK));

    // Step s of the pipeline reads K step (k_start + s) mod KT: an integer dot product does not care
    // about the order, and workgroups that start at different depths do not all pull on the same
    // memory channels at the same moment (their weight streams lie a fixed stride apart).
    // Issues the loads of pipeline step s_idx whose index i (activation loads first, then the weight
    // loads) satisfies i % nparts == part.
    auto issue_part = [&](int s_idx, int stage, int part, int nparts) {
        int step = t.k_start + s_idx;
        step = step >= KT ? step - KT : step;
        const unsigned sbase = lds0 + (unsigned)(stage * kStageBytes);
#pragma unroll
        for (int j = 0; j < AI; ++j) {
            if (j % nparts == part) {
                dma16(a_src[j] + (long long)step * kBK, sbase + a_dst[j]);
            }
        }
        const int8_t *bp = t.wp + (long long)step * (kBLoads * kWave * 16);
#pragma unroll
        for (int i = 0; i < kBLoads; ++i) {
            if ((AI + i) % nparts == part) {
                dma16(bp + i * (kWave * 16), sbase + b_dst + (unsigned)(i * 1024));
            }
        }
    };
    auto issue = [&](int s_idx, int stage) { issue_part(s_idx, stage, 0, 1); };

    const int a_row = lane & 31;
    const int a_half = lane >> 5;
    constexpr int HF = MF == 4 ? 2 : MF;        // fragments per half
    constexpr int NH = MF / HF;                 // halves per sub-step

    // Multiplies one stage.  Fragment reads run one half sub-step ahead of the MFMAs that use them.
    // The loads of the step two ahead are issued from inside the phases, a few at a time between the
    // MFMA groups: a wave that issued them all at once would sit at the memory pipe's input while it
    // drains, with its MFMAs waiting behind the loads in program order.
    auto compute = [&](const int8_t *stage, int next_idx, int next_stage) {
        const int8_t *sa = stage;
        const int8_t *sb = stage + kStageA + wave * (kWaveCols * kBK) + lane * 16;
        v4i af[2][HF];
        v4i bf[kKK][kNF];
        auto load_frags = [&](v4i *dst, int kk, int half) {
#pragma unroll
            for (int f = 0; f < HF; ++f) {
                dst[f] = *(const v4i *)(sa + a_lds_offset((half * HF + f) * 32 + a_row, kk * 2 + a_half));
            }
        };
#pragma unroll
        for (int kk = 0; kk < kKK; ++kk) {
#pragma unroll
            for (int nf = 0; nf < kNF; ++nf) {
                bf[kk][nf] = *(const v4i *)(sb + (kk * kNF + nf) * 1024);
            }
        }
        load_frags(af[0], 0, 0);
#pragma unroll
        for (int q = 0; q < kKK * NH; ++q) {
            const int kk = q / NH;
            const int half = q % NH;
            if (q + 1 < kKK * NH) {
                load_frags(af[(q + 1) & 1], (q + 1) / NH, (q + 1) % NH);
            }
            // Keep the LDS reads of the next half ahead of this half's MFMAs: the scheduler would
            // otherwise sink them to just before their first use and expose the LDS latency.
            __builtin_amdgcn_sched_barrier(0);
            issue_part(next_idx, next_stage, q, kKK * NH);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int f = 0; f < HF; ++f) {
#pragma unroll
                for (int nf = 0; nf < kNF; ++nf) {
                    // Weights as the first operand: the result tile comes out transposed, i.e. a lane
                    // holds ONE activation row and 4 consecutive weight columns per register quad.
                    acc[half * HF + f][nf] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[kk][nf], af[q & 1][f],
                                                                                   acc[half * HF + f][nf], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Pipeline.  Every step issues exactly PER_STEP loads per wave and loads retire in order, so "at
    // most (kStages-2)*PER_STEP outstanding" means that this wave's part of the current step has
    // landed; the barrier then makes every wave's part visible and also guarantees that all waves
    // are done reading the previous stage, which the loads issued next overwrite.  Step indices past
    // the end are clamped (the last step is fetched again), so the loop body has no control flow.
#pragma unroll
    for (int p = 0; p < kStages - 1; ++p) {
        issue(min(p, last), p);
    }
    for (int kt = 0; kt < KT; ++kt) {
        wait_loads_outstanding<(kStages - 2) * PER_STEP>();
        barrier_no_fence();
        compute(lds + (kt % kStages) * kStageBytes, min(kt + kStages - 1, last), (kt + kStages - 1) % kStages);
    }
    wait_loads_outstanding<0>();

    // ---- epilogue, accumulators in registers.
    // Lane l holds activation row (l & 31) of each 32x32 fragment; registers 4j .. 4j+3 hold the four
    // consecutive weight columns 8j + 4*(l/32) + 0..3.  Dequantisation runs on that layout with one
    // row scale per lane and fragment and the column scales fetched as 16-byte vectors.  To store
    // whole 128-byte lines, every wave passes its results through its own slice of LDS (the pipeline
    // stages are free by now): 128 staged bytes per row, then 16 bytes per lane and 8 rows per store.
    barrier_no_fence();  // all waves are done with the pipeline stages
    if (!t.wave_live) {
        return;
    }
    const int rows = t.rows;
    const int m0 = t.m0;
    const int N = t.N;
    const int nw = t.nw;
    const int row_in = lane & 31;
    const int col_half = (lane >> 5) * 4;
    int8_t *slice = lds + wave * (kBM * kEpiRowBytes);

    // Copies the wave's staged rows (128 bytes each) to `dst` + row * row_pitch_bytes.
    auto flush_rows = [&](int8_t *dst, long long row_pitch_bytes) {
        const int sub = lane >> 3;    // row inside a group of 8
        const int piece = lane & 7;   // 16-byte piece of the 128-byte row
#pragma unroll
        for (int it = 0; it < MF * 4; ++it) {
            const int row = it * 8 + sub;
            const v4u v = *(const v4u *)(slice + row * kEpiRowBytes + piece * 16);
            if (row < rows) {
                *(v4u *)(dst + (long long)(m0 + row) * row_pitch_bytes + piece * 16) = v;
            }
        }
    };

    if (EPI == kEpiInt32) {
#pragma unroll
        for (int nf = 0; nf < kNF; ++nf) {
            const int col0 = a.gate_up ? (nf * (N / 2) + nw * 32) : (nw * kWaveCols + nf * 32);
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const v4i v = {acc[mf][nf][4 * j], acc[mf][nf][4 * j + 1], acc[mf][nf][4 * j + 2],
                                   acc[mf][nf][4 * j + 3]};
                    *(v4i *)(slice + (mf * 32 + row_in) * kEpiRowBytes + (8 * j + col_half) * 4) = v;
                }
            }
            flush_rows((int8_t *)a.out + (long long)col0 * 4, (long long)N * 4);
        }
    } else if (EPI == kEpiSwiglu) {
        // t = (float(C) * w_scale[n]) * x_scale[m]; y = silu(t_gate) * t_up
        const int I = N / 2;
        v4f sg_gate[4], sg_up[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sg_gate[j] = *(const v4f *)(t.sg + nw * 32 + 8 * j + col_half);
            sg_up[j] = *(const v4f *)(t.sg + I + nw * 32 + 8 * j + col_half);
        }
#pragma unroll
        for (int mf = 0; mf < MF; ++mf) {
            const float xs = row_scale_s[mf * 32 + row_in];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v4f y;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float tg = __fmul_rn(__fmul_rn((float)acc[mf][0][4 * j + e], sg_gate[j][e]), xs);
                    const float tu = __fmul_rn(__fmul_rn((float)acc[mf][1][4 * j + e], sg_up[j][e]), xs);
                    y[e] = __fmul_rn(cam_silu_spec(tg), tu);
                }
                *(v4f *)(slice + (mf * 32 + row_in) * kEpiRowBytes + (8 * j + col_half) * 4) = y;
            }
        }
        flush_rows((int8_t *)a.out + (long long)(nw * 32) * 4, (long long)I * 4);
    } else {
#pragma unroll
        for (int nf = 0; nf < kNF; ++nf) {
            v4f ws[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                ws[j] = *(const v4f *)(t.sg + nw * kWaveCols + nf * 32 + 8 * j + col_half);
            }
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
                const float xs = row_scale_s[mf * 32 + row_in];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t b[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        b[e] = f32_to_bf16_bits(__fmul_rn(__fmul_rn((float)acc[mf][nf][4 * j + e], ws[j][e]), xs));
                    }
                    const v2u v = {b[0] | (b[1] << 16), b[2] | (b[3] << 16)};
                    *(v2u *)(slice + (mf * 32 + row_in) * kEpiRowBytes + (nf * 32 + 8 * j + col_half) * 2) = v;
                }
            }
        }
        flush_rows((int8_t *)a.out + (long long)(nw * kWaveCols) * 2, (long long)N * 2);
    }
}

template <int EPI>
__global__ __launch_bounds__(kThreads, 2) void gemm_kernel(GemmArgs a)
{
    __shared__ __attribute__((aligned(1024))) int8_t lds[kLdsBytes];
    __shared__ float row_scale_s[kBM];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;

    // ---- which tile, which column block.
    // Each XCD takes one contiguous run of work ids (workgroup i runs on XCD i % 8).  Inside an expert
    // with n tiles the ids run: a group of column blocks, and inside the group the column block, and
    // inside the column block the expert's n tiles.  The workgroups that are resident together on an
    // XCD (64) then are all the row tiles of an expert for a few column blocks: they stream the same
    // weight panels at the same depth and find each other's lines in L2, so a panel is fetched once.
    const int num_tiles = min(a.tiles[0], a.max_tiles);
    const int nblocks = (a.N + kBlockCols - 1) / kBlockCols;
    const long long total_work = (long long)num_tiles * nblocks;
    const long long chunk = (total_work + kNumXcd - 1) / kNumXcd;
    const long long slot = blockIdx.x / kNumXcd;
    const long long wid = (long long)(blockIdx.x % kNumXcd) * chunk + slot;
    if (slot >= chunk || wid >= total_work) {
        return;
    }
    const int32_t *probe = a.tiles + kTileHeader + kTileRecord * (int)(wid / nblocks);
    const int first = probe[3];
    const int ntile = max(probe[4], 1);
    const int local = (int)(wid - (long long)first * nblocks);  // id inside the expert
    const int tile = first + local % ntile;
    const int nb = local / ntile;
    const int32_t *te = a.tiles + kTileHeader + kTileRecord * tile;
    const int g = te[0];
    TileCtx t;
    t.m0 = te[1];
    t.rows = te[2];
    if (t.rows <= 0) {
        return;
    }
    t.Kd = a.Kd;
    t.N = a.N;
    t.nw = nb * 4 + wave;  // this wave's 64-column group
    t.wave_live = t.nw * kWaveCols < t.N;
    const int8_t *wg = a.per_expert ? a.list.w[g] : a.w + (long long)g * t.Kd * t.N;
    t.sg = a.per_expert ? a.list.s[g] : a.w_scale + (long long)g * t.N;
    t.wp = wg + (long long)(t.wave_live ? t.nw : 0) * t.Kd * kWaveCols + lane * 16;
    t.a_tile = a.a + (long long)t.m0 * t.Kd;
    // The start depth depends on the expert only, so that all workgroups of an expert, which share
    // activation rows or weight panels, stay in step and find each other's lines in L2.
    t.k_start = (int)(((long long)g * 37) % (t.Kd / kBK));

    if (EPI != kEpiInt32) {
        for (int r = tid; r < kBM; r += kThreads) {
            row_scale_s[r] = a.a_scale[t.m0 + min(r, t.rows - 1)];
        }
    }

    const int mfrags = (t.rows + 31) >> 5;
    if (mfrags <= 1) {
        gemm_tile<EPI, 1>(a, t, lds, row_scale_s);
    } else if (mfrags <= 2) {
        gemm_tile<EPI, 2>(a, t, lds, row_scale_s);
    } else if (mfrags <= 3) {
        gemm_tile<EPI, 3>(a, t, lds, row_scale_s);
    } else {
        gemm_tile<EPI, 4>(a, t, lds, row_scale_s);
    }
}

// SwiGLU product rows (fp32) -> int8 rows + per-row scale:
//   m = max|y|; y_scale = m * (1/127); q = rint((y * 127) * (1/m)).   One workgroup per row.
__global__ __launch_bounds__(256) void requant_kernel(const float *__restrict__ y, int I,
                                                      const int32_t *__restrict__ tiles, long long max_rows,
                                                      int8_t *__restrict__ q, float *__restrict__ scale)
{
    __shared__ float wave_max_s[4];
    const long long row = blockIdx.x;
    const long long valid = tiles != nullptr ? min((long long)tiles[1], max_rows) : max_rows;
    if (row >= valid) {
        return;
    }
    const int tid = threadIdx.x;
    const int n4 = I >> 2;
    constexpr int kMaxPer = 4;  // I <= 4096
    v4f v[kMaxPer];
    float m = 0.0f;
    const v4f *src = (const v4f *)(y + row * I);
#pragma unroll
    for (int j = 0; j < kMaxPer; ++j) {
        const int c = tid + j * 256;
        v[j] = v4f{0.f, 0.f, 0.f, 0.f};
        if (c < n4) {
            v[j] = __builtin_nontemporal_load(src + c);
            m = fmaxf(m, fmaxf(fmaxf(fabsf(v[j][0]), fabsf(v[j][1])), fmaxf(fabsf(v[j][2]), fabsf(v[j][3]))));
        }
    }
    m = wave_max(m);
    if ((tid & 63) == 0) {
        wave_max_s[tid >> 6] = m;
    }
    __syncthreads();
    m = fmaxf(fmaxf(wave_max_s[0], wave_max_s[1]), fmaxf(wave_max_s[2], wave_max_s[3]));
    const bool zero_row = m == 0.0f;
    const float rcp = zero_row ? 0.0f : __fdiv_rn(1.0f, m);
    if (tid == 0) {
        scale[row] = zero_row ? 0.0f : __fmul_rn(m, 1.0f / 127.0f);
    }
    uint32_t *dst = (uint32_t *)(q + row * I);
#pragma unroll
    for (int j = 0; j < kMaxPer; ++j) {
        const int c = tid + j * 256;
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

// Row-major [G,Kd,N] int8 -> MFMA operand order.  One thread writes one 16-byte piece:
//   piece index = (((g*NW + nw)*KS + ks)*2 + nf)*64 + lane, holding K rows ks*32 + (lane/32)*16 + 0..15 of
//   logical column  gate_up ? nf*(N/2) + nw*32 + lane%32 : nw*64 + nf*32 + lane%32.
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
    *((v4u *)(dst + (long long)g * Kd * N) + p) = o;
}

}  // namespace

hipError_t launch_gemm(const GemmArgs &a, hipStream_t stream)
{
    if (a.max_tiles <= 0) {
        return hipSuccess;
    }
    if (a.Kd % 128 != 0 || a.N % kWaveCols != 0 || (a.gate_up && a.N % (2 * kWaveCols) != 0)) {
        return hipErrorInvalidValue;
    }
    const int nblocks = (a.N + kBlockCols - 1) / kBlockCols;
    long long work = (long long)a.max_tiles * nblocks;
    work = (work + kNumXcd - 1) / kNumXcd * kNumXcd;
    if (work > 0x7fffffffll) {
        return hipErrorInvalidValue;
    }
    dim3 grid((unsigned)work), block(kThreads);
    switch (a.epilogue) {
        case kEpiInt32:
            hipLaunchKernelGGL(gemm_kernel<kEpiInt32>, grid, block, 0, stream, a);
            break;
        case kEpiSwiglu:
            hipLaunchKernelGGL(gemm_kernel<kEpiSwiglu>, grid, block, 0, stream, a);
            break;
        case kEpiDequantBf16:
            hipLaunchKernelGGL(gemm_kernel<kEpiDequantBf16>, grid, block, 0, stream, a);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_requant(const float *y, int64_t max_rows, int I, const int32_t *tiles_for_rows, int8_t *q,
                          float *scale, hipStream_t stream)
{
    if (max_rows <= 0) {
        return hipSuccess;
    }
    if (I % 4 != 0 || I > 4096) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(requant_kernel, dim3((unsigned)max_rows), dim3(256), 0, stream, y, I, tiles_for_rows,
                       (long long)max_rows, q, scale);
    return hipGetLastError();
}

hipError_t launch_prepack(const int8_t *src, int8_t *dst, int G, int Kd, int N, int gate_up, hipStream_t stream)
{
    if (Kd % kBK != 0 || N % kWaveCols != 0 || (gate_up && N % (2 * kWaveCols) != 0)) {
        return hipErrorInvalidValue;
    }
    const long long pieces = (long long)Kd * N / 16;
    dim3 grid((unsigned)((pieces + 255) / 256), (unsigned)G);
    hipLaunchKernelGGL(prepack_kernel, grid, dim3(256), 0, stream, src, dst, Kd, N, gate_up, pieces);
    return hipGetLastError();
}

}  // namespace cam
