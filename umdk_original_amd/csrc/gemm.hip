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
//   * One workgroup = 4 waves = a tile of up to 256 rows of ONE expert x 256 packed weight columns.
//     Every wave covers all rows of the tile and its own 64 columns, so a weight byte is needed by
//     exactly one wave: weights go straight from HBM to registers in the lane order the MFMA wants
//     (they were laid out that way once by the prepack kernel), 16 bytes per lane, 1 KB contiguous
//     per wave and load, through a register ring two 128-deep K steps ahead.  No LDS for weights.
//     The grouped shape is bound by streaming the weights, so the tile is as tall as the register
//     file allows (256 int32 accumulators per lane): every weight byte fetched feeds up to 256 rows.
//   * Activations (shared by the 4 waves) are staged through LDS, double-buffered, with an XOR
//     swizzle of the 16-byte chunks so that both the cooperative stores and the ds_read_b128
//     fragment loads are bank-conflict free.
//   * The int32 accumulators stay in registers through the epilogue: dequantisation, SiLU and the
//     gate*up product are applied in place; the int32 tile never goes to memory.
//     For GMM1 the prepack pairs gate column c with up column I+c inside one wave.
//   * Variable rows per expert: a device-built tile table lists (expert, first row, rows); empty
//     experts own no tile.  The grid is sized for the worst case and surplus workgroups exit at once.
//     Work ids are dealt to the 8 XCDs in contiguous runs so that workgroups sharing activation rows
//     (same tile, neighbouring column blocks) run on one XCD and share its L2.
//   * The K order inside a 32-deep MFMA step is whatever the two operands agree on (an integer dot
//     product does not care), which is what lets both be loaded as plain 16-byte pieces.
#include "cam_device.h"
#include "cam_kernels.h"
#include "../../include/cam_expf_spec.h"

namespace cam {

namespace {

constexpr int kBM = kGemmTileM;  // rows per tile
constexpr int kMF = kBM / 32;    // row fragments per tile
constexpr int kNF = 2;           // 2 column fragments per wave (64 columns)
constexpr int kBK = 128;         // K bytes per main-loop step
constexpr int kKK = kBK / 32;    // MFMA steps per main-loop step
constexpr int kThreads = 256;
constexpr int kWaveCols = 64;
constexpr int kBlockCols = 4 * kWaveCols;
constexpr int kNumXcd = 8;
constexpr int kBDepth = 3;       // weight register ring: steps in flight

// LDS offset (bytes) of the 16-byte chunk `c` (0..7) of row `r` in one A stage.
__device__ __forceinline__ int a_lds_offset(int r, int c)
{
    return r * kBK + ((c ^ ((r >> 1) & 7)) << 4);
}

struct BRegs {
    v4i v[kKK][kNF];
};

__device__ __forceinline__ void load_b(BRegs &b, const v4i *__restrict__ wp, int kt)
{
    // wave-contiguous: [(kt*4 + kk)*2 + nf][lane] 16-byte pieces
    const v4i *p = wp + (long long)kt * (kKK * kNF * kWave);
#pragma unroll
    for (int kk = 0; kk < kKK; ++kk) {
#pragma unroll
        for (int nf = 0; nf < kNF; ++nf) {
            b.v[kk][nf] = p[(kk * kNF + nf) * kWave];
        }
    }
}

// Activation loads of one step for a tile of MF 32-row fragments: MF 16-byte loads per thread.
// Rows inside the last fragment but beyond the tile repeat its last row (their results are dropped in
// the epilogue).
template <int MF>
struct ARegs {
    v4i v[MF];
};

template <int MF>
__device__ __forceinline__ void load_a(ARegs<MF> &r, const int8_t *__restrict__ a_tile, int Kd, int rows, int kt,
                                       int tid)
{
    const int c = tid & 7;
#pragma unroll
    for (int i = 0; i < MF; ++i) {
        const int row = min((tid >> 3) + 32 * i, rows - 1);
        r.v[i] = *(const v4i *)(a_tile + (long long)row * Kd + kt * kBK + c * 16);
    }
}

template <int MF>
__device__ __forceinline__ void store_a(const ARegs<MF> &r, int8_t *stage, int tid)
{
    const int c = tid & 7;
#pragma unroll
    for (int i = 0; i < MF; ++i) {
        const int row = (tid >> 3) + 32 * i;
        *(v4i *)(stage + a_lds_offset(row, c)) = r.v[i];
    }
}

struct TileCtx {
    const int8_t *a_tile;   // first activation row of the tile
    const v4i *wp;          // this wave's weight stream (+ lane)
    const float *sg;        // this expert's per-channel scales
    int m0, rows, nw, Kd, N;
    bool wave_live;
};

// The whole tile for a compile-time number of row fragments, so that the main loop is branch-free.
template <int EPI, int MF>
__device__ __forceinline__ void gemm_tile(const GemmArgs &a, const TileCtx &t, int8_t (*a_s)[kBM * kBK],
                                          const float *row_scale_s)
{
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int KT = t.Kd / kBK;

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

    // Software pipeline: weights for steps kt+1 and kt+2 are in flight (register ring of three steps)
    // while step kt is multiplied; activations for step kt+1 travel global -> registers -> LDS.
    // Every load in the loop is unconditional (step indices are clamped to the last step, which is
    // then simply fetched again), so the loop body has no control flow and nothing forces a wait on
    // a load before its data is needed.
    BRegs bring[kBDepth];
    ARegs<MF> ar;
    const int last = KT - 1;
    load_b(bring[0], t.wp, 0);
    load_a<MF>(ar, t.a_tile, t.Kd, t.rows, 0, tid);
    load_b(bring[1], t.wp, min(1, last));
    store_a<MF>(ar, a_s[0], tid);
    __syncthreads();

    const int a_row = lane & 31;
    const int a_half = lane >> 5;

    // A fragments are double-buffered in registers across the four MFMA sub-steps of a step.
    auto load_frags = [&](v4i *af, const int8_t *stage, int kk) {
#pragma unroll
        for (int mf = 0; mf < MF; ++mf) {
            af[mf] = *(const v4i *)(stage + a_lds_offset(mf * 32 + a_row, kk * 2 + a_half));
        }
    };
    auto compute = [&](const int8_t *stage, const BRegs &b) {
        v4i af[2][MF];
        load_frags(af[0], stage, 0);
#pragma unroll
        for (int kk = 0; kk < kKK; ++kk) {
            if (kk + 1 < kKK) {
                load_frags(af[(kk + 1) & 1], stage, kk + 1);
            }
            // Keep the LDS reads of the next sub-step ahead of this sub-step's MFMAs: the scheduler
            // would otherwise sink them to just before their first use and expose the LDS latency.
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                for (int nf = 0; nf < kNF; ++nf) {
                    acc[mf][nf] =
                        __builtin_amdgcn_mfma_i32_32x32x32_i8(af[kk & 1][mf], b.v[kk][nf], acc[mf][nf], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // One step with static ring indices: fetch step KT_+2 into ring[(CUR+2)%3], multiply ring[CUR].
#define CAM_GEMM_STEP(CUR, KT_)                                               \
    {                                                                         \
        const int kt_ = (KT_);                                                \
        load_b(bring[((CUR) + 2) % kBDepth], t.wp, min(kt_ + 2, last));       \
        load_a<MF>(ar, t.a_tile, t.Kd, t.rows, min(kt_ + 1, last), tid);      \
        compute(a_s[kt_ & 1], bring[(CUR)]);                                  \
        store_a<MF>(ar, a_s[(kt_ + 1) & 1], tid);                             \
        __syncthreads();                                                      \
    }

    int kt = 0;
    for (; kt + kBDepth <= KT; kt += kBDepth) {
        CAM_GEMM_STEP(0, kt)
        CAM_GEMM_STEP(1, kt + 1)
        CAM_GEMM_STEP(2, kt + 2)
    }
    if (kt < KT) {
        CAM_GEMM_STEP(0, kt)
    }
    if (kt + 1 < KT) {
        CAM_GEMM_STEP(1, kt + 1)
    }
#undef CAM_GEMM_STEP

    if (!t.wave_live) {
        return;
    }

    // ---- epilogue, accumulators in registers.
    // Lane l holds column (l & 31) of each 32x32 fragment; register i holds row 8*(i/4) + 4*(l/32) + i%4.
    const int rows = t.rows;
    const int m0 = t.m0;
    const int N = t.N;
    const int nw = t.nw;
    const int col_in = lane & 31;
    const int row_half = (lane >> 5) * 4;
    if (EPI == kEpiInt32) {
        int32_t *out = (int32_t *)a.out;
#pragma unroll
        for (int nf = 0; nf < kNF; ++nf) {
            const int col = a.gate_up ? (nf * (N / 2) + nw * 32 + col_in) : (nw * kWaveCols + nf * 32 + col_in);
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = mf * 32 + 8 * (i >> 2) + row_half + (i & 3);
                    if (row < rows) {
                        out[(long long)(m0 + row) * N + col] = acc[mf][nf][i];
                    }
                }
            }
        }
    } else if (EPI == kEpiSwiglu) {
        // t = (float(C) * w_scale[n]) * x_scale[m]; y = silu(t_gate) * t_up
        float *out = (float *)a.out;
        const int I = N / 2;
        const int c = nw * 32 + col_in;
        const float sg_gate = t.sg[c];
        const float sg_up = t.sg[I + c];
#pragma unroll
        for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = mf * 32 + 8 * (i >> 2) + row_half + (i & 3);
                if (row < rows) {
                    const float xs = row_scale_s[row];
                    const float tg = __fmul_rn(__fmul_rn((float)acc[mf][0][i], sg_gate), xs);
                    const float tu = __fmul_rn(__fmul_rn((float)acc[mf][1][i], sg_up), xs);
                    out[(long long)(m0 + row) * I + c] = __fmul_rn(cam_silu_spec(tg), tu);
                }
            }
        }
    } else {
        uint16_t *out = (uint16_t *)a.out;
#pragma unroll
        for (int nf = 0; nf < kNF; ++nf) {
            const int col = nw * kWaveCols + nf * 32 + col_in;
            const float ws = t.sg[col];
#pragma unroll
            for (int mf = 0; mf < MF; ++mf) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = mf * 32 + 8 * (i >> 2) + row_half + (i & 3);
                    if (row < rows) {
                        const float v = __fmul_rn(__fmul_rn((float)acc[mf][nf][i], ws), row_scale_s[row]);
                        out[(long long)(m0 + row) * N + col] = (uint16_t)f32_to_bf16_bits(v);
                    }
                }
            }
        }
    }
}

template <int EPI>
__global__ __launch_bounds__(kThreads, 1) void gemm_kernel(GemmArgs a)
{
    __shared__ __attribute__((aligned(16))) int8_t a_s[2][kBM * kBK];
    __shared__ float row_scale_s[kBM];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid >> 6;

    // ---- which tile, which column block.  Work ids run (tile, column block) with the column block
    // fastest; each XCD takes one contiguous run of ids, so the workgroups that share a tile's
    // activation rows, and neighbouring tiles of one expert that share weight panels, meet in one L2.
    const int num_tiles = min(a.tiles[0], a.max_tiles);
    const int nblocks = (a.N + kBlockCols - 1) / kBlockCols;
    const long long total_work = (long long)num_tiles * nblocks;
    const long long chunk = (total_work + kNumXcd - 1) / kNumXcd;
    const long long slot = blockIdx.x / kNumXcd;
    const long long wid = (long long)(blockIdx.x % kNumXcd) * chunk + slot;
    if (slot >= chunk || wid >= total_work) {
        return;
    }
    const int tile = (int)(wid / nblocks);
    const int nb = (int)(wid - (long long)tile * nblocks);
    const int32_t *te = a.tiles + 4 + 4 * tile;
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
    t.wp = (const v4i *)(wg + (long long)(t.wave_live ? t.nw : 0) * t.Kd * kWaveCols) + lane;
    t.a_tile = a.a + (long long)t.m0 * t.Kd;

    if (EPI != kEpiInt32) {
        for (int r = tid; r < kBM; r += kThreads) {
            row_scale_s[r] = a.a_scale[t.m0 + min(r, t.rows - 1)];
        }
    }

    const int mfrags = (t.rows + 31) >> 5;
    if (mfrags <= 1) {
        gemm_tile<EPI, 1>(a, t, a_s, row_scale_s);
    } else if (mfrags <= 2) {
        gemm_tile<EPI, 2>(a, t, a_s, row_scale_s);
    } else if (mfrags <= 4) {
        gemm_tile<EPI, 4>(a, t, a_s, row_scale_s);
    } else {
        gemm_tile<EPI, 8>(a, t, a_s, row_scale_s);
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
    if (a.Kd % kBK != 0 || a.N % kWaveCols != 0 || (a.gate_up && a.N % (2 * kWaveCols) != 0)) {
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
