// Weighted un-permute and reduce back to token order (bandwidth-bound gather).
//
// Reference semantics (paths relative to the reference tree):
//   src/cam/comm_operator/ascend_kernels/moe_combine_normal/op_kernel/moe_combine_normal.h:303-338
//   src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/raw_distributed/
//   cam_moe_distribute_combine.h:726-780
// acc = 0 (fp32); for k ascending, skipping absent slots: acc = acc + (float(row) * w[t,k]) with the
// multiply and the add rounded separately; out = bf16 round-to-nearest-even of acc.
//
// Design.  The reference scatters every row into a per-(token,k) window slot and then reads the slots
// back; here the rows are gathered straight from the expert-major buffer.  A workgroup of 128
// threads owns 1024 contiguous columns of one token, so row indices and weights are uniform across
// the workgroup; each thread issues up to eight independent 16-byte row loads before it starts the
// ordered accumulation, then stores 16 bytes of bf16.  Every row byte is read exactly once.
//
// Rows quantised for the wire (src/cam/comm_operator/ascend_kernels/moe_combine_shmem/op_kernel/
// moe_combine_shmem.h, IsQuant): a row is H int8 values followed by H/8 bf16 scales, one per block of 8 columns.
//   quantise (:567-592):   m = max |x| over the block; s = m * (1/127); stored scale = bf16(s);
//                          q = int8_rne(fp16_rne(x / s)), with the unrounded s.
//   dequantise (:755-773): v = bf16_rne(float(q) * float(stored scale)), then the weighted sum as above.
// A thread of the gather owns exactly one block of 8 columns, so it reads 8 + 2 bytes per row instead of 16.
#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

namespace {

constexpr int kCombThreads = 128;
constexpr int kCombBatch = 8;

// Rows at or beyond *row_limit (the receive total, epRecvCounts[E-1] of moe_combine_normal.h:206-207) were
// never written by the dispatch that filled the buffers; whatever triple they hold is ignored.
__global__ void invert_src_info_kernel(const int32_t *src_info, long long A, const int32_t *row_limit, int T, int K,
                                       int32_t *slot_row)
{
    long long r = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (row_limit != nullptr) {
        A = min(A, (long long)*row_limit);
    }
    if (r >= A) {
        return;
    }
    int t = src_info[3 * r + 1];
    int k = src_info[3 * r + 2];
    if (t >= 0 && t < T && k >= 0 && k < K) {
        slot_row[(long long)t * K + k] = (int32_t)r;
    }
}

__global__ void rows_from_counts_kernel(const int32_t *__restrict__ ids, const int32_t *__restrict__ expand_idx,
                                        const int32_t *__restrict__ ep_send_counts, long long n, int E, long long A,
                                        int32_t *__restrict__ slot_row)
{
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    const int e = ids[i];
    long long row = -1;
    if (e >= 0 && e < E) {
        row = (long long)(e == 0 ? 0 : ep_send_counts[e - 1]) + expand_idx[i];
        if (row < 0 || row >= A) {
            row = -1;
        }
    }
    slot_row[i] = (int32_t)row;
}

// Rows of the activation type (ACT: 0 = bf16, 1 = IEEE fp16) -> wire rows, whose block scales are of that type
// too (moe_combine_shmem.h:567-592 keeps them as ExpandXType).  One thread per block of 8 columns.
template <int ACT>
__global__ __launch_bounds__(256) void comm_quant_kernel(const uint16_t *__restrict__ y, long long A, int H,
                                                         const int32_t *__restrict__ row_limit,
                                                         uint8_t *__restrict__ out)
{
    const int blocks_per_row = H / 8;
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long row = i / blocks_per_row;
    const int b = (int)(i - row * blocks_per_row);
    const long long rows = row_limit == nullptr ? A : min(A, (long long)*row_limit);
    if (row >= rows) {
        return;
    }
    const v4u v = __builtin_nontemporal_load((const v4u *)(y + row * H + b * 8));
    float x[8];
    float m = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        x[2 * c] = ACT == 0 ? bf16_bits_to_f32(v[c] & 0xffffu) : fp16_bits_to_f32(v[c] & 0xffffu);
        x[2 * c + 1] = ACT == 0 ? bf16_bits_to_f32(v[c] >> 16) : fp16_bits_to_f32(v[c] >> 16);
        m = fmaxf(m, fmaxf(fabsf(x[2 * c]), fabsf(x[2 * c + 1])));
    }
    const long long pitch = (long long)H + H / 4;
    uint32_t q[2] = {0u, 0u};
    uint16_t sbits = 0;
    if (m != 0.0f) {
        const float s = __fmul_rn(m, 1.0f / 127.0f);
        sbits = (uint16_t)(ACT == 0 ? f32_to_bf16_bits(s) : f32_to_fp16_bits(s));
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const _Float16 h = (_Float16)__fdiv_rn(x[j], s);  // round to nearest even
            const int qi = (int)rintf((float)h);
            q[j >> 2] |= (uint32_t)(qi & 0xff) << (8 * (j & 3));
        }
    }
    uint8_t *dst = out + row * pitch;
    *(v2u *)(dst + b * 8) = v2u{q[0], q[1]};
    *(uint16_t *)(dst + H + b * 2) = sbits;
}

// ACT: 0 = bf16 rows and output, 1 = IEEE fp16 (the layer's activation type).
template <int ACT>
__device__ __forceinline__ float comb_act_to_f32(uint32_t bits16)
{
    return ACT == 0 ? bf16_bits_to_f32(bits16) : fp16_bits_to_f32(bits16);
}

template <bool WIRE, int ACT>
__global__ __launch_bounds__(kCombThreads) void combine_kernel(CombineArgs a, int segs)
{
    const int t = blockIdx.x / segs;
    const int seg = blockIdx.x - t * segs;
    const int col = (seg * kCombThreads + threadIdx.x) * 8;
    if (col >= a.H) {
        return;
    }
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        acc[j] = 0.0f;
    }
    const bool live = a.t_active == nullptr || t < *a.t_active;
    const long long rows = a.row_limit == nullptr ? a.A : min(a.A, (long long)*a.row_limit);
    const bool add_shared = live && a.shared != nullptr;
    v4u sh = {0u, 0u, 0u, 0u};
    if (add_shared) {  // requested with the routed rows, used after them
        sh = __builtin_nontemporal_load((const v4u *)(a.shared + (long long)t * a.H + col));
    }
    if (live) {
        for (int k0 = 0; k0 < a.K; k0 += kCombBatch) {
            v4u v[kCombBatch];  // WIRE: x, y = the 8 int8 values, z = the block's scale (bf16 bits)
            float w[kCombBatch];
            bool ok[kCombBatch];
#pragma unroll
            for (int j = 0; j < kCombBatch; ++j) {
                const int k = k0 + j;
                ok[j] = false;
                w[j] = 0.0f;
                v[j] = v4u{0u, 0u, 0u, 0u};
                if (k < a.K) {
                    const long long slot = (long long)t * a.K + k;
                    const long long row = a.slot_row[slot];
                    bool good = row >= 0 && row < rows;
                    if (good && a.src_info != nullptr) {
                        // The inverse map is not pre-cleared: accept a row only if it names this slot.
                        good = a.src_info[3 * row + 1] == t && a.src_info[3 * row + 2] == k;
                    }
                    if (good) {
                        ok[j] = true;
                        w[j] = a.w[slot];
                        if (WIRE) {
                            const uint8_t *src = (const uint8_t *)a.y + row * ((long long)a.H + a.H / 4);
                            const v2u q = __builtin_nontemporal_load((const v2u *)(src + col));
                            const uint16_t sc = __builtin_nontemporal_load((const uint16_t *)(src + a.H) + (col >> 3));
                            v[j] = v4u{q[0], q[1], sc, 0u};
                        } else {
                            v[j] = __builtin_nontemporal_load((const v4u *)(a.y + row * a.H + col));
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kCombBatch; ++j) {
                if (ok[j] && WIRE) {
                    const float sc = comb_act_to_f32<ACT>(v[j][2]);
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        const int q = (int)(int8_t)((v[j][c >> 2] >> (8 * (c & 3))) & 0xffu);
                        // the row as it leaves the wire: rounded to the activation type (moe_combine_shmem.h:755-773)
                        const float p = __fmul_rn((float)q, sc);
                        const float x = ACT == 0 ? bf16_bits_to_f32(f32_to_bf16_bits(p))
                                                 : fp16_bits_to_f32(f32_to_fp16_bits(p));
                        acc[c] = __fadd_rn(acc[c], __fmul_rn(x, w[j]));
                    }
                } else if (ok[j]) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float x0 = comb_act_to_f32<ACT>(v[j][c] & 0xffffu);
                        float x1 = comb_act_to_f32<ACT>(v[j][c] >> 16);
                        acc[2 * c] = __fadd_rn(acc[2 * c], __fmul_rn(x0, w[j]));
                        acc[2 * c + 1] = __fadd_rn(acc[2 * c + 1], __fmul_rn(x1, w[j]));
                    }
                }
            }
        }
    }
    if (add_shared) {  // the shared expert's row: un-weighted, after the routed rows
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            acc[2 * c] = __fadd_rn(acc[2 * c], comb_act_to_f32<ACT>(sh[c] & 0xffffu));
            acc[2 * c + 1] = __fadd_rn(acc[2 * c + 1], comb_act_to_f32<ACT>(sh[c] >> 16));
        }
    }
    v4u o;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        o[c] = ACT == 0 ? f32x2_to_bf16x2_bits(acc[2 * c], acc[2 * c + 1])
                        : f32_to_fp16_bits(acc[2 * c]) | (f32_to_fp16_bits(acc[2 * c + 1]) << 16);
    }
    __builtin_nontemporal_store(o, (v4u *)(a.out + (long long)t * a.H + col));
}

// Wire rows whose pitch keeps every 16-byte piece aligned (H a multiple of 64): a thread owns two blocks of 8
// columns and reads 16 + 4 bytes per row, the widths of the bf16 gather.  The arithmetic is that of
// combine_kernel<true>; the rebuilt values are rounded to bf16 two at a time by the hardware conversion
// (round to nearest even, subnormals kept), which is what keeps the kernel bound by memory rather than by the
// vector ALU (5.2 TB/s against 4.1 TB/s with 8 columns per thread and integer rounding).
constexpr int kWireBatch = 4;
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__global__ __launch_bounds__(kCombThreads) void combine_wire16_kernel(CombineArgs a, int segs)
{
    const int t = blockIdx.x / segs;
    const int seg = blockIdx.x - t * segs;
    const int col = (seg * kCombThreads + threadIdx.x) * 16;
    if (col >= a.H) {
        return;
    }
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        acc[j] = 0.0f;
    }
    const bool live = a.t_active == nullptr || t < *a.t_active;
    const long long rows = a.row_limit == nullptr ? a.A : min(a.A, (long long)*a.row_limit);
    const long long pitch = (long long)a.H + a.H / 4;
    if (live) {
        for (int k0 = 0; k0 < a.K; k0 += kWireBatch) {
            v4u v[kWireBatch];
            uint32_t sc2[kWireBatch];
            float w[kWireBatch];
            bool ok[kWireBatch];
#pragma unroll
            for (int j = 0; j < kWireBatch; ++j) {
                const int k = k0 + j;
                ok[j] = false;
                w[j] = 0.0f;
                v[j] = v4u{0u, 0u, 0u, 0u};
                sc2[j] = 0u;
                if (k < a.K) {
                    const long long slot = (long long)t * a.K + k;
                    const long long row = a.slot_row[slot];
                    bool good = row >= 0 && row < rows;
                    if (good && a.src_info != nullptr) {
                        good = a.src_info[3 * row + 1] == t && a.src_info[3 * row + 2] == k;
                    }
                    if (good) {
                        ok[j] = true;
                        w[j] = a.w[slot];
                        const uint8_t *src = (const uint8_t *)a.y + row * pitch;
                        v[j] = __builtin_nontemporal_load((const v4u *)(src + col));
                        sc2[j] = __builtin_nontemporal_load((const uint32_t *)(src + a.H + (col >> 2)));
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kWireBatch; ++j) {
                if (ok[j]) {
                    const float s_lo = __uint_as_float(sc2[j] << 16);
                    const float s_hi = __uint_as_float(sc2[j] & 0xffff0000u);
#pragma unroll
                    for (int c = 0; c < 16; c += 2) {
                        const int q0 = (int)(int8_t)((v[j][c >> 2] >> (8 * (c & 3))) & 0xffu);
                        const int q1 = (int)(int8_t)((v[j][c >> 2] >> (8 * ((c + 1) & 3))) & 0xffu);
                        const float sc = c < 8 ? s_lo : s_hi;
                        // one conversion instruction rounds both products to bf16 (nearest even)
                        const f32x2 p = {__fmul_rn((float)q0, sc), __fmul_rn((float)q1, sc)};
                        const f32x2 x = __builtin_convertvector(__builtin_convertvector(p, bf16x2), f32x2);
                        acc[c] = __fadd_rn(acc[c], __fmul_rn(x[0], w[j]));
                        acc[c + 1] = __fadd_rn(acc[c + 1], __fmul_rn(x[1], w[j]));
                    }
                }
            }
        }
    }
    if (live && a.shared != nullptr) {
        const v4u *sp = (const v4u *)(a.shared + (long long)t * a.H + col);
        const v4u s[2] = {__builtin_nontemporal_load(sp), __builtin_nontemporal_load(sp + 1)};
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            acc[2 * c] = __fadd_rn(acc[2 * c], bf16_bits_to_f32(s[c >> 2][c & 3] & 0xffffu));
            acc[2 * c + 1] = __fadd_rn(acc[2 * c + 1], bf16_bits_to_f32(s[c >> 2][c & 3] >> 16));
        }
    }
    v4u o[2];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        o[c >> 2][c & 3] = f32x2_to_bf16x2_bits(acc[2 * c], acc[2 * c + 1]);
    }
    v4u *dst = (v4u *)(a.out + (long long)t * a.H + col);
    __builtin_nontemporal_store(o[0], dst);
    __builtin_nontemporal_store(o[1], dst + 1);
}

}  // namespace

hipError_t launch_invert_src_info(const int32_t *src_info, int64_t A, const int32_t *row_limit, int T, int K,
                                  int32_t *slot_row, hipStream_t stream)
{
    if (A <= 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(invert_src_info_kernel, dim3((unsigned)((A + 255) / 256)), dim3(256), 0, stream, src_info,
                       (long long)A, row_limit, T, K, slot_row);
    return hipGetLastError();
}

hipError_t launch_rows_from_counts(const int32_t *ids, const int32_t *expand_idx, const int32_t *ep_send_counts,
                                   int64_t n, int E, int64_t A, int32_t *slot_row, hipStream_t stream)
{
    if (n <= 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(rows_from_counts_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, ids,
                       expand_idx, ep_send_counts, (long long)n, E, (long long)A, slot_row);
    return hipGetLastError();
}

hipError_t launch_comm_quant(const uint16_t *y, int act_fp16, int64_t A, int H, const int32_t *row_limit,
                             uint8_t *out, hipStream_t stream)
{
    if (A <= 0) {
        return hipSuccess;
    }
    if (H % 8 != 0) {
        return hipErrorInvalidValue;
    }
    const long long n = (long long)A * (H / 8);
    const long long blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffll) {
        return hipErrorInvalidValue;
    }
    if (act_fp16) {
        hipLaunchKernelGGL(comm_quant_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, stream, y, (long long)A, H,
                           row_limit, out);
    } else {
        hipLaunchKernelGGL(comm_quant_kernel<0>, dim3((unsigned)blocks), dim3(256), 0, stream, y, (long long)A, H,
                           row_limit, out);
    }
    return hipGetLastError();
}

hipError_t launch_combine(const CombineArgs &a, hipStream_t stream)
{
    if (a.T <= 0) {
        return hipSuccess;
    }
    if (a.H % 8 != 0) {
        return hipErrorInvalidValue;
    }
    const int segs = (a.H / 8 + kCombThreads - 1) / kCombThreads;
    const long long blocks = (long long)a.T * segs;
    if (blocks > 0x7fffffffll) {
        return hipErrorInvalidValue;
    }
    if (a.wire_rows && a.act_fp16) {
        hipLaunchKernelGGL((combine_kernel<true, 1>), dim3((unsigned)blocks), dim3(kCombThreads), 0, stream, a, segs);
    } else if (a.wire_rows && a.H % 64 == 0) {
        const int segs16 = (a.H / 16 + kCombThreads - 1) / kCombThreads;
        hipLaunchKernelGGL(combine_wire16_kernel, dim3((unsigned)(a.T * segs16)), dim3(kCombThreads), 0, stream, a,
                           segs16);
    } else if (a.wire_rows) {
        hipLaunchKernelGGL((combine_kernel<true, 0>), dim3((unsigned)blocks), dim3(kCombThreads), 0, stream, a, segs);
    } else if (a.act_fp16) {
        hipLaunchKernelGGL((combine_kernel<false, 1>), dim3((unsigned)blocks), dim3(kCombThreads), 0, stream, a, segs);
    } else {
        hipLaunchKernelGGL((combine_kernel<false, 0>), dim3((unsigned)blocks), dim3(kCombThreads), 0, stream, a, segs);
    }
    return hipGetLastError();
}

}  // namespace cam
