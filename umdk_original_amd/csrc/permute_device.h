// Device code shared by the permute kernels: one wavefront loads one token row, quantises it in
// registers and stores it to any number of destination rows.
//
// Reference semantics (paths relative to the reference tree):
//   quant   src/cam/comm_operator/ascend_kernels/moe_dispatch_normal/op_kernel/moe_dispatch_normal.h:278-316
//           (scale = 127/(max|x| + 1e-12)), and the fused kernel's QuantToken,
//           src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/gemm/kernel/
//           grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:780-818 (no epsilon)
//   rows    moe_dispatch_normal.h:486-535 (int8 or 16-bit row, fp32 scale and (srcRank, token, k) per row)
#ifndef CAM_PERMUTE_DEVICE_H_
#define CAM_PERMUTE_DEVICE_H_

#include "cam_device.h"
#include "cam_kernels.h"

namespace cam {

constexpr int kDispWaves = 4;         // tokens (waves) per workgroup
constexpr int kDispMaxChunks = 14;    // 16-byte chunks per lane: H <= 14 * 64 * 8 = 7168

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d)
{
    return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) | ((uint32_t)(c & 0xff) << 16) |
           ((uint32_t)(d & 0xff) << 24);
}

// 16-bit activation formats.  ACT = 0: bf16 (the upper half of an fp32); ACT = 1: IEEE fp16.
template <int ACT>
__device__ __forceinline__ float act_bits_to_f32(uint32_t bits16)
{
    if (ACT == 0) {
        return bf16_bits_to_f32(bits16);
    }
    return (float)__builtin_bit_cast(_Float16, (unsigned short)bits16);  // exact
}

// One token row held by a wavefront: lane l owns the 16-byte chunks l, l+64, ... of the row.
struct TokenRow {
    v4u raw[kDispMaxChunks];
    v2u q[kDispMaxChunks];
    float scale_out;
};

__device__ __forceinline__ void load_token_row(const uint16_t *x, int t, int H, int lane, TokenRow &r)
{
    const int nch = H >> 3;  // 8 values per chunk
    const v4u *src = (const v4u *)(x + (long long)t * H);
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
        const int c = j * kWave + lane;
        r.raw[j] = v4u{0u, 0u, 0u, 0u};
        if (c < nch) {
            r.raw[j] = __builtin_nontemporal_load(src + c);
        }
    }
}

// QUANT 1: scale = 127 / (max|x| + 1e-12); QUANT 2: scale = 127 / max|x|, an all-zero row giving zeros and scale 0.
template <int QUANT, int ACT>
__device__ __forceinline__ void quant_token_row(TokenRow &r)
{
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            m = fmaxf(m, fabsf(act_bits_to_f32<ACT>(r.raw[j][i] & 0xffffu)));
            m = fmaxf(m, fabsf(act_bits_to_f32<ACT>(r.raw[j][i] >> 16)));
        }
    }
    m = wave_max(m);
    float s;
    bool zero_row = false;
    if (QUANT == 1) {
        s = __fdiv_rn(127.0f, __fadd_rn(m, 1e-12f));
    } else {
        zero_row = (m == 0.0f);
        s = zero_row ? 0.0f : __fdiv_rn(127.0f, m);
    }
    r.scale_out = zero_row ? 0.0f : __fdiv_rn(1.0f, s);
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
        int v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = (int)rintf(__fmul_rn(act_bits_to_f32<ACT>(r.raw[j][i] & 0xffffu), s));
            v[2 * i + 1] = (int)rintf(__fmul_rn(act_bits_to_f32<ACT>(r.raw[j][i] >> 16), s));
        }
        r.q[j] = v2u{pack4(v[0], v[1], v[2], v[3]), pack4(v[4], v[5], v[6], v[7])};
    }
}

// Stores the row (quantised or raw) to output row `row`, with its scale and triple.
template <int QUANT>
__device__ __forceinline__ void store_token_row(const TokenRow &r, void *out, float *scales, int32_t *src_info,
                                                int src_rank, long long row, int t, int k, int H, int lane)
{
    const int nch = H >> 3;
    if (QUANT != 0) {
        v2u *dst = (v2u *)((int8_t *)out + row * H);
#pragma unroll
        for (int j = 0; j < kDispMaxChunks; ++j) {
            const int c = j * kWave + lane;
            if (c < nch) {
                __builtin_nontemporal_store(r.q[j], dst + c);
            }
        }
    } else {
        v4u *dst = (v4u *)((uint16_t *)out + row * H);
#pragma unroll
        for (int j = 0; j < kDispMaxChunks; ++j) {
            const int c = j * kWave + lane;
            if (c < nch) {
                __builtin_nontemporal_store(r.raw[j], dst + c);
            }
        }
    }
    if (lane == 0) {
        if (QUANT != 0) {
            scales[row] = r.scale_out;
        }
        if (src_info != nullptr) {
            src_info[3 * row + 0] = src_rank;
            src_info[3 * row + 1] = t;
            src_info[3 * row + 2] = k;
        }
    }
}

}  // namespace cam

#endif  // CAM_PERMUTE_DEVICE_H_
