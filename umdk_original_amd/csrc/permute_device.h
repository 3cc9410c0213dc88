// Device code shared by the permute kernels: one wavefront loads one token row, quantises it in
// registers and stores it to any number of destination rows.
//
// Reference semantics (paths relative to the reference tree):
//   quant   src/cam/comm_operator/ascend_kernels/moe_dispatch_normal/op_kernel/moe_dispatch_normal.h:278-316
//           (scale = 127/(max|x| + 1e-12)), and the fused kernel's QuantToken,
//           src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/gemm/kernel/
//           grouped_matmul_slice_m_per_token_dequant_swiglu_quant_multistage_workspace.h:780-818 (no epsilon)
//   rows    moe_dispatch_normal.h:486-535 (int8 or 16-bit row, fp32 scale and (srcRank, token, k) per row)
// QUANT 3 has no counterpart in the reference: OCP FP8 E4M3 values with one power-of-two (E8M0) scale per row
// and 128 columns, as include/cam_fp8_spec.h defines them.
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
    uint32_t scale8[kDispMaxChunks];  // QUANT 3: E8M0 scale of the 128-column block chunk j of this lane lies in
};

// Exponent x of the smallest power of two 2^x with amax / 2^x <= 448 (amax = m * 2^e: e - 8, one more when
// m > 1.75), 0 for amax == 0, clamped to [-127, 127].
__device__ __forceinline__ int fp8_block_scale_exp(float amax)
{
    const uint32_t a = __float_as_uint(amax);
    if (a == 0u) {
        return 0;
    }
    int e;
    uint32_t frac;
    if ((a >> 23) == 0u) {
        const int lead = __clz(a) - 9;  // shifts that bring the leading one to bit 22
        e = -127 - lead;
        frac = (a << (lead + 1)) & 0x7fffffu;
    } else {
        e = (int)(a >> 23) - 127;
        frac = a & 0x7fffffu;
    }
    const int x = e - 8 + (frac > 0x600000u ? 1 : 0);
    return min(max(x, -127), 127);
}

__device__ __forceinline__ float exp2_int(int x)
{
    return x >= -126 ? __uint_as_float((uint32_t)(x + 127) << 23) : __uint_as_float(0x00400000u);
}

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

// FP8 with one scale per 128 columns.  Chunk c = 64 j + lane holds columns 8c .. 8c+7, so a block of 128
// columns is the 16 chunks of lanes 16 q .. 16 q + 15 at one j: its largest magnitude is a maximum over a
// quarter of the wave.  The scaled values lie within +-448, where the hardware conversion (round to nearest
// even) needs no saturation.
template <int ACT>
__device__ __forceinline__ void quant_token_row_fp8(TokenRow &r)
{
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
        float x[8];
        float m = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = act_bits_to_f32<ACT>(r.raw[j][i] & 0xffffu);
            x[2 * i + 1] = act_bits_to_f32<ACT>(r.raw[j][i] >> 16);
            m = fmaxf(m, fmaxf(fabsf(x[2 * i]), fabsf(x[2 * i + 1])));
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            m = fmaxf(m, __shfl_xor(m, off, kWave));
        }
        const int e = fp8_block_scale_exp(m);
        r.scale8[j] = (uint32_t)(e + 127);
        const float f1 = exp2_int(-(e / 2)), f2 = exp2_int(-(e - e / 2));
        int lo = 0, hi = 0;
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[0], f1), f2), __fmul_rn(__fmul_rn(x[1], f1), f2), lo,
                                             false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[2], f1), f2), __fmul_rn(__fmul_rn(x[3], f1), f2), lo,
                                             true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[4], f1), f2), __fmul_rn(__fmul_rn(x[5], f1), f2), hi,
                                             false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(__fmul_rn(__fmul_rn(x[6], f1), f2), __fmul_rn(__fmul_rn(x[7], f1), f2), hi,
                                             true);
        r.q[j] = v2u{(uint32_t)lo, (uint32_t)hi};
    }
}

// QUANT 1: scale = 127 / (max|x| + 1e-12); QUANT 2: scale = 127 / max|x|, an all-zero row giving zeros and scale 0.
template <int QUANT, int ACT>
__device__ __forceinline__ void quant_token_row(TokenRow &r)
{
    if (QUANT == 3) {
        quant_token_row_fp8<ACT>(r);
        return;
    }
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
    // Keep the row as its 16-bit words across the two passes: left alone, the compiler holds the 112 converted
    // floats of the maximum pass for the scaling pass (a shift each to redo) and the kernel needs a third more
    // registers.
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            asm volatile("" : "+v"(r.raw[j][i]));
        }
    }
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

// Quantisation of one COPY of a token row under a per-expert smooth scale
// (src/cam/comm_operator/ascend_kernels/moe_dispatch_shmem/op_kernel/moe_dispatch_shmem.h:693-733):
// xf = float(x) * smooth[h] (one rounded multiply), then the no-epsilon variant on xf.  r.raw is left untouched.
template <int ACT>
__device__ __forceinline__ void quant_token_row_smooth(TokenRow &r, const float *__restrict__ smooth, int H, int lane)
{
    const int nch = H >> 3;
    float m = 0.0f;
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
        const int c = j * kWave + lane;
        if (c < nch) {
            const v4f s0 = *(const v4f *)(smooth + c * 8);
            const v4f s1 = *(const v4f *)(smooth + c * 8 + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float sa = i < 2 ? s0[2 * i] : s1[2 * i - 4], sb = i < 2 ? s0[2 * i + 1] : s1[2 * i - 3];
                m = fmaxf(m, fabsf(__fmul_rn(act_bits_to_f32<ACT>(r.raw[j][i] & 0xffffu), sa)));
                m = fmaxf(m, fabsf(__fmul_rn(act_bits_to_f32<ACT>(r.raw[j][i] >> 16), sb)));
            }
        }
    }
    m = wave_max(m);
    const bool zero_row = m == 0.0f;
    const float s = zero_row ? 0.0f : __fdiv_rn(127.0f, m);
    r.scale_out = zero_row ? 0.0f : __fdiv_rn(1.0f, s);
#pragma unroll
    for (int j = 0; j < kDispMaxChunks; ++j) {
        const int c = j * kWave + lane;
        int v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (c < nch) {
            const v4f s0 = *(const v4f *)(smooth + c * 8);
            const v4f s1 = *(const v4f *)(smooth + c * 8 + 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float sa = i < 2 ? s0[2 * i] : s1[2 * i - 4], sb = i < 2 ? s0[2 * i + 1] : s1[2 * i - 3];
                v[2 * i] = (int)rintf(__fmul_rn(__fmul_rn(act_bits_to_f32<ACT>(r.raw[j][i] & 0xffffu), sa), s));
                v[2 * i + 1] = (int)rintf(__fmul_rn(__fmul_rn(act_bits_to_f32<ACT>(r.raw[j][i] >> 16), sb), s));
            }
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
    if (QUANT == 3) {
        // one E8M0 byte per 128 columns, written by the first lane of each quarter of the wave
        uint8_t *sc = (uint8_t *)scales + row * (H >> 7);
        if ((lane & 15) == 0) {
#pragma unroll
            for (int j = 0; j < kDispMaxChunks; ++j) {
                const int c = j * kWave + lane;
                if (c < nch) {
                    sc[c >> 4] = (uint8_t)r.scale8[j];
                }
            }
        }
    }
    if (lane == 0) {
        if (QUANT == 1 || QUANT == 2) {
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
