// Device-side helpers shared by the CAM kernels (gfx950, 64-wide wavefronts).
#ifndef CAM_DEVICE_H_
#define CAM_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cam {

constexpr int kWave = 64;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16)
{
    return __uint_as_float(bits16 << 16);
}

// Round-to-nearest-even fp32 -> bf16 bit pattern (NaN stays a quiet NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    const uint32_t u = __float_as_uint(f);
    const uint32_t rounded = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    const uint32_t quiet = (u >> 16) | 0x0040u;
    return (u & 0x7fffffffu) > 0x7f800000u ? quiet : rounded;  // both sides computed: a select, no branch
}

// Two fp32 values -> two bf16 bit patterns (lo in bits 0..15) with ONE hardware conversion instruction.  Its results
// equal f32_to_bf16_bits on every one of the 2^32 inputs, NaNs included (checked exhaustively on the GPU by
// camCalibBf16Conversion and tests/test_gpu_gemm.py); it takes one vector instruction where the arithmetic form
// takes nine per value.
typedef float cam_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 cam_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi)
{
    const cam_f32x2 p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, cam_bf16x2));
}

// Round-to-nearest-even fp32 -> IEEE fp16 bit pattern (the hardware conversion; overflow gives infinity).
__device__ __forceinline__ uint32_t f32_to_fp16_bits(float f)
{
    return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f);
}

__device__ __forceinline__ float fp16_bits_to_f32(uint32_t bits16)
{
    return (float)__builtin_bit_cast(_Float16, (unsigned short)bits16);  // exact
}

__device__ __forceinline__ int lane_id()
{
    return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v = fmaxf(v, __shfl_xor(v, off, kWave));
    }
    return v;
}

__device__ __forceinline__ int wave_sum(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, kWave);
    }
    return v;
}

// Inclusive scan across the 64 lanes of a wave.
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane)
{
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        int n = __shfl_up(v, off, kWave);
        if (lane >= off) {
            v += n;
        }
    }
    return v;
}

}  // namespace cam

#endif  // CAM_DEVICE_H_
