/*
 * cam_fp8_spec.h -- the block-scaled FP8 variant of the CAM MoE layer, fully specified.
 *
 * The reference has no FP8 path: its fused operator is W8A8 int8 only (src/cam/README.md:20-21).  This header
 * is therefore a definition, not a restatement.  It fixes the three pieces of arithmetic the FP8 layer adds to
 * the int8 one, in a form that both the CPU oracle and a reader can evaluate by hand.
 *
 * 1. The element type: OCP FP8 E4M3 ("e4m3fn"): 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities;
 *    S.1111.111 is NaN; largest finite value 448; subnormals m/8 * 2^-6.
 *    cam_f32_to_e4m3() rounds to nearest, ties to even, and SATURATES: every |x| above 448 becomes +-448.
 * 2. The scale type: E8M0, a power of two stored as its biased exponent, value 2^(byte - 127).
 * 3. The block scale of a run of values with largest magnitude `amax`: the smallest power of two s with
 *    amax / s <= 448, computed on the bits of amax (no division, no logarithm):
 *        amax = m * 2^e, 1 <= m < 2:   s = 2^(e - 8) if m <= 1.75, else 2^(e - 7);      (448 = 1.75 * 2^8)
 *    amax == 0 gives s = 1.  The exponent is clamped to [-127, 127].  Dividing by s is exact, so no value of the
 *    block saturates and the largest scaled value lies in (224, 448] before it is rounded.
 *
 * Blocks: activations carry one scale per row and per 128 consecutive columns of K; weights carry one scale per
 * 128 x 128 block of (K, N).  A product of the layer is
 *        out[m, n] = sum over K-blocks kb of  2^(sa[m, kb] + sw[kb, n / 128]) * sum_{k in kb} a[m, k] * w[k, n]
 * with the inner sums and the outer sum accumulated in fp32 in an order the hardware chooses; results are
 * compared with a tolerance, not bit for bit.
 */
#ifndef CAM_FP8_SPEC_H_
#define CAM_FP8_SPEC_H_

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define CAM_FP8_FN static __host__ __device__ __forceinline__
#else
#define CAM_FP8_FN static inline
#endif

#define CAM_FP8_BLOCK 128
#define CAM_E4M3_MAX 448.0f

CAM_FP8_FN uint32_t cam_fp8_f32_bits_(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof(u));
    return u;
}

CAM_FP8_FN float cam_fp8_bits_f32_(uint32_t u)
{
    float f;
    memcpy(&f, &u, sizeof(f));
    return f;
}

CAM_FP8_FN float cam_e4m3_to_f32(uint8_t v)
{
    const uint32_t sign = (uint32_t)(v & 0x80u) << 24;
    const uint32_t exp = (v >> 3) & 0xfu;
    const uint32_t man = v & 0x7u;
    if (exp == 0xfu && man == 0x7u) {
        return cam_fp8_bits_f32_(sign | 0x7fc00000u);
    }
    if (exp == 0) {
        /* subnormal: man * 2^-9, exact in fp32 */
        const float mag = (float)man * 0.001953125f;
        return cam_fp8_bits_f32_(sign | cam_fp8_f32_bits_(mag));
    }
    return cam_fp8_bits_f32_(sign | ((exp + 120u) << 23) | (man << 20));
}

CAM_FP8_FN uint8_t cam_f32_to_e4m3(float f)
{
    const uint32_t u = cam_fp8_f32_bits_(f);
    const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    const uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) {
        return (uint8_t)(sign | 0x7fu); /* NaN */
    }
    if (a > 0x43e00000u) {
        return (uint8_t)(sign | 0x7eu); /* above 448 (infinity included): saturate */
    }
    if (a <= 0x3a800000u) {
        return sign; /* at most 2^-10, half the smallest subnormal 2^-9: zero (the tie goes to even) */
    }
    const int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t man = (a & 0x7fffffu) | 0x800000u; /* 24-bit significand, value man * 2^(e - 23) */
    int shift;                                  /* bits dropped */
    uint32_t base;
    if (e < -6) {
        shift = 14 - e; /* subnormal result, unit 2^-9: man * 2^(e - 23) / 2^-9 = man >> (14 - e) */
        base = 0;
    } else {
        shift = 20;
        base = (uint32_t)(e + 7) << 3;
        man &= 0x7fffffu;
    }
    uint32_t kept = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) {
        ++kept; /* a carry out of the mantissa lands in the exponent field, as it should */
    }
    return (uint8_t)(sign | (uint8_t)(base + kept));
}

/* Exponent x of the block scale 2^x for a block whose largest magnitude is amax (finite, >= 0). */
CAM_FP8_FN int cam_fp8_block_scale_exp(float amax)
{
    const uint32_t a = cam_fp8_f32_bits_(amax) & 0x7fffffffu;
    if (a == 0) {
        return 0;
    }
    int e;
    uint32_t frac; /* 23 fraction bits of m in [1, 2) */
    if ((a >> 23) == 0) {
        /* subnormal input: normalise */
        int lead = 0;
        uint32_t m = a;
        while ((m & 0x400000u) == 0) {
            m <<= 1;
            ++lead;
        }
        e = -127 - lead;
        frac = (m << 1) & 0x7fffffu;
    } else {
        e = (int)(a >> 23) - 127;
        frac = a & 0x7fffffu;
    }
    int x = e - 8 + (frac > 0x600000u ? 1 : 0); /* m > 1.75 */
    if (x < -127) {
        x = -127;
    }
    if (x > 127) {
        x = 127;
    }
    return x;
}

CAM_FP8_FN uint8_t cam_e8m0_from_exp(int x) { return (uint8_t)(x + 127); }

/* 2^x for x in [-127, 127] (2^-127 is subnormal in fp32 and still exact). */
CAM_FP8_FN float cam_exp2_int(int x)
{
    return x >= -126 ? cam_fp8_bits_f32_((uint32_t)(x + 127) << 23) : cam_fp8_bits_f32_(0x00400000u);
}

#endif /* CAM_FP8_SPEC_H_ */
