/*
 * cam_expf_spec.h -- the one transcendental on the CAM MoE path, fully specified.
 *
 * The reference's GMM1 epilogue computes SiLU as t / (1 + Exp(-t)) with the Ascend vector unit's
 * Exp (src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/epilogue/block/
 * block_epilogue_per_token_dequant_swiglu.h:253-260).  The bits of that Exp are not portable, so this
 * build fixes an exp() made only of IEEE-754 binary32 add / sub / mul (one rounding each, never fused),
 * rint and integer bit operations.  The HIP kernels and the CPU oracle both include this header, which
 * makes everything downstream of SiLU (the second int8 quantisation, the bf16 output) reproducible
 * bit-for-bit between x86 and gfx950.
 *
 * Host code including this header must be compiled with -ffp-contract=off.
 * Device code uses the __f*_rn intrinsics, which the compiler never contracts.
 *
 * Algorithm: Cody-Waite reduction x = n*ln2 + r, |r| <= ln2/2, degree-7 polynomial for exp(r)
 * (Horner, coefficients of the classic single-precision Cephes expf), scaling by 2^n in two exact
 * power-of-two multiplies.  Max error ~1 ulp against the real exp on [-87, 88].
 */
#ifndef CAM_EXPF_SPEC_H_
#define CAM_EXPF_SPEC_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define CAM_SPEC_FN static __host__ __device__ __forceinline__
#else
#define CAM_SPEC_FN static inline
#endif

#if defined(__HIP_DEVICE_COMPILE__)
#define CAM_FMUL(a, b) __fmul_rn((a), (b))
#define CAM_FADD(a, b) __fadd_rn((a), (b))
#define CAM_FSUB(a, b) __fsub_rn((a), (b))
#define CAM_RINT(a) rintf(a)
#define CAM_BITS_TO_F(u) __uint_as_float(u)
#else
#include <math.h>
#include <string.h>
#define CAM_FMUL(a, b) ((a) * (b))
#define CAM_FADD(a, b) ((a) + (b))
#define CAM_FSUB(a, b) ((a) - (b))
#define CAM_RINT(a) rintf(a)
static inline float cam_bits_to_f_(uint32_t u)
{
    float f;
    memcpy(&f, &u, sizeof(f));
    return f;
}
#define CAM_BITS_TO_F(u) cam_bits_to_f_(u)
#endif

CAM_SPEC_FN float cam_expf_spec(float x)
{
    if (x != x) {
        return x; /* NaN in, NaN out */
    }
    if (x > 88.72283f) {
        return CAM_BITS_TO_F(0x7f800000u); /* +inf */
    }
    if (x < -103.9f) {
        return 0.0f;
    }
    const float kLog2e = 1.44269504088896341f;
    const float kLn2Hi = 0.693359375f;       /* 0x3f318000: 9 significant bits, n*kLn2Hi is exact */
    const float kLn2Lo = -2.12194440e-4f;    /* ln2 - kLn2Hi */
    float n = CAM_RINT(CAM_FMUL(x, kLog2e));
    float r = CAM_FSUB(x, CAM_FMUL(n, kLn2Hi));
    r = CAM_FSUB(r, CAM_FMUL(n, kLn2Lo));
    float p = 1.9875691500e-4f;
    p = CAM_FADD(CAM_FMUL(p, r), 1.3981999507e-3f);
    p = CAM_FADD(CAM_FMUL(p, r), 8.3334519073e-3f);
    p = CAM_FADD(CAM_FMUL(p, r), 4.1665795894e-2f);
    p = CAM_FADD(CAM_FMUL(p, r), 1.6666665459e-1f);
    p = CAM_FADD(CAM_FMUL(p, r), 5.0000001201e-1f);
    float r2 = CAM_FMUL(r, r);
    float y = CAM_FADD(CAM_FADD(CAM_FMUL(p, r2), r), 1.0f);
    int ni = (int)n; /* |n| <= 150, exact */
#if defined(__HIP_DEVICE_COMPILE__)
    /* One v_ldexp_f32 gives the bits of the two multiplies below: y * s1 is exact (y in [0.7, 1.5], |n1| <= 75, the
     * product stays normal), so the second multiply is the only rounding, and it rounds y * 2^n to nearest even
     * exactly as ldexp does, into the subnormals and up to infinity alike. */
    return __builtin_ldexpf(y, ni);
#else
    int n1 = ni / 2;
    int n2 = ni - n1;
    float s1 = CAM_BITS_TO_F((uint32_t)(n1 + 127) << 23);
    float s2 = CAM_BITS_TO_F((uint32_t)(n2 + 127) << 23);
    return CAM_FMUL(CAM_FMUL(y, s1), s2);
#endif
}

/* SiLU exactly as the reference orders it: e = exp(-t); d = 1 + e; out = t / d (IEEE division). */
CAM_SPEC_FN float cam_silu_spec(float t)
{
    float e = cam_expf_spec(-t);
    float d = CAM_FADD(e, 1.0f);
#if defined(__HIP_DEVICE_COMPILE__)
    return __fdiv_rn(t, d);
#else
    return t / d;
#endif
}

#endif /* CAM_EXPF_SPEC_H_ */
