/*
 * cam_expf_spec.h -- the one transcendental on the CAM MoE path, fully specified.
 *
 * The reference's GMM1 epilogue computes SiLU as t / (1 + Exp(-t)) with the Ascend vector unit's
 * Exp (src/cam/comm_operator/ascend_kernels/fused_deep_moe/op_kernel/fused_deep_moe/epilogue/block/
 * block_epilogue_per_token_dequant_swiglu.h:253-260).  The bits of that Exp are not portable, so this
 * build fixes its own functions, made only of correctly rounded IEEE-754 binary32 operations that x86 and
 * gfx950 share.  The HIP kernels and the CPU oracle both include this header, which makes everything
 * downstream of SiLU (the second int8 quantisation, the bf16 output) reproducible bit-for-bit between them.
 * Two functions: cam_silu_spec() further down is what the layer uses; cam_expf_spec() is a stand-alone exp()
 * accurate to an ulp, kept as a yardstick for it.
 *
 * Host code including this header must be compiled with -ffp-contract=off (a fused multiply-add happens where
 * fmaf() is written and nowhere else).  Device code uses the __f*_rn intrinsics, which the compiler never
 * contracts.
 *
 * cam_expf_spec: Cody-Waite reduction x = n*ln2 + r, |r| <= ln2/2, degree-7 polynomial for exp(r)
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

/*
 * SiLU of the GMM1 epilogue, silu(t) = t / (1 + exp(-t)), as this build specifies it.
 *
 * The reference divides t by 1 + Exp(-t) with the Ascend vector unit's approximate Exp and accepts the result
 * to atol 2 / rtol 0.02 (block_epilogue_per_token_dequant_swiglu.h:253-260; test/cam/ut/fused_deep_moe/
 * test_fused_deep_moe.py:416-419).  The specification here is chosen for the epilogue of a matrix-core kernel,
 * where every instruction per product keeps the matrix pipes waiting: 19 operations, no division, no branch,
 * every one of them a correctly rounded IEEE-754 binary32 operation (min, max, multiply, add, fused
 * multiply-add, round-to-nearest-even, exact scaling by a power of two) that x86 and gfx950 both have, so the
 * CPU oracle and the kernels agree bit for bit.
 *
 *   a = min(|t|, 86)                         e^-86 is far below anything that survives the int8 re-quantisation
 *   z = a * -log2(e);  n = rint(z);  f = z - n       (f exact, |f| <= 1/2, -125 < n <= 0)
 *   p = 2^f   by a degree-4 polynomial (Horner in fused multiply-adds), relative error <= 2.6e-6
 *   e = p * 2^n = exp(-a)                    exact scaling, the result stays a normal number
 *   d = 1 + e  in (1, 2];   r0 = quadratic seed of 1/d (relative error <= 1.02e-2)
 *   u = 1 - d*r0;  r = r0 * (1 + u + u*u)    one cubically convergent step: relative error <= 1.1e-6
 *   q = e * r  = sigmoid(-a)
 *   silu(t) = max(t, 0) - a * q              t >= 0: t * (1 - q);  t < 0: t * q
 * Accuracy against the real function (tests pin it against float64): |error| <= 6e-6 * |silu(t)| for
 * |t| <= 20, <= 1.2e-5 * |silu(t)| for |t| <= 86, and below 4e-36 in absolute terms beyond (t < -86 gives
 * -86 e^-86 = -3.8e-36, t > 86 gives t); silu(0) = 0, silu(+inf) = +inf.
 * A NaN input does not come out as a NaN (min and max drop it); the dequantised sums that reach this function
 * are finite.
 */
#if defined(__HIP_DEVICE_COMPILE__)
#define CAM_FMA(a, b, c) __fmaf_rn((a), (b), (c))
#define CAM_FMIN(a, b) fminf((a), (b))
#define CAM_FMAX(a, b) fmaxf((a), (b))
#define CAM_FABS(a) fabsf(a)
#define CAM_LDEXP(a, n) __builtin_ldexpf((a), (n))
#else
#define CAM_FMA(a, b, c) fmaf((a), (b), (c))
#define CAM_FMIN(a, b) fminf((a), (b))
#define CAM_FMAX(a, b) fmaxf((a), (b))
#define CAM_FABS(a) fabsf(a)
#define CAM_LDEXP(a, n) ldexpf((a), (n))
#endif

CAM_SPEC_FN float cam_silu_spec(float t)
{
    const float a = CAM_FMIN(CAM_FABS(t), 86.0f);
    const float z = CAM_FMUL(a, -1.44269504088896341f);
    const float n = CAM_RINT(z);
    const float f = CAM_FSUB(z, n);
    float p = CAM_FMA(f, 9.570102e-3f, 5.591786e-2f);  /* minimax of 2^f on [-1/2, 1/2] for the relative error */
    p = CAM_FMA(f, p, 2.4024744e-1f);
    p = CAM_FMA(f, p, 6.931218e-1f);
    p = CAM_FMA(f, p, 9.999993e-1f);
    const float e = CAM_LDEXP(p, (int)n);
    const float d = CAM_FADD(e, 1.0f);
    float r = CAM_FMA(d, 3.2323232e-1f, -1.4545455f);  /* minimax of 1/d on [1, 2]: 32/99 d^2 - 144/99 d + 210/99 */
    r = CAM_FMA(d, r, 2.121212f);
    const float u = CAM_FMA(-d, r, 1.0f);
    r = CAM_FMA(CAM_FMA(u, u, u), r, r);
    const float q = CAM_FMUL(e, r);
    return CAM_FMA(-a, q, CAM_FMAX(t, 0.0f));
}

#endif /* CAM_EXPF_SPEC_H_ */
