/*
 * cam_oracle.c -- CPU restatement of the CAM MoE hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP kernels are compared against.  Nothing in the shipped library
 * links, loads or calls it; only tests/, the smoke test and the benchmark's cpu_baseline leg do.
 *
 * Every function restates one piece of the reference's arithmetic, in the reference's operation
 * order, with IEEE-754 binary32 operations rounded once each.  Compile with -ffp-contract=off.
 * Paths are relative to the reference tree; AK = src/cam/comm_operator/ascend_kernels,
 * PB = src/cam/comm_operator/pybind, FDM = AK/fused_deep_moe/op_kernel/fused_deep_moe.
 *
 * Parity status.  Integer functions (layout, offsets, ranks, receive bookkeeping, int32 GEMM) and the
 * dispatch quantisation are pinned by closed forms and brute-force definitions in tests/test_oracle.py.
 * The reference ships no golden vectors for this path, and its kernels cannot be built without the
 * Ascend toolkit, so no function here is checked against reference *outputs*.  These functions rest on
 * a deliberate definition the reference does not give portably and are therefore "parity unpinned"
 * against the Ascend hardware bit-for-bit:
 *   - cam_oracle_gmm1_epilogue: SiLU is cam_silu_spec() (a fixed sequence of 19 rounded operations, within
 *     1.2e-5 relative of the exact function) in place of the Ascend Exp and Div instructions;
 *   - everything downstream of it (cam_oracle_swiglu_quant's int8 values, the bf16 layer output)
 *     inherits that; the reference's own acceptance bound there is atol 2.0 / rtol 0.02;
 *   - cam_oracle_comm_quant_rows(_act) and cam_oracle_dispatch_shmem take the Ascend Div to be the IEEE quotient
 *     and every written operation to round once.
 * All-zero rows (division by zero in the reference, AK/.../grouped_matmul_slice_m_per_token_dequant_
 * swiglu_quant_multistage_workspace.h:804 and :252-255) are defined here as q = 0, scale = 0.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#include "../include/cam_expf_spec.h"
#include "../include/cam_fp8_spec.h"

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ---------------------------------------------------------------- bf16 helpers */

static inline float bf16_to_f32(uint16_t v)
{
    uint32_t u = (uint32_t)v << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, the CAST_RINT of FDM/raw_distributed/cam_moe_distribute_combine.h:778 */
static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* IEEE binary16 -> binary32, exact (the reference's dispatch accepts fp16 activations as well as bf16:
 * AK/moe_dispatch_normal/op_host/moe_dispatch_normal.cpp:17-22; its Cast to float is exact either way). */
static inline float fp16_to_f32(uint16_t v)
{
    uint32_t sign = (uint32_t)(v & 0x8000u) << 16;
    uint32_t exp = (v >> 10) & 0x1fu;
    uint32_t man = v & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: value = man * 2^-24 */
            float f = (float)man * 5.9604644775390625e-8f;
            memcpy(&u, &f, 4);
            u |= sign;
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* act: 0 = bf16 bits, 1 = fp16 bits */
static inline float act_to_f32(uint16_t v, int act) { return act ? fp16_to_f32(v) : bf16_to_f32(v); }

ORACLE_API float cam_oracle_fp16_to_f32(uint16_t v) { return fp16_to_f32(v); }

ORACLE_API int cam_oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Threads used by the row-parallel loops from now on (the benchmark's single-thread CPU figure uses 1). */
ORACLE_API void cam_oracle_set_num_threads(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n < 1 ? 1 : n);
#else
    (void)n;
#endif
}

ORACLE_API float cam_oracle_expf(float x) { return cam_expf_spec(x); }
ORACLE_API float cam_oracle_silu(float x) { return cam_silu_spec(x); }
ORACLE_API uint16_t cam_oracle_f32_to_bf16(float x) { return f32_to_bf16(x); }

/* ---------------------------------------------------------------- A.1 layout
 * AK/dispatch_layout/op_kernel/dispatch_layout.h:83-134 (counts, rank = e / (E/R), first-seen flag
 * per token and rank); negative ids are skipped as in PB/moe_dispatch_prefill.cpp:106.
 * The reference kernel indexes its count table with the id unguarded (dispatch_layout.h:113-118), so an
 * id >= E has no defined result there.  skip_out_of_range == 0: such an id is an error (returns -1);
 * != 0: it is skipped like a negative one, which is what the HIP kernels are specified to do. */
ORACLE_API int cam_oracle_layout(const int64_t *idx, int64_t T, int64_t K, int64_t E, int64_t R,
                                 int skip_out_of_range, int32_t *cnt, int32_t *per_rank, uint8_t *in_rank)
{
    int64_t epr = E / R;
    memset(cnt, 0, sizeof(int32_t) * (size_t)E);
    memset(per_rank, 0, sizeof(int32_t) * (size_t)R);
    memset(in_rank, 0, (size_t)(T * R));
    for (int64_t t = 0; t < T; ++t) {
        for (int64_t k = 0; k < K; ++k) {
            int64_t e = idx[t * K + k];
            if (e < 0) {
                continue;
            }
            if (e >= E) {
                if (skip_out_of_range) {
                    continue;
                }
                return -1;
            }
            cnt[e] += 1;
            int64_t r = e / epr;
            if (!in_rank[t * R + r]) {
                in_rank[t * R + r] = 1;
                per_rank[r] += 1;
            }
        }
    }
    return 0;
}

/* ---------------------------------------------------------------- A.2 offsets
 * AK/notify_dispatch/op_kernel/notify_dispatch.h:121-152: exclusive prefix sum in global expert
 * order, and the (count, offset, numTokens) triplet per expert. */
ORACLE_API void cam_oracle_offsets(const int32_t *cnt, int64_t E, int32_t num_tokens, int32_t *off,
                                   int32_t *triplets)
{
    int32_t run = 0;
    for (int64_t e = 0; e < E; ++e) {
        off[e] = run;
        if (triplets) {
            triplets[3 * e + 0] = cnt[e];
            triplets[3 * e + 1] = run;
            triplets[3 * e + 2] = num_tokens;
        }
        run += cnt[e];
    }
}

/* ---------------------------------------------------------------- A.3 within-expert rank
 * PB/moe_dispatch_prefill.cpp:96-112 (running counter per expert over the flat (t,k) order); the
 * fused kernel's CalExpandxIdx (…swiglu_quant_multistage_workspace.h:680-708) computes the same
 * number by counting earlier equal ids.  Entries with idx < 0 receive -1 (the reference leaves
 * them uninitialised). */
ORACLE_API void cam_oracle_send_token_idx(const int64_t *idx, int64_t T, int64_t K, int64_t E,
                                          int32_t *pos)
{
    int32_t *run = (int32_t *)calloc((size_t)E, sizeof(int32_t));
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = idx[i];
        if (e < 0 || e >= E) {
            pos[i] = -1;
            continue;
        }
        pos[i] = run[e];
        run[e] += 1;
    }
    free(run);
}

/* ---------------------------------------------------------------- A.4 receive bookkeeping
 * PB/moe_dispatch_prefill.cpp:126-145.  recv_data is what rank `me` holds after the count exchange:
 * for source rank s and local expert le the triplet sits at 3*(s*Epr + le).  Emits the inclusive
 * cumsum in (local expert, source rank) order, the per-pair source offset, and the per-expert totals
 * (int64, the binding's fourth return value; the fused kernel's expert_token_nums,
 * …swiglu_quant_multistage_workspace.h:1540-1544).  Returns the total row count. */
ORACLE_API int64_t cam_oracle_recv_bookkeeping(const int32_t *recv_data, int64_t R, int64_t epr,
                                               int32_t *recv_count, int32_t *recv_offset,
                                               int64_t *tokens_per_expert, int64_t *max_bs)
{
    int64_t total = 0;
    int64_t mx = 0;
    for (int64_t le = 0; le < epr; ++le) {
        int64_t local = 0;
        for (int64_t s = 0; s < R; ++s) {
            int64_t index = le * R + s;
            int64_t pair = 3 * (s * epr + le);
            total += recv_data[pair];
            recv_count[index] = (int32_t)total;
            recv_offset[index] = recv_data[pair + 1];
            if (recv_data[pair + 2] > mx) {
                mx = recv_data[pair + 2];
            }
            local += recv_data[pair];
        }
        tokens_per_expert[le] = local;
    }
    if (max_bs) {
        *max_bs = mx;
    }
    return total;
}

/* ---------------------------------------------------------------- A.6 per-token int8 quantisation
 * variant 1 ("Q1"): AK/moe_dispatch_normal/op_kernel/moe_dispatch_normal.h:278-316
 *     s = 127.0f / (max|x| + 1e-12f); q = int8(rint(x * s)); scale_out = 1.0f / s
 * variant 2 ("Q2"): FDM/gemm/kernel/…swiglu_quant_multistage_workspace.h:780-818
 *     s = 127.0f / max|x| (no epsilon); an all-zero row is defined as q = 0, scale_out = 0. */
static void quant_token(const uint16_t *x, int64_t H, int variant, int act, int8_t *q, float *scale_out)
{
    float m = 0.0f;
    for (int64_t h = 0; h < H; ++h) {
        float a = fabsf(act_to_f32(x[h], act));
        if (a > m) {
            m = a;
        }
    }
    float s;
    if (variant == 1) {
        s = 127.0f / (m + 1e-12f);
    } else {
        if (m == 0.0f) {
            memset(q, 0, (size_t)H);
            *scale_out = 0.0f;
            return;
        }
        s = 127.0f / m;
    }
    for (int64_t h = 0; h < H; ++h) {
        float v = act_to_f32(x[h], act) * s;
        q[h] = (int8_t)(int32_t)nearbyintf(v);
    }
    *scale_out = 1.0f / s;
}

/* variant: 1 / 2 as above, + 16 when x holds fp16 bits instead of bf16 bits. */
ORACLE_API void cam_oracle_quant_rows(const uint16_t *x, int64_t rows, int64_t H, int variant,
                                      int8_t *q, float *scales)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        quant_token(x + r * H, H, variant & 15, variant >> 4, q + r * H, scales + r);
    }
}

/* ---------------------------------------------------------------- A.5 permute (+quant)
 * moe_dispatch_normal.h:330-396 (send side: row = send_offset[e] + send_token_idx, source row
 * tokenIndex / K, triple (srcRank, token, k) :318-328) and :486-535 (receive side: rows land at
 * recv_count[i-1] + j).  With one rank the window row equals the output row.
 * quant: 0 = copy the 16-bit rows, 1 = Q1, 2 = Q2 (+ 16: x holds fp16 bits).  out is 16-bit [A,H] or int8 [A,H]. */
ORACLE_API void cam_oracle_dispatch(const uint16_t *x, const int64_t *idx, const int32_t *off,
                                    const int32_t *pos, int64_t T, int64_t K, int64_t H, int64_t E,
                                    int quant, int32_t src_rank, void *out, float *scales,
                                    int32_t *src_info)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = idx[i];
        if (e < 0 || e >= E) {
            continue;
        }
        int64_t t = i / K;
        int64_t row = (int64_t)off[e] + pos[i];
        if ((quant & 15) == 0) {
            memcpy((uint16_t *)out + row * H, x + t * H, (size_t)H * 2);
        } else {
            quant_token(x + t * H, H, quant & 15, quant >> 4, (int8_t *)out + row * H, scales + row);
        }
        if (src_info) {
            src_info[3 * row + 0] = src_rank;
            src_info[3 * row + 1] = (int32_t)t;
            src_info[3 * row + 2] = (int32_t)(i % K);
        }
    }
}

/* ---------------------------------------------------------------- A.7 / A.9 grouped int8 GEMM
 * …swiglu_quant_multistage_workspace.h:558-632 and …per_token_dequant_multistage_workspace.h:115-215:
 * for local expert g with rows [group_list[g-1], group_list[g]):  C[m,n] = sum_k A[m,k] * W[g][k][n],
 * int8 x int8 accumulated exactly in int32.  group_list is cumulative (int64).  W is [G, Kd, N]. */
ORACLE_API void cam_oracle_gmm_int32(const int8_t *a, const int8_t *w, const int64_t *group_list,
                                     int64_t G, int64_t Kd, int64_t N, int32_t *c)
{
    for (int64_t g = 0; g < G; ++g) {
        int64_t m0 = g == 0 ? 0 : group_list[g - 1];
        int64_t m1 = group_list[g];
        const int8_t *wg = w + g * Kd * N;
#pragma omp parallel for schedule(static)
        for (int64_t m = m0; m < m1; ++m) {
            int32_t *cr = c + m * N;
            for (int64_t n = 0; n < N; ++n) {
                cr[n] = 0;
            }
            const int8_t *ar = a + m * Kd;
            for (int64_t k = 0; k < Kd; ++k) {
                int32_t av = ar[k];
                if (av == 0) {
                    continue;
                }
                const int8_t *wr = wg + k * N;
                for (int64_t n = 0; n < N; ++n) {
                    cr[n] += av * (int32_t)wr[n];
                }
            }
        }
    }
}

/* ---------------------------------------------------------------- A.7 GMM1 epilogue
 * FDM/epilogue/block/block_epilogue_per_token_dequant_swiglu.h:236-264:
 *   t = (float(C) * w_scale[g][n]) * x_scale[m]   (weight scale first, then token scale)
 *   left half n < I: d = t / (1 + exp(-t));  right half: d = t.   d is fp32 [M, 2I]. */
ORACLE_API void cam_oracle_gmm1_epilogue(const int32_t *c, const float *w_scale, const float *x_scale,
                                         const int64_t *group_list, int64_t G, int64_t I, float *d)
{
    int64_t N = 2 * I;
    for (int64_t g = 0; g < G; ++g) {
        int64_t m0 = g == 0 ? 0 : group_list[g - 1];
        int64_t m1 = group_list[g];
        const float *ws = w_scale + g * N;
#pragma omp parallel for schedule(static)
        for (int64_t m = m0; m < m1; ++m) {
            for (int64_t n = 0; n < N; ++n) {
                float t = ((float)c[m * N + n] * ws[n]) * x_scale[m];
                d[m * N + n] = n < I ? cam_silu_spec(t) : t;
            }
        }
    }
}

/* ---------------------------------------------------------------- A.8 SwiGLU product + re-quant
 * …swiglu_quant_multistage_workspace.h:198-265:  y = d_left * d_right; m = max|y|;
 *   y_scale = m * (1.0f/127.0f);  q = int8(rint((y * 127.0f) * (1.0f / m))). */
ORACLE_API void cam_oracle_swiglu_quant(const float *d, int64_t M, int64_t I, int8_t *q,
                                        float *y_scale)
{
    const float inv127 = 1.0f / 127.0f;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        const float *dl = d + m * 2 * I;
        const float *dr = dl + I;
        float mx = 0.0f;
        for (int64_t i = 0; i < I; ++i) {
            float a = fabsf(dl[i] * dr[i]);
            if (a > mx) {
                mx = a;
            }
        }
        if (mx == 0.0f) {
            memset(q + m * I, 0, (size_t)I);
            y_scale[m] = 0.0f;
            continue;
        }
        y_scale[m] = mx * inv127;
        float rcp = 1.0f / mx;
        for (int64_t i = 0; i < I; ++i) {
            float y = dl[i] * dr[i];
            q[m * I + i] = (int8_t)(int32_t)nearbyintf((y * 127.0f) * rcp);
        }
    }
}

/* ---------------------------------------------------------------- A.9 GMM2 epilogue
 * FDM/epilogue/block/block_epilogue_per_token_dequant.hpp:665-684:
 *   out = bf16_rne((float(C2) * w2_scale[g][h]) * y_scale[m]). */
static inline uint16_t f32_to_fp16(float f);
static inline uint16_t f32_to_act(float f, int act) { return act ? f32_to_fp16(f) : f32_to_bf16(f); }

/* act: 0 = bf16 rows, 1 = fp16 rows (the output takes the activation type of the layer's input,
 * FDM/epilogue/block/block_epilogue_per_token_dequant.hpp:665-684 with ElementD = the token type). */
ORACLE_API void cam_oracle_gmm2_epilogue_act(const int32_t *c, const float *w_scale, const float *y_scale,
                                             const int64_t *group_list, int64_t G, int64_t H, int act,
                                             uint16_t *out)
{
    for (int64_t g = 0; g < G; ++g) {
        int64_t m0 = g == 0 ? 0 : group_list[g - 1];
        int64_t m1 = group_list[g];
        const float *ws = w_scale + g * H;
#pragma omp parallel for schedule(static)
        for (int64_t m = m0; m < m1; ++m) {
            for (int64_t h = 0; h < H; ++h) {
                out[m * H + h] = f32_to_act(((float)c[m * H + h] * ws[h]) * y_scale[m], act);
            }
        }
    }
}

ORACLE_API void cam_oracle_gmm2_epilogue(const int32_t *c, const float *w_scale, const float *y_scale,
                                         const int64_t *group_list, int64_t G, int64_t H,
                                         uint16_t *out)
{
    for (int64_t g = 0; g < G; ++g) {
        int64_t m0 = g == 0 ? 0 : group_list[g - 1];
        int64_t m1 = group_list[g];
        const float *ws = w_scale + g * H;
#pragma omp parallel for schedule(static)
        for (int64_t m = m0; m < m1; ++m) {
            for (int64_t h = 0; h < H; ++h) {
                out[m * H + h] = f32_to_bf16(((float)c[m * H + h] * ws[h]) * y_scale[m]);
            }
        }
    }
}

/* ---------------------------------------------------------------- A.10 combine
 * FDM/raw_distributed/cam_moe_distribute_combine.h:726-780 and
 * AK/moe_combine_normal/op_kernel/moe_combine_normal.h:303-338:  acc = 0; for k ascending, skipping
 * idx < 0:  acc = acc + (float(row) * w[t,k])  (rounded multiply, then rounded add); bf16_rne(acc).
 * row_of[t*K+k] is the expert-output row of slot (t,k), or < 0 to skip. */
ORACLE_API void cam_oracle_combine(const uint16_t *y, const int32_t *row_of, const float *w, int64_t T,
                                   int64_t K, int64_t H, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        float *acc = (float *)calloc((size_t)H, sizeof(float));
        for (int64_t k = 0; k < K; ++k) {
            int32_t row = row_of[t * K + k];
            if (row < 0) {
                continue;
            }
            float wk = w[t * K + k];
            const uint16_t *yr = y + (int64_t)row * H;
            for (int64_t h = 0; h < H; ++h) {
                float p = bf16_to_f32(yr[h]) * wk;
                acc[h] = acc[h] + p;
            }
        }
        for (int64_t h = 0; h < H; ++h) {
            out[t * H + h] = f32_to_bf16(acc[h]);
        }
        free(acc);
    }
}

/* ---------------------------------------------------------------- A.10b combine rows quantised for the wire
 * AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h (IsQuant instantiation).
 * A quantised row is H int8 values followed by H/8 scales in the activation type (:564, :570-571, :781):
 * blocks of 8 columns (one BlockReduceMax result per 32-byte block of fp32, :301-305, :577).
 *   quantise (:567-592):  xf = float(x);  m = max |xf| over the block;  s = m * (1/127) (:300, :579);
 *     stored scale = bf16_rne(s) (:581);  q = int8_rne(fp16_rne(xf / s)) with the UNROUNDED s (:583-589).
 *   dequantise (:755-773):  v = bf16_rne(float(q) * float(stored scale)).
 * Deliberate definitions: an all-zero block (0/0 in the reference) gives q = 0 and scale 0; Div is taken to be
 * the IEEE correctly rounded quotient ("parity unpinned" against the Ascend Div instruction bit for bit). */
static inline uint16_t f32_to_fp16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t absu = u & 0x7fffffffu;
    if (absu >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((absu > 0x7f800000u) ? 0x200u : 0u));
    }
    if (absu >= 0x477ff000u) { /* rounds to 65520 or more: overflow to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absu < 0x33000001u) { /* at most half the smallest subnormal (2^-25): rounds to zero */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(absu >> 23) - 127;
    uint32_t man = (absu & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;                                     /* bits dropped from the significand */
    uint32_t base;
    if (e < -14) { /* subnormal result: value = man * 2^(e-23), unit 2^-24 */
        shift = -e - 1;  /* (e - 23) - (-24) = e + 1 -> drop -(e+1) bits */
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t kept = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) {
        ++kept; /* a carry out of the mantissa moves into the exponent field, which is what is wanted */
    }
    return (uint16_t)(sign | (base + kept));
}

ORACLE_API uint16_t cam_oracle_f32_to_fp16(float x) { return f32_to_fp16(x); }

#define CAM_COMMQ_BLOCK 8

/* x [A,H] bits of the activation type (act: 0 bf16, 1 fp16) -> out [A, H + H/4] bytes: H int8 values, then one
 * scale of the activation type per block of 8 columns (moe_combine_shmem.h:567-592: block maximum * 1/127, kept in
 * fp32 for the division, stored rounded to ExpandXType; quotient rounded to fp16, then to int8, both to nearest even). */
ORACLE_API void cam_oracle_comm_quant_rows_act(const uint16_t *x, int64_t A, int64_t H, int act, uint8_t *out)
{
    const int64_t pitch = H + H / 4;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < A; ++r) {
        const uint16_t *xr = x + r * H;
        int8_t *q = (int8_t *)(out + r * pitch);
        uint16_t *sc = (uint16_t *)(out + r * pitch + H);
        for (int64_t b = 0; b < H / CAM_COMMQ_BLOCK; ++b) {
            float m = 0.0f;
            for (int j = 0; j < CAM_COMMQ_BLOCK; ++j) {
                uint16_t bits = xr[b * CAM_COMMQ_BLOCK + j];
                float a = fabsf(act ? fp16_to_f32(bits) : bf16_to_f32(bits));
                m = a > m ? a : m;
            }
            if (m == 0.0f) {
                sc[b] = 0;
                for (int j = 0; j < CAM_COMMQ_BLOCK; ++j) {
                    q[b * CAM_COMMQ_BLOCK + j] = 0;
                }
                continue;
            }
            float s = m * (1.0f / 127.0f);
            sc[b] = act ? f32_to_fp16(s) : f32_to_bf16(s);
            for (int j = 0; j < CAM_COMMQ_BLOCK; ++j) {
                uint16_t bits = xr[b * CAM_COMMQ_BLOCK + j];
                float v = (act ? fp16_to_f32(bits) : bf16_to_f32(bits)) / s;
                q[b * CAM_COMMQ_BLOCK + j] = (int8_t)nearbyintf(fp16_to_f32(f32_to_fp16(v)));
            }
        }
    }
}

ORACLE_API void cam_oracle_comm_quant_rows(const uint16_t *x, int64_t A, int64_t H, uint8_t *out)
{
    cam_oracle_comm_quant_rows_act(x, A, H, 0, out);
}

/* packed [A, H + H/4] -> bits of the activation type [A,H] (moe_combine_shmem.h:755-773: int8 -> fp32, times the
 * block's scale widened to fp32, rounded to ExpandXType) */
ORACLE_API void cam_oracle_comm_dequant_rows_act(const uint8_t *packed, int64_t A, int64_t H, int act, uint16_t *out)
{
    const int64_t pitch = H + H / 4;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < A; ++r) {
        const int8_t *q = (const int8_t *)(packed + r * pitch);
        const uint16_t *sc = (const uint16_t *)(packed + r * pitch + H);
        for (int64_t h = 0; h < H; ++h) {
            uint16_t sb = sc[h / CAM_COMMQ_BLOCK];
            float p = (float)q[h] * (act ? fp16_to_f32(sb) : bf16_to_f32(sb));
            out[r * H + h] = act ? f32_to_fp16(p) : f32_to_bf16(p);
        }
    }
}

ORACLE_API void cam_oracle_comm_dequant_rows(const uint8_t *packed, int64_t A, int64_t H, uint16_t *out)
{
    cam_oracle_comm_dequant_rows_act(packed, A, H, 0, out);
}

/* the same with rows and output in the activation type `act` (0 bf16, 1 fp16) */
ORACLE_API void cam_oracle_combine_act(const uint16_t *y, const int32_t *row_of, const float *w, int64_t T,
                                       int64_t K, int64_t H, int act, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        float *acc = (float *)calloc((size_t)H, sizeof(float));
        for (int64_t k = 0; k < K; ++k) {
            int32_t row = row_of[t * K + k];
            if (row < 0) {
                continue;
            }
            float wk = w[t * K + k];
            const uint16_t *yr = y + (int64_t)row * H;
            for (int64_t h = 0; h < H; ++h) {
                float p = act_to_f32(yr[h], act) * wk;
                acc[h] = acc[h] + p;
            }
        }
        for (int64_t h = 0; h < H; ++h) {
            out[t * H + h] = f32_to_act(acc[h], act);
        }
        free(acc);
    }
}

/* The combine with the shared expert's row added back (FDM/raw_distributed/cam_moe_distribute_combine.h:757-774,
 * AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:873-907): after the K routed rows, in the same fp32
 * accumulator, acc = acc + float(shared[t]) -- un-weighted, one rounded add -- and only then the rounding to the
 * activation type.  shared is [T,H] in the activation type, or NULL for the plain combine. */
ORACLE_API void cam_oracle_combine_shared(const uint16_t *y, const int32_t *row_of, const float *w,
                                          const uint16_t *shared, int64_t T, int64_t K, int64_t H, int act,
                                          uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t) {
        float *acc = (float *)calloc((size_t)H, sizeof(float));
        for (int64_t k = 0; k < K; ++k) {
            int32_t row = row_of[t * K + k];
            if (row < 0) {
                continue;
            }
            float wk = w[t * K + k];
            const uint16_t *yr = y + (int64_t)row * H;
            for (int64_t h = 0; h < H; ++h) {
                float p = act_to_f32(yr[h], act) * wk;
                acc[h] = acc[h] + p;
            }
        }
        if (shared) {
            for (int64_t h = 0; h < H; ++h) {
                acc[h] = acc[h] + act_to_f32(shared[t * H + h], act);
            }
        }
        for (int64_t h = 0; h < H; ++h) {
            out[t * H + h] = f32_to_act(acc[h], act);
        }
        free(acc);
    }
}

/* ---------------------------------------------------------------- the SHMEM operator pair on one rank
 * Dispatch: AK/moe_dispatch_shmem/op_kernel/moe_dispatch_shmem.h.
 *   send side (:492-549): entry i = t*K + k goes to expert e = expertIds[i]; its place inside the expert is
 *     expertCount(i), the number of earlier flat entries with the same id, which is also what expandIdx[i]
 *     reports (:541-548); rows are quantised per COPY, not per token, because the optional smooth scale is the
 *     destination expert's (:693-733): xf = float(x) * smooth[e][h] (one rounded multiply), m = max |xf|,
 *     s = 127 / m (no epsilon, :720), q = int8(rint(xf * s)), stored scale = 1 / s.  An all-zero row is
 *     defined as q = 0, scale 0 (0 * inf in the reference).
 *   receive side (:840-933): rows in (local expert, source rank) order, epRecvCount = inclusive running
 *     total in that order (:853-856,:927-931); with one rank that is the inclusive prefix sum of the counts.
 *   expertTokenNums (:1022-1051): type 0 = running total through each local expert, type 1 = per expert.
 * quant: 0 copies the 16-bit rows (smooth is ignored, as in the reference's non-quantising instantiation),
 * 2 quantises.  act: 0 bf16, 1 fp16.  Ids outside [0,E) name no expert: no row, expandIdx -1.
 * Returns the number of rows written. */
ORACLE_API int64_t cam_oracle_dispatch_shmem(const uint16_t *x, const int32_t *ids, const float *smooth,
                                             int64_t T, int64_t K, int64_t H, int64_t E, int quant, int act,
                                             int token_nums_type, void *out, float *scales,
                                             int32_t *expand_idx, int64_t *expert_token_nums,
                                             int32_t *ep_recv_count)
{
    int32_t *cnt = (int32_t *)calloc((size_t)E, 4);
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = ids[i];
        if (e < 0 || e >= E) {
            expand_idx[i] = -1;
            continue;
        }
        expand_idx[i] = cnt[e];
        cnt[e] += 1;
    }
    int64_t run = 0;
    for (int64_t e = 0; e < E; ++e) {
        run += cnt[e];
        ep_recv_count[e] = (int32_t)run;
        expert_token_nums[e] = token_nums_type == 0 ? run : (int64_t)cnt[e];
    }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = ids[i];
        if (e < 0 || e >= E) {
            continue;
        }
        const uint16_t *xr = x + (i / K) * H;
        int64_t row = (e == 0 ? 0 : ep_recv_count[e - 1]) + expand_idx[i];
        if (quant == 0) {
            memcpy((uint16_t *)out + row * H, xr, (size_t)H * 2);
            continue;
        }
        int8_t *q = (int8_t *)out + row * H;
        const float *sm = smooth ? smooth + e * H : NULL;
        float m = 0.0f;
        for (int64_t h = 0; h < H; ++h) {
            float v = act_to_f32(xr[h], act);
            if (sm) {
                v = v * sm[h];
            }
            float a = fabsf(v);
            m = a > m ? a : m;
        }
        if (m == 0.0f) {
            memset(q, 0, (size_t)H);
            scales[row] = 0.0f;
            continue;
        }
        float s = 127.0f / m;
        for (int64_t h = 0; h < H; ++h) {
            float v = act_to_f32(xr[h], act);
            if (sm) {
                v = v * sm[h];
            }
            q[h] = (int8_t)(int32_t)nearbyintf(v * s);
        }
        scales[row] = 1.0f / s;
    }
    free(cnt);
    return run;
}

/* Combine: AK/moe_combine_shmem/op_kernel/moe_combine_shmem.h:775-917 on one rank.  The row of slot (t,k) is
 * found from the dispatch's outputs: rows of expert e start at epSendCounts[e-1] (:514-556 walks the same
 * running totals) and the slot's place inside them is expandIdx[t*K+k] (:833-837).  comm_quant != 0 passes every
 * row through the int8 wire format on its way (quantise :567-592, dequantise :755-773) before it is weighted;
 * then acc = acc + float(row) * w[t,k] for k ascending, and one rounding to the activation type (:908-912).
 * Ids outside [0,E) are skipped (the reference does not guard them). */
ORACLE_API void cam_oracle_combine_shmem(const uint16_t *expand_x, const int32_t *ids, const int32_t *expand_idx,
                                         const int32_t *ep_send_counts, const float *w, int64_t A, int64_t T,
                                         int64_t K, int64_t H, int64_t E, int act, int comm_quant, uint16_t *out)
{
    int32_t *row_of = (int32_t *)malloc((size_t)(T * K > 0 ? T * K : 1) * 4);
    for (int64_t i = 0; i < T * K; ++i) {
        int64_t e = ids[i];
        int64_t row = -1;
        if (e >= 0 && e < E) {
            row = (e == 0 ? 0 : ep_send_counts[e - 1]) + expand_idx[i];
            if (row < 0 || row >= A) {
                row = -1;
            }
        }
        row_of[i] = (int32_t)row;
    }
    if (comm_quant) {
        uint8_t *wire = (uint8_t *)malloc((size_t)(A > 0 ? A : 1) * (size_t)(H + H / 4));
        uint16_t *rows = (uint16_t *)malloc((size_t)(A > 0 ? A : 1) * (size_t)H * 2);
        cam_oracle_comm_quant_rows_act(expand_x, A, H, act, wire);
        cam_oracle_comm_dequant_rows_act(wire, A, H, act, rows);
        cam_oracle_combine_shared(rows, row_of, w, NULL, T, K, H, act, out);
        free(wire);
        free(rows);
    } else {
        cam_oracle_combine_shared(expand_x, row_of, w, NULL, T, K, H, act, out);
    }
    free(row_of);
}

/* row_of for the fused op: off[e] + pos (cam_moe_distribute_combine.h:737-742), -1 where idx < 0. */
ORACLE_API void cam_oracle_rows_from_pos(const int64_t *idx, const int32_t *off, const int32_t *pos,
                                         int64_t n, int64_t E, int32_t *row_of)
{
    for (int64_t i = 0; i < n; ++i) {
        int64_t e = idx[i];
        row_of[i] = (e < 0 || e >= E) ? -1 : off[e] + pos[i];
    }
}

/* row_of for the "normal" op: invert the (srcRank, token, k) triples each row carries
 * (moe_combine_normal.h:232-238: row r goes to slot token*K + k of its source rank). */
ORACLE_API void cam_oracle_rows_from_src_info(const int32_t *src_info, int64_t A, int64_t T, int64_t K,
                                              int32_t *row_of)
{
    for (int64_t i = 0; i < T * K; ++i) {
        row_of[i] = -1;
    }
    for (int64_t r = 0; r < A; ++r) {
        int64_t t = src_info[3 * r + 1];
        int64_t k = src_info[3 * r + 2];
        if (t >= 0 && t < T && k >= 0 && k < K) {
            row_of[t * K + k] = (int32_t)r;
        }
    }
}

/* ---------------------------------------------------------------- the whole layer, one rank
 * Composition of AK/fused_deep_moe/op_kernel/fused_deep_moe.h:346-440 for epRankSize == 1:
 * counts -> offsets -> ranks -> Q2 permute -> GMM1 -> dequant+SiLU -> product+requant -> GMM2 ->
 * dequant -> combine.  n_active tokens (x_active_mask prefix semantics,
 * …swiglu_quant_multistage_workspace.h:647-678); output rows >= n_active are zero.
 * w1 is [E, H, 2I], w2 is [E, I, H].  Optional debug outputs may be NULL. */
ORACLE_API int cam_oracle_fused_layer(const uint16_t *x, const int64_t *idx, const float *topk_w,
                                      const int8_t *w1, const float *w1_scale, const int8_t *w2,
                                      const float *w2_scale, int64_t T, int64_t n_active, int64_t K,
                                      int64_t H, int64_t I, int64_t E, uint16_t *out,
                                      int64_t *expert_token_nums, int8_t *dbg_x1, float *dbg_x1_scale,
                                      int8_t *dbg_x2, float *dbg_x2_scale, uint16_t *dbg_y)
{
    int64_t Ta = n_active;
    int64_t A = Ta * K;
    int32_t *cnt = (int32_t *)calloc((size_t)E, 4);
    int32_t *off = (int32_t *)calloc((size_t)E, 4);
    int32_t per_rank = 0;
    uint8_t *in_rank = (uint8_t *)calloc((size_t)(Ta > 0 ? Ta : 1), 1);
    if (cam_oracle_layout(idx, Ta, K, E, 1, 0, cnt, &per_rank, in_rank) != 0) {
        free(cnt);
        free(off);
        free(in_rank);
        return -1;
    }
    cam_oracle_offsets(cnt, E, (int32_t)Ta, off, NULL);
    int64_t *gl = (int64_t *)calloc((size_t)E, 8);
    int64_t run = 0;
    for (int64_t e = 0; e < E; ++e) {
        run += cnt[e];
        gl[e] = run;
        expert_token_nums[e] = cnt[e];
    }
    int64_t rows = run;
    size_t ra = (size_t)(A > 0 ? A : 1);
    int32_t *pos = (int32_t *)malloc(ra * 4);
    int32_t *row_of = (int32_t *)malloc(ra * 4);
    cam_oracle_send_token_idx(idx, Ta, K, E, pos);
    cam_oracle_rows_from_pos(idx, off, pos, A, E, row_of);
    int8_t *x1 = (int8_t *)malloc(ra * (size_t)H);
    float *x1s = (float *)malloc(ra * 4);
    cam_oracle_dispatch(x, idx, off, pos, Ta, K, H, E, 2, 0, x1, x1s, NULL);
    int32_t *c1 = (int32_t *)malloc(ra * (size_t)(2 * I) * 4);
    cam_oracle_gmm_int32(x1, w1, gl, E, H, 2 * I, c1);
    float *d = (float *)malloc(ra * (size_t)(2 * I) * 4);
    cam_oracle_gmm1_epilogue(c1, w1_scale, x1s, gl, E, I, d);
    int8_t *x2 = (int8_t *)malloc(ra * (size_t)I);
    float *x2s = (float *)malloc(ra * 4);
    cam_oracle_swiglu_quant(d, rows, I, x2, x2s);
    int32_t *c2 = (int32_t *)malloc(ra * (size_t)H * 4);
    cam_oracle_gmm_int32(x2, w2, gl, E, I, H, c2);
    uint16_t *y = (uint16_t *)malloc(ra * (size_t)H * 2);
    cam_oracle_gmm2_epilogue(c2, w2_scale, x2s, gl, E, H, y);
    memset(out, 0, (size_t)(T * H) * 2);
    cam_oracle_combine(y, row_of, topk_w, Ta, K, H, out);
    if (dbg_x1) memcpy(dbg_x1, x1, (size_t)rows * (size_t)H);
    if (dbg_x1_scale) memcpy(dbg_x1_scale, x1s, (size_t)rows * 4);
    if (dbg_x2) memcpy(dbg_x2, x2, (size_t)rows * (size_t)I);
    if (dbg_x2_scale) memcpy(dbg_x2_scale, x2s, (size_t)rows * 4);
    if (dbg_y) memcpy(dbg_y, y, (size_t)rows * (size_t)H * 2);
    free(cnt); free(off); free(in_rank); free(gl); free(pos); free(row_of); free(x1); free(x1s);
    free(c1); free(d); free(x2); free(x2s); free(c2); free(y);
    return 0;
}

/* ================================================================ block-scaled FP8 layer
 * No counterpart in the reference (W8A8 only, src/cam/README.md:20-21): these functions evaluate the definition
 * in include/cam_fp8_spec.h.  The matrix products accumulate in double and round once to fp32, which is what a
 * tolerance test of an fp32-accumulating kernel should be measured against. */
ORACLE_API float cam_oracle_e4m3_to_f32(uint8_t v) { return cam_e4m3_to_f32(v); }
ORACLE_API uint8_t cam_oracle_f32_to_e4m3(float x) { return cam_f32_to_e4m3(x); }
ORACLE_API int cam_oracle_fp8_block_scale_exp(float amax) { return cam_fp8_block_scale_exp(amax); }

/* x [A,H] fp32 -> q [A,H] e4m3 bytes, scale [A, H/128] e8m0 bytes.  H % 128 == 0. */
ORACLE_API void cam_oracle_fp8_quant_rows_f32(const float *x, int64_t A, int64_t H, uint8_t *q, uint8_t *scale)
{
    const int64_t nb = H / CAM_FP8_BLOCK;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < A; ++r) {
        for (int64_t b = 0; b < nb; ++b) {
            const float *xb = x + r * H + b * CAM_FP8_BLOCK;
            float m = 0.0f;
            for (int j = 0; j < CAM_FP8_BLOCK; ++j) {
                float a = fabsf(xb[j]);
                m = a > m ? a : m;
            }
            const int e = cam_fp8_block_scale_exp(m);
            scale[r * nb + b] = cam_e8m0_from_exp(e);
            /* x * 2^-e in two exact steps so that neither factor leaves the normal range */
            const float f1 = cam_exp2_int(-(e / 2)), f2 = cam_exp2_int(-(e - e / 2));
            for (int j = 0; j < CAM_FP8_BLOCK; ++j) {
                q[r * H + b * CAM_FP8_BLOCK + j] = cam_f32_to_e4m3((xb[j] * f1) * f2);
            }
        }
    }
}

/* the same from bf16 (act == 0) or fp16 (act == 1) activations */
ORACLE_API void cam_oracle_fp8_quant_rows(const uint16_t *x, int act, int64_t A, int64_t H, uint8_t *q,
                                          uint8_t *scale)
{
    float *xf = (float *)malloc((size_t)(A > 0 ? A : 1) * (size_t)H * 4);
    for (int64_t i = 0; i < A * H; ++i) {
        xf[i] = act_to_f32(x[i], act);
    }
    cam_oracle_fp8_quant_rows_f32(xf, A, H, q, scale);
    free(xf);
}

/* out[m, n] = sum_kb 2^(sa[m,kb] + sw[g,kb,n/128] - 254) * sum_{k in kb} a[m,k] * w[g,k,n]   (double, then fp32)
 * a [A,K] e4m3, sa [A,K/128] e8m0, w [G,K,N] e4m3 row-major, sw [G,K/128,N/128] e8m0, group_list cumulative. */
ORACLE_API void cam_oracle_fp8_gemm(const uint8_t *a, const uint8_t *sa, const uint8_t *w, const uint8_t *sw,
                                    const int64_t *group_list, int64_t G, int64_t K, int64_t N, float *out)
{
    float lut[256];
    for (int i = 0; i < 256; ++i) {
        lut[i] = cam_e4m3_to_f32((uint8_t)i);
    }
    const int64_t kb_n = K / CAM_FP8_BLOCK, nb_n = N / CAM_FP8_BLOCK;
    for (int64_t g = 0; g < G; ++g) {
        const int64_t m0 = g == 0 ? 0 : group_list[g - 1], m1 = group_list[g];
        const uint8_t *wg = w + g * K * N;
        const uint8_t *swg = sw + g * kb_n * nb_n;
#pragma omp parallel for schedule(dynamic, 4)
        for (int64_t m = m0; m < m1; ++m) {
            double *acc = (double *)calloc((size_t)N, sizeof(double));
            double *part = (double *)malloc((size_t)N * sizeof(double));
            for (int64_t kb = 0; kb < kb_n; ++kb) {
                memset(part, 0, (size_t)N * sizeof(double));
                for (int64_t k = kb * CAM_FP8_BLOCK; k < (kb + 1) * CAM_FP8_BLOCK; ++k) {
                    const double av = lut[a[m * K + k]];
                    if (av == 0.0) {
                        continue;
                    }
                    const uint8_t *wr = wg + k * N;
                    for (int64_t n = 0; n < N; ++n) {
                        part[n] += av * (double)lut[wr[n]];
                    }
                }
                const int ea = (int)sa[m * kb_n + kb] - 127;
                for (int64_t n = 0; n < N; ++n) {
                    const int eb = (int)swg[kb * nb_n + n / CAM_FP8_BLOCK] - 127;
                    acc[n] += ldexp(part[n], ea + eb);
                }
            }
            for (int64_t n = 0; n < N; ++n) {
                out[m * N + n] = (float)acc[n];
            }
            free(acc);
            free(part);
        }
    }
}

/* y[m, i] = silu(c[m, i]) * c[m, I + i]: gate = columns [0, I), up = [I, 2I), as in the int8 layer
 * (FDM/epilogue/block/block_epilogue_per_token_dequant_swiglu.h:178, :253-264). */
ORACLE_API void cam_oracle_fp8_swiglu(const float *c, int64_t M, int64_t I, float *y)
{
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t i = 0; i < I; ++i) {
            y[m * I + i] = cam_silu_spec(c[m * 2 * I + i]) * c[m * 2 * I + I + i];
        }
    }
}

ORACLE_API void cam_oracle_f32_rows_to_bf16(const float *x, int64_t n, uint16_t *out)
{
    for (int64_t i = 0; i < n; ++i) {
        out[i] = f32_to_bf16(x[i]);
    }
}
