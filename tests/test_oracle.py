"""Pins the CPU oracle against closed forms, brute-force definitions and library routines.

The reference holds no golden vectors for this path and cannot be built or imported here, so every
oracle function is checked against what the mathematics fixes, with cases chosen so that a plausible
mistake (dropped epsilon, swapped halves, wrong scale order, fused multiply-add, wrong rounding) fails.
"""
import math

import numpy as np
import pytest
import torch

from umdk_original_amd import synth


def _rng(seed):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------ layout / offsets / ranks
@pytest.mark.parametrize("T,K,E,R", [(1, 1, 1, 1), (17, 3, 8, 2), (128, 8, 256, 8), (33, 16, 48, 48), (64, 2, 8, 1)])
def test_layout_matches_bincount_and_set_logic(oracle, T, K, E, R):
    rng = _rng(T * 1000 + E)
    idx = rng.integers(-1, E, size=(T, K)).astype(np.int64)  # -1 entries are skipped
    per_rank, cnt, in_rank = oracle.layout(idx, E, R)
    valid = idx[idx >= 0]
    assert np.array_equal(cnt, np.bincount(valid, minlength=E).astype(np.int32))
    epr = E // R
    want = np.zeros((T, R), bool)
    for t in range(T):
        for e in idx[t]:
            if e >= 0:
                want[t, e // epr] = True
    assert np.array_equal(in_rank, want)
    assert np.array_equal(per_rank, want.sum(0).astype(np.int32))


def test_layout_duplicate_expert_counts_rank_once(oracle):
    idx = np.array([[3, 3, 3, 1]], np.int64)
    per_rank, cnt, in_rank = oracle.layout(idx, 4, 2)
    assert cnt.tolist() == [0, 1, 0, 3]
    assert per_rank.tolist() == [1, 1]  # token counted once per rank although three ids hit rank 1
    assert in_rank.tolist() == [[True, True]]


def test_layout_rejects_out_of_range(oracle):
    with pytest.raises(ValueError):
        oracle.layout(np.array([[0, 8]], np.int64), 8, 1)


def test_layout_can_skip_out_of_range_ids(oracle):
    """The skipping mode equals the strict mode run on the same ids with the out-of-range ones set to -1."""
    rng = _rng(77)
    idx = rng.integers(-2, 12, size=(50, 4)).astype(np.int64)  # E = 8: ids 8..11 are out of range
    got = oracle.layout(idx, 8, 2, skip_out_of_range=True)
    want = oracle.layout(np.where(idx >= 8, -1, idx), 8, 2)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    assert got[1].sum() == ((idx >= 0) & (idx < 8)).sum() == np.bincount(idx[(idx >= 0) & (idx < 8)], minlength=8).sum()
    pos = oracle.send_token_idx(idx, 8)
    assert ((pos == -1) == ((idx < 0) | (idx >= 8))).all()


def test_fp16_conversion_matches_numpy_on_every_pattern(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.fp16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp16_quant_rows_follow_the_float32_definition(oracle):
    """Same arithmetic as the bf16 rows, on exactly converted fp16 inputs."""
    rng = _rng(5)
    x = (rng.standard_normal((9, 256)) * 3).astype(np.float16)
    x[3] = 0
    for variant in (1, 2):
        q, s = oracle.quant_rows(x.view(np.uint16), variant, fp16=True)
        xf = x.astype(np.float32)
        m = np.abs(xf).max(axis=1)
        with np.errstate(divide="ignore", invalid="ignore"):
            sc = np.float32(127.0) / (m + np.float32(1e-12)) if variant == 1 else np.float32(127.0) / m
        want_q = np.rint(xf * sc[:, None].astype(np.float32)).astype(np.float32)
        want_s = (np.float32(1.0) / sc).astype(np.float32)
        if variant == 2:
            want_q[3] = 0
            want_s[3] = 0
        assert np.array_equal(q.astype(np.float32), want_q)
        assert np.array_equal(s.view(np.uint32), want_s.view(np.uint32))


def test_offsets_are_exclusive_cumsum_with_triplets(oracle):
    cnt = _rng(1).integers(0, 50, size=37).astype(np.int32)
    off, trip = oracle.offsets(cnt, 99)
    want = np.concatenate([[0], np.cumsum(cnt)[:-1]]).astype(np.int32)
    assert np.array_equal(off, want)
    assert np.array_equal(trip.reshape(-1, 3)[:, 0], cnt)
    assert np.array_equal(trip.reshape(-1, 3)[:, 1], want)
    assert (trip.reshape(-1, 3)[:, 2] == 99).all()


def test_send_token_idx_brute_force_definition(oracle):
    rng = _rng(2)
    idx = rng.integers(-1, 5, size=(23, 4)).astype(np.int64)
    pos = oracle.send_token_idx(idx, 5).reshape(-1)
    flat = idx.reshape(-1)
    for i, e in enumerate(flat):
        if e < 0:
            assert pos[i] == -1
        else:
            assert pos[i] == sum(1 for j in range(i) if flat[j] == e)


@pytest.mark.parametrize("T,K,E", [(4096, 8, 256), (777, 6, 64)])
def test_permutation_is_the_stable_sort_by_expert(oracle, T, K, E):
    ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=44)
    idx = ids.numpy()
    _, cnt, _ = oracle.layout(idx, E, 1)
    off, _ = oracle.offsets(cnt, T)
    pos = oracle.send_token_idx(idx, E)
    row = oracle.rows_from_pos(idx, off, pos, E).reshape(-1)
    order = np.argsort(idx.reshape(-1), kind="stable")
    # entry order[p] must land on row p
    assert np.array_equal(row[order], np.arange(T * K, dtype=np.int32))
    # bijection onto [0, A)
    assert np.array_equal(np.sort(row), np.arange(T * K))


def test_recv_bookkeeping_one_rank_closed_form(oracle):
    cnt = _rng(3).integers(0, 9, size=16).astype(np.int32)
    off, trip = oracle.offsets(cnt, 40)
    total, rc, ro, tpe, mx = oracle.recv_bookkeeping(trip, 1, 16)
    assert total == cnt.sum()
    assert np.array_equal(rc, np.cumsum(cnt).astype(np.int32))
    assert np.array_equal(ro, off)
    assert np.array_equal(tpe, cnt.astype(np.int64))
    assert mx == 40


def test_recv_bookkeeping_two_ranks_hand_example(oracle):
    # rank "me" owns 2 local experts; source ranks 0 and 1 send (count, offset, bs):
    #   src0: le0 (3, 10, 7)  le1 (0, 13, 7)      src1: le0 (2, 0, 5)   le1 (4, 2, 5)
    recv = np.array([3, 10, 7, 0, 13, 7, 2, 0, 5, 4, 2, 5], np.int32)
    total, rc, ro, tpe, mx = oracle.recv_bookkeeping(recv, 2, 2)
    # order (le0,s0) (le0,s1) (le1,s0) (le1,s1): counts 3,2,0,4 -> inclusive cumsum 3,5,5,9
    assert rc.tolist() == [3, 5, 5, 9]
    assert ro.tolist() == [10, 0, 13, 2]
    assert tpe.tolist() == [5, 4]
    assert total == 9 and mx == 7


# ------------------------------------------------------------------ bf16 rounding
def test_bf16_rounding_matches_torch(oracle):
    x = torch.randn(20000, generator=torch.Generator().manual_seed(5)) * 100
    x[:8] = torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895313892515355e38, 65504.0, 1e-40])
    got = oracle.f32_to_bf16_bits(x.numpy())
    want = synth.bf16_bits(x.bfloat16())
    assert np.array_equal(got, want)
    one = np.array([oracle.lib().cam_oracle_f32_to_bf16(float(v)) for v in x[:64].tolist()], np.uint16)
    assert np.array_equal(one, want[:64])


# ------------------------------------------------------------------ token quantisation
def _quant_ref_f32(xf, variant):
    """Vectorised float32 restatement used as an independent implementation (numpy, not C)."""
    m = np.max(np.abs(xf), axis=1).astype(np.float32)
    if variant == 1:
        s = np.float32(127.0) / (m + np.float32(1e-12))
    else:
        with np.errstate(divide="ignore"):
            s = np.float32(127.0) / m
    q = np.rint(xf * s[:, None]).astype(np.int32)
    inv = np.float32(1.0) / s
    if variant == 2:
        zero = m == 0
        q[zero] = 0
        inv[zero] = 0
    return q.astype(np.int8), inv.astype(np.float32)


@pytest.mark.parametrize("variant", [1, 2])
def test_quant_invariants_and_numpy_cross_check(oracle, variant):
    x = synth.normal_bf16(257, 1024, seed=6)
    bits = synth.bf16_bits(x)
    q, s = oracle.quant_rows(bits, variant)
    xf = x.float().numpy()
    q_np, s_np = _quant_ref_f32(xf, variant)
    assert np.array_equal(q, q_np)
    assert np.array_equal(s.view(np.uint32), s_np.view(np.uint32))
    assert (np.abs(q.astype(np.int32)).max(axis=1) == 127).all()
    # reconstruction error bounded by half a step
    err = np.abs(xf - q.astype(np.float32) * s[:, None])
    assert (err <= s[:, None] * 0.5 * (1 + 1e-4)).all()
    # against exact arithmetic: scale_out ~ max/127 and q ~ rint(x*127/max) up to rare ties
    m = np.abs(xf.astype(np.float64)).max(axis=1)
    assert np.allclose(s, m / 127.0, rtol=3e-7)
    q64 = np.rint(xf.astype(np.float64) * 127.0 / m[:, None])
    assert (q64 != q).mean() < 1e-3 and np.abs(q64 - q).max() <= 1


def test_quant_special_rows(oracle):
    H = 64
    rows = np.zeros((5, H), np.float32)
    rows[0] = 3.0 * np.where(np.arange(H) % 2 == 0, 1, -1)  # equal magnitudes -> all +-127
    rows[1] = 2.0 ** -(np.arange(H) % 7)                      # powers of two: 127 * 2^-j
    rows[2] = 0.0                                             # all-zero row
    rows[3, 0] = 1e-13                                        # the epsilon matters here
    rows[4] = np.linspace(-1, 1, H)
    bits = synth.bf16_bits(torch.from_numpy(rows).bfloat16())
    xf = oracle.bf16_bits_to_f32(bits)
    for variant in (1, 2):
        q, s = oracle.quant_rows(bits, variant)
        assert (np.abs(q[0]) == 127).all() and (np.sign(q[0]) == np.sign(rows[0])).all()
        assert np.array_equal(q[1], np.rint(127.0 * xf[1].astype(np.float64)).astype(np.int8))
        assert (q[2] == 0).all()
    q1, s1 = oracle.quant_rows(bits, 1)
    q2, s2 = oracle.quant_rows(bits, 2)
    # zero row: variant 1 keeps the reference's finite scale 1/(127/1e-12); variant 2 is defined as 0
    assert s1[2] == np.float32(1.0) / (np.float32(127.0) / np.float32(1e-12)) and s2[2] == 0.0
    # tiny row: with the epsilon the maximum maps to 127*m/(m+1e-12), without it to exactly 127
    m = float(xf[3, 0])
    assert q1[3, 0] == int(np.rint(127.0 * m / (m + 1e-12))) and q1[3, 0] < 127
    assert q2[3, 0] == 127
    # ordinary rows: both variants agree bit for bit (epsilon vanishes in float32)
    assert np.array_equal(q1[4], q2[4]) and s1[4] == s2[4]


def test_dispatch_rows_and_triples(oracle):
    T, K, E, H = 50, 4, 8, 64
    ids, _ = synth.softmax_topk_routing(T, E, K, seed=7)
    idx = ids.numpy().copy()
    idx[3, 1] = -1
    x = synth.normal_bf16(T, H, seed=8)
    bits = synth.bf16_bits(x)
    _, cnt, _ = oracle.layout(idx, E, 1)
    off, _ = oracle.offsets(cnt, T)
    pos = oracle.send_token_idx(idx, E)
    total = int(cnt.sum())
    assert total == T * K - 1
    out, scales, src = oracle.dispatch(bits, idx, off, pos, E, 0, total)
    src = src.reshape(-1, 3)
    for r in range(total):
        _, t, k = src[r]
        assert idx[t, k] >= 0 and off[idx[t, k]] + pos[t, k] == r
        assert np.array_equal(out[r], bits[t])
    outq, sq, _ = oracle.dispatch(bits, idx, off, pos, E, 1, total)
    q_all, s_all = oracle.quant_rows(bits, 1)
    for r in range(total):
        t = src[r, 1]
        assert np.array_equal(outq[r], q_all[t]) and sq[r] == s_all[t]
    # rows of one expert are contiguous and in ascending flat order
    flat = (src[:, 1] * K + src[:, 2])
    experts = idx.reshape(-1)[flat]
    assert (np.diff(experts) >= 0).all()
    for e in range(E):
        assert (np.diff(flat[experts == e]) > 0).all()


# ------------------------------------------------------------------ GEMM and epilogues
def test_gmm_int32_matches_int64_matmul(oracle):
    rng = _rng(9)
    G, Kd, N = 5, 96, 40
    sizes = np.array([7, 0, 13, 1, 4])
    gl = np.cumsum(sizes).astype(np.int64)
    a = rng.integers(-128, 128, size=(int(gl[-1]), Kd)).astype(np.int8)
    w = rng.integers(-128, 128, size=(G, Kd, N)).astype(np.int8)
    c = oracle.gmm_int32(a, w, gl)
    m0 = 0
    for g in range(G):
        want = a[m0:gl[g]].astype(np.int64) @ w[g].astype(np.int64)
        assert np.array_equal(c[m0:gl[g]], want.astype(np.int32))
        m0 = gl[g]


def test_gmm_int32_extreme_values_do_not_overflow(oracle):
    Kd = 7168
    a = np.full((1, Kd), -128, np.int8)
    w = np.full((1, Kd, 2), -128, np.int8)
    c = oracle.gmm_int32(a, w, np.array([1], np.int64))
    assert c[0, 0] == Kd * 128 * 128 and c[0, 0] < 2 ** 31


def test_expf_spec_accuracy_and_edges(oracle):
    xs = np.concatenate([np.linspace(-87.0, 88.0, 40001), _rng(10).normal(0, 5, 20000)]).astype(np.float32)
    got = np.array([oracle.expf(float(v)) for v in xs], np.float64)
    want = np.exp(xs.astype(np.float64))
    rel = np.abs(got - want) / want
    assert rel.max() < 2.5e-7, rel.max()  # about 2 ulp of float32
    assert oracle.expf(0.0) == 1.0
    assert oracle.expf(-200.0) == 0.0 and math.isinf(oracle.expf(100.0))
    assert math.isnan(oracle.expf(float("nan")))
    mono = np.array([oracle.expf(float(v)) for v in np.linspace(-3, 3, 5001, dtype=np.float32)])
    assert (np.diff(mono) >= 0).all()


def test_expf_scaling_by_two_multiplies_equals_ldexp():
    """The exp specification scales y in [0.7, 1.5] by 2^n with two power-of-two multiplies; the device code uses one
    ldexp instead.  Both round y * 2^n once, to nearest even: identical bits for every n the specification can
    produce (-150 .. 128), subnormal results, zero and infinity included."""
    rng = _rng(123)
    y = np.concatenate([rng.uniform(0.70, 1.42, 200000), [0.70710677, 1.0, 1.4142135, 1.0000001, 1.5]]).astype(np.float32)
    with np.errstate(over="ignore", under="ignore"):
        for n in range(-150, 129):
            n1 = int(n / 2)  # C division truncates toward zero
            n2 = n - n1
            s1 = np.float32(2.0) ** np.float32(n1)
            s2 = np.float32(2.0) ** np.float32(n2)
            two_step = (y * s1) * s2
            one_step = np.ldexp(y, n).astype(np.float32)
            assert two_step.dtype == np.float32
            assert np.array_equal(two_step.view(np.uint32), one_step.view(np.uint32)), n


def _silu64(t):
    t = np.asarray(t, np.float64)
    with np.errstate(over="ignore"):
        return t / (1.0 + np.exp(-t))


def test_silu_spec_accuracy_against_float64(oracle):
    """The bounds the specification states (include/cam_expf_spec.h): 6e-6 relative for |t| <= 20, 1.2e-5 for
    |t| <= 86, below 4e-36 absolute beyond; exact at 0 and at +inf."""
    rng = _rng(11)
    ts = np.concatenate([np.linspace(-86, 86, 60001), rng.normal(0, 4, 30000), rng.uniform(-20, 20, 30000),
                         [2.0 ** -k for k in range(0, 140, 3)], [-(2.0 ** -k) for k in range(0, 140, 3)]]).astype(np.float32)
    got = np.array([oracle.silu(float(t)) for t in ts], np.float64)
    want = _silu64(ts)
    err = np.abs(got - want)
    near = np.abs(ts) <= 20
    assert (err[near] <= 6e-6 * np.abs(want[near]) + 1e-45).all(), (err[near] / np.abs(want[near]).clip(1e-300)).max()
    assert (err <= 1.2e-5 * np.abs(want) + 1e-45).all(), (err / np.abs(want).clip(1e-300)).max()
    far = np.array([87.0, 100.0, 1e4, 1e30, 3e38], np.float32)
    for t in far:
        assert oracle.silu(float(t)) == float(t)                       # t - 86 q with q ~ 4e-38
        assert abs(oracle.silu(-float(t)) - _silu64(-float(t))) < 4e-36
    assert oracle.silu(0.0) == 0.0 and oracle.silu(-0.0) == 0.0
    assert math.isinf(oracle.silu(float("inf"))) and oracle.silu(float("inf")) > 0
    assert abs(oracle.silu(float("-inf"))) < 4e-36
    # silu(t) - silu(-t) == t up to the roundings of the two results
    pos = np.abs(ts[:60001:7])
    d = np.array([oracle.silu(float(t)) - oracle.silu(-float(t)) for t in pos])
    assert np.allclose(d, pos, rtol=3e-7, atol=1e-37)


def _round_f32(fr):
    """Correctly rounded (nearest, ties to even) binary32 value of an exact Fraction, as np.float32 (normal range)."""
    from fractions import Fraction
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = fr.numerator.bit_length() - fr.denominator.bit_length()
    if Fraction(2) ** e > fr:
        e -= 1
    assert -126 <= e <= 127, e                      # the specification never leaves the normal range
    scaled = fr / Fraction(2) ** (e - 23)           # in [2^23, 2^24)
    m = scaled.numerator // scaled.denominator
    rem = scaled - m
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and m % 2 == 1):
        m += 1
    return np.float32(sign * float(m) * 2.0 ** (e - 23))   # m <= 2^24 and the power are exact in a double


def test_silu_spec_is_the_written_operation_sequence_bit_for_bit(oracle):
    """An independent restatement in exact rational arithmetic, every written operation rounded to binary32 once
    (a fused multiply-add is ONE rounding of a*b + c).  It fails if the C build splits a fused operation, fuses a
    split one, evaluates the polynomial in another order or scales by the power of two inexactly."""
    from fractions import Fraction as F

    def fr(v):
        return F(float(v))

    def fma(a, b, c):
        return _round_f32(fr(a) * fr(b) + fr(c))

    def spec(t):
        t = np.float32(t)
        a = np.float32(min(abs(float(t)), 86.0))
        z = _round_f32(fr(a) * fr(np.float32(-1.44269504088896341)))
        n = np.float32(np.rint(z))
        f = _round_f32(fr(z) - fr(n))
        p = fma(f, np.float32(9.570102e-3), np.float32(5.591786e-2))
        p = fma(f, p, np.float32(2.4024744e-1))
        p = fma(f, p, np.float32(6.931218e-1))
        p = fma(f, p, np.float32(9.999993e-1))
        e = _round_f32(fr(p) * F(2) ** int(n))
        d = _round_f32(fr(e) + 1)
        r = fma(d, np.float32(3.2323232e-1), np.float32(-1.4545455))
        r = fma(d, r, np.float32(2.121212))
        u = fma(-d, r, np.float32(1.0))
        r = fma(fma(u, u, u), r, r)
        q = _round_f32(fr(e) * fr(r))
        return fma(-a, q, np.float32(max(float(t), 0.0)))

    rng = _rng(12)
    ts = np.concatenate([rng.normal(0, 3, 1500), rng.uniform(-90, 90, 600), [0.5, -0.5, 1.0, -1.0, 86.0, -86.0, 1e-20, 20.0, -20.0],
                         np.float32(np.arange(-40, 41)) * np.float32(0.6931472)]).astype(np.float32)
    for t in ts:
        got, want = np.float32(oracle.silu(float(t))), spec(t)
        assert got.view(np.uint32) == want.view(np.uint32), (float(t), float(got), float(want))


def test_gmm1_epilogue_halves_scale_order_and_grouping(oracle):
    rng = _rng(12)
    G, I = 3, 8
    sizes = np.array([4, 0, 5])
    gl = np.cumsum(sizes).astype(np.int64)
    M = int(gl[-1])
    c = rng.integers(-2 ** 20, 2 ** 20, size=(M, 2 * I)).astype(np.int32)
    ws = rng.uniform(0.0015, 0.0045, size=(G, 2 * I)).astype(np.float32)
    xs = rng.uniform(0.01, 0.05, size=M).astype(np.float32)
    d = oracle.gmm1_epilogue(c, ws, xs, gl)
    grp = np.repeat(np.arange(G), sizes)
    t32 = (c.astype(np.float32) * ws[grp]) * xs[:, None]  # weight scale first, then token scale
    # right half is the dequantised value itself, bit for bit
    assert np.array_equal(d[:, I:].view(np.uint32), t32[:, I:].view(np.uint32))
    # the other association differs somewhere, so the order is really pinned
    t_other = c.astype(np.float32) * (ws[grp] * xs[:, None])
    assert not np.array_equal(t_other[:, I:].view(np.uint32), t32[:, I:].view(np.uint32))
    # left half is SiLU of the dequantised value
    t64 = t32[:, :I].astype(np.float64)
    # (the specified SiLU is within 1.2e-5 relative of the exact one over this range; its own tests pin that)
    assert np.allclose(d[:, :I], t64 / (1 + np.exp(-t64)), rtol=1.5e-5, atol=1e-30)
    assert not np.allclose(d[:, :I], t32[:, :I])  # and not the identity


def test_swiglu_quant_definition(oracle):
    rng = _rng(13)
    M, I = 9, 64
    d = rng.normal(0, 3, size=(M, 2 * I)).astype(np.float32)
    d[4] = 0.0
    q, s = oracle.swiglu_quant(d)
    y = d[:, :I] * d[:, I:]
    m = np.abs(y).max(axis=1)
    inv127 = np.float32(1.0) / np.float32(127.0)
    want_s = (m * inv127).astype(np.float32)
    want_s[4] = 0
    assert np.array_equal(s.view(np.uint32), want_s.view(np.uint32))
    with np.errstate(divide="ignore", invalid="ignore"):
        rcp = np.float32(1.0) / m
        want_q = np.rint((y * np.float32(127.0)) * rcp[:, None])
    want_q[4] = 0
    assert np.array_equal(q, want_q.astype(np.int8))
    assert (q[4] == 0).all()
    live = [i for i in range(M) if i != 4]
    assert (np.abs(q[live].astype(int)).max(axis=1) == 127).all()
    # gate*up really is left*right: swapping in a wrong pairing changes the result
    assert not np.array_equal(y, d[:, :I] * d[:, :I])
    # m * (1/127) is not always m / 127: the constant is rounded first
    mm = np.float32(1.0) + np.arange(1, 4000, dtype=np.float32) * np.float32(1e-3)
    assert (mm * inv127 != mm / np.float32(127.0)).any()


def test_gmm2_epilogue_bits(oracle):
    rng = _rng(14)
    G, H = 2, 16
    gl = np.array([3, 7], np.int64)
    c = rng.integers(-2 ** 22, 2 ** 22, size=(7, H)).astype(np.int32)
    ws = rng.uniform(0.0015, 0.0045, size=(G, H)).astype(np.float32)
    ys = rng.uniform(0.001, 0.01, size=7).astype(np.float32)
    out = oracle.gmm2_epilogue(c, ws, ys, gl)
    grp = np.array([0, 0, 0, 1, 1, 1, 1])
    v = (c.astype(np.float32) * ws[grp]) * ys[:, None]
    want = synth.bf16_bits(torch.from_numpy(v).bfloat16())
    assert np.array_equal(out, want)


# ------------------------------------------------------------------ combine
def test_combine_sequential_fp32_semantics(oracle):
    rng = _rng(15)
    T, K, H, A = 6, 8, 32, 60
    y = torch.from_numpy(rng.normal(0, 1, size=(A, H)).astype(np.float32)).bfloat16()
    bits = synth.bf16_bits(y)
    row_of = rng.permutation(A)[: T * K].reshape(T, K).astype(np.int32)
    row_of[2, 3] = -1
    w = rng.uniform(0, 1, size=(T, K)).astype(np.float32)
    out = oracle.combine(bits, row_of, w)
    yf = y.float().numpy()
    acc = np.zeros((T, H), np.float32)
    for k in range(K):  # ascending k, multiply rounded, then add rounded
        ok = row_of[:, k] >= 0
        p = yf[np.maximum(row_of[:, k], 0)] * w[:, k][:, None]
        acc = np.where(ok[:, None], acc + p, acc)
    want = synth.bf16_bits(torch.from_numpy(acc).bfloat16())
    assert np.array_equal(out, want)
    # float64 cross-check within bf16 rounding
    acc64 = np.zeros((T, H))
    for k in range(K):
        ok = (row_of[:, k] >= 0)[:, None]
        acc64 += np.where(ok, yf[np.maximum(row_of[:, k], 0)].astype(np.float64) * w[:, k][:, None], 0)
    got = oracle.bf16_bits_to_f32(out).astype(np.float64)
    assert np.allclose(got, acc64, rtol=2 ** -8, atol=1e-6)


def test_combine_identity_mean_and_no_fma(oracle):
    H = 16
    y = torch.arange(1, 4 * H + 1, dtype=torch.float32).view(4, H).bfloat16()
    bits = synth.bf16_bits(y)
    # K = 1, weight 1 -> the un-permute alone
    out = oracle.combine(bits, np.array([[2], [0], [3], [1]], np.int32), np.ones((4, 1), np.float32))
    assert np.array_equal(out, bits[[2, 0, 3, 1]])
    # equal weights -> mean
    out = oracle.combine(bits, np.array([[0, 1, 2, 3]], np.int32), np.full((1, 4), 0.25, np.float32))
    want = synth.bf16_bits((y.float().sum(0, keepdim=True) * 0.25).bfloat16())
    assert np.array_equal(out, want)
    # a*b + c with a separately rounded product differs from a fused multiply-add here
    a = np.float32(1.0 + 2.0 ** -7)          # exactly representable in bf16
    wv = np.float32(1.0 + 2.0 ** -23)
    prod = np.float32(a * wv)                 # rounded product
    c = -prod
    yb = synth.bf16_bits(torch.tensor([[float(a)] * 8, [1.0] * 8]).bfloat16())
    out = oracle.combine(yb, np.array([[0, 1]], np.int32), np.array([[wv, c]], np.float32))
    assert (oracle.bf16_bits_to_f32(out) == 0.0).all()  # fused arithmetic would leave a residue


# ------------------------------------------------------------------ rows quantised for the wire
def test_f32_to_fp16_matches_numpy(oracle):
    rng = np.random.default_rng(11)
    f = rng.integers(0, 2 ** 32, size=60000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    f = f[np.isfinite(f)]
    edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 65536.0, 6.1e-5, 5.96e-8, 2.98e-8, 2.9802322e-8,
                     2.9802326e-8, 1.4999, 1.5, 2.5, 0.5, 1e-10, -1.49999, 127.03125, 100.3], np.float32)
    f = np.concatenate([f, edge, rng.uniform(-130, 130, 40000).astype(np.float32)])
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_fp16_bits(f), want)


def _comm_quant_numpy(x_bits):
    """The wire quantisation with numpy's own float32 / float16 arithmetic (independent of the C code)."""
    xf = oracle_bits_to_f32(x_bits)
    A, H = xf.shape
    blk = xf.reshape(A, H // 8, 8)
    m = np.max(np.abs(blk), axis=2).astype(np.float32)
    s = (m * np.float32(1.0 / 127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = (blk / s[:, :, None]).astype(np.float32)
    q = np.rint(v.astype(np.float16).astype(np.float32))
    q[m == 0] = 0
    return q.astype(np.int8).reshape(A, H), s


def oracle_bits_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def test_comm_quant_rows_definition_and_layout(oracle):
    A, H = 37, 1024
    x = synth.normal_bf16(A, H, seed=71)
    x[3] = 0                      # all-zero row: every block q = 0, scale 0
    x[4, :8] = 0                  # one zero block in a live row
    x[5, 8:16] = torch.tensor([2.0, -2.0, 2.0, 2.0, -2.0, 2.0, 2.0, -2.0])  # equal magnitudes -> +-127
    x[6, 16:24] = torch.tensor([1.0, 0.5, 0.25, -0.125, 0.0, 1.0, -1.0, 0.0625])
    bits = synth.bf16_bits(x)
    packed = oracle.comm_quant_rows(bits)
    assert packed.shape == (A, H + H // 4) and packed.dtype == np.uint8
    q = packed[:, :H].view(np.int8)
    sc_bits = np.ascontiguousarray(packed[:, H:]).view(np.uint16)
    assert sc_bits.shape == (A, H // 8)
    want_q, s = _comm_quant_numpy(bits)
    assert np.array_equal(q, want_q)
    assert np.array_equal(sc_bits, oracle.f32_to_bf16_bits(s))
    assert not q[3].any() and not sc_bits[3].any() and not q[4, :8].any() and sc_bits[4, 0] == 0
    assert np.array_equal(q[5, 8:16], np.array([127, -127, 127, 127, -127, 127, 127, -127], np.int8))
    # every live block reaches +-127 at its largest element and nothing exceeds it
    live = s > 0
    assert (np.abs(q.astype(np.int32)).reshape(A, H // 8, 8).max(axis=2)[live] == 127).all()
    # dequantised values: bf16(q * bf16(scale)), within one quantisation step (plus bf16 rounding) of the input
    back = oracle.comm_dequant_rows(packed, H)
    scf = oracle_bits_to_f32(sc_bits)
    want_back = oracle.f32_to_bf16_bits((q.astype(np.float32).reshape(A, H // 8, 8) * scf[:, :, None]).reshape(A, H))
    assert np.array_equal(back, want_back)
    err = np.abs(oracle_bits_to_f32(back) - oracle_bits_to_f32(bits)).reshape(A, H // 8, 8)
    assert (err <= scf[:, :, None] * 0.51 + np.abs(oracle_bits_to_f32(bits)).reshape(A, H // 8, 8) * 2 ** -6 + 1e-30).all()


def test_comm_quant_rows_of_fp16_rows_keep_fp16_scales(oracle):
    """The same wire format from IEEE fp16 rows: the block scales are stored as fp16 (the reference keeps them in the
    rows' type, moe_combine_shmem.h:572,581) and the rows come back rounded to fp16.  Checked against numpy's own
    float16 / float32 arithmetic."""
    A, H = 29, 1024
    rng = np.random.default_rng(12)
    x = rng.normal(0, 1, size=(A, H)).astype(np.float16)
    x[2] = 0
    x[3, :8] = 0
    x[4, 8:16] = np.array([6e-5, -3e-5, 1e-5, 0, 6e-8, 0, 0, 0], np.float16)   # a block of (near-)subnormals
    x[5, 16:24] = np.array([60000, -65504, 1, 2, 3, 4, 5, 6], np.float16)      # the top of the range
    bits = x.view(np.uint16)
    packed = oracle.comm_quant_rows(bits, fp16=True)
    q = packed[:, :H].view(np.int8)
    sc_bits = np.ascontiguousarray(packed[:, H:]).view(np.uint16)
    blk = x.astype(np.float32).reshape(A, H // 8, 8)
    m = np.max(np.abs(blk), axis=2).astype(np.float32)
    s = (m * np.float32(1.0 / 127.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        v = (blk / s[:, :, None]).astype(np.float32)
        want_q = np.rint(v.astype(np.float16).astype(np.float32))
        want_s = s.astype(np.float16)
    want_q[m == 0] = 0
    assert np.array_equal(q, want_q.astype(np.int8).reshape(A, H))
    assert np.array_equal(sc_bits, want_s.view(np.uint16))
    back = oracle.comm_dequant_rows(packed, H, fp16=True)
    with np.errstate(over="ignore"):
        want_back = (q.astype(np.float32).reshape(A, H // 8, 8) * want_s.astype(np.float32)[:, :, None]).astype(np.float16)
    assert np.array_equal(back, want_back.reshape(A, H).view(np.uint16))
    # bf16 rows through the same entry points are unchanged by the new argument
    xb = synth.bf16_bits(synth.normal_bf16(5, H, seed=3))
    assert np.array_equal(oracle.comm_quant_rows(xb), oracle.comm_quant_rows(xb, fp16=False))


def test_comm_quant_double_rounding_is_kept(oracle):
    """x / s just below a half-integer rounds up to it in fp16 and then to the even neighbour: the reference casts
    float -> half -> int8 (moe_combine_shmem.h:587-589), and so must a restatement."""
    # block maximum 127 makes s = 127 * (1/127), which is 1 up to rounding; 1.4990234375 is a bf16 value whose fp16
    # image is itself, so pick a neighbour scale instead: search a few blocks for a case where the two roundings differ.
    rng = np.random.default_rng(5)
    x = synth.bf16_bits(torch.from_numpy(rng.uniform(-3, 3, size=(4000, 8)).astype(np.float32)).bfloat16())
    xf = oracle_bits_to_f32(x)
    m = np.max(np.abs(xf), axis=1).astype(np.float32)
    s = (m * np.float32(1.0 / 127.0)).astype(np.float32)
    v = (xf / s[:, None]).astype(np.float32)
    direct = np.rint(v)
    via_half = np.rint(v.astype(np.float16).astype(np.float32))
    rows = np.nonzero((direct != via_half).any(axis=1))[0]
    assert len(rows) > 0, "the sample holds no double-rounding case"
    packed = oracle.comm_quant_rows(x[rows])
    assert np.array_equal(packed[:, :8].view(np.int8), via_half[rows].astype(np.int8))


def test_rows_from_src_info_inverts_dispatch(oracle):
    T, K, E, H = 31, 3, 6, 16
    ids, _ = synth.softmax_topk_routing(T, E, K, seed=16)
    idx = ids.numpy()
    _, cnt, _ = oracle.layout(idx, E, 1)
    off, _ = oracle.offsets(cnt, T)
    pos = oracle.send_token_idx(idx, E)
    x = synth.normal_bf16(T, H, seed=17)
    _, _, src = oracle.dispatch(synth.bf16_bits(x), idx, off, pos, E, 0, T * K)
    assert np.array_equal(oracle.rows_from_src_info(src, T * K, T, K), oracle.rows_from_pos(idx, off, pos, E))


# ------------------------------------------------------------------ whole layer
def test_fused_layer_is_the_composition_and_close_to_exact_math(oracle):
    d = synth.ut_recipe(batch_size=24, hidden=256, intermediate=128, num_experts=6, top_k=4, seed=42)
    bits = synth.bf16_bits(d["x"])
    idx = d["ids"].numpy().astype(np.int64)
    out, etn, dbg = oracle.fused_layer(bits, idx, d["gates"].numpy(), d["w1"].numpy(), d["w1_scale"].numpy(),
                                       d["w2"].numpy(), d["w2_scale"].numpy(), debug=True)
    T, K = idx.shape
    E = 6
    assert np.array_equal(etn, np.bincount(idx.reshape(-1), minlength=E))
    # exact-arithmetic model of the same pipeline (float64 everywhere except the two int8 roundings)
    xf = d["x"].double().numpy()
    w1 = d["w1"].double().numpy() * d["w1_scale"].double().numpy()[:, None, :]
    w2 = d["w2"].double().numpy() * d["w2_scale"].double().numpy()[:, None, :]
    I = 128
    want = np.zeros_like(xf)
    for t in range(T):
        m = np.abs(xf[t]).max()
        xq = np.rint(xf[t] * 127 / m) * (m / 127)
        for k in range(K):
            e = idx[t, k]
            h1 = xq @ w1[e]
            y = h1[:I] / (1 + np.exp(-h1[:I])) * h1[I:]
            my = np.abs(y).max()
            yq = np.rint(y * 127 / my) * (my / 127)
            want[t] += d["gates"][t, k].item() * (yq @ w2[e])
    got = oracle.bf16_bits_to_f32(out).astype(np.float64)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 0.02 * scale
    assert np.corrcoef(got.reshape(-1), want.reshape(-1))[0, 1] > 0.9995


def test_fused_layer_active_mask_prefix(oracle):
    d = synth.ut_recipe(batch_size=10, hidden=128, intermediate=64, num_experts=4, top_k=2, seed=43)
    bits = synth.bf16_bits(d["x"])
    idx = d["ids"].numpy().astype(np.int64)
    args = (d["gates"].numpy(), d["w1"].numpy(), d["w1_scale"].numpy(), d["w2"].numpy(), d["w2_scale"].numpy())
    full, _ = oracle.fused_layer(bits, idx, *args)
    part, etn = oracle.fused_layer(bits, idx, *args, n_active=6)
    assert np.array_equal(part[:6], full[:6])  # tokens are independent
    assert (part[6:] == 0).all()
    assert etn.sum() == 6 * 2


# ------------------------------------------------------------------ block-scaled FP8 (definition: include/cam_fp8_spec.h)
def _e4m3_closed_form(code):
    s = -1.0 if code & 0x80 else 1.0
    e, m = (code >> 3) & 0xf, code & 7
    if e == 0xf and m == 7:
        return float("nan")
    if e == 0:
        return s * math.ldexp(m / 8.0, -6)
    return s * math.ldexp(1.0 + m / 8.0, e - 7)


def test_e4m3_decode_table_closed_form_and_torch(oracle):
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.e4m3_to_f32(codes)
    want = np.array([_e4m3_closed_form(int(c)) for c in codes], np.float32)
    assert np.array_equal(got, want, equal_nan=True)
    assert got[0x7e] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9
    via_torch = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(got, via_torch, equal_nan=True)


def test_e4m3_encode_is_nearest_even_and_saturates(oracle):
    rng = np.random.default_rng(21)
    table = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8)).astype(np.float64)
    finite = np.array([c for c in range(256) if not math.isnan(table[c])])
    x = np.concatenate([rng.uniform(-470, 470, 3000), rng.normal(0, 1, 3000), rng.uniform(-0.02, 0.02, 2000),
                        table[finite], (table[finite[:-1]] + table[finite[1:]]) / 2,   # representable values and ties
                        [448.0, 449.0, 463.9, 464.0, 1e9, -1e9, 2.0 ** -10, 2.0 ** -10 * 1.0001, 0.0]]).astype(np.float32)
    got = oracle.f32_to_e4m3(x)
    # brute force: the nearest finite value, ties to the even code, everything above 448 clamped
    for xv, g in zip(x.tolist(), got.tolist()):
        c = min(max(xv, -448.0), 448.0)
        d = np.abs(table[finite] - c)
        best = finite[np.nonzero(d == d.min())[0]]
        if len(best) > 1:
            best = [b for b in best if (b & 1) == 0] if c != 0 else [0x80 if math.copysign(1, xv) < 0 else 0]
        assert table[g] == table[best[0]], (xv, g, best)
    # and torch's conversion wherever it is defined the same way (no saturation there)
    inr = np.abs(x) <= 448
    via_torch = torch.from_numpy(x[inr]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got[inr], via_torch)
    assert oracle.f32_to_e4m3(np.array([np.inf, -np.inf], np.float32)).tolist() == [0x7e, 0xfe]


def test_fp8_block_scale_is_the_smallest_power_of_two(oracle):
    from fractions import Fraction
    rng = np.random.default_rng(22)
    vals = np.concatenate([np.exp(rng.uniform(-60, 60, 2000)), [448.0, 448.0001, 447.99, 224.0, 1.0, 1.75, 1.7500001,
                                                                 3.5, 2.0 ** -100, 7 * 2.0 ** 40]]).astype(np.float32)
    for v in vals.tolist():
        x = oracle.fp8_block_scale_exp(v)
        fv = Fraction(v)
        assert fv / Fraction(2) ** x <= 448, (v, x)
        assert fv / Fraction(2) ** (x - 1) > 448, (v, x)
    assert oracle.fp8_block_scale_exp(0.0) == 0


def test_fp8_quant_rows_matches_torch_conversion_of_scaled_values(oracle):
    x = torch.randn(19, 512, generator=torch.Generator().manual_seed(23)) * 5
    x[0] = 0
    x[1] *= 1e-12
    x[2, :128] = 448.0
    xb = x.bfloat16()
    q, sc = oracle.fp8_quant_rows(synth.bf16_bits(xb))
    xf = xb.float().reshape(19, 4, 128)
    amax = xf.abs().amax(dim=2)
    exps = torch.tensor([[oracle.fp8_block_scale_exp(float(v)) for v in row] for row in amax])
    assert np.array_equal(sc, (exps + 127).to(torch.uint8).numpy())
    scaled = xf * torch.pow(2.0, -exps.float())[:, :, None]
    assert float(scaled.abs().max()) <= 448.0
    want = scaled.to(torch.float8_e4m3fn).view(torch.uint8).reshape(19, 512).numpy()
    assert np.array_equal(q, want)
    # the largest scaled value of a live block lies in (224, 448]; rounding keeps it within [224, 448]
    deq = oracle.e4m3_to_f32(q).reshape(19, 4, 128)
    big = np.abs(deq).max(axis=2)
    live = amax.numpy() > 0
    assert ((big[live] >= 224) & (big[live] <= 448)).all()
    pre = scaled.abs().amax(dim=2).numpy()
    assert ((pre[live] > 224) & (pre[live] <= 448)).all()
    q32, sc32 = oracle.fp8_quant_rows_f32(xb.float().numpy())
    assert np.array_equal(q32, q) and np.array_equal(sc32, sc)


def test_fp8_gemm_against_float64_and_swiglu(oracle):
    g = torch.Generator().manual_seed(24)
    sizes = [3, 0, 5]
    G, K, N = 3, 256, 256
    A = sum(sizes)
    a = (torch.randn(A, K, generator=g) * 2).to(torch.float8_e4m3fn)
    w = torch.randn(G, K, N, generator=g).to(torch.float8_e4m3fn)
    sa = (torch.randint(-5, 4, (A, K // 128), generator=g) + 127).to(torch.uint8)
    sw = (torch.randint(-5, 4, (G, K // 128, N // 128), generator=g) + 127).to(torch.uint8)
    gl = np.cumsum(sizes).astype(np.int64)
    got = oracle.fp8_gemm(a.view(torch.uint8).numpy(), sa.numpy(), w.view(torch.uint8).numpy(), sw.numpy(), gl)
    af = a.double() * torch.pow(2.0, sa.double() - 127).repeat_interleave(128, dim=1)
    want = np.zeros((A, N))
    m0 = 0
    for e, n in enumerate(sizes):
        wf = w[e].double() * torch.pow(2.0, sw[e].double() - 127).repeat_interleave(128, dim=0).repeat_interleave(128, dim=1)
        want[m0:m0 + n] = (af[m0:m0 + n] @ wf).numpy()
        m0 += n
    assert np.array_equal(got, want.astype(np.float32))
    # scaling every operand block by a power of two scales the result exactly
    got2 = oracle.fp8_gemm(a.view(torch.uint8).numpy(), (sa + 3).numpy(), w.view(torch.uint8).numpy(), (sw - 1).numpy(), gl)
    assert np.array_equal(got2, got * 4.0)
    c = torch.randn(7, 64, generator=g).numpy() * 3
    y = oracle.fp8_swiglu(c.astype(np.float32))
    c64 = c.astype(np.float32).astype(np.float64)
    ref = c64[:, :32] / (1 + np.exp(-c64[:, :32])) * c64[:, 32:]
    assert np.allclose(y, ref, rtol=3e-6, atol=1e-7)


def test_fp16_activation_variants_of_gmm2_epilogue_and_combine(oracle):
    """The fp16 forms differ from the bf16 ones only in the 16-bit conversions, which numpy's float16 pins."""
    g = torch.Generator().manual_seed(31)
    c = torch.randint(-200000, 200000, (6, 128), generator=g, dtype=torch.int32).numpy()
    ws = (torch.rand(2, 128, generator=g) * 1e-3).numpy()
    ys = (torch.rand(6, generator=g) * 1e-2).numpy()
    gl = np.array([4, 6], np.int64)
    got = oracle.gmm2_epilogue_act(c, ws, ys, gl, True)
    grp = np.array([0, 0, 0, 0, 1, 1])
    want = ((c.astype(np.float32) * ws[grp]) * ys[:, None]).astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.gmm2_epilogue_act(c, ws, ys, gl, False), oracle.gmm2_epilogue(c, ws, ys, gl))
    y = (torch.randn(8, 64, generator=g) * 2).half()
    row_of = np.array([[0, 3], [5, -1], [7, 2]], np.int32)
    w = np.array([[0.25, 0.5], [1.0, 9.0], [0.3, 0.7]], np.float32)
    got = oracle.combine_act(y.view(torch.int16).numpy().view(np.uint16), row_of, w, True)
    yf = y.float().numpy()
    acc = np.zeros((3, 64), np.float32)
    for t in range(3):
        for k in range(2):
            if row_of[t, k] >= 0:
                acc[t] = acc[t] + (yf[row_of[t, k]] * w[t, k]).astype(np.float32)
    assert np.array_equal(got, acc.astype(np.float16).view(np.uint16))


# ------------------------------------------------------------------ shared expert add-back
def test_combine_shared_row_is_added_last_and_unweighted(oracle):
    rng = _rng(91)
    T, K, H, A = 5, 4, 32, 24
    y = torch.from_numpy(rng.normal(0, 1, size=(A, H)).astype(np.float32)).bfloat16()
    sh = torch.from_numpy(rng.normal(0, 1, size=(T, H)).astype(np.float32)).bfloat16()
    row_of = rng.permutation(A)[: T * K].reshape(T, K).astype(np.int32)
    row_of[1, 2] = -1
    w = rng.uniform(0, 2, size=(T, K)).astype(np.float32)
    out = oracle.combine_shared(synth.bf16_bits(y), row_of, w, synth.bf16_bits(sh))
    # independent numpy float32 restatement: routed rows in k order, then the shared row, then ONE rounding
    yf, acc = y.float().numpy(), np.zeros((T, H), np.float32)
    for k in range(K):
        ok = (row_of[:, k] >= 0)[:, None]
        acc = np.where(ok, acc + yf[np.maximum(row_of[:, k], 0)] * w[:, k][:, None], acc)
    acc = acc + sh.float().numpy()
    assert np.array_equal(out, synth.bf16_bits(torch.from_numpy(acc).bfloat16()))
    # no shared rows -> the plain combine
    assert np.array_equal(oracle.combine_shared(synth.bf16_bits(y), row_of, w), oracle.combine(synth.bf16_bits(y), row_of, w))
    # no routed rows at all -> the shared rows come back bit for bit (un-weighted: a weight would change them)
    none = np.full((T, K), -1, np.int32)
    assert np.array_equal(oracle.combine_shared(synth.bf16_bits(y), none, w, synth.bf16_bits(sh)), synth.bf16_bits(sh))


def test_combine_shared_order_and_single_rounding_witnesses(oracle):
    """(a + b) + s with s last differs from (s + a) + b here, and rounding the routed sum to bf16 before adding
    the shared row differs from rounding once at the end."""
    H = 8
    big, small = 2.0 ** 24, 1.0
    rows = synth.bf16_bits(torch.tensor([[big] * H, [small] * H]).bfloat16())
    shared = synth.bf16_bits(torch.tensor([[-big] * H]).bfloat16())
    w = np.ones((1, 2), np.float32)
    out = oracle.bf16_bits_to_f32(oracle.combine_shared(rows, np.array([[0, 1]], np.int32), w, shared))
    # routed first: 2^24 + 1 rounds to 2^24 in fp32, minus 2^24 -> 0; shared first would leave 1
    assert (out == 0.0).all()
    # single rounding: 1 + 2^-9 is not a bf16 value; with the shared row -1 the exact fp32 sum 2^-9 survives,
    # while a bf16 rounding of the routed sum (-> 1.0) first would give 0
    a = synth.bf16_bits(torch.tensor([[1.0] * H, [2.0 ** -9] * H]).bfloat16())
    sh = synth.bf16_bits(torch.tensor([[-1.0] * H]).bfloat16())
    out = oracle.bf16_bits_to_f32(oracle.combine_shared(a, np.array([[0, 1]], np.int32), w, sh))
    assert (out == np.float32(2.0 ** -9)).all()


# ------------------------------------------------------------------ the SHMEM operator pair on one rank
@pytest.mark.parametrize("T,K,E,H", [(1, 1, 1, 16), (37, 4, 8, 64), (64, 8, 32, 128)])
def test_dispatch_shmem_bookkeeping_closed_forms(oracle, T, K, E, H):
    rng = _rng(7 * T + E)
    ids = rng.integers(-1, E + 1, size=(T, K)).astype(np.int32)  # -1 and E name no expert
    x = torch.from_numpy(rng.normal(0, 1, size=(T, H)).astype(np.float32)).bfloat16()
    xb = synth.bf16_bits(x)
    for ttype in (0, 1):
        out, _, eidx, etn, rc, total = oracle.dispatch_shmem(xb, ids, E, 0, token_nums_type=ttype)
        flat = ids.ravel()
        ok = (flat >= 0) & (flat < E)
        cnt = np.bincount(flat[ok], minlength=E)
        assert total == ok.sum()
        assert np.array_equal(rc, np.cumsum(cnt).astype(np.int32))           # inclusive running totals
        assert np.array_equal(etn, np.cumsum(cnt) if ttype == 0 else cnt)    # type 0 cumulative, 1 per expert
        # expandIdx: number of earlier flat entries with the same id (brute force)
        want = np.array([-1 if not ok[i] else int((flat[:i] == flat[i]).sum()) for i in range(flat.size)], np.int32)
        assert np.array_equal(eidx, want)
        # rows: the stable sort of the valid entries by expert; row r holds the token of the r-th sorted entry
        order = np.argsort(np.where(ok, flat, E), kind="stable")[: ok.sum()]
        assert np.array_equal(out[:total], xb[order // K])
        rows = np.where(ok, np.concatenate([[0], np.cumsum(cnt)])[np.clip(flat, 0, E - 1)] + eidx, -1)
        assert np.array_equal(np.sort(rows[ok]), np.arange(total))


def test_dispatch_shmem_quant_and_smooth_scales(oracle):
    rng = _rng(5)
    T, K, E, H = 20, 3, 6, 64
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
    x = torch.from_numpy(rng.normal(0, 2, size=(T, H)).astype(np.float32)).bfloat16()
    x[3] = 0  # an all-zero token: zeros and scale 0 by definition
    xb = synth.bf16_bits(x)
    # without smooth scales every copy equals the token's no-epsilon quantisation (variant 2)
    q, sc, eidx, _, rc, total = oracle.dispatch_shmem(xb, ids, E, 2)
    q2, s2 = oracle.quant_rows(xb, 2)
    start = np.concatenate([[0], rc[:-1]])
    rows = start[ids.ravel()] + eidx
    assert np.array_equal(q[rows], np.repeat(q2, K, axis=0)) and np.array_equal(sc[rows], np.repeat(s2, K))
    assert (q[rows[3 * K:4 * K]] == 0).all() and (sc[rows[3 * K:4 * K]] == 0).all()
    # smooth scales of all ones change nothing; powers of two leave q alone and scale the stored scale exactly
    ones = np.ones((E, H), np.float32)
    q1, s1 = oracle.dispatch_shmem(xb, ids, E, 2, smooth=ones)[:2]
    assert np.array_equal(q1, q) and np.array_equal(s1, sc)
    pw = (2.0 ** rng.integers(-3, 4, size=E)).astype(np.float32)
    qp, sp = oracle.dispatch_shmem(xb, ids, E, 2, smooth=np.repeat(pw[:, None], H, 1))[:2]
    assert np.array_equal(qp, q)
    assert np.array_equal(sp[rows], (sc[rows] * np.repeat(pw[None, :], T, 0)[np.arange(T)[:, None], ids].ravel()))
    # general smooth scales: independent numpy float32 restatement, copy by copy
    sm = rng.uniform(0.25, 4.0, size=(E, H)).astype(np.float32)
    qs, ss = oracle.dispatch_shmem(xb, ids, E, 2, smooth=sm)[:2]
    xf = x.float().numpy()
    for t in range(T):
        for k in range(K):
            e = ids[t, k]
            v = (xf[t] * sm[e]).astype(np.float32)                    # one rounded multiply
            m = np.abs(v).max()
            r = rows[t * K + k]
            if m == 0:
                assert (qs[r] == 0).all() and ss[r] == 0
                continue
            s = np.float32(127.0) / m
            assert np.array_equal(qs[r], np.rint((v * s).astype(np.float32)).astype(np.int8))
            assert ss[r] == np.float32(1.0) / s
            assert np.abs(qs[r]).max() == 127
    # the copies of one token now differ (the scale row is the destination expert's)
    assert not np.array_equal(qs[rows[0]], qs[rows[1]])


def test_combine_shmem_locates_rows_like_the_dispatch_and_applies_the_wire_rounding(oracle):
    rng = _rng(6)
    T, K, E, H = 24, 4, 8, 64
    ids = np.stack([rng.permutation(E + 1)[:K] - 1 for _ in range(T)]).astype(np.int32)  # some -1
    x = torch.from_numpy(rng.normal(0, 1, size=(T, H)).astype(np.float32)).bfloat16()
    _, _, eidx, _, rc, total = oracle.dispatch_shmem(synth.bf16_bits(x), ids, E, 0)
    y = torch.from_numpy(rng.normal(0, 1, size=(total, H)).astype(np.float32)).bfloat16()
    yb = synth.bf16_bits(y)
    w = rng.uniform(0, 1, size=(T, K)).astype(np.float32)
    out = oracle.combine_shmem(yb, ids, eidx, rc, w, E)
    # the same rows as the plan-based map (offset of the expert + place inside it), then the plain combine
    cnt = np.bincount(ids[ids >= 0], minlength=E).astype(np.int32)
    off, _ = oracle.offsets(cnt, T)
    row_of = oracle.rows_from_pos(ids.astype(np.int64), off, eidx.reshape(T, K), E)
    assert np.array_equal(out, oracle.combine(yb, row_of, w))
    # K = 1, weight 1: combine(dispatch(x)) == x, the un-permute round trip
    ids1 = rng.integers(0, E, size=(T, 1)).astype(np.int32)
    rows1, _, e1, _, rc1, _ = oracle.dispatch_shmem(synth.bf16_bits(x), ids1, E, 0)
    assert np.array_equal(oracle.combine_shmem(rows1, ids1, e1, rc1, np.ones((T, 1), np.float32), E), synth.bf16_bits(x))
    # commQuantMode 2: every row first goes through the int8 wire format
    wired = oracle.comm_dequant_rows(oracle.comm_quant_rows(yb), H)
    assert np.array_equal(oracle.combine_shmem(yb, ids, eidx, rc, w, E, comm_quant=True), oracle.combine(wired, row_of, w))
    assert not np.array_equal(wired, yb)
