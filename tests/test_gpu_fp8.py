"""GPU parity of the block-scaled FP8 layer against the CPU oracle.

The FP8 layer is this library's own definition (include/cam_fp8_spec.h); the reference is W8A8 int8 only
(src/cam/README.md:20-21), so nothing here is pinned against reference outputs.  Quantised values and scales
are compared bit for bit; the matrix products accumulate in fp32 in hardware order and are compared with the
tolerances written in each test.
"""
import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce

pytestmark = pytest.mark.gpu


def _rand_fp8(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(torch.float8_e4m3fn)


def _rand_e8m0(shape, seed, lo=-9, hi=-5):
    g = torch.Generator().manual_seed(seed)
    return (torch.randint(lo, hi + 1, shape, generator=g) + 127).to(torch.uint8)


def _u8(t):
    return t.view(torch.uint8).cpu().numpy()


def test_dispatch_fp8_rows_and_scales_bit_exact(gpu, oracle):
    announce("fp8 dispatch T=77 H=4096")
    T, H, E, K = 77, 4096, 16, 4
    ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=3)
    x = synth.normal_bf16(T, H, seed=4)
    x[0] = 0
    x[1] = (x[1].float() * 1e-30).bfloat16()
    x[2] = (x[2].float() * 1e30).bfloat16()
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(torch.int32).to(gpu), E, quant_mode=4)
    q, sc = oracle.fp8_quant_rows(synth.bf16_bits(x))
    slot = d["slot_row"].cpu().numpy()
    rx, rs = _u8(d["recv_x"]), d["recv_x_scales"].cpu().numpy()
    assert rx.shape == (T * K, H) and rs.shape == (T * K, H // 128)
    for t in range(T):
        for k in range(K):
            r = slot[t, k]
            assert r >= 0
            assert np.array_equal(rx[r], q[t]), (t, k)
            assert np.array_equal(rs[r], sc[t]), (t, k)


def test_dispatch_fp8_from_fp16_activations(gpu, oracle):
    announce("fp8 dispatch from fp16")
    T, H, E, K = 33, 1024, 8, 2
    ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=5)
    x = torch.randn(T, H, generator=torch.Generator().manual_seed(6)).half()
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(torch.int32).to(gpu), E, quant_mode=4)
    q, sc = oracle.fp8_quant_rows(x.view(torch.int16).numpy().view(np.uint16), fp16=True)
    slot = d["slot_row"].cpu().numpy()
    rx, rs = _u8(d["recv_x"]), d["recv_x_scales"].cpu().numpy()
    for t in range(T):
        for k in range(K):
            assert np.array_equal(rx[slot[t, k]], q[t]) and np.array_equal(rs[slot[t, k]], sc[t])


def test_quant_rows_fp8_bit_exact(gpu, oracle):
    announce("fp8 re-quantisation of fp32 rows")
    y = torch.randn(300, 1536, generator=torch.Generator().manual_seed(9)) * 3
    y[0] = 0
    y[1] *= 1e-20
    y[2] *= 1e20
    q, sc = cam.quant_rows_fp8(y.to(gpu))
    wq, wsc = oracle.fp8_quant_rows_f32(y.numpy())
    assert np.array_equal(_u8(q), wq)
    assert np.array_equal(sc.cpu().numpy(), wsc)


def _gemm_case(gpu, oracle, sizes, K, N, gate_up, seed, out_dtype=torch.float32):
    G = len(sizes)
    gl = torch.tensor(np.cumsum(sizes), dtype=torch.int64)
    A = int(gl[-1])
    a = _rand_fp8((max(A, 1), K), seed, 2.0)
    sa = _rand_e8m0((max(A, 1), K // 128), seed + 1, -6, 2)
    w = _rand_fp8((G, K, N), seed + 2)
    sw = _rand_e8m0((G, K // 128, N // 128), seed + 3, -6, 2)
    wp = cam.prepack_weight(w.to(gpu), gate_up)
    out = cam.grouped_matmul_fp8(a.to(gpu), sa.to(gpu), wp, sw.to(gpu), gl.to(gpu), out_dtype=out_dtype)
    c = oracle.fp8_gemm(_u8(a), sa.numpy(), _u8(w), sw.numpy(), gl.numpy())
    want = oracle.fp8_swiglu(c) if gate_up else c
    return out.float().cpu().numpy()[:A], want[:A]


@pytest.mark.parametrize("sizes,K,N,gate_up", [
    ([5, 0, 130, 60], 256, 256, False),
    ([300, 77], 512, 1024, False),          # two row tiles of one expert, flat and tall shapes
    ([33, 257], 1024, 512, True),
    ([129, 3, 64], 4096, 768, True),        # K of the C5 layer, ragged column block (768 = 3 x 256)
    ([700, 1], 128, 384, False),            # shortest K loop
])
def test_grouped_matmul_fp8_sums(gpu, oracle, sizes, K, N, gate_up):
    """fp32 sums (or SwiGLU products) of the scaled FP8 MFMA against double accumulation.
    Tolerance: |diff| <= 1e-3 |want| + 2e-4 max|want| (measured: 3e-5 of the maximum; the matrix core aligns the
    64 products of an instruction to a common exponent before adding them)."""
    announce("fp8 gemm sizes=%s K=%d N=%d gate_up=%s" % (sizes, K, N, gate_up))
    got, want = _gemm_case(gpu, oracle, sizes, K, N, gate_up, seed=K + N)
    tol = 1e-3 * np.abs(want) + 2e-4 * np.abs(want).max()
    assert (np.abs(got - want) <= tol).all(), float(np.abs(got - want).max())


def test_grouped_matmul_fp8_bf16_output(gpu, oracle):
    """bf16 output: within one bf16 rounding step (2^-8 relative) of the oracle's sums plus the sum tolerance."""
    announce("fp8 gemm bf16 output")
    got, want = _gemm_case(gpu, oracle, [200, 31], 1536, 1024, False, seed=77, out_dtype=torch.bfloat16)
    tol = (2.0 ** -8 + 1e-3) * np.abs(want) + 2e-4 * np.abs(want).max()
    assert (np.abs(got - want) <= tol).all()


@pytest.mark.parametrize("sizes,K,N", [
    ([33, 257, 0, 5], 1024, 512),      # flat and tall experts, an empty one, two product blocks
    ([129, 3, 64], 4096, 768),         # three product blocks, K of the C5 layer
    ([700, 130, 1], 256, 1280),        # 1280 = 2.5 flat column blocks: the last flat item has one live team
    ([520], 512, 3072),                # three row tiles, N of the C5 layer
])
def test_grouped_matmul_fp8_quantised_product_bit_exact(gpu, oracle, sizes, K, N):
    """The epilogue that quantises the SwiGLU product (E4M3 + E8M0 per 128 columns) against the two-step form on
    the same device sums: fp32 product, then QuantRowsFp8.  Same arithmetic on the same values: bit for bit.
    The fp32 product itself is pinned against the oracle by test_grouped_matmul_fp8_sums, QuantRowsFp8 by
    test_quant_rows_fp8_bit_exact."""
    announce("fp8 gemm quantised product sizes=%s K=%d N=%d" % (sizes, K, N))
    G = len(sizes)
    gl = torch.tensor(np.cumsum(sizes), dtype=torch.int64)
    A = int(gl[-1])
    a = _rand_fp8((A, K), K + N, 2.0)
    sa = _rand_e8m0((A, K // 128), K + N + 1, -6, 2)
    w = _rand_fp8((G, K, N), K + N + 2)
    sw = _rand_e8m0((G, K // 128, N // 128), K + N + 3, -6, 2)
    wp = cam.prepack_weight(w.to(gpu), True)
    prod = cam.grouped_matmul_fp8(a.to(gpu), sa.to(gpu), wp, sw.to(gpu), gl.to(gpu))
    want_q, want_s = cam.quant_rows_fp8(prod)
    got_q, got_s = cam.grouped_matmul_fp8(a.to(gpu), sa.to(gpu), wp, sw.to(gpu), gl.to(gpu),
                                          out_dtype=torch.float8_e4m3fn)
    assert np.array_equal(got_s.cpu().numpy(), want_s.cpu().numpy())
    assert np.array_equal(_u8(got_q), _u8(want_q))
    # and against the oracle's quantisation of the oracle's product, where the device sums are within tolerance:
    # scales may differ only where a block maximum sits on a power-of-two boundary, so compare dequantised values
    c = oracle.fp8_gemm(_u8(a), sa.numpy(), _u8(w), sw.numpy(), gl.numpy())
    oq, osc = oracle.fp8_quant_rows_f32(oracle.fp8_swiglu(c)[:A].astype(np.float32))
    lut = oracle.e4m3_to_f32(np.arange(256, dtype=np.uint8)).astype(np.float64)
    deq = lambda qq, ss: lut[qq] * np.repeat(np.exp2(ss.astype(np.float64) - 127), 128, axis=1)
    dv, dw = deq(_u8(got_q), got_s.cpu().numpy()), deq(oq, osc)
    blockmax = np.repeat(np.abs(dw).reshape(A, -1, 128).max(axis=2), 128, axis=1)
    assert (np.abs(dv - dw) <= 0.13 * blockmax + 1e-30).all()


def _layer_inputs(T, H, E, K, I, seed):
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=seed)
    x = synth.normal_bf16(T, H, seed=seed + 1)
    w1 = _rand_fp8((E, H, 2 * I), seed + 2)
    s1 = _rand_e8m0((E, H // 128, 2 * I // 128), seed + 3)
    w2 = _rand_fp8((E, I, H), seed + 4)
    s2 = _rand_e8m0((E, I // 128, H // 128), seed + 5)
    return ids, w, x, w1, s1, w2, s2


def _check_layer(got, want_bits):
    """bf16 layer output against the oracle's.  An FP8 re-quantisation sits between the two GEMMs: a product that
    differs in its last bits can land on the other side of an E4M3 rounding boundary (a 6-12 % step on one of I
    inputs of a GMM2 sum), so single outputs move by a fraction of a percent of the output scale.  Tolerance:
    max |diff| <= 2e-2 max|want| and mean |diff| <= 2e-3 max|want| (measured: 1e-2 and 6e-4)."""
    want = (want_bits.astype(np.uint32) << 16).view(np.float32)
    err = np.abs(got - want)
    mx = np.abs(want).max()
    assert err.max() <= 2e-2 * mx, (float(err.max()), float(mx))
    assert err.mean() <= 2e-3 * mx, (float(err.mean()), float(mx))


@pytest.mark.parametrize("T,H,E,K,I", [(64, 1024, 8, 2, 512), (200, 2048, 16, 4, 768)])
def test_fused_layer_fp8_against_oracle(gpu, oracle, T, H, E, K, I):
    announce("fp8 fused layer T=%d H=%d E=%d K=%d I=%d" % (T, H, E, K, I))
    ids, w, x, w1, s1, w2, s2 = _layer_inputs(T, H, E, K, I, seed=T)
    out, etn = cam.fused_deep_moe_fp8(x.to(gpu), ids.to(torch.int32).to(gpu), cam.prepack_weight(w1.to(gpu), True),
                                      s1.to(gpu), cam.prepack_weight(w2.to(gpu), False), s2.to(gpu), w.to(gpu))
    want, dbg = oracle.fp8_fused_layer(synth.bf16_bits(x), ids.numpy(), w.numpy(), _u8(w1), s1.numpy(), _u8(w2),
                                       s2.numpy(), debug=True)
    assert np.array_equal(etn.cpu().numpy(), dbg["cnt"])
    _check_layer(out.float().cpu().numpy(), want)
    # stage by stage with the operators: the quantised input rows are exact, and so is the re-quantisation of a
    # given product tensor; the product tensor itself is within the GEMM tolerance and the E4M3 codes made from
    # it differ from the oracle's in a small fraction of places, never by more than one code
    gl = torch.from_numpy(np.cumsum(dbg["cnt"]).astype(np.int64)).to(gpu)
    x1 = torch.from_numpy(dbg["x1"]).to(gpu).view(torch.float8_e4m3fn)
    y = cam.grouped_matmul_fp8(x1, torch.from_numpy(dbg["s1"]).to(gpu), cam.prepack_weight(w1.to(gpu), True),
                               s1.to(gpu), gl)
    yw = dbg["y"]
    assert (np.abs(y.cpu().numpy() - yw) <= 1e-3 * np.abs(yw) + 2e-4 * np.abs(yw).max()).all()
    q, sc = cam.quant_rows_fp8(y)
    same_scale = sc.cpu().numpy() == dbg["s2"]
    assert same_scale.mean() > 0.999
    codes, wcodes = _u8(q), dbg["x2"]
    blocks_ok = np.repeat(same_scale, 128, axis=1)
    differ = (codes != wcodes) & blocks_ok
    assert differ.mean() < 0.01
    # where they differ, by one E4M3 step (12.5 % at most) or, near zero, by a sliver of the block's range (448)
    dv, dw = oracle.e4m3_to_f32(codes[differ]), oracle.e4m3_to_f32(wcodes[differ])
    assert (np.abs(dv - dw) <= 0.125 * np.maximum(np.abs(dv), np.abs(dw)) + 0.5).all()


def test_fused_layer_fp8_decode_shape_full_size(gpu, oracle):
    """The FP8 layer configuration at its decode size: 128 tokens, hidden 4096, 128 experts, top-8, intermediate 1536."""
    announce("fp8 fused layer, 128-token full-size configuration")
    T, H, E, K, I = 128, 4096, 128, 8, 1536
    ids, w, x, w1, s1, w2, s2 = _layer_inputs(T, H, E, K, I, seed=3)
    out, etn = cam.fused_deep_moe_fp8(x.to(gpu), ids.to(torch.int32).to(gpu), cam.prepack_weight(w1.to(gpu), True),
                                      s1.to(gpu), cam.prepack_weight(w2.to(gpu), False), s2.to(gpu), w.to(gpu))
    want, dbg = oracle.fp8_fused_layer(synth.bf16_bits(x), ids.numpy(), w.numpy(), _u8(w1), s1.numpy(), _u8(w2),
                                       s2.numpy(), debug=True)
    assert np.array_equal(etn.cpu().numpy(), dbg["cnt"])
    _check_layer(out.float().cpu().numpy(), want)


def test_fused_layer_fp8_prefill_shape_sampled_tokens(gpu, oracle):
    """8192 tokens (65536 rows): a token's output depends on its own routing and the weights only, so the oracle is
    run on a sample of tokens and compared with those tokens' rows of the full-size result."""
    announce("fp8 fused layer, 8192-token full-size configuration, sampled tokens")
    T, H, E, K, I = 8192, 4096, 128, 8, 1536
    ids, w, x, w1, s1, w2, s2 = _layer_inputs(T, H, E, K, I, seed=11)
    out, etn = cam.fused_deep_moe_fp8(x.to(gpu), ids.to(torch.int32).to(gpu), cam.prepack_weight(w1.to(gpu), True),
                                      s1.to(gpu), cam.prepack_weight(w2.to(gpu), False), s2.to(gpu), w.to(gpu))
    assert np.array_equal(etn.cpu().numpy(), np.bincount(ids.numpy().reshape(-1), minlength=E))
    pick = np.unique(np.concatenate([[0, 1, T - 1], np.random.default_rng(12).integers(0, T, 45)]))
    want = oracle.fp8_fused_layer(synth.bf16_bits(x)[pick], ids.numpy()[pick], w.numpy()[pick], _u8(w1), s1.numpy(),
                                  _u8(w2), s2.numpy())
    _check_layer(out.float().cpu().numpy()[pick], want)
    assert torch.isfinite(out.float()).all()
