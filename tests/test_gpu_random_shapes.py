"""GPU parity on seeded random shapes: the operators of the path against the oracle, bit for bit, at sizes nobody
picked by hand (odd token counts, ragged hidden sizes, empty and single-row experts, duplicate and negative expert
ids, top-k up to 16).  Every case prints its parameters before it touches the GPU; the seeds are fixed, so a failure
names a case that can be run again.  The cases are small: the whole file runs in seconds.  CAM_RANDOM_SHAPE_SCALE=n
runs n times as many seeds of each kind (a longer hunt, by hand)."""
import os

import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce, to_np, plan_oracle, assert_bits_equal
from test_gpu_dispatch import _check_fused

pytestmark = pytest.mark.gpu

SCALE = max(1, int(os.environ.get("CAM_RANDOM_SHAPE_SCALE", "1")))


def _ids(rng, T, K, E, neg_frac, dup):
    """[T,K] expert ids: distinct per token unless `dup`, a fraction of them -1."""
    if dup:
        ids = rng.integers(0, E, size=(T, K))
    else:
        ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]) if K <= E else rng.integers(0, E, size=(T, K))
    drop = rng.random((T, K)) < neg_frac
    ids = np.where(drop, -1, ids)
    return torch.from_numpy(ids.astype(np.int64))


@pytest.mark.parametrize("seed", range(12 * SCALE))
def test_dispatch_prefill_then_combine_random_shape(gpu, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    T = int(rng.integers(1, 400))
    E = int(rng.choice([2, 3, 8, 17, 64, 100, 256, 384, 512]))
    K = int(rng.integers(1, min(16, E) + 1))
    H = int(rng.choice([1024, 1032, 1536, 2048, 2064, 4096, 5120, 7168]))
    quant_mode = int(rng.choice([0, 2, 3]))
    if quant_mode == 3 and H % 128 != 0:
        quant_mode = 2
    neg = float(rng.choice([0.0, 0.0, 0.1, 0.5]))
    dup = bool(rng.integers(0, 2))
    dtype = torch.int32 if rng.integers(0, 2) else torch.int64
    announce("random dispatch+combine seed=%d T=%d K=%d E=%d H=%d quant=%d neg=%.1f dup=%s %s" %
             (seed, T, K, E, H, quant_mode, neg, dup, dtype))
    ids = _ids(rng, T, K, E, neg, dup)
    x = synth.normal_bf16(T, H, seed=seed + 7)
    if T > 2:
        x[int(rng.integers(0, T))] = 0  # an all-zero token
    idx_np = ids.numpy()
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(dtype).to(gpu), E, quant_mode=quant_mode)
    _check_fused(oracle, d, x, idx_np, E, quant_mode)
    # the way back: a gather with the dispatch's own map, from rows of the activation type
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E, skip_out_of_range=True)
    total = int(cnt.sum())
    w = torch.from_numpy(rng.random((T, K)).astype(np.float32))
    y = synth.normal_bf16(max(total, 1), H, seed=seed + 9)
    row_of = oracle.rows_from_pos(idx_np, off, pos, E)
    got = cam.moe_combine_gather(y.to(gpu), None, d["slot_row"], w.to(gpu))
    want = oracle.combine(synth.bf16_bits(y), row_of, w.numpy())
    assert_bits_equal(to_np(got), want, "combined x")


@pytest.mark.parametrize("seed", range(10 * SCALE))
def test_grouped_gemm_operators_random_shape(gpu, oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    G = int(rng.integers(1, 40))
    kind = int(rng.integers(0, 3))
    sizes = [int(v) for v in rng.choice([0, 1, 5, 31, 64, 127, 128, 129, 200, 257, 400], size=G)]
    if sum(sizes) == 0:
        sizes[0] = 3
    Kd = int(rng.choice([128, 256, 384, 512, 1024, 1536]))
    A = sum(sizes)
    if kind == 0:  # int32 sums, plain or gate/up layout
        N = int(rng.choice([64, 128, 320, 512, 1152]))
        gate_up = bool(rng.integers(0, 2)) and N % 128 == 0
        announce("random gemm int32 seed=%d sizes=%s Kd=%d N=%d gate_up=%s" % (seed, sizes, Kd, N, gate_up))
        a = synth.uniform_int8((A, Kd), seed)
        w = synth.uniform_int8((G, Kd, N), seed + 1)
        gl = torch.tensor(np.cumsum(sizes), dtype=torch.int64)
        got = cam.grouped_matmul_int32(a.to(gpu), cam.prepack_weight(w.to(gpu), gate_up), gl.to(gpu))
        assert_bits_equal(to_np(got)[:A], oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())[:A], "int32 sums")
    elif kind == 1:  # gate/up GEMM + SwiGLU + per-row quantisation
        I = int(rng.choice([64, 128, 320, 512]))
        announce("random gmm1 seed=%d sizes=%s H=%d I=%d" % (seed, sizes, Kd, I))
        a = synth.uniform_int8((A, Kd), seed)
        w = synth.uniform_int8((G, Kd, 2 * I), seed + 1, -16, 16)
        gl = torch.tensor(np.cumsum(sizes), dtype=torch.int64)
        ws = synth.channel_scales((G, 2 * I), seed=seed + 2)
        xs = synth.channel_scales((A,), seed=seed + 3, lo=0.005, hi=0.05)
        y, ysc = cam.grouped_matmul_swiglu_quant(a.to(gpu), xs.to(gpu), cam.prepack_weight(w.to(gpu), True),
                                                 ws.to(gpu), gl.to(gpu))
        c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
        want_q, want_s = oracle.swiglu_quant(oracle.gmm1_epilogue(c, ws.numpy(), xs.numpy(), gl.numpy()), rows=A)
        assert_bits_equal(to_np(ysc)[:A].view(np.uint32), want_s[:A].view(np.uint32), "y_scale")
        assert_bits_equal(to_np(y)[:A], want_q[:A], "y int8")
    else:  # down GEMM + dequantisation to bf16
        H = int(rng.choice([64, 256, 1024, 1088]))
        announce("random gmm2 seed=%d sizes=%s I=%d H=%d" % (seed, sizes, Kd, H))
        a = synth.uniform_int8((A, Kd), seed)
        w = synth.uniform_int8((G, Kd, H), seed + 1, -16, 16)
        gl = torch.tensor(np.cumsum(sizes), dtype=torch.int64)
        ws = synth.channel_scales((G, H), seed=seed + 2)
        xs = synth.channel_scales((A,), seed=seed + 3, lo=0.001, hi=0.01)
        out = cam.grouped_matmul_dequant(a.to(gpu), xs.to(gpu), cam.prepack_weight(w.to(gpu), False), ws.to(gpu),
                                         gl.to(gpu))
        c = oracle.gmm_int32(a.numpy(), w.numpy(), gl.numpy())
        assert_bits_equal(to_np(out)[:A], oracle.gmm2_epilogue(c, ws.numpy(), xs.numpy(), gl.numpy())[:A], "bf16 rows")


@pytest.mark.parametrize("seed", range(8 * SCALE))
def test_fused_layer_random_shape(gpu, oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    T = int(rng.integers(1, 200))
    E = int(rng.choice([2, 4, 8, 16, 24, 48]))
    K = int(rng.integers(1, min(12, E) + 1))
    H = int(rng.choice([512, 1024, 1536]))
    I = int(rng.choice([512, 768, 1024]))
    n_active = int(rng.integers(0, T + 1)) if rng.integers(0, 3) == 0 else None
    announce("random fused layer seed=%d T=%d K=%d E=%d H=%d I=%d active=%s" % (seed, T, K, E, H, I, n_active))
    d = synth.ut_recipe(batch_size=T, hidden=H, intermediate=I, num_experts=E, top_k=K, seed=seed + 60)
    if rng.integers(0, 2):
        d["ids"][::5, 0] = -1
    w1 = [cam.prepack_weight(d["w1"].to(gpu), True)]
    w2 = [cam.prepack_weight(d["w2"].to(gpu), False)]
    mask = None
    if n_active is not None:
        mask = torch.zeros(T, dtype=torch.bool)
        mask[:n_active] = True
    out, etn = cam.fused_deep_moe(d["x"].to(gpu), d["ids"].to(torch.int32).to(gpu), w1, [d["w1_scale"].to(gpu)], w2,
                                  [d["w2_scale"].to(gpu)], d["gates"].to(gpu), None,
                                  None if mask is None else mask.to(gpu), "ep_group", 1, 0, E, 1, 0, 0, 0)
    want, want_etn = oracle.fused_layer(synth.bf16_bits(d["x"]), d["ids"].numpy().astype(np.int64), d["gates"].numpy(),
                                        d["w1"].numpy(), d["w1_scale"].numpy(), d["w2"].numpy(), d["w2_scale"].numpy(),
                                        n_active=n_active)
    assert_bits_equal(to_np(etn), want_etn, "expert_token_nums")
    assert_bits_equal(to_np(out), want, "layer output")


def _bits16(t):
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("seed", range(10 * SCALE))
def test_shmem_pair_random_shape(gpu, oracle, seed):
    rng = np.random.default_rng(4000 + seed)
    T = int(rng.integers(1, 300))
    E = int(rng.choice([2, 8, 24, 64, 256]))
    K = int(rng.integers(1, min(16, E) + 1))
    H = int(rng.choice([1024, 1032, 2048, 4096, 7168]))
    quant = int(rng.choice([0, 2]))
    smooth = quant == 2 and bool(rng.integers(0, 2))
    fp16 = bool(rng.integers(0, 2))
    ttype = int(rng.integers(0, 2))
    comm = int(rng.choice([0, 2]))
    announce("random shmem pair seed=%d T=%d K=%d E=%d H=%d quant=%d smooth=%d fp16=%d type=%d comm=%d" %
             (seed, T, K, E, H, quant, smooth, fp16, ttype, comm))
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=seed + 70)
    ids = ids.to(torch.int32)
    drop = torch.from_numpy(rng.random((T, K)) < 0.1)
    ids[drop] = -1
    x = synth.normal_bf16(T, H, seed=seed + 71)
    if fp16:
        x = x.half()
    sm = None
    if smooth:
        sm = torch.from_numpy((rng.random((E, H)) * 3.75 + 0.25).astype(np.float32))
    want = oracle.dispatch_shmem(_bits16(x), ids.numpy(), E, quant, smooth=None if sm is None else sm.numpy(), fp16=fp16,
                                 token_nums_type=ttype)
    got = cam.moe_dispatch_shmem(x.to(gpu), ids.to(gpu), None if sm is None else sm.to(gpu), None, 1, 0, E, 1, 0, 0, 1, 0,
                                 quant, 0, ttype, 0)
    total = want[5]
    assert_bits_equal(to_np(got[2]), want[2], "expandIdx")
    assert_bits_equal(to_np(got[3]), want[3], "expertTokenNums")
    assert_bits_equal(to_np(got[4]), want[4], "epRecvCount")
    if quant:
        assert_bits_equal(to_np(got[0])[:total], want[0][:total], "expandX (int8)")
        assert_bits_equal(to_np(got[1])[:total].view(np.uint32), want[1][:total].view(np.uint32), "dynamicScales")
    else:
        assert_bits_equal(_bits16(got[0])[:total], want[0][:total], "expandX (copy)")
    # the way back, from rows of the activation type
    y = synth.normal_bf16(got[0].size(0), H, seed=seed + 72)
    if fp16:
        y = y.half()
    back = cam.moe_combine_shmem(y.to(gpu), ids.to(gpu), got[2], got[4], w.to(gpu), epWorldSize=1, moeExpertNum=E,
                                 commQuantMode=comm)
    want_back = oracle.combine_shmem(_bits16(y), ids.numpy(), to_np(got[2]), to_np(got[4]), w.numpy(), E, fp16=fp16,
                                     comm_quant=comm == 2)
    assert_bits_equal(_bits16(back), want_back, "combined rows")


@pytest.mark.parametrize("seed", range(4 * SCALE))
def test_fp8_fused_layer_random_shape(gpu, oracle, seed):
    from test_gpu_fp8 import _layer_inputs, _check_layer, _u8
    rng = np.random.default_rng(5000 + seed)
    T = int(rng.integers(1, 160))
    E = int(rng.choice([2, 4, 8, 16, 32]))
    K = int(rng.integers(1, min(8, E) + 1))
    H = int(rng.choice([1024, 1536, 2048]))
    I = int(rng.choice([512, 768, 1024]))
    announce("random fp8 layer seed=%d T=%d K=%d E=%d H=%d I=%d" % (seed, T, K, E, H, I))
    ids, w, x, w1, s1, w2, s2 = _layer_inputs(T, H, E, K, I, seed=seed + 90)
    out, etn = cam.fused_deep_moe_fp8(x.to(gpu), ids.to(torch.int32).to(gpu), cam.prepack_weight(w1.to(gpu), True),
                                      s1.to(gpu), cam.prepack_weight(w2.to(gpu), False), s2.to(gpu), w.to(gpu))
    want, dbg = oracle.fp8_fused_layer(synth.bf16_bits(x), ids.numpy(), w.numpy(), _u8(w1), s1.numpy(), _u8(w2),
                                       s2.numpy(), debug=True)
    assert np.array_equal(etn.cpu().numpy(), dbg["cnt"])
    _check_layer(out.float().cpu().numpy(), want)


def test_dispatch_and_combine_at_the_largest_parameters(gpu, oracle):
    """Every parameter at its limit at once: 512 experts, top-16, hidden 7168, and twice the batch the reference's
    tiling admits (16384 tokens, 262144 routing entries of which one in 513 names no expert)."""
    T, K, E, H = 16384, 16, 512, 7168
    announce("largest parameters: T=%d K=%d E=%d H=%d" % (T, K, E, H))
    rng = np.random.default_rng(T)
    ids = torch.from_numpy(rng.integers(-1, E, size=(T, K)).astype(np.int64))
    x = synth.normal_bf16(T, H, seed=T + 1)
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(gpu), E, quant_mode=2)
    idx_np = ids.numpy()
    _check_fused(oracle, d, x, idx_np, E, 2)
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E, skip_out_of_range=True)
    total = int(cnt.sum())
    w = torch.from_numpy(rng.random((T, K)).astype(np.float32))
    y = synth.normal_bf16(total, H, seed=T + 2)
    got = cam.moe_combine_gather(y.to(gpu), None, d["slot_row"], w.to(gpu))
    want = oracle.combine(synth.bf16_bits(y), oracle.rows_from_pos(idx_np, off, pos, E), w.numpy())
    assert_bits_equal(to_np(got), want, "combined x")
