"""GPU parity: routing plan, layout and permute+quant kernels against the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce, to_np, plan_oracle, assert_bits_equal

pytestmark = pytest.mark.gpu


def _random_ids(T, K, E, seed, neg_frac=0.0, dtype=torch.int64):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int64)
    if neg_frac > 0:
        ids[torch.rand(T, K, generator=g) < neg_frac] = -1
    return ids.to(dtype)


@pytest.mark.parametrize("T,K,E,R,dtype,neg", [
    (1, 1, 1, 1, torch.int64, 0.0),
    (17, 3, 8, 2, torch.int64, 0.2),
    (128, 8, 256, 8, torch.int64, 0.0),
    (333, 16, 384, 384, torch.int32, 0.1),
    (4096, 8, 256, 1, torch.int64, 0.0),
    (5000, 6, 512, 64, torch.int64, 0.05),
])
def test_get_dispatch_layout(gpu, oracle, T, K, E, R, dtype, neg):
    announce("layout T=%d K=%d E=%d R=%d" % (T, K, E, R))
    ids = _random_ids(T, K, E, seed=T + E, neg_frac=neg, dtype=dtype)
    per_rank, per_expert, in_rank = cam.get_dispatch_layout(ids.to(gpu), E, R)
    want_rank, want_cnt, want_in = oracle.layout(ids.numpy().astype(np.int64), E, R)
    assert per_rank.dtype == torch.int32 and per_expert.dtype == torch.int32 and in_rank.dtype == torch.bool
    assert_bits_equal(to_np(per_expert), want_cnt, "num_tokens_per_expert")
    assert_bits_equal(to_np(per_rank), want_rank, "num_tokens_per_rank")
    assert_bits_equal(to_np(in_rank), want_in, "is_token_in_rank")


def test_notify_dispatch_scan(gpu, oracle):
    announce("notify E=256")
    cnt = torch.randint(0, 300, (256,), generator=torch.Generator().manual_seed(1), dtype=torch.int32)
    send, off, recv = cam.notify_dispatch(cnt.to(gpu), 4096)
    want_off, want_trip = oracle.offsets(cnt.numpy(), 4096)
    assert_bits_equal(to_np(off), want_off, "send_data_offset")
    assert_bits_equal(to_np(send), want_trip, "send_data")
    assert_bits_equal(to_np(recv), want_trip, "recv_data")


@pytest.mark.parametrize("T,K,E,dtype,neg", [
    (1, 1, 4, torch.int64, 0.0),
    (3, 2, 2, torch.int32, 0.0),
    (65, 5, 7, torch.int64, 0.3),
    (128, 2, 8, torch.int64, 0.0),
    (1023, 8, 512, torch.int32, 0.0),
    (4096, 8, 256, torch.int64, 0.0),
    (8000, 16, 512, torch.int64, 0.02),
])
def test_dispatch_plan(gpu, oracle, T, K, E, dtype, neg):
    announce("plan T=%d K=%d E=%d" % (T, K, E))
    if (T, K, E) == (4096, 8, 256):
        ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=44)
        ids = ids.to(dtype)
    else:
        ids = _random_ids(T, K, E, seed=T * 7 + K, neg_frac=neg, dtype=dtype)
    plan = cam.moe_dispatch_plan(ids.to(gpu), E)
    idx_np = ids.numpy().astype(np.int64)
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    assert_bits_equal(to_np(plan["send_token_idx"]), pos, "send_token_idx")
    assert_bits_equal(to_np(plan["num_tokens_per_expert"]), cnt, "num_tokens_per_expert")
    assert_bits_equal(to_np(plan["send_offset"]), off, "send_offset")
    assert_bits_equal(to_np(plan["recv_offset"]), off, "recv_offset")
    assert_bits_equal(to_np(plan["recv_count"]), (off + cnt).astype(np.int32), "recv_count")
    assert_bits_equal(to_np(plan["num_recv_tokens_per_expert"]), cnt.astype(np.int64), "tokens per expert")
    assert int(plan["total"].item()) == int(cnt.sum())
    # the plan is a permutation: stable argsort of the flat ids
    flat = idx_np.reshape(-1)
    valid = flat >= 0
    rows = (off[np.maximum(flat, 0)] + pos.reshape(-1))[valid]
    order = np.argsort(flat[valid], kind="stable")
    assert np.array_equal(rows[order], np.arange(valid.sum()))


def test_dispatch_plan_is_deterministic(gpu):
    announce("plan determinism")
    ids, _ = synth.sigmoid_zipf_routing(4096, 256, 8, seed=44)
    ids = ids.to(gpu)
    a = cam.moe_dispatch_plan(ids, 256)["send_token_idx"].clone()
    for _ in range(5):
        b = cam.moe_dispatch_plan(ids, 256)["send_token_idx"]
        assert torch.equal(a, b)


def _dispatch_case(gpu, oracle, T, K, E, H, quant_mode, seed, neg=0.0, zero_rows=()):
    ids = _random_ids(T, K, E, seed=seed, neg_frac=neg, dtype=torch.int64)
    x = synth.normal_bf16(T, H, seed=seed + 1)
    for r in zero_rows:
        x[r] = 0
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    total = int(cnt.sum())
    plan = cam.moe_dispatch_plan(ids.to(gpu), E)
    recv_x, scales, assist = cam.moe_dispatch_normal(
        x.to(gpu), ids.to(gpu), plan["send_offset"], plan["send_token_idx"], plan["recv_offset"], plan["recv_count"],
        total, E, quant_mode=quant_mode)
    variant = {0: 0, 2: 1, 3: 2}[quant_mode]
    want_x, want_s, want_src = oracle.dispatch(synth.bf16_bits(x), idx_np, off, pos, E, variant, total)
    n = max(total, 0)
    assert_bits_equal(to_np(recv_x)[:n], want_x[:n], "recv_x")
    assert_bits_equal(to_np(assist)[:3 * n], want_src[:3 * n], "assist_info")
    if quant_mode != 0:
        assert_bits_equal(to_np(scales)[:n].view(np.uint32), want_s[:n].view(np.uint32), "recv_x_scales")


@pytest.mark.parametrize("quant_mode", [0, 2, 3])
@pytest.mark.parametrize("T,K,E,H", [(1, 1, 2, 1024), (37, 3, 8, 1024), (128, 2, 8, 1024), (64, 8, 32, 7168),
                                      (50, 16, 64, 4096), (19, 4, 16, 2064), (9, 2, 4, 1032)])
def test_dispatch_normal_bit_exact(gpu, oracle, T, K, E, H, quant_mode):
    announce("dispatch T=%d K=%d E=%d H=%d quant=%d" % (T, K, E, H, quant_mode))
    _dispatch_case(gpu, oracle, T, K, E, H, quant_mode, seed=T + H)


@pytest.mark.parametrize("quant_mode", [2, 3])
def test_dispatch_negative_ids_and_zero_rows(gpu, oracle, quant_mode):
    announce("dispatch edge quant=%d" % quant_mode)
    _dispatch_case(gpu, oracle, 77, 4, 16, 1024, quant_mode, seed=5, neg=0.25, zero_rows=(0, 13, 76))


def test_dispatch_full_size_config(gpu, oracle):
    """Dispatch-only benchmark shape: 4096 x 7168 bf16, 256 experts, top-8, int8 rows + fp32 scales."""
    announce("dispatch C2 full size")
    T, K, E, H = 4096, 8, 256, 7168
    ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=44)
    x = synth.normal_bf16(T, H, seed=44)
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    plan = cam.moe_dispatch_plan(ids.to(gpu), E)
    recv_x, scales, assist = cam.moe_dispatch_normal(
        x.to(gpu), ids.to(gpu), plan["send_offset"], plan["send_token_idx"], plan["recv_offset"], plan["recv_count"],
        T * K, E, quant_mode=2)
    want_x, want_s, want_src = oracle.dispatch(synth.bf16_bits(x), idx_np, off, pos, E, 1, T * K)
    assert_bits_equal(to_np(assist), want_src, "assist_info")
    assert_bits_equal(to_np(scales).view(np.uint32), want_s.view(np.uint32), "scales")
    assert_bits_equal(to_np(recv_x), want_x, "recv_x")
    # size-independent property: every row dequantises back to its source token within half a step
    src_t = torch.from_numpy(want_src.reshape(-1, 3)[:, 1].astype(np.int64)).to(gpu)
    xs = x.to(gpu).float()[src_t[:4096]]
    back = recv_x[:4096].float() * scales[:4096, None]
    assert ((back - xs).abs() <= scales[:4096, None] * 0.5001).all()


def test_moe_dispatch_prefill_surface(gpu, oracle):
    """The binding-level op: shapes, dtypes and devices of the four return values."""
    announce("moe_dispatch_prefill surface")
    T, K, E, H = 96, 4, 16, 1024
    ids, w = synth.softmax_topk_routing(T, E, K, seed=9)
    x = synth.normal_bf16(T, H, seed=10).to(gpu)
    per_rank, per_expert, in_rank = cam.get_dispatch_layout(ids.to(gpu), E, 1)
    ex, eidx, recv_count, per_expert_cpu = torch.ops.umdk_cam_op_lib.moe_dispatch_prefill(
        x, ids.to(gpu), w.to(gpu), per_rank, in_rank, per_expert, 0, "group", 0, 1)
    assert ex.shape == (T * K, H) and ex.dtype == torch.bfloat16
    assert eidx.shape == (3 * T * K,) and eidx.dtype == torch.int32
    assert recv_count.dtype == torch.int32 and recv_count.is_cuda
    assert per_expert_cpu.dtype == torch.int64 and not per_expert_cpu.is_cuda
    cnt, off, pos, _ = plan_oracle(oracle, ids.numpy(), E)
    want_x, _, want_src = oracle.dispatch(synth.bf16_bits(x.cpu()), ids.numpy(), off, pos, E, 0, T * K)
    assert_bits_equal(to_np(ex), want_x, "expand_x")
    assert_bits_equal(to_np(eidx), want_src, "expand_idx")
    assert_bits_equal(per_expert_cpu.numpy(), cnt.astype(np.int64), "num_recv_tokens_per_expert")
    # and back: combine of the un-quantised rows with weights summing to one returns x (K copies averaged)
    comb = torch.ops.umdk_cam_op_lib.moe_combine_prefill(ex, ids.to(gpu), w.to(gpu), eidx, recv_count, "group", 0, 1)
    assert (comb.float() - x.float()).abs().max().item() <= 0.04


def test_ids_at_or_above_E_are_skipped(gpu, oracle):
    """Ids >= E (which the reference kernel does not guard against) behave like negative ids everywhere."""
    announce("ids >= E")
    T, K, E, H = 90, 4, 16, 1024
    g = torch.Generator().manual_seed(31)
    ids = torch.randint(-2, E + 5, (T, K), generator=g, dtype=torch.int64)  # -2..20 with E = 16
    idx_np = ids.numpy()
    assert (idx_np >= E).sum() > 20 and (idx_np < 0).sum() > 10
    per_rank, per_expert, in_rank = cam.get_dispatch_layout(ids.to(gpu), E, 4)
    want_rank, want_cnt, want_in = oracle.layout(idx_np, E, 4, skip_out_of_range=True)
    assert_bits_equal(to_np(per_expert), want_cnt, "num_tokens_per_expert")
    assert_bits_equal(to_np(per_rank), want_rank, "num_tokens_per_rank")
    assert_bits_equal(to_np(in_rank), want_in, "is_token_in_rank")
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E, skip_out_of_range=True)
    plan = cam.moe_dispatch_plan(ids.to(gpu), E)
    assert_bits_equal(to_np(plan["send_token_idx"]), pos, "send_token_idx")
    assert_bits_equal(to_np(plan["num_tokens_per_expert"]), cnt, "num_tokens_per_expert")
    assert_bits_equal(to_np(plan["slot_row"]), oracle.rows_from_pos(idx_np, off, pos, E), "slot_row")
    total = int(cnt.sum())
    assert int(plan["total"].item()) == total == int(((idx_np >= 0) & (idx_np < E)).sum())
    x = synth.normal_bf16(T, H, seed=32)
    recv_x, scales, assist = cam.moe_dispatch_normal(
        x.to(gpu), ids.to(gpu), plan["send_offset"], plan["send_token_idx"], plan["recv_offset"], plan["recv_count"],
        total, E, quant_mode=2)
    want_x, want_s, want_src = oracle.dispatch(synth.bf16_bits(x), idx_np, off, pos, E, 1, total)
    assert_bits_equal(to_np(recv_x), want_x, "recv_x")
    assert_bits_equal(to_np(assist), want_src, "assist_info")
    assert_bits_equal(to_np(scales).view(np.uint32), want_s.view(np.uint32), "scales")


def _check_fused(oracle, d, x, idx_np, E, quant_mode, fp16=False):
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E, skip_out_of_range=True)
    total = int(cnt.sum())
    variant = {0: 0, 2: 1, 3: 2}[quant_mode]
    bits = x.view(torch.int16).numpy().view(np.uint16)
    want_x, want_s, want_src = oracle.dispatch(bits, idx_np, off, pos, E, variant, total, fp16=fp16)
    assert int(d["total"].item()) == total
    assert_bits_equal(to_np(d["send_token_idx"]), pos, "send_token_idx")
    assert_bits_equal(to_np(d["slot_row"]), oracle.rows_from_pos(idx_np, off, pos, E), "slot_row")
    assert_bits_equal(to_np(d["num_tokens_per_expert"]), cnt, "num_tokens_per_expert")
    assert_bits_equal(to_np(d["send_offset"]), off, "send_offset")
    assert_bits_equal(to_np(d["recv_count"]), (off + cnt).astype(np.int32), "recv_count")
    assert_bits_equal(to_np(d["num_recv_tokens_per_expert"]), cnt.astype(np.int64), "tokens per expert")
    got_x = d["recv_x"].view(torch.int16) if quant_mode == 0 else d["recv_x"]
    assert_bits_equal(got_x.cpu().numpy()[:total].view(want_x.dtype), want_x[:total], "recv_x")
    assert_bits_equal(to_np(d["expand_idx"])[:3 * total], want_src[:3 * total], "expand_idx")
    if quant_mode != 0:
        assert_bits_equal(to_np(d["recv_x_scales"])[:total].view(np.uint32), want_s[:total].view(np.uint32), "scales")


@pytest.mark.parametrize("quant_mode", [0, 2, 3])
@pytest.mark.parametrize("T,K,E,H,dtype,neg", [
    (1, 1, 2, 1024, torch.int64, 0.0),
    (37, 3, 8, 1024, torch.int32, 0.2),
    (300, 8, 256, 7168, torch.int64, 0.0),     # two chunks of 2048 ids
    (1500, 16, 512, 1032, torch.int64, 0.05),  # twelve chunks, odd row length
])
def test_dispatch_prefill_operator(gpu, oracle, T, K, E, H, dtype, neg, quant_mode):
    announce("dispatch prefill T=%d K=%d E=%d H=%d quant=%d" % (T, K, E, H, quant_mode))
    ids = _random_ids(T, K, E, seed=T + K + E, neg_frac=neg, dtype=dtype)
    x = synth.normal_bf16(T, H, seed=T + 3)
    if T > 4:
        x[4] = 0
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(gpu), E, quant_mode=quant_mode)
    _check_fused(oracle, d, x, ids.numpy().astype(np.int64), E, quant_mode)


def test_dispatch_prefill_workspace_reuse_and_garbage(gpu, oracle):
    """The same workspace, first filled with arbitrary bytes, serves several launches with different routings."""
    announce("dispatch prefill workspace reuse")
    from umdk_original_amd import _lib
    T, K, E, H = 513, 8, 64, 2048
    ws = torch.full((1 << 20,), 0xA5, dtype=torch.uint8, device=gpu)
    for seed, fill in ((1, None), (2, None), (3, 0xFF), (4, None)):
        if fill is not None:
            ws.fill_(fill)
        ids = _random_ids(T, K, E, seed=seed, neg_frac=0.1)
        x = synth.normal_bf16(T, H, seed=seed + 10)
        A = T * K
        i32 = dict(dtype=torch.int32, device=gpu)
        d = dict(recv_x=torch.empty((A, H), dtype=torch.int8, device=gpu),
                 recv_x_scales=torch.empty(A, dtype=torch.float32, device=gpu), expand_idx=torch.empty(3 * A, **i32),
                 send_token_idx=torch.empty((T, K), **i32), slot_row=torch.empty((T, K), **i32),
                 num_tokens_per_expert=torch.empty(E, **i32), send_offset=torch.empty(E, **i32),
                 recv_count=torch.empty(E, **i32),
                 num_recv_tokens_per_expert=torch.empty(E, dtype=torch.int64, device=gpu),
                 total=torch.empty(1, dtype=torch.int64, device=gpu))
        _lib.call("MoeDispatchPrefill", [x.to(gpu), ids.to(gpu), E, 1, 0, 2, d["recv_x"], d["recv_x_scales"],
                                         d["expand_idx"], d["send_token_idx"], d["slot_row"],
                                         d["num_tokens_per_expert"], d["send_offset"], d["recv_count"],
                                         d["num_recv_tokens_per_expert"], d["total"]], workspace=ws)
        _check_fused(oracle, d, x, ids.numpy(), E, 2)


def test_dispatch_prefill_full_size_config(gpu, oracle):
    announce("dispatch prefill C2 full size")
    T, K, E, H = 4096, 8, 256, 7168
    ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=44)
    x = synth.normal_bf16(T, H, seed=44)
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(gpu), E, quant_mode=2)
    _check_fused(oracle, d, x, ids.numpy(), E, 2)
    again = cam.moe_dispatch_fused(x.to(gpu), ids.to(gpu), E, quant_mode=2)
    assert torch.equal(again["recv_x"], d["recv_x"]) and torch.equal(again["send_token_idx"], d["send_token_idx"])


@pytest.mark.parametrize("quant_mode", [0, 2, 3])
def test_dispatch_fp16_activations(gpu, oracle, quant_mode):
    """fp16 activations (moe_dispatch_normal.cpp op_host :17-22 lists them beside bf16), both dispatch operators."""
    announce("dispatch fp16 quant=%d" % quant_mode)
    T, K, E, H = 70, 4, 16, 2048
    ids = _random_ids(T, K, E, seed=61, neg_frac=0.1)
    x = (torch.randn(T, H, generator=torch.Generator().manual_seed(62)) * 4).half()
    x[9] = 0
    x[10, :5] = torch.tensor([6e-8, -6e-5, 65504.0, -1e-3, 3e-7]).half()  # subnormals and the largest value
    idx_np = ids.numpy()
    d = cam.moe_dispatch_fused(x.to(gpu), ids.to(gpu), E, quant_mode=quant_mode)
    _check_fused(oracle, d, x, idx_np, E, quant_mode, fp16=True)
    plan = cam.moe_dispatch_plan(ids.to(gpu), E)
    total = int(plan["total"].item())
    recv_x, scales, assist = cam.moe_dispatch_normal(
        x.to(gpu), ids.to(gpu), plan["send_offset"], plan["send_token_idx"], plan["recv_offset"], plan["recv_count"],
        total, E, quant_mode=quant_mode)
    assert torch.equal(recv_x[:total], d["recv_x"][:total])
    assert torch.equal(assist[:3 * total], d["expand_idx"][:3 * total])
    if quant_mode:
        assert torch.equal(scales[:total], d["recv_x_scales"][:total])


def test_plain_c_caller_runs_layout_and_notify(gpu):
    """The C ABI called from a program in plain C (csrc/abi_consumer.c; no torch, no C++): DispatchLayout and
    NotifyDispatch on device memory from hipMalloc, compared with loops on the host."""
    import subprocess
    from umdk_original_amd import build
    announce("plain C caller of the ABI")
    p = subprocess.run([build.ABI_CONSUMER_PATH, "run"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=120)
    assert p.returncode == 0 and "run ok" in p.stdout, p.stdout
