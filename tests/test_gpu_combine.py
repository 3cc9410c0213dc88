"""GPU parity: weighted un-permute / reduce against the CPU oracle (bit-exact bf16)."""
import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce, to_np, plan_oracle, assert_bits_equal

pytestmark = pytest.mark.gpu


def _case(gpu, oracle, T, K, E, H, seed, drop=0):
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=seed)
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    A = T * K
    y = synth.normal_bf16(A, H, seed=seed + 1)
    _, _, src = oracle.dispatch(np.zeros((T, 8), np.uint16), idx_np, off, pos, E, 0, A)
    if drop:  # rows that name no slot: their slots must contribute nothing
        src = src.copy().reshape(-1, 3)
        src[:drop, 1] = -1
        src = src.reshape(-1)
    row_of = oracle.rows_from_src_info(src, A, T, K)
    want = oracle.combine(synth.bf16_bits(y), row_of, w.numpy())
    recv_count = torch.from_numpy((off + cnt).astype(np.int32)).to(gpu)
    got = cam.moe_combine_normal(y.to(gpu), torch.from_numpy(src).to(gpu), recv_count, w.to(gpu))
    assert got.dtype == torch.bfloat16 and got.shape == (T, H)
    assert_bits_equal(to_np(got), want, "combined x")
    return got


@pytest.mark.parametrize("T,K,E,H", [(1, 1, 2, 1024), (128, 2, 8, 1024), (33, 8, 64, 7168), (57, 16, 32, 4096),
                                      (21, 3, 8, 1032)])
def test_combine_bit_exact(gpu, oracle, T, K, E, H):
    announce("combine T=%d K=%d E=%d H=%d" % (T, K, E, H))
    _case(gpu, oracle, T, K, E, H, seed=T + K)


def test_combine_missing_slots(gpu, oracle):
    announce("combine with absent slots")
    _case(gpu, oracle, 64, 4, 16, 2048, seed=3, drop=9)


def test_combine_decode_shape(gpu, oracle):
    announce("combine decode T=128 H=7168 K=8")
    _case(gpu, oracle, 128, 8, 256, 7168, seed=46)


def test_combine_full_size_config(gpu, oracle):
    """Combine-only benchmark shape: 32768 bf16 rows x 7168 gathered back to 4096 tokens, top-8."""
    announce("combine C4 full size")
    got = _case(gpu, oracle, 4096, 8, 256, 7168, seed=46)
    assert torch.isfinite(got.float()).all()


def _wire_case(gpu, oracle, T, K, E, H, seed):
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=seed)
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    A = T * K
    y = synth.normal_bf16(A, H, seed=seed + 1)
    y[0] = 0  # an all-zero row: q = 0, scale 0
    if A > 2:   # tiny and huge rows: scales and rebuilt values at both ends of the bf16 range
        y[1] = (y[1].float() * 1e-37).bfloat16()
        y[2] = (y[2].float() * 1e36).bfloat16()
    packed = oracle.comm_quant_rows(synth.bf16_bits(y))
    row_of = oracle.rows_from_pos(idx_np, off, pos, E)
    want = oracle.combine(oracle.comm_dequant_rows(packed, H), row_of, w.numpy())
    got = cam.moe_combine_gather(torch.from_numpy(packed.view(np.int8)).to(gpu), None,
                                 torch.from_numpy(row_of.reshape(T, K)).to(gpu), w.to(gpu))
    assert got.dtype == torch.bfloat16 and got.shape == (T, H)
    assert_bits_equal(to_np(got), want, "combined x from wire rows")
    return y, packed, row_of, w, got


@pytest.mark.parametrize("T,K,E,H", [(1, 1, 2, 1024), (33, 8, 64, 7168), (57, 16, 32, 4096), (21, 3, 8, 1032)])
def test_combine_from_wire_rows_bit_exact(gpu, oracle, T, K, E, H):
    """Rows quantised for the wire (int8 + bf16 scale per 8 columns) are dequantised inside the gather."""
    announce("combine from wire rows T=%d K=%d E=%d H=%d" % (T, K, E, H))
    _wire_case(gpu, oracle, T, K, E, H, seed=T + K + 5)


@pytest.mark.parametrize("T,K,E,H", [(33, 8, 64, 7168), (21, 3, 8, 1032)])
def test_combine_from_wire_rows_of_fp16_rows(gpu, oracle, T, K, E, H):
    """Wire rows made from IEEE fp16 rows carry fp16 block scales; an fp16 output selects that reading."""
    announce("combine from fp16 wire rows T=%d K=%d E=%d H=%d" % (T, K, E, H))
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=T + 9)
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    A = T * K
    y = synth.normal_bf16(A, H, seed=T + 10).half()
    y[0] = 0
    y[1] = y[1] * 1e-4   # block scales in fp16's subnormal range
    y[2] = y[2] * 1e4
    bits = y.view(torch.int16).numpy().view(np.uint16)
    packed = oracle.comm_quant_rows(bits, fp16=True)
    row_of = oracle.rows_from_pos(idx_np, off, pos, E)
    want = oracle.combine_act(oracle.comm_dequant_rows(packed, H, fp16=True), row_of, w.numpy(), True)
    out = torch.empty((T, H), dtype=torch.float16, device=gpu)
    got = cam.moe_combine_gather(torch.from_numpy(packed.view(np.int8)).to(gpu), None,
                                 torch.from_numpy(row_of.reshape(T, K)).to(gpu), w.to(gpu), out=out)
    assert_bits_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), want, "combined x from fp16 wire rows")


def test_combine_from_wire_rows_full_size(gpu, oracle):
    """C4 shape with wire rows: bit-exact against the oracle, and close to the combine of the unquantised rows."""
    announce("combine from wire rows, C4 full size")
    T, K, E, H = 4096, 8, 256, 7168
    y, packed, row_of, w, got = _wire_case(gpu, oracle, T, K, E, H, seed=46)
    exact = cam.moe_combine_gather(y.to(gpu), None, torch.from_numpy(row_of.reshape(T, K)).to(gpu), w.to(gpu))
    diff = (got.float() - exact.float()).abs().max().item()
    assert diff <= 0.02 * exact.float().abs().max().item() + 1e-3


def test_combine_identity_and_linearity(gpu, oracle):
    announce("combine properties")
    T, K, E, H = 256, 1, 16, 1024
    ids, _ = synth.softmax_topk_routing(T, E, K, seed=11)
    cnt, off, pos, _ = plan_oracle(oracle, ids.numpy(), E)
    x = synth.normal_bf16(T, H, seed=12).to(gpu)
    plan = cam.moe_dispatch_plan(ids.to(gpu), E)
    rx, _, assist = cam.moe_dispatch_normal(x, ids.to(gpu), plan["send_offset"], plan["send_token_idx"],
                                            plan["recv_offset"], plan["recv_count"], T, E)
    ones = torch.ones(T, 1, device=gpu)
    back = cam.moe_combine_normal(rx, assist, plan["recv_count"], ones)
    assert torch.equal(back, x)  # K = 1, weight 1: combine undoes dispatch exactly
    half = cam.moe_combine_normal(rx, assist, plan["recv_count"], ones * 0.5)
    assert torch.equal(half.float(), (x.float() * 0.5).bfloat16().float())


def test_combine_index_then_gather_equals_normal(gpu, oracle):
    announce("combine index + gather")
    T, K, E, H = 200, 8, 64, 2048
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=21)
    cnt, off, pos, _ = plan_oracle(oracle, ids.numpy(), E)
    A = T * K
    _, _, src = oracle.dispatch(np.zeros((T, 8), np.uint16), ids.numpy(), off, pos, E, 0, A)
    src_d = torch.from_numpy(src).to(gpu)
    recv_count = torch.from_numpy((off + cnt).astype(np.int32)).to(gpu)
    slot = cam.moe_combine_index(src_d, A, T, K)
    assert_bits_equal(to_np(slot), oracle.rows_from_src_info(src, A, T, K), "slot_row")
    for seed in (1, 2):  # one index, several gathers
        y = synth.normal_bf16(A, H, seed=seed).to(gpu)
        got = cam.moe_combine_gather(y, src_d, slot, w.to(gpu))
        want = cam.moe_combine_normal(y, src_d, recv_count, w.to(gpu))
        assert torch.equal(got, want)
        # the map the dispatch operators hand out, trusted as it stands (no triples)
        plan = cam.moe_dispatch_plan(ids.to(gpu), E)
        got2 = cam.moe_combine_gather(y, None, plan["slot_row"], w.to(gpu), ep_recv_counts=recv_count)
        assert torch.equal(got2, want)


def test_combine_ignores_rows_past_the_receive_total(gpu, oracle):
    """Buffers sized for a worst case: rows at or past epRecvCounts[E-1] hold triples of an earlier routing that
    name valid slots; they must not be read (moe_combine_normal.h:206-207 stops at the receive total)."""
    announce("combine with a stale tail")
    T, K, E, H = 64, 4, 16, 1024
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=71)
    ids[::3, 1] = -1  # fewer than T*K rows this time
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    total = int(cnt.sum())
    A = T * K
    assert total < A
    y = synth.normal_bf16(A, H, seed=72)
    _, _, src_now = oracle.dispatch(np.zeros((T, 8), np.uint16), idx_np, off, pos, E, 0, A)
    src = src_now.copy().reshape(-1, 3)
    # the tail keeps triples from an earlier, full routing: they name slots that exist now as well
    tail = np.arange(total, A)
    src[tail, 0] = 0
    src[tail, 1] = tail % T
    src[tail, 2] = (tail // T) % K
    src = src.reshape(-1)
    row_of = oracle.rows_from_src_info(src_now, total, T, K)
    want = oracle.combine(synth.bf16_bits(y), row_of, w.numpy())
    recv_count = torch.from_numpy((off + cnt).astype(np.int32)).to(gpu)
    ws = torch.full((T * K * 4 + 256,), 0xFF, dtype=torch.uint8, device=gpu)
    from umdk_original_amd import _lib
    for _ in range(2):
        out = torch.empty((T, H), dtype=torch.bfloat16, device=gpu)
        _lib.call("MoeCombineNormal", [y.to(gpu), torch.from_numpy(src).to(gpu), recv_count, w.to(gpu), None, "", 1, 0,
                                       "", 1, 0, E, 0, out], workspace=ws)
        assert_bits_equal(to_np(out), want, "combined x")
        # poison the inverse map with the stale rows, as a racing stale triple would have left it
        ws[:T * K * 4].view(torch.int32).copy_(torch.from_numpy(
            oracle.rows_from_src_info(src, A, T, K).reshape(-1)).to(gpu))


def test_prefill_with_worst_case_rows_then_combine(gpu, oracle):
    """moe_dispatch_prefill with num_worst_tokens > 0 leaves the tail of expand_x / expand_idx unwritten;
    moe_combine_prefill must still return the right tokens."""
    announce("prefill worst-case sizing + combine")
    T, K, E, H = 48, 4, 8, 1024
    ids, w = synth.softmax_topk_routing(T, E, K, seed=81)
    ids[::4, 0] = -1
    x = synth.normal_bf16(T, H, seed=82).to(gpu)
    per_rank, per_expert, in_rank = cam.get_dispatch_layout(ids.to(gpu), E, 1)
    # first a full routing into the same allocator blocks, so that the tail holds plausible triples
    full_ids, _ = synth.softmax_topk_routing(T, E, K, seed=83)
    first = cam.moe_dispatch_prefill(x, full_ids.to(gpu), w.to(gpu), per_rank, in_rank, per_expert, T * K, "g", 0, 1)
    del first
    ex, eidx, recv_count, _ = cam.moe_dispatch_prefill(x, ids.to(gpu), w.to(gpu), per_rank, in_rank, per_expert,
                                                       T * K, "g", 0, 1)
    assert ex.shape[0] == T * K
    comb = cam.moe_combine_prefill(ex, ids.to(gpu), w.to(gpu), eidx, recv_count, "g", 0, 1)
    cnt, off, pos, _ = plan_oracle(oracle, ids.numpy(), E)
    total = int(cnt.sum())
    want_x, _, want_src = oracle.dispatch(synth.bf16_bits(x.cpu()), ids.numpy(), off, pos, E, 0, total)
    want = oracle.combine(want_x, oracle.rows_from_src_info(want_src, total, T, K), w.numpy())
    assert_bits_equal(to_np(comb), want, "combined x")


def test_combine_fp16_rows_bit_exact(gpu, oracle):
    """fp16 rows in, fp16 out (moe_combine_normal.cpp(op_host):18,49 lists bf16 and fp16)."""
    announce("combine fp16 rows")
    T, K, E, H = 45, 4, 16, 2048
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=61)
    idx_np = ids.numpy()
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    y = (torch.randn(T * K, H, generator=torch.Generator().manual_seed(62)) * 3).half()
    row_of = oracle.rows_from_pos(idx_np, off, pos, E)
    want = oracle.combine_act(y.view(torch.int16).numpy().view(np.uint16), row_of, w.numpy(), True)
    got = cam.moe_combine_gather(y.to(gpu), None, torch.from_numpy(row_of.reshape(T, K)).to(gpu), w.to(gpu))
    assert got.dtype == torch.float16
    assert_bits_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), want, "combined fp16 x")


@pytest.mark.parametrize("T,K,E,H,wire,fp16", [(33, 8, 64, 7168, False, False), (21, 3, 8, 1032, False, False),
                                                 (57, 16, 32, 4096, True, False), (19, 4, 8, 1032, True, False),
                                                 (40, 8, 32, 2048, False, True)])
def test_combine_with_shared_expert_rows(gpu, oracle, T, K, E, H, wire, fp16):
    """The shared expert's row is added un-weighted after the routed rows, before the one rounding
    (cam_moe_distribute_combine.h:757-774), for 16-bit rows of either type and for wire rows."""
    announce("combine + shared rows T=%d K=%d E=%d H=%d wire=%d fp16=%d" % (T, K, E, H, wire, fp16))
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=T)
    idx_np = ids.numpy()
    idx_np[T // 2, 0] = -1  # an absent slot; and one token with no routed rows at all
    idx_np[0, :] = -1
    cnt, off, pos, _ = plan_oracle(oracle, idx_np, E)
    A = T * K
    row_of = oracle.rows_from_pos(idx_np, off, pos, E)
    y = synth.normal_bf16(A, H, seed=T + 1)
    sh = synth.normal_bf16(T, H, seed=T + 2)
    if fp16:
        y, sh = y.half(), sh.half()
        yb, sb = y.view(torch.int16).numpy().view(np.uint16), sh.view(torch.int16).numpy().view(np.uint16)
    else:
        yb, sb = synth.bf16_bits(y), synth.bf16_bits(sh)
    slot = torch.from_numpy(row_of.reshape(T, K)).to(gpu)
    if wire:
        packed = oracle.comm_quant_rows(yb)
        want = oracle.combine_shared(oracle.comm_dequant_rows(packed, H), row_of, w.numpy(), sb)
        got = cam.moe_combine_gather(torch.from_numpy(packed.view(np.int8)).to(gpu), None, slot, w.to(gpu),
                                     shared_x=sh.to(gpu))
    else:
        want = oracle.combine_shared(yb, row_of, w.numpy(), sb, fp16=fp16)
        got = cam.moe_combine_gather(y.to(gpu), None, slot, w.to(gpu), shared_x=sh.to(gpu))
    gb = got.cpu().view(torch.int16).numpy().view(np.uint16)
    assert_bits_equal(gb, want, "combined x with shared rows")
    assert np.array_equal(gb[0], sb[0])  # no routed rows: the shared row alone, bit for bit
