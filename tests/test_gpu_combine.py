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
