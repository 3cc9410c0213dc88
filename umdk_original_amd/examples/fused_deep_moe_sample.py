"""One rank's share of the reference's sample (src/cam/examples/fused_deep_moe_sample.py:295-468) on one MI355X.

The reference sample spawns 16 NPU processes, builds bs x H tokens, round-robin expert ids, int8 weights with
bf16-rounded per-channel scales, calls torch.ops.umdk_cam_op_lib.fused_deep_moe and compares it with a chain of small
operators under atol 2.0 / rtol 0.02, with exact equality of expert_token_nums (…/test_fused_deep_moe.py:416-419).
This script does the same on one GPU: the fused operator against the chain dispatch -> GMM1 + SwiGLU + re-quant ->
GMM2 -> combine built from this library's stand-alone operators.

    python -m umdk_original_amd.examples.fused_deep_moe_sample [--bs 64] [--hidden 7168] [--inter 2048]
                                                                [--experts 64] [--topk 8]
"""
import argparse

import torch

import umdk_original_amd as cam
from umdk_original_amd import synth


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--bs", type=int, default=64)
    ap.add_argument("--hidden", type=int, default=7168)
    ap.add_argument("--inter", type=int, default=2048)
    ap.add_argument("--experts", type=int, default=64)
    ap.add_argument("--topk", type=int, default=8)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    d = synth.ut_recipe(batch_size=args.bs, hidden=args.hidden, intermediate=args.inter, num_experts=args.experts,
                        top_k=args.topk, seed=42)
    x, ids, gates = d["x"].to(dev), d["ids"].to(torch.int32).to(dev), d["gates"].to(dev)
    w1 = cam.prepack_weight(d["w1"].to(dev), True)     # once after loading: the FRACTAL_NZ cast of the reference
    w2 = cam.prepack_weight(d["w2"].to(dev), False)
    w1s, w2s = d["w1_scale"].to(dev), d["w2_scale"].to(dev)

    # the fused operator, through the reference's torch schema
    out, expert_token_nums = torch.ops.umdk_cam_op_lib.fused_deep_moe(
        x, ids, [w1], [w1s], [w2], [w2s], gates, None, None, "", 1, 0, args.experts, 1, 0, 0, 0)

    # the same layer as a chain of stand-alone operators
    disp = cam.moe_dispatch_fused(x, ids, args.experts, quant_mode=3)            # plan + permute + per-token int8
    group_list = torch.cumsum(disp["num_tokens_per_expert"].to(torch.int64), 0)
    y, y_scale = cam.grouped_matmul_swiglu_quant(disp["recv_x"], disp["recv_x_scales"], w1, w1s, group_list)
    rows = cam.grouped_matmul_dequant(y, y_scale, w2, w2s, group_list)
    chain = cam.moe_combine_gather(rows, None, disp["slot_row"], gates)
    torch.cuda.synchronize()

    torch.testing.assert_close(out.float(), chain.float(), atol=2.0, rtol=0.02)
    assert torch.equal(expert_token_nums.cpu(), disp["num_tokens_per_expert"].to(torch.int64).cpu())
    same = bool(torch.equal(out.view(torch.int16), chain.view(torch.int16)))
    print("fused_deep_moe vs operator chain: within atol 2.0 / rtol 0.02, expert_token_nums equal; "
          "bit-identical: %s; output %s, %d rows dispatched" % (same, tuple(out.shape), int(group_list[-1])))


if __name__ == "__main__":
    main()
