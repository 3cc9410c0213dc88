"""GPU: the operators recorded into a HIP graph and replayed.  Phase 2 of every operator only enqueues kernels (no
allocation, no synchronisation, no memset nodes), so a caller may capture it; a replay must give what the same calls
give eagerly on the inputs the buffers hold at that moment, every time, with other work between the replays."""
import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce

pytestmark = pytest.mark.gpu


def _same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.view(torch.uint8), b.view(torch.uint8))


def test_graph_replays_of_the_whole_path_equal_eager_calls(gpu):
    announce("HIP graph: dispatch, GEMM operators, combine and the fused layer, three replays on changing inputs")
    T, E, K, H, I = 300, 32, 4, 1024, 512
    d = synth.ut_recipe(batch_size=T, hidden=H, intermediate=I, num_experts=E, top_k=K, seed=21)
    w1 = cam.prepack_weight(d["w1"].to(gpu), True)
    w2 = cam.prepack_weight(d["w2"].to(gpu), False)
    w1s, w2s = d["w1_scale"].to(gpu), d["w2_scale"].to(gpu)
    x = d["x"].to(gpu).clone()
    ids = d["ids"].to(torch.int32).to(gpu).clone()
    gates = d["gates"].to(gpu).clone()

    def path():
        """The stand-alone operators chained like the layer, and the fused layer itself."""
        dd = cam.moe_dispatch_fused(x, ids, E, quant_mode=2)
        gl = torch.cumsum(dd["num_recv_tokens_per_expert"], 0)
        y, ysc = cam.grouped_matmul_swiglu_quant(dd["recv_x"], dd["recv_x_scales"], w1, w1s, gl)
        rows = cam.grouped_matmul_dequant(y, ysc, w2, w2s, gl)
        chain = cam.moe_combine_gather(rows, None, dd["slot_row"], gates)
        fused, etn = cam.fused_deep_moe(x, ids, [w1], [w1s], [w2], [w2s], gates, None, None, "ep_group", 1, 0, E, 1, 0, 0,
                                        0)
        return chain, fused, etn, dd["slot_row"]

    warm = path()  # first-use initialisation outside the capture
    torch.cuda.synchronize()
    assert _same(warm[0], warm[1])  # the chain of operators and the fused operator agree bit for bit
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        recorded = path()
    for rep in range(3):
        # new tokens, routing and gates in the buffers the graph reads
        nd = synth.ut_recipe(batch_size=T, hidden=H, intermediate=I, num_experts=E, top_k=K, seed=30 + rep)
        x.copy_(nd["x"].to(gpu))
        ids.copy_(nd["ids"].to(torch.int32).to(gpu))
        gates.copy_(nd["gates"].to(gpu))
        if rep == 1:
            ids[::7, 1] = -1  # dropped entries change every count
        eager = [t.clone() for t in path()]  # the program's own eager work between the replays
        junk = torch.randn(1 << 20, device=gpu).sum()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("chain of operators", "fused layer", "expert_token_nums", "slot -> row map"), recorded,
                              eager):
            assert _same(a, b), "replay %d: %s differs from the eager call" % (rep, name)
        assert torch.isfinite(junk)


def test_graph_replay_of_the_fp8_layer_equals_eager(gpu):
    from test_gpu_fp8 import _layer_inputs
    announce("HIP graph: FP8 fused layer, three replays")
    T, H, E, K, I = 96, 1024, 8, 2, 512
    ids, w, x, w1, s1, w2, s2 = _layer_inputs(T, H, E, K, I, seed=5)
    w1p, w2p = cam.prepack_weight(w1.to(gpu), True), cam.prepack_weight(w2.to(gpu), False)
    s1, s2 = s1.to(gpu), s2.to(gpu)
    xs, idx, ws = x.to(gpu).clone(), ids.to(torch.int32).to(gpu).clone(), w.to(gpu).clone()

    def layer():
        return cam.fused_deep_moe_fp8(xs, idx, w1p, s1, w2p, s2, ws)

    layer()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        recorded = layer()
    for rep in range(3):
        nids, nw, nx = _layer_inputs(T, H, E, K, I, seed=40 + rep)[:3]
        xs.copy_(nx.to(gpu))
        idx.copy_(nids.to(torch.int32).to(gpu))
        ws.copy_(nw.to(gpu))
        eager = [t.clone() for t in layer()]
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert _same(recorded[0], eager[0]) and _same(recorded[1], eager[1]), "replay %d" % rep
