"""GPU parity of the entry point that allocates nothing: MoeDispatchPlanNoAlloc against MoeDispatchPlan.

Two calls in a row share the library's built-in scratch array; the second is smaller than the first, so
whatever the first left behind in the array lies beyond what the second rewrites."""
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import _lib, synth
from gpu_util import announce

pytestmark = pytest.mark.gpu

OUTPUTS = ("send_token_idx", "num_tokens_per_expert", "send_offset", "recv_offset", "recv_count",
           "num_recv_tokens_per_expert", "total", "slot_row")


def _plan_no_alloc(ids, E):
    T, K = ids.shape
    dev = ids.device
    i32 = dict(dtype=torch.int32, device=dev)
    out = dict(send_token_idx=torch.empty((T, K), **i32), num_tokens_per_expert=torch.empty(E, **i32),
               send_offset=torch.empty(E, **i32), recv_offset=torch.empty(E, **i32), recv_count=torch.empty(E, **i32),
               num_recv_tokens_per_expert=torch.empty(E, dtype=torch.int64, device=dev),
               total=torch.empty(1, dtype=torch.int64, device=dev), slot_row=torch.empty((T, K), **i32))
    _lib.call_direct("MoeDispatchPlanNoAlloc", [ids, E, 1, 0] + [out[k] for k in OUTPUTS])
    return out


def test_plan_no_alloc_matches_plan_on_two_calls_in_a_row(gpu):
    announce("plan, no-alloc entry point: T=4096 K=8 E=256, then T=77 K=3 E=16")
    cases = []
    ids, _ = synth.sigmoid_zipf_routing(4096, 256, 8, seed=44)
    cases.append((ids.to(gpu), 256))
    g = torch.Generator().manual_seed(5)
    small = torch.randint(-1, 16, (77, 3), generator=g, dtype=torch.int64).to(torch.int32)
    cases.append((small.to(gpu), 16))
    for ids_d, E in cases:  # back to back on one stream, nothing in between
        got = _plan_no_alloc(ids_d, E)
        want = cam.moe_dispatch_plan(ids_d, E)
        for k in OUTPUTS:
            assert torch.equal(got[k], want[k]), (k, tuple(ids_d.shape))
    # and in the other order of issue: both no-alloc calls first, then both references
    got = [_plan_no_alloc(i, e) for i, e in cases]
    want = [cam.moe_dispatch_plan(i, e) for i, e in cases]
    for gd, wd in zip(got, want):
        for k in OUTPUTS:
            assert torch.equal(gd[k], wd[k]), k


def test_plan_no_alloc_rejects_oversized_input(gpu):
    announce("plan, no-alloc entry point: size limit")
    ids = torch.zeros((131072 // 8 + 1, 8), dtype=torch.int32, device=gpu)
    with pytest.raises(cam.CamError) as err:
        _plan_no_alloc(ids, 8)
    assert err.value.status == _lib.CAM_ERR_RANGE and "131072" in str(err.value)
    ok = torch.zeros((131072 // 8, 8), dtype=torch.int32, device=gpu)  # exactly at the limit
    got = _plan_no_alloc(ok, 8)
    assert int(got["total"].item()) == 131072 and int(got["num_tokens_per_expert"][0].item()) == 131072


def test_plan_no_alloc_under_graph_capture(gpu):
    """What the entry point is for: two calls recorded into one HIP graph (after a call outside any capture has
    resolved the scratch array's address on this device), replayed several times with eager work in between, every
    replay compared with MoeDispatchPlan."""
    announce("plan, no-alloc entry point: captured in a HIP graph")
    ids_a, _ = synth.sigmoid_zipf_routing(2048, 64, 8, seed=3)
    ids_a = ids_a.to(torch.int32).to(gpu)
    ids_b = torch.randint(0, 16, (300, 4), generator=torch.Generator().manual_seed(4)).to(torch.int32).to(gpu)
    _plan_no_alloc(ids_b, 16)  # outside capture: the first call on a device looks the array up
    torch.cuda.synchronize()
    T, K = ids_a.shape
    i32 = dict(dtype=torch.int32, device=gpu)

    def outputs(t, k, e):
        return dict(send_token_idx=torch.empty((t, k), **i32), num_tokens_per_expert=torch.empty(e, **i32),
                    send_offset=torch.empty(e, **i32), recv_offset=torch.empty(e, **i32),
                    recv_count=torch.empty(e, **i32),
                    num_recv_tokens_per_expert=torch.empty(e, dtype=torch.int64, device=gpu),
                    total=torch.empty(1, dtype=torch.int64, device=gpu), slot_row=torch.empty((t, k), **i32))

    oa, ob = outputs(T, K, 64), outputs(300, 4, 16)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            _lib.call_direct("MoeDispatchPlanNoAlloc", [ids_a, 64, 1, 0] + [oa[k] for k in OUTPUTS])
            _lib.call_direct("MoeDispatchPlanNoAlloc", [ids_b, 16, 1, 0] + [ob[k] for k in OUTPUTS])
    torch.cuda.current_stream().wait_stream(side)
    want_a, want_b = cam.moe_dispatch_plan(ids_a, 64), cam.moe_dispatch_plan(ids_b, 16)
    for replay in range(3):
        for d in (oa, ob):
            for k in OUTPUTS:
                d[k].fill_(-7)  # eager work between the replays; also proves a replay rewrites every output
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for got, want in ((oa, want_a), (ob, want_b)):
            for k in OUTPUTS:
                assert torch.equal(got[k], want[k]), (replay, k)
