"""GPU parity of the SHMEM operator pair on one rank (MoeDispatchShmem / MoeCombineShmem) against the CPU oracle:
every integer output, the int8 rows and their scales, and the combined rows are compared bit for bit."""
import numpy as np
import pytest
import torch

import umdk_original_amd as cam
from umdk_original_amd import synth
from gpu_util import announce, to_np, assert_bits_equal

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("T,K,E,H,quant,smooth,fp16,ttype", [
    (1, 1, 2, 1024, 2, False, False, 1), (64, 8, 32, 7168, 2, False, False, 0), (37, 4, 8, 1032, 2, True, False, 1),
    (300, 8, 64, 4096, 2, True, True, 0), (128, 2, 8, 1024, 0, False, False, 1), (50, 3, 16, 2048, 0, False, True, 0),
    (700, 8, 256, 7168, 2, True, False, 1)])
def test_dispatch_shmem_bit_exact(gpu, oracle, T, K, E, H, quant, smooth, fp16, ttype):
    announce("dispatch shmem T=%d K=%d E=%d H=%d quant=%d smooth=%d fp16=%d type=%d" % (T, K, E, H, quant, smooth, fp16, ttype))
    ids, _ = synth.sigmoid_zipf_routing(T, E, K, seed=T + E)
    ids = ids.to(torch.int32)
    if T > 4:
        ids[2, 0] = -1      # names no expert
        ids[3, K - 1] = E   # neither does an id past the table
    x = synth.normal_bf16(T, H, seed=T + 1)
    if T > 8:
        x[5] = 0            # an all-zero token
    if fp16:
        x = x.half()
    sm = None
    if smooth:
        g = torch.Generator().manual_seed(T)
        sm = (torch.rand(E, H, generator=g) * 3.75 + 0.25).float()
    want = oracle.dispatch_shmem(_bits(x), ids.numpy(), E, quant, smooth=None if sm is None else sm.numpy(), fp16=fp16,
                                 token_nums_type=ttype)
    got = cam.moe_dispatch_shmem(x.to(gpu), ids.to(gpu), None if sm is None else sm.to(gpu), None, 1, 0, E, 1, 0, 0, 1, 0,
                                 quant, 0, ttype, 0)
    total = want[5]
    assert got[0].shape == (T * min(K, E), H) and got[2].shape == (T * K,) and got[3].dtype == torch.int64
    assert_bits_equal(to_np(got[2]), want[2], "expandIdx")
    assert_bits_equal(to_np(got[3]), want[3], "expertTokenNums")
    assert_bits_equal(to_np(got[4]), want[4], "epRecvCount")
    if quant:
        assert_bits_equal(to_np(got[0])[:total], want[0][:total], "expandX (int8)")
        assert_bits_equal(to_np(got[1])[:total].view(np.uint32), want[1][:total].view(np.uint32), "dynamicScales")
    else:
        assert_bits_equal(_bits(got[0])[:total], want[0][:total], "expandX (copy)")


@pytest.mark.parametrize("T,K,E,H,comm,fp16", [(1, 1, 2, 1024, 0, False), (64, 8, 32, 7168, 0, False),
                                                (37, 4, 8, 1032, 2, False), (300, 8, 64, 4096, 2, False),
                                                (50, 3, 16, 2048, 0, True), (45, 4, 8, 1032, 2, True),
                                                (200, 8, 64, 7168, 2, True)])
def test_combine_shmem_bit_exact(gpu, oracle, T, K, E, H, comm, fp16):
    announce("combine shmem T=%d K=%d E=%d H=%d comm=%d fp16=%d" % (T, K, E, H, comm, fp16))
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=T + E + 1)
    ids = ids.to(torch.int32)
    if T > 4:
        ids[1, 0] = -1
    x = synth.normal_bf16(T, H, seed=T + 2)
    d = cam.moe_dispatch_shmem(x.to(gpu), ids.to(gpu), None, None, 1, 0, E, 1, 0, 0, 1, 0, 0, 0, 1, 0)
    A = d[0].size(0)
    y = synth.normal_bf16(A, H, seed=T + 3)
    y[0] = 0
    if fp16:
        y = y.half()
    got = cam.moe_combine_shmem(y.to(gpu), ids.to(gpu), d[2], d[4], w.to(gpu), epWorldSize=1, moeExpertNum=E,
                                commQuantMode=comm)
    want = oracle.combine_shmem(_bits(y), ids.numpy(), to_np(d[2]), to_np(d[4]), w.numpy(), E, fp16=fp16,
                                comm_quant=comm == 2)
    assert got.dtype == y.dtype and got.shape == (T, H)
    assert_bits_equal(_bits(got), want, "combined rows")


def test_shmem_round_trip_restores_the_tokens(gpu):
    """K = 1, weight 1, no quantisation: combine(dispatch(x)) == x (a size-independent property, at C2's width)."""
    announce("shmem dispatch -> combine round trip")
    T, E, H = 2048, 64, 7168
    x = synth.normal_bf16(T, H, seed=9).to(gpu)
    ids = torch.randint(0, E, (T, 1), generator=torch.Generator().manual_seed(9)).to(torch.int32).to(gpu)
    d = cam.moe_dispatch_shmem(x, ids, None, None, 1, 0, E, 1, 0, 0, 1, 0, 0, 0, 1, 0)
    out = cam.moe_combine_shmem(d[0], ids, d[2], d[4], torch.ones(T, 1, device=gpu), epWorldSize=1, moeExpertNum=E)
    assert torch.equal(out, x)


def test_shmem_torch_ops_are_registered_with_the_reference_schemas(gpu, oracle):
    """torch.ops.umdk_cam_op_lib.moe_dispatch_shmem / moe_combine_shmem (src/cam/comm_operator/pybind/pybind.cpp:
    32-41): positional calls with the reference's argument lists give the oracle's results."""
    announce("shmem ops through torch.ops")
    T, K, E, H = 48, 4, 16, 2048
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=3)
    ids = ids.to(torch.int32)
    x = synth.normal_bf16(T, H, seed=4)
    ops = torch.ops.umdk_cam_op_lib
    d = ops.moe_dispatch_shmem(x.to(gpu), ids.to(gpu), None, None, 1, 0, E, 1, 0, 0, 1, 0, 2, 0, 1, 0)
    assert len(d) == 6
    want = oracle.dispatch_shmem(synth.bf16_bits(x), ids.numpy(), E, 2)
    total = want[5]
    assert_bits_equal(to_np(d[0])[:total], want[0][:total], "expandX")
    assert_bits_equal(to_np(d[2]), want[2], "expandIdx")
    y = synth.normal_bf16(d[0].size(0), H, seed=5)
    out = ops.moe_combine_shmem(y.to(gpu), ids.to(gpu), d[2], d[4], w.to(gpu), None, None, None, None, None, None,
                                1, 0, E, 1, 0, 0, 1, 0, 0, 0, 0, 0, 0)
    assert_bits_equal(to_np(out), oracle.combine_shmem(synth.bf16_bits(y), ids.numpy(), want[2], want[4], w.numpy(), E),
                      "combined rows")


def test_operators_accept_inputs_that_require_grad_and_return_no_gradients(gpu):
    """The autograd registrations (the reference's backward returns undefined gradients for every input,
    src/cam/comm_operator/pybind/fused_deep_moe.cpp:179-191, moe_combine_shmem.cpp:125-160)."""
    announce("autograd registrations")
    T, K, E, H = 16, 2, 8, 1024
    ids, w = synth.sigmoid_zipf_routing(T, E, K, seed=1)
    ids = ids.to(torch.int32).to(gpu)
    x = synth.normal_bf16(T, H, seed=2).to(gpu).requires_grad_(True)
    ops = torch.ops.umdk_cam_op_lib
    d = ops.moe_dispatch_shmem(x, ids, None, None, 1, 0, E, 1, 0, 0, 1, 0, 0, 0, 1, 0)
    assert d[0].requires_grad and d[0].grad_fn is not None and not d[2].requires_grad
    wg = w.to(gpu).requires_grad_(True)
    out = ops.moe_combine_shmem(d[0], ids, d[2], d[4], wg, None, None, None, None, None, None,
                                1, 0, E, 1, 0, 0, 1, 0, 0, 0, 0, 0, 0)
    assert out.requires_grad
    out.float().sum().backward()
    assert x.grad is None and wg.grad is None
    with torch.no_grad():
        ref = ops.moe_combine_shmem(d[0], ids, d[2], d[4], wg, None, None, None, None, None, None,
                                    1, 0, E, 1, 0, 0, 1, 0, 0, 0, 0, 0, 0)
    assert torch.equal(ref, out.detach()) and not ref.requires_grad
