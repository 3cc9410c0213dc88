"""Seeded synthetic inputs for the CAM MoE path (CPU tensors; callers move them to the device).

Two families:
  * the reference's own unit-test recipe (test/cam/ut/fused_deep_moe/test_fused_deep_moe.py:269-337):
    x = rand*10-5 in bf16, round-robin expert ids, int8 weights randint(-16,16), scales
    rand*0.003+0.0015 rounded through bf16, un-normalised rand gate weights;
  * the benchmark shapes: N(0,1) activations, softmax / sigmoid+Zipf-biased top-k routing (gating is
    not part of CAM -- it receives ids and weights -- so these are plain torch on the CPU), Zipf-skewed
    rows per expert with some experts empty.
Every generator takes a seed; the benchmark uses 42 + configuration number.
"""
import math

import torch


def _gen(seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    return g


def ut_recipe(batch_size, hidden, intermediate, num_experts, top_k=8, rank=0, seed=42):
    """The reference unit test's data, for one rank that owns all `num_experts` experts."""
    g = _gen(seed)
    x = (torch.rand([batch_size, hidden], generator=g) * 10 - 5).bfloat16()
    ids = torch.arange(rank * batch_size * top_k, (rank + 1) * batch_size * top_k).to(torch.int32)
    ids = (ids.view(batch_size, top_k) % num_experts).contiguous()
    w1 = torch.randint(-16, 16, [num_experts, hidden, 2 * intermediate], generator=g).to(torch.int8)
    w2 = torch.randint(-16, 16, [num_experts, intermediate, hidden], generator=g).to(torch.int8)
    w1s = (torch.rand([num_experts, 2 * intermediate], generator=g) * 0.003 + 0.0015).bfloat16().float()
    w2s = (torch.rand([num_experts, hidden], generator=g) * 0.003 + 0.0015).bfloat16().float()
    gates = torch.rand(batch_size, top_k, generator=g)
    return dict(x=x, ids=ids, gates=gates, w1=w1, w1_scale=w1s, w2=w2, w2_scale=w2s)


def softmax_topk_routing(tokens, num_experts, top_k, seed):
    """N(0,1) logits -> softmax -> top-k (ties: lowest index), gate weights renormalised to sum 1."""
    g = _gen(seed)
    logits = torch.randn(tokens, num_experts, generator=g)
    probs = torch.softmax(logits, dim=-1)
    w, ids = torch.topk(probs, top_k, dim=-1)
    w = w / w.sum(dim=-1, keepdim=True)
    return ids.to(torch.int64).contiguous(), w.float().contiguous()


def sigmoid_zipf_routing(tokens, num_experts, top_k, seed, s=1.1, bias_scale=1.0):
    """sigmoid(N(0,1) logits) + Zipf(s) expert bias on a random expert order -> top-k ids;
    gate weights are the selected sigmoid scores renormalised (DeepSeek-V3 style)."""
    g = _gen(seed)
    logits = torch.randn(tokens, num_experts, generator=g)
    scores = torch.sigmoid(logits)
    order = torch.randperm(num_experts, generator=g)
    zipf = torch.arange(1, num_experts + 1, dtype=torch.float32).pow(-s)
    bias = torch.empty(num_experts)
    bias[order] = zipf * bias_scale
    _, ids = torch.topk(scores + bias, top_k, dim=-1)
    w = torch.gather(scores, 1, ids)
    w = w / w.sum(dim=-1, keepdim=True)
    return ids.to(torch.int64).contiguous(), w.float().contiguous()


def zipf_group_sizes(num_groups, total_rows, seed, s=1.1, num_empty=3):
    """Rows per expert ~ Zipf(s) over a random expert order, summing to total_rows, `num_empty` experts at 0."""
    g = _gen(seed)
    live = num_groups - num_empty
    zipf = torch.arange(1, live + 1, dtype=torch.float64).pow(-s)
    share = zipf / zipf.sum() * total_rows
    rows = torch.floor(share).to(torch.int64)
    rem = int(total_rows - rows.sum().item())
    frac = share - rows
    rows[torch.argsort(frac, descending=True)[:rem]] += 1
    order = torch.randperm(num_groups, generator=g)
    out = torch.zeros(num_groups, dtype=torch.int64)
    out[order[:live]] = rows
    assert int(out.sum()) == total_rows
    return out


def normal_bf16(rows, cols, seed):
    return torch.randn(rows, cols, generator=_gen(seed)).bfloat16()


def uniform_int8(shape, seed, lo=-127, hi=127):
    return torch.randint(lo, hi + 1, list(shape), generator=_gen(seed), dtype=torch.int16).to(torch.int8)


def channel_scales(shape, seed, lo=0.0015, hi=0.0045):
    return (torch.rand(list(shape), generator=_gen(seed)) * (hi - lo) + lo).float()


def absmax_int8_weights(num_experts, kd, n, seed):
    """N(0,1) fp32 weights quantised per output channel: scale = absmax/127, w = rint(w/scale)."""
    g = _gen(seed)
    w = torch.randn(num_experts, kd, n, generator=g)
    scale = w.abs().amax(dim=1) / 127.0
    q = torch.round(w / scale[:, None, :]).clamp_(-127, 127).to(torch.int8)
    return q.contiguous(), scale.float().contiguous()


# Algorithmic byte / op counts (the roofline numerators).
def dispatch_bytes(tokens, hidden, top_k, num_experts):
    """Read x once + ids; write int8 rows, fp32 scales, positions, counts and offsets."""
    rows = tokens * top_k
    return tokens * hidden * 2 + rows * 4 + rows * hidden + rows * 4 + rows * 4 + 2 * num_experts * 4


def combine_bytes(tokens, hidden, top_k):
    rows = tokens * top_k
    return rows * hidden * 2 + rows * 4 + rows * 4 + tokens * hidden * 2


def gemm_ops(rows, hidden, intermediate):
    return 2 * rows * hidden * 2 * intermediate + 2 * rows * intermediate * hidden


def bf16_bits(t):
    """torch bf16 tensor -> numpy uint16 bit patterns."""
    return t.contiguous().view(torch.int16).numpy().view("uint16")


def bits_to_bf16(a):
    import numpy as np
    return torch.from_numpy(np.ascontiguousarray(a).view("int16")).view(torch.bfloat16)


def _isclose_count(a, b, atol, rtol):
    d = (a.double() - b.double()).abs()
    return int((d > atol + rtol * b.double().abs()).sum())


def max_rel_err(a, b):
    """max |a-b| / max(|b|, tiny) over elements where b != 0, plus max |a| where b == 0."""
    a = a.double()
    b = b.double()
    nz = b != 0
    rel = ((a[nz] - b[nz]).abs() / b[nz].abs()).max().item() if nz.any() else 0.0
    zero = a[~nz].abs().max().item() if (~nz).any() else 0.0
    return max(rel, zero) if not math.isnan(rel) else float("nan")
