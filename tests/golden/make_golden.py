"""Writes tests/golden/cam_c1_golden.npz: inputs' fingerprints and expected outputs of the CPU-golden MoE
layer (128 tokens, hidden 1024, 8 experts, softmax top-2, intermediate 512) as computed by the CPU oracle.

The reference ships no golden vectors for this path and cannot run here, so these vectors freeze the
oracle's results (after the oracle itself was pinned by tests/test_oracle.py): a later change to the oracle,
to the seeded generators or to the HIP kernels that alters any of them is caught without a GPU-vs-oracle
run.  Usage: python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

import cam_oracle  # noqa: E402
from umdk_original_amd import synth  # noqa: E402

T, H, E, K, I = 128, 1024, 8, 2, 512


def sha(a):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), dtype=np.uint8)


def inputs():
    ids, gates = synth.softmax_topk_routing(T, E, K, seed=43)
    w1, w1s = synth.absmax_int8_weights(E, H, 2 * I, seed=431)
    w2, w2s = synth.absmax_int8_weights(E, I, H, seed=432)
    x = synth.normal_bf16(T, H, seed=433)
    return dict(x=x, ids=ids, gates=gates, w1=w1, w1_scale=w1s, w2=w2, w2_scale=w2s)


def compute():
    d = inputs()
    xb = synth.bf16_bits(d["x"])
    idx = d["ids"].numpy()
    _, cnt, _ = cam_oracle.layout(idx, E, 1)
    off, _ = cam_oracle.offsets(cnt, T)
    pos = cam_oracle.send_token_idx(idx, E)
    out, etn, dbg = cam_oracle.fused_layer(xb, idx, d["gates"].numpy(), d["w1"].numpy(), d["w1_scale"].numpy(),
                                           d["w2"].numpy(), d["w2_scale"].numpy(), debug=True)
    q1, s1 = cam_oracle.quant_rows(xb, 1)
    return dict(
        ids=idx, gates=d["gates"].numpy(), x_sha=sha(xb), w1_sha=sha(d["w1"].numpy()), w2_sha=sha(d["w2"].numpy()),
        w1_scale_sha=sha(d["w1_scale"].numpy()), w2_scale_sha=sha(d["w2_scale"].numpy()),
        cnt=cnt, off=off, pos=pos, expert_token_nums=etn,
        x1_head=dbg["x1"][:4], x1_scale=dbg["x1_scale"], x1_sha=sha(dbg["x1"]),
        q1_eps_head=q1[:4], q1_eps_scale=s1,
        x2_head=dbg["x2"][:4], x2_scale=dbg["x2_scale"], x2_sha=sha(dbg["x2"]),
        y_head=dbg["y"][:4], y_sha=sha(dbg["y"]),
        out_head=out[:8], out_sha=sha(out),
    )


if __name__ == "__main__":
    g = compute()
    path = os.path.join(HERE, "cam_c1_golden.npz")
    np.savez_compressed(path, **g)
    print("wrote", path, os.path.getsize(path), "bytes")
