"""Helpers shared by the GPU parity tests (which call the HIP path through the C ABI)."""
import numpy as np
import torch

from umdk_original_amd import synth


def announce(msg):
    # Names the case before any GPU work so a lost box still tells which test was running.
    print("[gpu-case] " + msg, flush=True)


def to_np(t):
    if t.dtype == torch.bfloat16:
        return synth.bf16_bits(t.cpu())
    return t.cpu().numpy()


def plan_oracle(oracle, idx_np, E, skip_out_of_range=False):
    T = idx_np.shape[0]
    _, cnt, _ = oracle.layout(idx_np, E, 1, skip_out_of_range=skip_out_of_range)
    off, trip = oracle.offsets(cnt, T)
    pos = oracle.send_token_idx(idx_np, E)
    return cnt, off, pos, trip


def assert_bits_equal(got, want, what):
    got = np.asarray(got)
    want = np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        raise AssertionError("%s: %d of %d elements differ; first at %s: got %s want %s" % (
            what, len(bad), got.size, bad[0].tolist(), got[tuple(bad[0])], want[tuple(bad[0])]))
