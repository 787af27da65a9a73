"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

RTOL, ATOL = 1e-5, 1e-6     # fp32 tolerance of the sparse path (relative / absolute)


def dev():
    return torch.device("cuda:0")


def to_gpu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev())


def rand_graph(rng, V, E, hubs=0, hub_share=0.3):
    """Random directed multigraph; `hubs` destinations/sources get hub_share of the edges."""
    src = rng.integers(0, V, E).astype(np.int32)
    dst = rng.integers(0, V, E).astype(np.int32)
    if hubs and E:
        pick = rng.random(E) < hub_share
        dst[pick] = rng.integers(0, hubs, pick.sum()).astype(np.int32)
        pick = rng.random(E) < hub_share
        src[pick] = (V - 1 - rng.integers(0, hubs, pick.sum())).astype(np.int32)
    w = rng.standard_normal(E).astype(np.float32)
    return np.stack([src, dst]), w


def assert_close(got, want, scale=None, rtol=RTOL, atol=ATOL, what=""):
    """|got - want| <= atol + rtol * scale, where scale defaults to |want| and may be
    the sum of absolute terms of a reduction (summation-order differences grow
    with it, not with the possibly cancelled result)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.abs(want) if scale is None else np.asarray(scale, dtype=np.float64)
    err = np.abs(got - want)
    bad = err > atol + rtol * scale
    if bad.any():
        i = np.unravel_index(np.argmax(err - (atol + rtol * scale)), err.shape)
        raise AssertionError("%s: %d/%d out of tolerance; worst at %s: got %r want %r scale %r"
                             % (what, bad.sum(), bad.size, i, got[i], want[i], scale[i]))
