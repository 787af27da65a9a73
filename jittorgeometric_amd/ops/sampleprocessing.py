"""Neighbour sampling of one layer.  Same call as jittor_geometric.ops.sampleprocessing
(ops/sampleprocessing.py:29-35) plus an optional seed.  The reference draws with rand()
or a clock-seeded curand state (ops/cpp/sampleprocessing_op.cc:66-69,122-124), so it has
no reproducible output; here a destination's sample is a function of (seed, its id):
csrc/sample.hip.  Without a seed, successive calls use torch's initial seed plus a call
counter, so a run is reproducible after torch.manual_seed."""
import torch

from .. import _lib
from ._common import as_i32

_calls = 0


def sampleprocessing(fanout_i, csc_layer_dst, csc_layer_column_offset, csc_global_column_offset,
                     csc_global_row_indices, seed=None):
    global _calls
    lib = _lib.load()
    dev = _lib.require_gpu(csc_layer_dst, csc_layer_column_offset, csc_global_column_offset, csc_global_row_indices)
    dst = as_i32(csc_layer_dst, "csc_layer_dst")
    loff = as_i32(csc_layer_column_offset, "csc_layer_column_offset")
    goff = as_i32(csc_global_column_offset, "csc_global_column_offset")
    gidx = as_i32(csc_global_row_indices, "csc_global_row_indices")
    if seed is None:
        seed = (torch.initial_seed() + 0x9E3779B97F4A7C15 * _calls) & (2 ** 64 - 1)
        _calls += 1
    n_out = int(loff[-1].item()) if loff.numel() else 0          # sized as the reference does (:31)
    out = torch.zeros(n_out, dtype=torch.int32, device=dev)
    _lib.check(lib.jgamd_sample_neighbors(_lib.ptr(dst), _lib.ptr(loff), _lib.ptr(goff), _lib.ptr(gidx),
                                          dst.shape[0], goff.shape[0] - 1, int(fanout_i), n_out,
                                          int(seed) & (2 ** 64 - 1), _lib.ptr(out), _lib.stream_ptr(dev)))
    return out
