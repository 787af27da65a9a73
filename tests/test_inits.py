"""Parameter initialisers against the reference's formulas (nn/inits.py:19-22,59-61):
glorot draws from U(-s, s) with s = sqrt(6 / (size(-2) + size(-1))); zeros fills with 0;
both ignore None."""
import math

import torch

from jittorgeometric_amd.nn.inits import glorot, zeros


def test_glorot_bound_uses_the_last_two_dimensions():
    torch.manual_seed(0)
    for shape in ((1433, 256), (256, 7), (3, 40, 50), (32, 1)):
        t = torch.full(shape, 9.0)
        glorot(t)
        s = math.sqrt(6.0 / (shape[-2] + shape[-1]))
        assert t.abs().max().item() <= s
        if t.numel() >= 1000:                       # the draw fills the interval and is centred
            assert t.abs().max().item() > 0.98 * s
            assert abs(t.mean().item()) < 0.05 * s
            assert abs(t.std().item() - s / math.sqrt(3.0)) < 0.05 * s      # std of U(-s, s)
    assert glorot(None) is None


def test_zeros_and_layer_defaults():
    t = torch.ones(5)
    zeros(t)
    assert not t.any()
    assert zeros(None) is None
    from jittorgeometric_amd.nn import GATConv, GCNConv, SAGEConv
    torch.manual_seed(1)
    layer = GCNConv(1433, 256)
    assert layer.weight.abs().max().item() <= math.sqrt(6.0 / (1433 + 256)) and not layer.bias.any()
    gat = GATConv(64, 16, 0)
    assert gat.edge_weight.shape == (32, 1) and gat.edge_weight.abs().max().item() <= math.sqrt(6.0 / 33)
    sage = SAGEConv(100, 256)
    assert sage.root_weight.abs().max().item() <= math.sqrt(6.0 / 356) and not sage.bias.any()
