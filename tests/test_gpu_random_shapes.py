"""Randomly drawn column layouts and edge lists, a fixed number per seed, through the operators:
edge softmax (forward and backward, twice, so that the first pass partitions on the fly and the
second goes through the plans kept with the offsets), the product at a random width, and both
conversions, against float64 models and numpy's stable sort.  The layouts mix the cases the
kernels treat differently: columns of 0-3 entries, a few thousand-entry columns among short
ones, half the columns empty, lengths around the lane and tile sizes, one column only."""
import numpy as np
import pytest
import torch

from util import dev, to_gpu

pytestmark = pytest.mark.gpu


def draw_lengths(rng):
    kind = int(rng.integers(0, 7))
    V = int(rng.integers(1, 5000))
    if kind == 0:
        return rng.integers(0, 4, V)
    if kind == 1:
        return rng.integers(0, 40, V)
    if kind == 2:
        return np.where(rng.random(V) < 0.01, rng.integers(1000, 9000, V), rng.integers(0, 3, V))
    if kind == 3:
        return np.where(rng.random(V) < 0.5, 0, rng.integers(1, 20, V))
    if kind == 4:
        return rng.choice([0, 1, 7, 8, 9, 1023, 1024, 1025, 2047, 2048, 2049], min(V, 40))
    if kind == 5:
        return np.array([int(rng.integers(1, 60000))])
    return rng.integers(0, 2, V) * rng.integers(1, 300, V)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_layouts_against_float64_models(seed):
    from jittorgeometric_amd import CSC
    from jittorgeometric_amd.ops import EdgeSoftmax, cootocsc, cootocsr
    from jittorgeometric_amd.ops._common import spmm
    rng = np.random.default_rng(seed)
    for case in range(16):
        lens = np.asarray(draw_lengths(rng), np.int64)
        V, E = len(lens), int(lens.sum())
        what = "seed %d case %d (V=%d, E=%d)" % (seed, case, V, E)
        if E > 0:
            off = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
            seg = np.repeat(np.arange(V), lens)
            row = rng.integers(0, V, E).astype(np.int32)
            w = rng.standard_normal(E).astype(np.float32)
            csc = CSC(to_gpu(row), to_gpu(off), to_gpu(w))
            H = int(rng.choice([1, 2, 4, 8, 3, 16]))
            x = (rng.standard_normal((E, H)) * rng.choice([0.5, 4, 30])).astype(np.float32)
            g = rng.standard_normal((E, H)).astype(np.float32)
            x64 = x.astype(np.float64)
            mx = np.full((V, H), -np.inf)
            np.maximum.at(mx, seg, x64)
            p = np.exp(x64 - mx[seg])
            den = np.zeros((V, H))
            np.add.at(den, seg, p)
            y64 = p / den[seg]
            dot, absdot = np.zeros((V, H)), np.zeros((V, H))
            np.add.at(dot, seg, y64 * g)
            np.add.at(absdot, seg, np.abs(y64 * g))
            xt = to_gpu(x).requires_grad_(True)
            for use in range(2):
                xt.grad = None
                y = EdgeSoftmax(xt, csc)
                y.backward(to_gpu(g))
                assert np.abs(y.detach().cpu().numpy() - y64).max() < 2e-6, what + " softmax, use %d, H=%d" % (use, H)
                tol = 1e-6 + 1e-5 * (np.abs(y64 * g) + y64 * absdot[seg])
                assert (np.abs(xt.grad.cpu().numpy() - y64 * (g - dot[seg])) <= tol).all(), \
                    what + " softmax backward, use %d, H=%d" % (use, H)
                F = int(rng.choice([1, 2, 4, 8, 5, 32, 64, 128, 100]))
                feat = rng.standard_normal((V, F)).astype(np.float32)
                out = spmm(csc.column_offset, csc.row_indices, csc.edge_weight, to_gpu(feat), V).cpu().numpy()
                terms = w.astype(np.float64)[:, None] * feat.astype(np.float64)[row]
                want, mag = np.zeros((V, F)), np.zeros((V, F))
                np.add.at(want, seg, terms)
                np.add.at(mag, seg, np.abs(terms))
                assert (np.abs(out - want) <= 1e-6 + 1e-5 * mag).all(), what + " product, use %d, F=%d" % (use, F)
        n = int(rng.integers(1, 200000))
        ei = np.stack([rng.integers(0, V, n), rng.integers(0, V, n)]).astype(np.int32)
        if rng.random() < 0.3:
            ei[int(rng.integers(0, 2))].sort()
        wc = rng.standard_normal(n).astype(np.float32)
        for fn, key in ((cootocsr, 0), (cootocsc, 1)):
            r = fn(to_gpu(ei), to_gpu(wc), V)
            offs, idxs = (r.row_offset, r.column_indices) if key == 0 else (r.column_offset, r.row_indices)
            order = np.argsort(ei[key], kind="stable")
            assert np.array_equal(offs.cpu().numpy(), np.concatenate([[0], np.cumsum(np.bincount(ei[key], minlength=V))]))
            assert np.array_equal(idxs.cpu().numpy(), ei[1 - key][order]), what + " conversion by row %d" % key
            assert np.array_equal(r.edge_weight.cpu().numpy(), wc[order])
    assert torch.cuda.is_available() and dev().type == "cuda"
