"""The column-blocked product (csrc/spmm_blocked.hip) through the C ABI: the regrouping is a
stable partition of every row by column block (checked bit for bit against numpy), the product
over the regrouped arrays equals the oracle's row sums (aggregate_op.cc:107-114) within 1e-5
of the sum of absolute terms, and equals the unblocked kernels' result within the same bound.
Small shapes with explicit block counts; the benchmark configuration that takes this path by
itself (V = 233k, 492 entries per row) is covered by tests/test_gpu_configs.py."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu


def lib():
    from jittorgeometric_amd import _lib
    return _lib, _lib.load()


def block_columns(off, idx, w, R, nb, cols):
    L, l = lib()
    E = idx.shape[0]
    b_off = torch.empty(nb * R + 1, dtype=torch.int32, device=dev())
    b_idx = torch.full((E,), -7, dtype=torch.int32, device=dev())
    b_w = torch.full((E,), -7.0, dtype=torch.float32, device=dev()) if w is not None else None
    nbytes = L.query(l.jgamd_csx_block_columns_workspace, R, nb)
    ws = L.workspace(nbytes, dev())
    L.check(l.jgamd_csx_block_columns(L.ptr(off), L.ptr(idx), L.ptr(w), R, E, cols, nb, L.ptr(b_off), L.ptr(b_idx),
                                      L.ptr(b_w), L.ptr(ws), nbytes, L.stream_ptr(dev())))
    return b_off, b_idx, b_w


def blocked_product(b_off, b_idx, b_w, x, R, E, nb, beta=1.0, alpha=0.0, h=None):
    L, l = lib()
    C, F = x.shape
    out = torch.empty((R, F), dtype=torch.float32, device=dev())
    nbytes = L.query(l.jgamd_spmm_csx_blocked_workspace, R, C, E, F, nb)
    ws = L.workspace(nbytes, dev())
    h_rows = R if h is None or h.dim() == 2 else 1
    L.check(l.jgamd_spmm_csx_blocked(L.ptr(b_off), L.ptr(b_idx), L.ptr(b_w), L.ptr(x), L.ptr(out), beta, alpha,
                                     L.ptr(h), h_rows, R, C, E, F, nb, L.ptr(ws), nbytes, L.stream_ptr(dev())))
    return out


def numpy_blocks(off, idx, w, R, nb, cols):
    """Stable partition of every row by min(idx // cols, nb - 1)."""
    E = int(off[R])
    row = np.repeat(np.arange(R), np.diff(off[:R + 1]))
    blk = np.minimum(idx[:E].astype(np.int64) // cols, nb - 1)
    key = blk * R + row
    order = np.argsort(key, kind="stable")
    b_off = np.zeros(nb * R + 1, np.int64)
    np.add.at(b_off, key + 1, 1)
    return np.cumsum(b_off).astype(np.int32), idx[:E][order], (w[:E][order] if w is not None else None)


@pytest.mark.parametrize("V,E,nb,cols,hubs,seed", [(300, 9000, 5, 64, 2, 0), (1000, 200000, 16, 64, 3, 1),
                                                   (50, 40, 3, 20, 0, 2), (2000, 60000, 64, 32, 1, 3),
                                                   (700, 30000, 1, 1000, 0, 4), (64, 5000, 7, 8, 1, 5)])
def test_regrouping_is_a_stable_partition_by_block(V, E, nb, cols, hubs, seed):
    rng = np.random.default_rng(seed)
    ei, w = rand_graph(rng, V, E, hubs)
    idx, off, wt = oracle.cootocsc(ei, w, V)
    b_off, b_idx, b_w = block_columns(to_gpu(off), to_gpu(idx), to_gpu(wt), V, nb, cols)
    want_off, want_idx, want_w = numpy_blocks(off, idx, wt, V, nb, cols)
    assert np.array_equal(b_off.cpu().numpy(), want_off)
    assert np.array_equal(b_idx.cpu().numpy(), want_idx)
    assert np.array_equal(b_w.cpu().numpy().view(np.int32), want_w.view(np.int32))


def test_regrouping_without_weights_and_with_entries_past_the_last_offset():
    rng = np.random.default_rng(7)
    V = 400
    ei, w = rand_graph(rng, V, 20000, 1)
    idx, off, wt = oracle.cootocsc(ei, w, V)
    off = off.copy()
    off[-1] -= 37                                          # the last 37 entries belong to no row
    b_off, b_idx, b_w = block_columns(to_gpu(off), to_gpu(idx), None, V, 6, 70)
    want_off, want_idx, _ = numpy_blocks(off, idx, None, V, 6, 70)
    assert b_w is None
    assert np.array_equal(b_off.cpu().numpy(), want_off)
    covered = int(off[-1])
    assert np.array_equal(b_idx.cpu().numpy()[:covered], want_idx)
    assert (b_idx.cpu().numpy()[covered:] == -7).all()      # slots past the covered entries are left alone


@pytest.mark.parametrize("F", [1, 3, 4, 8, 9, 41, 64, 100, 130, 256])
@pytest.mark.parametrize("V,E,nb,cols", [(600, 90000, 8, 80), (3000, 40000, 5, 700)])
def test_blocked_product_matches_oracle_and_unblocked(V, E, nb, cols, F):
    from jittorgeometric_amd.ops._common import spmm
    rng = np.random.default_rng(F + V)
    ei, w = rand_graph(rng, V, E, 2)
    idx, off, wt = oracle.cootocsc(ei, w, V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    off_g, idx_g, w_g, x_g = to_gpu(off), to_gpu(idx), to_gpu(wt), to_gpu(x)
    b_off, b_idx, b_w = block_columns(off_g, idx_g, w_g, V, nb, cols)
    got = blocked_product(b_off, b_idx, b_w, x_g, V, E, nb).cpu().numpy()
    want = oracle.aggregate(x, idx, off, wt)
    terms = oracle.aggregate(np.abs(x), idx, off, np.abs(wt))
    assert_close(got, want, terms, what="blocked product F=%d" % F)
    plain = spmm(off_g, idx_g, w_g, x_g, V).cpu().numpy()
    assert_close(got, plain, terms, what="blocked vs unblocked F=%d" % F)
    again = blocked_product(b_off, b_idx, b_w, x_g, V, E, nb).cpu().numpy()
    assert np.array_equal(got.view(np.int32), again.view(np.int32))           # run-to-run identical


@pytest.mark.parametrize("F,bias_row", [(48, True), (48, False), (41, False), (128, True)])
def test_blocked_product_with_scaled_sum_and_added_rows(F, bias_row):
    rng = np.random.default_rng(11 + F)
    V, E, nb, cols = 900, 70000, 6, 160
    ei, w = rand_graph(rng, V, E, 1)
    idx, off, wt = oracle.cootocsc(ei, w, V)
    x = rng.standard_normal((V, F)).astype(np.float32)
    h = rng.standard_normal((F,) if bias_row else (V, F)).astype(np.float32)
    b_off, b_idx, b_w = block_columns(to_gpu(off), to_gpu(idx), to_gpu(wt), V, nb, cols)
    got = blocked_product(b_off, b_idx, b_w, to_gpu(x), V, E, nb, beta=0.9, alpha=0.1, h=to_gpu(h)).cpu().numpy()
    ax = oracle.aggregate(x, idx, off, wt).astype(np.float64)
    terms = oracle.aggregate(np.abs(x), idx, off, np.abs(wt))
    assert_close(got, 0.9 * ax + 0.1 * h.astype(np.float64), 0.9 * terms + 0.1 * np.abs(h), what="beta A x + alpha h")


def test_plan_takes_long_rows_only():
    L, l = lib()

    def plan(R, C, E, F):
        nb, cols = ctypes.c_int32(-1), ctypes.c_int32(-1)
        L.check(l.jgamd_spmm_block_plan(R, C, E, F, ctypes.byref(nb), ctypes.byref(cols)))
        return nb.value, cols.value
    nb, cols = plan(232_965, 232_965, 114_848_857, 256)
    assert 3 <= nb <= 64 and cols * nb >= 232_965 and cols * 64 * 4 <= 8 << 20
    assert plan(1_000_000, 1_000_000, 16_997_439, 128)[0] == 0        # 17 entries per row
    assert plan(2_449_029, 2_449_029, 126_000_000, 100)[0] == 0       # too many blocks
    assert plan(232_965, 232_965, 114_848_857, 8)[0] == 0             # narrow rows take the tile kernels
    assert plan(1000, 1000, 500_000, 64)[0] == 0                      # x fits anyway
    assert plan(100_000, 100_000, 20_000_000, 16)[0] == 0             # 6.4 MB of narrow rows


def test_blocked_entry_points_reject_bad_sizes():
    from jittorgeometric_amd import JgamdError
    L, l = lib()
    with pytest.raises(JgamdError):
        L.query(l.jgamd_csx_block_columns_workspace, 10, 65)
    with pytest.raises(JgamdError):
        L.query(l.jgamd_spmm_csx_blocked_workspace, 1 << 26, 1 << 26, 10, 4, 64)    # nb * R above 2^31


def test_blocked_product_without_weights_and_with_columns_out_of_range():
    """w = NULL means weight 1 (ScatterToVertex-style sums); an index outside [0, C) contributes
    nothing, as in the unblocked kernels, whichever block it was filed under."""
    rng = np.random.default_rng(23)
    V, E, nb, cols, F = 800, 50000, 7, 120, 44
    ei, w = rand_graph(rng, V, E, 1)
    idx, off, wt = oracle.cootocsc(ei, w, V)
    bad = idx.copy()
    where = rng.choice(E, 300, replace=False)
    bad[where[:150]] = V + 5
    bad[where[150:]] = -3
    keep = np.ones(E, bool)
    keep[where] = False
    x = rng.standard_normal((V, F)).astype(np.float32)
    ones = np.ones(E, np.float32)
    # exact row sums: the hub row has 15,000 same-weight terms, where the oracle's sequential fp32
    # loop has itself drifted past 1e-5 of the sum of absolute terms
    want, terms = oracle.aggregate_f64(x, idx, off, np.where(keep, ones, 0).astype(np.float32))
    b_off, b_idx, b_w = block_columns(to_gpu(off), to_gpu(bad), None, V, nb, cols)
    assert b_w is None
    got = blocked_product(b_off, b_idx, None, to_gpu(x), V, E, nb).cpu().numpy()
    assert_close(got, want, terms, what="unweighted blocked product with dropped indices")
