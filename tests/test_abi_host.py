"""Host-side checks that need no GPU: the C-ABI library loads, exports every
symbol include/jgamd.h declares, sizes its workspaces, and rejects bad
arguments with an error code instead of touching the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from jittorgeometric_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from jittorgeometric_amd import build
        build.build()
    return _lib.load()


def test_every_declared_symbol_is_exported_and_bound(lib):
    from jittorgeometric_amd import _lib
    header = open(os.path.join(ROOT, "include", "jgamd.h")).read()
    declared = set(re.findall(r"\b(jgamd_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 15
    for name in declared:
        assert hasattr(lib, name), name
    assert declared - {"jgamd_version", "jgamd_last_error"} == set(_lib.SIGNATURES)


def test_version_and_error_text(lib):
    assert lib.jgamd_version() >= 100
    rc = lib.jgamd_coo_to_csx(None, None, 5, 4, 0, None, None, None, None, None, 0, None)
    assert rc == -1 and b"out_off" in lib.jgamd_last_error()


def test_workspace_queries_are_host_only(lib):
    n = ctypes.c_size_t(0)
    assert lib.jgamd_coo_to_csx_workspace(17_000_000, 1_000_000, 0, ctypes.byref(n)) == 0
    plain = n.value
    assert 17_000_000 * 12 <= plain < 17_000_000 * 16
    assert lib.jgamd_coo_to_csx_workspace(17_000_000, 1_000_000, 1, ctypes.byref(n)) == 0
    assert n.value >= plain + 17_000_000 * 4 - 4096
    assert lib.jgamd_spmm_csx_workspace(1_000_000, 17_000_000, 128, ctypes.byref(n)) == 0
    assert 0 < n.value < 100 << 20
    assert lib.jgamd_spmm_csx_workspace(0, 0, 128, ctypes.byref(n)) == 0 and n.value == 0
    assert lib.jgamd_gat_fwd_workspace(169_343, 1_335_586, 8, 16, ctypes.byref(n)) == 0 and n.value > 0
    assert lib.jgamd_gat_bwd_workspace(169_343, 1_335_586, 8, 16, ctypes.byref(n)) == 0 and n.value > 0
    assert lib.jgamd_csx_transpose_workspace(1000, 10, 10, ctypes.byref(n)) == 0 and n.value > 0


def test_argument_errors_are_reported_not_launched(lib):
    n = ctypes.c_size_t(0)
    bad = ctypes.c_void_p(256)          # never dereferenced: every call below fails validation first
    assert lib.jgamd_coo_to_csx_workspace(-1, 4, 0, ctypes.byref(n)) == -2
    assert lib.jgamd_coo_to_csx_workspace(1 << 31, 4, 0, ctypes.byref(n)) == -2
    assert lib.jgamd_coo_to_csx_workspace(10, (1 << 22) + 1, 0, ctypes.byref(n)) == 0      # LSD path
    assert lib.jgamd_coo_to_csx_workspace(10, 2**31 - 1, 0, ctypes.byref(n)) == -2
    assert lib.jgamd_coo_to_csx_workspace(10, 4, 0, None) == -1
    assert lib.jgamd_coo_to_csx(bad, bad, 5, 4, 2, bad, bad, bad, None, bad, 1 << 30, None) == -2      # key_row
    assert lib.jgamd_coo_to_csx(bad, bad, 5, 4, 0, bad, bad, bad, None, None, 0, None) == -3          # no workspace
    assert lib.jgamd_coo_to_csx(bad, bad, 5, 4, 0, bad, bad, bad, None, bad, 16, None) == -3          # too small
    assert lib.jgamd_coo_to_csx(bad, bad, 5, 4, 0, bad, bad, bad, None, ctypes.c_void_p(260), 1 << 30, None) == -5
    assert lib.jgamd_coo_to_csx(None, bad, 5, 4, 0, bad, bad, bad, None, bad, 1 << 30, None) == -1
    assert lib.jgamd_spmm_csx(None, bad, bad, bad, bad, 4, 4, 5, 8, bad, 1 << 30, None) == -1
    assert lib.jgamd_spmm_csx(bad, bad, bad, bad, bad, -4, 4, 5, 8, bad, 1 << 30, None) == -2
    assert lib.jgamd_spmm_csx(bad, bad, bad, bad, bad, 4, 0, 5, 8, bad, 1 << 30, None) == -2          # E>0, no x rows
    assert lib.jgamd_spmm_csx(bad, bad, bad, ctypes.c_void_p(258), bad, 4, 4, 5, 8, bad, 1 << 30, None) == -5
    assert lib.jgamd_spmm_csx(bad, bad, bad, bad, bad, 4, 4, 5, 8, bad, 8, None) == -3
    assert lib.jgamd_spmm_csx(bad, bad, bad, bad, bad, 0, 4, 0, 8, None, 0, None) == 0                # nothing to do
    assert lib.jgamd_edge_softmax_fwd(bad, bad, bad, 4, 5, 0, bad, 1 << 20, None) == -2
    assert lib.jgamd_edge_softmax_fwd(None, bad, bad, 4, 5, 1, bad, 1 << 20, None) == -1
    assert lib.jgamd_edge_softmax_fwd(bad, bad, bad, 4, 5, 1, None, 0, None) == -3
    assert lib.jgamd_edge_softmax_bwd(bad, bad, None, bad, 4, 5, 1, bad, 1 << 20, None) == -1
    assert lib.jgamd_edge_softmax_workspace(4, 5, ctypes.byref(n)) == 0 and n.value >= 260
    assert lib.jgamd_scatter_to_edge(bad, bad, bad, bad, 4, 5, 8, 3, None) == -2
    assert lib.jgamd_gat_fwd_workspace(10, 10, 4, 1024, ctypes.byref(n)) == -4
    assert lib.jgamd_gat_bwd_workspace(10, 10, 3, 7, ctypes.byref(n)) == -4
    assert lib.jgamd_gat_bwd_workspace(10, 10, 1, 7, ctypes.byref(n)) == 0
    # rows without classes: refused on the host, nothing is launched on a [V,0] array's NULL address
    assert lib.jgamd_cross_entropy_fwd(None, bad, 0, 0, 5, 0, bad, bad, bad, bad, 1 << 20, None) == -2
    assert b"C=0" in lib.jgamd_last_error()


def test_operators_refuse_cpu_tensors():
    import torch
    from jittorgeometric_amd import CSC, _lib
    from jittorgeometric_amd.ops import EdgeSoftmax, aggregateWithWeight, cootocsc
    with pytest.raises(_lib.JgamdError):
        cootocsc(torch.zeros((2, 3), dtype=torch.int32), torch.ones(3), 4)
    csc = CSC(torch.zeros(3, dtype=torch.int32), torch.tensor([0, 1, 2, 3], dtype=torch.int32), torch.ones(3))
    with pytest.raises(_lib.JgamdError):
        aggregateWithWeight(torch.ones(3, 4), csc, None)
    with pytest.raises(_lib.JgamdError):
        EdgeSoftmax(torch.ones(3), csc)


def test_synthetic_generators_are_seeded_and_shaped():
    import numpy as np
    from jittorgeometric_amd import synthetic
    a, V = synthetic.make("cora_like")
    b, _ = synthetic.make("cora_like")
    assert V == 2708 and a.shape == (2, 10556) and np.array_equal(a, b) and a.dtype == np.int32
    assert (a[0] != a[1]).all()
    pairs = set(map(tuple, a.T))
    assert len(pairs) == 10556 and all((v, u) in pairs for u, v in list(pairs)[:200])
    g = synthetic.chung_lu(20000, 300000, 2.1, max_degree=500, seed=1)
    deg = np.bincount(g[1], minlength=20000)
    assert g.dtype == np.int32 and 0.9 * 300000 < g.shape[1] <= 300000 and deg.max() < 700 and np.median(deg) < 15
    d = synthetic.lognormal_degree(2000, 50.0, 1.0, seed=2)
    assert 0.8 * 100000 < d.shape[1] < 1.2 * 100000
