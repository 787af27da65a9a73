"""jgamd_spmm_csx_noalloc (scratch in a fixed device array inside the library)
against jgamd_spmm_csx (scratch from the caller), through the C ABI: the two
share their kernels and their chunking, so the outputs must agree bit for bit.
Two calls in a row, the second on a smaller input, so that whatever the first
call left in the shared array is there when the second one runs."""
import ctypes

import numpy as np
import pytest
import torch

from util import dev, rand_graph, to_gpu

pytestmark = pytest.mark.gpu


def _csc(ei, w, V):
    from jittorgeometric_amd.ops import cootocsc
    return cootocsc(to_gpu(ei), to_gpu(w), V)


def _both(csc, x, V, E, F):
    from jittorgeometric_amd import _lib
    lib = _lib.load()
    st = _lib.stream_ptr(x.device)
    off, idx, w = csc.column_offset, csc.row_indices, csc.edge_weight
    n = _lib.query(lib.jgamd_spmm_csx_workspace, V, E, F)
    ws = _lib.workspace(n, x.device)
    want = torch.full((V, F), float("nan"), device=x.device)
    got = torch.full((V, F), float("nan"), device=x.device)
    _lib.check(lib.jgamd_spmm_csx(off.data_ptr(), idx.data_ptr(), w.data_ptr(), x.data_ptr(), want.data_ptr(),
                                  V, V, E, F, ws.data_ptr(), ws.numel(), st))
    _lib.check(lib.jgamd_spmm_csx_noalloc(off.data_ptr(), idx.data_ptr(), w.data_ptr(), x.data_ptr(),
                                          got.data_ptr(), V, V, E, F, st))
    torch.cuda.synchronize()
    return got, want


@pytest.mark.parametrize("F", [128, 41, 8])
def test_two_calls_in_a_row_match_the_workspace_entry_point(F):
    import oracle
    rng = np.random.default_rng(7 + F)
    shapes = [(60_000, 1_500_000, 40), (900, 20_000, 3)]      # large with hub rows cut into pieces, then small
    for V, E, hubs in shapes:
        ei, w = rand_graph(rng, V, E, hubs=hubs)
        x = rng.standard_normal((V, F)).astype(np.float32)
        csc = _csc(ei, w, V)
        got, want = _both(csc, to_gpu(x), V, E, F)
        assert not torch.isnan(got).any()
        assert torch.equal(got, want), "V=%d E=%d F=%d" % (V, E, F)
        if V < 1000:      # and the small one against the CPU oracle
            o = oracle.cootocsc(ei, w, V)
            ref = oracle.aggregate_with_weight(x, o)
            scale = oracle.aggregate(np.abs(x), o[0], o[1], np.abs(o[2]))
            assert np.all(np.abs(got.cpu().numpy() - ref) <= 1e-6 + 1e-5 * scale)


def test_shape_beyond_the_fixed_array_is_rejected_without_a_launch():
    from jittorgeometric_amd import _lib
    lib = _lib.load()
    n = ctypes.c_size_t(0)
    V, E, F = 1_000_000, 17_000_000, 512
    assert lib.jgamd_spmm_csx_workspace(V, E, F, ctypes.byref(n)) == 0 and n.value > 64 << 20
    bad = ctypes.c_void_p(256)     # never dereferenced
    rc = lib.jgamd_spmm_csx_noalloc(bad, bad, bad, bad, bad, V, V, E, F, None)
    assert rc == -2
    assert b"67108864" in lib.jgamd_last_error()
