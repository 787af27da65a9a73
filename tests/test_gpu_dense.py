"""The matrix-core dense transform (csrc/dense_rows.hip, jgamd_dense_rows) against float64
products of the same operands: out = x1 @ w1 (+ x2 @ w2) (+ bias), which stands for
`x @ self.weight` (gcn_conv.py:95) and `out @ weight1 + x @ root_weight + bias`
(sage_conv.py:186-190).  Tolerance 1e-5 of the sum of absolute terms plus 1e-6."""
import numpy as np
import pytest
import torch

from util import assert_close, dev

pytestmark = pytest.mark.gpu


def reference(x1, w1, x2, w2, bias):
    ref = x1.double() @ w1.double()
    scale = x1.double().abs() @ w1.double().abs()
    if x2 is not None:
        ref += x2.double() @ w2.double()
        scale += x2.double().abs() @ w2.double().abs()
    if bias is not None:
        ref += bias.double()
        scale += bias.double().abs()
    return ref.cpu().numpy(), scale.cpu().numpy()


@pytest.mark.parametrize("V,K1,K2,N,bias", [
    (4096, 128, 0, 128, False), (4097, 128, 0, 128, True), (5000, 100, 0, 256, True), (9001, 256, 0, 256, False),
    (7000, 128, 128, 128, True), (4100, 4, 0, 4, False), (6000, 36, 60, 44, True), (5003, 64, 0, 32, False),
    (4111, 132, 124, 136, True), (20000, 16, 0, 600, True), (4096, 252, 4, 252, False)])
def test_dense_rows_matches_float64(V, K1, K2, N, bias):
    from jittorgeometric_amd import _lib
    from jittorgeometric_amd.nn.dense import rows_times
    assert _lib.load().jgamd_dense_rows_supported(K1, K2, N) == 1
    gen = torch.Generator(device=dev()).manual_seed(V + K1 + N)
    x1 = torch.randn((V, K1), device=dev(), generator=gen)
    w1 = torch.randn((K1, N), device=dev(), generator=gen)
    x2 = torch.randn((V, K2), device=dev(), generator=gen) if K2 else None
    w2 = torch.randn((K2, N), device=dev(), generator=gen) if K2 else None
    b = torch.randn((N,), device=dev(), generator=gen) if bias else None
    got = rows_times(x1, w1, x2, w2, b)
    ref, scale = reference(x1, w1, x2, w2, b)
    assert_close(got.cpu().numpy(), ref, scale, what="dense rows V=%d K=%d+%d N=%d" % (V, K1, K2, N))
    again = rows_times(x1, w1, x2, w2, b)
    assert torch.equal(got, again)


def test_rows_past_the_inputs_are_not_touched_and_special_values_stay_in_their_rows():
    """V is not a multiple of the 16-row tile: the slots after the last row keep their contents;
    an infinity in one row of x reaches that row's outputs only (the padding lanes of the last
    tile re-read the last row and must not leak it)."""
    from jittorgeometric_amd import _lib
    L, l = _lib, _lib.load()
    V, K, N = 4099, 100, 72
    gen = torch.Generator(device=dev()).manual_seed(3)
    x = torch.randn((V, K), device=dev(), generator=gen)
    x[V - 1, 5] = float("inf")
    x[17, 99] = float("nan")
    w = torch.randn((K, N), device=dev(), generator=gen)
    buf = torch.full((V + 16, N), 7.0, device=dev())
    L.check(l.jgamd_dense_rows(L.ptr(x), L.ptr(w), K, None, None, 0, None, L.ptr(buf), V, N, 0, L.stream_ptr(dev())))
    out = buf.cpu().numpy()
    assert (out[V:] == 7.0).all()
    finite = np.isfinite(out[:V]).all(axis=1)
    assert not finite[V - 1] and not finite[17] and finite.sum() == V - 2


def test_shapes_outside_the_kernel_fall_back_and_are_refused_by_the_entry_point():
    from jittorgeometric_amd import JgamdError, _lib
    from jittorgeometric_amd.nn.dense import rows_times
    L, l = _lib, _lib.load()
    for K1, K2, N in ((47, 0, 128), (128, 0, 47), (200, 100, 64), (128, 6, 64)):
        assert l.jgamd_dense_rows_supported(K1, K2, N) == 0
    gen = torch.Generator(device=dev()).manual_seed(5)
    x = torch.randn((5000, 47), device=dev(), generator=gen)
    w = torch.randn((47, 41), device=dev(), generator=gen)
    b = torch.randn((41,), device=dev(), generator=gen)
    ref, scale = reference(x, w, None, None, b)
    assert_close(rows_times(x, w, bias=b).cpu().numpy(), ref, scale, what="BLAS route")
    out = torch.empty((5000, 41), device=dev())
    with pytest.raises(JgamdError):
        L.check(l.jgamd_dense_rows(L.ptr(x), L.ptr(w), 47, None, None, 0, None, L.ptr(out), 5000, 41, 0, L.stream_ptr(dev())))
    xs = torch.randn((5000, 256), device=dev(), generator=gen)[:, ::2]          # not contiguous: BLAS route
    w2 = torch.randn((128, 64), device=dev(), generator=gen)
    ref, scale = reference(xs, w2, None, None, None)
    assert_close(rows_times(xs, w2).cpu().numpy(), ref, scale, what="strided x")
