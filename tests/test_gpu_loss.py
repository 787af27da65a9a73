"""The mean cross-entropy kernel against the oracle's float64 restatement and against
torch's own float64 loss on the CPU."""
import numpy as np
import pytest
import torch

import oracle
from util import assert_close, dev, to_gpu

pytestmark = pytest.mark.gpu


def run(x, y, ydtype=torch.int64, upstream=None):
    from jittorgeometric_amd.nn import cross_entropy_loss
    xt = to_gpu(x).requires_grad_(True)
    yt = to_gpu(np.asarray(y)).to(ydtype)
    loss = cross_entropy_loss(xt, yt)
    (loss if upstream is None else loss * upstream).backward()
    return loss.item(), xt.grad.cpu().numpy()


@pytest.mark.parametrize("V,C,seed", [
    (1, 1, 0), (3, 2, 1), (100, 7, 2), (2049, 47, 3), (5000, 32, 4), (5000, 33, 5), (777, 64, 6),
    (300, 100, 7), (513, 256, 8), (64, 257, 9), (40, 1433, 10), (4097, 8, 11),
])
def test_against_oracle(V, C, seed):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((V, C)) * 4).astype(np.float32)
    y = rng.integers(0, C, V)
    want, wgrad = oracle.cross_entropy_loss(x, y)
    for ydtype in (torch.int64, torch.int32):
        got, grad = run(x, y, ydtype)
        assert abs(got - want) <= 1e-6 + 1e-5 * abs(want)
        # a gradient entry is (p - onehot) / V with p a ratio of float32 exponentials
        assert_close(grad, wgrad, scale=np.full_like(wgrad, 1.0 / V), rtol=1e-5, atol=0, what="grad")


def test_against_torch_float64_and_upstream_gradient():
    rng = np.random.default_rng(30)
    V, C = 10_000, 47
    x = (rng.standard_normal((V, C)) * 2).astype(np.float32)
    y = rng.integers(0, C, V)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(xt, torch.from_numpy(y))
    (ref * 2.5).backward()
    got, grad = run(x, y, upstream=2.5)
    assert abs(got - ref.item()) <= 1e-5 * abs(ref.item())
    assert_close(grad, xt.grad.numpy(), scale=np.full((V, C), 2.5 / V), rtol=1e-5, atol=0, what="grad")


def test_rows_without_a_label_are_left_out():
    rng = np.random.default_rng(31)
    V, C = 3000, 10
    x = rng.standard_normal((V, C)).astype(np.float32)
    y = rng.integers(0, C, V)
    y[::7] = -100
    y[5] = C
    want, wgrad = oracle.cross_entropy_loss(x, y)
    got, grad = run(x, y)
    assert abs(got - want) <= 1e-5 * abs(want)
    assert not grad[::7].any() and not grad[5].any()
    assert_close(grad, wgrad, scale=np.full_like(wgrad, 1.0 / V), rtol=1e-5, atol=0)
    none, gnone = run(x, np.full(V, -1))
    assert np.isnan(none) and not gnone.any()


def test_large_logits_and_infinities_stay_in_their_rows():
    x = np.zeros((4, 5), np.float32)
    x[0] = (1e4, -1e4, 0, 0, 0)
    x[1] = (88.0, 88.5, 89.0, -200.0, 3.0)
    x[2, 3] = -np.inf                      # one class ruled out
    x[3] = (1, 2, 3, 4, 5)
    y = np.array([1, 2, 0, 4])
    want, wgrad = oracle.cross_entropy_loss(x, y)
    got, grad = run(x, y)
    assert np.isfinite(got) and abs(got - want) <= 1e-5 * abs(want)
    assert_close(grad, wgrad, scale=np.full_like(wgrad, 0.25), rtol=1e-5, atol=0)


def test_run_to_run_identical_and_other_dtypes():
    from jittorgeometric_amd.nn import cross_entropy_loss, nll_loss
    rng = np.random.default_rng(32)
    V, C = 200_000, 47
    x = rng.standard_normal((V, C)).astype(np.float32)
    y = rng.integers(0, C, V)
    a = run(x, y)
    b = run(x, y)
    assert a[0] == b[0] and np.array_equal(a[1], b[1])
    # float64 logits are narrowed, a strided view is copied; the gradient comes back in the input's dtype
    xt = to_gpu(x[:500].astype(np.float64)).requires_grad_(True)
    cross_entropy_loss(xt, to_gpu(y[:500])).backward()
    want, wgrad = oracle.cross_entropy_loss(x[:500], y[:500])
    assert xt.grad.dtype == torch.float64
    assert_close(xt.grad.cpu().numpy(), wgrad, scale=np.full_like(wgrad, 1 / 500), rtol=1e-5, atol=0)
    wide = to_gpu(np.concatenate([x[:500], x[:500]], axis=1))
    view = wide[:, :C]
    assert not view.is_contiguous()
    assert abs(cross_entropy_loss(view, to_gpu(y[:500])).item() - want) <= 1e-5 * abs(want)
    # rows of log-probabilities: the same number as log_softmax + nll_loss, a gradient of -1 / rows at
    # the labels, and through torch's log_softmax the gradient of the fused loss
    xs = to_gpu(x[:500]).requires_grad_(True)
    logp = torch.log_softmax(xs, dim=1)
    logp.retain_grad()
    got = nll_loss(logp, to_gpu(y[:500]))
    got.backward()
    assert abs(got.item() - want) <= 1e-5 * abs(want)
    onehot = np.zeros((500, C))
    onehot[np.arange(500), y[:500]] = 1
    assert np.array_equal(logp.grad.cpu().numpy(), (-onehot / 500).astype(np.float32))
    assert_close(xs.grad.cpu().numpy(), wgrad, scale=np.full_like(wgrad, 1 / 500), rtol=1e-5, atol=0)
    # not log-probabilities: still -mean(row[label]), whatever the rows sum to
    raw = to_gpu(x[:500])
    assert abs(nll_loss(raw, to_gpu(y[:500])).item() + x[np.arange(500), y[:500]].astype(np.float64).mean()) <= 1e-5


def test_bad_arguments_are_refused():
    from jittorgeometric_amd import _lib
    from jittorgeometric_amd.nn import cross_entropy_loss
    with pytest.raises(_lib.JgamdError):
        cross_entropy_loss(torch.zeros(4, 3), torch.zeros(4, dtype=torch.int64))            # CPU tensors
    with pytest.raises(_lib.JgamdError):
        cross_entropy_loss(torch.zeros(4, 3, device=dev()), torch.zeros(5, dtype=torch.int64, device=dev()))
    with pytest.raises(_lib.JgamdError):
        cross_entropy_loss(torch.zeros(4, device=dev()), torch.zeros(4, dtype=torch.int64, device=dev()))
