"""Pins the classifier-head oracle (mean, matrix product / linear, log-softmax, NLL loss) with
torch CPU as a library routine and closed forms."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

import oracle


def test_mean_over_spatial_dimensions():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, 5, 7, 7)).astype(np.float32)
    for dim, keep in [((-1, -2), True), ((2, 3), False), (None, False), (3, True)]:
        y = oracle.mean_forward(x, dim, keep)
        xt = torch.from_numpy(x).requires_grad_()
        yt = xt.mean() if dim is None else xt.mean(dim, keepdim=keep)
        np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-6, atol=1e-7)
        g = rng.standard_normal(np.shape(y)).astype(np.float32)
        yt.backward(torch.from_numpy(np.asarray(g)))
        dx = oracle.mean_backward(np.asarray(g), x.shape, dim, keep)
        np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-6, atol=1e-8)
    # closed form: every element receives g / count
    dx = oracle.mean_backward(np.float32([[2.0], [4.0]]).reshape(2, 1, 1, 1), (2, 1, 2, 2), (-1, -2), True)
    np.testing.assert_array_equal(dx.ravel(), [0.5] * 4 + [1.0] * 4)


def test_linear_is_x_wT_plus_b_with_torch_gradients():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((6, 10)).astype(np.float32)
    w = rng.standard_normal((4, 10)).astype(np.float32)
    b = rng.standard_normal(4).astype(np.float32)
    g = rng.standard_normal((6, 4)).astype(np.float32)
    y = oracle.linear_forward(x, w, b)
    xt, wt, bt = (torch.from_numpy(a).requires_grad_() for a in (x, w, b))
    yt = TF.linear(xt, wt, bt)
    yt.backward(torch.from_numpy(g))
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-5, atol=1e-6)
    dx, dw, db = oracle.linear_backward(g, x, w)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-5, atol=1e-6)
    # element by element, in float64
    want = np.array([[sum(float(x[i, k]) * float(w[j, k]) for k in range(10)) + float(b[j]) for j in range(4)]
                     for i in range(6)])
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-6)
    ga, gb = oracle.mm_backward(g, x, w.T.copy())
    np.testing.assert_allclose(ga, g @ w, rtol=1e-6)
    np.testing.assert_allclose(gb, x.T @ g, rtol=1e-6)


def test_log_softmax_normalisation_and_torch():
    rng = np.random.default_rng(2)
    x = (5 * rng.standard_normal((7, 13))).astype(np.float32)
    x[0] += 80                      # large logits: the shift by the row maximum keeps exp finite
    y = oracle.log_softmax_forward(x, -1)
    np.testing.assert_allclose(np.exp(y.astype(np.float64)).sum(-1), 1.0, rtol=1e-6)
    xt = torch.from_numpy(x).requires_grad_()
    yt = TF.log_softmax(xt, -1)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-5, atol=1e-6)
    g = rng.standard_normal(x.shape).astype(np.float32)
    yt.backward(torch.from_numpy(g))
    dx = oracle.log_softmax_backward(g, y, -1)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-5, atol=1e-6)
    # shifting a row by a constant leaves y unchanged, so a gradient row sums to zero
    np.testing.assert_allclose(dx.sum(-1), 0, atol=1e-5)


@pytest.mark.parametrize('reduction', ['mean', 'sum', 'none'])
@pytest.mark.parametrize('weighted', [False, True])
@pytest.mark.parametrize('ignore_index', [-100, 2])
def test_nll_loss_against_torch(reduction, weighted, ignore_index):
    rng = np.random.default_rng(3)
    n, c = 12, 5
    logp = oracle.log_softmax_forward(rng.standard_normal((n, c)).astype(np.float32))
    target = rng.integers(0, c, n)
    target[:3] = 2
    weight = rng.uniform(0.5, 2.0, c).astype(np.float32) if weighted else None
    loss, count = oracle.nll_loss_forward(logp, target, weight, ignore_index, reduction)
    lt = torch.from_numpy(logp).requires_grad_()
    out = TF.nll_loss(lt, torch.from_numpy(target), None if weight is None else torch.from_numpy(weight),
                      ignore_index=ignore_index, reduction=reduction)
    if reduction == 'mean' and weighted:
        # torch divides by the sum of the weights, the reference by the number of non-zero weights (:317-318)
        w_rows = weight[target] * (target != ignore_index if ignore_index >= 0 else 1)
        np.testing.assert_allclose(loss * count, out.item() * w_rows.sum(), rtol=1e-5)
    else:
        np.testing.assert_allclose(loss, out.detach().numpy(), rtol=1e-5, atol=1e-7)
    g = rng.standard_normal(np.shape(loss)).astype(np.float32) if reduction == 'none' else np.float32(1.5)
    grad = oracle.nll_loss_backward(g, logp.shape, target, weight, ignore_index, reduction, count)
    out.backward(torch.from_numpy(np.asarray(g)))
    want = lt.grad.numpy()
    if reduction == 'mean' and weighted:
        want = want * (w_rows.sum() / count)
    np.testing.assert_allclose(grad, want, rtol=1e-5, atol=1e-7)


def test_nll_loss_closed_forms():
    logp = np.log(np.float32([[1.0, 1e-30], [0.25, 0.75]]))
    loss, count = oracle.nll_loss_forward(logp, np.array([0, 1]))
    assert count == 2
    np.testing.assert_allclose(loss, -np.log(0.75) / 2, rtol=1e-6)
    grad = oracle.nll_loss_backward(np.float32(1.0), logp.shape, np.array([0, 1]), count=count)
    np.testing.assert_array_equal(grad, [[-0.5, 0], [0, -0.5]])
    with pytest.raises(ValueError):
        oracle.nll_loss_forward(logp, np.array([0, 1]), reduction='median')
