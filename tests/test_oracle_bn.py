"""Pins the CPU oracle's BatchNorm without the reference: closed forms, invariants,
torch CPU (forward, running buffers, autograd) and float64 finite differences."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

import oracle

SHAPES = [(4, 3, 5, 5), (2, 8, 1, 3), (16, 5, 4, 4), (3, 2, 7, 9)]


def _inputs(shape, dtype=np.float32, seed=0):
    rng = np.random.default_rng(seed)
    c = shape[1]
    x = (2 + 3 * rng.standard_normal(shape)).astype(dtype)
    gamma = rng.uniform(0.5, 1.5, c).astype(dtype)
    beta = (0.1 * rng.standard_normal(c)).astype(dtype)
    gy = rng.standard_normal(shape).astype(dtype)
    return x, gamma, beta, gy


@pytest.mark.parametrize('shape', SHAPES)
def test_forward_closed_forms(shape):
    x, gamma, beta, _ = _inputs(shape, np.float64)
    eps = 1e-5
    y, saved, rm, rv = oracle.batch_norm_forward(x, gamma, beta, np.zeros(shape[1]), np.ones(shape[1]),
                                                 True, 0.1, eps)
    ax = (0, 2, 3)
    m = x.size // shape[1]
    mu = x.sum(ax) / m
    var = ((x - mu[:, None, None]) ** 2).sum(ax) / m
    np.testing.assert_allclose(y.mean(ax), beta, atol=1e-12)
    np.testing.assert_allclose(y.var(ax), gamma ** 2 * var / (var + eps), rtol=1e-11)
    np.testing.assert_allclose(saved['mean'].ravel(), mu, rtol=1e-12)
    np.testing.assert_allclose(saved['var'].ravel(), var + eps, rtol=1e-12)     # 'var' includes eps
    np.testing.assert_allclose(saved['sd'].ravel(), np.sqrt(var + eps), rtol=1e-12)
    assert saved['mean'].shape == (shape[1], 1, 1)
    np.testing.assert_allclose(rm, 0.9 * 0 + 0.1 * mu, rtol=1e-12)
    np.testing.assert_allclose(rv, 0.9 * 1 + 0.1 * var * m / (m - 1), rtol=1e-12)   # unbiased running var


def test_running_stat_recurrence_over_steps():
    rng = np.random.default_rng(7)
    c, mom = 3, 0.3
    rm, rv = np.zeros(c), np.ones(c)
    exp_m, exp_v = rm.copy(), rv.copy()
    for _ in range(4):
        x = rng.standard_normal((5, c, 2, 3)) * 2 + 1
        _, _, rm, rv = oracle.batch_norm_forward(x, None, None, rm, rv, True, mom, 1e-5)
        exp_m = (1 - mom) * exp_m + mom * x.mean((0, 2, 3))
        exp_v = (1 - mom) * exp_v + mom * x.var((0, 2, 3), ddof=1)
    np.testing.assert_allclose(rm, exp_m, rtol=1e-12)
    np.testing.assert_allclose(rv, exp_v, rtol=1e-12)


@pytest.mark.parametrize('shape', SHAPES)
def test_matches_torch_cpu_fp32(shape):
    x, gamma, beta, gy = _inputs(shape)
    c = shape[1]
    rm0 = np.linspace(-1, 1, c).astype(np.float32)
    rv0 = np.linspace(0.5, 2, c).astype(np.float32)
    y, saved, rm, rv = oracle.batch_norm_forward(x, gamma, beta, rm0, rv0, True, 0.1, 1e-5)
    dx, dg, db = oracle.batch_norm_backward(gy, x, gamma, saved)
    xt = torch.tensor(x, requires_grad=True)
    gt = torch.tensor(gamma, requires_grad=True)
    bt = torch.tensor(beta, requires_grad=True)
    rmt, rvt = torch.tensor(rm0.copy()), torch.tensor(rv0.copy())
    yt = TF.batch_norm(xt, rmt, rvt, gt, bt, True, 0.1, 1e-5)
    yt.backward(torch.tensor(gy))
    assert y.dtype == np.float32 and rm.dtype == np.float32 and dx.dtype == np.float32
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(rm, rmt.numpy(), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(rv, rvt.numpy(), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-4, atol=2e-6)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize('shape', SHAPES)
def test_backward_invariants_and_closed_forms(shape):
    x, gamma, beta, gy = _inputs(shape, np.float64)
    y, saved, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, True, 0.1, 1e-5)
    dx, dg, db = oracle.batch_norm_backward(gy, x, gamma, saved)
    xhat = (x - saved['mean']) / saved['sd']
    ax = (0, 2, 3)
    np.testing.assert_allclose(dx.sum(ax), 0, atol=1e-11)
    # sum(dx*xhat) vanishes only up to eps: sum(xhat^2) = M*var/(var+eps), which leaves
    # (gamma/sd) * sum(dy*xhat) * eps/(var+eps)
    resid = gamma / saved['sd'].ravel() * (gy * xhat).sum(ax) * 1e-5 / saved['var'].ravel()
    np.testing.assert_allclose((dx * xhat).sum(ax), resid, atol=1e-11)
    np.testing.assert_allclose(db, gy.sum(ax), rtol=1e-12)
    np.testing.assert_allclose(dg, (gy * xhat).sum(ax), rtol=1e-12)
    m = x.size // shape[1]
    closed = (gamma[:, None, None] / saved['sd']) * (
        gy - gy.sum(ax, keepdims=True)[0] / m - xhat * (gy * xhat).sum(ax, keepdims=True)[0] / m)
    np.testing.assert_allclose(dx, closed, rtol=1e-9, atol=1e-12)


def test_backward_finite_differences_float64():
    x, gamma, beta, gy = _inputs((3, 2, 2, 3), np.float64, seed=3)

    def loss(xx, gg, bb):
        y = oracle.batch_norm_forward(xx, gg, bb, None, None, True, 0.1, 1e-5)[0]
        return float((y * gy).sum())

    _, saved, _, _ = oracle.batch_norm_forward(x, gamma, beta, None, None, True, 0.1, 1e-5)
    dx, dg, db = oracle.batch_norm_backward(gy, x, gamma, saved)
    h = 1e-6
    for idx in [(0, 0, 0, 0), (2, 1, 1, 2), (1, 0, 1, 1)]:
        xp_, xm_ = x.copy(), x.copy()
        xp_[idx] += h
        xm_[idx] -= h
        assert abs((loss(xp_, gamma, beta) - loss(xm_, gamma, beta)) / (2 * h) - dx[idx]) < 1e-6
    for c in range(2):
        gp, gm = gamma.copy(), gamma.copy()
        gp[c] += h
        gm[c] -= h
        assert abs((loss(x, gp, beta) - loss(x, gm, beta)) / (2 * h) - dg[c]) < 1e-6
        bp, bm = beta.copy(), beta.copy()
        bp[c] += h
        bm[c] -= h
        assert abs((loss(x, gamma, bp) - loss(x, gamma, bm)) / (2 * h) - db[c]) < 1e-6


def test_eval_mode_uses_running_stats_and_no_affine():
    x, _, _, _ = _inputs((4, 3, 2, 2), np.float64)
    rm = np.array([0.5, 1.0, 2.0])
    rv = np.array([1.0, 4.0, 9.0])
    y, saved, nrm, nrv = oracle.batch_norm_forward(x, None, None, rm, rv, False, 0.1, 1e-5)
    assert nrm is None and nrv is None
    np.testing.assert_allclose(y, (x - rm[:, None, None]) / np.sqrt(rv + 1e-5)[:, None, None], rtol=1e-12)


def test_single_value_per_channel_raises():
    with pytest.raises(ValueError, match='Expected more than 1 value per channel'):
        oracle.batch_norm_forward(np.zeros((1, 3, 1, 1), np.float32), None, None, None, None, True, 0.1, 1e-5)
