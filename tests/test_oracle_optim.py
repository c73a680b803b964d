"""Pins the optimiser oracle with torch CPU optimisers and closed forms."""
import numpy as np
import pytest
import torch

import oracle


def _trajectory(shape, steps, seed):
    rng = np.random.default_rng(seed)
    p0 = rng.standard_normal(shape).astype(np.float32)
    grads = [rng.standard_normal(shape).astype(np.float32) for _ in range(steps)]
    return p0, grads


@pytest.mark.parametrize('kw', [
    dict(momentum=0, dampening=0, weight_decay=0, nesterov=False),
    dict(momentum=0.9, dampening=0, weight_decay=0, nesterov=False),
    dict(momentum=0.9, dampening=0.1, weight_decay=5e-4, nesterov=False),
    dict(momentum=0.8, dampening=0, weight_decay=1e-3, nesterov=True),
])
def test_sgd_against_torch(kw):
    p0, grads = _trajectory((7, 5), 6, 0)
    p = p0.copy()
    bufs = [None]
    pt = torch.from_numpy(p0.copy()).requires_grad_()
    opt = torch.optim.SGD([pt], lr=0.05, **kw)
    for g in grads:
        oracle.optim.sgd([p], [g.copy()], bufs, kw['weight_decay'], kw['momentum'], 0.05, kw['dampening'],
                         kw['nesterov'])
        pt.grad = torch.from_numpy(g.copy())
        opt.step()
    np.testing.assert_allclose(p, pt.detach().numpy(), rtol=2e-6, atol=1e-7)


def test_sgd_closed_forms():
    p = np.float32([1.0, -2.0, 0.5])
    g = np.float32([0.5, 0.25, -1.0])
    oracle.optim.sgd([p], [g.copy()], [None], 0, 0, 0.1, 0, False)
    np.testing.assert_allclose(p, [0.95, -2.025, 0.6], rtol=1e-6)
    # constant gradient, momentum mu: buffer after k steps = g * (1 - mu^k) / (1 - mu)
    p = np.zeros(3, np.float32)
    bufs = [None]
    for _ in range(5):
        oracle.optim.sgd([p], [g.copy()], bufs, 0, 0.5, 1.0, 0, False)
    np.testing.assert_allclose(bufs[0], g * (1 - 0.5 ** 5) / 0.5, rtol=1e-6)
    np.testing.assert_allclose(p, -g * sum((1 - 0.5 ** k) / 0.5 for k in range(1, 6)), rtol=1e-6)


@pytest.mark.parametrize('decoupled', [False, True])
@pytest.mark.parametrize('amsgrad', [False, True])
@pytest.mark.parametrize('weight_decay', [0, 1e-2])
def test_adam_against_torch(decoupled, amsgrad, weight_decay):
    p0, grads = _trajectory((6, 4), 8, 1)
    p = p0.copy()
    m, v, vmax = np.zeros_like(p), np.zeros_like(p), np.zeros_like(p)
    pt = torch.from_numpy(p0.copy()).requires_grad_()
    cls = torch.optim.AdamW if decoupled else torch.optim.Adam
    opt = cls([pt], lr=1e-2, betas=(0.9, 0.99), eps=1e-8, weight_decay=weight_decay, amsgrad=amsgrad)
    for step, g in enumerate(grads, 1):
        oracle.optim.adam([p], [g], [m], [v], [vmax], [step], amsgrad, 0.9, 0.99, 1e-2, weight_decay, 1e-8, decoupled)
        pt.grad = torch.from_numpy(g.copy())
        opt.step()
    assert p.dtype == np.float32
    np.testing.assert_allclose(p, pt.detach().numpy(), rtol=5e-6, atol=1e-7)


def test_adam_first_step_moves_by_lr_times_sign():
    p = np.zeros(4, np.float32)
    g = np.float32([3.0, -0.01, 100.0, -7.0])
    m, v = np.zeros_like(p), np.zeros_like(p)
    oracle.optim.adam([p], [g], [m], [v], [None], [1], False, 0.9, 0.999, 1e-3, 0, 1e-12)
    np.testing.assert_allclose(p, -1e-3 * np.sign(g), rtol=1e-5)
