"""Pins the MaxPool2d and activation oracles without the reference: loop-level definitions,
torch CPU as a library routine, closed forms."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

import oracle
from tests import brute
from tests.cases import POOL_CASES, random_pool_cases


def _data(case, seed=0, ties=False):
    n, c, h, w = case[:4]
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    if ties:
        x = np.round(x)          # many equal values: the first maximum must win
    return x, rng


def _where_from_pos(pos, case):
    """(input row, input column) of each arg-max from the oracle's (kernel row, kernel column)."""
    (kh, kw), (sh, sw), (ph, pw), (dh, dw) = case[4:8]
    idx2, idx1_m = (np.moveaxis(a, -1, 1) for a in pos)           # [N,C,P,Q]
    p = np.arange(idx2.shape[2])[None, None, :, None]
    q = np.arange(idx2.shape[3])[None, None, None, :]
    return p * sh - ph + idx2 * dh, q * sw - pw + idx1_m * dw


@pytest.mark.parametrize('ties', [False, True])
@pytest.mark.parametrize('case', POOL_CASES)
def test_max_pool_forward_against_loops_and_torch(case, ties):
    x, _ = _data(case, ties=ties)
    ks, st, pd, dl, cm = case[4:]
    y, pos = oracle.max_pool2d(x, ks, st, pd, dl, cm)
    out_hw = tuple(oracle.pool_output_size(x.shape[2 + a], ks[a], st[a], pd[a], dl[a], cm) for a in (0, 1))
    assert y.shape[-2:] == out_hw
    y_def, arg = brute.max_pool2d_def(x, ks, st, pd, dl, out_hw)
    np.testing.assert_array_equal(y, y_def)
    hh, ww = _where_from_pos(pos, case)
    for idx in np.ndindex(*y.shape):
        if arg[idx] is not None:
            assert (hh[idx], ww[idx]) == arg[idx]
    yt, it = TF.max_pool2d(torch.from_numpy(x), ks, st, pd, dl, ceil_mode=cm, return_indices=True)
    np.testing.assert_array_equal(y, yt.numpy())
    np.testing.assert_array_equal(hh * x.shape[3] + ww, it.numpy())     # same arg-max, ties included


@pytest.mark.parametrize('ties', [False, True])
@pytest.mark.parametrize('case', POOL_CASES)
def test_max_pool_backward_assigns_last_window(case, ties):
    x, rng = _data(case, seed=1, ties=ties)
    ks, st, pd, dl, cm = case[4:]
    y, pos = oracle.max_pool2d(x, ks, st, pd, dl, cm)
    g = rng.standard_normal(y.shape).astype(np.float32)
    dx = oracle.max_pool2d_backward(x.shape, g, pos, ks, st, pd, dl, cm)
    _, arg = brute.max_pool2d_def(x, ks, st, pd, dl, y.shape[-2:])
    np.testing.assert_array_equal(dx, brute.max_pool2d_backward_def(x.shape, g, arg))
    # where no pixel is chosen twice, assignment equals the summed (torch) gradient
    summed = brute.max_pool2d_backward_def(x.shape, g, arg, accumulate=True)
    xt = torch.from_numpy(x).requires_grad_()
    TF.max_pool2d(xt, ks, st, pd, dl, ceil_mode=cm).backward(torch.from_numpy(g))
    np.testing.assert_allclose(summed, xt.grad.numpy(), rtol=1e-6, atol=1e-6)
    chosen = np.zeros(x.shape, int)
    for idx in np.ndindex(*y.shape):
        if arg[idx] is not None:
            chosen[idx[0], idx[1], arg[idx][0], arg[idx][1]] += 1
    once = chosen <= 1
    np.testing.assert_array_equal(dx[once], summed[once])
    if ties and ks[0] > st[0]:
        assert (chosen > 1).any()           # the overlapping cases do exercise the difference


def test_max_pool_three_dimensional_input_and_output_size_rule():
    x = np.random.default_rng(2).standard_normal((3, 7, 6)).astype(np.float32)
    y, pos = oracle.max_pool2d(x, (2, 2), (2, 2))
    assert y.shape == (3, 3, 3)
    np.testing.assert_array_equal(y, oracle.max_pool2d(x[None], (2, 2), (2, 2))[0][0])
    dx = oracle.max_pool2d_backward(x.shape, np.ones_like(y), pos, (2, 2), (2, 2))
    assert dx.shape == x.shape and dx.sum() == y.size
    for size, k, s, p, d in [(112, 3, 2, 1, 1), (7, 3, 3, 0, 1), (6, 2, 2, 1, 1), (10, 3, 2, 1, 2), (5, 2, 4, 1, 1)]:
        for cm in (False, True):
            t = TF.max_pool2d(torch.zeros(1, 1, size, size), k, s, p, d, ceil_mode=cm)
            assert oracle.pool_output_size(size, k, s, p, d, cm) == t.shape[-1]


def test_relu_and_leaky_relu_closed_forms_and_torch():
    x = np.array([-2.0, -0.5, 0.0, 0.5, 3.0, np.nan], np.float32)
    g = np.array([1.0, 2.0, 3.0, 4.0, 5.0, 6.0], np.float32)
    y = oracle.relu_forward(x)
    np.testing.assert_array_equal(y[:5], [0, 0, 0, 0.5, 3.0])
    assert np.isnan(y[5])
    np.testing.assert_array_equal(oracle.relu_backward(g, y)[:5], [0, 0, 0, 4, 5])
    yl = oracle.leaky_relu_forward(x, 0.2)
    np.testing.assert_allclose(yl[:5], [-0.4, -0.1, 0, 0.5, 3.0], rtol=1e-7)
    assert np.isnan(yl[5])
    gl = oracle.leaky_relu_backward(g, x, 0.2)
    np.testing.assert_allclose(gl, [0.2, 0.4, 3, 4, 5, 6], rtol=1e-7)
    np.testing.assert_array_equal(g, [1, 2, 3, 4, 5, 6])          # the caller's array is left alone
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    g = rng.standard_normal(x.shape).astype(np.float32)
    for slope in (0.01, 0.2):
        xt = torch.from_numpy(x).requires_grad_()
        yt = TF.leaky_relu(xt, slope)
        yt.backward(torch.from_numpy(g))
        np.testing.assert_allclose(oracle.leaky_relu_forward(x, slope), yt.detach().numpy(), rtol=1e-7)
        np.testing.assert_allclose(oracle.leaky_relu_backward(g, x, slope), xt.grad.numpy(), rtol=1e-7)
    xt = torch.from_numpy(x).requires_grad_()
    yt = TF.relu(xt)
    yt.backward(torch.from_numpy(g))
    np.testing.assert_array_equal(oracle.relu_forward(x), yt.detach().numpy())
    np.testing.assert_array_equal(oracle.relu_backward(g, oracle.relu_forward(x)), xt.grad.numpy())


@pytest.mark.parametrize('case', random_pool_cases(60, 77))
def test_max_pool_random_geometries_against_torch(case):
    """Values and arg-max positions against torch on the geometries the GPU sweep uses (rounded
    inputs, so ties are everywhere); windows that lie wholly in the padding are left out of the
    index comparison (torch reports an index there, the reference's tap points into the padding)."""
    x, _ = _data(case, seed=3, ties=True)
    ks, st, pd, dl, cm = case[4:]
    y, pos = oracle.max_pool2d(x, ks, st, pd, dl, cm)
    yt, it = TF.max_pool2d(torch.from_numpy(x), ks, st, pd, dl, ceil_mode=cm, return_indices=True)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_array_equal(y, yt.numpy())
    hh, ww = _where_from_pos(pos, case)
    inside = (hh >= 0) & (hh < x.shape[2]) & (ww >= 0) & (ww < x.shape[3])
    np.testing.assert_array_equal((hh * x.shape[3] + ww)[inside], it.numpy()[inside])
