"""Pins the CPU oracle's convolution routines without the reference:
brute-force definitions, adjoint identities in float64, torch CPU, special cases."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

import oracle
from tests import brute
from tests.cases import CONV_CASES, CONVT_CASES, random_conv_cases, random_convt_cases


def _rand(shape, rng, dtype=np.float64):
    return rng.standard_normal(shape).astype(dtype)


@pytest.mark.parametrize('case', CONV_CASES)
def test_conv_forward_backward_match_definition(case):
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(1)
    x = _rand((n, c, h, w_), rng)
    w = _rand((k, c // g, r, s), rng)
    b = _rand((k,), rng)
    y_def = brute.conv2d_def(x, w, b, st, pd, dl, g)
    y, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, g)
    assert y.shape == y_def.shape
    assert y.shape[-2:] == (oracle.conv_output_size(h, r, st[0], pd[0], dl[0]),
                            oracle.conv_output_size(w_, s, st[1], pd[1], dl[1]))
    np.testing.assert_allclose(y, y_def, rtol=1e-12, atol=1e-12)
    gy = _rand(y.shape, rng)
    dx_def, dw_def, db_def = brute.conv2d_grads_def(x, w, gy, st, pd, dl, g)
    dx, dw, db = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
    assert dx.shape == x.shape and dw.shape == w.shape and db.shape == (k,)
    np.testing.assert_allclose(dx, dx_def, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dw, dw_def, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(db, db_def, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize('case', CONV_CASES)
def test_conv_adjoint_identities(case):
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(2)
    x = _rand((n, c, h, w_), rng)
    w = _rand((k, c // g, r, s), rng)
    y, xpad = oracle.convolution_forward(x, w, None, st, pd, dl, g)
    gy = _rand(y.shape, rng)
    dx, dw, _ = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
    lhs = float((y * gy).sum())
    assert abs(lhs - float((x * dx).sum())) <= 1e-10 * max(1.0, abs(lhs))
    assert abs(lhs - float((w * dw).sum())) <= 1e-10 * max(1.0, abs(lhs))


@pytest.mark.parametrize('case', CONV_CASES + random_conv_cases(60, 2024))
def test_conv_matches_torch_cpu_fp32(case):
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(3)
    x = _rand((n, c, h, w_), rng, np.float32)
    w = _rand((k, c // g, r, s), rng, np.float32)
    b = _rand((k,), rng, np.float32)
    xt = torch.tensor(x, requires_grad=True)
    wt = torch.tensor(w, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    yt = TF.conv2d(xt, wt, bt, st, pd, dl, g)
    y, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, g)
    assert y.dtype == np.float32
    gy = _rand(y.shape, rng, np.float32)
    yt.backward(torch.tensor(gy))
    dx, dw, db = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-4, atol=1e-5)
    scale = max(1.0, float(np.abs(dw).max()), float(np.abs(db).max()))     # sums over N*P*Q terms
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-4, atol=2e-5 * scale)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-4, atol=2e-5 * scale)


def test_conv_1x1_is_matrix_product():
    rng = np.random.default_rng(4)
    x = _rand((3, 5, 4, 6), rng)
    w = _rand((7, 5, 1, 1), rng)
    y, _ = oracle.conv2d(x, w)
    ref = np.einsum('kc,nchw->nkhw', w[:, :, 0, 0], x)
    np.testing.assert_allclose(y, ref, rtol=1e-13, atol=1e-13)


def test_conv_padding_zero_returns_same_array_as_padded():
    # grad_nn.py:465-469: with no padding the "padded" input is the input itself
    x = np.ones((1, 1, 3, 3), np.float32)
    w = np.ones((1, 1, 2, 2), np.float32)
    assert oracle.conv2d(x, w)[1] is x


def test_notebook_case_shapes_and_torch_parity():
    """examples/conv2d_result_speed_comparison.ipynb cells 1-7: N=128, C=4, 64x64,
    weight (16,2,3,2), stride (1,3), padding (2,3), dilation (1,2), groups=2; the notebook
    expects output (128,16,66,23), y/dx allclose(atol=1e-5, rtol=1e-5) and dw/db at rtol=1e-3
    against PyTorch (its data are unseeded, so only the configuration is a fixture)."""
    rng = np.random.default_rng(5)
    x = _rand((128, 4, 64, 64), rng, np.float32)
    w = _rand((16, 2, 3, 2), rng, np.float32)
    b = _rand((16,), rng, np.float32)
    st, pd, dl, g = (1, 3), (2, 3), (1, 2), 2
    y, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, g)
    assert y.shape == (128, 16, 66, 23)
    gy = _rand(y.shape, rng, np.float32)
    dx, dw, db = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
    xt = torch.tensor(x, requires_grad=True)
    wt = torch.tensor(w, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    yt = TF.conv2d(xt, wt, bt, st, pd, dl, g)
    yt.backward(torch.tensor(gy))
    assert np.allclose(y, yt.detach().numpy(), atol=1e-5, rtol=1e-5)
    assert np.allclose(dx, xt.grad.numpy(), atol=1e-5, rtol=1e-5)
    assert np.allclose(dw, wt.grad.numpy(), atol=1e-5, rtol=1e-3)
    assert np.allclose(db, bt.grad.numpy(), atol=1e-5, rtol=1e-3)


@pytest.mark.parametrize('case', CONVT_CASES)
def test_conv_transpose_matches_definition_and_torch(case):
    n, ci, h, w_, co, r, s, st, pd, op, dl, g = case
    rng = np.random.default_rng(6)
    x = _rand((n, ci, h, w_), rng)
    w = _rand((ci, co // g, r, s), rng)
    b = _rand((co,), rng)
    y_def = brute.conv_transpose2d_def(x, w, b, st, pd, op, dl, g)
    y = oracle.transposed_convolution_forward(x, w, b, st, pd, op, dl, g)
    assert y.shape == y_def.shape
    np.testing.assert_allclose(y, y_def, rtol=1e-12, atol=1e-12)
    xt = torch.tensor(x, requires_grad=True)
    wt = torch.tensor(w, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    yt = TF.conv_transpose2d(xt, wt, bt, st, pd, op, g, dl)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-11, atol=1e-11)
    gy = _rand(y.shape, rng)
    yt.backward(torch.tensor(gy))
    dx, dw, db = oracle.transposed_convolution_backward(gy, x, w, st, pd, dl, g)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-11, atol=1e-11)
    # adjointness with the forward convolution that has this layer as its input gradient
    lhs = float((y_def - b[None, :, None, None]).ravel() @ gy.ravel())
    assert abs(lhs - float((x * dx).sum())) <= 1e-10 * max(1.0, abs(lhs))
    assert abs(lhs - float((w * dw).sum())) <= 1e-10 * max(1.0, abs(lhs))


@pytest.mark.parametrize('case', random_convt_cases(40, 99))
def test_conv_transpose_random_geometries_against_torch(case):
    n, ci, h, w_, co, r, s, st, pd, op, dl, g = case
    rng = np.random.default_rng(8)
    x, w, b = _rand((n, ci, h, w_), rng), _rand((ci, co // g, r, s), rng), _rand((co,), rng)
    y = oracle.transposed_convolution_forward(x, w, b, st, pd, op, dl, g)
    xt, wt, bt = (torch.tensor(a, requires_grad=True) for a in (x, w, b))
    yt = TF.conv_transpose2d(xt, wt, bt, st, pd, op, g, dl)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-11, atol=1e-11)
    gy = _rand(y.shape, rng)
    yt.backward(torch.tensor(gy))
    dx, dw, db = oracle.transposed_convolution_backward(gy, x, w, st, pd, dl, g)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-11, atol=1e-11)


def test_conv_transpose_output_size_formula():
    # nn/modules/conv.py:132-136 and grad_nn.py:677-678
    assert oracle.conv_transpose_output_size(4, 4, 2, 1, 1, 0) == 8
    assert oracle.conv_transpose_output_size(1, 4, 1, 0, 1, 0) == 4
    assert oracle.conv_transpose_output_size(5, 3, 2, 1, 1, 1) == 10


def test_seeded_conv_parameters_follow_reference_draw_order():
    """weight first, then bias, both U(-1/sqrt(fan_in), 1/sqrt(fan_in)) from np.random's
    legacy stream (nn/init.py:6-10, :91-96; nn/modules/conv.py:48-56)."""
    np.random.seed(0)
    w, b = oracle.conv_parameters(16, 32, (3, 3))
    bound = 1 / np.sqrt(16 * 9)
    np.random.seed(0)
    w2 = np.random.uniform(-1, 1, size=(32, 16, 3, 3))
    b2 = np.random.uniform(-1, 1, size=(32,))
    np.testing.assert_allclose(w, (w2 * bound).astype(np.float32), rtol=2e-6)
    np.testing.assert_allclose(b, (b2 * bound).astype(np.float32), rtol=2e-6)
    assert w.dtype == np.float32 and np.abs(w).max() <= bound
