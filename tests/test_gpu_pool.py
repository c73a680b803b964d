"""GPU parity: MaxPool2d forward / backward and LeakyReLU through the C ABI vs the CPU oracle.

Max pooling copies values, so everything here is compared bit for bit."""
import numpy as np
import pytest

import oracle
from tests.cases import POOL_CASES, random_pool_cases

pytestmark = pytest.mark.gpu


def _run_pool(case, seed, ties):
    from pytortto_amd import ops
    from pytortto_amd.autograd.grad_nn import pool_output_size
    from pytortto_amd.xparray import hiparray
    n, c, h, w, ks, st, pd, dl, cm = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    if ties:
        x = np.round(x)
    y_ref, (idx2, idx1_m) = oracle.max_pool2d(x, ks, st, pd, dl, cm)
    g = rng.standard_normal(y_ref.shape).astype(np.float32)
    dx_ref = oracle.max_pool2d_backward(x.shape, g, (idx2, idx1_m), ks, st, pd, dl, cm)
    out_hw = tuple(pool_output_size(x.shape[2 + a], ks[a], st[a], pd[a], dl[a], cm) for a in (0, 1))
    assert out_hw == y_ref.shape[-2:]
    y, tap = ops.maxpool2d_fwd(hiparray(x), out_hw, ks, st, pd, dl)
    np.testing.assert_array_equal(y.get(), y_ref)
    np.testing.assert_array_equal(tap.get(), np.moveaxis(idx2 * ks[1] + idx1_m, -1, 1))
    dx = ops.maxpool2d_bwd(hiparray(g), tap, (h, w), ks, st, pd, dl)
    np.testing.assert_array_equal(dx.get(), dx_ref)


@pytest.mark.parametrize('ties', [False, True])
@pytest.mark.parametrize('case', POOL_CASES)
def test_max_pool_small_geometries(case, ties):
    _run_pool(case, seed=4, ties=ties)


def test_max_pool_resnet_stem_shape_reduced_batch():
    _run_pool((4, 64, 112, 112, (3, 3), (2, 2), (1, 1), (1, 1), False), seed=5, ties=False)
    _run_pool((2, 16, 113, 57, (3, 3), (2, 2), (1, 1), (1, 1), True), seed=6, ties=True)


def test_max_pool_rows_too_wide_for_the_lds_stage():
    # three input rows of 1500 (forward) / two gradient rows of 1100 (backward) exceed the staged
    # span: both passes take the direct kernels
    _run_pool((1, 2, 8, 1500, (3, 3), (2, 2), (1, 1), (1, 1), False), seed=10, ties=True)
    _run_pool((1, 1, 6, 2200, (3, 3), (2, 2), (1, 1), (1, 1), False), seed=11, ties=False)
    _run_pool((1, 2, 40, 700, (5, 2), (1, 1), (2, 1), (1, 1), False), seed=12, ties=True)   # one output row per block


def test_max_pool_more_than_65535_planes():
    _run_pool((1100, 60, 4, 6, (2, 2), (2, 2), (0, 0), (1, 1), False), seed=13, ties=True)


def test_max_pool_full_size_properties():
    """[64,64,112,112], 3x3 stride 2 padding 1 (the ResNet-50 stem pooling): with dy = y every
    assigned gradient equals the input at that pixel, each window's maximum is found in the
    input plane, and the plane maximum survives."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(7)
    x = rng.standard_normal((64, 64, 112, 112), dtype=np.float32)
    xd = hiparray(x)
    y, tap = ops.maxpool2d_fwd(xd, (56, 56), (3, 3), (2, 2), (1, 1), (1, 1))
    dx = ops.maxpool2d_bwd(y, tap, (112, 112), (3, 3), (2, 2), (1, 1), (1, 1)).get()
    yh, th = y.get(), tap.get()
    assert th.min() >= 0 and th.max() <= 8
    np.testing.assert_array_equal(yh.max(axis=(2, 3)), x.max(axis=(2, 3)))
    chosen = dx != 0
    np.testing.assert_array_equal(dx[chosen], x[chosen])
    # the arg-max of window (p, q) is x[2p-1+i, 2q-1+j]: rebuild y from x and tap
    p = np.arange(56)[:, None]
    q = np.arange(56)[None, :]
    hh, ww = 2 * p - 1 + th // 3, 2 * q - 1 + th % 3
    n_i = np.arange(64)[:, None, None, None]
    c_i = np.arange(64)[None, :, None, None]
    np.testing.assert_array_equal(x[n_i, c_i, hh, ww], yh)
    # every pixel of the 3x3 neighbourhood is <= the window maximum (interior windows)
    up = np.repeat(np.repeat(yh, 2, axis=2), 2, axis=3)          # y at [h//2, w//2]: that window covers (h, w)
    assert (x <= up).all()


def test_max_pool_module_autograd_and_errors():
    import pytortto_amd as tt
    from pytortto_amd import nn
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 3, 9, 9)).astype(np.float32)
    g = rng.standard_normal((2, 3, 5, 5)).astype(np.float32)
    leaf = tt.tensor(x, requires_grad=True)
    xt = leaf.cuda()
    pool = nn.MaxPool2d(3, stride=2, padding=1)
    y = pool(xt)
    y.backward(tt.tensor(g).cuda())
    y_ref, pos = oracle.max_pool2d(x, (3, 3), (2, 2), (1, 1))
    np.testing.assert_array_equal(y.data.get(), y_ref)
    np.testing.assert_array_equal(leaf.grad, oracle.max_pool2d_backward(x.shape, g, pos, (3, 3), (2, 2), (1, 1)))
    # default stride = kernel size; 3-D input; return_indices gives the reference's index tuple
    y3, got = nn.MaxPool2d(2, return_indices=True)(tt.tensor(x[0]).cuda())
    y3_ref, pos3 = oracle.max_pool2d(x[0], (2, 2), (2, 2))
    np.testing.assert_array_equal(y3.data.get(), y3_ref)
    assert len(got) == 6 and got[0].shape == (1, 1, 1, 1)
    np.testing.assert_array_equal(got[4], pos3[0])
    np.testing.assert_array_equal(got[5], pos3[1])
    with pytest.raises(RuntimeError, match='pad should be smaller than or equal to half of kernel size'):
        nn.MaxPool2d(2, padding=2)(xt)
    with pytest.raises(RuntimeError, match='3D or 4D'):
        nn.MaxPool2d(2)(tt.tensor(x[0, 0]).cuda())


@pytest.mark.parametrize('inplace', [False, True])
def test_leaky_relu_module(inplace):
    import pytortto_amd as tt
    from pytortto_amd import nn
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 5, 7, 6)).astype(np.float32)     # 630 elements: exercises the scalar tail
    x.flat[:4] = [0.0, -0.0, np.nan, -3.0]
    g = rng.standard_normal(x.shape).astype(np.float32)
    leaf = tt.tensor(x, requires_grad=True)
    act = nn.LeakyReLU(0.2, inplace=inplace)
    y = act(leaf.cuda())                                          # a non-leaf input, so in-place is allowed
    gd = tt.tensor(g).cuda()
    y.backward(gd)
    np.testing.assert_array_equal(y.data.get(), oracle.leaky_relu_forward(x, 0.2))
    # in-place mode saves the overwritten tensor, as the reference does (grad_nn.py:81-86)
    saved = oracle.leaky_relu_forward(x, 0.2) if inplace else x
    want = oracle.leaky_relu_backward(g, saved, 0.2)
    np.testing.assert_array_equal(leaf.grad, want)
    np.testing.assert_array_equal(gd.data.get(), g)               # backward() seeds with a copy (tensor.py:583)
    # the node scales the gradient array it receives in place, as the reference does (:94)
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    buf = hiparray(g)
    assert ops.leaky_relu_bwd(buf, hiparray(saved), 0.2, out=buf) is buf
    np.testing.assert_array_equal(buf.get(), want)


def test_relu_keeps_nan():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x = np.array([np.nan, -1.0, 0.0, 2.0, -0.0], np.float32)
    y = ops.relu_fwd(hiparray(x)).get()
    np.testing.assert_array_equal(y, oracle.relu_forward(x))


@pytest.mark.parametrize('case', random_pool_cases(60, 77), ids=lambda c: '%dx%d_k%d%d_s%d%d_p%d%d_d%d%d_%s' % (
    c[2], c[3], *c[4], *c[5], *c[6], *c[7], 'ceil' if c[8] else 'floor'))
def test_max_pool_random_geometries(case):
    _run_pool(case, seed=14, ties=True)
