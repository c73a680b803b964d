"""GPU: tensors of 2^31 elements and more (8.8 GB each) through the C ABI.

The reference has no size limit (``grad_nn.py:595-611``); the kernels index with 32-bit element
offsets, so the library cuts such a batch into runs of images (forward, input gradient: separate
calls; weight gradient: separate partial sums added by the one reduce) and BatchNorm / elementwise
kernels use 64-bit offsets.  The tensors here are zero except for a few images -- the first ones,
the last ones of the first run, the first of the second run and the very last -- which hold random
values: convolution is per image, so those images of y and dx must equal the oracle's on the same
images alone, dw equals the oracle's on the batch of those images, and the BatchNorm statistics
have closed forms over "these values plus zeros".
"""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

N, C, H, W, K = 2100, 64, 128, 128, 16          # x: 2100 * 64 * 128 * 128 = 2.2e9 elements
IMAGES = [0, 1, 2046, 2047, 2099]              # images per run: 2047, so 2047 opens the second run


def _sparse(shape, rng):
    """Device array of zeros with random values in IMAGES; returns (array, {image: host values}).
    The first value of every channel stays zero: the BatchNorm kernels take their moments about
    x[0, c, 0, 0], which is a typical value of the channel in any real input -- and here, where
    all but five images are zero, has to be one too."""
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    arr = hiparray.zeros(shape)
    per = int(np.prod(shape[1:]))
    host = {}
    for n in IMAGES:
        host[n] = rng.standard_normal(shape[1:]).astype(np.float32)
        host[n][:, 0, 0] = 0
        _hip.call('tt_memcpy_h2d', arr.ptr + 4 * per * n, host[n].ctypes.data, 4 * per)
    return arr, host


def _image(arr, n):
    from pytortto_amd import _hip
    per = int(np.prod(arr.shape[1:]))
    out = np.empty(arr.shape[1:], np.float32)
    _hip.call('tt_memcpy_d2h', out.ctypes.data, arr.ptr + 4 * per * n, 4 * per)
    return out


def test_convolution_over_a_batch_of_more_than_2_to_31_elements():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    assert N * C * H * W > 2 ** 31
    rng = np.random.default_rng(0)
    x, xh = _sparse((N, C, H, W), rng)
    w = (rng.standard_normal((K, C, 3, 3)) / 24).astype(np.float32)
    geo = ((1, 1), (1, 1), (1, 1), 1)
    wd = hiparray(w)
    y = ops.conv2d_fwd(x, wd, None, *geo)
    assert y.shape == (N, K, H, W)
    xs = np.stack([xh[n] for n in IMAGES])
    y_ref, xpad = oracle.convolution_forward(xs, w, None, *geo)
    for i, n in enumerate(IMAGES):
        np.testing.assert_allclose(_image(y, n), y_ref[i], rtol=1e-4, atol=1e-5, err_msg=f'y[{n}]')
    assert not _image(y, 1000).any() and not _image(y, 2098).any()
    del y

    dy, dyh = _sparse((N, K, H, W), rng)
    dys = np.stack([dyh[n] for n in IMAGES])
    dx_ref, dw_ref, _ = oracle.convolution_backward(dys, xs, xpad, w, *geo, need=(True, True, False))
    dw = ops.conv2d_wgrad(x, dy, w.shape, *geo).get()
    np.testing.assert_allclose(dw, dw_ref, rtol=1e-4, atol=1e-5 * float(np.abs(dw_ref).max()), err_msg='dw')
    del x
    dx = ops.conv2d_dgrad(dy, wd, None, (H, W), *geo)
    for i, n in enumerate(IMAGES):
        np.testing.assert_allclose(_image(dx, n), dx_ref[i], rtol=1e-4, atol=1e-5, err_msg=f'dx[{n}]')
    assert not _image(dx, 2046 - 1).any()


def test_batchnorm_and_relu_over_more_than_2_to_31_elements():
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(1)
    x, xh = _sparse((N, C, H, W), rng)
    gamma = rng.uniform(0.5, 1.5, C).astype(np.float32)
    beta = (0.1 * rng.standard_normal(C)).astype(np.float32)
    m = N * H * W
    xs = np.stack([xh[n] for n in IMAGES]).astype(np.float64)
    mean = xs.sum((0, 2, 3)) / m                                     # the other images are zero
    var = (xs ** 2).sum((0, 2, 3)) / m - mean ** 2
    sd = np.sqrt(var + 1e-5)
    gd = hiparray(gamma)
    y, mu_d, var_d, sd_d, rm, rv = ops.bn_fwd_train(x, gd, hiparray(beta), hiparray(np.zeros(C, np.float32)),
                                                    hiparray(np.ones(C, np.float32)), 0.1, 1e-5)
    np.testing.assert_allclose(mu_d.get(), mean, rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(var_d.get(), var + 1e-5, rtol=1e-5)
    np.testing.assert_allclose(rv.get(), 0.9 + 0.1 * var * (m / (m - 1)), rtol=1e-5)
    col = lambda v: v[:, None, None]
    for n in IMAGES + [1234]:
        xn = xh.get(n, np.zeros((C, H, W), np.float32)).astype(np.float64)
        np.testing.assert_allclose(_image(y, n), (xn - col(mean)) / col(sd) * col(gamma) + col(beta), rtol=1e-5, atol=1e-5,
                                   err_msg=f'y[{n}]')
    # ReLU over the same 2.2e9 elements, in place of y: head, tail and a zero image
    r = ops.relu_fwd(y)
    for n in (0, 1234, 2099):
        np.testing.assert_array_equal(_image(r, n), np.maximum(_image(y, n), 0))
    del r, y

    dy, dyh = _sparse((N, C, H, W), rng)
    dys = np.stack([dyh[n] for n in IMAGES]).astype(np.float64)
    xhat = (xs - mean[None, :, None, None]) / sd[None, :, None, None]
    s_dy = dys.sum((0, 2, 3))
    s_dyxhat = (dys * xhat).sum((0, 2, 3))
    dx, dg, db = ops.bn_bwd(x, dy, gd, mu_d, var_d, sd_d)
    np.testing.assert_allclose(db.get(), s_dy, rtol=1e-5, atol=1e-5 * np.abs(s_dy).max())
    np.testing.assert_allclose(dg.get(), s_dyxhat, rtol=1e-5, atol=1e-5 * np.abs(s_dyxhat).max())
    for i, n in enumerate(IMAGES):
        want = col(gamma / sd) * (dys[i] - col(s_dy) / m - xhat[i] * col(s_dyxhat) / m)
        np.testing.assert_allclose(_image(dx, n), want, rtol=1e-4, atol=1e-5, err_msg=f'dx[{n}]')
    _hip.call('tt_empty_cache')
