"""The convolution shapes of the baseline configurations at their full sizes: the 23 unique
ResNet-50 shapes of the benchmark (batch 64, 3x224x224 input), the 11 unique shapes of the
PreAct-ResNet-18 stack (batch 128, 3x32x32) and the five ConvTranspose2d layers of the DCGAN
generator (batch 128).

At full size the oracle is too slow, so the kernels are checked at the benchmark's own shapes
through properties that do not depend on the size:

* convolution acts on every image separately: the first images of y and dx computed at batch 64
  must equal the oracle's result for those images alone;
* the weight gradient is linear in dy: with dy zero outside the first images, dw at batch 64
  must equal the oracle's dw for those images alone;
* adjointness: <conv(x, u), g> = <u, wgrad(x, g)> for random weight-shaped probes u, and
  <conv(x, w), g> = <x, dgrad(g, w)> (float64 inner products on the host).

At batch 2 every shape is compared with the oracle directly.
Tolerances: the convolution bar, allclose(rtol=1e-4, atol=1e-5 * max|ref|); inner products 2e-4
relative to the product of the norms' scale.
"""
import numpy as np
import pytest

import oracle
from bench import RESNET50_CONVS

pytestmark = pytest.mark.gpu

FULL_BATCH = 64
# PreAct-ResNet-18 on 32x32 inputs: (C, H, K, kernel, stride, padding, count) as in bench.RESNET50_CONVS
PREACT18_CONVS = [(3, 32, 64, 3, 1, 1, 1), (64, 32, 64, 3, 1, 1, 4), (64, 32, 128, 3, 2, 1, 1), (128, 16, 128, 3, 1, 1, 3),
                  (64, 32, 128, 1, 2, 0, 1), (128, 16, 256, 3, 2, 1, 1), (256, 8, 256, 3, 1, 1, 3), (128, 16, 256, 1, 2, 0, 1),
                  (256, 8, 512, 3, 2, 1, 1), (512, 4, 512, 3, 1, 1, 3), (256, 8, 512, 1, 2, 0, 1)]
# DCGAN generator: (C_in, H_in, C_out, kernel, stride, padding)
DCGAN_CONVTS = [(100, 1, 512, 4, 1, 0), (512, 4, 256, 4, 2, 1), (256, 8, 128, 4, 2, 1), (128, 16, 64, 4, 2, 1),
                (64, 32, 3, 4, 2, 1)]
HEAD = 2        # images checked against the oracle


def _tensors(spec, batch, seed):
    c, h, k, r, s, p, _ = spec
    rng = np.random.default_rng(seed)
    q = (h + 2 * p - r) // s + 1
    x = rng.standard_normal((batch, c, h, h), dtype=np.float32)
    w = (rng.standard_normal((k, c, r, r), dtype=np.float32) / np.float32(np.sqrt(c * r * r))).astype(np.float32)
    g = rng.standard_normal((batch, k, q, q), dtype=np.float32)
    return x, w, g, ((s, s), (p, p), (1, 1), 1)


def _close(got, ref, name):
    scale = float(np.abs(ref).max()) or 1.0
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5 * max(1.0, scale), err_msg=name)


def _dot(a, b):
    return float(np.dot(a.ravel().astype(np.float64), b.ravel().astype(np.float64)))


@pytest.mark.parametrize('spec', RESNET50_CONVS, ids=lambda s: 'C%d_H%d_K%d_k%d_s%d' % s[:5])
def test_shape_at_batch_2_matches_oracle(spec):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x, w, g, geo = _tensors(spec, 2, 0)
    y_ref, xpad = oracle.convolution_forward(x, w, None, *geo)
    dx_ref, dw_ref, _ = oracle.convolution_backward(g, x, xpad, w, *geo)
    xd, wd, gd = hiparray(x), hiparray(w), hiparray(g)
    _close(ops.conv2d_fwd(xd, wd, None, *geo).get(), y_ref, 'y')
    _close(ops.conv2d_dgrad(gd, wd, None, x.shape[-2:], *geo).get(), dx_ref, 'dx')
    _close(ops.conv2d_wgrad(xd, gd, w.shape, *geo).get(), dw_ref, 'dw')


FULL_SIZE = [(s, FULL_BATCH) for s in RESNET50_CONVS] + [(s, 128) for s in PREACT18_CONVS]


@pytest.mark.parametrize('spec,batch', FULL_SIZE, ids=lambda v: 'C%d_H%d_K%d_k%d_s%d' % v[:5] if isinstance(v, tuple) else 'N%d' % v)
def test_shape_at_full_batch_properties(spec, batch):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x, w, g, geo = _tensors(spec, batch, 1)
    xd, wd, gd = hiparray(x), hiparray(w), hiparray(g)
    y = ops.conv2d_fwd(xd, wd, None, *geo).get()
    dx = ops.conv2d_dgrad(gd, wd, None, x.shape[-2:], *geo).get()
    dw = ops.conv2d_wgrad(xd, gd, w.shape, *geo).get()

    # every image separately: the first images against the oracle
    y_ref, xpad = oracle.convolution_forward(x[:HEAD], w, None, *geo)
    dx_ref, dw_head_ref, _ = oracle.convolution_backward(g[:HEAD], x[:HEAD], xpad, w, *geo)
    _close(y[:HEAD], y_ref, 'y[:2]')
    _close(dx[:HEAD], dx_ref, 'dx[:2]')

    # linear in dy: only the first images carry a gradient
    g_head = np.zeros_like(g)
    g_head[:HEAD] = g[:HEAD]
    dw_head = ops.conv2d_wgrad(xd, hiparray(g_head), w.shape, *geo).get()
    _close(dw_head, dw_head_ref, 'dw from the first images')

    # adjointness at full size
    yg = _dot(y, g)
    scale = np.sqrt(_dot(y, y) * _dot(g, g))
    assert abs(yg - _dot(x, dx)) <= 2e-4 * scale, ('<y,g> vs <x,dx>', yg, _dot(x, dx))
    assert abs(yg - _dot(w, dw)) <= 2e-4 * scale, ('<y,g> vs <w,dw>', yg, _dot(w, dw))
    rng = np.random.default_rng(2)
    for _ in range(2):
        u = rng.standard_normal(w.shape, dtype=np.float32) / np.float32(np.sqrt(w[0].size))
        yu = ops.conv2d_fwd(xd, hiparray(u), None, *geo).get()
        lhs, rhs = _dot(yu, g), _dot(u, dw)
        assert abs(lhs - rhs) <= 2e-4 * np.sqrt(_dot(yu, yu) * _dot(g, g)), ('<conv(x,u),g> vs <u,dw>', lhs, rhs)


@pytest.mark.parametrize('spec', DCGAN_CONVTS, ids=lambda s: 'Cin%d_H%d_Cout%d' % s[:3])
def test_dcgan_conv_transpose_layers_at_batch_128(spec):
    """ConvTranspose2d forward runs on the input-gradient kernel, its input gradient on the forward
    kernel, its weight gradient on the weight-gradient kernel with the roles of x and dy swapped:
    per-image parity with the oracle on the first images, linearity of dw, adjointness."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    ci, h, co, r, st, pd = spec
    geo = ((st, st), (pd, pd), (1, 1), 1)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((128, ci, h, h), dtype=np.float32)
    w = (rng.standard_normal((ci, co, r, r), dtype=np.float32) / np.float32(np.sqrt(ci * r * r))).astype(np.float32)
    y_ref = oracle.transposed_convolution_forward(x[:HEAD], w, None, geo[0], geo[1], (0, 0), (1, 1), 1)
    ho = y_ref.shape[-1]
    g = rng.standard_normal((128, co, ho, ho), dtype=np.float32)
    xd, wd, gd = hiparray(x), hiparray(w), hiparray(g)
    y = ops.conv2d_dgrad(xd, wd, None, (ho, ho), *geo).get()
    dx = ops.conv2d_fwd(gd, wd, None, *geo).get()
    dw = ops.conv2d_wgrad(gd, xd, w.shape, *geo).get()
    dx_ref, dw_head_ref, _ = oracle.transposed_convolution_backward(g[:HEAD], x[:HEAD], w, geo[0], geo[1], (1, 1), 1)
    _close(y[:HEAD], y_ref, 'y[:2]')
    _close(dx[:HEAD], dx_ref, 'dx[:2]')
    x_head = np.zeros_like(x)
    x_head[:HEAD] = x[:HEAD]
    _close(ops.conv2d_wgrad(gd, hiparray(x_head), w.shape, *geo).get(), dw_head_ref, 'dw from the first images')
    yg = _dot(y, g)
    scale = np.sqrt(_dot(y, y) * _dot(g, g))
    assert abs(yg - _dot(x, dx)) <= 2e-4 * scale, ('<y,g> vs <x,dx>', yg, _dot(x, dx))
    assert abs(yg - _dot(w, dw)) <= 2e-4 * scale, ('<y,g> vs <w,dw>', yg, _dot(w, dw))
