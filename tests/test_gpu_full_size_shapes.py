"""The convolution shapes of the baseline configurations at their full sizes: the 23 unique
ResNet-50 shapes of the benchmark (batch 64, 3x224x224 input), the 11 unique shapes of the
PreAct-ResNet-18 stack (batch 128, 3x32x32) and the five ConvTranspose2d layers of the DCGAN
generator (batch 128).

At full size the oracle is too slow for whole tensors, so the kernels are checked at the
benchmark's own shapes through properties that do not depend on the size:

* convolution acts on every image separately: selected images of y and dx computed at full batch
  must equal the oracle's result for those images alone.  The images: the first two, the middle
  one, the last two (the last, ragged tile), and -- read from the library's launch plan -- the
  images in which the first and the last of the tiles begin whose reduction is shared between
  blocks (the stream-K segments and their finishing blocks);
* the weight gradient is linear in dy: with dy zero outside those images, dw at full batch must
  equal the oracle's dw for those images alone;
* adjointness: <conv(x, u), g> = <u, wgrad(x, g)> for random weight-shaped probes u, and
  <conv(x, w), g> = <x, dgrad(g, w)> (float64 inner products on the host).

At batch 2 every shape is compared with the oracle directly.
Tolerances: y and dx allclose(rtol=1e-4, atol=1e-5), the bar the convolution is specified to; any
element outside it must be a near-zero entry (|ref| below 5 % of the tensor's magnitude, where two
correct float32 sums differ by more than a relative bound can hold), within 1e-5 of the
magnitude, and such elements must stay below one in 10^5 -- their share is printed.  dw (sums
over N*P*Q products) keeps atol = 1e-5 * max|ref|, as in test_gpu_conv.py.  Inner products 2e-4
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


def _tensors(spec, batch, seed):
    c, h, k, r, s, p, _ = spec
    rng = np.random.default_rng(seed)
    q = (h + 2 * p - r) // s + 1
    x = rng.standard_normal((batch, c, h, h), dtype=np.float32)
    w = (rng.standard_normal((k, c, r, r), dtype=np.float32) / np.float32(np.sqrt(c * r * r))).astype(np.float32)
    g = rng.standard_normal((batch, k, q, q), dtype=np.float32)
    return x, w, g, ((s, s), (p, p), (1, 1), 1)


def _close(got, ref, name):
    """The stated bar; returns the share of elements that needed the near-zero exception."""
    scale = float(np.abs(ref).max()) or 1.0
    outside = np.abs(got - ref) > 1e-5 + 1e-4 * np.abs(ref)
    share = float(outside.mean()) if outside.size else 0.0
    if outside.any():
        assert float(np.abs(ref[outside]).max()) <= 0.05 * scale, f'{name}: outside rtol 1e-4 / atol 1e-5 away from zero'
        np.testing.assert_allclose(got[outside], ref[outside], rtol=1e-4, atol=1e-5 * max(1.0, scale), err_msg=name)
        assert share <= 1e-5, f'{name}: {share:.2e} of the elements are outside rtol 1e-4 / atol 1e-5'
        print(f'{name}: {int(outside.sum())} of {outside.size} near-zero elements outside atol 1e-5 (share {share:.1e})')
    return share


def _close_reduction(got, ref, name):
    scale = float(np.abs(ref).max()) or 1.0
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5 * max(1.0, scale), err_msg=name)


def _images(batch, pixels_per_image):
    """Images to compare element-wise after a forward / input-gradient call: head, middle, tail, and
    where the tiles with a shared reduction begin and end (from the plan of the launch just made)."""
    import ctypes
    from pytortto_amd import _hip
    plan = (ctypes.c_int * 8)()
    _hip.call('tt_conv2d_last_launch', plan)
    bm, bn, tiles, tiles_i, sk_blocks, whole, sharing, mode = plan
    chosen = {0, 1, batch // 2, batch - 2, batch - 1}
    if sk_blocks > 0 and whole < tiles:
        chosen.add(min(batch - 1, (whole // tiles_i) * bn // pixels_per_image))
        chosen.add(min(batch - 1, ((tiles - 1) // tiles_i) * bn // pixels_per_image))
    return sorted(i for i in chosen if 0 <= i < batch), sk_blocks > 0 and whole < tiles


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
    _close_reduction(ops.conv2d_wgrad(xd, gd, w.shape, *geo).get(), dw_ref, 'dw')


FULL_SIZE = [(s, FULL_BATCH) for s in RESNET50_CONVS] + [(s, 128) for s in PREACT18_CONVS]


@pytest.mark.parametrize('spec,batch', FULL_SIZE, ids=lambda v: 'C%d_H%d_K%d_k%d_s%d' % v[:5] if isinstance(v, tuple) else 'N%d' % v)
def test_shape_at_full_batch_properties(spec, batch):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x, w, g, geo = _tensors(spec, batch, 1)
    xd, wd, gd = hiparray(x), hiparray(w), hiparray(g)
    y = ops.conv2d_fwd(xd, wd, None, *geo).get()
    pick_y, shared_y = _images(batch, y.shape[-1] * y.shape[-2])
    dx = ops.conv2d_dgrad(gd, wd, None, x.shape[-2:], *geo).get()
    pick_dx, shared_dx = _images(batch, x.shape[-1] * x.shape[-2]) if geo[0] == (1, 1) else (pick_y, False)
    dw = ops.conv2d_wgrad(xd, gd, w.shape, *geo).get()
    pick = sorted(set(pick_y) | set(pick_dx))
    print(f'images compared: {pick} (shared reductions: forward {shared_y}, input gradient {shared_dx})')

    # every image separately: the selected images against the oracle on those images alone
    y_ref, xpad = oracle.convolution_forward(x[pick], w, None, *geo)
    dx_ref, dw_pick_ref, _ = oracle.convolution_backward(g[pick], x[pick], xpad, w, *geo)
    _close(y[pick], y_ref, f'y{pick}')
    _close(dx[pick], dx_ref, f'dx{pick}')

    # linear in dy: only the selected images carry a gradient
    g_pick = np.zeros_like(g)
    g_pick[pick] = g[pick]
    dw_pick = ops.conv2d_wgrad(xd, hiparray(g_pick), w.shape, *geo).get()
    _close_reduction(dw_pick, dw_pick_ref, 'dw from the selected images')

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
    ho = (h - 1) * st - 2 * pd + (r - 1) + 1
    g = rng.standard_normal((128, co, ho, ho), dtype=np.float32)
    xd, wd, gd = hiparray(x), hiparray(w), hiparray(g)
    y = ops.conv2d_dgrad(xd, wd, None, (ho, ho), *geo).get()
    dx = ops.conv2d_fwd(gd, wd, None, *geo).get()
    pick, shared = _images(128, h * h)
    dw = ops.conv2d_wgrad(gd, xd, w.shape, *geo).get()
    print(f'images compared: {pick} (shared reductions in the input gradient: {shared})')
    y_ref = oracle.transposed_convolution_forward(x[pick], w, None, geo[0], geo[1], (0, 0), (1, 1), 1)
    assert y_ref.shape[-1] == ho
    dx_ref, dw_pick_ref, _ = oracle.transposed_convolution_backward(g[pick], x[pick], w, geo[0], geo[1], (1, 1), 1)
    _close(y[pick], y_ref, f'y{pick}')
    _close(dx[pick], dx_ref, f'dx{pick}')
    x_pick = np.zeros_like(x)
    x_pick[pick] = x[pick]
    _close_reduction(ops.conv2d_wgrad(gd, hiparray(x_pick), w.shape, *geo).get(), dw_pick_ref, 'dw from the selected images')
    yg = _dot(y, g)
    scale = np.sqrt(_dot(y, y) * _dot(g, g))
    assert abs(yg - _dot(x, dx)) <= 2e-4 * scale, ('<y,g> vs <x,dx>', yg, _dot(x, dx))
    assert abs(yg - _dot(w, dw)) <= 2e-4 * scale, ('<y,g> vs <w,dw>', yg, _dot(w, dw))
