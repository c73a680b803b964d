"""GPU parity: Conv2d / ConvTranspose2d forward, dgrad, wgrad through the C ABI vs the CPU oracle.

Tolerance (fp32): allclose(rtol=1e-4, atol=1e-5) against the oracle for forward/dgrad.  For
weight/bias gradients -- reductions over N*P*Q terms -- two correct float32 evaluations differ
on near-zero entries by more than an element-wise rtol allows (the reference's own notebook
check used rtol=1e-3 for them), so those use atol scaled by the tensor's magnitude, and every
tensor is additionally required to be as close to a float64 evaluation as the oracle itself.
"""
import numpy as np
import pytest

import oracle
from tests.cases import CONV_CASES, CONVT_CASES, random_conv_cases, random_convt_cases, random_large_kernel_cases

pytestmark = pytest.mark.gpu


def _check(name, got, ref32, ref64, reduction=False):
    scale = float(np.abs(ref64).max()) or 1.0
    err_gpu = float(np.abs(got - ref64).max()) / scale
    err_cpu = float(np.abs(ref32 - ref64).max()) / scale
    assert err_gpu <= max(3 * err_cpu, 5e-6), f'{name}: gpu err {err_gpu:.3g} vs oracle err {err_cpu:.3g}'
    atol = 1e-5 * max(1.0, scale) if reduction else 1e-5
    np.testing.assert_allclose(got, ref32, rtol=1e-4, atol=atol, err_msg=name)


def _run_conv(case, seed=0, bias=True):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
    w = (rng.standard_normal((k, c // g, r, s)) / np.sqrt(c // g * r * s)).astype(np.float32)
    b = rng.standard_normal(k).astype(np.float32) if bias else None
    y32, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, g)
    gy = rng.standard_normal(y32.shape).astype(np.float32)
    dx32, dw32, db32 = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
    x64, w64, gy64 = x.astype(np.float64), w.astype(np.float64), gy.astype(np.float64)
    y64, xpad64 = oracle.convolution_forward(x64, w64, None if b is None else b.astype(np.float64), st, pd, dl, g)
    dx64, dw64, db64 = oracle.convolution_backward(gy64, x64, xpad64, w64, st, pd, dl, g)

    xd, wd, gyd = hiparray(x), hiparray(w), hiparray(gy)
    bd = None if b is None else hiparray(b)
    y = ops.conv2d_fwd(xd, wd, bd, st, pd, dl, g)
    assert y.shape == y32.shape
    dx = ops.conv2d_dgrad(gyd, wd, None, (h, w_), st, pd, dl, g)
    dw = ops.conv2d_wgrad(xd, gyd, w.shape, st, pd, dl, g)
    db = ops.channel_sum(gyd)
    _check('y', y.get(), y32, y64)
    _check('dx', dx.get(), dx32, dx64)
    _check('dw', dw.get(), dw32, dw64, reduction=True)
    _check('db', db.get(), db32, db64, reduction=True)


@pytest.mark.parametrize('case', CONV_CASES)
def test_conv_small_geometries(case):
    _run_conv(case)


# shapes that exercise every tile configuration, ragged tiles, split reductions and groups
TILE_CASES = [
    (32, 16, 32, 32, 32, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # the CPU-runnable baseline config
    (4, 64, 28, 28, 64, 1, 1, (1, 1), (0, 0), (1, 1), 1),       # 64-row tile x 256 pixels
    (4, 64, 28, 28, 256, 1, 1, (1, 1), (0, 0), (1, 1), 1),      # 128x128 tiles
    (3, 96, 15, 15, 200, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # ragged rows (200) and pixels (675)
    (4, 128, 28, 28, 128, 3, 3, (2, 2), (1, 1), (1, 1), 1),     # stride 2: four parity classes in dgrad
    (4, 256, 14, 14, 512, 1, 1, (2, 2), (0, 0), (1, 1), 1),     # strided 1x1 shortcut
    (8, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3), (1, 1), 1),        # stem: C=3, Kred=147 (not a multiple of 4)
    (2, 512, 7, 7, 512, 3, 3, (1, 1), (1, 1), (1, 1), 1),       # small M, long reduction
    (4, 64, 20, 20, 96, 3, 3, (1, 1), (2, 2), (2, 2), 4),       # groups + dilation
    (128, 4, 64, 64, 16, 3, 2, (1, 3), (2, 3), (1, 2), 2),      # the reference notebook's configuration
    (8, 128, 28, 28, 128, 3, 3, (1, 1), (1, 1), (1, 1), 1),     # 49 tiles of 128x128: split reduction (stream-K)
    (16, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # 196 tiles of 64x256: stream-K
    (8, 256, 14, 14, 256, 3, 3, (2, 2), (1, 1), (1, 1), 1),     # stream-K in every dgrad parity class
    (2, 40, 8, 8, 72, 1, 1, (1, 1), (0, 0), (1, 1), 1),         # plain-GEMM path, 64x64 tiles, C not a multiple of 16
    (16, 256, 14, 14, 1024, 1, 1, (1, 1), (0, 0), (1, 1), 1),   # plain-GEMM path with split left-over tiles
    (3, 64, 6, 6, 64, 1, 1, (1, 1), (0, 0), (1, 1), 2),         # plain-GEMM path with groups, ragged pixel tile
    (70, 16, 3, 3, 32, 3, 3, (1, 1), (1, 1), (1, 1), 1),        # tiny images: a pixel tile spans 15-29 images (buffer re-basing)
    (5, 32, 13, 9, 48, 5, 5, (2, 1), (4, 2), (2, 1), 2),        # 25 taps, dilation + stride + groups: tap masks, negative table steps in dgrad
    (3, 16, 14, 14, 16, 6, 6, (1, 1), (2, 2), (1, 1), 1),       # 36 taps > 31: 64-bit tap masks in forward and weight gradient, compare-and-select in the input gradient
    (2, 8, 20, 18, 24, 7, 9, (1, 1), (3, 4), (1, 1), 1),        # 63 taps: the most a 64-bit tap mask holds (its top bit is the padding tap)
    (4, 6, 23, 25, 40, 7, 7, (2, 2), (3, 3), (1, 1), 2),        # 49 taps with groups, stride 2 and an odd image
    (2, 4, 30, 30, 16, 6, 7, (1, 2), (5, 6), (2, 2), 1),        # 42 taps with dilation 2 and padding wider than the kernel's reach on one side
    (3, 16, 14, 14, 16, 9, 9, (1, 1), (4, 4), (1, 1), 1),       # 81 taps > 63: compare-and-select addressing in all three passes
    (2, 2, 20, 22, 4, 13, 11, (2, 2), (6, 5), (1, 1), 1),       # few channels, stride 2, 13x11 kernel: the dense input gradient's union window has 7x6 = 42 taps (64-bit masks there too)
    (2, 32, 12, 12, 64, 1, 1, (1, 1), (1, 1), (1, 1), 1),       # padded 1x1: not the plain-GEMM geometry, one-tap mask
    (4, 48, 10, 10, 24, 3, 3, (1, 1), (0, 0), (1, 1), 1),       # unpadded 3x3, rows (24) and weight rows shorter than a tile
    (6, 20, 9, 9, 36, 3, 3, (1, 1), (1, 1), (1, 1), 1),         # C*R*S = 180: weight rows not a whole number of 16-wide chunks (repacked copy)
    (8, 64, 18, 20, 32, 1, 1, (3, 2), (0, 0), (1, 1), 1),       # strided 1x1, whole cells: the input gradient stores value + zeros of a 3x2 cell itself
    (4, 64, 16, 12, 64, 1, 1, (4, 2), (0, 0), (1, 1), 1),       # the same with cells four rows high (the tallest the whole-cell stores take)
    (8, 256, 28, 28, 512, 1, 1, (2, 2), (0, 0), (1, 1), 1),     # whole cells with the reduction of every tile split between blocks: the second stage stores the cells
    (48, 128, 21, 28, 256, 1, 1, (3, 2), (0, 0), (1, 1), 1),    # split reduction and cells three rows high
    (4, 40, 15, 14, 24, 1, 1, (2, 2), (0, 0), (1, 1), 1),        # strided 1x1, last row of dx not covered by the forward: cleared beforehand instead
    (4, 32, 12, 12, 16, 1, 1, (2, 2), (0, 0), (1, 1), 2),        # strided 1x1 with groups
    # tiny C with stride > 1: the input gradient stacks the pixel classes of a cell of one or more stride periods as GEMM rows
    (3, 3, 45, 43, 16, 7, 7, (2, 2), (3, 3), (1, 1), 1),        # stem taps, odd image: cells two periods wide, ragged last cell and last column
    (2, 1, 21, 30, 8, 3, 3, (2, 2), (1, 1), (1, 1), 1),         # one channel: cells widened both ways
    (2, 2, 17, 19, 8, 4, 4, (2, 2), (1, 1), (1, 1), 1),         # 4x4 stride 2 (the transposed generator's taps), rows left uncovered by the forward
    (2, 3, 20, 22, 8, 5, 3, (3, 2), (2, 1), (1, 1), 1),         # stride 3 x 2: 18 classes x 3 channels stay in one period
    (2, 2, 19, 21, 8, 3, 3, (2, 2), (2, 2), (2, 2), 1),         # dilation shares a factor with the stride: classes without taps
    (2, 5, 16, 9, 8, 3, 5, (2, 2), (1, 2), (1, 1), 1),          # five channels, image narrower than a four-period cell
    (4, 3, 3, 40, 8, 3, 3, (2, 2), (1, 1), (1, 1), 1),          # image too low for a taller cell: two periods wide instead
    (4, 1, 3, 40, 8, 3, 3, (2, 2), (1, 1), (1, 1), 1),          # the same with one channel: four periods wide
]


def test_tile_case_list_is_complete():
    """A case that slips into the comment of the line above it would silently drop out."""
    assert len(TILE_CASES) == 41
    assert all(len(c) == 11 for c in TILE_CASES)
    strided_1x1 = [c for c in TILE_CASES if c[5:7] == (1, 1) and c[7] != (1, 1) and c[10] == 1]
    assert {c[7][0] for c in strided_1x1} == {2, 3, 4}      # cells two, three and four rows high


@pytest.mark.parametrize('case', TILE_CASES)
def test_conv_tile_configurations(case):
    _run_conv(case, seed=1)


@pytest.mark.parametrize('case', [c for c in TILE_CASES if c[1] <= 5 and c[7] != (1, 1)])
def test_conv_dense_input_gradient_with_larger_cells(case):
    """Strided layers with very few input channels: without the tile-count threshold these small
    inputs take the larger cells (several stride periods per cell) of the dense input gradient;
    between them the cases take cells of 2x1, 1x2, 2x2, 1x4 and 2x4 periods."""
    from pytortto_amd import _hip
    _hip.call('tt_set_conv_dense_cell_min_tiles', 0)
    try:
        _run_conv(case, seed=3)
    finally:
        _hip.call('tt_set_conv_dense_cell_min_tiles', -1)        # back to the default


STREAM_K_CASES = [c for c in TILE_CASES if c[:3] in ((8, 128, 28), (16, 64, 56), (16, 256, 14))]


def _last_launch():
    import ctypes
    from pytortto_amd import _hip
    plan = (ctypes.c_int * 8)()
    _hip.call('tt_conv2d_last_launch', plan)
    return dict(zip(('bm', 'bn', 'tiles', 'tiles_i', 'persistent_blocks', 'whole_tiles', 'sharing_blocks', 'mode'), plan))


def test_persistent_grid_kernels_fit_the_device():
    """The blocks of a persistent launch wait for each other's partial sums; that is safe only while
    two blocks (three with bf16 arithmetic) of every such kernel are resident per compute unit."""
    import ctypes
    from pytortto_amd import _hip
    held = ctypes.c_int()
    _hip.call('tt_conv2d_stream_k_blocks_per_cu', 0, ctypes.byref(held))
    assert held.value >= 2, held.value
    _hip.call('tt_conv2d_stream_k_blocks_per_cu', 1, ctypes.byref(held))
    assert held.value >= 3, held.value
    _hip.call('tt_conv2d_stream_k_blocks_per_cu', 3, ctypes.byref(held))   # float32 arithmetic in three bf16 terms
    assert held.value >= 2, held.value


@pytest.mark.parametrize('case', STREAM_K_CASES)
def test_persistent_grid_falls_back_to_one_tile_per_block_when_it_would_not_fit(case):
    """With the device reporting (here: made to report) one resident block per compute unit, the
    launches that would share reductions between blocks run data-parallel, and still match."""
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    assert len(STREAM_K_CASES) == 3
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(9)
    x = hiparray(rng.standard_normal((n, c, h, w_)).astype(np.float32))
    w = hiparray((rng.standard_normal((k, c // g, r, s)) / np.sqrt(c // g * r * s)).astype(np.float32))
    y_shared = ops.conv2d_fwd(x, w, None, st, pd, dl, g).get()
    assert _last_launch()['persistent_blocks'] > 0 and _last_launch()['sharing_blocks'] > 0
    _hip.call('tt_conv2d_stream_k_force_occupancy', 1)
    try:
        y_plain = ops.conv2d_fwd(x, w, None, st, pd, dl, g).get()
        plan = _last_launch()
        assert plan['persistent_blocks'] == 0 and plan['whole_tiles'] == plan['tiles']
        _run_conv(case, seed=2)
    finally:
        _hip.call('tt_conv2d_stream_k_force_occupancy', -1)
    np.testing.assert_allclose(y_plain, y_shared, rtol=1e-5, atol=1e-5)     # summation order of the shared tiles only


def test_a_wait_that_ran_out_is_reported_by_the_next_synchronisation():
    """Host side of the failure path: the word a block sets when its bounded wait runs out (set here by
    a one-thread kernel; nothing waits) makes the next tt_sync / device-to-host copy fail with the
    documented message, once; afterwards the library works as before."""
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    _hip.synchronize()
    _hip.call('tt_conv2d_selftest_raise_async_error')
    with pytest.raises(RuntimeError, match='timed out waiting for another block'):
        _hip.synchronize()
    _hip.synchronize()                                  # reported once, then clear
    a = hiparray(np.arange(8, dtype=np.float32))
    _hip.call('tt_conv2d_selftest_raise_async_error')
    with pytest.raises(RuntimeError, match='results since the last synchronisation are invalid'):
        a.get()
    np.testing.assert_array_equal(a.get(), np.arange(8, dtype=np.float32))
    _run_conv(STREAM_K_CASES[0], seed=4)


# Images too large for 32-bit byte offsets relative to a tile's (a chunk's) first image: the
# kernels must fall back from buffer addressing to 64-bit addresses with compared bounds.
LARGE_IMAGE_CASES = [
    (2, 32, 720, 720, 8, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # 66 MB per image, a chunk may span 34 images: weight gradient falls back
    (2, 20, 3300, 3300, 4, 1, 1, (1, 1), (0, 0), (1, 1), 1),    # 871 MB per image: forward / input gradient fall back too
]


@pytest.mark.parametrize('case', LARGE_IMAGE_CASES)
def test_conv_large_images_use_64_bit_addressing(case):
    _run_conv(case, seed=3)


def test_conv_without_bias():
    _run_conv((2, 4, 8, 8, 6, 3, 3, (1, 1), (1, 1), (1, 1), 1), bias=False)


@pytest.mark.parametrize('case', TILE_CASES + random_conv_cases(24, 77))
def test_conv_tile_configurations_without_bias(case):
    """Without a bias the stores take the scalar-addressed path when the row count is a multiple of 8."""
    _run_conv(case, seed=5, bias=False)


CONVT_TILE_CASES = [
    (16, 100, 1, 1, 512, 4, 4, (1, 1), (0, 0), (0, 0), (1, 1), 1),   # DCGAN layer 1 (reduced batch)
    (8, 256, 8, 8, 128, 4, 4, (2, 2), (1, 1), (0, 0), (1, 1), 1),    # DCGAN upsampling layer
    (8, 64, 16, 16, 3, 4, 4, (2, 2), (1, 1), (0, 0), (1, 1), 1),     # DCGAN last layer: 3 output channels
    (130, 24, 1, 1, 40, 3, 5, (2, 3), (0, 0), (0, 0), (1, 1), 1),    # 1x1 input, rectangular kernel, stride irrelevant: one matrix product
    (4, 24, 1, 1, 40, 3, 3, (2, 2), (0, 0), (1, 1), (1, 1), 1),      # 1x1 input with output padding: not that case
]


@pytest.mark.parametrize('case', CONVT_CASES + CONVT_TILE_CASES + random_convt_cases(40, 99))
def test_conv_transpose_forward_backward(case):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    n, ci, h, w_, co, r, s, st, pd, op, dl, g = case
    rng = np.random.default_rng(2)
    x = rng.standard_normal((n, ci, h, w_)).astype(np.float32)
    w = (rng.standard_normal((ci, co // g, r, s)) / np.sqrt(ci // g * r * s)).astype(np.float32)
    b = rng.standard_normal(co).astype(np.float32)
    y32 = oracle.transposed_convolution_forward(x, w, b, st, pd, op, dl, g)
    gy = rng.standard_normal(y32.shape).astype(np.float32)
    dx32, dw32, db32 = oracle.transposed_convolution_backward(gy, x, w, st, pd, dl, g)
    x64, w64, gy64 = x.astype(np.float64), w.astype(np.float64), gy.astype(np.float64)
    y64 = oracle.transposed_convolution_forward(x64, w64, b.astype(np.float64), st, pd, op, dl, g)
    dx64, dw64, db64 = oracle.transposed_convolution_backward(gy64, x64, w64, st, pd, dl, g)

    xd, wd, gyd = hiparray(x), hiparray(w), hiparray(gy)
    # forward = input gradient of the convolution whose weight is w: "K" = C_in, "C" = C_out
    y = ops.conv2d_dgrad(xd, wd, hiparray(b), y32.shape[-2:], st, pd, dl, g)
    assert y.shape == y32.shape
    dx = ops.conv2d_fwd(gyd, wd, None, st, pd, dl, g)
    assert dx.shape == x.shape
    dw = ops.conv2d_wgrad(gyd, xd, w.shape, st, pd, dl, g)
    db = ops.channel_sum(gyd)
    _check('y', y.get(), y32, y64)
    # without a bias (a 1x1 input spread over the whole kernel then runs as one matrix product)
    y0 = ops.conv2d_dgrad(xd, wd, None, y32.shape[-2:], st, pd, dl, g)
    bb, bb64 = b.reshape(1, -1, 1, 1), b.astype(np.float64).reshape(1, -1, 1, 1)
    _check('y without bias', y0.get(), y32 - bb, y64 - bb64)
    _check('dx', dx.get(), dx32, dx64)
    _check('dw', dw.get(), dw32, dw64, reduction=True)
    _check('db', db.get(), db32, db64, reduction=True)


def test_conv_rejects_bad_arguments():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    x = hiparray(np.zeros((1, 4, 4, 4), np.float32))
    w = hiparray(np.zeros((4, 4, 3, 3), np.float32))
    with pytest.raises(RuntimeError):
        ops.conv2d_fwd(x, w, None, (1, 1), (0, 0), (1, 1), 3)      # channels not divisible by groups
    with pytest.raises(RuntimeError):
        ops.conv2d_fwd(x, w, None, (1, 1), (0, 0), (2, 2), 1)      # dilated kernel larger than the input


@pytest.mark.parametrize('case', random_conv_cases(60, 2024), ids=lambda c: 'n%d_c%d_%dx%d_k%d_%dx%d_s%s_p%s_d%s_g%d' % (
    c[0], c[1], c[2], c[3], c[4], c[5], c[6], '%d%d' % c[7], '%d%d' % c[8], '%d%d' % c[9], c[10]))
def test_conv_random_geometries(case):
    _run_conv(case, seed=5)


@pytest.mark.parametrize('case', random_large_kernel_cases(40, 99), ids=lambda c: 'n%d_c%d_%dx%d_k%d_%dx%d_s%s_p%s_d%s_g%d' % (
    c[0], c[1], c[2], c[3], c[4], c[5], c[6], '%d%d' % c[7], '%d%d' % c[8], '%d%d' % c[9], c[10]))
def test_conv_random_large_kernels(case):
    """Kernels of 26 to 81 taps with random stride, padding, dilation and groups: 32-bit tap masks,
    64-bit tap masks (32 to 63 taps) and per-element bounds (more than 63) in all three passes."""
    _run_conv(case, seed=6)


@pytest.mark.parametrize('case', [
    (16, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # stream-K forward and input gradient, split weight gradient
    (8, 256, 14, 14, 256, 3, 3, (2, 2), (1, 1), (1, 1), 1),     # parity classes in one grid
    (16, 256, 14, 14, 1024, 1, 1, (1, 1), (0, 0), (1, 1), 1),   # 64x64 tiles
])
def test_conv_is_bit_reproducible(case):
    """Split reductions are added in a fixed order: the same call gives the same bits every time."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(6)
    x = hiparray(rng.standard_normal((n, c, h, w_), dtype=np.float32))
    w = hiparray(rng.standard_normal((k, c // g, r, s), dtype=np.float32))
    p = (h + 2 * pd[0] - dl[0] * (r - 1) - 1) // st[0] + 1
    q = (w_ + 2 * pd[1] - dl[1] * (s - 1) - 1) // st[1] + 1
    gy = hiparray(rng.standard_normal((n, k, p, q), dtype=np.float32))

    def once():
        return (ops.conv2d_fwd(x, w, None, st, pd, dl, g).get(), ops.conv2d_dgrad(gy, w, None, (h, w_), st, pd, dl, g).get(),
                ops.conv2d_wgrad(x, gy, w.shape, st, pd, dl, g).get())

    first = once()
    ops.conv2d_fwd(hiparray(rng.standard_normal((4, 8, 9, 9), dtype=np.float32)),           # other work in between
                   hiparray(rng.standard_normal((8, 8, 3, 3), dtype=np.float32)), None, (1, 1), (1, 1), (1, 1), 1)
    for a, b in zip(first, once()):
        np.testing.assert_array_equal(a, b)


def test_stream_k_partial_sums_across_many_launches():
    """The partial sums of a split tile pass from block to block through memory, announced by a flag
    per block whose value changes from launch to launch.  Launches of different layers back to
    back -- each re-using the same partial slots and flag words -- must give the same bits every
    time, and the right ones: a partial read too early, or left over from the launch before, would
    show here."""
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    geo = ((1, 1), (1, 1), (1, 1), 1)
    rng = np.random.default_rng(21)
    layers = []
    for n, c, h, k in ((8, 128, 28, 128), (8, 256, 14, 256), (4, 512, 7, 512), (16, 64, 56, 64)):   # tiles: 49, 98 x ..., all split
        x = rng.standard_normal((n, c, h, h), dtype=np.float32)
        w = (rng.standard_normal((k, c, 3, 3)) / np.sqrt(9 * c)).astype(np.float32)
        y_ref, _ = oracle.convolution_forward(x, w, None, *geo)
        layers.append((hiparray(x), hiparray(w), y_ref))
    outs = [[] for _ in layers]
    for _ in range(12):
        for i, (x, w, _) in enumerate(layers):
            outs[i].append(ops.conv2d_fwd(x, w, None, *geo))        # enqueued back to back, read afterwards
    _hip.synchronize()
    for (x, w, y_ref), ys in zip(layers, outs):
        first = ys[0].get()
        np.testing.assert_allclose(first, y_ref, rtol=1e-4, atol=1e-5)
        for y in ys[1:]:
            np.testing.assert_array_equal(y.get(), first)


def _last_wgrad():
    import ctypes
    from pytortto_amd import _hip
    plan = (ctypes.c_int * 4)()
    _hip.call('tt_conv2d_last_wgrad_launch', plan)
    return dict(zip(('tiles', 'splits', 'added_in_kernel', 'slots'), plan))


# weight gradients whose partial sums are added inside the kernel (one round of resident blocks):
# ragged rows and columns, 1x1 / 3x3 / stem taps, groups, one tile with hundreds of splits, many tiles with few
WGRAD_FUSED_CASES = [
    (16, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1),       # 64x64 tiles, J = 576: nine tiles, 56 splits each
    (16, 64, 56, 56, 64, 1, 1, (1, 1), (0, 0), (1, 1), 1),       # one 64x64 tile, hundreds of splits: two float4s per block
    (8, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3), (1, 1), 1),         # stem: J = 147 in three 64-column tiles, 64-bit tap masks
    (24, 96, 15, 15, 200, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # ragged rows (200) and columns (864), 128x128 tiles
    (8, 256, 14, 14, 512, 1, 1, (1, 1), (0, 0), (1, 1), 1),      # 128x64 tiles, 16 tiles
    (4, 64, 20, 20, 96, 3, 3, (1, 1), (2, 2), (2, 2), 4),        # groups: tiles of every group share the grid
    (32, 256, 14, 14, 256, 3, 3, (1, 1), (1, 1), (1, 1), 1),     # 36 tiles of 128x128, 14 splits
    (6, 20, 9, 9, 36, 3, 3, (1, 1), (1, 1), (1, 1), 1),          # J = 180, rows 36: small ragged tiles
]


@pytest.mark.parametrize('case', WGRAD_FUSED_CASES)
def test_weight_gradient_with_partial_sums_added_in_the_kernel(case):
    """dw against the oracle and float64 with the in-kernel adding, the same bits on a second call, and
    the same values (to float64-sum rounding) from the separate reduce kernel, which the library takes
    when the device would not hold the whole grid (forced here)."""
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(21)
    x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
    p = (h + 2 * pd[0] - dl[0] * (r - 1) - 1) // st[0] + 1
    q = (w_ + 2 * pd[1] - dl[1] * (s - 1) - 1) // st[1] + 1
    gy = rng.standard_normal((n, k, p, q)).astype(np.float32)
    w_shape = (k, c // g, r, s)
    zero_w = np.zeros(w_shape, np.float32)
    _, xpad = oracle.convolution_forward(x, zero_w, None, st, pd, dl, g)
    _, dw32, _ = oracle.convolution_backward(gy, x, xpad, zero_w, st, pd, dl, g, need=(False, True, False))
    _, xpad64 = oracle.convolution_forward(x.astype(np.float64), zero_w.astype(np.float64), None, st, pd, dl, g)
    _, dw64, _ = oracle.convolution_backward(gy.astype(np.float64), x.astype(np.float64), xpad64, zero_w.astype(np.float64),
                                             st, pd, dl, g, need=(False, True, False))
    xd, gyd = hiparray(x), hiparray(gy)
    dw = ops.conv2d_wgrad(xd, gyd, w_shape, st, pd, dl, g).get()
    plan = _last_wgrad()
    assert plan['added_in_kernel'] == 1 and plan['splits'] > 1, plan
    _check('dw', dw, dw32, dw64, reduction=True)
    ops.conv2d_fwd(xd, hiparray(rng.standard_normal(w_shape).astype(np.float32)), None, st, pd, dl, g)   # other work in between
    np.testing.assert_array_equal(ops.conv2d_wgrad(xd, gyd, w_shape, st, pd, dl, g).get(), dw)
    _hip.call('tt_conv2d_wgrad_force_occupancy', 0)
    try:
        dw_two_kernels = ops.conv2d_wgrad(xd, gyd, w_shape, st, pd, dl, g).get()
        assert _last_wgrad()['added_in_kernel'] == 0
    finally:
        _hip.call('tt_conv2d_wgrad_force_occupancy', -1)
    _check('dw (reduce kernel)', dw_two_kernels, dw32, dw64, reduction=True)
    scale = float(np.abs(dw64).max())
    np.testing.assert_allclose(dw, dw_two_kernels, rtol=0, atol=2e-7 * scale)     # both sum float32 partials in float64


def test_weight_gradient_fused_launches_back_to_back_reuse_their_flags():
    """Different layers one after the other re-use the same partial-sum slots and flag words; the flag
    value changes from launch to launch, so nothing left over from the launch before can be taken for
    this launch's: the same bits every time, and the right ones."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(22)
    layers = []
    for case in WGRAD_FUSED_CASES[:5]:
        n, c, h, w_, k, r, s, st, pd, dl, g = case
        p = (h + 2 * pd[0] - dl[0] * (r - 1) - 1) // st[0] + 1
        q = (w_ + 2 * pd[1] - dl[1] * (s - 1) - 1) // st[1] + 1
        layers.append((hiparray(rng.standard_normal((n, c, h, w_)).astype(np.float32)),
                       hiparray(rng.standard_normal((n, k, p, q)).astype(np.float32)), (k, c // g, r, s), (st, pd, dl, g)))
    first = None
    for _ in range(6):
        outs = [ops.conv2d_wgrad(x, gy, shape, *geo) for x, gy, shape, geo in layers]
        got = [o.get() for o in outs]
        if first is None:
            first = got
        for a, b in zip(first, got):
            np.testing.assert_array_equal(a, b)
