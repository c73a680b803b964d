"""GPU checks of the optional bf16 MFMA variant of the three convolution passes.

The reference is float32 throughout, so this variant has no counterpart to be identical to; what
it computes is pinned exactly instead: both operands rounded to bfloat16 (nearest even), products
accumulated in float32, bias added in float32.  Products of two bfloat16 values are exact in
float32, so the oracle run on operands rounded the same way on the host must agree to the
float32 bar (rtol=1e-4, atol=1e-5 of the tensor's magnitude) -- only the summation order differs.
Against the oracle on the unrounded operands the stated bound is max|error| <= 1e-2 * max|ref|
(measured: 2-3e-3); for the weight gradient, a sum over all N*P*Q pixels, it is taken relative to
max|ref| too.  Everything else (bias gradient, BatchNorm, ...) must not change with the mode.
"""
import numpy as np
import pytest

import oracle
from tests.brute import bf16_round
from tests.cases import CONV_CASES, CONVT_CASES, random_conv_cases, random_convt_cases
from tests.test_gpu_conv import TILE_CASES, CONVT_TILE_CASES

pytestmark = pytest.mark.gpu

LOOSE_BOUND = 1e-2


@pytest.fixture
def bf16_math():
    """bf16 arithmetic, with every launch the bf16-first kernels support sent to them (by default the
    small tile counts of test shapes with long reductions would stay on the other kernels)."""
    from pytortto_amd import _hip
    _hip.set_conv_math('bf16')
    _hip.call('tt_conv2d_bf16_first_enable', 2)
    try:
        yield
    finally:
        _hip.call('tt_conv2d_bf16_first_enable', 1)
        _hip.set_conv_math('f32')


def _close(name, got, model, plain):
    scale = max(1.0, float(np.abs(model).max()))
    np.testing.assert_allclose(got, model, rtol=1e-4, atol=1e-5 * scale, err_msg=name + ' vs oracle on rounded operands')
    err = float(np.abs(got - plain).max()) / (float(np.abs(plain).max()) or 1.0)
    assert err <= LOOSE_BOUND, f'{name}: {err:.3g} of max|ref| against the float32 oracle'


@pytest.mark.parametrize('case', CONV_CASES + TILE_CASES + random_conv_cases(40, 123))
def test_conv_bf16_forward_and_input_gradient(case, bf16_math):
    _forward_and_input_gradient(case)


def _forward_and_input_gradient(case):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(4)
    x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
    w = (rng.standard_normal((k, c // g, r, s)) / np.sqrt(c // g * r * s)).astype(np.float32)
    b = rng.standard_normal(k).astype(np.float32)
    y32, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, g)
    gy = rng.standard_normal(y32.shape).astype(np.float32)
    dx32, dw32, _ = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
    xr, wr, gyr = (bf16_round(a).astype(np.float64) for a in (x, w, gy))
    y_model, xpad_r = oracle.convolution_forward(xr, wr, b.astype(np.float64), st, pd, dl, g)
    dx_model = oracle.conv2d_backward_x(gyr, wr, st, pd, dl, g, x_hw=(h, w_))
    dw_model = oracle.convolution_backward(gyr, xr, xpad_r, wr, st, pd, dl, g)[1]

    xd, wd, gyd = hiparray(x), hiparray(w), hiparray(gy)
    y = ops.conv2d_fwd(xd, wd, hiparray(b), st, pd, dl, g).get()
    dx = ops.conv2d_dgrad(gyd, wd, None, (h, w_), st, pd, dl, g).get()
    dw = ops.conv2d_wgrad(xd, gyd, w.shape, st, pd, dl, g).get()
    _close('y', y, y_model, y32)
    _close('dx', dx, dx_model, dx32)
    _close('dw', dw, dw_model, dw32)


@pytest.mark.parametrize('case', CONVT_CASES + CONVT_TILE_CASES + random_convt_cases(12, 321))
def test_conv_transpose_bf16_forward_and_input_gradient(case, bf16_math):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    n, ci, h, w_, co, r, s, st, pd, op, dl, g = case
    rng = np.random.default_rng(5)
    x = rng.standard_normal((n, ci, h, w_)).astype(np.float32)
    w = (rng.standard_normal((ci, co // g, r, s)) / np.sqrt(ci // g * r * s)).astype(np.float32)
    b = rng.standard_normal(co).astype(np.float32)
    y32 = oracle.transposed_convolution_forward(x, w, b, st, pd, op, dl, g)
    gy = rng.standard_normal(y32.shape).astype(np.float32)
    dx32, dw32, _ = oracle.transposed_convolution_backward(gy, x, w, st, pd, dl, g)
    xr, wr, gyr = (bf16_round(a).astype(np.float64) for a in (x, w, gy))
    y_model = oracle.transposed_convolution_forward(xr, wr, b.astype(np.float64), st, pd, op, dl, g)
    dx_model, dw_model, _ = oracle.transposed_convolution_backward(gyr, xr, wr, st, pd, dl, g)

    xd, wd, gyd = hiparray(x), hiparray(w), hiparray(gy)
    y = ops.conv2d_dgrad(xd, wd, hiparray(b), y32.shape[-2:], st, pd, dl, g).get()
    dx = ops.conv2d_fwd(gyd, wd, None, st, pd, dl, g).get()
    dw = ops.conv2d_wgrad(gyd, xd, w.shape, st, pd, dl, g).get()
    _close('y', y, y_model, y32)
    _close('dx', dx, dx_model, dx32)
    _close('dw', dw, dw_model, dw32)


def _persistent_blocks_of_last_launch():
    import ctypes
    from pytortto_amd import _hip
    plan = (ctypes.c_int * 8)()
    _hip.call('tt_conv2d_last_launch', plan)
    return plan[4]


# shapes the bf16-first kernels take, one per way they fetch their operands: (forward, input gradient)
BF16_FIRST_CASES = [
    ((4, 64, 28, 28, 256, 1, 1, (1, 1), (0, 0), (1, 1), 1), (True, True)),      # 1x1: rows in place / columns in place, 128- and 64-row tiles
    ((16, 256, 14, 14, 1024, 1, 1, (1, 1), (0, 0), (1, 1), 1), (True, True)),   # 1x1, 128-row tiles both ways, ragged last pixel tile
    ((4, 64, 28, 28, 64, 1, 1, (1, 1), (0, 0), (1, 1), 1), (True, True)),       # 64-row tiles
    ((8, 128, 28, 28, 128, 3, 3, (1, 1), (1, 1), (1, 1), 1), (True, True)),     # 3x3: tap masks, rows in place / repacked quads
    ((16, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1), (True, True)),      # 3x3 with 64-row tiles
    ((2, 32, 12, 12, 64, 1, 1, (1, 1), (1, 1), (1, 1), 1), (True, True)),       # padded 1x1: one-tap mask, columns in place
    ((3, 64, 6, 6, 64, 1, 1, (1, 1), (0, 0), (1, 1), 2), (True, True)),         # groups
    ((4, 128, 28, 28, 128, 3, 3, (2, 2), (1, 1), (1, 1), 1), (True, False)),    # stride 2: forward only (the input gradient's classes share a grid)
    ((5, 32, 13, 9, 48, 5, 5, (2, 1), (4, 2), (2, 1), 2), (False, False)),      # 16 channels per group x 25 taps: not whole chunks
    ((8, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3), (1, 1), 1), (False, False)),      # stem: 49 taps, dense input gradient
]


@pytest.mark.parametrize('case,takes', BF16_FIRST_CASES)
def test_bf16_first_kernels_and_the_other_bf16_kernels_agree(case, takes, bf16_math):
    """Which launches go to the bf16-first kernels, and that they and the float32 kernels' bf16
    instantiations -- both "the convolution of the bf16-rounded operands in float32" -- agree to the
    float32 bar on the same inputs (the summation order differs)."""
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(8)
    x = hiparray(rng.standard_normal((n, c, h, w_)).astype(np.float32))
    w = hiparray((rng.standard_normal((k, c // g, r, s)) / np.sqrt(c // g * r * s)).astype(np.float32))
    p = (h + 2 * pd[0] - dl[0] * (r - 1) - 1) // st[0] + 1
    q = (w_ + 2 * pd[1] - dl[1] * (s - 1) - 1) // st[1] + 1
    gy = hiparray(rng.standard_normal((n, k, p, q)).astype(np.float32))
    y = ops.conv2d_fwd(x, w, None, st, pd, dl, g).get()
    assert (_persistent_blocks_of_last_launch() == -1) == takes[0]
    dx = ops.conv2d_dgrad(gy, w, None, (h, w_), st, pd, dl, g).get()
    assert (_persistent_blocks_of_last_launch() == -1) == takes[1]
    _hip.call('tt_conv2d_bf16_first_enable', 0)
    try:
        y_other = ops.conv2d_fwd(x, w, None, st, pd, dl, g).get()
        assert _persistent_blocks_of_last_launch() != -1
        dx_other = ops.conv2d_dgrad(gy, w, None, (h, w_), st, pd, dl, g).get()
    finally:
        _hip.call('tt_conv2d_bf16_first_enable', 2)
    for name, a, b in (('y', y, y_other), ('dx', dx, dx_other)):
        np.testing.assert_allclose(a, b, rtol=1e-4, atol=1e-5 * max(1.0, float(np.abs(b).max())), err_msg=name)


@pytest.mark.parametrize('case', TILE_CASES)
def test_conv_bf16_on_the_float32_kernels_instantiations(case, bf16_math):
    """The same pins as above with the bf16-first kernels switched off: the instantiations that serve
    whatever those do not take stay covered on every tile shape."""
    from pytortto_amd import _hip
    _hip.call('tt_conv2d_bf16_first_enable', 0)
    try:
        _forward_and_input_gradient(case)
    finally:
        _hip.call('tt_conv2d_bf16_first_enable', 2)


def test_other_ops_do_not_depend_on_the_mode_and_it_switches_back():
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(6)
    x = hiparray(rng.standard_normal((8, 32, 14, 14), dtype=np.float32))
    gy = hiparray(rng.standard_normal((8, 48, 14, 14), dtype=np.float32))
    w = hiparray(rng.standard_normal((48, 32, 3, 3), dtype=np.float32))
    args = ((1, 1), (1, 1), (1, 1), 1)
    assert _hip.get_conv_math() == 'f32'
    dw = ops.conv2d_wgrad(x, gy, (48, 32, 3, 3), *args).get()
    y = ops.conv2d_fwd(x, w, None, *args).get()
    db = ops.channel_sum(gy).get()
    _hip.set_conv_math('bf16')
    try:
        assert _hip.get_conv_math() == 'bf16'
        np.testing.assert_array_equal(ops.channel_sum(gy).get(), db)
        assert np.abs(ops.conv2d_fwd(x, w, None, *args).get() - y).max() > 0          # the mode is really in effect
        assert np.abs(ops.conv2d_wgrad(x, gy, (48, 32, 3, 3), *args).get() - dw).max() > 0
    finally:
        _hip.set_conv_math('f32')
    np.testing.assert_array_equal(ops.conv2d_fwd(x, w, None, *args).get(), y)   # and really off again
    np.testing.assert_array_equal(ops.conv2d_wgrad(x, gy, (48, 32, 3, 3), *args).get(), dw)
    with pytest.raises(ValueError):
        _hip.set_conv_math('fp8')


def test_per_call_bf16_entry_points_leave_the_process_wide_mode_alone():
    """tt_conv2d_*_bf16: bf16 arithmetic for one call; the same bits as the float32-named entry points
    give under tt_set_conv_math(bf16), and the mode other callers see is float32 before and after."""
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(10)
    n, c, h, k = 4, 32, 14, 48
    x = hiparray(rng.standard_normal((n, c, h, h), dtype=np.float32))
    w = hiparray(rng.standard_normal((k, c, 3, 3), dtype=np.float32))
    gy = hiparray(rng.standard_normal((n, k, h, h), dtype=np.float32))
    geo = ((1, 1), (1, 1), (1, 1), 1)
    a = (n, c, h, h, k, 3, 3, 1, 1, 1, 1, 1, 1, 1)
    y, dx, dw = hiparray.empty((n, k, h, h)), hiparray.empty((n, c, h, h)), hiparray.empty((k, c, 3, 3))
    assert _hip.get_conv_math() == 'f32'
    _hip.call('tt_conv2d_fwd_bf16', x.ptr, w.ptr, None, y.ptr, *a)
    _hip.call('tt_conv2d_dgrad_bf16', gy.ptr, w.ptr, None, dx.ptr, *a, h, h)
    _hip.call('tt_conv2d_wgrad_bf16', x.ptr, gy.ptr, dw.ptr, *a, h, h)
    assert _hip.get_conv_math() == 'f32'
    y32 = ops.conv2d_fwd(x, w, None, *geo).get()
    _hip.set_conv_math('bf16')
    try:
        want = (ops.conv2d_fwd(x, w, None, *geo).get(), ops.conv2d_dgrad(gy, w, None, (h, h), *geo).get(),
                ops.conv2d_wgrad(x, gy, (k, c, 3, 3), *geo).get())
    finally:
        _hip.set_conv_math('f32')
    for got, ref in zip((y, dx, dw), want):
        np.testing.assert_array_equal(got.get(), ref)
    assert np.abs(y.get() - y32).max() > 0                       # really bf16
    np.testing.assert_array_equal(ops.conv2d_fwd(x, w, None, *geo).get(), y32)   # and float32 for everybody else


def test_module_api_switch():
    import pytortto_amd as tt
    tt.manual_seed(0)
    conv = tt.nn.Conv2d(16, 32, 3, padding=1).cuda()
    x = tt.randn(4, 16, 12, 12).cuda()
    y = conv(x).data.get()
    tt.cuda.set_conv_math('bf16')
    try:
        assert tt.cuda.get_conv_math() == 'bf16'
        y_bf = conv(x).data.get()
    finally:
        tt.cuda.set_conv_math('f32')
    err = np.abs(y_bf - y).max() / np.abs(y).max()
    assert 0 < err <= LOOSE_BOUND
