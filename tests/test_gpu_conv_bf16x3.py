"""GPU checks of float32 convolution arithmetic carried out on the bf16 matrix instructions
(tt_set_conv_math(TT_CONV_MATH_BF16X3), tt.cuda.set_conv_math('bf16x3')).

Inside the kernels every operand element becomes three bfloat16 terms that add up to it exactly and
all products of terms except the three smallest are accumulated in float32 (what is left out stays
below 2^-24 of a product, half an ulp of it: tests/test_bf16_round.py).  Forward and input gradient
run that way for every geometry (the float32 kernels with another matrix step); the weight gradient
keeps the float32 instructions and must not change with the mode.  The mode therefore has to meet the float32
path's own bar, and these tests hold it to exactly that: the same cases through the same checks as
tests/test_gpu_conv.py -- allclose(rtol=1e-4, atol=1e-5) against the oracle (atol scaled by the
tensor's magnitude for the weight / bias gradients) and no further from a float64 evaluation than
three times the oracle's own float32 error.  The reference has no such mode.
"""
import ctypes

import numpy as np
import pytest

import oracle
from bench import RESNET50_CONVS
from tests.cases import CONV_CASES, CONVT_CASES, random_conv_cases, random_convt_cases
from tests.test_gpu_conv import CONVT_TILE_CASES, LARGE_IMAGE_CASES, TILE_CASES, _check, _run_conv
from tests.test_gpu_conv import test_conv_transpose_forward_backward as _conv_transpose_checks
from tests.test_gpu_full_size_shapes import test_shape_at_full_batch_properties as _full_size_checks

pytestmark = pytest.mark.gpu


@pytest.fixture
def three_terms():
    from pytortto_amd import _hip
    _hip.set_conv_math('bf16x3')
    try:
        yield
    finally:
        _hip.set_conv_math('f32')


def _terms_of_last_launch():
    """bf16 terms per operand element of the matrix instructions the last forward / input-gradient
    launch used: 0 = float32 instructions."""
    from pytortto_amd import _hip
    plan = (ctypes.c_int * 8)()
    _hip.call('tt_conv2d_last_launch', plan)
    return plan[7] >> 8


@pytest.mark.parametrize('case', CONV_CASES + TILE_CASES + random_conv_cases(40, 31))
def test_conv_meets_the_float32_bar(case, three_terms):
    _run_conv(case)


@pytest.mark.parametrize('case', TILE_CASES[:16])
def test_conv_without_bias_meets_the_float32_bar(case, three_terms):
    _run_conv(case, seed=9, bias=False)


@pytest.mark.parametrize('case', LARGE_IMAGE_CASES)
def test_conv_large_images_meet_the_float32_bar(case, three_terms):
    """Images too large for 32-bit offsets: 64-bit addresses with compared bounds, also in this arithmetic."""
    _run_conv(case, seed=3)


@pytest.mark.parametrize('case', CONVT_CASES + CONVT_TILE_CASES + random_convt_cases(12, 17))
def test_conv_transpose_meets_the_float32_bar(case, three_terms):
    _conv_transpose_checks(case)


# one shape per way the kernels address their operands
TAKEN = [
    (4, 64, 28, 28, 256, 1, 1, (1, 1), (0, 0), (1, 1), 1),       # 1x1: rows / columns of w in place
    (8, 128, 28, 28, 128, 3, 3, (1, 1), (1, 1), (1, 1), 1),      # 3x3: tap masks, shared reductions
    (16, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), (1, 1), 1),       # 64-row tiles
    (3, 64, 6, 6, 64, 1, 1, (1, 1), (0, 0), (1, 1), 2),          # groups
    (4, 128, 28, 28, 128, 3, 3, (2, 2), (1, 1), (1, 1), 1),      # stride 2: the gradient's classes share a grid
    (8, 3, 64, 64, 64, 7, 7, (2, 2), (3, 3), (1, 1), 1),         # 49 taps: 64-bit masks, dense input gradient
    (3, 16, 14, 14, 16, 9, 9, (1, 1), (4, 4), (1, 1), 1),        # 81 taps: compared bounds
]


@pytest.mark.parametrize('case', TAKEN)
def test_the_three_term_kernels_are_the_ones_that_ran(case, three_terms):
    """The launch plan names the matrix instructions; the weight gradient does not depend on the mode."""
    from pytortto_amd import _hip, ops
    from pytortto_amd.xparray import hiparray
    n, c, h, w_, k, r, s, st, pd, dl, g = case
    rng = np.random.default_rng(3)
    x = hiparray(rng.standard_normal((n, c, h, w_)).astype(np.float32))
    w = hiparray(rng.standard_normal((k, c // g, r, s)).astype(np.float32))
    y = ops.conv2d_fwd(x, w, None, st, pd, dl, g)
    assert _terms_of_last_launch() == 3
    gy = hiparray(rng.standard_normal(y.shape).astype(np.float32))
    ops.conv2d_dgrad(gy, w, None, (h, w_), st, pd, dl, g)
    assert _terms_of_last_launch() == 3
    dw3 = ops.conv2d_wgrad(x, gy, w.shape, st, pd, dl, g).get()
    _hip.set_conv_math('f32')
    ops.conv2d_fwd(x, w, None, st, pd, dl, g)
    assert _terms_of_last_launch() == 0
    dw1 = ops.conv2d_wgrad(x, gy, w.shape, st, pd, dl, g).get()
    _hip.set_conv_math('bf16x3')
    np.testing.assert_array_equal(dw3, dw1)


def test_operands_far_from_one_keep_float32_accuracy(three_terms):
    """bfloat16 has float32's exponent range: operands of 1e-20 and 1e+15 need no scaling (a split into
    float16 terms would lose them), and zeros stay zeros."""
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(6)
    n, c, h, k = 4, 64, 28, 128
    x = (rng.standard_normal((n, c, h, h)) * 1e-20).astype(np.float32)
    x[:, ::3] = 0.0
    w = (rng.standard_normal((k, c, 3, 3)) * 1e15).astype(np.float32)
    geo = ((1, 1), (1, 1), (1, 1), 1)
    y32, xpad = oracle.convolution_forward(x, w, None, *geo)
    y64, _ = oracle.convolution_forward(x.astype(np.float64), w.astype(np.float64), None, *geo)
    y = ops.conv2d_fwd(hiparray(x), hiparray(w), None, *geo).get()
    assert _terms_of_last_launch() == 3
    scale = float(np.abs(y64).max())
    assert 1e-5 < scale < 1e-2
    assert float(np.abs(y - y64).max()) <= max(3 * float(np.abs(y32 - y64).max()), 5e-6 * scale)
    np.testing.assert_allclose(y, y32, rtol=1e-4, atol=1e-5 * scale)
    gy = (rng.standard_normal(y.shape) * 1e-12).astype(np.float32)
    dw32 = oracle.convolution_backward(gy, x, xpad, w, *geo)[1]
    dw = ops.conv2d_wgrad(hiparray(x), hiparray(gy), w.shape, *geo).get()
    np.testing.assert_allclose(dw, dw32, rtol=1e-4, atol=1e-5 * float(np.abs(dw32).max()))


def test_entry_points_for_one_call_leave_the_mode_alone():
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(7)
    n, c, h, k = 64, 128, 28, 128
    x = hiparray(rng.standard_normal((n, c, h, h)).astype(np.float32))
    w = hiparray((rng.standard_normal((k, c, 3, 3)) / 34.0).astype(np.float32))
    gy = hiparray(rng.standard_normal((n, k, h, h)).astype(np.float32))
    outs = {}
    for how in ('call', 'mode'):
        y, dx, dw = (hiparray(np.zeros(s, np.float32)) for s in ((n, k, h, h), (n, c, h, h), (k, c, 3, 3)))
        if how == 'mode':
            _hip.set_conv_math('bf16x3')
        sfx = 'bf16x3' if how == 'call' else 'f32'
        try:
            _hip.call('tt_conv2d_fwd_' + sfx, x.ptr, w.ptr, None, y.ptr, n, c, h, h, k, 3, 3, 1, 1, 1, 1, 1, 1, 1)
            taken = _terms_of_last_launch()
            _hip.call('tt_conv2d_dgrad_' + sfx, gy.ptr, w.ptr, None, dx.ptr, n, c, h, h, k, 3, 3, 1, 1, 1, 1, 1, 1, 1, h, h)
            _hip.call('tt_conv2d_wgrad_f32', x.ptr, gy.ptr, dw.ptr, n, c, h, h, k, 3, 3, 1, 1, 1, 1, 1, 1, 1, h, h)
        finally:
            _hip.set_conv_math('f32')
        assert taken == 3
        assert _hip.get_conv_math() == 'f32'
        outs[how] = (y.get(), dx.get(), dw.get())
    for a, b in zip(outs['call'], outs['mode']):
        np.testing.assert_array_equal(a, b)


FULL_SIZE = [s for s in RESNET50_CONVS if (s[0], s[1], s[2], s[3]) in {
    (64, 56, 256, 1), (256, 56, 64, 1), (64, 56, 64, 3), (256, 56, 512, 1), (128, 28, 128, 3), (512, 28, 256, 1), (256, 14, 1024, 1),
    (256, 14, 256, 3)}]


@pytest.mark.parametrize('spec', FULL_SIZE, ids=lambda s: 'C%d_H%d_K%d_k%d_s%d' % s[:5])
def test_benchmark_shapes_at_full_batch(spec, three_terms):
    """The benchmark's shapes at batch 64 with the routing the mode uses by default, through the
    float32 path's own full-size checks (selected images against the oracle at rtol 1e-4 / atol 1e-5,
    linearity of the weight gradient, adjointness)."""
    assert len(FULL_SIZE) == 8
    _full_size_checks(spec, 64)
