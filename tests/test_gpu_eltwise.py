"""GPU: the elementwise glue kernels straight through the C ABI, bit for bit against NumPy
expressions of the reference (``gd0 * (yd0 > 0)``, ``a + b``, ``acc += alpha * v``): sizes that are
not a multiple of four (scalar tail), sizes below one vector, non-finite gradients at masked
elements, a large array that wraps the capped grid several times, and misaligned pointers."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 4, 5, 7, 1023, 1025, 4099, (1 << 20) + 3]


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _same_bits(got, want, name):
    got, want = _bits(got), _bits(want)
    nan_got, nan_want = np.isnan(got.view(np.float32)), np.isnan(want.view(np.float32))
    assert np.array_equal(nan_got, nan_want), f'{name}: NaN pattern differs'
    assert np.array_equal(got[~nan_got], want[~nan_want]), f'{name}: bits differ'   # -0.0 and +0.0 are told apart


def _special_gradient(rng, n):
    g = rng.standard_normal(n).astype(np.float32)
    if n >= 5:
        g[:5] = [np.inf, -np.inf, np.nan, -2.5, 0.0]
    return g


@pytest.mark.parametrize('n', SIZES)
def test_relu_backward_multiplies_by_the_mask(n):
    """dx = dy * (y > 0) (grad_nn.py:67): where y <= 0, an infinite or NaN dy gives NaN and a
    negative dy gives -0.0 -- a select would give +0.0 there."""
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(n)
    y = np.maximum(rng.standard_normal(n).astype(np.float32), 0)
    if n >= 8:
        y[:8] = [0, 0, 0, 0, 0, 1.5, np.nan, 2.0]      # masked: elements 0-4 and the NaN
    dy = _special_gradient(rng, n)
    with np.errstate(invalid='ignore'):
        want = dy * (y > 0)
    dx, dyd, yd = hiparray.empty((n,)), hiparray(dy), hiparray(y)
    _hip.call('tt_relu_bwd_f32', dyd.ptr, yd.ptr, dx.ptr, n)
    _same_bits(dx.get(), want, 'relu_bwd')


@pytest.mark.parametrize('n', SIZES)
def test_add_and_axpy(n):
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(1000 + n)
    a, b = _special_gradient(rng, n), rng.standard_normal(n).astype(np.float32)
    out, ad, bd = hiparray.empty((n,)), hiparray(a), hiparray(b)
    _hip.call('tt_add_f32', ad.ptr, bd.ptr, out.ptr, n)
    with np.errstate(invalid='ignore'):
        _same_bits(out.get(), a + b, 'add')
    # gradient accumulation acc += v (tensor.py:596-599): alpha = 1, so the fused multiply-add is exact
    acc = hiparray(b)
    _hip.call('tt_axpy_f32', 1.0, ad.ptr, acc.ptr, n)
    with np.errstate(invalid='ignore'):
        _same_bits(acc.get(), b + a, 'axpy')
    # a general alpha is a fused multiply-add (one rounding): within one unit in the last place of
    # the float64 product-sum (which itself rounds twice)
    acc = hiparray(b)
    fin = np.isfinite(a)
    _hip.call('tt_axpy_f32', 0.3, ad.ptr, acc.ptr, n)
    want = (np.float64(np.float32(0.3)) * a[fin].astype(np.float64) + b[fin].astype(np.float64)).astype(np.float32)
    np.testing.assert_array_max_ulp(acc.get()[fin], want, maxulp=1)


def test_elementwise_kernels_refuse_misaligned_pointers():
    """Tensor pointers at the C ABI are 16-byte aligned; a pointer offset by one float is refused
    with a message instead of being used for 16-byte vector accesses."""
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    buf, out = hiparray.empty((64,)), hiparray.empty((64,))
    off = buf.ptr + 4
    for name, args in (('tt_relu_fwd_f32', (off, out.ptr, 32)), ('tt_add_f32', (buf.ptr, off, out.ptr, 32)),
                       ('tt_bn_fwd_eval_f32', (off, None, None, out.ptr, buf.ptr, buf.ptr, buf.ptr, buf.ptr, buf.ptr,
                                               1e-5, 2, 4, 4))):
        with pytest.raises(RuntimeError, match='16-byte aligned'):
            _hip.call(name, *args)
