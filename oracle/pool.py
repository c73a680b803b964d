"""MaxPool2d restated from ``src/tortto/autograd/grad_nn.py`` -- TEST INFRASTRUCTURE ONLY.

``max_pool2d`` follows ``_max_pool2d`` (:784-808) over ``_sliding_window_view`` (:557-592) with
``val=-inf``; ``max_pool2d_backward`` follows ``_max_pool2d_backward`` (:811-824).  Two things
are specific to the reference and kept: the arg-max is found in two stages (first column per
kernel row, then first row), which selects the first maximum in (row, column) order; and the
backward *assigns* through an overlapping strided view (:818), so where several windows chose
the same pixel the one NumPy writes last -- the last in (p, q) order -- wins and nothing is
summed.

One deliberate difference: with ``ceil_mode`` the reference drops the bottom/right padding of
*both* axes as soon as one axis loses its last window (``aug``, :573-582, :520-522) and may
then read beyond its padded array; here the padded array always covers every window, which
gives the same values wherever the reference stays inside its array.

Pinned by (tests/test_oracle_pool.py): nested-loop brute force with sequential assignment,
torch CPU ``F.max_pool2d`` for the forward (padding, dilation, ceil_mode) and torch autograd for
the backward where windows do not overlap (there assignment and summation coincide).
"""
import math

import numpy as np


def pool_output_size(size, k, stride, pad, dil, ceil_mode=False):
    """grad_nn.py:565-579 (one axis)."""
    span = size + 2 * pad - dil * (k - 1) - 1
    if not ceil_mode:
        return math.floor(span / stride + 1)
    out = math.ceil(span / stride + 1)
    extra = (out - 1) * stride - span
    if extra + pad >= (k - 1) * dil + 1:
        out -= 1
    return out


def _windows(x, kernel_size, stride, padding, dilation, ceil_mode, fill):
    """(view [N,P,Q,C,kh,kw] into the padded copy, padded copy) -- grad_nn.py:557-592."""
    n, c, h, w = x.shape
    (kh, kw), (sh, sw), (ph, pw), (dh, dw) = kernel_size, stride, padding, dilation
    p = pool_output_size(h, kh, sh, ph, dh, ceil_mode)
    q = pool_output_size(w, kw, sw, pw, dw, ceil_mode)
    rows = max(h + 2 * ph, (p - 1) * sh + (kh - 1) * dh + 1)
    cols = max(w + 2 * pw, (q - 1) * sw + (kw - 1) * dw + 1)
    padded = np.full((n, c, rows, cols), fill, dtype=x.dtype)
    padded[:, :, ph:ph + h, pw:pw + w] = x
    sn, sc, s_h, s_w = padded.strides
    view = np.lib.stride_tricks.as_strided(padded, shape=(n, p, q, c, kh, kw),
                                           strides=(sn, s_h * sh, s_w * sw, sc, s_h * dh, s_w * dw))
    return view, padded


def max_pool2d(x, kernel_size, stride, padding=(0, 0), dilation=(1, 1), ceil_mode=False):
    """y [N,C,P,Q] and pos = (kernel-row index, kernel-column index), each [N,P,Q,C]."""
    low_dim = x.ndim == 3
    if low_dim:
        x = x[None]
    win, _ = _windows(x, kernel_size, stride, padding, dilation, ceil_mode, -np.inf)
    idx1 = np.nanargmax(win, -1)                                        # first column per kernel row
    row_max = np.take_along_axis(win, idx1[..., None], -1)[..., 0]
    idx2 = np.nanargmax(row_max, -1)                                    # first row among the row maxima
    value = np.take_along_axis(row_max, idx2[..., None], -1)[..., 0]
    idx1_m = np.take_along_axis(idx1, idx2[..., None], -1)[..., 0]
    y = np.ascontiguousarray(np.moveaxis(value, -1, -3))
    return (y[0] if low_dim else y), (idx2, idx1_m)


def max_pool2d_backward(x_shape, grad, pos, kernel_size, stride, padding=(0, 0), dilation=(1, 1),
                        ceil_mode=False):
    low_dim = len(x_shape) == 3
    if low_dim:
        x_shape, grad = (1,) + tuple(x_shape), grad[None]
    idx2, idx1_m = pos
    win, padded = _windows(np.zeros(x_shape, dtype=grad.dtype), kernel_size, stride, padding, dilation,
                           ceil_mode, -np.inf)
    n, p, q, c = idx2.shape
    ax = np.ix_(np.arange(n), np.arange(p), np.arange(q), np.arange(c))
    win[ax[0], ax[1], ax[2], ax[3], idx2, idx1_m] = np.moveaxis(grad, -3, -1)   # assignment, not +=
    (ph, pw), (h, w) = padding, x_shape[-2:]
    dx = np.ascontiguousarray(padded[..., ph:ph + h, pw:pw + w])
    return dx[0] if low_dim else dx
