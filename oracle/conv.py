"""NumPy restatement of the reference's CPU convolution (test infrastructure only).

Follows ``src/tortto/autograd/grad_nn.py`` of samrere/pytortto 1.3.4:
zero-pad -> strided sliding-window view -> ``np.einsum(..., optimize=True)`` (which NumPy
lowers to tensordot, i.e. an im2col copy and an OpenBLAS sgemm), zero-insertion + flipped
weights for the input gradient, and a stride<->dilation swapped convolution for the weight
gradient.  Keeping that formulation makes this both the parity target and a fair CPU
baseline.  All arrays are NCHW; weights are ``[K, C/g, R, S]`` (``[C_in, C_out/g, R, S]``
for the transposed convolution).
"""
import math

import numpy as np
from numpy.lib.stride_tricks import as_strided


def conv_output_size(size, k, stride, pad, dil):
    """Output extent of one spatial dim (grad_nn.py:565-566: floor of a float division + 1)."""
    return math.floor((size + 2 * pad - dil * (k - 1) - 1) / stride + 1)


def conv_transpose_output_size(size, k, stride, pad, dil, out_pad):
    """Output extent of a transposed convolution (grad_nn.py:677-678)."""
    return (size - 1) * stride - 2 * pad + dil * (k - 1) + out_pad + 1


def _zero_pad(a, pad_hw, extra_hw=(0, 0)):
    """Zero-pad the last two dims (grad_nn.py:509-526).  Like the reference's cached wrapper
    (grad_nn.py:465-469) it hands back the very same array when nothing is to be padded."""
    ph, pw = pad_hw
    eh, ew = extra_hw
    if ph + pw + eh + ew == 0:
        return a
    widths = [(0, 0)] * (a.ndim - 2) + [(ph, ph + eh), (pw, pw + ew)]
    return np.pad(a, widths, constant_values=0)


def _zero_insert(a, step_hw):
    """Spread the last two dims by ``step`` with zeros in between (grad_nn.py:496-506)."""
    sh, sw = step_hw
    if sh == 1 and sw == 1:
        return a
    h, w = a.shape[-2:]
    out = np.zeros(a.shape[:-2] + ((h - 1) * sh + 1, (w - 1) * sw + 1), dtype=a.dtype)
    out[..., ::sh, ::sw] = a
    return out


def _windows(xpad, ksize, stride, dilation):
    """View ``[N, P, Q, C, R, S]`` over an already padded input (grad_nn.py:557-592)."""
    n, c, h, w = xpad.shape
    r, s = ksize
    p = conv_output_size(h, r, stride[0], 0, dilation[0])
    q = conv_output_size(w, s, stride[1], 0, dilation[1])
    sn, sc, sy, sx = xpad.strides
    return as_strided(xpad, shape=(n, p, q, c, r, s),
                      strides=(sn, sy * stride[0], sx * stride[1], sc, sy * dilation[0], sx * dilation[1]),
                      writeable=False)


def _split_channels(a, axis, groups):
    """Reshape-view ``axis`` into ``(groups, size/groups)`` (grad_nn.py:437-442)."""
    axis %= a.ndim
    gs = a.shape[axis] // groups
    shape = a.shape[:axis] + (groups, gs) + a.shape[axis + 1:]
    strides = a.strides[:axis] + (gs * a.strides[axis], a.strides[axis]) + a.strides[axis + 1:]
    return as_strided(a, shape=shape, strides=strides, writeable=False)


def conv2d(x, w, stride=(1, 1), padding=(0, 0), dilation=(1, 1), groups=1,
           backward_w=False, backward_x=False):
    """The reference's ``_conv2d`` NumPy branch (grad_nn.py:595-622).

    Returns ``(value, padded_input)``.  ``backward_x`` contracts over the weight's axis 0
    instead of axis 1; ``backward_w`` treats ``w`` as the upstream gradient and contracts
    over the batch axis.  The groups>1 branch loops over groups and concatenates.
    """
    xpad = _zero_pad(x, padding)
    if groups == 1:
        win = _windows(xpad, w.shape[-2:], stride, dilation)
        if backward_x:
            w = np.swapaxes(w, -3, -4)
        if backward_w:
            win = np.swapaxes(win, -3, 0)
            w = np.swapaxes(w, -3, 0)
        val = np.einsum('NHWihw,oihw->NoHW', win, w, optimize=True)
        if backward_w:
            val = np.swapaxes(val, 1, 0)
    else:
        wsplit = _split_channels(w, -3 if backward_w else -4, groups)
        xsplit = _split_channels(xpad, -3, groups)
        parts = []
        for g in range(groups):
            xg = xsplit[:, g]
            wg = wsplit[:, g] if backward_w else wsplit[g]
            parts.append(conv2d(xg, wg, stride, (0, 0), dilation, 1, backward_w, backward_x)[0])
        val = np.concatenate(parts, axis=-4 if backward_w else -3)
    return val, xpad


def conv2d_backward_w(x, grad, stride, padding, dilation, groups, weight_shape):
    """Weight gradient (grad_nn.py:646-656): crop the padded input to the rows/columns the
    forward pass read, then convolve it with ``grad`` using stride and dilation swapped.
    Returns ``(dw, padded_input)``."""
    xpad = _zero_pad(x, padding)
    r, s = weight_shape[-2:]
    p, q = grad.shape[-2:]
    hv = (p - 1) * stride[0] + 1 + dilation[0] * (r - 1)
    wv = (q - 1) * stride[1] + 1 + dilation[1] * (s - 1)
    dw, _ = conv2d(xpad[..., :hv, :wv], grad, stride=dilation, padding=(0, 0), dilation=stride,
                   groups=groups, backward_w=True)
    return dw, xpad


def conv2d_backward_x(grad, w, stride, padding, dilation, groups, x_hw=None, output_padding=(0, 0)):
    """Input gradient / transposed-convolution forward (grad_nn.py:659-682).

    Zero-insert ``grad`` by ``stride``, pad by ``(R-1)*dil``, run a stride-1 convolution with
    the spatially flipped, channel-swapped weights, crop the forward padding away and
    zero-fill bottom/right rows the forward pass never covered.  ``x_hw`` is the target
    spatial size (conv backward); when ``None`` it follows from ``output_padding``.
    """
    gz = _zero_insert(grad, stride)
    wf = np.flip(w, axis=(-1, -2))
    r, s = w.shape[-2:]
    gp = _zero_pad(gz, ((r - 1) * dilation[0], (s - 1) * dilation[1]))
    full, _ = conv2d(gp, wf, (1, 1), (0, 0), dilation, groups, backward_x=True)
    if x_hw is not None:
        hx, wx = x_hw
    else:
        oph = output_padding[0]
        opw = oph if len(output_padding) == 1 else output_padding[1]
        hx = conv_transpose_output_size(grad.shape[-2], r, stride[0], padding[0], dilation[0], oph)
        wx = conv_transpose_output_size(grad.shape[-1], s, stride[1], padding[1], dilation[1], opw)
    ph, pw = padding
    out = full[..., ph:hx + ph, pw:wx + pw]
    hh, ww = out.shape[-2:]
    return np.pad(out, ((0, 0), (0, 0), (0, hx - hh), (0, wx - ww)))


# ---- autograd-node level (grad_nn.py:684-779) ------------------------------------------

def convolution_forward(x, w, b, stride, padding, dilation, groups):
    """``Convolution.forward`` (grad_nn.py:686-715): returns ``(y, padded_input)``."""
    y, xpad = conv2d(x, w, stride, padding, dilation, groups)
    if b is not None:
        y += b[:, None, None]
    return y, xpad


def convolution_backward(gy, x, xpad, w, stride, padding, dilation, groups,
                         need=(True, True, True)):
    """``Convolution.backward`` (grad_nn.py:718-734): returns ``(dx, dw, db)``."""
    dx = dw = db = None
    if need[2]:
        db = gy.sum((0, 2, 3))
    if need[1]:
        dw = conv2d_backward_w(xpad, gy, stride, (0, 0), dilation, groups, w.shape)[0]
    if need[0]:
        dx = conv2d_backward_x(gy, w, stride, padding, dilation, groups, x_hw=x.shape[-2:])
    return dx, dw, db


def transposed_convolution_forward(x, w, b, stride, padding, output_padding, dilation, groups):
    """``TransposedConvolution.forward`` (grad_nn.py:739-760)."""
    y = conv2d_backward_x(x, w, stride, padding, dilation, groups, output_padding=output_padding)
    if b is not None:
        y += b[:, None, None]
    return y


def transposed_convolution_backward(gy, x, w, stride, padding, dilation, groups,
                                    need=(True, True, True)):
    """``TransposedConvolution.backward`` (grad_nn.py:762-779): returns ``(dx, dw, db)``.

    The reference reuses the padded upstream gradient produced by the weight-gradient
    call for the input gradient and falls back to the *unpadded* gradient when the weight
    needs no gradient (grad_nn.py:778), which is only correct for padding 0.  This
    restatement always pads, i.e. it returns the mathematically correct dx.
    """
    dx = dw = db = None
    if need[2]:
        db = gy.sum((0, 2, 3))
    gpad = _zero_pad(gy, padding)
    if need[1]:
        dw = conv2d_backward_w(gy, x, stride, padding, dilation, groups, w.shape)[0]
    if need[0]:
        dx = conv2d(gpad, w, stride, (0, 0), dilation, groups)[0]
    return dx, dw, db
