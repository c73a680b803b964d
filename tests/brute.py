"""Direct, loop-level definitions used to pin the oracle (float64, tiny shapes only).

These are written from the textbook definitions, not from the oracle's formulation:
the forward is a gather over taps, the input gradient a scatter of every forward
contribution, the weight gradient an accumulation of every forward contribution.
"""
import numpy as np


def conv_out(size, k, s, p, d):
    return (size + 2 * p - d * (k - 1) - 1) // s + 1


def conv2d_def(x, w, b, stride, padding, dilation, groups):
    x = x.astype(np.float64)
    w = w.astype(np.float64)
    n, c, h, wd = x.shape
    k, cg, r, s = w.shape
    kg = k // groups
    p = conv_out(h, r, stride[0], padding[0], dilation[0])
    q = conv_out(wd, s, stride[1], padding[1], dilation[1])
    y = np.zeros((n, k, p, q))
    for ko in range(k):
        g = ko // kg
        for ci in range(cg):
            cc = g * cg + ci
            for rr in range(r):
                for ss in range(s):
                    for pp in range(p):
                        ih = pp * stride[0] + rr * dilation[0] - padding[0]
                        if ih < 0 or ih >= h:
                            continue
                        for qq in range(q):
                            iw = qq * stride[1] + ss * dilation[1] - padding[1]
                            if iw < 0 or iw >= wd:
                                continue
                            y[:, ko, pp, qq] += x[:, cc, ih, iw] * w[ko, ci, rr, ss]
    if b is not None:
        y += b.astype(np.float64)[None, :, None, None]
    return y


def conv2d_grads_def(x, w, gy, stride, padding, dilation, groups):
    """(dx, dw, db) by scattering every forward product term."""
    x = x.astype(np.float64)
    w = w.astype(np.float64)
    gy = gy.astype(np.float64)
    n, c, h, wd = x.shape
    k, cg, r, s = w.shape
    kg = k // groups
    p, q = gy.shape[-2:]
    dx = np.zeros_like(x)
    dw = np.zeros_like(w)
    for ko in range(k):
        g = ko // kg
        for ci in range(cg):
            cc = g * cg + ci
            for rr in range(r):
                for ss in range(s):
                    for pp in range(p):
                        ih = pp * stride[0] + rr * dilation[0] - padding[0]
                        if ih < 0 or ih >= h:
                            continue
                        for qq in range(q):
                            iw = qq * stride[1] + ss * dilation[1] - padding[1]
                            if iw < 0 or iw >= wd:
                                continue
                            dx[:, cc, ih, iw] += gy[:, ko, pp, qq] * w[ko, ci, rr, ss]
                            dw[ko, ci, rr, ss] += (gy[:, ko, pp, qq] * x[:, cc, ih, iw]).sum()
    db = gy.sum((0, 2, 3))
    return dx, dw, db


def conv_transpose2d_def(x, w, b, stride, padding, output_padding, dilation, groups):
    """Scatter definition: every input pixel paints a weighted kernel into the output."""
    x = x.astype(np.float64)
    w = w.astype(np.float64)
    n, cin, h, wd = x.shape
    _, kg, r, s = w.shape
    cg = cin // groups
    k = kg * groups
    ho = (h - 1) * stride[0] - 2 * padding[0] + dilation[0] * (r - 1) + output_padding[0] + 1
    wo = (wd - 1) * stride[1] - 2 * padding[1] + dilation[1] * (s - 1) + output_padding[1] + 1
    y = np.zeros((n, k, ho, wo))
    for ci in range(cin):
        g = ci // cg
        for kk in range(kg):
            ko = g * kg + kk
            for rr in range(r):
                for ss in range(s):
                    for ih in range(h):
                        oh = ih * stride[0] + rr * dilation[0] - padding[0]
                        if oh < 0 or oh >= ho:
                            continue
                        for iw in range(wd):
                            ow = iw * stride[1] + ss * dilation[1] - padding[1]
                            if ow < 0 or ow >= wo:
                                continue
                            y[:, ko, oh, ow] += x[:, ci, ih, iw] * w[ci, kk, rr, ss]
    if b is not None:
        y += b.astype(np.float64)[None, :, None, None]
    return y


def max_pool2d_def(x, kernel_size, stride, padding, dilation, out_hw):
    """(y, arg): window maxima over the -inf padded input, first maximum in (row, column)
    order; arg[n,c,p,q] = (input row, input column) of the chosen element, or None when it
    lies in the padding."""
    n, c, h, w = x.shape
    (kh, kw), (sh, sw), (ph, pw), (dh, dw) = kernel_size, stride, padding, dilation
    p_out, q_out = out_hw
    y = np.empty((n, c, p_out, q_out), x.dtype)
    arg = np.empty((n, c, p_out, q_out), object)
    for nn in range(n):
        for cc in range(c):
            for p in range(p_out):
                for q in range(q_out):
                    best, where = -np.inf, None
                    first = True
                    for i in range(kh):
                        for j in range(kw):
                            hh, ww = p * sh - ph + i * dh, q * sw - pw + j * dw
                            inside = 0 <= hh < h and 0 <= ww < w
                            v = x[nn, cc, hh, ww] if inside else -np.inf
                            if first or v > best:
                                best, where = v, ((hh, ww) if inside else None)
                            first = False
                    y[nn, cc, p, q] = best
                    arg[nn, cc, p, q] = where
    return y, arg


def max_pool2d_backward_def(x_shape, grad, arg, accumulate=False):
    """Visit the windows in (n, c, p, q) order and write (or add) each gradient at its arg-max."""
    dx = np.zeros(x_shape, grad.dtype)
    n, c, p_out, q_out = grad.shape
    for nn in range(n):
        for cc in range(c):
            for p in range(p_out):
                for q in range(q_out):
                    where = arg[nn, cc, p, q]
                    if where is None:
                        continue
                    if accumulate:
                        dx[nn, cc, where[0], where[1]] += grad[nn, cc, p, q]
                    else:
                        dx[nn, cc, where[0], where[1]] = grad[nn, cc, p, q]
    return dx


def bf16_round(a):
    """float32 -> nearest bfloat16 (ties to even), returned as float32: the operand rounding of the
    optional bf16 convolution variant."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))
