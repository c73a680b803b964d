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
