"""NumPy restatement of the reference's CPU BatchNorm (test infrastructure only).

Follows ``BatchNorm.forward`` / ``BatchNorm.backward`` in
``src/tortto/autograd/grad_nn.py:907-989`` of samrere/pytortto 1.3.4, pass by pass, so the
float32 rounding class and the CPU cost (about ten sweeps forward, twelve backward) are
those of the reference.
"""
from math import prod

import numpy as np


def batch_norm_forward(x, gamma, beta, running_mean, running_var, training, momentum, eps):
    """Returns ``(y, saved, new_running_mean, new_running_var)``.

    ``saved`` holds ``mean``, ``var`` (already including ``eps``, grad_nn.py:942) and ``sd``,
    each shaped ``[C, 1, ...]`` as the reference stores them (grad_nn.py:963).  The running
    buffers are not modified in place: like the reference (grad_nn.py:929-930) new arrays
    are produced; they are ``None`` when no update happens.
    """
    axis = (0,) + tuple(range(2, x.ndim))
    red_shape = (x.shape[0],) + x.shape[2:]
    cshape = (x.shape[1],) + (1,) * (x.ndim - 2)
    new_rm = new_rv = None
    if training:
        if prod(red_shape) == 1:  # grad_nn.py:899-904
            raise ValueError(f'Expected more than 1 value per channel when training, got input size {x.shape}')
        mean = np.mean(x, axis=axis)
        var = np.var(x, axis=axis)  # biased, two-pass
        if running_mean is not None and running_var is not None:
            m = prod(red_shape)
            unbiased = var * (m / (m - 1))  # ratio first, in Python float (grad_nn.py:928)
            new_rm = (1 - momentum) * running_mean + momentum * mean
            new_rv = (1 - momentum) * running_var + momentum * unbiased
    elif running_mean is not None and running_var is not None:
        mean, var = running_mean, running_var
    else:
        mean = np.mean(x, axis=axis)
        var = np.var(x, axis=axis)
    var = var + eps
    sd = np.sqrt(var)
    mean, var, sd = mean.reshape(cshape), var.reshape(cshape), sd.reshape(cshape)
    y = (x - mean) / sd
    if gamma is not None:
        y *= gamma.reshape(cshape)
    if beta is not None:
        y += beta.reshape(cshape)
    return y, {'mean': mean, 'var': var, 'sd': sd}, new_rm, new_rv


def batch_norm_backward(gy, x, gamma, saved, need=(True, True, True)):
    """Returns ``(dx, dgamma, dbeta)`` (grad_nn.py:966-989)."""
    axis = (0,) + tuple(range(2, x.ndim))
    m = prod((x.shape[0],) + x.shape[2:])
    mu, var, sd = saved['mean'], saved['var'], saved['sd']
    dx = dgamma = dbeta = None
    if need[2]:
        dbeta = gy.sum(axis)
    if need[1]:
        dgamma = (((x - mu) / sd) * gy).sum(axis)
    if need[0]:
        g = gy
        if gamma is not None:
            g = g * gamma.reshape(gamma.shape + (1,) * (x.ndim - 2))
        a = m * g - g.sum(axis=axis, keepdims=True)
        b = (x - mu) / var * (g * (x - mu)).sum(axis=axis, keepdims=True)
        dx = np.divide(a - b, m, dtype=g.dtype) / sd
    return dx, dgamma, dbeta
