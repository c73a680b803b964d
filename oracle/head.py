"""The classifier head restated from the reference -- TEST INFRASTRUCTURE ONLY.

``mean_*`` follows ``Mean`` (src/tortto/autograd/grad_fcn.py:1058-1093), ``mm_*`` follows ``Mm``
(:907-932), ``linear_*`` composes them as ``F.linear`` does (src/tortto/nn/functional.py:54-63:
``matmul(input, weight.T) + bias``), ``log_softmax_*`` follows ``LogSoftmax``
(src/tortto/autograd/grad_nn.py:373-392) and ``nll_loss_*`` follows ``NllLoss`` (:287-349).

Pinned by (tests/test_oracle_head.py): torch CPU ``mean`` / ``F.linear`` / ``F.log_softmax`` /
``F.nll_loss`` with autograd (weights, ``ignore_index``, all three reductions), and closed forms
(rows of exp(log_softmax) sum to 1, its gradient rows sum to 0 for a constant upstream row, the
mean's gradient is g / count everywhere, loss of a one-hot-certain prediction is 0).
"""
import numpy as np


def mean_forward(x, dim=None, keepdim=False):
    return np.mean(x, axis=dim, keepdims=keepdim)                                   # :1066


def mean_backward(g, x_shape, dim=None, keepdim=False):
    if dim is None:                                                                  # :1079-1082
        return np.broadcast_to(np.divide(g, int(np.prod(x_shape)), dtype=g.dtype), x_shape).copy()
    if not isinstance(dim, tuple):
        dim = (dim,)
    if not keepdim:
        g = np.expand_dims(g, dim)
    count = 1
    for i in dim:
        count *= x_shape[i]
    return np.broadcast_to(np.divide(g, count, dtype=g.dtype), x_shape).copy()       # :1084-1093


def mm_forward(a, b):
    return a @ b                                                                     # :916


def mm_backward(g, a, b):
    return g @ b.T, a.T @ g                                                          # :927-930


def linear_forward(x, w, b=None):
    y = mm_forward(x, w.T)
    return y if b is None else y + b


def linear_backward(g, x, w, has_bias=True):
    """(dx, dw, db): ``Add`` hands g to both inputs (the bias sums it over rows), ``Mm`` gives
    g @ (w.T).T and x.T @ g, and ``Transpose`` turns the latter back into the weight's layout."""
    dx, dwt = mm_backward(g, x, w.T)
    return dx, dwt.T, (g.sum(0) if has_bias else None)


def log_softmax_forward(x, dim=-1):
    aug = x - np.max(x, axis=dim, keepdims=True)                                     # :379
    return aug - np.log(np.sum(np.exp(aug), axis=dim, keepdims=True))                # :380-381


def log_softmax_backward(g, y, dim=-1):
    return g - g.sum(axis=dim, keepdims=True) * np.exp(y)                            # :390


def _nll_weights(target, weight, ignore_index):
    w = None
    if weight is not None:                                                           # :299-305
        w = weight[target]
        if ignore_index >= 0:
            w = w * (target != ignore_index)
    elif ignore_index >= 0:
        w = target != ignore_index
    return w


def nll_loss_forward(logp, target, weight=None, ignore_index=-100, reduction='mean'):
    """(loss, N) for logp [N, C] and target [N]; N is the divisor of the mean (else None)."""
    w = _nll_weights(target, weight, ignore_index)
    y = -logp[np.arange(target.shape[0]), target]                                    # :306-308
    if w is not None:
        y = y * w
    count = None
    if reduction == 'sum':
        y = y.sum()
    elif reduction == 'mean':
        if w is None:                                                                # :313-319
            count = y.size
            y = y.mean()
        else:
            count = np.count_nonzero(w)
            y = np.divide(y.sum(), count, dtype=logp.dtype)
    elif reduction != 'none':
        raise ValueError(f'{reduction} is not a valid value for reduction')
    return y, count


def nll_loss_backward(g, logp_shape, target, weight=None, ignore_index=-100, reduction='mean', count=None):
    w = _nll_weights(target, weight, ignore_index)
    if reduction == 'mean':
        g = g / count                                                                # :343-344
    grad = np.zeros(logp_shape, dtype=np.result_type(g, np.float32) if np.ndim(g) else np.float32)
    grad[np.arange(target.shape[0]), target] = -g if w is None else -g * w          # :346-347
    return grad
