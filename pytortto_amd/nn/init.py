"""Parameter initialisers (``src/tortto/nn/init.py``).  Values are drawn on the host with
``np.random`` in float64 and cast, as the reference does (init.py:6-17), so ``manual_seed(s)``
reproduces the reference's parameters bit for bit.  Filling a device tensor uploads the draw."""
import math

import numpy as np

from ..xparray import hiparray


def _assign(tensor, values):
    d = tensor.data
    values = values.astype(d.dtype)
    if d.__class__ is hiparray:
        d.set(values)
    else:
        d[...] = values
    return tensor


def _no_grad_uniform_(tensor, a, b):
    return _assign(tensor, np.random.uniform(low=a, high=b, size=tensor.data.shape))


def _no_grad_normal_(tensor, mean, std):
    return _assign(tensor, np.random.normal(loc=mean, scale=std, size=tensor.data.shape))


def _no_grad_fill_(tensor, val):
    tensor.data.fill(val)
    return tensor


def ones_(tensor):
    return _no_grad_fill_(tensor, 1.)


def zeros_(tensor):
    return _no_grad_fill_(tensor, 0.)


def constant_(tensor, val):
    return _no_grad_fill_(tensor, val)


def uniform_(tensor, a=0, b=1):
    return _no_grad_uniform_(tensor, a, b)


def normal_(tensor, mean=0., std=1.):
    return _no_grad_normal_(tensor, mean, std)


def _calculate_fan_in_and_fan_out(tensor):
    if tensor.dim() < 2:
        raise ValueError('Fan in and fan out can not be computed for tensor with fewer than 2 dimensions')
    receptive = 1
    for s in tensor.shape[2:]:
        receptive *= s
    return tensor.shape[1] * receptive, tensor.shape[0] * receptive


def _calculate_correct_fan(tensor, mode):
    mode = mode.lower()
    if mode not in ('fan_in', 'fan_out'):
        raise ValueError('Mode {} not supported, please use one of {}'.format(mode, ['fan_in', 'fan_out']))
    fan_in, fan_out = _calculate_fan_in_and_fan_out(tensor)
    return fan_in if mode == 'fan_in' else fan_out


def calculate_gain(nonlinearity, param=None):
    linear = ['linear', 'conv1d', 'conv2d', 'conv3d', 'conv_transpose1d', 'conv_transpose2d', 'conv_transpose3d']
    if nonlinearity in linear or nonlinearity == 'sigmoid':
        return 1
    if nonlinearity == 'tanh':
        return 5.0 / 3
    if nonlinearity == 'relu':
        return math.sqrt(2.0)
    if nonlinearity == 'leaky_relu':
        if param is None:
            slope = 0.01
        elif not isinstance(param, bool) and isinstance(param, int) or isinstance(param, float):
            slope = param
        else:
            raise ValueError('negative_slope {} not a valid number'.format(param))
        return math.sqrt(2.0 / (1 + slope ** 2))
    if nonlinearity == 'selu':
        return 3.0 / 4
    raise ValueError('Unsupported nonlinearity {}'.format(nonlinearity))


def kaiming_uniform_(tensor, a=0, mode='fan_in', nonlinearity='leaky_relu'):
    fan = _calculate_correct_fan(tensor, mode)
    std = calculate_gain(nonlinearity, a) / math.sqrt(fan)
    bound = math.sqrt(3.0) * std
    return _no_grad_uniform_(tensor, -bound, bound)
