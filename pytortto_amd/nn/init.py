"""Parameter initialisers with the names and formulas of ``src/tortto/nn/init.py``.  Every draw
comes from NumPy's global legacy stream in float64 and is then cast to the parameter's dtype
(init.py:6-17) -- so after ``manual_seed(s)`` the parameters equal the reference's bit for bit.
A device tensor receives the host draw by upload."""
import math

import numpy as np

from ..xparray import hiparray

# gain of a nonlinearity = the factor that keeps the variance of its output (init.py:58-88)
_UNIT_GAIN = {'linear', 'conv1d', 'conv2d', 'conv3d', 'conv_transpose1d', 'conv_transpose2d', 'conv_transpose3d',
              'sigmoid'}
_FIXED_GAIN = {'tanh': 5.0 / 3, 'relu': math.sqrt(2.0), 'selu': 3.0 / 4}


def _store(tensor, values):
    target = tensor.data
    values = values.astype(target.dtype)
    if target.__class__ is hiparray:
        target.set(values)
    else:
        target[...] = values
    return tensor


def uniform_(tensor, a=0, b=1):
    return _store(tensor, np.random.uniform(low=a, high=b, size=tensor.data.shape))


def normal_(tensor, mean=0., std=1.):
    return _store(tensor, np.random.normal(loc=mean, scale=std, size=tensor.data.shape))


def constant_(tensor, val):
    tensor.data.fill(val)
    return tensor


def ones_(tensor):
    return constant_(tensor, 1.)


def zeros_(tensor):
    return constant_(tensor, 0.)


_no_grad_uniform_, _no_grad_normal_, _no_grad_fill_ = uniform_, normal_, constant_


def _calculate_fan_in_and_fan_out(tensor):
    """(inputs per output unit, outputs per input unit): shape[1] resp. shape[0] times the
    receptive field shape[2:] (init.py:41-52)."""
    if tensor.dim() < 2:
        raise ValueError('Fan in and fan out can not be computed for tensor with fewer than 2 dimensions')
    field = math.prod(tensor.shape[2:])
    return tensor.shape[1] * field, tensor.shape[0] * field


def _calculate_correct_fan(tensor, mode):
    fans = dict(zip(('fan_in', 'fan_out'), _calculate_fan_in_and_fan_out(tensor)))
    if mode.lower() not in fans:
        raise ValueError('Mode {} not supported, please use one of {}'.format(mode.lower(), list(fans)))
    return fans[mode.lower()]


def calculate_gain(nonlinearity, param=None):
    if nonlinearity in _UNIT_GAIN:
        return 1
    if nonlinearity in _FIXED_GAIN:
        return _FIXED_GAIN[nonlinearity]
    if nonlinearity != 'leaky_relu':
        raise ValueError('Unsupported nonlinearity {}'.format(nonlinearity))
    slope = 0.01 if param is None else param
    if isinstance(slope, bool) or not isinstance(slope, (int, float)):
        raise ValueError('negative_slope {} not a valid number'.format(param))
    return math.sqrt(2.0 / (1 + slope ** 2))


def kaiming_uniform_(tensor, a=0, mode='fan_in', nonlinearity='leaky_relu'):
    """U(-b, b) with b = gain * sqrt(3 / fan) (init.py:91-96)."""
    std = calculate_gain(nonlinearity, a) / math.sqrt(_calculate_correct_fan(tensor, mode))
    return uniform_(tensor, -math.sqrt(3.0) * std, math.sqrt(3.0) * std)
