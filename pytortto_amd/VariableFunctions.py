"""Creation functions (``src/tortto/VariableFunctions.py``): all draw from / allocate with NumPy on
the host, exactly as the reference does; ``manual_seed`` seeds NumPy's legacy global stream."""
import warnings

import numpy as np

from .tensor import Tensor, float32


def manual_seed(seed):
    np.random.seed(seed)


def _shape(shape):
    return shape[0] if hasattr(shape[0], '__iter__') else shape


def empty(*shape, dtype=None, requires_grad=False):
    dtype = dtype or float32
    return Tensor(np.empty(_shape(shape), dtype=dtype), dtype=dtype, copy=False, requires_grad=requires_grad)


def zeros(*shape, dtype=None, requires_grad=False):
    dtype = dtype or float32
    return Tensor(np.zeros(_shape(shape), dtype=dtype), dtype=dtype, copy=False, requires_grad=requires_grad)


def ones(*shape, dtype=None, requires_grad=False):
    dtype = dtype or float32
    return Tensor(np.ones(_shape(shape), dtype=dtype), dtype=dtype, copy=False, requires_grad=requires_grad)


def randn(*shape, dtype=None, requires_grad=False):
    return Tensor(np.random.randn(*_shape(shape)), dtype=dtype, copy=False, requires_grad=requires_grad)


def tensor(data, requires_grad=False, dtype=None, copy=True, **kwargs):
    if isinstance(data, Tensor):
        warnings.warn('Input is already a tensor, returning without deepcopy', UserWarning)
        return data
    if dtype is None:
        dtype = getattr(data, 'dtype', float32)
    return Tensor(data, requires_grad=requires_grad, dtype=dtype, copy=copy, **kwargs)
