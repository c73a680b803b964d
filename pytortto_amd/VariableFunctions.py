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


# ---- the few array functions the classifier head of the ResNet examples uses ----------------------

def transpose(input, dim0, dim1):
    return input.transpose(dim0, dim1)


swapaxes = transpose
swapdims = transpose


def mean(input, dim=None, keepdim=False):
    return input.mean(dim, keepdim)


def flatten(x, start_dim=0, end_dim=-1):
    """Collapse dimensions ``start_dim`` .. ``end_dim`` (inclusive, negative values count from the
    end) into one (interface of VariableFunctions.py:108-127).  Returns ``x`` itself when nothing
    would change, else a view."""
    rank = len(x.shape)
    first, last = start_dim % rank if rank else 0, end_dim % rank if rank else 0
    if first > last:
        raise RuntimeError('flatten() has invalid args: start_dim cannot come after end_dim')
    if first == last:
        return x
    return x.view(x.shape[:first] + (-1,) + x.shape[last + 1:])


def mm(input, mat2):
    from .autograd.grad_fcn import Mm
    return Mm.apply(input, mat2)


def matmul(input, other):
    """VariableFunctions.py:365-396, for the cases the head needs: matrix @ matrix, and a tensor with
    leading dimensions @ matrix (collapsed to a matrix product and restored)."""
    from .autograd.grad_fcn import Mm, View
    if input.ndim == 0 or other.ndim == 0:
        raise RuntimeError(f'both arguments to matmul need to be at least 1D, but they are {input.ndim}D and '
                           f'{other.ndim}D')
    if input.ndim == 2 and other.ndim == 2:
        return Mm.apply(input, other)
    if other.ndim == 2 and input.ndim > 2:
        leading_dims = input.shape[:-1]
        input = View.apply(input, shape=(-1, input.shape[-1]))
        result = Mm.apply(input, other)
        return View.apply(result, shape=(*leading_dims, result.shape[-1]))
    raise NotImplementedError(f'matmul of a {input.ndim}D and a {other.ndim}D tensor is outside this build')
