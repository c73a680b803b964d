"""``Tensor`` with the part of the reference's API the convolution / BatchNorm path sits behind
(``src/tortto/tensor.py``): data/grad/grad_fn/requires_grad/_version, ``.cuda()`` / ``.cpu()`` as
differentiable ``ToCopy`` nodes, ``backward()``.  ``data`` is an ``nparray`` (host) or a
``hiparray`` (device); ``grad`` is a raw array of the same kind."""
import numpy as np

from . import xparray
from .xparray import hiparray, nparray

float16 = np.float16
float32 = np.float32
float64 = np.float64
int16 = np.int16
int32 = np.int32
int64 = np.int64

_default_dtypes = {np.int64, np.float32, np.complex64, np.bool_}


class Tensor:
    def __init__(self, data, requires_grad=False, dtype=None, copy=True, **kwargs):
        if dtype is None:
            dtype = float32
        if data.__class__ is hiparray:
            self.data = hiparray(data, dtype=dtype)
        else:
            self.data = nparray(data, dtype=dtype, copy=copy)
        self.grad = None
        self.grad_fn = kwargs.get('grad_fn')
        self._requires_grad = requires_grad
        self._output_idx = kwargs.get('_output_idx')

    # ---- properties --------------------------------------------------------------------------
    @property
    def _version(self):
        return self.data._version[0]

    @property
    def requires_grad(self):
        return self._requires_grad

    @requires_grad.setter
    def requires_grad(self, val):
        if val.__class__ is not bool:
            raise RuntimeError('requires_grad must be a bool')
        if val and not issubclass(self.data.dtype.type, (np.floating, np.complexfloating)):
            raise RuntimeError('only Tensors of floating point and complex dtype can require gradients')
        self._requires_grad = val

    def requires_grad_(self, val=True):
        self.requires_grad = val

    @property
    def is_cuda(self):
        return self.data.__class__ is hiparray

    @property
    def device(self):
        return self.data.device if self.data.__class__ is hiparray else 'cpu'

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def shape(self):
        return self.data.shape

    @property
    def is_leaf(self):
        return self.grad_fn is None

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def itemsize(self):
        return self.data.itemsize

    @property
    def strides(self):
        return self.data.strides

    def __len__(self):
        return self.shape[0]

    def __hash__(self):
        return id(self)

    def __repr__(self):
        dev = f", device='{self.device}'" if self.device != 'cpu' else ''
        dt = f', dtype={self.dtype}' if self.dtype.type not in _default_dtypes else ''
        fn = f', grad_fn=<{self.grad_fn.__class__.__name__}>' if self.grad_fn else ''
        rg = ', requires_grad=True' if self.requires_grad and not self.grad_fn else ''
        host = self.data.get() if self.data.__class__ is hiparray else self.data
        body = np.array2string(np.asarray(host), separator=', ', precision=4).replace('\n', '\n' + ' ' * 7)
        return f'tensor({body}{dev}{dt}{fn}{rg})'

    # ---- shape queries -------------------------------------------------------------------------
    def dim(self):
        return self.ndim

    def size(self, dim=None):
        if dim is None:
            return self.shape
        n = len(self.shape)
        if dim < -n or dim > n - 1:
            raise IndexError(f'Dimension out of range (expected to be in range of [-{n}, {n - 1}], but got {dim})')
        return self.shape[dim]

    def numel(self):
        return self.data.size

    def item(self):
        return self.data.item()

    def data_ptr(self):
        return self.data.ptr if self.data.__class__ is hiparray else self.data.ctypes.data

    # ---- device movement ------------------------------------------------------------------------
    def cuda(self):
        from .autograd.grad_fcn import ToCopy
        return ToCopy.apply(self, target_device='cuda')

    def cpu(self):
        from .autograd.grad_fcn import ToCopy
        return ToCopy.apply(self, target_device='cpu')

    def detach(self):
        return Tensor(self.data, requires_grad=False, dtype=self.data.dtype, copy=False)

    def numpy(self):
        if self.data.__class__ is hiparray:
            raise TypeError(f"can't convert {self.device} device type tensor to numpy. "
                            f"Use Tensor.cpu() to copy the tensor to host memory first.")
        if self.requires_grad:
            raise RuntimeError("Can't call numpy() on Tensor that requires grad. "
                               "Use tensor.detach().numpy() instead.")
        return self.data

    def copy_(self, src):
        """In-place copy of values from a tensor or array of the same shape (used by
        ``load_state_dict``, nn/modules/module.py:56-57)."""
        from .autograd.helper import inplace_precheck
        inplace_precheck(self)
        sd = src.data if isinstance(src, Tensor) else src
        if sd.__class__ is hiparray:
            sd = sd.get()
        if self.data.__class__ is hiparray:
            self.data.set(sd)
        else:
            self.data[...] = sd
        self.data._version[0] += 1
        return self

    def __add__(self, other):
        from .autograd.grad_fcn import Add
        return Add.apply(self, other)

    def __matmul__(self, other):
        from .VariableFunctions import matmul
        return matmul(self, other)

    @property
    def T(self):
        """tensor.py:56-60."""
        if self.ndim != 2:
            raise RuntimeError(f'x.T expects a tensor with 2 dimensions, but self is {self.ndim}D')
        return self.transpose(1, 0)

    def transpose(self, dim0, dim1):
        from .autograd.grad_fcn import Transpose
        return Transpose.apply(self, dim0=dim0, dim1=dim1)

    swapaxes = transpose
    swapdims = transpose

    def mean(self, dim=None, keepdim=False):
        from .autograd.grad_fcn import Mean
        return Mean.apply(self, dim=dim, keepdim=keepdim)

    def view(self, *shape):
        """tensor.py:408-411."""
        from .autograd.grad_fcn import View
        if shape[0].__class__ is not int:
            shape = shape[0]
        return View.apply(self, shape=tuple(shape))

    def flatten(self, start_dim=0, end_dim=-1):
        from .VariableFunctions import flatten
        return flatten(self, start_dim, end_dim)

    # ---- autograd ------------------------------------------------------------------------------
    def backward(self, gradient=None):
        """tensor.py:568-613."""
        from .autograd.function import AccumulateGrad
        from .autograd.helper import toposort
        if not self.requires_grad:
            raise RuntimeError('element 0 of tensors does not require grad and does not have a grad_fn')
        on_device = self.data.__class__ is hiparray
        if gradient is None:
            one = np.ones((1,) * self.data.ndim, dtype=self.data.dtype)
            gradient = hiparray(one) if on_device else one
        elif isinstance(gradient, Tensor):
            if gradient.device != self.device:
                raise RuntimeError(f'invalid gradient at index 0 - expected device {self.device} '
                                   f'but got {gradient.device}')
            gradient = gradient.data.copy() if on_device else gradient.data.copy().view(np.ndarray)
        if self.data.shape != gradient.shape:
            raise RuntimeError('grad can be implicitly created only for scalar outputs')
        if self.grad_fn:
            self.grad_fn.grad[self._output_idx] = gradient
            for node in toposort(self.grad_fn):
                grads = node.apply(*node.grad)
                for i, (fn, idx) in enumerate(node.next_functions):   # empty for leaf accumulators
                    g = grads[i]
                    if g is None:
                        continue
                    if fn.grad[idx] is None:
                        fn.grad[idx] = g if g.__class__ is hiparray else np.ascontiguousarray(g)
                    elif fn.grad[idx].__class__ is hiparray and fn.grad[idx]._shared and g.__class__ is hiparray:
                        # the first arrival is an alias of somebody else's gradient (hiparray.alias):
                        # the sum goes to a new array instead of copying it and adding in place
                        from . import ops
                        fn.grad[idx] = ops.add(fn.grad[idx], g)
                    else:
                        fn.grad[idx] += g
                node.clear()
        else:
            acc = AccumulateGrad()
            acc.variable = self
            acc.grad = (gradient,)
            acc.apply(*acc.grad)


class Parameter(Tensor):
    """``nn.Parameter`` (``src/tortto/nn/parameter.py``): a leaf tensor that asks for a gradient by
    default and adopts -- does not copy -- the array of the tensor it is made from."""

    def __init__(self, data=None, requires_grad=True, **kwargs):
        if data is not None and not isinstance(data, Tensor):
            raise TypeError(f'input must be Tensor, not {data.__class__.__name__}')
        array = None if data is None else data.data
        super().__init__(array, requires_grad=requires_grad, dtype=float32 if array is None else array.dtype,
                         copy=False)

    def __repr__(self):
        return 'Parameter containing:\n' + super().__repr__()
