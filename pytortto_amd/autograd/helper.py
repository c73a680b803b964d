"""Autograd helpers with the reference's contracts (``src/tortto/autograd/helper.py``)."""
from .grad_mode import is_grad_enabled


def inplace_precheck(t):
    """helper.py:5-7"""
    if is_grad_enabled() and t.requires_grad and t.grad_fn is None:
        raise RuntimeError('a leaf Variable that requires grad is being used in an in-place operation.')


def inplace_update(t, grad_fn):
    """helper.py:10-16: bump the shared version counter and re-point the tensor at ``grad_fn``."""
    t.data._version[0] += 1
    t._output_idx = 0
    t.requires_grad = grad_fn.requires_grad
    if grad_fn.requires_grad:
        t.grad_fn = grad_fn
    return t


def get_data(pair):
    """helper.py:19-29: hand back the saved tensor's array unless it was modified in place."""
    if pair is None:
        return None
    t, version = pair
    if t._version != version:
        origin = '' if t.grad_fn is None else f', which is the output of {t.grad_fn.__class__.__name__},'
        raise RuntimeError(f'one of the variables needed for gradient computation has been modified '
                           f'by an inplace operation: [shape: {t.shape}]{origin} is at version '
                           f'{t._version}; expected version {version} instead.')
    return t.data


def build_links(data, grad_fn, copy=False, _output_idx=0):
    """helper.py:45-50: wrap a forward result, attached to ``grad_fn`` when gradients flow."""
    from ..tensor import Tensor
    dtype = getattr(data, 'dtype', None)
    if grad_fn.requires_grad and is_grad_enabled():
        return Tensor(data, requires_grad=True, dtype=dtype, copy=copy, grad_fn=grad_fn, _output_idx=_output_idx)
    return Tensor(data, dtype=dtype, copy=copy)


def toposort(end_node):
    """helper.py:53-82: yield nodes so that a node comes after everything that feeds gradient
    into it; nodes whose other consumers are not part of this backward pass are taken from
    the ``waiting`` set once nothing else is ready."""
    ready = [end_node]
    waiting = set()
    while ready or waiting:
        node = ready.pop() if ready else waiting.pop()
        yield node
        for fn, _ in node.next_functions or ():
            if fn is None:
                continue
            fn.prev_function_counts -= 1
            if fn.prev_function_counts == 0:
                ready.append(fn)
                waiting.discard(fn)
            else:
                waiting.add(fn)
