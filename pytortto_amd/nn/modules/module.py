"""``Module`` (``src/tortto/nn/modules/module.py``): parameter/buffer/submodule registries,
``cuda()`` / ``cpu()`` re-wrapping every parameter as a new ``Parameter`` (:351-385),
``state_dict`` that always yields NumPy arrays (:108-131), ``load_state_dict`` (:41-106)."""
import itertools
from collections import OrderedDict, namedtuple

import numpy as np

from ...autograd.grad_mode import no_grad
from ...tensor import Tensor
from ...VariableFunctions import tensor as _tensor
from ...xparray import hiparray
from ..parameter import Parameter


class _IncompatibleKeys(namedtuple('IncompatibleKeys', ['missing_keys', 'unexpected_keys'])):
    def __repr__(self):
        if not self.missing_keys and not self.unexpected_keys:
            return '<All keys matched successfully>'
        return super().__repr__()

    __str__ = __repr__


def _indent(text, spaces):
    lines = text.split('\n')
    if len(lines) == 1:
        return text
    return lines[0] + '\n' + '\n'.join(' ' * spaces + l for l in lines[1:])


def _check_name(kind, name, owner, registry):
    if not isinstance(name, str):
        raise TypeError('{} name should be a string. Got {}'.format(kind, type(name)))
    if '.' in name:
        raise KeyError('{} name can\'t contain "."'.format(kind))
    if name == '':
        raise KeyError('{} name can\'t be empty string ""'.format(kind))
    if hasattr(owner, name) and name not in registry:
        raise KeyError("attribute '{}' already exists".format(name))


class Module:
    def __init__(self):
        self.training = True
        self._parameters = OrderedDict()
        self._modules = OrderedDict()
        self._buffers = OrderedDict()

    # ---- registration ------------------------------------------------------------------------
    def register_buffer(self, name, tensor):
        if '_buffers' not in self.__dict__:
            raise AttributeError('cannot assign buffer before Module.__init__() call')
        _check_name('buffer', name, self, self._buffers)
        if tensor is not None and not isinstance(tensor, Tensor):
            raise TypeError("cannot assign '{}' object to buffer '{}' (tortto.Tensor or None required)"
                            .format(type(tensor), name))
        self._buffers[name] = tensor

    def register_parameter(self, name, param):
        if '_parameters' not in self.__dict__:
            raise AttributeError('cannot assign parameter before Module.__init__() call')
        _check_name('parameter', name, self, self._parameters)
        if param is None:
            self._parameters[name] = None
        elif not isinstance(param, Parameter):
            raise TypeError("cannot assign '{}' object to parameter '{}' (tortto.nn.Parameter or None required)"
                            .format(type(param), name))
        elif param.grad_fn:
            raise ValueError("Cannot assign non-leaf Tensor to parameter '{0}'. Model parameters must be created "
                             "explicitly. To express '{0}' as a function of another Tensor, compute the value in "
                             "the forward() method.".format(name))
        else:
            self._parameters[name] = param

    def add_module(self, name, module):
        if not isinstance(module, Module) and module is not None:
            raise TypeError('{} is not a Module subclass'.format(type(module)))
        _check_name('module', name, self, self._modules)
        self._modules[name] = module

    def __getattr__(self, name):
        for registry in ('_parameters', '_buffers', '_modules'):
            table = self.__dict__.get(registry)
            if table is not None and name in table:
                return table[name]
        raise AttributeError("'{}' object has no attribute '{}'".format(type(self).__name__, name))

    def __setattr__(self, name, value):
        if isinstance(value, Parameter):
            self._parameters[name] = value
        elif isinstance(value, Module):
            self._modules[name] = value
        else:
            buffers = self.__dict__.get('_buffers')
            if buffers is not None and name in buffers:
                if value is not None and not isinstance(value, Tensor):
                    raise TypeError("cannot assign '{}' as buffer '{}' (tortto.Tensor or None expected)"
                                    .format(type(value), name))
                buffers[name] = value
            else:
                object.__setattr__(self, name, value)

    def __delattr__(self, name):
        for table in (self._parameters, self._buffers, self._modules):
            if name in table:
                del table[name]
                return
        object.__delattr__(self, name)

    # ---- calling -----------------------------------------------------------------------------
    def forward(self, *input, **kwargs):
        raise NotImplementedError

    def _call_impl(self, *input, **kwargs):
        return self.forward(*input, **kwargs)

    __call__ = _call_impl

    # ---- traversal ---------------------------------------------------------------------------
    def named_modules(self, memo=None, prefix=''):
        memo = set() if memo is None else memo
        if self in memo:
            return
        memo.add(self)
        yield prefix, self
        for name, module in self._modules.items():
            if module is not None:
                yield from module.named_modules(memo, prefix + ('.' if prefix else '') + name)

    def modules(self):
        for _, module in self.named_modules():
            yield module

    def named_children(self):
        seen = set()
        for name, module in self._modules.items():
            if module is not None and module not in seen:
                seen.add(module)
                yield name, module

    def children(self):
        for _, module in self.named_children():
            yield module

    def _named_members(self, get_members, prefix='', recurse=True):
        seen = set()
        modules = self.named_modules(prefix=prefix) if recurse else [(prefix, self)]
        for mod_prefix, module in modules:
            for k, v in get_members(module):
                if v is None or v in seen:
                    continue
                seen.add(v)
                yield mod_prefix + ('.' if mod_prefix else '') + k, v

    def named_parameters(self, prefix='', recurse=True):
        yield from self._named_members(lambda m: m._parameters.items(), prefix=prefix, recurse=recurse)

    def parameters(self, recurse=True):
        for _, p in self.named_parameters(recurse=recurse):
            yield p

    def named_buffers(self, prefix='', recurse=True):
        yield from self._named_members(lambda m: m._buffers.items(), prefix=prefix, recurse=recurse)

    def buffers(self, recurse=True):
        for _, b in self.named_buffers(recurse=recurse):
            yield b

    # ---- modes -------------------------------------------------------------------------------
    def train(self, mode=True):
        self.training = mode
        for module in self.children():
            module.train(mode)
        return self

    def eval(self):
        return self.train(False)

    def requires_grad_(self, requires_grad=True):
        for p in self.parameters():
            p.requires_grad_(requires_grad)
        return self

    def zero_grad(self):
        for p in self.parameters():
            p.grad = None

    def apply(self, fn):
        for module in self.children():
            module.apply(fn)
        fn(self)
        return self

    # ---- device movement ---------------------------------------------------------------------
    def cuda(self):
        return self._apply(lambda t: t.cuda())

    def cpu(self):
        return self._apply(lambda t: t.cpu())

    def _apply(self, fn):
        for module in self.children():
            module._apply(fn)
        for key, param in self._parameters.items():
            if param is None:
                continue
            with no_grad():
                moved = fn(param)
            new_param = Parameter(moved, param.requires_grad)
            self._parameters[key] = new_param
            if param.grad is not None:
                with no_grad():
                    new_param.grad = fn(_tensor(param.grad, copy=False)).data
        for key, buf in self._buffers.items():
            if buf is not None:
                self._buffers[key] = fn(buf)
        return self

    # ---- checkpoints ---------------------------------------------------------------------------
    def _save_to_state_dict(self, destination, prefix):
        for name, t in itertools.chain(self._parameters.items(), self._buffers.items()):
            if t is not None:
                d = t.data
                destination[prefix + name] = d.get() if d.__class__ is hiparray else d.view(np.ndarray)

    def state_dict(self, destination=None, prefix=''):
        if destination is None:
            destination = OrderedDict()
        self._save_to_state_dict(destination, prefix)
        for name, module in self._modules.items():
            if module is not None:
                module.state_dict(destination, prefix + name + '.')
        return destination

    def _check_shape_mismatch(self, input_param, param):
        return input_param.shape != param.shape

    def _load_from_state_dict(self, state_dict, prefix, strict, missing_keys, unexpected_keys, error_msgs):
        local = {k: v for k, v in itertools.chain(self._parameters.items(), self._buffers.items()) if v is not None}
        for name, param in local.items():
            key = prefix + name
            if key in state_dict:
                value = state_dict[key]
                if self._check_shape_mismatch(value, param):
                    error_msgs.append('size mismatch for {}: copying a param with shape {} from checkpoint, '
                                      'the shape in current model is {}.'.format(key, value.shape, param.shape))
                    continue
                try:
                    with no_grad():
                        param.copy_(value)
                except Exception as ex:
                    error_msgs.append('While copying the parameter named "{}", whose dimensions in the model are {} '
                                      'and whose dimensions in the checkpoint are {}, an exception occurred : {}.'
                                      .format(key, param.size(), value.shape, ex.args))
            elif strict:
                missing_keys.append(key)
        if strict:
            for key in state_dict.keys():
                if key.startswith(prefix):
                    head = key[len(prefix):].split('.', 1)[0]
                    if head not in self._modules and head not in local:
                        unexpected_keys.append(key)

    def load_state_dict(self, state_dict, strict=True):
        missing, unexpected, errors = [], [], []
        state_dict = state_dict.copy()

        def load(module, prefix=''):
            module._load_from_state_dict(state_dict, prefix, True, missing, unexpected, errors)
            for name, child in module._modules.items():
                if child is not None:
                    load(child, prefix + name + '.')

        load(self)
        if strict:
            if unexpected:
                errors.insert(0, 'Unexpected key(s) in state_dict: {}. '.format(
                    ', '.join('"{}"'.format(k) for k in unexpected)))
            if missing:
                errors.insert(0, 'Missing key(s) in state_dict: {}. '.format(
                    ', '.join('"{}"'.format(k) for k in missing)))
        if errors:
            raise RuntimeError('Error(s) in loading state_dict for {}:\n\t{}'.format(
                self.__class__.__name__, '\n\t'.join(errors)))
        return _IncompatibleKeys(missing, unexpected)

    # ---- printing ------------------------------------------------------------------------------
    def _get_name(self):
        return self.__class__.__name__

    def extra_repr(self):
        return ''

    def __repr__(self):
        extra = self.extra_repr()
        extra_lines = extra.split('\n') if extra else []
        child_lines = ['(' + k + '): ' + _indent(repr(m), 2) for k, m in self._modules.items()]
        lines = extra_lines + child_lines
        text = self._get_name() + '('
        if lines:
            if len(extra_lines) == 1 and not child_lines:
                text += extra_lines[0]
            else:
                text += '\n  ' + '\n  '.join(lines) + '\n'
        return text + ')'
