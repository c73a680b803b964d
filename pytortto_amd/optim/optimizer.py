"""``Optimizer``: parameter groups with per-group hyper-parameters, per-parameter state,
``zero_grad`` and the ``state_dict`` layout of ``src/tortto/optim/optimizer.py`` (groups refer to
parameters by running index; state arrays are saved as host NumPy arrays, :68-79, and moved to
each parameter's device when loaded, :108-123)."""
import warnings
from collections import defaultdict

import numpy as np

from ..tensor import Tensor
from ..xparray import hiparray


class _RequiredParameter:
    """Marks a hyper-parameter that every group has to supply (``lr`` of SGD)."""

    def __repr__(self):
        return '<required parameter>'


required = _RequiredParameter()


def _to_host(value):
    return value.get() if value.__class__ is hiparray else value


def _like(param, value):
    """``value`` of a loaded checkpoint, with arrays placed where ``param`` lives."""
    if isinstance(value, np.ndarray):
        return hiparray(value) if param.data.__class__ is hiparray else value
    if isinstance(value, dict):
        return {k: _like(param, v) for k, v in value.items()}
    if isinstance(value, (list, tuple)):
        return type(value)(_like(param, v) for v in value)
    return value


class Optimizer:
    def __init__(self, params, defaults):
        if isinstance(params, Tensor):
            raise TypeError('params argument given to the optimizer should be an iterable of Tensors or dicts, '
                            'but got ' + params.__class__.__name__)
        self.defaults = defaults
        self.state = defaultdict(dict)
        self.param_groups = []
        groups = list(params)
        if not groups:
            raise ValueError('optimizer got an empty parameter list')
        if not isinstance(groups[0], dict):
            groups = [{'params': groups}]
        for group in groups:
            self.add_param_group(group)

    # ---- groups -------------------------------------------------------------------------------------
    def add_param_group(self, param_group):
        assert isinstance(param_group, dict), 'param group must be a dict'
        members = param_group['params']
        if isinstance(members, set):
            raise TypeError('optimizer parameters need to be organized in ordered collections, but the ordering of '
                            'tensors in sets will change between runs. Please use a list instead.')
        members = [members] if isinstance(members, Tensor) else list(members)
        for p in members:
            if not isinstance(p, Tensor):
                raise TypeError('optimizer can only optimize Tensors, but one of the params is ' +
                                p.__class__.__name__)
            if not p.is_leaf:
                raise ValueError("can't optimize a non-leaf Tensor")
        param_group['params'] = members
        for name, default in self.defaults.items():
            if default is required and name not in param_group:
                raise ValueError("parameter group didn't specify a value of required optimization parameter " + name)
            param_group.setdefault(name, default)
        if len(set(members)) != len(members):
            warnings.warn('optimizer contains a parameter group with duplicate parameters.', stacklevel=3)
        taken = {p for group in self.param_groups for p in group['params']}
        if taken & set(members):
            raise ValueError('some parameters appear in more than one parameter group')
        self.param_groups.append(param_group)

    def _with_grad(self):
        """(group, parameters of the group that received a gradient) for every group."""
        for group in self.param_groups:
            yield group, [p for p in group['params'] if p.grad is not None and p.grad.__class__ is not int]

    def zero_grad(self):
        for group in self.param_groups:
            for p in group['params']:
                p.grad = None

    def step(self):
        raise NotImplementedError

    # ---- (de)serialisation ---------------------------------------------------------------------------
    def __getstate__(self):
        return {'defaults': self.defaults, 'state': self.state, 'param_groups': self.param_groups}

    def __setstate__(self, state):
        self.__dict__.update(state)

    def state_dict(self):
        number = {}
        for group in self.param_groups:
            for p in group['params']:
                number.setdefault(id(p), len(number))
        groups = [{**{k: v for k, v in g.items() if k != 'params'}, 'params': [number[id(p)] for p in g['params']]}
                  for g in self.param_groups]
        state = {(number[id(k)] if isinstance(k, Tensor) else k): {name: _to_host(v) for name, v in entry.items()}
                 for k, entry in self.state.items()}
        return {'state': state, 'param_groups': groups}

    def load_state_dict(self, state_dict):
        saved_groups = state_dict['param_groups']
        if len(saved_groups) != len(self.param_groups):
            raise ValueError('loaded state dict has a different number of parameter groups')
        for mine, saved in zip(self.param_groups, saved_groups):
            if len(mine['params']) != len(saved['params']):
                raise ValueError("loaded state dict contains a parameter group that doesn't match the size of "
                                 "optimizer's group")
        owner = {index: p for mine, saved in zip(self.param_groups, saved_groups)
                 for index, p in zip(saved['params'], mine['params'])}
        state = defaultdict(dict)
        for key, entry in state_dict['state'].items():
            if key in owner:
                state[owner[key]] = _like(owner[key], entry)
            else:
                state[key] = entry
        groups = [{**saved, 'params': mine['params']} for mine, saved in zip(self.param_groups, saved_groups)]
        self.__setstate__({'state': state, 'param_groups': groups})

    def __repr__(self):
        lines = [self.__class__.__name__ + ' (']
        for i, group in enumerate(self.param_groups):
            lines.append(f'Parameter Group {i}')
            lines += [f'    {key}: {group[key]}' for key in sorted(group) if key != 'params']
        return '\n'.join(lines) + '\n)'
