"""``Optimizer`` base class (``src/tortto/optim/optimizer.py``): parameter groups, per-parameter
state, ``zero_grad``, ``state_dict`` / ``load_state_dict`` (state arrays are saved as NumPy
arrays and moved to the parameter's device on load, :68-79, :108-123)."""
import collections.abc
import warnings
from collections import defaultdict
from itertools import chain

import numpy as np

from ..tensor import Tensor
from ..xparray import hiparray


class _RequiredParameter:
    def __repr__(self):
        return '<required parameter>'


required = _RequiredParameter()


class Optimizer:
    def __init__(self, params, defaults):
        self.defaults = defaults
        if isinstance(params, Tensor):
            raise TypeError('params argument given to the optimizer should be an iterable of Tensors or dicts, '
                            'but got ' + params.__class__.__name__)
        self.state = defaultdict(dict)
        self.param_groups = []
        param_groups = list(params)
        if len(param_groups) == 0:
            raise ValueError('optimizer got an empty parameter list')
        if not isinstance(param_groups[0], dict):
            param_groups = [{'params': param_groups}]
        for group in param_groups:
            self.add_param_group(group)

    def __getstate__(self):
        return {'defaults': self.defaults, 'state': self.state, 'param_groups': self.param_groups}

    def __setstate__(self, state):
        self.__dict__.update(state)

    def __repr__(self):
        text = self.__class__.__name__ + ' ('
        for i, group in enumerate(self.param_groups):
            text += f'\nParameter Group {i}\n'
            for key in sorted(group.keys()):
                if key != 'params':
                    text += f'    {key}: {group[key]}\n'
        return text + ')'

    def state_dict(self):
        index_of = {}
        start = 0
        packed_groups = []
        for group in self.param_groups:
            packed = {k: v for k, v in group.items() if k != 'params'}
            index_of.update({id(p): i for i, p in enumerate(group['params'], start) if id(p) not in index_of})
            packed['params'] = [index_of[id(p)] for p in group['params']]
            start += len(packed['params'])
            packed_groups.append(packed)

        def to_host(entry):
            return {k: v.get() if v.__class__ is hiparray else v for k, v in entry.items()}

        packed_state = {(index_of[id(k)] if isinstance(k, Tensor) else k): to_host(v) for k, v in self.state.items()}
        return {'state': packed_state, 'param_groups': packed_groups}

    def load_state_dict(self, state_dict):
        state_dict = state_dict.copy()
        groups, saved_groups = self.param_groups, state_dict['param_groups']
        if len(groups) != len(saved_groups):
            raise ValueError('loaded state dict has a different number of parameter groups')
        if any(len(g['params']) != len(s['params']) for g, s in zip(groups, saved_groups)):
            raise ValueError("loaded state dict contains a parameter group that doesn't match the size of "
                             "optimizer's group")
        by_index = dict(zip(chain.from_iterable(g['params'] for g in saved_groups),
                            chain.from_iterable(g['params'] for g in groups)))

        def cast(param, value):
            if isinstance(value, np.ndarray):
                return hiparray(value) if param.data.__class__ is hiparray else value
            if isinstance(value, dict):
                return {k: cast(param, v) for k, v in value.items()}
            if isinstance(value, collections.abc.Iterable) and not isinstance(value, str):
                return type(value)(cast(param, v) for v in value)
            return value

        state = defaultdict(dict)
        for k, v in state_dict['state'].items():
            if k in by_index:
                state[by_index[k]] = cast(by_index[k], v)
            else:
                state[k] = v
        new_groups = []
        for group, saved in zip(groups, saved_groups):
            saved = dict(saved)
            saved['params'] = group['params']
            new_groups.append(saved)
        self.__setstate__({'state': state, 'param_groups': new_groups})

    def zero_grad(self):
        for group in self.param_groups:
            for p in group['params']:
                p.grad = None

    def step(self):
        raise NotImplementedError

    def add_param_group(self, param_group):
        assert isinstance(param_group, dict), 'param group must be a dict'
        params = param_group['params']
        if isinstance(params, Tensor):
            param_group['params'] = [params]
        elif isinstance(params, set):
            raise TypeError('optimizer parameters need to be organized in ordered collections, but the ordering of '
                            'tensors in sets will change between runs. Please use a list instead.')
        else:
            param_group['params'] = list(params)
        for param in param_group['params']:
            if not isinstance(param, Tensor):
                raise TypeError('optimizer can only optimize Tensors, but one of the params is ' +
                                param.__class__.__name__)
            if not param.is_leaf:
                raise ValueError("can't optimize a non-leaf Tensor")
        for name, default in self.defaults.items():
            if default is required and name not in param_group:
                raise ValueError("parameter group didn't specify a value of required optimization parameter " + name)
            param_group.setdefault(name, default)
        params = param_group['params']
        if len(params) != len(set(params)):
            warnings.warn('optimizer contains a parameter group with duplicate parameters.', stacklevel=3)
        seen = set()
        for group in self.param_groups:
            seen.update(group['params'])
        if not seen.isdisjoint(param_group['params']):
            raise ValueError('some parameters appear in more than one parameter group')
        self.param_groups.append(param_group)
