"""``Sequential``: modules applied one after the other (interface of
``src/tortto/nn/modules/container.py:8-54``).

Children live in ``Module._modules`` under string keys: ``'0', '1', ...`` for positional
arguments, the given names for a single ``OrderedDict`` argument.  Integer positions (negative
ones count from the end) and slices address them in registration order.
"""
from collections import OrderedDict

from .module import Module


class Sequential(Module):
    def __init__(self, *modules):
        super().__init__()
        named = modules[0].items() if len(modules) == 1 and isinstance(modules[0], OrderedDict) \
            else ((str(i), m) for i, m in enumerate(modules))
        for name, module in named:
            self.add_module(name, module)

    def _key_at(self, position):
        """Name of the child at an integer position."""
        keys = list(self._modules)
        position = position.__index__()
        if position < -len(keys) or position >= len(keys):
            raise IndexError(f'index {position} is out of range')
        return keys[position]

    def __len__(self):
        return len(self._modules)

    def __iter__(self):
        return iter(self._modules.values())

    def __getitem__(self, where):
        if isinstance(where, slice):
            picked = list(self._modules.items())[where]
            return type(self)(OrderedDict(picked))
        return self._modules[self._key_at(where)]

    def __setitem__(self, position, module):
        setattr(self, self._key_at(position), module)

    def __delitem__(self, where):
        doomed = list(self._modules)[where] if isinstance(where, slice) else [self._key_at(where)]
        for name in doomed:
            delattr(self, name)

    def forward(self, x):
        for stage in self:
            x = stage(x)
        return x
