"""``Sequential`` (``src/tortto/nn/modules/container.py:8-54``)."""
import operator
from collections import OrderedDict
from itertools import islice

from .module import Module


class Sequential(Module):
    def __init__(self, *args):
        super().__init__()
        if len(args) == 1 and isinstance(args[0], OrderedDict):
            for key, module in args[0].items():
                self.add_module(key, module)
        else:
            for idx, module in enumerate(args):
                self.add_module(str(idx), module)

    def _item(self, iterator, idx):
        size = len(self)
        idx = operator.index(idx)
        if not -size <= idx < size:
            raise IndexError('index {} is out of range'.format(idx))
        return next(islice(iterator, idx % size, None))

    def __getitem__(self, idx):
        if isinstance(idx, slice):
            return self.__class__(OrderedDict(list(self._modules.items())[idx]))
        return self._item(self._modules.values(), idx)

    def __setitem__(self, idx, module):
        return setattr(self, self._item(self._modules.keys(), idx), module)

    def __delitem__(self, idx):
        keys = list(self._modules.keys())[idx] if isinstance(idx, slice) else [self._item(self._modules.keys(), idx)]
        for key in keys:
            delattr(self, key)

    def __len__(self):
        return len(self._modules)

    def __iter__(self):
        return iter(self._modules.values())

    def forward(self, inpt):
        for module in self._modules.values():
            inpt = module(inpt)
        return inpt
