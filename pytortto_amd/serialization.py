"""``tt.save`` / ``tt.load`` (``src/tortto/serialization.py:1-12``): the checkpoint wire format is a
``.npy`` file holding one pickled object, the dict ``{'data': obj}``.  ``state_dict()`` entries are
always host NumPy arrays (nn/modules/module.py:109-122), so a checkpoint written from device
modules loads anywhere."""
import numpy as np


def save(obj, f, allow_pickle=True):
    np.save(f, {'data': obj}, allow_pickle=allow_pickle)


def load(file, mmap_mode=None, allow_pickle=True, encoding='ASCII'):
    return np.load(file, mmap_mode=mmap_mode, allow_pickle=allow_pickle, encoding=encoding).item()['data']
