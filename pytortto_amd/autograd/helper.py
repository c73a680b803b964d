"""The helpers of ``src/tortto/autograd/helper.py`` live with the node classes in ``function.py``;
this module keeps the reference's import path."""
from .function import build_links, get_data, inplace_precheck, inplace_update, toposort

__all__ = ['build_links', 'get_data', 'inplace_precheck', 'inplace_update', 'toposort']
