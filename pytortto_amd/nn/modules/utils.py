"""Argument helpers of the modules (``src/tortto/nn/modules/utils.py``)."""


def _ntuple(n):
    """int -> n-tuple of it; a sequence -> its first n entries."""
    def parse(x):
        return tuple(x[:n]) if hasattr(x, '__iter__') else (x,) * n
    return parse


_single, _pair = _ntuple(1), _ntuple(2)
