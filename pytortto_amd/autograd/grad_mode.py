"""Gradient-mode switches (``src/tortto/autograd/grad_mode.py``): ``no_grad`` / ``enable_grad`` /
``set_grad_enabled`` usable as context managers and as decorators."""
import functools

_enabled = True


def is_grad_enabled():
    return _enabled


class set_grad_enabled:
    def __init__(self, mode):
        global _enabled
        self.prev = _enabled
        self.mode = bool(mode)
        _enabled = self.mode      # takes effect immediately when used as a plain call

    def __enter__(self):
        global _enabled
        _enabled = self.mode

    def __exit__(self, *exc):
        global _enabled
        _enabled = self.prev
        return False


class _GradSwitch:
    _mode = True

    def __enter__(self):
        global _enabled
        self.prev = _enabled
        _enabled = self._mode

    def __exit__(self, *exc):
        global _enabled
        _enabled = self.prev
        return False

    def __call__(self, fn):
        @functools.wraps(fn)
        def wrapped(*args, **kwargs):
            with self.__class__():
                return fn(*args, **kwargs)
        return wrapped


class no_grad(_GradSwitch):
    _mode = False


class enable_grad(_GradSwitch):
    _mode = True
