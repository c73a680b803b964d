"""ctypes binding of ``libtortto_hip.so`` -- the only door from Python to the GPU.

The prototypes below restate ``include/tortto_hip.h``.  The library is loaded on first use
(``lib()``); if it has not been built, or no MI355X is visible, that raises -- there is no
CPU fallback behind this module.
"""
import ctypes
import os
import threading
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_void_p

from ._paths import LIB_PATH

_P = c_void_p
_I = c_int

# name -> argument types (every function returns int, except tt_last_error)
PROTOTYPES = {
    'tt_init': [_I],
    'tt_device_info': [c_char_p, _I, POINTER(c_int), POINTER(c_int), POINTER(c_int), POINTER(c_size_t)],
    'tt_malloc': [POINTER(c_void_p), c_size_t],
    'tt_free': [_P],
    'tt_empty_cache': [],
    'tt_mem_stats': [POINTER(c_size_t), POINTER(c_size_t), POINTER(c_size_t)],
    'tt_memcpy_h2d': [_P, _P, c_size_t],
    'tt_memcpy_d2h': [_P, _P, c_size_t],
    'tt_memcpy_d2d': [_P, _P, c_size_t],
    'tt_memset': [_P, _I, c_size_t],
    'tt_sync': [],
    'tt_set_conv_math': [_I],
    'tt_get_conv_math': [POINTER(c_int)],
    'tt_set_conv_dense_cell_min_tiles': [_I],
    'tt_event_create': [POINTER(c_void_p)],
    'tt_event_record': [_P],
    'tt_event_elapsed_ms': [_P, _P, POINTER(c_float)],
    'tt_event_destroy': [_P],
    'tt_profile_enable': [_I],
    'tt_profile_read': [_I, POINTER(ctypes.c_longlong), POINTER(c_double)],
    'tt_probe_mfma_f32': [_I, POINTER(c_double), POINTER(c_double), POINTER(c_double)],
    'tt_probe_hbm_f32': [c_size_t, POINTER(c_double), POINTER(c_double)],
    'tt_conv2d_fwd_f32': [_P, _P, _P, _P] + [_I] * 14,
    'tt_conv2d_dgrad_f32': [_P, _P, _P, _P] + [_I] * 16,
    'tt_conv2d_wgrad_f32': [_P, _P, _P] + [_I] * 16,
    'tt_conv2d_fwd_bf16': [_P, _P, _P, _P] + [_I] * 14,
    'tt_conv2d_dgrad_bf16': [_P, _P, _P, _P] + [_I] * 16,
    'tt_conv2d_wgrad_bf16': [_P, _P, _P] + [_I] * 16,
    'tt_conv2d_fwd_bf16x3': [_P, _P, _P, _P] + [_I] * 14,
    'tt_conv2d_dgrad_bf16x3': [_P, _P, _P, _P] + [_I] * 16,
    'tt_conv2d_check_tables_fwd_f32': [_I] * 14,
    'tt_conv2d_check_tables_dgrad_f32': [_I] * 16,
    'tt_conv2d_check_tables_wgrad_f32': [_I] * 16,
    'tt_conv2d_check_tables_selftest': [],
    'tt_conv2d_check_tables_selftest_wgrad': [],
    'tt_conv2d_stream_k_blocks_per_cu': [_I, POINTER(c_int)],
    'tt_conv2d_stream_k_force_occupancy': [_I],
    'tt_conv2d_selftest_raise_async_error': [],
    'tt_conv2d_last_launch': [POINTER(c_int)],
    'tt_conv2d_last_wgrad_launch': [POINTER(c_int)],
    'tt_conv2d_bf16_first_enable': [_I],
    'tt_conv2d_wgrad_force_occupancy': [_I],
    'tt_conv2d_images_per_run': [_I, ctypes.c_longlong, ctypes.c_longlong, POINTER(c_int)],
    'tt_channel_sum_f32': [_P, _P, _I, _I, _I],
    'tt_workspace_size_conv2d_fwd_f32': [POINTER(c_size_t)] + [_I] * 14,
    'tt_workspace_size_conv2d_dgrad_f32': [POINTER(c_size_t)] + [_I] * 16,
    'tt_workspace_size_conv2d_wgrad_f32': [POINTER(c_size_t)] + [_I] * 16,
    'tt_workspace_size_bn_f32': [POINTER(c_size_t), _I, _I, _I],
    'tt_bn_fwd_train_f32': [_P] * 12 + [c_double, c_double, _I, _I, _I],
    'tt_bn_fwd_train_noalloc_f32': [_P] * 12 + [c_double, c_double, _I, _I, _I],
    'tt_bn_relu_fwd_train_f32': [_P] * 12 + [c_double, c_double, _I, _I, _I],
    'tt_bn_relu_bwd_f32': [_P] * 10 + [_I, _I, _I],
    'tt_bn_fwd_eval_f32': [_P] * 9 + [c_double, _I, _I, _I],
    'tt_bn_bwd_f32': [_P] * 9 + [_I, _I, _I],
    'tt_relu_fwd_f32': [_P, _P, c_size_t],
    'tt_relu_bwd_f32': [_P, _P, _P, c_size_t],
    'tt_leaky_relu_fwd_f32': [_P, _P, c_float, c_size_t],
    'tt_leaky_relu_bwd_f32': [_P, _P, _P, c_float, c_size_t],
    'tt_maxpool2d_fwd_f32': [_P, _P, _P] + [_I] * 13,
    'tt_maxpool2d_bwd_f32': [_P, _P, _P] + [_I] * 13,
    'tt_mean_rows_f32': [_P, _P, _I, _I],
    'tt_mean_rows_bwd_f32': [_P, _P, _I, _I],
    'tt_transpose2d_f32': [_P, _P, _I, _I],
    'tt_add_rowvec_f32': [_P, _P, _P, _I, _I],
    'tt_log_softmax_fwd_f32': [_P, _P, _I, _I],
    'tt_log_softmax_bwd_f32': [_P, _P, _P, _I, _I],
    'tt_nll_loss_fwd_f32': [_P, _P, _P, _P, _P, _I, _I, ctypes.c_longlong, _I],
    'tt_nll_loss_bwd_f32': [_P, _P, _P, _P, _P, _I, _I, ctypes.c_longlong, _I],
    'tt_sgd_step_f32': [_P, _P, _P, c_size_t, c_double, c_double, c_double, c_double, _I, _I],
    'tt_sgd_step_multi_f32': [_I, _P, _P, _P, _P, _P, c_double, c_double, c_double, c_double, _I],
    'tt_adam_step_f32': [_P, _P, _P, _P, _P, c_size_t, _I, c_double, c_double, c_double, c_double, c_double, _I, _I],
    'tt_adam_step_multi_f32': [_I, _P, _P, _P, _P, _P, _P, _P, c_double, c_double, c_double, c_double, c_double, _I, _I],
    'tt_add_f32': [_P, _P, _P, c_size_t],
    'tt_add_relu_f32': [_P, _P, _P, c_size_t],
    'tt_axpy_f32': [c_float, _P, _P, c_size_t],
    'tt_add_scalar_f32': [_P, c_float, c_size_t],
    'tt_fill_f32': [_P, c_float, c_size_t],
}

_lib = None
_ready = False


def load_library(path=None):
    """dlopen the library and attach prototypes (no GPU call is made)."""
    global _lib
    if _lib is None:
        path = path or LIB_PATH
        if not os.path.exists(path):
            raise RuntimeError(f'{path} has not been built: run `python -m pytortto_amd.build` '
                               f'(there is no CPU fallback for the device path)')
        handle = ctypes.CDLL(path)
        handle.tt_last_error.restype = c_char_p
        handle.tt_last_error.argtypes = []
        for name, args in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = c_int
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status):
    if status != 0:
        raise RuntimeError(_lib.tt_last_error().decode(errors='replace'))


def lib():
    """The loaded library with ``tt_init(0)`` done."""
    global _ready
    handle = load_library()
    if not _ready:
        check(handle.tt_init(0))
        _ready = True
    return handle


# ---- one deferred operation ----------------------------------------------------------------------
# An operation whose result the very next operation may absorb (BatchNorm's normalisation into a
# following ReLU, a ReLU's gradient mask into the BatchNorm backward behind it) is not launched at
# once: its caller parks it here.  The next operation either takes it over (``take_pending_if`` and
# a fused launch) or, like any other call into the library, finds it run first -- ``call`` flushes
# before it does anything else, so a deferred operation never outlives the next library call and
# nothing can read or overwrite its operands in between.
#
# The slot is shared by all threads (a buffer that thread A's parked operation will fill may be
# read by thread B, whose first use of it must find the operation run), so every access goes
# through one re-entrant lock: parking, the test-and-take of a fusing successor and the flush are
# each atomic, and a flush started by one thread is finished before another thread's call proceeds.
_pending = None
_lock = threading.RLock()


def defer(op):
    """Park ``op`` (an object with ``run()``); whatever was parked before runs now."""
    global _pending
    with _lock:
        flush()
        _pending = op


def pending():
    return _pending


def take_pending():
    global _pending
    with _lock:
        op, _pending = _pending, None
    return op


def take_pending_if(wanted):
    """The parked operation, removed from the slot, if ``wanted(op)`` holds for it -- test and take
    in one step, so that no other thread can run or steal it in between; otherwise None (and the
    operation stays parked)."""
    global _pending
    with _lock:
        op = _pending
        if op is None or not wanted(op):
            return None
        _pending = None
    return op


def flush():
    """Run the parked operation, if any.  Should it fail, the arrays it was to fill are marked:
    any later use of them raises the same error instead of reading memory nobody wrote."""
    with _lock:
        op = take_pending()
        if op is None:
            return
        try:
            op.run()
        except Exception as exc:
            poison = getattr(op, 'poison', None)
            if poison is not None:
                poison(exc)
            raise


def call(name, *args):
    """Call ``name`` through the C ABI and raise ``RuntimeError(tt_last_error())`` on failure.
    A deferred operation runs first."""
    if _pending is not None:
        flush()
    check(getattr(lib(), name)(*args))


def is_available():
    """True when the library is built and a gfx950 device answers."""
    try:
        lib()
        return True
    except (RuntimeError, OSError):
        return False


def device_info():
    name = ctypes.create_string_buffer(256)
    cus, khz, lds, mem = c_int(), c_int(), c_int(), c_size_t()
    call('tt_device_info', name, 256, ctypes.byref(cus), ctypes.byref(khz), ctypes.byref(lds), ctypes.byref(mem))
    return {'name': name.value.decode(), 'compute_units': cus.value, 'clock_khz': khz.value,
            'lds_bytes_per_block': lds.value, 'total_mem_bytes': mem.value}


PROF_KERNELS = {
    'conv_igemm_fwd': 0, 'conv_igemm_dgrad': 1, 'conv_wgrad': 2, 'conv_wgrad_reduce': 3, 'conv_prep': 4,
    'bn_fwd_reduce': 5, 'bn_fwd_apply': 6, 'bn_bwd_reduce': 7, 'bn_bwd_apply': 8, 'maxpool_fwd': 9, 'maxpool_bwd': 10,
}


def profile_enable(on=True):
    call('tt_profile_enable', 1 if on else 0)


def profile_read():
    """{kernel name: (launches, total milliseconds)} since ``profile_enable(True)``."""
    out = {}
    for name, kid in PROF_KERNELS.items():
        n, ms = ctypes.c_longlong(), c_double()
        call('tt_profile_read', kid, ctypes.byref(n), ctypes.byref(ms))
        out[name] = (n.value, ms.value)
    return out


def probe_mfma(launches=100):
    """Sustained dense fp32 MFMA TFLOP/s: (mean, min, max) over ``launches`` launches."""
    mean, lo, hi = c_double(), c_double(), c_double()
    call('tt_probe_mfma_f32', launches, ctypes.byref(mean), ctypes.byref(lo), ctypes.byref(hi))
    return mean.value, lo.value, hi.value


def probe_hbm(nbytes=2 << 30):
    """Streaming bandwidth in GB/s: (read only, copy counting read + written bytes)."""
    rd, cp = c_double(), c_double()
    call('tt_probe_hbm_f32', nbytes, ctypes.byref(rd), ctypes.byref(cp))
    return rd.value, cp.value


CONV_MATH = {'f32': 0, 'bf16': 1, 'bf16x3': 2}


def set_conv_math(mode):
    """Matrix arithmetic of the three convolution passes: 'f32' (default: float32 matrix
    instructions), 'bf16' (operands rounded to bfloat16 inside the kernel, float32 accumulation;
    tensors stay float32) or 'bf16x3' (float32 arithmetic on the bf16 matrix pipe: every operand
    element as three bf16 terms that add up to it exactly, six products per step; meets the same
    tolerances as 'f32')."""
    if mode not in CONV_MATH:
        raise ValueError(f"conv math must be one of {sorted(CONV_MATH)}, got {mode!r}")
    call('tt_set_conv_math', CONV_MATH[mode])


def get_conv_math():
    mode = c_int()
    call('tt_get_conv_math', ctypes.byref(mode))
    return {v: k for k, v in CONV_MATH.items()}[mode.value]


def synchronize():
    call('tt_sync')


class Event:
    """HIP event on the library stream."""

    def __init__(self):
        self._h = c_void_p()
        call('tt_event_create', ctypes.byref(self._h))

    def record(self):
        call('tt_event_record', self._h)
        return self

    def elapsed_ms(self, later):
        ms = c_float()
        call('tt_event_elapsed_ms', self._h, later._h, ctypes.byref(ms))
        return ms.value

    def __del__(self):
        try:
            if self._h:
                _lib.tt_event_destroy(self._h)
        except Exception:
            pass
