"""GPU: ``tt_bn_fwd_train_noalloc_f32`` (the entry point that allocates nothing) against
``tt_bn_fwd_train_f32`` through the C ABI.

Both run the same kernels in the same order, so every output must be bit-identical; the first
shape is also held to the oracle.  Two calls in a row, the second on a smaller input, check that
what the first call left in the shared scratch array does not leak into the second.  The library
workspace is released beforehand and must still be empty afterwards.
"""
import ctypes

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

# (N, C, H, W): two-sweep path with several splits per channel, then a smaller input of the same
# kind, then the single-kernel path for small channels (no scratch at all)
CALLS = [(96, 12, 28, 28), (6, 5, 12, 20), (4, 128, 7, 7)]


def _run(entry, x, gamma, beta, rm0, rv0):
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    n, c = x.shape[:2]
    hw = x.size // (n * c)
    xd, gd, bd = hiparray(x), hiparray(gamma), hiparray(beta)
    rmd, rvd = hiparray(rm0), hiparray(rv0)
    y = hiparray.empty(x.shape)
    outs = [hiparray.empty((c,)) for _ in range(5)]   # mean, var+eps, sd, running mean, running var
    counter = hiparray(np.array([7.0], np.float32))   # num_batches_tracked: incremented by the call
    _hip.call(entry, xd.ptr, gd.ptr, bd.ptr, y.ptr, outs[0].ptr, outs[1].ptr, outs[2].ptr, rmd.ptr, rvd.ptr,
              outs[3].ptr, outs[4].ptr, counter.ptr, 0.1, 1e-5, n, c, hw)
    assert counter.get()[0] == 8.0
    return [y.get()] + [o.get() for o in outs]


def _workspace_bytes():
    from pytortto_amd import _hip
    ws = ctypes.c_size_t()
    _hip.call('tt_mem_stats', None, None, ctypes.byref(ws))
    return ws.value


def test_noalloc_entry_matches_allocating_entry_on_consecutive_calls():
    from pytortto_amd import _hip
    _hip.call('tt_empty_cache')
    assert _workspace_bytes() == 0
    inputs = []
    got = []
    for i, shape in enumerate(CALLS):
        np.random.seed(100 + i)
        c = shape[1]
        x = (2 + 3 * np.random.randn(*shape)).astype(np.float32)
        gamma, beta = oracle.bn_affine_c4(c)
        rm0 = np.random.randn(c).astype(np.float32)
        rv0 = np.random.uniform(0.5, 2.0, c).astype(np.float32)
        inputs.append((x, gamma, beta, rm0, rv0))
        got.append(_run('tt_bn_fwd_train_noalloc_f32', x, gamma, beta, rm0, rv0))
    assert _workspace_bytes() == 0, 'the no-allocation entry point grew the library workspace'

    names = ['y', 'save_mean', 'save_var_eps', 'save_sd', 'running_mean', 'running_var']
    for shape, args, res in zip(CALLS, inputs, got):
        want = _run('tt_bn_fwd_train_f32', *args)
        for name, a, b in zip(names, res, want):
            assert a.dtype == b.dtype and a.shape == b.shape
            assert np.array_equal(a, b), f'{name} differs between the two entry points at {shape}'
    # the first call also against the oracle (rtol 1e-5, floor for values that cancel to ~0)
    x, gamma, beta, rm0, rv0 = inputs[0]
    y_ref, saved, rm_ref, rv_ref = oracle.batch_norm_forward(x, gamma, beta, rm0, rv0, True, 0.1, 1e-5)
    for name, a, ref in zip(names, got[0], [y_ref, saved['mean'].ravel(), saved['var'].ravel(), saved['sd'].ravel(),
                                            rm_ref, rv_ref]):
        np.testing.assert_allclose(a, ref, rtol=1e-5, atol=2e-6 * float(np.abs(ref).max()), err_msg=name)


def test_noalloc_entry_rejects_sizes_beyond_the_scratch_array():
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    size = ctypes.c_size_t()
    # [64, 2048, 64, 64]: 8 splits of 8192 float4 vectors per channel = 16384 partial moments: the limit
    _hip.call('tt_workspace_size_bn_f32', ctypes.byref(size), 64, 2048, 4096)
    assert size.value == 16 * 16384
    # one channel more does not fit; the call must fail before any launch (the pointers are never touched)
    _hip.call('tt_workspace_size_bn_f32', ctypes.byref(size), 64, 2049, 4096)
    assert size.value > 16 * 16384
    dummy = hiparray.empty((16,))
    with pytest.raises(RuntimeError, match='fixed scratch array'):
        _hip.call('tt_bn_fwd_train_noalloc_f32', dummy.ptr, None, None, dummy.ptr, dummy.ptr, dummy.ptr, dummy.ptr,
                  None, None, None, None, None, 0.1, 1e-5, 64, 2049, 4096)
