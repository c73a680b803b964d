"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the oracle).

CPU part: the oracle still reproduces its frozen float32 results (to a few ulps: only the
summation order of the BLAS underneath may differ) -- any change to the checker shows up here.  GPU part: the HIP path matches the same frozen vectors within the path's
tolerances (conv rtol 1e-4 / atol 1e-5, reductions with an absolute floor scaled by the tensor's
magnitude; BatchNorm rtol 1e-5 for outputs and statistics, 1e-4 for gradients)."""
import os

import numpy as np
import pytest

import oracle
from tests.cases import CONV_CASES, CONVT_CASES
from tests.golden.make_golden import BN_SHAPES

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def _load(name):
    with np.load(os.path.join(GOLDEN, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _same(a, b, what):
    """Equal up to float32 summation order (BLAS kernels differ between hosts and thread counts)."""
    assert a.shape == b.shape, what
    scale = float(np.abs(b).max()) or 1.0
    np.testing.assert_allclose(np.asarray(a, np.float32), b, rtol=2e-6, atol=2e-6 * scale, err_msg=what)


def test_oracle_reproduces_conv_fixture():
    z = _load('conv_small.npz')
    for i, (n, c, h, w_, k, r, s, st, pd, dl, g) in enumerate(CONV_CASES):
        y, xpad = oracle.convolution_forward(z[f'{i}/x'], z[f'{i}/w'], z[f'{i}/b'], st, pd, dl, g)
        dx, dw, db = oracle.convolution_backward(z[f'{i}/gy'], z[f'{i}/x'], xpad, z[f'{i}/w'], st, pd, dl, g)
        for name, a in (('y', y), ('dx', dx), ('dw', dw), ('db', db)):
            _same(a, z[f'{i}/{name}'], f'conv case {i} {name}')


def test_oracle_reproduces_conv_transpose_fixture():
    z = _load('conv_transpose_small.npz')
    for i, (n, ci, h, w_, co, r, s, st, pd, op, dl, g) in enumerate(CONVT_CASES):
        y = oracle.transposed_convolution_forward(z[f'{i}/x'], z[f'{i}/w'], z[f'{i}/b'], st, pd, op, dl, g)
        dx, dw, db = oracle.transposed_convolution_backward(z[f'{i}/gy'], z[f'{i}/x'], z[f'{i}/w'], st, pd, dl, g)
        for name, a in (('y', y), ('dx', dx), ('dw', dw), ('db', db)):
            _same(a, z[f'{i}/{name}'], f'conv-transpose case {i} {name}')


def test_oracle_reproduces_batchnorm_fixture():
    z = _load('batchnorm_small.npz')
    for i, shape in enumerate(BN_SHAPES):
        c = shape[1]
        y, saved, rm, rv = oracle.batch_norm_forward(z[f'{i}/x'], z[f'{i}/gamma'], z[f'{i}/beta'],
                                                     np.zeros(c, np.float32), np.ones(c, np.float32), True, 0.1, 1e-5)
        dx, dg, db = oracle.batch_norm_backward(z[f'{i}/dy'], z[f'{i}/x'], z[f'{i}/gamma'], saved)
        for name, a in (('y', y), ('mean', saved['mean'].ravel()), ('var_eps', saved['var'].ravel()),
                        ('sd', saved['sd'].ravel()), ('running_mean', rm), ('running_var', rv),
                        ('dx', dx), ('dgamma', dg), ('dbeta', db)):
            _same(a, z[f'{i}/{name}'], f'batchnorm case {i} {name}')


def _close(got, ref, rtol, atol, name):
    np.testing.assert_allclose(got, ref, rtol=rtol, atol=atol, err_msg=name)


@pytest.mark.gpu
def test_hip_conv_matches_fixture():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    z = _load('conv_small.npz')
    for i, (n, c, h, w_, k, r, s, st, pd, dl, g) in enumerate(CONV_CASES):
        x, w, b, gy = (hiparray(z[f'{i}/{t}']) for t in ('x', 'w', 'b', 'gy'))
        y = ops.conv2d_fwd(x, w, b, st, pd, dl, g)
        dx = ops.conv2d_dgrad(gy, w, None, (h, w_), st, pd, dl, g)
        dw = ops.conv2d_wgrad(x, gy, z[f'{i}/w'].shape, st, pd, dl, g)
        db = ops.channel_sum(gy)
        _close(y.get(), z[f'{i}/y'], 1e-4, 1e-5, f'case {i} y')
        _close(dx.get(), z[f'{i}/dx'], 1e-4, 1e-5, f'case {i} dx')
        for got, name in ((dw, 'dw'), (db, 'db')):
            ref = z[f'{i}/{name}']
            _close(got.get(), ref, 1e-4, 1e-5 * max(1.0, float(np.abs(ref).max())), f'case {i} {name}')


@pytest.mark.gpu
def test_hip_conv_transpose_matches_fixture():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    z = _load('conv_transpose_small.npz')
    for i, (n, ci, h, w_, co, r, s, st, pd, op, dl, g) in enumerate(CONVT_CASES):
        x, w, b, gy = (hiparray(z[f'{i}/{t}']) for t in ('x', 'w', 'b', 'gy'))
        y = ops.conv2d_dgrad(x, w, b, z[f'{i}/y'].shape[-2:], st, pd, dl, g)
        dx = ops.conv2d_fwd(gy, w, None, st, pd, dl, g)
        dw = ops.conv2d_wgrad(gy, x, z[f'{i}/w'].shape, st, pd, dl, g)
        db = ops.channel_sum(gy)
        _close(y.get(), z[f'{i}/y'], 1e-4, 1e-5, f'case {i} y')
        _close(dx.get(), z[f'{i}/dx'], 1e-4, 1e-5, f'case {i} dx')
        for got, name in ((dw, 'dw'), (db, 'db')):
            ref = z[f'{i}/{name}']
            _close(got.get(), ref, 1e-4, 1e-5 * max(1.0, float(np.abs(ref).max())), f'case {i} {name}')


@pytest.mark.gpu
def test_hip_batchnorm_matches_fixture():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    z = _load('batchnorm_small.npz')
    for i, shape in enumerate(BN_SHAPES):
        c = shape[1]
        x, gamma, beta, dy = (hiparray(z[f'{i}/{t}']) for t in ('x', 'gamma', 'beta', 'dy'))
        y, mean, var_eps, sd, rm, rv = ops.bn_fwd_train(x, gamma, beta, hiparray(np.zeros(c, np.float32)),
                                                         hiparray(np.ones(c, np.float32)), 0.1, 1e-5)
        dx, dg, db = ops.bn_bwd(x, dy, gamma, mean, var_eps, sd)
        for got, name in ((y, 'y'), (mean, 'mean'), (var_eps, 'var_eps'), (sd, 'sd'), (rm, 'running_mean'),
                          (rv, 'running_var')):
            ref = z[f'{i}/{name}']
            _close(got.get(), ref, 1e-5, 2e-6 * float(np.abs(ref).max()), f'case {i} {name}')
        for got, name in ((dx, 'dx'), (dg, 'dgamma'), (db, 'dbeta')):
            ref = z[f'{i}/{name}']
            _close(got.get(), ref, 1e-4, 1e-5 * max(1.0, float(np.abs(ref).max())), f'case {i} {name}')
