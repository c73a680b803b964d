"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the oracle).

CPU part: the oracle still reproduces its frozen float32 results (to a few ulps: only the
summation order of the BLAS underneath may differ) -- any change to the checker shows up here.  GPU part: the HIP path matches the same frozen vectors within the path's
tolerances (conv rtol 1e-4 / atol 1e-5, reductions with an absolute floor scaled by the tensor's
magnitude; BatchNorm rtol 1e-5 for outputs and statistics, 1e-4 for gradients; pooling, LeakyReLU and the
optimiser trajectories bit for bit; the head rtol 1e-5 for means and the loss, the convolution
bar for what goes through the matrix products)."""
import os

import numpy as np
import pytest

import oracle
from tests.cases import CONV_CASES, CONVT_CASES, POOL_CASES
from tests.golden.make_golden import ADAM_SETTINGS, BN_SHAPES, HEAD_SHAPES, SGD_SETTINGS

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


def test_oracle_reproduces_pool_fixture():
    z = _load('pool_small.npz')
    for i, (n, c, h, w_, ks, st, pd, dl, cm) in enumerate(POOL_CASES):
        y, (idx2, idx1_m) = oracle.max_pool2d(z[f'{i}/x'], ks, st, pd, dl, cm)
        np.testing.assert_array_equal(y, z[f'{i}/y'])
        np.testing.assert_array_equal(np.moveaxis(idx2 * ks[1] + idx1_m, -1, 1), z[f'{i}/tap'])
        dx = oracle.max_pool2d_backward(z[f'{i}/x'].shape, z[f'{i}/gy'], (idx2, idx1_m), ks, st, pd, dl, cm)
        np.testing.assert_array_equal(dx, z[f'{i}/dx'])
        np.testing.assert_array_equal(oracle.leaky_relu_forward(z[f'{i}/x'], 0.2), z[f'{i}/leaky'])
        np.testing.assert_array_equal(oracle.leaky_relu_backward(dx, z[f'{i}/x'], 0.2), z[f'{i}/dleaky'])


def test_oracle_reproduces_head_fixture():
    z = _load('head_small.npz')
    for i, (n, f, k) in enumerate(HEAD_SHAPES):
        feat = oracle.mean_forward(z[f'{i}/x'], (-1, -2), True).reshape(n, f)
        logp = oracle.log_softmax_forward(oracle.linear_forward(feat, z[f'{i}/w'], z[f'{i}/b']))
        loss, count = oracle.nll_loss_forward(logp, z[f'{i}/target'])
        _same(feat, z[f'{i}/feat'], f'head case {i} feat')
        _same(logp, z[f'{i}/logp'], f'head case {i} logp')
        _same(np.float32(loss), z[f'{i}/loss'], f'head case {i} loss')
        dlogits = oracle.log_softmax_backward(oracle.nll_loss_backward(np.float32(1.0), logp.shape, z[f'{i}/target'],
                                                                       count=count), logp)
        dfeat, dw, db = oracle.linear_backward(dlogits, feat, z[f'{i}/w'])
        _same(dw, z[f'{i}/dw'], f'head case {i} dw')
        _same(db, z[f'{i}/db'], f'head case {i} db')
        _same(oracle.mean_backward(dfeat.reshape(n, f, 1, 1), z[f'{i}/x'].shape, (-1, -2), True), z[f'{i}/dx'],
              f'head case {i} dx')


def test_oracle_reproduces_optim_fixture():
    z = _load('optim_small.npz')
    for i, (mom, damp, wd, nest) in enumerate(SGD_SETTINGS):
        p, bufs = z[f'sgd{i}/p0'].copy(), [None]
        for t in range(5):
            oracle.optim.sgd([p], [z[f'sgd{i}/g{t}'].copy()], bufs, wd, mom, 0.05, damp, nest)
            np.testing.assert_array_equal(p, z[f'sgd{i}/p{t + 1}'])
    for i, (ams, dec, wd) in enumerate(ADAM_SETTINGS):
        p = z[f'adam{i}/p0'].copy()
        m, v, vmax = np.zeros_like(p), np.zeros_like(p), np.zeros_like(p)
        for t in range(5):
            oracle.optim.adam([p], [z[f'adam{i}/g{t}']], [m], [v], [vmax], [t + 1], ams, 0.9, 0.99, 1e-2, wd, 1e-8, dec)
            np.testing.assert_array_equal(p, z[f'adam{i}/p{t + 1}'])


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


@pytest.mark.gpu
def test_hip_pool_and_leaky_relu_match_fixture():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    z = _load('pool_small.npz')
    for i, (n, c, h, w_, ks, st, pd, dl, cm) in enumerate(POOL_CASES):
        x = hiparray(z[f'{i}/x'])
        y, tap = ops.maxpool2d_fwd(x, z[f'{i}/y'].shape[-2:], ks, st, pd, dl)
        np.testing.assert_array_equal(y.get(), z[f'{i}/y'])
        np.testing.assert_array_equal(tap.get(), z[f'{i}/tap'])
        dx = ops.maxpool2d_bwd(hiparray(z[f'{i}/gy']), tap, (h, w_), ks, st, pd, dl)
        np.testing.assert_array_equal(dx.get(), z[f'{i}/dx'])
        np.testing.assert_array_equal(ops.leaky_relu_fwd(x, 0.2).get(), z[f'{i}/leaky'])
        np.testing.assert_array_equal(ops.leaky_relu_bwd(dx, x, 0.2).get(), z[f'{i}/dleaky'])


@pytest.mark.gpu
def test_hip_head_matches_fixture():
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    z = _load('head_small.npz')
    for i, (n, f, k) in enumerate(HEAD_SHAPES):
        x, w, b, target = (hiparray(z[f'{i}/{t}']) for t in ('x', 'w', 'b', 'target'))
        feat = ops.mean_trailing(x, 2, True).reshape((n, f))
        wt = ops.transpose2d(w)
        logits = ops.add_rowvec(ops.mm(feat, wt), b)
        logp = ops.log_softmax_fwd(logits)
        loss, count = ops.nll_loss_fwd(logp, target, None, -100, 'mean')
        _close(feat.get(), z[f'{i}/feat'], 1e-5, 1e-6, f'case {i} feat')
        _close(logits.get(), z[f'{i}/logits'], 1e-4, 1e-5, f'case {i} logits')
        _close(logp.get(), z[f'{i}/logp'], 1e-4, 1e-5, f'case {i} logp')
        _close(loss.get(), z[f'{i}/loss'], 1e-5, 1e-6, f'case {i} loss')
        dlogp = ops.nll_loss_bwd(hiparray(np.float32(1.0)), (n, k), target, None, count, -100, 'mean')
        _close(dlogp.get(), z[f'{i}/dlogp'], 1e-6, 1e-8, f'case {i} dlogp')
        dlogits = ops.log_softmax_bwd(dlogp, logp)
        _close(dlogits.get(), z[f'{i}/dlogits'], 1e-4, 1e-6, f'case {i} dlogits')
        dw = ops.transpose2d(ops.mm_grad_b(feat, dlogits))
        _close(dw.get(), z[f'{i}/dw'], 1e-4, 1e-6, f'case {i} dw')
        _close(ops.sum_rows(dlogits, k).get(), z[f'{i}/db'], 1e-4, 1e-6, f'case {i} db')
        dfeat = ops.mm_grad_a(dlogits, wt)
        dx = ops.mean_trailing_bwd(dfeat.reshape((n, f, 1, 1)), (n, f, 3, 3), 2)
        _close(dx.get(), z[f'{i}/dx'], 1e-4, 1e-7, f'case {i} dx')


@pytest.mark.gpu
def test_hip_optimiser_trajectories_match_fixture():
    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    z = _load('optim_small.npz')
    for i, (mom, damp, wd, nest) in enumerate(SGD_SETTINGS):
        p = hiparray(z[f'sgd{i}/p0'])
        buf = hiparray.empty(p.shape) if mom else None
        for t in range(5):
            g = hiparray(z[f'sgd{i}/g{t}'])
            _hip.call('tt_sgd_step_f32', p.ptr, g.ptr, None if buf is None else buf.ptr, p.size, 0.05, mom, damp, wd,
                      int(nest), int(t == 0))
            np.testing.assert_array_equal(p.get(), z[f'sgd{i}/p{t + 1}'])
    for i, (ams, dec, wd) in enumerate(ADAM_SETTINGS):
        p = hiparray(z[f'adam{i}/p0'])
        m, v, vmax = (hiparray.zeros(p.shape) for _ in range(3))
        for t in range(5):
            g = hiparray(z[f'adam{i}/g{t}'])
            _hip.call('tt_adam_step_f32', p.ptr, g.ptr, m.ptr, v.ptr, vmax.ptr if ams else None, p.size, t + 1, 1e-2,
                      0.9, 0.99, 1e-8, wd, int(ams), int(dec))
            np.testing.assert_array_equal(p.get(), z[f'adam{i}/p{t + 1}'])
