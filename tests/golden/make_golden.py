"""Writes the golden fixtures in this directory from the CPU oracle.

    python tests/golden/make_golden.py

The reference publishes no vectors for this path (its one parity
notebook uses unseeded data) and cannot be imported under the NumPy of this image, so the
fixtures are produced by ``oracle/`` -- after ``tests/test_oracle_*.py`` have pinned it against
brute-force definitions, adjoint identities, closed forms and torch CPU.  They freeze its
float32 results on fixed seeded inputs: ``tests/test_golden.py`` checks that the oracle still
reproduces them (a regression pin for the checker itself) and that the HIP path matches them.

One ``.npz`` per family; arrays are named ``<case index>/<tensor>``.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from tests.cases import CONV_CASES, CONVT_CASES, POOL_CASES  # noqa: E402

BN_SHAPES = [(4, 3, 5, 5), (16, 5, 4, 4), (6, 16, 16, 16)]
HEAD_SHAPES = [(6, 10, 4), (16, 33, 10)]          # (batch, features, classes)
SGD_SETTINGS = [(0.0, 0.0, 0.0, False), (0.9, 0.1, 5e-4, False), (0.8, 0.0, 1e-3, True)]   # momentum, dampening, wd, nesterov
ADAM_SETTINGS = [(False, False, 0.0), (True, False, 1e-2), (False, True, 1e-2)]             # amsgrad, decoupled, wd


def conv_fixture():
    out = {}
    for i, (n, c, h, w_, k, r, s, st, pd, dl, g) in enumerate(CONV_CASES):
        rng = np.random.default_rng(100 + i)
        x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
        w = (rng.standard_normal((k, c // g, r, s)) / np.sqrt(c // g * r * s)).astype(np.float32)
        b = rng.standard_normal(k).astype(np.float32)
        y, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, g)
        gy = rng.standard_normal(y.shape).astype(np.float32)
        dx, dw, db = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, g)
        for name, a in (('x', x), ('w', w), ('b', b), ('gy', gy), ('y', y), ('dx', dx), ('dw', dw), ('db', db)):
            out[f'{i}/{name}'] = np.ascontiguousarray(a, dtype=np.float32)
    return out


def convt_fixture():
    out = {}
    for i, (n, ci, h, w_, co, r, s, st, pd, op, dl, g) in enumerate(CONVT_CASES):
        rng = np.random.default_rng(200 + i)
        x = rng.standard_normal((n, ci, h, w_)).astype(np.float32)
        w = (rng.standard_normal((ci, co // g, r, s)) / np.sqrt(ci // g * r * s)).astype(np.float32)
        b = rng.standard_normal(co).astype(np.float32)
        y = oracle.transposed_convolution_forward(x, w, b, st, pd, op, dl, g)
        gy = rng.standard_normal(y.shape).astype(np.float32)
        dx, dw, db = oracle.transposed_convolution_backward(gy, x, w, st, pd, dl, g)
        for name, a in (('x', x), ('w', w), ('b', b), ('gy', gy), ('y', y), ('dx', dx), ('dw', dw), ('db', db)):
            out[f'{i}/{name}'] = np.ascontiguousarray(a, dtype=np.float32)
    return out


def bn_fixture():
    out = {}
    for i, shape in enumerate(BN_SHAPES):
        rng = np.random.default_rng(300 + i)
        c = shape[1]
        x = (2 + 3 * rng.standard_normal(shape)).astype(np.float32)
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = (0.1 * rng.standard_normal(c)).astype(np.float32)
        dy = rng.standard_normal(shape).astype(np.float32)
        rm0, rv0 = np.zeros(c, np.float32), np.ones(c, np.float32)
        y, saved, rm, rv = oracle.batch_norm_forward(x, gamma, beta, rm0, rv0, True, 0.1, 1e-5)
        dx, dg, db = oracle.batch_norm_backward(dy, x, gamma, saved)
        for name, a in (('x', x), ('gamma', gamma), ('beta', beta), ('dy', dy), ('y', y),
                        ('mean', saved['mean'].ravel()), ('var_eps', saved['var'].ravel()), ('sd', saved['sd'].ravel()),
                        ('running_mean', rm), ('running_var', rv), ('dx', dx), ('dgamma', dg), ('dbeta', db)):
            out[f'{i}/{name}'] = np.ascontiguousarray(a, dtype=np.float32)
    return out


def pool_fixture():
    """MaxPool2d on rounded inputs (many ties) and LeakyReLU; `tap` = kernel row * kw + kernel column."""
    out = {}
    for i, (n, c, h, w_, ks, st, pd, dl, cm) in enumerate(POOL_CASES):
        rng = np.random.default_rng(400 + i)
        x = np.round(2 * rng.standard_normal((n, c, h, w_))).astype(np.float32) / 2
        y, (idx2, idx1_m) = oracle.max_pool2d(x, ks, st, pd, dl, cm)
        gy = rng.standard_normal(y.shape).astype(np.float32)
        dx = oracle.max_pool2d_backward(x.shape, gy, (idx2, idx1_m), ks, st, pd, dl, cm)
        tap = np.moveaxis(idx2 * ks[1] + idx1_m, -1, 1).astype(np.int32)
        act = oracle.leaky_relu_forward(x, 0.2)
        dact = oracle.leaky_relu_backward(dx, x, 0.2)
        for name, a in (('x', x), ('gy', gy), ('y', y), ('tap', tap), ('dx', dx), ('leaky', act), ('dleaky', dact)):
            out[f'{i}/{name}'] = np.ascontiguousarray(a)
    return out


def head_fixture():
    """mean over (H, W) -> Linear -> LogSoftmax -> NLLLoss (mean), forward and backward."""
    out = {}
    for i, (n, f, k) in enumerate(HEAD_SHAPES):
        rng = np.random.default_rng(500 + i)
        x = rng.standard_normal((n, f, 3, 3)).astype(np.float32)
        w = (rng.standard_normal((k, f)) / np.sqrt(f)).astype(np.float32)
        b = rng.standard_normal(k).astype(np.float32)
        target = rng.integers(0, k, n).astype(np.int64)
        feat = oracle.mean_forward(x, (-1, -2), True).reshape(n, f)
        logits = oracle.linear_forward(feat, w, b)
        logp = oracle.log_softmax_forward(logits)
        loss, count = oracle.nll_loss_forward(logp, target)
        dlogp = oracle.nll_loss_backward(np.float32(1.0), logp.shape, target, count=count)
        dlogits = oracle.log_softmax_backward(dlogp, logp)
        dfeat, dw, db = oracle.linear_backward(dlogits, feat, w)
        dx = oracle.mean_backward(dfeat.reshape(n, f, 1, 1), x.shape, (-1, -2), True)
        for name, a in (('x', x), ('w', w), ('b', b), ('target', target), ('feat', feat), ('logits', logits),
                        ('logp', logp), ('loss', np.float32(loss)), ('dlogp', dlogp), ('dlogits', dlogits),
                        ('dw', dw), ('db', db), ('dx', dx)):
            out[f'{i}/{name}'] = np.ascontiguousarray(a).reshape(np.shape(a))   # (0-d stays 0-d)
    return out


def optim_fixture():
    """Five steps of SGD / Adam / AdamW on one parameter: `p0`, the gradients and the trajectory."""
    out = {}
    lr = 0.05
    for i, (mom, damp, wd, nest) in enumerate(SGD_SETTINGS):
        rng = np.random.default_rng(600 + i)
        p = rng.standard_normal((5, 7)).astype(np.float32)
        out[f'sgd{i}/p0'] = p.copy()
        bufs = [None]
        for t in range(5):
            g = rng.standard_normal(p.shape).astype(np.float32)
            out[f'sgd{i}/g{t}'] = g.copy()
            oracle.optim.sgd([p], [g], bufs, wd, mom, lr, damp, nest)
            out[f'sgd{i}/p{t + 1}'] = p.copy()
    for i, (ams, dec, wd) in enumerate(ADAM_SETTINGS):
        rng = np.random.default_rng(700 + i)
        p = rng.standard_normal((5, 7)).astype(np.float32)
        out[f'adam{i}/p0'] = p.copy()
        m, v, vmax = np.zeros_like(p), np.zeros_like(p), np.zeros_like(p)
        for t in range(5):
            g = rng.standard_normal(p.shape).astype(np.float32)
            out[f'adam{i}/g{t}'] = g.copy()
            oracle.optim.adam([p], [g], [m], [v], [vmax], [t + 1], ams, 0.9, 0.99, 1e-2, wd, 1e-8, dec)
            out[f'adam{i}/p{t + 1}'] = p.copy()
    return out


if __name__ == '__main__':
    for fname, make in (('conv_small.npz', conv_fixture), ('conv_transpose_small.npz', convt_fixture),
                        ('batchnorm_small.npz', bn_fixture), ('pool_small.npz', pool_fixture),
                        ('head_small.npz', head_fixture), ('optim_small.npz', optim_fixture)):
        arrays = make()
        np.savez_compressed(os.path.join(HERE, fname), **arrays)
        print(fname, len(arrays), 'arrays', os.path.getsize(os.path.join(HERE, fname)), 'bytes')
