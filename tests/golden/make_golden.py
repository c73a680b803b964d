"""Writes the golden fixtures in this directory from the CPU oracle.

    python tests/golden/make_golden.py

The reference publishes no vectors for the convolution / BatchNorm path (its one parity
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
from tests.cases import CONV_CASES, CONVT_CASES  # noqa: E402

BN_SHAPES = [(4, 3, 5, 5), (16, 5, 4, 4), (6, 16, 16, 16)]


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


if __name__ == '__main__':
    for fname, make in (('conv_small.npz', conv_fixture), ('conv_transpose_small.npz', convt_fixture),
                        ('batchnorm_small.npz', bn_fixture)):
        arrays = make()
        np.savez_compressed(os.path.join(HERE, fname), **arrays)
        print(fname, len(arrays), 'arrays', os.path.getsize(os.path.join(HERE, fname)), 'bytes')
