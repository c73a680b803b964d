"""Error report of the device path against the CPU oracle and a float64 evaluation.

Run on a machine with an MI355X:  ``python -m tests.parity_report``  (a few minutes; the oracle's
float64 passes dominate).  For every tensor it prints, as the worst case over the layers of a
configuration:

    d(gpu, ref)   max|gpu - oracle_f32| / max|oracle_f32|
    e(gpu)        max|gpu - f64| / max|f64|
    e(ref)        max|oracle_f32 - f64| / max|f64|

The configurations are the benchmark's: the baseline Conv2d(16, 32, 3, padding=1) at
[32,16,32,32]; the PreAct-ResNet-18 and ResNet-50 convolution shapes (batch 8 and 2: the oracle's
float64 pass sets the size); the DCGAN generator's ConvTranspose2d layers (batch 16); BatchNorm2d
at [64,256,56,56] and [128,64,112,112] with x ~ N(2, 3).  The parity tests assert on the same
quantities; this script only tabulates them.
"""
import sys

import numpy as np

import oracle

PREACT18 = [(3, 32, 64, 3, 1, 1), (64, 32, 64, 3, 1, 1), (64, 32, 128, 1, 2, 0), (64, 32, 128, 3, 2, 1),
            (128, 16, 128, 3, 1, 1), (128, 16, 256, 1, 2, 0), (128, 16, 256, 3, 2, 1), (256, 8, 256, 3, 1, 1),
            (256, 8, 512, 1, 2, 0), (256, 8, 512, 3, 2, 1), (512, 4, 512, 3, 1, 1)]
DCGAN = [(100, 1, 512, 4, 1, 0), (512, 4, 256, 4, 2, 1), (256, 8, 128, 4, 2, 1), (128, 16, 64, 4, 2, 1), (64, 32, 3, 4, 2, 1)]


def rel(a, b):
    return float(np.abs(a - b).max()) / (float(np.abs(b).max()) or 1.0)


class Worst:
    def __init__(self):
        self.rows = {}

    def add(self, name, gpu, ref32, ref64):
        d, eg, er = rel(gpu, ref32), rel(gpu, ref64), rel(ref32, ref64)
        old = self.rows.get(name, (0.0, 0.0, 0.0))
        self.rows[name] = (max(old[0], d), max(old[1], eg), max(old[2], er))

    def show(self, title):
        print(title)
        for name, (d, eg, er) in self.rows.items():
            print(f'    {name:<14} d(gpu,ref) {d:9.2e}   e(gpu) {eg:9.2e}   e(ref) {er:9.2e}')
        sys.stdout.flush()


def conv_layers(title, specs, batch, seed):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(seed)
    worst = Worst()
    for c, h, k, r, s, p in specs:
        st, pd, dl = (s, s), (p, p), (1, 1)
        x = rng.standard_normal((batch, c, h, h)).astype(np.float32)
        w = rng.uniform(-1, 1, (k, c, r, r)).astype(np.float32) / np.float32(np.sqrt(c * r * r))
        b = rng.uniform(-1, 1, k).astype(np.float32)
        y32, xpad = oracle.convolution_forward(x, w, b, st, pd, dl, 1)
        gy = rng.standard_normal(y32.shape).astype(np.float32)
        dx32, dw32, db32 = oracle.convolution_backward(gy, x, xpad, w, st, pd, dl, 1)
        x64, w64, gy64 = (a.astype(np.float64) for a in (x, w, gy))
        y64, xpad64 = oracle.convolution_forward(x64, w64, b.astype(np.float64), st, pd, dl, 1)
        dx64, dw64, db64 = oracle.convolution_backward(gy64, x64, xpad64, w64, st, pd, dl, 1)
        xd, wd, gyd = hiparray(x), hiparray(w), hiparray(gy)
        worst.add('y', ops.conv2d_fwd(xd, wd, hiparray(b), st, pd, dl, 1).get(), y32, y64)
        worst.add('x.grad', ops.conv2d_dgrad(gyd, wd, None, (h, h), st, pd, dl, 1).get(), dx32, dx64)
        worst.add('weight.grad', ops.conv2d_wgrad(xd, gyd, w.shape, st, pd, dl, 1).get(), dw32, dw64)
        worst.add('bias.grad', ops.channel_sum(gyd).get(), db32, db64)
    worst.show(title)


def conv_transpose_layers(title, specs, batch, seed):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(seed)
    worst = Worst()
    for ci, h, co, r, s, p in specs:
        st, pd, dl, op = (s, s), (p, p), (1, 1), (0, 0)
        x = rng.standard_normal((batch, ci, h, h)).astype(np.float32)
        w = rng.uniform(-1, 1, (ci, co, r, r)).astype(np.float32) / np.float32(np.sqrt(ci * r * r))
        y32 = oracle.transposed_convolution_forward(x, w, None, st, pd, op, dl, 1)
        gy = rng.standard_normal(y32.shape).astype(np.float32)
        dx32, dw32, _ = oracle.transposed_convolution_backward(gy, x, w, st, pd, dl, 1)
        x64, w64, gy64 = (a.astype(np.float64) for a in (x, w, gy))
        y64 = oracle.transposed_convolution_forward(x64, w64, None, st, pd, op, dl, 1)
        dx64, dw64, _ = oracle.transposed_convolution_backward(gy64, x64, w64, st, pd, dl, 1)
        xd, wd, gyd = hiparray(x), hiparray(w), hiparray(gy)
        worst.add('y', ops.conv2d_dgrad(xd, wd, None, y32.shape[-2:], st, pd, dl, 1).get(), y32, y64)
        worst.add('x.grad', ops.conv2d_fwd(gyd, wd, None, st, pd, dl, 1).get(), dx32, dx64)
        worst.add('weight.grad', ops.conv2d_wgrad(gyd, xd, w.shape, st, pd, dl, 1).get(), dw32, dw64)
    worst.show(title)


def batchnorm(title, shapes, seed):
    from pytortto_amd import ops
    from pytortto_amd.xparray import hiparray
    rng = np.random.default_rng(seed)
    worst = Worst()
    for shape in shapes:
        c = shape[1]
        x = (2 + 3 * rng.standard_normal(shape)).astype(np.float32)
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = rng.normal(0, 0.1, c).astype(np.float32)
        gy = rng.standard_normal(shape).astype(np.float32)
        rm, rv = np.zeros(c, np.float32), np.ones(c, np.float32)
        res = {}
        for dt in (np.float32, np.float64):
            xx, gg, bb, gyy = (a.astype(dt) for a in (x, gamma, beta, gy))
            y, saved, nrm, nrv = oracle.batch_norm_forward(xx, gg, bb, rm.astype(dt), rv.astype(dt), True, 0.1, 1e-5)
            dx, dgamma, dbeta = oracle.batch_norm_backward(gyy, xx, gg, saved)
            res[dt] = (y, nrm, nrv, dx, dgamma, dbeta)
            del xx, gyy, y, dx
        xd, gyd, gd = hiparray(x), hiparray(gy), hiparray(gamma)
        y, mean, var_eps, sd, nrm, nrv = ops.bn_fwd_train(xd, gd, hiparray(beta), hiparray(rm), hiparray(rv), 0.1, 1e-5)
        dx, dgamma, dbeta = ops.bn_bwd(xd, gyd, gd, mean, var_eps, sd)
        got = (y, nrm, nrv, dx, dgamma, dbeta)
        for i, name in enumerate(('y', 'running_mean', 'running_var', 'x.grad', 'weight.grad', 'bias.grad')):
            worst.add(name, got[i].get(), res[np.float32][i], res[np.float64][i])
        del res, xd, gyd, y, dx, got
    worst.show(title)


def main():
    import bench
    conv_layers('Conv2d(16, 32, 3, padding=1), x [32,16,32,32] (baseline configuration)', [(16, 32, 32, 3, 1, 1)], 32, 0)
    conv_layers('PreAct-ResNet-18 convolution shapes, batch 8 (11 shapes)', PREACT18, 8, 1)
    conv_layers('ResNet-50 convolution shapes, batch 2 (23 shapes)', [s[:6] for s in bench.RESNET50_CONVS], 2, 2)
    conv_transpose_layers('DCGAN generator ConvTranspose2d layers, batch 16 (5 layers)', DCGAN, 16, 3)
    batchnorm('BatchNorm2d training, x ~ N(2, 3), [64,256,56,56] and [128,64,112,112]', [(64, 256, 56, 56), (128, 64, 112, 112)], 4)


if __name__ == '__main__':
    main()
