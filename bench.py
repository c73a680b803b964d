#!/usr/bin/env python3
"""Benchmark of the convolution / BatchNorm hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  Primary metric: fp32 conv fwd+dgrad+wgrad TFLOP/s over the 53
convolutions of ResNet-50 at batch 64, 224x224 (one "step" = one pass over all of them, inputs
resident in HBM, synthetic N(0,1) data, Kaiming-uniform weights).  Secondary (same line, key
"bn"): BatchNorm2d training fwd+bwd GB/s at [64,256,56,56] and [128,64,112,112].

Timing: W warm-up steps, then exactly K steps between stream synchronisations (HIP events on
the library's stream give ms_per_step; the wall clock around the same region is reported
too).  A second pass of K steps runs with the library's per-kernel event brackets switched on
and yields the average launch duration of each kernel for the roofline objects; event records
between kernels cost a few microseconds each, which is why they are not part of the first pass.
The CPU baseline (NumPy restatement of the reference's CPU path, ``oracle/``) is timed on a
bounded sample of the same workloads on the host cores.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0   # dense, published
PEAK_HBM_GBS = 8000.0

# ResNet-50 convolutions at 224x224: (C_in, H_in, C_out, kernel, stride, pad, occurrences)
RESNET50_CONVS = [
    (3, 224, 64, 7, 2, 3, 1),
    (64, 56, 256, 1, 1, 0, 4), (64, 56, 64, 1, 1, 0, 1), (64, 56, 64, 3, 1, 1, 3), (256, 56, 64, 1, 1, 0, 2),
    (256, 56, 512, 1, 2, 0, 1), (256, 56, 128, 1, 1, 0, 1), (128, 56, 128, 3, 2, 1, 1),
    (128, 28, 512, 1, 1, 0, 4), (512, 28, 128, 1, 1, 0, 3), (128, 28, 128, 3, 1, 1, 3),
    (512, 28, 1024, 1, 2, 0, 1), (512, 28, 256, 1, 1, 0, 1), (256, 28, 256, 3, 2, 1, 1),
    (256, 14, 1024, 1, 1, 0, 6), (1024, 14, 256, 1, 1, 0, 5), (256, 14, 256, 3, 1, 1, 5),
    (1024, 14, 2048, 1, 2, 0, 1), (1024, 14, 512, 1, 1, 0, 1), (512, 14, 512, 3, 2, 1, 1),
    (512, 7, 2048, 1, 1, 0, 3), (2048, 7, 512, 1, 1, 0, 2), (512, 7, 512, 3, 1, 1, 2),
]
BATCH = 64
# HBM bytes per launch of the dominant kernels come from rocprofv3 FETCH_SIZE + WRITE_SIZE runs of this
# workload (each counter scaled by what it reads for the 2 GiB copy probe of the same run).  Counters
# cannot be read from inside this script, so the figures are read from the committed summary of the
# last counter run, a table keyed on the kernel instantiation name that also records the hashes of
# the kernel sources it was taken with: a kernel that was renamed is not found, and sources that
# changed since make the figure stale -- both give `traffic: null` with the reason beside it.
TRAFFIC_SUMMARY = os.path.join(ROOT, 'profiles', 'bench_hbm_traffic_fetch_write_size.txt')
BRACKETED_IGEMM_LAUNCHES_PER_STEP = 106       # forward + input gradient of the 53 layers


def _sha16(path):
    import hashlib
    with open(path, 'rb') as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def traffic_table(path=TRAFFIC_SUMMARY):
    """({kernel name: (dispatches, bytes per dispatch)}, conv steps in the counter run, None or why the
    table cannot be used)."""
    import re
    rows, steps, sources = {}, None, {}
    try:
        with open(path) as f:
            for line in f:
                m = re.match(r'^(\S.*?)\s{2,}(\d+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$', line)
                if m:
                    rows[m.group(1).strip()] = (int(m.group(2)), float(m.group(5)) * 1e6)
                m = re.match(r'^kernel source (\S+) sha256 (\w+)', line)
                if m:
                    sources[m.group(1)] = m.group(2)
                m = re.match(r'^conv steps per precision in each run: (\d+)', line)
                if m:
                    steps = int(m.group(1))
    except OSError as exc:
        return {}, None, f'no counter summary ({exc})'
    if not rows or not steps or not sources:
        return rows, steps, 'the counter summary holds no table, step count or source hashes'
    for name, sha in sources.items():
        src = os.path.join(ROOT, 'pytortto_amd', 'csrc', name)
        if not os.path.exists(src) or _sha16(src) != sha:
            return rows, steps, f'stale: {name} changed since the counter run'
    return rows, steps, None


def traffic_per_launch(prefixes, launches_per_step=None):
    """Bytes per launch of the kernels whose instantiation names start with one of `prefixes`: the
    mean over their dispatches, or -- with `launches_per_step` -- their bytes per step divided by
    that many bracketed launches.  (None, reason) when the table cannot serve it."""
    rows, steps, why = traffic_table()
    if why:
        return None, why
    hit = {n: v for n, v in rows.items() if any(n == p or n.startswith(p + '<') for p in prefixes)}
    if not hit:
        return None, f'no kernel named {" / ".join(prefixes)} in the counter summary'
    total = sum(d * b for d, b in hit.values())
    if launches_per_step:
        return total / (steps * launches_per_step), None
    return total / sum(d for d, _ in hit.values()), None


BN_SHAPES = [(64, 256, 56, 56), (128, 64, 112, 112)]


def progress(text):
    """A line on stderr (stdout carries the one JSON line): long phases, the host-side baseline above
    all, say that they are alive."""
    print(f'[bench] {text}', file=sys.stderr, flush=True)


def conv_flops(n, c, h, k, r, s, p):
    q = (h + 2 * p - r) // s + 1
    return 2.0 * n * k * c * r * r * q * q, q


class ConvLayer:
    """Device buffers of one convolution shape and the three C-ABI calls on them."""

    def __init__(self, spec, batch, rng):
        from pytortto_amd.xparray import hiparray
        c, h, k, r, s, p, count = spec
        self.spec, self.count, self.batch = spec, count, batch
        self.flops, q = conv_flops(batch, c, h, k, r, s, p)
        bound = 1.0 / np.sqrt(c * r * r)
        self.x = hiparray(rng.standard_normal((batch, c, h, h), dtype=np.float32))
        self.w = hiparray(rng.uniform(-bound, bound, (k, c, r, r)).astype(np.float32))
        self.dy = hiparray(rng.standard_normal((batch, k, q, q), dtype=np.float32))
        self.y = hiparray.empty((batch, k, q, q))
        self.dx = hiparray.empty((batch, c, h, h))
        self.dw = hiparray.empty((k, c, r, r))
        self.args = (batch, c, h, h, k, r, r, s, s, p, p, 1, 1, 1)
        self.q = q
        self.label = f'{c}x{h}x{h}->{k} k{r} s{s} p{p}'
        self.nbytes = 4.0 * (self.x.size + self.w.size + self.y.size)

    def passes(self, call):
        a = self.args
        return {'fwd': lambda: call('tt_conv2d_fwd_f32', self.x.ptr, self.w.ptr, None, self.y.ptr, *a),
                'dgrad': lambda: call('tt_conv2d_dgrad_f32', self.dy.ptr, self.w.ptr, None, self.dx.ptr, *a, self.q, self.q),
                'wgrad': lambda: call('tt_conv2d_wgrad_f32', self.x.ptr, self.dy.ptr, self.dw.ptr, *a, self.q, self.q)}

    def run(self, call):
        a = self.args
        call('tt_conv2d_fwd_f32', self.x.ptr, self.w.ptr, None, self.y.ptr, *a)
        call('tt_conv2d_dgrad_f32', self.dy.ptr, self.w.ptr, None, self.dx.ptr, *a, self.q, self.q)
        call('tt_conv2d_wgrad_f32', self.x.ptr, self.dy.ptr, self.dw.ptr, *a, self.q, self.q)


# PreAct-ResNet-18 basic-block stack on 3x32x32 inputs: the 11 unique convolution shapes, as RESNET50_CONVS
PREACT18_CONVS = [(3, 32, 64, 3, 1, 1, 1), (64, 32, 64, 3, 1, 1, 4), (64, 32, 128, 3, 2, 1, 1), (128, 16, 128, 3, 1, 1, 3),
                  (64, 32, 128, 1, 2, 0, 1), (128, 16, 256, 3, 2, 1, 1), (256, 8, 256, 3, 1, 1, 3), (128, 16, 256, 1, 2, 0, 1),
                  (256, 8, 512, 3, 2, 1, 1), (512, 4, 512, 3, 1, 1, 3), (256, 8, 512, 1, 2, 0, 1)]
# DCGAN generator: (C_in, H_in, C_out, kernel, stride, padding) of the five ConvTranspose2d layers
DCGAN_CONVTS = [(100, 1, 512, 4, 1, 0), (512, 4, 256, 4, 2, 1), (256, 8, 128, 4, 2, 1), (128, 16, 64, 4, 2, 1),
                (64, 32, 3, 4, 2, 1)]


class ConvTransposeLayer:
    """One ConvTranspose2d shape: its forward is the input-gradient call of the convolution with the
    same geometry, its input gradient that convolution's forward call, its weight gradient the
    weight-gradient call with the roles of x and dy exchanged (grad_nn.py:755, :776-778).  Useful
    FLOPs per pass: 2*N*C_in*C_out*R*S*H_in*W_in (the reference's zero-insertion executes stride^2
    times that)."""

    def __init__(self, spec, batch, rng):
        from pytortto_amd.xparray import hiparray
        ci, h, co, r, st, pd = spec
        ho = (h - 1) * st - 2 * pd + (r - 1) + 1
        self.spec, self.count, self.batch = spec, 1, batch
        self.flops = 2.0 * batch * ci * co * r * r * h * h
        bound = 1.0 / np.sqrt(co * r * r)
        self.x = hiparray(rng.standard_normal((batch, ci, h, h), dtype=np.float32))
        self.w = hiparray(rng.uniform(-bound, bound, (ci, co, r, r)).astype(np.float32))
        self.g = hiparray(rng.standard_normal((batch, co, ho, ho), dtype=np.float32))
        self.y, self.dx, self.dw = hiparray.empty((batch, co, ho, ho)), hiparray.empty((batch, ci, h, h)), hiparray.empty((ci, co, r, r))
        self.args = (batch, co, ho, ho, ci, r, r, st, st, pd, pd, 1, 1, 1)
        self.h = h
        self.label = f'{ci}x{h}x{h}->{co}x{ho}x{ho} k{r} s{st} p{pd} (transposed)'
        self.nbytes = 4.0 * (self.x.size + self.w.size + self.y.size)

    def passes(self, call):
        a, h = self.args, self.h
        return {'fwd': lambda: call('tt_conv2d_dgrad_f32', self.x.ptr, self.w.ptr, None, self.y.ptr, *a, h, h),
                'dgrad': lambda: call('tt_conv2d_fwd_f32', self.g.ptr, self.w.ptr, None, self.dx.ptr, *a),
                'wgrad': lambda: call('tt_conv2d_wgrad_f32', self.g.ptr, self.x.ptr, self.dw.ptr, *a, h, h)}


class BnLayer:
    def __init__(self, shape, rng):
        from pytortto_amd.xparray import hiparray
        n, c, h, w = shape
        self.shape = shape
        self.bytes = 4.0 * n * c * h * w
        self.x = hiparray((2 + 3 * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32))
        self.dy = hiparray(rng.standard_normal(shape, dtype=np.float32))
        self.gamma = hiparray(rng.uniform(0.5, 1.5, c).astype(np.float32))
        self.beta = hiparray((0.1 * rng.standard_normal(c)).astype(np.float32))
        self.rm, self.rv = hiparray(np.zeros(c, np.float32)), hiparray(np.ones(c, np.float32))
        self.y, self.dx = hiparray.empty(shape), hiparray.empty(shape)
        self.mean, self.var, self.sd = (hiparray.empty((c,)) for _ in range(3))
        self.dg, self.db = hiparray.empty((c,)), hiparray.empty((c,))
        self.dims = (n, c, h * w)

    def run_fwd(self, call):
        call('tt_bn_fwd_train_f32', self.x.ptr, self.gamma.ptr, self.beta.ptr, self.y.ptr, self.mean.ptr,
             self.var.ptr, self.sd.ptr, self.rm.ptr, self.rv.ptr, self.rm.ptr, self.rv.ptr, None, 0.1, 1e-5, *self.dims)

    def run_bwd(self, call):
        call('tt_bn_bwd_f32', self.x.ptr, self.dy.ptr, self.gamma.ptr, self.mean.ptr, self.var.ptr, self.sd.ptr,
             self.dx.ptr, self.dg.ptr, self.db.ptr, *self.dims)

    def run(self, call):
        self.run_fwd(call)
        self.run_bwd(call)


def bn_passes_separately(hip, call, bns, steps, cold):
    """Forward and backward of every BatchNorm shape bracketed by their own HIP events.  With
    `cold`, 2.3 GB are streamed through the device between the passes (an elementwise add over
    three 768 MB arrays, outside the events), so a pass finds none of its tensors in the 256 MB
    memory-side cache -- the way a network, which runs other layers in between, meets it.  Without,
    the passes follow each other directly on the same tensors, as in the headline figure."""
    from pytortto_amd.xparray import hiparray
    fa = fb = None
    if cold:
        n = 192 << 20
        fa, fb = hiparray.empty((n,)), hiparray.empty((n,))
        call('tt_fill_f32', fa.ptr, 1.0, n)
        call('tt_fill_f32', fb.ptr, 0.0, n)

    def flush():
        if cold:
            call('tt_add_f32', fa.ptr, fb.ptr, fb.ptr, fa.size)

    out = {}
    for b in bns:
        pairs = []
        for it in range(steps + 2):
            flush()
            e0 = hip.Event().record()
            b.run_fwd(call)
            e1 = hip.Event().record()
            flush()
            e2 = hip.Event().record()
            b.run_bwd(call)
            e3 = hip.Event().record()
            if it >= 2:
                pairs.append((e0, e1, e2, e3))
        hip.synchronize()
        fwd = sum(e0.elapsed_ms(e1) for e0, e1, _, _ in pairs) / steps
        bwd = sum(e2.elapsed_ms(e3) for _, _, e2, e3 in pairs) / steps
        out['x'.join(map(str, b.shape))] = {
            'fwd_ms': round(fwd, 4), 'bwd_ms': round(bwd, 4),
            'fwd_gbs': round(3 * b.bytes / (fwd * 1e-3) / 1e9, 1), 'bwd_gbs': round(5 * b.bytes / (bwd * 1e-3) / 1e9, 1),
            'fwd_bwd_gbs': round(8 * b.bytes / ((fwd + bwd) * 1e-3) / 1e9, 1)}
    total_bytes = sum(8 * b.bytes for b in bns)
    total_ms = sum(v['fwd_ms'] + v['bwd_ms'] for v in out.values())
    out['both_shapes_fwd_bwd_gbs'] = round(total_bytes / (total_ms * 1e-3) / 1e9, 1)
    out['both_shapes_pct_of_peak'] = round(100 * total_bytes / (total_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 1)
    del fa, fb
    return out


def timed_steps(hip, step, steps, warmup):
    """(ms per step from HIP events on the library stream, wall-clock ms per step)."""
    for _ in range(warmup):
        step()
    hip.synchronize()
    t0 = time.perf_counter()
    e0 = hip.Event().record()
    for _ in range(steps):
        step()
    e1 = hip.Event().record()
    ms = e0.elapsed_ms(e1)
    hip.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    return ms / steps, wall / steps


def profiled_steps(hip, step, steps):
    hip.profile_enable(True)
    for _ in range(steps):
        step()
    prof = hip.profile_read()
    hip.profile_enable(False)
    return prof


def per_layer_table(hip, call, layers, reps):
    """Forward, input gradient and weight gradient of every unique shape timed on their own
    (HIP events on the library stream around `reps` back-to-back calls after 3 warm-up calls; the
    weight gradient includes its float64 reduce, the input gradient its weight repack).  The
    per-layer roofline is min(fp32 MFMA peak, AI * 8 TB/s) with AI = F / (4 * (|x| + |w| + |y|)):
    the three passes of a layer move the same three tensors' worth of bytes."""
    rows = []
    for l in layers:
        ai = l.flops / l.nbytes
        roof = min(PEAK_FP32_MFMA_TFLOPS, ai * PEAK_HBM_GBS / 1e3)
        row = {'shape': l.label, 'count': l.count, 'gflop': round(l.flops / 1e9, 3),
               'ai_flop_per_byte': round(ai, 1), 'roofline_tflops': round(roof, 1)}
        for name, fn in l.passes(call).items():
            ms, _ = timed_steps(hip, fn, reps, 3)
            tf = l.flops / (ms * 1e-3) / 1e12
            row[name] = {'ms': round(ms, 4), 'tflops': round(tf, 1), 'frac_of_roofline': round(tf / roof, 3)}
        rows.append(row)
    return rows


def table_totals(rows):
    """Time and rate of one step made of the rows' passes (every occurrence of every shape)."""
    ms = sum(r['count'] * (r['fwd']['ms'] + r['dgrad']['ms'] + r['wgrad']['ms']) for r in rows)
    gflop = sum(3 * r['count'] * r['gflop'] for r in rows)
    return {'layers_ms_summed': round(ms, 3), 'gflop': round(gflop, 2), 'tflops': round(gflop / ms, 2),
            'frac_of_fp32_mfma_peak': round(gflop / ms / PEAK_FP32_MFMA_TFLOPS, 4)}


def single_layer_config(hip, call, rng, reps=200):
    """The CPU-runnable baseline configuration on the GPU: Conv2d(16, 32, 3, padding=1, bias) on
    x [32,16,32,32], forward (with bias), input gradient, weight gradient and bias gradient.  At 0.3
    GFLOP per pass every call is one launch of a few microseconds: the figures are bound by launch
    and ramp-up, not by the matrix pipe, and say so."""
    from pytortto_amd.xparray import hiparray
    x = hiparray(rng.standard_normal((32, 16, 32, 32), dtype=np.float32))
    w = hiparray(rng.uniform(-1 / 12, 1 / 12, (32, 16, 3, 3)).astype(np.float32))
    b = hiparray(rng.uniform(-1 / 12, 1 / 12, 32).astype(np.float32))
    dy = hiparray(rng.standard_normal((32, 32, 32, 32), dtype=np.float32))
    y, dx, dw, db = hiparray.empty(dy.shape), hiparray.empty(x.shape), hiparray.empty(w.shape), hiparray.empty((32,))
    a = (32, 16, 32, 32, 32, 3, 3, 1, 1, 1, 1, 1, 1, 1)
    flops = 2.0 * 32 * 32 * 16 * 9 * 32 * 32
    nbytes = 4.0 * (x.size + w.size + y.size)
    roof = min(PEAK_FP32_MFMA_TFLOPS, flops / nbytes * PEAK_HBM_GBS / 1e3)
    passes = {'fwd': lambda: call('tt_conv2d_fwd_f32', x.ptr, w.ptr, b.ptr, y.ptr, *a),
              'dgrad': lambda: call('tt_conv2d_dgrad_f32', dy.ptr, w.ptr, None, dx.ptr, *a, 32, 32),
              'wgrad': lambda: call('tt_conv2d_wgrad_f32', x.ptr, dy.ptr, dw.ptr, *a, 32, 32),
              'bias_grad': lambda: call('tt_channel_sum_f32', dy.ptr, db.ptr, 32, 32, 1024)}
    out = {'config': {'workload': 'Conv2d(16, 32, 3, padding=1, bias) on x [32,16,32,32], fwd + dgrad + wgrad + bias gradient; '
                                  '0.302 GFLOP per pass'},
           'roofline_tflops': round(roof, 1), 'ai_flop_per_byte': round(flops / nbytes, 1)}
    total = 0.0
    for name, fn in passes.items():
        ms, _ = timed_steps(hip, fn, reps, 10)
        total += ms
        out[name] = {'ms': round(ms, 5)}
        if name != 'bias_grad':
            tf = flops / (ms * 1e-3) / 1e12
            out[name].update(tflops=round(tf, 2), frac_of_roofline=round(tf / roof, 3))

    def whole():
        for fn in passes.values():
            fn()
    ms, wall = timed_steps(hip, whole, reps, 10)
    tf = 3 * flops / (ms * 1e-3) / 1e12
    out.update(value=round(tf, 2), unit='TFLOP/s', ms_per_step=round(ms, 5), wall_ms_per_step=round(wall, 5),
               frac_of_roofline=round(tf / roof, 3),
               note='launch-bound: each pass is one to three kernels of 5-15 us; back-to-back launches overlap their ramp-up, '
                    'so the step is shorter than the sum of the passes timed alone')
    return out


def resnet50_train_step(hip, steps, warmup, batch=BATCH):
    """Whole ResNet-50 training steps through the module API (the network of the reference's
    examples/resnet/resnet50_finetune notebook, 10 classes): forward, NLL loss, backward, SGD with
    momentum, everything on the device.  Returns (images/s, ms per step from HIP events, wall ms)."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    F = nn.functional

    def conv3x3(cin, cout, stride=1):
        return nn.Conv2d(cin, cout, kernel_size=3, stride=stride, padding=1, bias=False)

    def conv1x1(cin, cout, stride=1):
        return nn.Conv2d(cin, cout, kernel_size=1, stride=stride, bias=False)

    class Bottleneck(nn.Module):
        def __init__(self, cin, width, stride=1, downsample=None):
            super().__init__()
            self.conv1, self.bn1 = conv1x1(cin, width), nn.BatchNorm2d(width)
            self.conv2, self.bn2 = conv3x3(width, width, stride), nn.BatchNorm2d(width)
            self.conv3, self.bn3 = conv1x1(width, width * 4), nn.BatchNorm2d(width * 4)
            self.downsample = downsample

        def forward(self, x):
            shortcut = x if self.downsample is None else self.downsample(x)
            out = F.relu(self.bn1(self.conv1(x)))
            out = F.relu(self.bn2(self.conv2(out)))
            out = self.bn3(self.conv3(out))
            return F.relu(out + shortcut)

    class ResNet50(nn.Module):
        def __init__(self, classes=10):
            super().__init__()
            self.conv1 = nn.Conv2d(3, 64, kernel_size=7, stride=2, padding=3, bias=False)
            self.bn1 = nn.BatchNorm2d(64)
            self.maxpool = nn.MaxPool2d(kernel_size=3, stride=2, padding=1)
            blocks, cin = [], 64
            for width, count, stride in ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)):
                for i in range(count):
                    down = None
                    if i == 0:
                        down = nn.Sequential(conv1x1(cin, width * 4, stride), nn.BatchNorm2d(width * 4))
                    blocks.append(Bottleneck(cin, width, stride if i == 0 else 1, down))
                    cin = width * 4
            self.layers = nn.Sequential(*blocks)
            self.classifier = nn.Linear(2048, classes)

        def forward(self, x):
            x = self.maxpool(F.relu(self.bn1(self.conv1(x))))
            x = self.layers(x)
            x = tt.flatten(tt.mean(x, (-1, -2), True), 1)
            return F.log_softmax(self.classifier(x), -1)

    tt.manual_seed(0)
    net = ResNet50()
    net.cuda()
    opt = tt.optim.SGD(net.parameters(), lr=0.001, momentum=0.9)
    rng = np.random.default_rng(0)
    x = tt.tensor(rng.standard_normal((batch, 3, 224, 224), dtype=np.float32)).cuda()
    target = tt.tensor(rng.integers(0, 10, batch)).cuda()
    losses = []

    def step():
        opt.zero_grad()
        loss = F.nll_loss(net(x), target)
        loss.backward()
        opt.step()
        return loss

    for _ in range(warmup):
        losses.append(step().item())
    ms, wall = timed_steps(hip, step, steps, 0)
    losses.append(step().item())
    del net, opt, x
    return batch / (wall * 1e-3), ms, wall, losses


def preact18_stack_step(hip, steps, warmup, batch=128):
    """Forward + backward of the PreAct-ResNet-18 basic-block stack of the reference's
    examples/resnet/preact_resnet18 notebook at batch 128, 3x32x32, through the module API: conv3x3
    3->64, stages (64, 128, 256, 512) of two blocks, block = BN-ReLU -> [conv3x3(stride) - BN - ReLU -
    conv3x3] + shortcut (identity, or conv1x1 stride 2 on the block input), no biases, BatchNorm in
    training mode, upstream gradient on the last stage's output.  Returns (ms per step, wall ms)."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    F = nn.functional

    class Block(nn.Module):
        def __init__(self, cin, cout, stride):
            super().__init__()
            self.bn1, self.conv1 = nn.BatchNorm2d(cin), nn.Conv2d(cin, cout, 3, stride, 1, bias=False)
            self.bn2, self.conv2 = nn.BatchNorm2d(cout), nn.Conv2d(cout, cout, 3, 1, 1, bias=False)
            self.shortcut = None if stride == 1 and cin == cout else nn.Conv2d(cin, cout, 1, stride, bias=False)

        def forward(self, x):
            out = self.conv1(F.relu(self.bn1(x)))
            out = self.conv2(F.relu(self.bn2(out)))
            return out + (x if self.shortcut is None else self.shortcut(x))

    tt.manual_seed(0)
    layers, cin = [nn.Conv2d(3, 64, 3, 1, 1, bias=False)], 64
    for cout, stride in ((64, 1), (128, 2), (256, 2), (512, 2)):
        layers += [Block(cin, cout, stride), Block(cout, cout, 1)]
        cin = cout
    net = nn.Sequential(*layers)
    net.cuda()
    rng = np.random.default_rng(0)
    x = tt.tensor(rng.standard_normal((batch, 3, 32, 32), dtype=np.float32)).cuda()
    g = tt.tensor(rng.standard_normal((batch, 512, 4, 4), dtype=np.float32)).cuda()

    def step():
        for q in net.parameters():
            q.grad = None
        net(x).backward(g)

    ms, wall = timed_steps(hip, step, steps, warmup)
    del net, x, g
    return ms, wall


def dcgan_generator_step(hip, steps, warmup, batch=128):
    """Forward + backward of the DCGAN-style generator: latent [batch,100,1,1] -> ConvTranspose2d
    4x4 stride 1 to 512 channels, then 4x4 / stride 2 / padding 1 to 256, 128, 64 and 3 channels
    (64x64), BatchNorm2d + ReLU between, no biases.  Returns (ms per step, wall ms)."""
    import pytortto_amd as tt
    from pytortto_amd import nn
    tt.manual_seed(0)
    layers, cin = [], 100
    for cout, stride, pad in ((512, 1, 0), (256, 2, 1), (128, 2, 1), (64, 2, 1)):
        layers += [nn.ConvTranspose2d(cin, cout, 4, stride, pad, bias=False), nn.BatchNorm2d(cout), nn.ReLU()]
        cin = cout
    layers.append(nn.ConvTranspose2d(cin, 3, 4, 2, 1, bias=False))
    net = nn.Sequential(*layers)
    net.cuda()
    rng = np.random.default_rng(0)
    z = tt.tensor(rng.standard_normal((batch, 100, 1, 1), dtype=np.float32)).cuda()
    g = tt.tensor(rng.standard_normal((batch, 3, 64, 64), dtype=np.float32)).cuda()

    def step():
        for q in net.parameters():
            q.grad = None
        net(z).backward(g)

    ms, wall = timed_steps(hip, step, steps, warmup)
    del net, z, g
    return ms, wall


def cpu_baseline_pool(batch):
    """(bytes counted, seconds) of the oracle's MaxPool2d forward + backward."""
    import oracle
    rng = np.random.default_rng(0)
    x = rng.standard_normal((batch, 64, 112, 112), dtype=np.float32)
    t0 = time.perf_counter()
    y, pos = oracle.max_pool2d(x, (3, 3), (2, 2), (1, 1))
    oracle.max_pool2d_backward(x.shape, y, pos, (3, 3), (2, 2), (1, 1))
    sec = time.perf_counter() - t0
    return 2 * (x.nbytes + 2 * y.nbytes), sec


def cpu_threads():
    try:
        from threadpoolctl import threadpool_info
        blas = [p for p in threadpool_info() if p.get('user_api') == 'blas']
        if blas:
            return max(p['num_threads'] for p in blas)
    except Exception:
        pass
    return len(os.sched_getaffinity(0))


def cpu_baseline_conv(batch):
    """Oracle fwd + dgrad + wgrad, once per unique ResNet-50 shape, at the given batch."""
    import oracle
    rng = np.random.default_rng(0)
    flops = 0.0
    seconds = 0.0
    for c, h, k, r, s, p, _count in RESNET50_CONVS:
        f, q = conv_flops(batch, c, h, k, r, s, p)
        x = rng.standard_normal((batch, c, h, h), dtype=np.float32)
        w = rng.standard_normal((k, c, r, r), dtype=np.float32)
        dy = rng.standard_normal((batch, k, q, q), dtype=np.float32)
        t0 = time.perf_counter()
        _, xpad = oracle.convolution_forward(x, w, None, (s, s), (p, p), (1, 1), 1)
        oracle.convolution_backward(dy, x, xpad, w, (s, s), (p, p), (1, 1), 1, need=(True, True, False))
        seconds += time.perf_counter() - t0
        flops += 3 * f
        progress(f'cpu baseline, batch {batch}: {c}x{h}x{h}->{k} k{r} s{s} done, {seconds:.1f} s so far')
    return flops, seconds


def cpu_baseline_c1(reps=5):
    """Oracle forward + backward of the single-layer baseline configuration at its full size:
    Conv2d(16, 32, 3, padding=1, bias) on x [32,16,32,32].  (flops counted, median seconds)"""
    import oracle
    rng = np.random.default_rng(0)
    x = rng.standard_normal((32, 16, 32, 32), dtype=np.float32)
    w = rng.uniform(-1 / 12, 1 / 12, (32, 16, 3, 3)).astype(np.float32)
    b = rng.uniform(-1 / 12, 1 / 12, 32).astype(np.float32)
    dy = rng.standard_normal((32, 32, 32, 32), dtype=np.float32)
    times = []
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        _, xpad = oracle.convolution_forward(x, w, b, (1, 1), (1, 1), (1, 1), 1)
        oracle.convolution_backward(dy, x, xpad, w, (1, 1), (1, 1), (1, 1), 1)
        times.append(time.perf_counter() - t0)
    return 3 * 2.0 * 32 * 32 * 16 * 9 * 32 * 32, float(np.median(times[1:]))


def cpu_baseline_bn(batch_div):
    import oracle
    rng = np.random.default_rng(0)
    nbytes = 0.0
    seconds = 0.0
    for n, c, h, w in BN_SHAPES:
        shape = (max(1, n // batch_div), c, h, w)
        x = (2 + 3 * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)
        dy = rng.standard_normal(shape, dtype=np.float32)
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = np.zeros(c, np.float32)
        rm, rv = np.zeros(c, np.float32), np.ones(c, np.float32)
        t0 = time.perf_counter()
        _, saved, _, _ = oracle.batch_norm_forward(x, gamma, beta, rm, rv, True, 0.1, 1e-5)
        oracle.batch_norm_backward(dy, x, gamma, saved)
        seconds += time.perf_counter() - t0
        nbytes += 8 * x.nbytes
    return nbytes, seconds


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=10)
    ap.add_argument('--warmup', type=int, default=3)
    ap.add_argument('--no-cpu-baseline', action='store_true', help='skip the host-side oracle timing')
    ap.add_argument('--cpu-batch', type=int, default=BATCH,
                    help='batch of the CPU baseline over the 23 ResNet-50 shapes (default: the benchmark batch, 64; '
                         'about 2.5 minutes of host time)')
    ap.add_argument('--no-model-step', action='store_true', help='skip the whole-network ResNet-50 training step')
    ap.add_argument('--model-step-only', action='store_true',
                    help='run only the whole-network ResNet-50 training step and print its object (for profiling)')
    ap.add_argument('--no-per-layer', action='store_true',
                    help='skip the per-layer table (profiling runs: keeps the launch counts of a trace to whole steps)')
    ap.add_argument('--per-layer-only', action='store_true',
                    help='print only the per-layer table of the 23 ResNet-50 convolution shapes (for profiling)')
    ap.add_argument('--stack-only', choices=('preact', 'dcgan'),
                    help='run only the PreAct-ResNet-18 stack or the DCGAN generator stack and print its object '
                         '(for profiling)')
    args = ap.parse_args()
    if args.gpus != 1:
        print(f'bench.py: this path runs on exactly one GPU (asked for --gpus {args.gpus}); '
              f'nothing in it is sharded (it would shard by batch: one all-reduce of the weight gradients, and of the '
              f'per-channel BatchNorm moments between the two sweeps)', file=sys.stderr)
        sys.exit(2)

    from pytortto_amd import _hip
    from pytortto_amd.xparray import hiparray
    from pytortto_amd._paths import LIB_PATH
    if not os.path.exists(LIB_PATH):
        from pytortto_amd.build import build_library
        build_library()
    info = _hip.device_info()
    call = _hip.call
    rng = np.random.default_rng(0)
    if args.stack_only:
        fn = preact18_stack_step if args.stack_only == 'preact' else dcgan_generator_step
        gflop = 142.19 if args.stack_only == 'preact' else 26.78
        s_ms, s_wall = fn(_hip, args.steps, args.warmup)   # the full run uses at least 50 steps after 20 warm-up steps
        print(json.dumps({'metric': f'{args.stack_only} stack fwd+bwd through the module API', 'value': round(s_wall, 3),
                          'unit': 'ms', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
                          'ms_per_step': round(s_wall, 3), 'gpu_ms_per_step': round(s_ms, 3),
                          'higher_is_better': False, 'dtype': 'f32', 'data': 'synthetic',
                          'conv_tflops_equivalent': round(3 * gflop * 1e9 / (s_wall * 1e-3) / 1e12, 2)}))
        return
    if args.model_step_only:
        ips, m_ms, m_wall, m_losses = resnet50_train_step(_hip, args.steps, args.warmup)
        print(json.dumps({'metric': 'ResNet-50 training step images/s (module API)', 'value': round(ips, 1),
                          'unit': 'images/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
                          'ms_per_step': round(m_wall, 2), 'gpu_ms_per_step': round(m_ms, 2), 'batch': BATCH,
                          'higher_is_better': True, 'dtype': 'f32', 'data': 'synthetic',
                          'loss_first_last': [round(m_losses[0], 4), round(m_losses[-1], 4)]}))
        return

    # ---- convolution: ResNet-50, batch 64 ------------------------------------------------------
    layers = [ConvLayer(spec, BATCH, rng) for spec in RESNET50_CONVS]
    flops_per_pass = sum(l.flops * l.count for l in layers)
    assert abs(flops_per_pass / 1e9 - 523.15) < 0.05, flops_per_pass
    if args.per_layer_only:
        rows = per_layer_table(_hip, call, layers, max(args.steps, 20))
        print(json.dumps({'metric': 'per-layer conv fwd / dgrad / wgrad of the 23 unique ResNet-50 shapes, batch 64',
                          'unit': 'ms, TFLOP/s', 'n_gpus': 1, 'steps': max(args.steps, 20), 'warmup': 3,
                          'dtype': 'f32', 'data': 'synthetic', 'per_layer': rows}))
        return

    def conv_step():
        for l in layers:
            for _ in range(l.count):
                l.run(call)

    progress('calibration probes, then the convolution step')
    # ---- what the device sustains on the two bounding resources, measured in this run ----------
    # (first: 0.2 s of dense matrix work and 8 GiB of streaming also bring the device from idle to
    # its sustained clocks before anything is timed; with 3 warm-up steps alone the first timed
    # steps still run on the ramp)
    mfma_mean, mfma_min, mfma_max = _hip.probe_mfma(100)
    hbm_read, hbm_copy = _hip.probe_hbm(2 << 30)

    conv_ms, conv_wall_ms = timed_steps(_hip, conv_step, args.steps, args.warmup)
    conv_tflops = 3 * flops_per_pass / (conv_ms * 1e-3) / 1e12
    prof = profiled_steps(_hip, conv_step, args.steps)
    # dominant kernel: igemm_f32 (forward and input-gradient launches); algorithmic flops per
    # launch = 2*N*K*C*R*S*P*Q of the layer, summed over the launches of one step
    n_fwd, ms_fwd = prof['conv_igemm_fwd']
    n_dg, ms_dg = prof['conv_igemm_dgrad']
    igemm_flops = 2 * flops_per_pass * args.steps
    igemm_tflops = igemm_flops / ((ms_fwd + ms_dg) * 1e-3) / 1e12
    n_wg, ms_wg = prof['conv_wgrad']
    wgrad_tflops = flops_per_pass * args.steps / (ms_wg * 1e-3) / 1e12
    kernel_ms = {k: round(v[1] / args.steps, 4) for k, v in prof.items() if v[0]}
    progress('per-layer table of the 23 shapes')
    layer_rows = None if args.no_per_layer else per_layer_table(_hip, call, layers, 20)
    c1_gpu = None if args.no_per_layer else single_layer_config(_hip, call, rng)   # (kept out of profiling runs)

    progress('convolution step with bf16 arithmetic')
    # optional reduced-precision variant, reported separately and never part of `value`: the three
    # passes on bf16 MFMA (operands rounded inside the kernels, fp32 accumulation and tensors)
    _hip.set_conv_math('bf16')
    try:
        bf_ms, _ = timed_steps(_hip, conv_step, args.steps, args.warmup)
        bf_prof = profiled_steps(_hip, conv_step, args.steps)
    finally:
        _hip.set_conv_math('f32')
    bf_igemm_ms = bf_prof['conv_igemm_fwd'][1] + bf_prof['conv_igemm_dgrad'][1]
    bf_igemm_tflops = igemm_flops / (bf_igemm_ms * 1e-3) / 1e12
    bf16_variant = {
        'metric': 'conv fwd+bwd TFLOP/s on bf16 MFMA (forward, input gradient, weight gradient)',
        'value': round(3 * flops_per_pass / (bf_ms * 1e-3) / 1e12, 2), 'unit': 'TFLOP/s',
        'ms_per_step': round(bf_ms, 3), 'dtype': 'bf16 operands, f32 accumulation, f32 tensors in memory',
        'error_bound': 'max|y - y_f32| <= 1e-2 * max|y_f32| (measured 2-3e-3); exact against the oracle on '
                       'bf16-rounded operands to the f32 tolerance',
        'roofline': {'bound': 'mfma', 'kernel': 'igemm_bf16 (Conv2d forward + input gradient)',
                     'achieved': round(bf_igemm_tflops, 2), 'peak': PEAK_BF16_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': round(bf_igemm_tflops / PEAK_BF16_MFMA_TFLOPS, 4), 'traffic': None,
                     'speedup_over_f32_kernel': round((ms_fwd + ms_dg) / bf_igemm_ms, 2),
                     'note': 'tensors stay fp32 in HBM.  Forward and stride-1 input gradients run on bf16-first kernels '
                             '(operands converted on their way into LDS, 32-deep chunks): their 1x1 layers move their bytes at '
                             'HBM speed, their 3x3 layers are bound by the address unit (one 4-byte gathered element per lane); '
                             'launches with fewer tiles than compute units and long reductions, strided input gradients and the '
                             'stem stay on the float32 kernels\' bf16 instantiations'},
        'wgrad_tflops': round(flops_per_pass * args.steps / (bf_prof['conv_wgrad'][1] * 1e-3) / 1e12, 2),
        'kernels_ms_per_step': {k: round(v[1] / args.steps, 4) for k, v in bf_prof.items() if v[0]}}
    progress('convolution step in float32 arithmetic on the bf16 matrix instructions (three terms)')
    # the other optional variant, also reported separately and never part of `value`: float32
    # arithmetic carried out on the bf16 matrix pipe (every operand element as three exact bf16
    # terms, six products per step); it meets the float32 tolerances
    _hip.set_conv_math('bf16x3')
    try:
        x3_ms, _ = timed_steps(_hip, conv_step, args.steps, args.warmup)
        x3_prof = profiled_steps(_hip, conv_step, args.steps)
    finally:
        _hip.set_conv_math('f32')
    x3_igemm_ms = x3_prof['conv_igemm_fwd'][1] + x3_prof['conv_igemm_dgrad'][1]
    x3_igemm_tflops = igemm_flops / (x3_igemm_ms * 1e-3) / 1e12
    x3_peak = PEAK_BF16_MFMA_TFLOPS / 6.0
    bf16x3_variant = {
        'metric': 'conv fwd+bwd TFLOP/s, float32 arithmetic on bf16 MFMA (forward and input gradient; weight gradient on fp32 MFMA)',
        'value': round(3 * flops_per_pass / (x3_ms * 1e-3) / 1e12, 2), 'unit': 'TFLOP/s',
        'ms_per_step': round(x3_ms, 3), 'speedup_over_f32_step': round(conv_ms / x3_ms, 3),
        'dtype': 'f32 operands as three exact bf16 terms each, six bf16 MFMAs per product step, f32 accumulation',
        'error_bound': 'the float32 tolerances (rtol 1e-4 / atol 1e-5 against the oracle): the three products of terms left '
                       'out stay below 2^-24 of a product',
        'roofline': {'bound': 'mfma', 'kernel': 'igemm_bf16x3 (Conv2d forward + input gradient)',
                     'achieved': round(x3_igemm_tflops, 2), 'peak': round(x3_peak, 1), 'unit': 'TFLOP/s',
                     'frac': round(x3_igemm_tflops / x3_peak, 4), 'traffic': None,
                     'speedup_over_f32_kernel': round((ms_fwd + ms_dg) / x3_igemm_ms, 2),
                     'note': 'peak = the bf16 MFMA peak divided by the six matrix instructions a product step takes; '
                             'achieved = useful float32 FLOPs (2*N*K*C*R*S*P*Q) per second.  The kernels are bound by the '
                             'chain fetch -> LDS -> matrix instructions of a 16-deep chunk, which the two blocks of a compute unit '
                             'run in step: in throw-away builds the kernel without any matrix instruction still takes 55 % as long, '
                             'and the parts add up'},
        'wgrad_tflops': round(flops_per_pass * args.steps / (x3_prof['conv_wgrad'][1] * 1e-3) / 1e12, 2),
        'kernels_ms_per_step': {k: round(v[1] / args.steps, 4) for k, v in x3_prof.items() if v[0]}}
    del layers
    call('tt_empty_cache')

    progress('BatchNorm shapes')
    # ---- BatchNorm2d training fwd+bwd -----------------------------------------------------------
    bns = [BnLayer(s, rng) for s in BN_SHAPES]
    bn_bytes = sum(8 * b.bytes for b in bns)

    def bn_step():
        for b in bns:
            b.run(call)

    bn_ms, bn_wall_ms = timed_steps(_hip, bn_step, args.steps, args.warmup)
    bn_gbs = bn_bytes / (bn_ms * 1e-3) / 1e9
    per_shape = {}
    for b in bns:
        ms, _ = timed_steps(_hip, lambda: b.run(call), args.steps, 1)
        per_shape['x'.join(map(str, b.shape))] = round(8 * b.bytes / (ms * 1e-3) / 1e9, 1)
    bprof = profiled_steps(_hip, bn_step, args.steps)
    bn_kernel_ms = {k: round(v[1] / args.steps, 4) for k, v in bprof.items() if v[0]}
    # dominant kernel: bn_bwd_apply (reads x, dy, writes dx: 3*S algorithmic bytes per launch)
    n_ba, ms_ba = bprof['bn_bwd_apply']
    bwd_apply_gbs = sum(3 * b.bytes for b in bns) * args.steps / (ms_ba * 1e-3) / 1e9
    bn_warm = bn_passes_separately(_hip, call, bns, args.steps, cold=False)
    bn_cold = bn_passes_separately(_hip, call, bns, args.steps, cold=True)
    del bns
    call('tt_empty_cache')

    progress('MaxPool2d and elementwise kernels')
    # ---- rows either side of the path: MaxPool2d (ResNet-50 stem pooling) and the activations ---
    pool_shape, pool_args = (BATCH, 64, 112, 112), (3, 3, 2, 2, 1, 1, 1, 1)
    px = hiparray(rng.standard_normal(pool_shape, dtype=np.float32))
    py = hiparray.empty((BATCH, 64, 56, 56))
    ptap = hiparray.empty((BATCH, 64, 56, 56), np.int32)
    pdx = hiparray.empty(pool_shape)
    pool_dims = (BATCH * 64, 112, 112, 56, 56)

    def pool_step():
        call('tt_maxpool2d_fwd_f32', px.ptr, py.ptr, ptap.ptr, *pool_dims, *pool_args)
        call('tt_maxpool2d_bwd_f32', py.ptr, ptap.ptr, pdx.ptr, *pool_dims, *pool_args)

    pool_ms, _ = timed_steps(_hip, pool_step, args.steps, args.warmup)
    pprof = profiled_steps(_hip, pool_step, args.steps)
    # algorithmic bytes: forward reads x, writes y and the int32 taps; backward reads dy and taps, writes dx
    pool_fwd_bytes = px.nbytes + py.nbytes + ptap.nbytes
    pool_bytes = 2 * pool_fwd_bytes
    n_pb, ms_pb = pprof['maxpool_bwd']
    n_pf, ms_pf = pprof['maxpool_fwd']
    pool_bwd_gbs = pool_fwd_bytes * n_pb / (ms_pb * 1e-3) / 1e9
    act = {}
    for name, fn, nbytes in (
            ('relu_fwd', lambda: call('tt_relu_fwd_f32', px.ptr, pdx.ptr, px.size), 2 * px.nbytes),
            ('relu_bwd', lambda: call('tt_relu_bwd_f32', px.ptr, pdx.ptr, pdx.ptr, px.size), 3 * px.nbytes),
            ('leaky_relu_fwd', lambda: call('tt_leaky_relu_fwd_f32', px.ptr, pdx.ptr, 0.2, px.size), 2 * px.nbytes),
            ('add', lambda: call('tt_add_f32', px.ptr, pdx.ptr, pdx.ptr, px.size), 3 * px.nbytes)):
        ms, _ = timed_steps(_hip, fn, args.steps, 2)
        act[name] = round(nbytes / (ms * 1e-3) / 1e9, 1)
    cpu_pool = None
    if not args.no_cpu_baseline:
        nb, sec = cpu_baseline_pool(32)
        cpu_pool = {'value': round(nb / sec / 1e9, 3), 'unit': 'GB/s', 'cores': 1, 'kind': 'port',
                    'sample': f'oracle MaxPool2d fwd+bwd at [32,64,112,112] ({nb / 1e9:.2f} GB counted, {sec:.1f} s)'}
    del px, py, ptap, pdx
    call('tt_empty_cache')

    progress('whole ResNet-50 training step')
    # ---- the whole network through the module API ---------------------------------------------
    model = None
    if not args.no_model_step:
        ips, m_ms, m_wall, m_losses = resnet50_train_step(_hip, max(3, args.steps // 2), 2)
        model = {'metric': 'ResNet-50 training step images/s (module API: forward, NLL loss, backward, SGD momentum)',
                 'value': round(ips, 1), 'unit': 'images/s', 'ms_per_step': round(m_wall, 2),
                 'gpu_ms_per_step': round(m_ms, 2), 'batch': BATCH,
                 'loss_first_last': [round(m_losses[0], 4), round(m_losses[-1], 4)],
                 'note': 'wall clock around the Python loop, launches asynchronous; fp32, synthetic 3x224x224 input'}
        call('tt_empty_cache')
        _hip.set_conv_math('bf16')   # the optional variant, reported beside the fp32 figure
        try:
            b_ips, b_ms, b_wall, b_losses = resnet50_train_step(_hip, max(3, args.steps // 2), 2)
        finally:
            _hip.set_conv_math('f32')
        model['with_bf16_conv_math'] = {'value': round(b_ips, 1), 'unit': 'images/s', 'ms_per_step': round(b_wall, 2),
                                        'loss_first_last': [round(b_losses[0], 4), round(b_losses[-1], 4)]}
        call('tt_empty_cache')
        _hip.set_conv_math('bf16x3')   # float32 arithmetic on the bf16 matrix instructions: same tolerances as fp32
        try:
            t_ips, t_ms, t_wall, t_losses = resnet50_train_step(_hip, max(3, args.steps // 2), 2)
        finally:
            _hip.set_conv_math('f32')
        model['with_bf16x3_conv_math'] = {'value': round(t_ips, 1), 'unit': 'images/s', 'ms_per_step': round(t_wall, 2),
                                          'loss_first_last': [round(t_losses[0], 4), round(t_losses[-1], 4)]}
        call('tt_empty_cache')

    progress('PreAct-ResNet-18 and DCGAN stacks')
    # ---- the other two stack configurations: per layer, then whole stacks through the module API ---
    stack_rows = {}
    if not args.no_per_layer:
        for key, cls, specs in (('preact_resnet18_stack', ConvLayer, PREACT18_CONVS),
                                ('dcgan_generator_stack', ConvTransposeLayer, DCGAN_CONVTS)):
            ls = [cls(spec, 128, rng) for spec in specs]
            rows = per_layer_table(_hip, call, ls, 30)
            stack_rows[key] = {'rows': rows, 'all_layers': table_totals(rows)}
            del ls
            call('tt_empty_cache')
    stacks = None
    if not args.no_model_step:
        # steps of 1-6 ms: enough of them that the first ones (pool refill after tt_empty_cache, clock
        # ramp after the host-side pause) do not set the figure
        s_steps, s_warmup = max(args.steps, 50), max(args.warmup, 20)
        p_ms, p_wall = preact18_stack_step(_hip, s_steps, s_warmup)
        call('tt_empty_cache')
        d_ms, d_wall = dcgan_generator_step(_hip, s_steps, s_warmup)
        call('tt_empty_cache')
        # convolution FLOPs of one pass (2*N*K*C*R*S*P*Q summed over the layers); forward, input
        # gradient and weight gradient each count it once
        stacks = {'preact_resnet18_stack': {
                      'metric': 'PreAct-ResNet-18 basic-block stack fwd+bwd (conv + BatchNorm + ReLU + shortcuts)',
                      'config': {'workload': 'batch 128, 3x32x32, 20 convolutions, 142.19 GFLOP per pass'},
                      'ms_per_step': round(p_wall, 3), 'gpu_ms_per_step': round(p_ms, 3),
                      'conv_tflops_equivalent': round(3 * 142.19e9 / (p_wall * 1e-3) / 1e12, 2),
                      'per_layer': stack_rows.get('preact_resnet18_stack')},
                  'dcgan_generator_stack': {
                      'metric': 'DCGAN generator fwd+bwd (ConvTranspose2d + BatchNorm + ReLU)',
                      'config': {'workload': 'batch 128, latent 100 -> 3x64x64, 5 transposed convolutions, '
                                             '26.78 GFLOP per pass'},
                      'ms_per_step': round(d_wall, 3), 'gpu_ms_per_step': round(d_ms, 3),
                      'conv_tflops_equivalent': round(3 * 26.78e9 / (d_wall * 1e-3) / 1e12, 2),
                      'per_layer': stack_rows.get('dcgan_generator_stack')},
                  'note': 'whole stacks, every kernel counted in the time, only convolution FLOPs in the rate; '
                          'the input of the first layer needs no gradient, so its input-gradient pass does not run.  '
                          'per_layer: every unique convolution shape of the stack at batch 128 timed alone (30 calls '
                          'after 3 warm-up calls), each with its own roofline min(157.3, AI * 8 TB/s); transposed '
                          'layers count useful FLOPs 2*N*C_in*C_out*R*S*H_in*W_in'}
    elif stack_rows:
        stacks = {k: {'per_layer': v} for k, v in stack_rows.items()}

    progress('CPU baseline (oracle on the host cores)')
    # ---- CPU baseline (oracle on the host cores) -------------------------------------------------
    cpu_conv = cpu_bn = None
    if not args.no_cpu_baseline:
        cores = cpu_threads()
        f, sec = cpu_baseline_conv(args.cpu_batch)
        cpu_conv = {'value': round(f / sec / 1e12, 4), 'unit': 'TFLOP/s', 'cores': cores, 'kind': 'port',
                    'sample': f'oracle fwd+dgrad+wgrad once over the 23 unique ResNet-50 conv shapes at batch '
                              f'{args.cpu_batch}{" (the benchmark batch)" if args.cpu_batch == BATCH else ""} '
                              f'({f / 1e9:.0f} GFLOP counted, {sec:.1f} s, one repetition per shape)'}
        if args.cpu_batch != 8:
            f8, sec8 = cpu_baseline_conv(8)
            cpu_conv['at_batch_8'] = {'value': round(f8 / sec8 / 1e12, 4), 'unit': 'TFLOP/s', 'cores': cores, 'kind': 'port',
                                      'sample': f'the same 23 shapes at batch 8 ({f8 / 1e9:.0f} GFLOP counted, {sec8:.1f} s)'}
        f1, sec1 = cpu_baseline_c1()
        cpu_conv['single_layer_config_full_size'] = {
            'value': round(f1 / sec1 / 1e12, 4), 'unit': 'TFLOP/s', 'cores': cores, 'kind': 'port',
            'sample': f'oracle Conv2d(16,32,3,padding=1) fwd+bwd on x [32,16,32,32], the CPU-runnable configuration at '
                      f'full size ({f1 / 1e9:.2f} GFLOP counted, median of 5 runs {sec1 * 1e3:.1f} ms)'}
        nb, sec = cpu_baseline_bn(1)
        cpu_bn = {'value': round(nb / sec / 1e9, 3), 'unit': 'GB/s', 'cores': cores, 'kind': 'port',
                  'sample': f'oracle BatchNorm fwd+bwd at both shapes, full batch ({nb / 1e9:.2f} GB counted, '
                            f'{sec:.1f} s)'}

    igemm_traffic, igemm_traffic_why = traffic_per_launch(('igemm_f32', 'igemm_multi_f32'), BRACKETED_IGEMM_LAUNCHES_PER_STEP)
    bn_traffic, bn_traffic_why = traffic_per_launch(('bn_bwd_apply',))
    pool_traffic, pool_traffic_why = traffic_per_launch(('maxpool_bwd_scatter',))
    out = {
        'metric': 'conv fwd+bwd TFLOP/s (% fp32 MFMA peak); BatchNorm2d fwd+bwd GB/s (% HBM)',
        'value': round(conv_tflops, 2), 'unit': 'TFLOP/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': round(conv_ms, 3), 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'ResNet-50 convolutions (53 layers, 23 unique shapes), batch 64, 3x224x224: '
                               'fwd + dgrad + wgrad of every layer per step, 1569.5 GFLOP',
                   'global_batch': BATCH, 'device': info['name'].strip(), 'compute_units': info['compute_units']},
        'pct_of_peak': round(100 * conv_tflops / PEAK_FP32_MFMA_TFLOPS, 1),
        'wall_ms_per_step': round(conv_wall_ms, 3),
        'roofline': {'bound': 'mfma', 'kernel': 'igemm_f32 (Conv2d forward + input gradient)',
                     'achieved': round(igemm_tflops, 2), 'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': round(igemm_tflops / PEAK_FP32_MFMA_TFLOPS, 4),
                     'traffic': igemm_traffic, 'traffic_note': igemm_traffic_why,
                     'sustained_peak_measured': {'mean': round(mfma_mean, 1), 'min': round(mfma_min, 1),
                                                 'max': round(mfma_max, 1), 'unit': 'TFLOP/s',
                                                 'what': '100 launches of dense v_mfma_f32_32x32x2_f32, '
                                                         'per-lane varying operands'},
                     'launches_per_step': (n_fwd + n_dg) // args.steps,
                     'avg_launch_ms': round((ms_fwd + ms_dg) / max(1, n_fwd + n_dg), 5)},
        'kernels_ms_per_step': kernel_ms,
        'wgrad_tflops': round(wgrad_tflops, 2),
        'per_layer': {'what': 'each unique shape and pass timed alone, 20 back-to-back calls after 3 warm-up calls; '
                              'roofline_tflops = min(157.3, AI * 8 TB/s), AI = F / (4 * (|x| + |w| + |y|))',
                      'rows': layer_rows},
        'conv_bf16_variant': bf16_variant,
        'conv_bf16x3_variant': bf16x3_variant,
        'cpu_baseline': cpu_conv,
        'single_layer_config': c1_gpu,
        'bn': {'metric': 'BatchNorm2d training fwd+bwd GB/s', 'value': round(bn_gbs, 1), 'unit': 'GB/s',
               'ms_per_step': round(bn_ms, 4), 'wall_ms_per_step': round(bn_wall_ms, 4),
               'pct_of_peak': round(100 * bn_gbs / PEAK_HBM_GBS, 1),
               'config': {'workload': 'BatchNorm2d train fwd+bwd fp32 NCHW at [64,256,56,56] and [128,64,112,112], '
                                      'x ~ N(2,3), 8*S algorithmic bytes per shape'},
               'per_shape_gbs': per_shape,
               'passes_back_to_back': bn_warm,
               'passes_cold_cache': dict(bn_cold, what='2.3 GB streamed through the device before each pass, outside '
                                                       'the events: no tensor of the pass is left in the 256 MB '
                                                       'memory-side cache; `value` above is the back-to-back figure'),
               'roofline': {'bound': 'hbm', 'kernel': 'bn_bwd_apply (reads x, dy; writes dx)',
                            'achieved': round(bwd_apply_gbs, 1), 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                            'frac': round(bwd_apply_gbs / PEAK_HBM_GBS, 4),
                            'traffic': bn_traffic, 'traffic_note': bn_traffic_why,
                            'sustained_measured': {'read_gbs': round(hbm_read, 1), 'copy_gbs': round(hbm_copy, 1),
                                                   'what': '2 GiB streamed, 16 KiB contiguous per block'},
                            'avg_launch_ms': round(ms_ba / max(1, n_ba), 5)},
               'kernels_ms_per_step': bn_kernel_ms,
               'cpu_baseline': cpu_bn},
        'maxpool': {'metric': 'MaxPool2d fwd+bwd GB/s', 'value': round(pool_bytes / (pool_ms * 1e-3) / 1e9, 1),
                    'unit': 'GB/s', 'ms_per_step': round(pool_ms, 4),
                    'pct_of_peak': round(100 * pool_bytes / (pool_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 1),
                    'config': {'workload': 'MaxPool2d(3, stride 2, padding 1) fwd+bwd fp32 NCHW at [64,64,112,112] '
                                           '(ResNet-50 stem pooling); bytes: x + y + int32 taps, both ways'},
                    'roofline': {'bound': 'hbm', 'kernel': 'maxpool_bwd_scatter (reads dy, taps; writes dx)',
                                 'achieved': round(pool_bwd_gbs, 1), 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                                 'frac': round(pool_bwd_gbs / PEAK_HBM_GBS, 4),
                                 'traffic': pool_traffic, 'traffic_note': pool_traffic_why,
                                 'avg_launch_ms': round(ms_pb / max(1, n_pb), 5)},
                    'kernels_ms_per_step': {'maxpool_fwd': round(ms_pf / max(1, n_pf), 4),
                                            'maxpool_bwd': round(ms_pb / max(1, n_pb), 4)},
                    'elementwise_gbs_at_same_size': act,
                    'cpu_baseline': cpu_pool},
        'resnet50_step': model,
        'stacks': stacks,
    }
    print(json.dumps(out))


if __name__ == '__main__':
    main()
