"""CPU tests of the host-side mirror of tortto's API (no GPU, no compute through the C ABI)."""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle
import pytortto_amd as tt
from pytortto_amd import nn
from pytortto_amd.build import LIB_PATH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, 'include', 'tortto_hip.h')).read()
    declared = set(re.findall(r'\b(tt_[a-z0-9_]+)\s*\(', header))
    assert len(declared) >= 25
    assert os.path.exists(LIB_PATH), 'libtortto_hip.so has not been built (python -m pytortto_amd.build)'
    lib = ctypes.CDLL(LIB_PATH)
    missing = [name for name in sorted(declared) if not hasattr(lib, name)]
    assert not missing, f'symbols declared in include/tortto_hip.h but not exported: {missing}'
    from pytortto_amd import _hip
    assert declared == set(_hip.PROTOTYPES) | {'tt_last_error'}
    _hip.load_library()     # attaches every prototype; makes no GPU call


def test_seeded_conv2d_parameters_match_reference_draw_order():
    tt.manual_seed(0)
    conv = nn.Conv2d(16, 32, 3, stride=1, padding=1, bias=True)
    x = tt.randn(2, 3)
    np.random.seed(0)
    w, b = oracle.conv_parameters(16, 32, (3, 3))
    np.testing.assert_array_equal(conv.weight.data, w)
    np.testing.assert_array_equal(conv.bias.data, b)
    np.testing.assert_array_equal(x.data, np.random.randn(2, 3).astype(np.float32))
    assert conv.weight.requires_grad and conv.weight.is_leaf and conv.weight.dtype == np.float32


def test_conv_transpose_weight_layout_and_output_padding():
    tt.manual_seed(1)
    m = nn.ConvTranspose2d(8, 6, 3, stride=2, padding=1, groups=2)
    assert m.weight.shape == (8, 3, 3, 3) and m.bias.shape == (6,)
    x = tt.zeros(1, 8, 5, 5)
    assert list(m._output_padding(x, None, m.stride, m.padding, m.kernel_size, m.dilation)) == [0]
    assert m._output_padding(x, (10, 10), m.stride, m.padding, m.kernel_size, m.dilation) == [1, 1]
    assert m._output_padding(x, (1, 6, 9, 10), m.stride, m.padding, m.kernel_size, m.dilation) == [0, 1]
    with pytest.raises(ValueError, match='requested an output size'):
        m._output_padding(x, (12, 12), m.stride, m.padding, m.kernel_size, m.dilation)
    with pytest.raises(ValueError, match='Only "zeros" padding mode'):
        nn.ConvTranspose2d(4, 4, 3, padding_mode='reflect')


def test_constructor_errors():
    with pytest.raises(ValueError, match='in_channels must be divisible by groups'):
        nn.Conv2d(3, 4, 3, groups=2)
    with pytest.raises(ValueError, match='out_channels must be divisible by groups'):
        nn.Conv2d(4, 3, 3, groups=2)
    with pytest.raises(ValueError, match='padding_mode must be one of'):
        nn.Conv2d(4, 4, 3, padding_mode='circular')


def test_host_tensors_are_refused_by_the_hot_path():
    conv = nn.Conv2d(2, 2, 1)
    with pytest.raises(RuntimeError, match='device \\(HIP\\) path only'):
        conv(tt.randn(1, 2, 4, 4))
    bn = nn.BatchNorm2d(2)
    with pytest.raises(RuntimeError, match='device \\(HIP\\) path only'):
        bn(tt.randn(2, 2, 4, 4))
    with pytest.raises(ValueError, match='expected 4D input'):
        bn(tt.randn(2, 2, 4))
    with pytest.raises(RuntimeError, match='Expected 3D \\(unbatched\\) or 4D \\(batched\\) input to conv2d'):
        conv(tt.randn(1, 1, 2, 4, 4))
    with pytest.raises(RuntimeError, match='expected input'):
        conv(tt.randn(1, 3, 4, 4))


def test_batchnorm_module_state():
    bn = nn.BatchNorm2d(5)
    sd = bn.state_dict()
    assert list(sd) == ['weight', 'bias', 'running_mean', 'running_var', 'num_batches_tracked']
    assert sd['num_batches_tracked'].dtype == np.float32 and sd['num_batches_tracked'].shape == ()
    np.testing.assert_array_equal(sd['running_var'], np.ones(5, np.float32))
    assert all(type(v) is np.ndarray for v in sd.values())
    bn2 = nn.BatchNorm2d(5, affine=False, track_running_stats=False)
    assert bn2.weight is None and bn2.running_mean is None and list(bn2.state_dict()) == []


def test_state_dict_round_trip_and_errors():
    tt.manual_seed(3)
    a = nn.Sequential(nn.Conv2d(2, 3, 3), nn.BatchNorm2d(3), nn.ReLU())
    b = nn.Sequential(nn.Conv2d(2, 3, 3), nn.BatchNorm2d(3), nn.ReLU())
    assert not np.array_equal(a[0].weight.data, b[0].weight.data)
    res = b.load_state_dict(a.state_dict())
    assert repr(res) == '<All keys matched successfully>'
    np.testing.assert_array_equal(a[0].weight.data, b[0].weight.data)
    bad = a.state_dict()
    bad.pop('1.running_mean')
    bad['extra'] = np.zeros(1)
    with pytest.raises(RuntimeError, match='Missing key\\(s\\).*\n.*Unexpected key'):
        b.load_state_dict(bad)
    wrong = a.state_dict()
    wrong['0.weight'] = np.zeros((3, 2, 1, 1), np.float32)
    with pytest.raises(RuntimeError, match='size mismatch for 0.weight'):
        b.load_state_dict(wrong)


def test_module_registry_and_repr():
    net = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1, bias=False), nn.BatchNorm2d(8), nn.ReLU(inplace=True))
    names = [n for n, _ in net.named_parameters()]
    assert names == ['0.weight', '1.weight', '1.bias']
    assert len(list(net.modules())) == 4 and len(net) == 3
    assert 'Conv2d(3, 8, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), bias=False)' in repr(net)
    net.eval()
    assert not net[1].training
    net.train()
    assert net[1].training
    with pytest.raises(KeyError):
        net.register_buffer('a.b', None)
    with pytest.raises(TypeError):
        net.register_parameter('p', tt.zeros(1))


def test_autograd_engine_on_host_add_relu():
    """Engine semantics the path relies on: AccumulateGrad on leaves, gradient accumulation when
    a tensor feeds two consumers (residual shortcut), grad_fn naming, cleared nodes."""
    x = tt.tensor(np.array([-1.0, 2.0, 3.0], np.float32), requires_grad=True)
    r = tt.nn.functional.relu(x)
    y = r + x                     # x is used twice
    assert y.grad_fn.__class__.__name__ == 'AddBackward' and r.grad_fn.__class__.__name__ == 'ReluBackward'
    y.backward(tt.tensor(np.array([1.0, 10.0, 100.0], np.float32)))
    np.testing.assert_array_equal(x.grad, np.array([1.0, 20.0, 200.0], np.float32))
    assert type(x.grad) is np.ndarray
    y2 = tt.nn.functional.relu(x)
    y2.backward(tt.tensor(np.ones(3, np.float32)))
    np.testing.assert_array_equal(x.grad, np.array([1.0, 21.0, 201.0], np.float32))   # accumulates
    with tt.no_grad():
        z = tt.nn.functional.relu(x)
    assert z.grad_fn is None and not z.requires_grad
    with pytest.raises(RuntimeError, match='does not require grad'):
        z.backward()


def test_inplace_version_check():
    x = tt.tensor(np.array([1.0, -2.0], np.float32), requires_grad=True)
    with pytest.raises(RuntimeError, match='leaf Variable that requires grad'):
        tt.nn.functional.relu(x, inplace=True)
    a = x + x
    b = tt.nn.functional.relu(a)          # saves its output
    tt.nn.functional.relu(b, inplace=True)  # bumps b's version
    with pytest.raises(RuntimeError, match='modified by an inplace operation'):
        b.backward(tt.tensor(np.ones(2, np.float32)))


def test_cpu_copy_is_a_no_op_on_host_and_numpy_rules():
    x = tt.randn(2, 2)
    assert x.cpu() is x and x.device == 'cpu'
    assert x.numpy() is x.data
    x.requires_grad_(True)
    with pytest.raises(RuntimeError, match="Can't call numpy\\(\\) on Tensor that requires grad"):
        x.numpy()


def test_optimizer_plumbing_on_host():
    """Parameter groups, defaults, validation and state_dict layout need no GPU."""
    import pytortto_amd as tt
    lin = tt.nn.Linear(4, 2)
    opt = tt.optim.SGD([{'params': [lin.weight]}, {'params': [lin.bias], 'lr': 0.5}], lr=0.1, momentum=0.9)
    assert [g['lr'] for g in opt.param_groups] == [0.1, 0.5] and opt.param_groups[1]['momentum'] == 0.9
    sd = opt.state_dict()
    assert sd['param_groups'][0]['params'] == [0] and sd['param_groups'][1]['params'] == [1]
    opt.load_state_dict(sd)
    with pytest.raises(ValueError, match='Nesterov momentum requires a momentum and zero dampening'):
        tt.optim.SGD(lin.parameters(), lr=0.1, nesterov=True)
    with pytest.raises(ValueError, match='Invalid beta parameter at index 0'):
        tt.optim.Adam(lin.parameters(), betas=(1.0, 0.9))
    with pytest.raises(ValueError, match='empty parameter list'):
        tt.optim.Adam([])
    with pytest.raises(TypeError, match='iterable of Tensors or dicts'):
        tt.optim.SGD(lin.weight, lr=0.1)
    with pytest.raises(ValueError, match='more than one parameter group'):
        tt.optim.SGD([{'params': [lin.weight]}, {'params': [lin.weight]}], lr=0.1)
    with pytest.raises(ValueError, match="can't optimize a non-leaf Tensor"):
        tt.optim.SGD([lin.weight + lin.weight], lr=0.1)
    assert tt.optim.AdamW(lin.parameters()).defaults['weight_decay'] == 1e-2
    assert 'lr: 0.1' in repr(opt)


def test_checkpoint_wire_format_round_trip(tmp_path):
    """tt.save writes {'data': obj} as one pickled object in a .npy file; a model's state_dict
    (parameters and BatchNorm buffers, host arrays) survives the round trip."""
    tt.manual_seed(5)
    net = nn.Sequential(nn.Conv2d(3, 4, 3, bias=True), nn.BatchNorm2d(4), nn.ReLU())
    net[1].running_mean.data[...] = np.arange(4, dtype=np.float32)
    sd = net.state_dict()
    assert list(sd) == ['0.weight', '0.bias', '1.weight', '1.bias', '1.running_mean', '1.running_var',
                        '1.num_batches_tracked']
    path = str(tmp_path / 'ckpt.npy')
    tt.save({'model': sd, 'epoch': 3}, path)
    raw = np.load(path, allow_pickle=True)
    assert raw.dtype == object and raw.shape == () and set(raw.item()) == {'data'}
    back = tt.load(path)
    assert back['epoch'] == 3
    other = nn.Sequential(nn.Conv2d(3, 4, 3, bias=True), nn.BatchNorm2d(4), nn.ReLU())
    other.load_state_dict(back['model'])
    for k, v in other.state_dict().items():
        assert type(v) is np.ndarray
        np.testing.assert_array_equal(v, sd[k])
    with pytest.raises(RuntimeError, match='Missing key'):
        other.load_state_dict({k: v for k, v in sd.items() if k != '1.running_var'})


def test_host_relu_while_a_device_operation_is_parked(monkeypatch):
    """A host ReLU must not look for a device buffer on its input: with a device BatchNorm or Add
    still parked, relu(host tensor) takes tortto's NumPy expression and leaves the parked operation
    alone.  (Stand-ins for the parked objects: nothing here touches a GPU.)"""
    from pytortto_amd import _hip, ops

    class _Out:
        _buf = object()

    for cls, field in ((ops.DeferredBatchNorm, 'y'), (ops.DeferredAdd, 'out')):
        fake = object.__new__(cls)
        setattr(fake, field, _Out())
        monkeypatch.setattr(_hip, '_pending', fake)
        for inplace in (False, True):
            x = tt.tensor(np.array([-1.0, 2.0, -3.0], np.float32))
            y = tt.nn.functional.relu(x, inplace=inplace)
            np.testing.assert_array_equal(y.data, np.array([0.0, 2.0, 0.0], np.float32))
        assert _hip.pending() is fake
    monkeypatch.setattr(_hip, '_pending', None)


def test_parked_operation_slot_is_atomic_and_poisons_on_failure():
    """take_pending_if tests and takes in one step; an operation that fails when it is flushed marks
    its outputs so that they raise instead of handing out memory nobody wrote."""
    from pytortto_amd import _hip
    from pytortto_amd.xparray import poison

    class Op:
        ran = 0

        def run(self):
            Op.ran += 1

    op = Op()
    _hip.defer(op)
    assert _hip.take_pending_if(lambda o: False) is None and _hip.pending() is op
    assert _hip.take_pending_if(lambda o: o is op) is op and _hip.pending() is None
    _hip.defer(op)
    _hip.flush()
    assert Op.ran == 1 and _hip.pending() is None

    class Buf:
        on_demand = None

    class Arr:
        def __init__(self):
            self._buf = Buf()

    class Failing:
        def __init__(self):
            self.out = Arr()

        def run(self):
            raise RuntimeError('shape limit')

        def poison(self, exc):
            poison([self.out, None], exc)

    bad = Failing()
    _hip.defer(bad)
    with pytest.raises(RuntimeError, match='shape limit'):
        _hip.flush()
    assert _hip.pending() is None
    for _ in range(2):                      # stays poisoned
        with pytest.raises(RuntimeError, match='shape limit'):
            bad.out._buf.on_demand(bad.out._buf)


def test_runs_of_a_long_batch_start_aligned():
    """Batches of 2^31 elements or more are cut into runs of images; every run but the first starts
    `per` images in, and the kernels need 16-byte aligned pointers: per * image must be a multiple of
    four elements for both tensors, whatever the image sizes."""
    import ctypes
    from pytortto_amd import _hip
    lib = _hip.load_library()

    def per_run(n, a, b):
        out = ctypes.c_int()
        assert lib.tt_conv2d_images_per_run(n, a, b, ctypes.byref(out)) == 0
        return out.value

    assert per_run(64, 3 * 224 * 224, 64 * 112 * 112) == 64              # fits: one run
    for image_a, image_b in [(2 ** 20, 2 ** 20), (3 * 333 * 333, 5 * 167 * 167), (7 * 1001 * 999, 3 * 501 * 500),
                             (1000003, 999983), (2 ** 20 + 2, 2 ** 19 + 1), (2 ** 30 + 1, 5)]:
        n = 3 * (2 ** 31) // max(image_a, image_b) + 7
        per = per_run(n, image_a, image_b)
        if per == 0:        # only when not even one image keeps the runs aligned
            assert max(image_a, image_b) * 4 > 2 ** 31 - 2 and (image_a % 4 or image_b % 4)
            continue
        assert 1 <= per < n and per * max(image_a, image_b) < 2 ** 31
        assert (per * image_a) % 4 == 0 and (per * image_b) % 4 == 0, (per, image_a, image_b)
        assert (per + 4) * max(image_a, image_b) >= 2 ** 31 - 1            # not needlessly short
