"""BASELINE config 3 on REAL activations: one forward / backward of a ResNet-50 (the
network the layer list of the benchmark comes from, built here as torch modules, random
weights) at batch 32, 224x224, through the hooks and SecondOrderOptimizer.step, all 54
Kronecker layers and 53 BatchNorm layers.  Post-ReLU inputs (non-negative, a dominant mean
direction) and rank-deficient output-gradient factors (2048 channels from 1568 positions)
are what the synthetic N(0,1) layer set of the benchmark does not have.  Asserts that
every one of the 108 factors was positive definite, and rechecks the factors, the
pi-damped inverses and the preconditioned gradients of ten layers of every kind in float64
on the device; inverses beside the reference's float32 result (scipy.linalg.inv) on the
same damped matrix."""
import os
import sys

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from test_gpu_bench_step import TOL, conv_a_float64, inverse_record, rel   # noqa: E402

pytestmark = pytest.mark.gpu

PICKED = ['conv1', 'layer1.0.conv1', 'layer1.0.conv2', 'layer2.0.conv2', 'layer3.0.downsample',
          'layer4.0.conv2', 'layer4.2.conv2', 'layer4.2.conv3', 'fc', 'layer3.1.bn2']


def test_resnet50_step_on_real_activations():
    import bench
    import torchsso
    from torchsso.curv import curvature as _curv
    dev = torch.device('cuda:0')
    specs = bench.resnet50_specs()
    torch.manual_seed(1)
    model = bench.build_resnet50().to(dev)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(32, 3, 224, 224, generator=gen).to(dev)
    y = torch.randint(0, 1000, (32,), generator=gen).to(dev)
    opt = torchsso.optim.SecondOrderOptimizer(
        model, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron', 'BatchNorm2d': 'Diag'},
        {'damping': 1e-3, 'ema_decay': 0.95}, lr=1e-3, momentum=0.9)
    groups = opt.param_groups
    assert len(groups) == len(specs) == 107
    names = [s['name'] for s in specs]
    picked = {names.index(n): n for n in PICKED}
    raw, bn_before = {}, {}

    def closure():
        opt.zero_grad()
        out = model(x)
        loss = F.cross_entropy(out, y)
        loss.backward()
        for i in picked:
            raw[i] = [p.grad.detach().clone() for p in groups[i]['params']]
            if specs[i]['kind'] == 'bn':
                bn_before[i] = [p.detach().clone() for p in groups[i]['params']]
        return loss, out

    loss, _ = opt.step(closure=closure)
    torch.cuda.synchronize()
    assert torch.isfinite(loss)

    kron = [g['curv'] for g in groups if g['curv'].kind == 'kron']
    info = torch.cat([c.info for c in kron]).cpu()
    assert info.numel() == 108 and int((info != 0).sum()) == 0, info.nonzero().flatten().tolist()
    _curv.check_spd_all(kron)
    for g in groups:
        for p in g['params']:
            assert torch.isfinite(p).all() and torch.isfinite(p.grad).all()

    worst, bounds = {}, {}
    for i, name in picked.items():
        s, g = specs[i], groups[i]
        curv, mod = g['curv'], g['curv'].module
        go = mod.grad_output
        n = go.shape[0]
        if s['kind'] == 'bn':
            w0, b0 = bn_before[i]
            xhat = (mod.data_output.detach().double() - b0.double().view(1, -1, 1, 1)) / \
                w0.double().view(1, -1, 1, 1)
            sx = (xhat * xhat).sum((2, 3))
            sg = (go.double() ** 2).sum((2, 3))
            want = [(sx * sg).mean(0) * n * n, sg.mean(0) * n * n]
            for k in range(2):
                worst['bn ema'] = max(worst.get('bn ema', 0.), rel(curv.ema[k], want[k]))
                worst['bn inv'] = max(worst.get('bn inv', 0.),
                                      rel(curv.inv[k], 1. / (curv.ema[k].double() + 1e-3)))
            continue
        xin = mod.data_input
        if isinstance(mod, nn.Conv2d):
            assert (mod.in_channels, mod.out_channels, mod.kernel_size[0]) == (s['cin'], s['cout'], s['k'])
            A = conv_a_float64(xin, s)
            hw = go.shape[2] * go.shape[3]
            gm = go.double().permute(1, 0, 2, 3).reshape(go.shape[1], -1)
            G = gm @ gm.t() * (float(n) / hw)
        else:
            xa = torch.cat([xin.double(), torch.ones(n, 1, dtype=torch.float64, device=dev)], 1)
            A = xa.t() @ xa / n
            G = go.double().t() @ go.double() * float(n)
        # first step: the running average is the factor itself
        worst['A'] = max(worst.get('A', 0.), rel(curv.ema[0], A))
        worst['G'] = max(worst.get('G', 0.), rel(curv.ema[1], G))
        del A, G
        eA, eG = curv.ema[0].double(), curv.ema[1].double()
        pi = ((eA.diagonal().sum() / eA.shape[0]) / (eG.diagonal().sum() / eG.shape[0])).sqrt()
        r = 1e-3 ** 0.5
        for tag, X, shift, Y in (('A', eA, r * pi, curv.inv[0]), ('G', eG, r / pi, curv.inv[1])):
            key = '%s %s inverse' % (name, tag)
            _, e_dev, e_ref, _, _ = inverse_record(key, X, shift.item(), Y)
            worst[key] = e_dev
            bounds[key] = max(TOL, 1.5 * e_ref)
        V = raw[i][0].reshape(raw[i][0].shape[0], -1).double()
        ps = g['params']
        got = ps[0].grad.reshape(ps[0].shape[0], -1).double()
        if len(ps) > 1:
            V = torch.cat([V, raw[i][1].double()[:, None]], 1)
            got = torch.cat([got, ps[1].grad.double()[:, None]], 1)
        want = curv.inv[1].double() @ V @ curv.inv[0].double()
        worst['preconditioned gradient'] = max(worst.get('preconditioned gradient', 0.), rel(got, want))
        del eA, eG
    print('resnet50 on real activations, worst rel. Frobenius errors:',
          {k: '%.2e' % v for k, v in worst.items()}, flush=True)
    for k, v in worst.items():
        assert v <= bounds.get(k, TOL), (k, v, bounds.get(k, TOL))
