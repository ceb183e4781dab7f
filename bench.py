"""K-FAC step benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload resnet50|alexnet_fc|convnet|mlp|noisy_kfac|resnet50_train]
                    [--factor-mode grouped|eager] [--factor-streams N] [--factor-flush-work W]
                    [--explicit-inverse] [--no-cpu-baseline] [--no-other-workloads]
                    [--copy-calibration]

A "step" is one pass of the K-FAC hot path over one batch of synthetic input,
driven through the public torchsso API: for every layer the two Kronecker
factors are built from that layer's input and output gradient (the forward hooks
in layer order, then the backward hooks in reverse order, as in a training pass;
they queue the products, which run in a few grouped engine calls), then
SecondOrderOptimizer.step() runs the running
average, the pi-damped inversion of all factors, the preconditioning of all
gradients and the parameter update.  The default workload is BASELINE config 3:
the 53 convolutions + fc of a ResNet-50 at batch 32, 224x224 (real per-layer
activation / gradient shapes, N(0,1) data), with diagonal curvature for the 53
BatchNorm layers.  All inputs are resident in HBM before the timed region.
`--workload noisy_kfac` is BASELINE config 5: VIOptimizer.step on config 2's
network, 4 MC samples, timed from the second step (forward and backward of the
network included: the factor products run inside its hooks).
`--workload resnet50_train` times whole training steps of the ResNet-50 itself (forward,
backward, K-FAC step on real activations) beside plain SGD steps of the same network.

Prints ONE JSON line.  `value` is the step time in ms; `host_enqueue_ms` the host's
own time to enqueue a step; `roofline.executed_*` come from the library's tile plan.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, 'pytorch-sso_amd'))
sys.path.insert(0, ROOT)

METRIC = 'K-FAC step ms (factor+invert+precondition) & fp32 MFMA TFLOP/s, 1 MI355X'
PEAK_FP32_MFMA_TFLOPS = 157.3
# rocprofv3 --pmc readings of the factor-build kernels of a resnet50 step, kept with the
# profile summary they come from (counter runs cannot be made from inside this script):
#   traffic_bytes_per_launch   HBM bytes per launch (FETCH_SIZE, WRITE_SIZE, calibrated)
#   executed_flop_per_step_pmc 512 x SQ_INSTS_VALU_MFMA_MOPS_F32
# The second one is the check on the plan arithmetic below: if the flops this script
# derives from the library's tile / split plan differ from it by more than 3 %, the plan
# has changed since the counters were read, and the line says so instead of quoting them.
PMC_SUMMARY = os.path.join(ROOT, 'profiles', 'factor_build_resnet50_b32_hbm_traffic.txt')


def read_pmc_summary(path=PMC_SUMMARY):
    vals = {}
    try:
        with open(path) as f:
            for line in f:
                parts = line.split('=')
                if len(parts) == 2 and parts[0].strip() in ('traffic_bytes_per_launch',
                                                            'executed_flop_per_step_pmc'):
                    vals[parts[0].strip()] = float(parts[1].split()[0])
    except OSError:
        pass
    return vals


# ---------------------------------------------------------------------------
# workloads: lists of layer specs with the real shapes
# ---------------------------------------------------------------------------

def conv_spec(name, cin, cout, k, stride, pad, hin, bias=False):
    hout = (hin + 2 * pad - k) // stride + 1
    return dict(kind='conv', name=name, cin=cin, cout=cout, k=k, stride=stride, pad=pad,
                hin=hin, hout=hout, bias=bias)


def resnet50_specs():
    """ResNet-50 (Bottleneck [3,4,6,3], stride on the 3x3 conv, conv bias=False,
    fc with bias), 224x224 input: 53 convs + fc, each conv followed by a BatchNorm."""
    specs = [conv_spec('conv1', 3, 64, 7, 2, 3, 224)]
    specs.append(dict(kind='bn', name='bn1', c=64, h=112))
    h = 56
    inplanes = 64
    for li, (planes, blocks, stride) in enumerate([(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)]):
        for b in range(blocks):
            s = stride if b == 0 else 1
            pre = 'layer%d.%d.' % (li + 1, b)
            specs.append(conv_spec(pre + 'conv1', inplanes, planes, 1, 1, 0, h))
            specs.append(dict(kind='bn', name=pre + 'bn1', c=planes, h=h))
            specs.append(conv_spec(pre + 'conv2', planes, planes, 3, s, 1, h))
            hout = specs[-1]['hout']
            specs.append(dict(kind='bn', name=pre + 'bn2', c=planes, h=hout))
            specs.append(conv_spec(pre + 'conv3', planes, planes * 4, 1, 1, 0, hout))
            specs.append(dict(kind='bn', name=pre + 'bn3', c=planes * 4, h=hout))
            if b == 0:
                specs.append(conv_spec(pre + 'downsample', inplanes, planes * 4, 1, s, 0, h))
                specs.append(dict(kind='bn', name=pre + 'downsample.bn', c=planes * 4, h=hout))
            inplanes = planes * 4
            h = hout
    specs.append(dict(kind='linear', name='fc', fin=2048, fout=1000, bias=True))
    return specs


def alexnet_fc_specs():
    return [dict(kind='linear', name='fc6', fin=9216, fout=4096, bias=True),
            dict(kind='linear', name='fc7', fin=4096, fout=4096, bias=True),
            dict(kind='linear', name='fc8', fin=4096, fout=1000, bias=True)]


def convnet_specs():
    return [conv_spec('conv1', 3, 64, 5, 1, 0, 32, bias=True),
            conv_spec('conv2', 64, 128, 5, 1, 0, 14, bias=True),
            dict(kind='linear', name='fc1', fin=3200, fout=384, bias=True),
            dict(kind='linear', name='fc2', fin=384, fout=192, bias=True),
            dict(kind='linear', name='fc3', fin=192, fout=10, bias=True)]


def mlp_specs():
    return [dict(kind='linear', name='l1', fin=784, fout=1000, bias=True),
            dict(kind='linear', name='l2', fin=1000, fout=1000, bias=True),
            dict(kind='linear', name='l3', fin=1000, fout=10, bias=True)]


WORKLOADS = {
    'resnet50': (resnet50_specs, 32, 'resnet50_kfac_layerset_batch32_224x224 (BASELINE config 3)'),
    'alexnet_fc': (alexnet_fc_specs, 256, 'alexnet_fc6-8_batch256 (BASELINE config 4)'),
    'convnet': (convnet_specs, 128, 'convnet_batch128 (BASELINE config 2)'),
    'mlp': (mlp_specs, 128, 'mlp_784-1000-1000-10_batch128 (BASELINE config 1)'),
}


def build_resnet50(num_classes=1000):
    """The network config 3's layer list comes from, as torch modules: ResNet-50 with
    Bottleneck blocks [3, 4, 6, 3], the stride of a stage on its first block's 3x3
    convolution, bias-free convolutions each followed by BatchNorm, a 1x1 projection on the
    first block of every stage, global average pooling and a 2048 -> classes linear layer.
    Module order = resnet50_specs() order (used by the tests that run the K-FAC step on
    real activations and by --workload resnet50_train)."""
    import torch.nn as nn
    import torch.nn.functional as F

    class Block(nn.Module):
        def __init__(self, inplanes, planes, stride, project):
            super(Block, self).__init__()
            self.conv1 = nn.Conv2d(inplanes, planes, 1, bias=False)
            self.bn1 = nn.BatchNorm2d(planes)
            self.conv2 = nn.Conv2d(planes, planes, 3, stride, 1, bias=False)
            self.bn2 = nn.BatchNorm2d(planes)
            self.conv3 = nn.Conv2d(planes, 4 * planes, 1, bias=False)
            self.bn3 = nn.BatchNorm2d(4 * planes)
            if project:
                self.downsample = nn.Conv2d(inplanes, 4 * planes, 1, stride, bias=False)
                self.downsample_bn = nn.BatchNorm2d(4 * planes)
            else:
                self.downsample = None

        def forward(self, x):
            y = F.relu(self.bn1(self.conv1(x)))
            y = F.relu(self.bn2(self.conv2(y)))
            y = self.bn3(self.conv3(y))
            skip = x if self.downsample is None else self.downsample_bn(self.downsample(x))
            return F.relu(y + skip)

    class Net(nn.Module):
        def __init__(self):
            super(Net, self).__init__()
            self.conv1 = nn.Conv2d(3, 64, 7, 2, 3, bias=False)
            self.bn1 = nn.BatchNorm2d(64)
            blocks, inplanes = [], 64
            for planes, count, stride in ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)):
                for b in range(count):
                    blocks.append(Block(inplanes, planes, stride if b == 0 else 1, b == 0))
                    inplanes = 4 * planes
            self.blocks = nn.Sequential(*blocks)
            self.fc = nn.Linear(2048, num_classes)

        def forward(self, x):
            x = F.max_pool2d(F.relu(self.bn1(self.conv1(x))), 3, 2, 1)
            x = self.blocks(x)
            return self.fc(x.mean(dim=(2, 3)))

    return Net()


def spec_dims(s, batch):
    """(dA, dG, L) of a Kron layer."""
    if s['kind'] == 'conv':
        return (s['cin'] * s['k'] * s['k'] + (1 if s['bias'] else 0), s['cout'],
                batch * s['hout'] * s['hout'])
    return s['fin'] + (1 if s['bias'] else 0), s['fout'], batch


def algorithmic_work(specs, batch):
    """Flops of the dense formulation (what the reference's einsum / mm / potrf+potri do)."""
    w = dict(factor=0., inverse=0., precondition=0., bn_bytes=0., update_bytes=0.)
    for s in specs:
        if s['kind'] == 'bn':
            w['bn_bytes'] += 8. * batch * s['c'] * s['h'] * s['h']
            continue
        dA, dG, L = spec_dims(s, batch)
        w['factor'] += 2. * dA * dA * L + 2. * dG * dG * L
        w['inverse'] += float(dA) ** 3 + float(dG) ** 3
        w['precondition'] += 2. * dG * dG * dA + 2. * dG * dA * dA
        w['update_bytes'] += 20. * dG * dA
    return w


def factor_executed_flops(specs, batch):
    """fp32 MFMA flops the factor kernels execute for one step, from the same tile / split /
    correlation plan the launches use (the library's plan queries): upper-triangular tiles x
    whole reduction chunks x 2 * tile^2 * chunk depth; 13 shared correlations instead of 45
    tap-pair products for a stride-1 3x3 layer."""
    import torchsso
    from torchsso import _hip
    lib = _hip.load()
    if torchsso.factor_mode() == 'grouped':
        # the plan of ONE engine call over all products (the figure does not depend on how the
        # hooks cut a pass into calls: it counts tiles x reduction chunks, not k-splits)
        jobs = []
        for s in specs:
            if s['kind'] == 'bn':
                continue
            for kind in ('a', 'g'):
                j = _hip.FactorJob()
                j.x, j.C, j.rows, j.alpha = 256, 256 * (len(jobs) + 2), batch, 1.   # (never dereferenced)
                if s['kind'] == 'conv' and kind == 'a':
                    j.kind, j.add_bias = _hip.FACTOR_CONV_A, int(s['bias'])
                    j.c, j.H, j.W = s['cin'], s['hin'], s['hin']
                    j.kh = j.kw = s['k']
                    j.sh = j.sw = s['stride']
                    j.ph = j.pw = s['pad']
                    j.dh = j.dw = 1
                elif s['kind'] == 'conv':
                    j.kind = _hip.FACTOR_CONV_G
                    j.c, j.H, j.W = s['cout'], s['hout'], s['hout']
                else:
                    j.kind = _hip.FACTOR_LINEAR
                    j.add_bias = int(s['bias']) if kind == 'a' else 0
                    j.c = s['fin'] if kind == 'a' else s['fout']
                jobs.append(j)
        arr = (_hip.FactorJob * len(jobs))(*jobs)
        return lib.kfac_factor_grouped_executed_flops(len(jobs), arr)
    total = 0.
    for s in specs:
        if s['kind'] == 'bn':
            continue
        dA, dG, L = spec_dims(s, batch)
        if s['kind'] == 'conv':
            total += lib.kfac_factor_conv_a_executed_flops(
                batch, s['cin'], s['hin'], s['hin'], s['k'], s['k'], s['stride'], s['stride'],
                s['pad'], s['pad'], 1, 1, int(s['bias']))
        else:
            total += lib.kfac_factor_executed_flops(dA, L)
        total += lib.kfac_factor_executed_flops(dG, L)
    return total


def inverse_precondition_executed_flops(specs, batch):
    """(inversion, preconditioning) fp32 MFMA flops executed per step, from the library's
    plan queries: whole 128 x 128 tiles; factors kept as the triangular factor of their
    inverse (KronCurvature.factored_inverse_min_dim) skip the Y Y^T third of the inversion
    and are applied as two triangular products."""
    from torchsso import _hip
    from torchsso.curv.curvature import KronCurvature
    lib = _hip.load()
    min_dim = KronCurvature.factored_inverse_min_dim
    fact = (lambda d: 0) if min_dim is None else (lambda d: int(d >= min_dim))
    dims, dG, dA = [], [], []
    for s in specs:
        if s['kind'] == 'bn':
            continue
        a, g, _ = spec_dims(s, batch)
        dims += [a, g]
        dA.append(a)
        dG.append(g)
    inv = lib.kfac_inverse_executed_flops(len(dims), _hip.int_array(dims),
                                          _hip.int_array([fact(d) for d in dims]))
    pre = lib.kfac_precondition_executed_flops(len(dG), _hip.int_array(dG), _hip.int_array(dA),
                                               _hip.int_array([fact(d) for d in dG]),
                                               _hip.int_array([fact(d) for d in dA]))
    return inv, pre


# ---------------------------------------------------------------------------
# GPU side
# ---------------------------------------------------------------------------

class LayerSet(object):
    """Modules + synthetic per-layer tensors on the device, wrapped by a
    SecondOrderOptimizer exactly as a user model would be."""

    def __init__(self, specs, batch, device, seed=0):
        import torch
        import torch.nn as nn
        import torchsso
        self.torch = torch
        self.batch = batch
        gen = torch.Generator(device='cpu').manual_seed(seed)
        torch.manual_seed(1)
        mods = []
        for s in specs:
            if s['kind'] == 'conv':
                m = nn.Conv2d(s['cin'], s['cout'], s['k'], s['stride'], s['pad'], bias=s['bias'])
            elif s['kind'] == 'linear':
                m = nn.Linear(s['fin'], s['fout'], bias=s['bias'])
            else:
                m = nn.BatchNorm2d(s['c'])
                with torch.no_grad():
                    m.weight.uniform_(0.5, 1.5, generator=gen)
                    m.bias.normal_(0, 0.1, generator=gen)
            mods.append(m)
        self.model = nn.ModuleList(mods).to(device)
        self.specs = specs
        self.opt = torchsso.optim.SecondOrderOptimizer(
            self.model, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron', 'BatchNorm2d': 'Diag'},
            {'damping': 1e-3, 'ema_decay': 0.95}, lr=1e-3, momentum=0.9)
        self.curvs = [g['curv'] for g in self.opt.param_groups]
        # synthetic layer inputs / output gradients / raw parameter gradients
        self.inputs, self.gouts = [], []
        for s, m in zip(specs, self.model):
            if s['kind'] == 'conv':
                xin = torch.randn(batch, s['cin'], s['hin'], s['hin'], device=device)
                g = torch.randn(batch, s['cout'], s['hout'], s['hout'], device=device) * 1e-2
            elif s['kind'] == 'linear':
                if s.get('relu_input', False):
                    xin = torch.randn(batch, s['fin'], device=device).clamp_(min=0)
                else:
                    xin = torch.randn(batch, s['fin'], device=device)
                g = torch.randn(batch, s['fout'], device=device) * 1e-2
            else:   # BatchNorm: the hook reads the OUTPUT and the output gradient
                xin = torch.randn(batch, s['c'], s['h'], s['h'], device=device)
                g = torch.randn(batch, s['c'], s['h'], s['h'], device=device) * 1e-2
            self.inputs.append(xin)
            self.gouts.append(g)
        # raw parameter gradients: every p.grad is a 256-byte aligned view into one
        # flat buffer, so that handing the step fresh gradients (what a backward pass
        # would do) is one device copy
        params = [p for m in self.model for p in m.parameters()]
        offs, total = [], 0
        for p in params:
            offs.append(total)
            total += (p.numel() + 63) // 64 * 64
        self.flat_raw = torch.randn(total, device=device) * 1e-2
        self.flat_grad = self.flat_raw.clone()
        for p, o in zip(params, offs):
            p.grad = self.flat_grad[o:o + p.numel()].view_as(p)

    def bytes_resident(self):
        n = 0
        for lst in (self.inputs, self.gouts):
            n += sum(t.numel() * 4 for t in lst)
        return n

    # -- the parts of a step ---------------------------------------------------
    def build_factors(self, kinds=('conv', 'linear', 'bn')):
        """The hooks of one training pass: the forward hooks in layer order, then the backward
        hooks in reverse order."""
        layers = [(s, m, c, xin, g) for s, m, c, xin, g in
                  zip(self.specs, self.model, self.curvs, self.inputs, self.gouts)
                  if s['kind'] in kinds]
        for s, m, c, xin, g in layers:
            if s['kind'] == 'bn':
                c.forward_postprocess(m, (xin,), xin)    # sum_hw xhat^2 from the layer output
            else:
                c.update_in_forward(xin)
        for s, m, c, xin, g in reversed(layers):
            c.update_in_backward(g)

    def restore_grads(self):
        self.flat_grad.copy_(self.flat_raw)

    def step(self):
        # the factor products go to the side streams; the copy that stands in for the
        # backward pass's fresh gradients runs beside them, as a backward pass would
        self.build_factors()
        self.restore_grads()
        self.opt.step()

    def timed_phases(self, iters):
        """Average ms of: Kronecker factor build (the syrk kernels only) / BatchNorm
        diagonal curvature / EMA / inversion / preconditioning / parameter update, bracketed by HIP
        events on the stream the kernels are launched on (torch's current stream)."""
        torch = self.torch
        import torchsso
        from torchsso.curv import curvature as _curv
        ev = lambda: torch.cuda.Event(enable_timing=True)
        acc = [0.] * 6
        groups = self.opt.param_groups
        for _ in range(iters):
            self.restore_grads()
            e = [ev() for _ in range(7)]
            e[0].record()
            self.build_factors(('conv', 'linear'))
            # (the products run on the library's side streams: eager mode from their hooks, grouped
            # mode in a few engine calls that the hooks and this join trigger)
            torchsso.join_factor_streams()
            e[1].record()
            self.build_factors(('bn',))
            e[2].record()
            _curv.update_ema_all(self.curvs)
            e[3].record()
            _curv.update_inv_all(self.curvs)
            e[4].record()
            _curv.precondition_all([(g['curv'], g['params']) for g in groups])
            e[5].record()
            self.opt._fused_update(groups, 'params')
            e[6].record()
            torch.cuda.synchronize()
            for i in range(6):
                acc[i] += e[i].elapsed_time(e[i + 1])
        return [a / iters for a in acc]


def time_steps(step, steps, warmup):
    """(ms per step by the slower of HIP events and the host clock, ms by events, host
    enqueue ms per step).  The third figure is the host's own time to enqueue one step
    (Python + ctypes + launch calls; the median over steps that each start on an idle
    device); where it approaches the first, the step is bound by the host."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        step()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ev_ms = start.elapsed_time(end) / steps
    # host enqueue time: each step starts on an idle device (with a backlog of several steps
    # the runtime makes the host wait for queue space, and the figure would drift towards the
    # device time)
    host = []
    for _ in range(min(steps, 10)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        step()
        host.append(time.perf_counter() - t0)
    torch.cuda.synchronize()
    host_ms = sorted(host)[len(host) // 2] * 1e3
    return max(wall_ms, ev_ms), ev_ms, host_ms


def run_gpu(specs, batch, steps, warmup):
    import torch
    dev = torch.device('cuda:0')
    ls = LayerSet(specs, batch, dev)
    ms, ev_ms, host_ms = time_steps(ls.step, steps, warmup)
    phases = ls.timed_phases(max(2, min(steps, 5)))
    infos = [c.info for c in ls.curvs if c.kind == 'kron']
    not_spd = int(sum(int((i != 0).sum().item()) for i in infos))
    resident = ls.bytes_resident()
    del ls
    torch.cuda.empty_cache()
    return ms, ev_ms, host_ms, phases, resident, not_spd


PEAK_HBM_TBS = 8.0


def phase_records(work, executed, phases):
    """Per phase of a step: algorithmic and executed work over the phase's HIP-event time.
    MFMA phases in TFLOP/s against the fp32 matrix peak, HBM-bound tails in TB/s against
    8 TB/s (algorithmic bytes: BatchNorm 8*n*c*h*w, update 20*|p|)."""
    f_ms, bn_ms, ema_ms, inv_ms, pre_ms, upd_ms = phases
    mfma = {}
    for name, key, t in (('factor', 'factor', f_ms), ('invert', 'inverse', inv_ms),
                         ('precondition', 'precondition', pre_ms)):
        alg, exe = work[key], executed[key]
        mfma[name] = {'ms': round(t, 4), 'algorithmic_gflop': round(alg / 1e9, 1),
                      'executed_gflop': round(exe / 1e9, 1),
                      'algorithmic_tflops': round(alg / t / 1e9, 2),
                      'executed_tflops': round(exe / t / 1e9, 2),
                      'executed_frac': round(exe / t / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)}
    hbm = {}
    # The factor products write the running averages of the Kronecker factors themselves
    # (no accumulation steps here), so the `ema` phase holds no pass over the factors: what
    # runs there is the tail of the BatchNorm work (the queued backward reductions not yet
    # flushed and the running average of the diagonals), priced with BatchNorm.
    for name, nbytes, t in (('batchnorm_diag', work['bn_bytes'], bn_ms + ema_ms),
                            ('update', work['update_bytes'], upd_ms)):
        if nbytes <= 0 or t < 0.02:
            continue
        hbm[name] = {'ms': round(t, 4), 'algorithmic_GB': round(nbytes / 1e9, 3),
                     'TB_per_s': round(nbytes / t / 1e9, 3),
                     'frac': round(nbytes / t / 1e9 / PEAK_HBM_TBS, 4)}
    return mfma, hbm


def layerset_summary(workload, steps, warmup):
    """One LayerSet workload, timed like the headline one: step ms and the phases."""
    make, batch, label = WORKLOADS[workload]
    specs = make()
    if workload == 'alexnet_fc':
        for s in specs:
            s['relu_input'] = True
    work = algorithmic_work(specs, batch)
    inv_x, pre_x = inverse_precondition_executed_flops(specs, batch)
    executed = {'factor': factor_executed_flops(specs, batch), 'inverse': inv_x, 'precondition': pre_x}
    ms, ev_ms, host_ms, phases, resident, not_spd = run_gpu(specs, batch, steps, warmup)
    mfma, hbm = phase_records(work, executed, phases)
    return {'workload': label, 'ms_per_step': round(ms, 4), 'steps': steps, 'warmup': warmup,
            'host_enqueue_ms': round(host_ms, 4), 'not_spd_factors': not_spd,
            'phases': mfma, 'hbm': hbm}


# ---------------------------------------------------------------------------
# BASELINE config 5: Noisy K-FAC (VIOptimizer) on config 2's network
# ---------------------------------------------------------------------------

class PhaseClock(object):
    """Brackets named functions with HIP events on the current stream while a step runs and
    sums the elapsed times per name; the functions are patched in place for the duration of
    `with clock:` only (an instrumented run, separate from the timed one)."""

    def __init__(self, targets):
        self.targets = targets            # name -> (object, attribute)
        self.pairs = {}
        self.saved = []

    def wrap(self, name, fn):
        import torch

        def timed(*a, **k):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = fn(*a, **k)
            e1.record()
            self.pairs.setdefault(name, []).append((e0, e1))
            return out
        return timed

    def __enter__(self):
        for name, (obj, attr) in self.targets.items():
            fn = getattr(obj, attr)
            self.saved.append((obj, attr, fn))
            setattr(obj, attr, self.wrap(name, fn))
        return self

    def __exit__(self, *exc):
        for obj, attr, fn in self.saved:
            setattr(obj, attr, fn)
        self.saved = []

    def totals_ms(self):
        import torch
        torch.cuda.synchronize()
        return {name: sum(a.elapsed_time(b) for a, b in pairs) for name, pairs in self.pairs.items()}


class NoisyKfacJob(object):
    """The network and data of BASELINE config 2 (conv 3->64 k5, pool, conv 64->128 k5, pool,
    3200-384-192-10; batch 128 of 3x32x32) under VIOptimizer with 4 MC samples per step,
    Kronecker curvature for Conv2d and Linear: per step 4 x (posterior sample, forward,
    backward with the factor products in the hooks, accumulation), then the running average,
    the pi-damped inversion, the Cholesky factors of the inverses, preconditioning and the
    update of the posterior means (reference: optim/vi.py:174-258)."""

    MC = 4

    def __init__(self, device, batch=128):
        import torch
        import torch.nn as nn
        import torch.nn.functional as F
        import torchsso
        torch.manual_seed(1)
        self.model = nn.Sequential(
            nn.Conv2d(3, 64, 5), nn.ReLU(), nn.MaxPool2d(2),
            nn.Conv2d(64, 128, 5), nn.ReLU(), nn.MaxPool2d(2), nn.Flatten(),
            nn.Linear(3200, 384), nn.ReLU(), nn.Linear(384, 192), nn.ReLU(),
            nn.Linear(192, 10)).to(device)
        gen = torch.Generator().manual_seed(0)
        self.x = torch.randn(batch, 3, 32, 32, generator=gen).to(device)
        self.y = torch.randint(0, 10, (batch,), generator=gen).to(device)
        self.opt = torchsso.optim.VIOptimizer(
            self.model, 50000, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron'},
            {'damping': 1e-3, 'ema_decay': 0.95}, lr=1e-3, momentum=0.9,
            num_mc_samples=self.MC, prior_variance=1, kl_weighting=1, seed=1)
        self.F = F

    def closure(self):
        self.model.zero_grad()
        out = self.model(self.x)
        loss = self.F.cross_entropy(out, self.y)
        loss.backward()
        return loss, out

    def step(self):
        self.opt.step(closure=self.closure)

    def timed_phases(self, iters):
        from torchsso.curv import curvature as _curv
        clock = PhaseClock({
            'sample': (_curv, 'sample_all'),
            'forward_backward_factor': (self, 'closure'),
            'accumulate': (self.opt, '_accumulate'),
            'ema': (_curv, 'update_ema_all'),
            'invert': (_curv, 'update_inv_all'),
            'cholesky': (_curv, 'update_std_all'),
            'precondition': (_curv, 'precondition_all'),
            'update': (self.opt, '_fused_update'),
        })
        with clock:
            for _ in range(iters):
                self.step()
        return {k: v / iters for k, v in clock.totals_ms().items()}


def run_noisy_kfac(args):
    import torch
    dev = torch.device('cuda:0')
    job = NoisyKfacJob(dev)
    job.step()                     # the first step has no posterior to sample from yet
    ms, ev_ms, host_ms = time_steps(job.step, args.steps, args.warmup)
    phases = job.timed_phases(max(2, min(args.steps, 5)))
    specs = convnet_specs()
    work = algorithmic_work(specs, 128)
    flops = {'factor': NoisyKfacJob.MC * work['factor'], 'inverse': work['inverse'],
             'cholesky': work['inverse'] / 3., 'sample': NoisyKfacJob.MC * work['precondition'],
             'precondition': work['precondition']}
    info = [g['curv'].info for g in job.opt.param_groups] + \
        [g['curv'].std_info for g in job.opt.param_groups]
    not_spd = int(sum(int((i != 0).sum().item()) for i in info if i is not None))
    total = sum(flops.values())
    # the Cholesky factors of the inverses come out of the inversion (the matrices are factored
    # back to front), so the `cholesky` phase is what is left of update_std: nearly nothing
    both = phases['invert'] + phases['cholesky']
    out = {
        'metric': METRIC, 'value': round(ms, 4), 'unit': 'ms', 'n_gpus': 1,
        'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms, 4),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'noisy_kfac_convnet_batch128_mc4 (BASELINE config 5)', 'batch': 128,
                   'kron_layers': 5, 'num_mc_samples': NoisyKfacJob.MC, 'dataset_size': 50000,
                   'damping': 1e-3, 'ema_decay': 0.95, 'measured_from_step': 2,
                   'step_includes': 'forward and backward of the network (torch) for every MC sample'},
        'tflops': round(total / (ms * 1e-3) / 1e12, 2),
        'algorithmic_gflop': {k: round(v / 1e9, 2) for k, v in flops.items()},
        'phases_ms': {k: round(v, 4) for k, v in phases.items()},
        'phases_tflops': {'invert': round(flops['inverse'] / phases['invert'] / 1e9, 2),
                          'sample': round(flops['sample'] / phases['sample'] / 1e9, 2),
                          'precondition': round(flops['precondition'] / phases['precondition'] / 1e9, 2)},
        'host_enqueue_ms': round(host_ms, 4),
        'not_spd_factors': not_spd,
        'roofline': {'bound': 'mfma',
                     'kernel': 'pi-damped inversion delivering the Cholesky factors of the inverses, '
                               'all layers (potrf_*, trtri_*, lauum, std_from_inverse_factor kernels)',
                     'achieved': round(flops['inverse'] / both / 1e9, 2),
                     'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': round(flops['inverse'] / both / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
                     'traffic': None,
                     'note': 'n^3 flops per factor over the inversion + update_std phases; the '
                             'reference\'s separate Cholesky factorisation of every inverse '
                             '(algorithmic_gflop.cholesky) is not executed: the factor is read off '
                             'the triangular inverse'},
    }
    return out


# ---------------------------------------------------------------------------
# a real training step: ResNet-50 forward + backward + K-FAC step (and plain SGD beside it)
# ---------------------------------------------------------------------------

def run_resnet50_train(args):
    """Whole training steps of the ResNet-50 itself (torch modules, batch 32, 224x224, fp32):
    forward, backward with the factor products in the hooks, SecondOrderOptimizer.step with
    every factor inverted every step; beside it the same network under torch.optim.SGD.
    What the optimizer adds to a step is the difference."""
    import torch
    import torch.nn.functional as F
    import torchsso
    dev = torch.device('cuda:0')
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(32, 3, 224, 224, generator=gen).to(dev)
    y = torch.randint(0, 1000, (32,), generator=gen).to(dev)

    torch.manual_seed(1)
    model = build_resnet50().to(dev)
    sgd = torch.optim.SGD(model.parameters(), lr=1e-3, momentum=0.9)

    def sgd_step():
        sgd.zero_grad()
        F.cross_entropy(model(x), y).backward()
        sgd.step()
    sgd_ms, _, _ = time_steps(sgd_step, args.steps, args.warmup)
    del sgd, model

    torch.manual_seed(1)
    model = build_resnet50().to(dev)
    opt = torchsso.optim.SecondOrderOptimizer(
        model, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron', 'BatchNorm2d': 'Diag'},
        {'damping': 1e-3, 'ema_decay': 0.95}, lr=1e-3, momentum=0.9)

    def closure():
        opt.zero_grad()
        out = model(x)
        loss = F.cross_entropy(out, y)
        loss.backward()
        return loss, out
    ms, ev_ms, host_ms = time_steps(lambda: opt.step(closure=closure), args.steps, args.warmup)
    info = torch.cat([g['curv'].info for g in opt.param_groups if g['curv'].kind == 'kron'])
    work = algorithmic_work(resnet50_specs(), 32)
    total = work['factor'] + work['inverse'] + work['precondition']
    return {
        'metric': 'ResNet-50 training step ms with the K-FAC step inside (forward + backward + '
                  'factor + invert + precondition + update), 1 MI355X',
        'value': round(ms, 4), 'unit': 'ms', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': round(ms, 4), 'higher_is_better': False,
        'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'resnet50_training_step_batch32_224x224 (real activations)',
                   'batch': 32, 'invert_every_step': True,
                   'factor_side_streams': torchsso.factor_streams()},
        'sgd_step_ms': round(sgd_ms, 4), 'kfac_overhead_ms': round(ms - sgd_ms, 4),
        'kfac_algorithmic_tflops_over_the_overhead': round(total / ((ms - sgd_ms) * 1e-3) / 1e12, 2),
        'host_enqueue_ms': round(host_ms, 4),
        'not_spd_factors': int((info != 0).sum().item()),
    }


# ---------------------------------------------------------------------------
# CPU baseline (the oracle = port of the reference's torch-CPU + SciPy path)
# ---------------------------------------------------------------------------

def run_cpu_baseline(specs, batch, budget_s=30.0):
    """Times the oracle on one layer of every distinct shape and weighs each by how often
    that shape occurs in the workload (a bounded sample of the same step).  Largest shapes
    first; the shapes that carry the first 80 % of the step's algorithmic flops get one
    untimed warm-up run and the median of two timed ones, the rest one timed run; shapes the
    budget does not reach are scaled in by flops.  Threads: the job's share of the host
    (OMP_NUM_THREADS where the environment sets it, else every core)."""
    import torch
    from oracle import kfac_oracle as O
    cores = os.cpu_count() or 1
    threads = int(os.environ.get('OMP_NUM_THREADS', '0')) or cores
    torch.set_num_threads(threads)
    groups = {}
    for s in specs:
        key = tuple(sorted((k, v) for k, v in s.items() if k != 'name'))
        groups.setdefault(key, [s, 0])[1] += 1

    def flops(s):
        if s['kind'] == 'bn':
            return 8. * batch * s['c'] * s['h'] * s['h']
        dA, dG, L = spec_dims(s, batch)
        return 2. * (dA * dA + dG * dG) * L + 2. * (float(dA) ** 3 + float(dG) ** 3) \
            + 2. * dG * dA * (dA + dG)

    def one_layer(s, x, g, gw, gb):
        if s['kind'] == 'bn':
            w, b = torch.rand(s['c']) + 0.5, torch.randn(s['c'])
            xhat = O.bn_restore_input(x, w, b)
            data = O.bn_diag(xhat, g, True)
            ema = O.ema_update(data, [d.clone() for d in data], 0.95)
            inv = [O.diag_inverse(e, 1e-3) for e in ema]
            return [i * torch.ones_like(i) for i in inv]
        if s['kind'] == 'conv':
            A = O.factor_conv_a(x, (s['k'], s['k']), (s['stride'],) * 2, (s['pad'],) * 2,
                                (1, 1), s['bias'])
            G = O.factor_conv_g(g)
        else:
            A = O.factor_linear_a(x, s['bias'])
            G = O.factor_linear_g(g)
        ema = O.ema_update([A, G], [A.clone(), G.clone()], 0.95)
        Ai, Gi = O.pi_damped_inverse(ema[0], ema[1], 1e-3)
        pw, pb = O.precondition(Gi, Ai, gw, gb)
        return O.sgd_tail(torch.zeros_like(pw), pw, torch.zeros_like(pw), 1e-3, 0.9, 0.)

    order = sorted(groups.values(), key=lambda sc: -flops(sc[0]))
    total_flops = sum(flops(s) * c for s, c in order)
    done_flops = 0.
    total_s = 0.
    spent = 0.
    measured = repeated = 0
    torch.manual_seed(0)
    for s, count in order:
        if spent > budget_s:
            break
        gw = gb = None
        if s['kind'] == 'conv':
            x = torch.randn(batch, s['cin'], s['hin'], s['hin'])
            g = torch.randn(batch, s['cout'], s['hout'], s['hout']) * 1e-2
            gw = torch.randn(s['cout'], s['cin'], s['k'], s['k']) * 1e-2
            gb = torch.randn(s['cout']) * 1e-2 if s['bias'] else None
        elif s['kind'] == 'linear':
            x = torch.randn(batch, s['fin'])
            if s.get('relu_input', False):
                x.clamp_(min=0)
            g = torch.randn(batch, s['fout']) * 1e-2
            gw = torch.randn(s['fout'], s['fin']) * 1e-2
            gb = torch.randn(s['fout']) * 1e-2 if s['bias'] else None
        else:
            x = torch.randn(batch, s['c'], s['h'], s['h'])
            g = torch.randn(batch, s['c'], s['h'], s['h']) * 1e-2
        heavy = done_flops < 0.8 * total_flops
        times = []
        for rep in range(3 if heavy else 1):
            t0 = time.perf_counter()
            one_layer(s, x, g, gw, gb)
            dt = time.perf_counter() - t0
            spent += dt
            if not (heavy and rep == 0):     # the first run of a heavy shape is the warm-up
                times.append(dt)
            if heavy and spent > budget_s and times:
                break
        times.sort()
        dt = times[len(times) // 2] if len(times) % 2 else 0.5 * (times[len(times) // 2 - 1]
                                                                   + times[len(times) // 2])
        total_s += dt * count
        done_flops += flops(s) * count
        measured += 1
        repeated += 1 if heavy else 0
    if done_flops < total_flops:      # extrapolate what the budget did not cover
        total_s *= total_flops / done_flops
    sample = ('%d of %d distinct layer shapes (largest first, %.0f%% of the step\'s algorithmic '
              'flops), weighted by multiplicity%s; the %d shapes carrying the first 80%% of the '
              'flops: warm-up + median of 2, the rest once; torch CPU einsum/unfold/mm + '
              'scipy.linalg.inv, fp32; %d threads = the job\'s share of a host with %d cores' % (
                  measured, len(order), 100. * done_flops / total_flops,
                  '' if done_flops >= total_flops else ', rest scaled by flops', repeated,
                  threads, cores))
    return total_s * 1e3, cores, threads, sample


# ---------------------------------------------------------------------------

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='resnet50', choices=sorted(WORKLOADS) + ['noisy_kfac', 'resnet50_train'])
    ap.add_argument('--factor-streams', type=int, default=None,
                    help='side streams for the factor products (library default: 2; 0 = none)')
    ap.add_argument('--factor-mode', default=None, choices=['grouped', 'eager'],
                    help='grouped (library default): the hooks queue their factor products and one '
                         'engine call runs them all; eager: a launch sequence per product, on the '
                         'side streams')
    ap.add_argument('--factor-flush-work', default=None,
                    help='grouped mode: multiply-adds of queued products from which the queue runs '
                         'without waiting for a reader (library default: 2.5e11); "none": never')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-other-workloads', action='store_true',
                    help='resnet50 only: leave out the short runs of the other BASELINE '
                         'configurations that the line carries in `other_workloads`')
    ap.add_argument('--factored-min-dim', type=int, default=None,
                    help='rows from which update_inv keeps an inverse as its triangular factor '
                         '(library default: KronCurvature.factored_inverse_min_dim)')
    ap.add_argument('--explicit-inverse', action='store_true',
                    help='form A^-1 and G^-1 explicitly in update_inv (as the reference does) '
                         'instead of keeping their triangular factors and applying those')
    ap.add_argument('--one-curvature-stream', action='store_true',
                    help='inversion and preconditioning of all layers on the caller\'s stream '
                         '(default: the layers with small factors take theirs to a side stream '
                         'beside the factorisation chain of the largest factors)')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run a plain 1 GiB device copy (reference for rocprofv3 --pmc '
                         'FETCH_SIZE / WRITE_SIZE readings)')
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py measures the one-GPU share of the K-FAC step; --gpus must be 1 '
              '(no collectives are part of this build)', file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print('no HIP device visible', file=sys.stderr)
        sys.exit(1)
    import torchsso
    if args.factor_streams is not None:
        torchsso.set_factor_streams(args.factor_streams)
    if args.factor_mode is not None:
        torchsso.set_factor_mode(args.factor_mode)
    if args.factor_flush_work is not None:
        torchsso.set_factor_flush_work(None if args.factor_flush_work == 'none'
                                       else float(args.factor_flush_work))
    factor_streams = torchsso.factor_streams()
    from torchsso.curv import curvature as _curvature
    from torchsso.curv.curvature import KronCurvature
    if args.one_curvature_stream:
        _curvature.two_stream_min_dim = None
    if args.explicit_inverse:
        KronCurvature.factored_inverse_min_dim = None
    elif args.factored_min_dim is not None:
        KronCurvature.factored_inverse_min_dim = args.factored_min_dim
    inverse_form = ('explicit' if KronCurvature.factored_inverse_min_dim is None else
                    'triangular factor Y (Y Y^T = inverse) for factors of >= %d rows, explicit below'
                    % KronCurvature.factored_inverse_min_dim)

    if args.workload == 'resnet50_train':
        print(json.dumps(run_resnet50_train(args)))
        return
    if args.workload == 'noisy_kfac':
        out = run_noisy_kfac(args)
        out['config']['factor_side_streams'] = factor_streams
        out['config']['inverse_form'] = inverse_form
        if not args.no_cpu_baseline:
            # the same step on the host: 4 x factors + inverse + Cholesky + 4 x sampling products
            specs = convnet_specs()
            cpu_ms, cores, threads, sample = run_cpu_baseline(specs, 128)
            out['cpu_baseline'] = {
                'value': round(cpu_ms, 1), 'unit': 'ms', 'cores': cores, 'threads': threads,
                'kind': 'port',
                'sample': 'ONE factor build + inversion + preconditioning of the same layers '
                          '(config 2\'s K-FAC step, a lower bound for the Noisy K-FAC step, which '
                          'builds the factors 4 times and adds the Cholesky factors and 4 '
                          'sampling products; the reference has no CPU Cholesky at all, '
                          'utils/cholesky_cupy.py is CuPy only); ' + sample}
        print(json.dumps(out))
        return

    make, batch, label = WORKLOADS[args.workload]
    specs = make()
    if args.workload == 'alexnet_fc':
        for s in specs:
            s['relu_input'] = True
    work = algorithmic_work(specs, batch)
    executed = factor_executed_flops(specs, batch)
    inv_x, pre_x = inverse_precondition_executed_flops(specs, batch)
    mfma_phases, hbm_phases = None, None

    ms, ev_ms, host_ms, phases, resident, not_spd = run_gpu(specs, batch, args.steps, args.warmup)
    mfma_phases, hbm_phases = phase_records(
        work, {'factor': executed, 'inverse': inv_x, 'precondition': pre_x}, phases)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device='cuda:0').normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    f_ms, bn_ms, ema_ms, inv_ms, pre_ms, upd_ms = phases
    total_flops = work['factor'] + work['inverse'] + work['precondition']

    out = {
        'metric': METRIC, 'value': round(ms, 4), 'unit': 'ms', 'n_gpus': 1,
        'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms, 4),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': label, 'batch': batch,
                   'kron_layers': sum(1 for s in specs if s['kind'] != 'bn'),
                   'bn_layers': sum(1 for s in specs if s['kind'] == 'bn'),
                   'damping': 1e-3, 'ema_decay': 0.95, 'invert_every_step': True, 'inverse_form': inverse_form,
                   'curvature_streams': 1 if _curvature.two_stream_min_dim is None else 2,
                   'factor_mode': torchsso.factor_mode(), 'factor_side_streams': factor_streams,
                   'inputs_resident_GB': round(resident / 1e9, 3)},
        'tflops': round(total_flops / (ms * 1e-3) / 1e12, 2),
        'algorithmic_gflop': {k: round(v / 1e9, 1) for k, v in work.items() if not k.endswith('bytes')},
        'phases_ms': {'factor': round(f_ms, 4), 'batchnorm_diag': round(bn_ms, 4),
                      'ema': round(ema_ms, 4),
                      'invert': round(inv_ms, 4), 'precondition': round(pre_ms, 4),
                      'update': round(upd_ms, 4)},
        # algorithmic flops (dense convention: 2*d^2*L per factor, n^3 per inverse,
        # 2*dG*dA*(dG+dA) per layer) over the phase time; what the matrix cores execute is in
        # roofline.phases
        'phases_tflops': {'factor': round(work['factor'] / f_ms / 1e9, 2),
                          'invert': round(work['inverse'] / inv_ms / 1e9, 2),
                          'precondition': round(work['precondition'] / pre_ms / 1e9, 2)},
        'host_enqueue_ms': round(host_ms, 4),
        'not_spd_factors': not_spd,
        'roofline': {'bound': 'mfma',
                     'kernel': 'Kronecker factor build, all layers (syrk_grouped_kernel, corr_grouped_kernel; '
                               'syrk_kernel, corr_kernel in eager mode)',
                     'achieved': round(work['factor'] / f_ms / 1e9, 2),
                     'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': round(work['factor'] / f_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
                     'traffic': None,
                     'note': 'achieved counts the algorithmic flops 2*d^2*L of every factor (dense '
                             'convention); the kernels execute fewer (one triangle of each symmetric '
                             'product, shared spatial correlations for stride-1 kxk convolutions), so '
                             'frac can exceed 1; executed_* prices what the matrix cores really do, '
                             'derived from the library\'s tile / split plan',
                     'executed_gflop': round(executed / 1e9, 1),
                     'executed_tflops': round(executed / f_ms / 1e9, 2),
                     'executed_frac': round(executed / f_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
                     # every MFMA phase and every HBM-bound tail of the step, each over its
                     # own HIP-event time: algorithmic and executed work (executed: the
                     # library's tile plans; the inversion forms no Y Y^T for the factors it
                     # keeps in triangular form, so it executes less than n^3)
                     'phases': mfma_phases, 'hbm': hbm_phases},
    }
    if args.workload == 'resnet50':
        pmc = read_pmc_summary()
        seen = pmc.get('executed_flop_per_step_pmc')
        if seen and abs(executed - seen) <= 0.03 * seen:
            out['roofline']['traffic'] = pmc.get('traffic_bytes_per_launch')
            out['roofline']['executed_gflop_pmc'] = round(seen / 1e9, 1)
            # (counter runs cannot be made from inside this script: both figures are read
            # from the summary of the rocprofv3 --pmc runs, not measured in this run)
            out['roofline']['traffic_source'] = os.path.relpath(PMC_SUMMARY, ROOT)
        else:
            msg = ('the factor plan executes %.1f GFLOP per step but the counter summary %s was '
                   'taken at %s: the plan changed since, traffic and the PMC cross-check are '
                   'left out until the counters are read again'
                   % (executed / 1e9, os.path.relpath(PMC_SUMMARY, ROOT),
                      'no reading' if not seen else '%.1f GFLOP' % (seen / 1e9)))
            print('bench.py: WARNING: ' + msg, file=sys.stderr)
            out['roofline']['pmc_check'] = 'STALE: ' + msg
    if args.workload == 'resnet50' and not args.no_other_workloads:
        # the other BASELINE configurations, timed in this same run (fewer steps): parity-test
        # cases, not the headline
        others = [layerset_summary(w, 10, 3) for w in ('mlp', 'convnet', 'alexnet_fc')]
        oargs = argparse.Namespace(steps=10, warmup=3)
        nk = run_noisy_kfac(oargs)
        others.append({'workload': nk['config']['workload'], 'ms_per_step': nk['value'],
                       'steps': 10, 'warmup': 3, 'host_enqueue_ms': nk['host_enqueue_ms'],
                       'not_spd_factors': nk['not_spd_factors'], 'phases_ms': nk['phases_ms'],
                       'step_includes': nk['config']['step_includes']})
        out['other_workloads'] = others
    if not args.no_cpu_baseline:
        cpu_ms, cores, threads, sample = run_cpu_baseline(specs, batch)
        out['cpu_baseline'] = {'value': round(cpu_ms, 1), 'unit': 'ms', 'cores': cores,
                               'threads': threads, 'kind': 'port', 'sample': sample}
        out['speedup_vs_cpu'] = round(cpu_ms / ms, 1)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
