"""K-FAC step benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50|alexnet_fc|convnet|mlp]
                    [--no-cpu-baseline] [--copy-calibration]

A "step" is one pass of the K-FAC hot path over one batch of synthetic input,
driven through the public torchsso API: for every layer the two Kronecker
factors are built from that layer's input and output gradient (what the
forward / backward hooks do), then SecondOrderOptimizer.step() runs the running
average, the pi-damped inversion of all factors, the preconditioning of all
gradients and the parameter update.  The default workload is BASELINE config 3:
the 53 convolutions + fc of a ResNet-50 at batch 32, 224x224 (real per-layer
activation / gradient shapes, N(0,1) data), with diagonal curvature for the 53
BatchNorm layers.  All inputs are resident in HBM before the timed region.

Prints ONE JSON line (see the keys below).  `value` is the step time in ms.
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
# HBM bytes per launch of the factor-build kernels (syrk_kernel, corr_kernel and their reduce /
# assemble kernels), averaged over the 226 launches of a resnet50 step, from two rocprofv3 --pmc runs
# (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0 after calibration with a 1 GiB copy): 48.0 MB read + 14.6 MB
# written (the reads include the previous running average, which the epilogues fold in).
RESNET50_FACTOR_TRAFFIC_BYTES = 62.6e6
# flops the matrix cores execute for the factor products of one resnet50 step
# (512 x SQ_INSTS_VALU_MFMA_MOPS_F32 from a rocprofv3 --pmc run): the symmetric products run one
# triangle, and the stride-1 3x3 layers take 13 spatial correlations instead of 45 block products
RESNET50_FACTOR_EXECUTED_FLOP = 560.6e9


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


def spec_dims(s, batch):
    """(dA, dG, L) of a Kron layer."""
    if s['kind'] == 'conv':
        return (s['cin'] * s['k'] * s['k'] + (1 if s['bias'] else 0), s['cout'],
                batch * s['hout'] * s['hout'])
    return s['fin'] + (1 if s['bias'] else 0), s['fout'], batch


def algorithmic_work(specs, batch):
    """Flops of the dense formulation (what the reference's einsum / mm / potrf+potri do)."""
    w = dict(factor=0., inverse=0., precondition=0., bn_bytes=0., ema_bytes=0., update_bytes=0.)
    for s in specs:
        if s['kind'] == 'bn':
            w['bn_bytes'] += 8. * batch * s['c'] * s['h'] * s['h']
            continue
        dA, dG, L = spec_dims(s, batch)
        w['factor'] += 2. * dA * dA * L + 2. * dG * dG * L
        w['inverse'] += float(dA) ** 3 + float(dG) ** 3
        w['precondition'] += 2. * dG * dG * dA + 2. * dG * dA * dA
        w['ema_bytes'] += 12. * (dA * dA + dG * dG)
        w['update_bytes'] += 20. * dG * dA
    return w


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

    # -- the three phases of a step -----------------------------------------
    def build_factors(self, kinds=('conv', 'linear', 'bn')):
        for s, m, c, xin, g in zip(self.specs, self.model, self.curvs, self.inputs, self.gouts):
            if s['kind'] not in kinds:
                continue
            if s['kind'] == 'bn':
                # forward hook: sum_hw xhat^2 from the layer output; backward hook: the rest
                c.forward_postprocess(m, (xin,), xin)
                c.update_in_backward(g)
            else:
                c.update_in_forward(xin)
                c.update_in_backward(g)

    def restore_grads(self):
        self.flat_grad.copy_(self.flat_raw)

    def step(self):
        self.restore_grads()
        self.build_factors()
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
            torchsso.join_factor_streams()   # the products run on the library's side streams
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


def run_gpu(args, specs, batch):
    import torch
    dev = torch.device('cuda:0')
    ls = LayerSet(specs, batch, dev)
    for _ in range(args.warmup):
        ls.step()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        ls.step()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ev_ms = start.elapsed_time(end) / args.steps
    phases = ls.timed_phases(max(2, min(args.steps, 5)))
    infos = [c.info for c in ls.curvs if c.kind == 'kron']
    not_spd = int(sum(int((i != 0).sum().item()) for i in infos))
    return max(wall_ms, ev_ms), ev_ms, phases, ls.bytes_resident(), not_spd


# ---------------------------------------------------------------------------
# CPU baseline (the oracle = port of the reference's torch-CPU + SciPy path)
# ---------------------------------------------------------------------------

def run_cpu_baseline(specs, batch, budget_s=30.0):
    """Times the oracle on one layer of every distinct shape and weighs each by
    how often that shape occurs in the workload (bounded sample of the same
    step).  Largest shapes first; stops adding shapes when the budget is spent
    and scales the remainder by algorithmic flops."""
    import torch
    from oracle import kfac_oracle as O
    threads = int(os.environ.get('OMP_NUM_THREADS', '0')) or min(os.cpu_count() or 1, 16)
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

    order = sorted(groups.values(), key=lambda sc: -flops(sc[0]))
    total_flops = sum(flops(s) * c for s, c in order)
    done_flops = 0.
    total_s = 0.
    spent = 0.
    measured = 0
    torch.manual_seed(0)
    for s, count in order:
        if spent > budget_s:
            break
        if s['kind'] == 'conv':
            x = torch.randn(batch, s['cin'], s['hin'], s['hin'])
            g = torch.randn(batch, s['cout'], s['hout'], s['hout']) * 1e-2
            gw = torch.randn(s['cout'], s['cin'], s['k'], s['k']) * 1e-2
            gb = torch.randn(s['cout']) * 1e-2 if s['bias'] else None
        elif s['kind'] == 'linear':
            x = torch.randn(batch, s['fin'])
            g = torch.randn(batch, s['fout']) * 1e-2
            gw = torch.randn(s['fout'], s['fin']) * 1e-2
            gb = torch.randn(s['fout']) * 1e-2 if s['bias'] else None
        else:
            x = torch.randn(batch, s['c'], s['h'], s['h'])
            g = torch.randn(batch, s['c'], s['h'], s['h']) * 1e-2
        t0 = time.perf_counter()
        if s['kind'] == 'bn':
            w, b = torch.rand(s['c']) + 0.5, torch.randn(s['c'])
            xhat = O.bn_restore_input(x, w, b)
            data = O.bn_diag(xhat, g, True)
            ema = O.ema_update(data, [d.clone() for d in data], 0.95)
            inv = [O.diag_inverse(e, 1e-3) for e in ema]
            _ = [i * torch.ones_like(i) for i in inv]
        else:
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
            O.sgd_tail(torch.zeros_like(pw), pw, torch.zeros_like(pw), 1e-3, 0.9, 0.)
        dt = time.perf_counter() - t0
        spent += dt
        total_s += dt * count
        done_flops += flops(s) * count
        measured += 1
    if done_flops < total_flops:      # extrapolate what the budget did not cover
        total_s *= total_flops / done_flops
    sample = ('%d of %d distinct layer shapes timed once each (largest first, %.0f%% of the '
              'step\'s algorithmic flops), weighted by multiplicity%s; torch CPU einsum/unfold/mm '
              '+ scipy.linalg.inv, fp32' % (
                  measured, len(order), 100. * done_flops / total_flops,
                  '' if done_flops >= total_flops else ', rest scaled by flops'))
    return total_s * 1e3, threads, sample


# ---------------------------------------------------------------------------

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='resnet50', choices=sorted(WORKLOADS))
    ap.add_argument('--factor-streams', type=int, default=None,
                    help='side streams for the factor products (library default: 3; 0 = none)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--copy-calibration', action='store_true',
                    help='also run a plain 1 GiB device copy (reference for rocprofv3 --pmc '
                         'FETCH_SIZE / WRITE_SIZE readings)')
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py measures the one-GPU share of the K-FAC step; --gpus must be 1 '
              '(no collectives are part of this build)', file=sys.stderr)
        sys.exit(2)

    make, batch, label = WORKLOADS[args.workload]
    specs = make()
    if args.workload == 'alexnet_fc':
        for s in specs:
            s['relu_input'] = True
    work = algorithmic_work(specs, batch)

    import torch
    if not torch.cuda.is_available():
        print('no HIP device visible', file=sys.stderr)
        sys.exit(1)
    import torchsso
    if args.factor_streams is not None:
        torchsso.set_factor_streams(args.factor_streams)
    factor_streams = torchsso.factor_streams()
    ms, ev_ms, phases, resident, not_spd = run_gpu(args, specs, batch)
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
                   'damping': 1e-3, 'ema_decay': 0.95, 'invert_every_step': True, 'factor_side_streams': factor_streams,
                   'inputs_resident_GB': round(resident / 1e9, 3)},
        'tflops': round(total_flops / (ms * 1e-3) / 1e12, 2),
        'algorithmic_gflop': {k: round(v / 1e9, 1) for k, v in work.items() if not k.endswith('bytes')},
        'phases_ms': {'factor': round(f_ms, 4), 'batchnorm_diag': round(bn_ms, 4),
                      'ema': round(ema_ms, 4),
                      'invert': round(inv_ms, 4), 'precondition': round(pre_ms, 4),
                      'update': round(upd_ms, 4)},
        'phases_tflops': {'factor': round(work['factor'] / f_ms / 1e9, 2),
                          'invert': round(work['inverse'] / inv_ms / 1e9, 2),
                          'precondition': round(work['precondition'] / pre_ms / 1e9, 2)},
        'not_spd_factors': not_spd,
        'roofline': {'bound': 'mfma',
                     'kernel': 'Kronecker factor build, all layers (syrk_kernel, corr_kernel)',
                     'achieved': round(work['factor'] / f_ms / 1e9, 2),
                     'peak': PEAK_FP32_MFMA_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': round(work['factor'] / f_ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
                     'traffic': RESNET50_FACTOR_TRAFFIC_BYTES if args.workload == 'resnet50' else None,
                     'note': 'achieved counts the algorithmic flops 2*d^2*L of every factor (dense '
                             'convention); the kernels execute fewer (one triangle of each symmetric '
                             'product, shared spatial correlations for stride-1 kxk convolutions), so '
                             'frac can exceed 1; executed_* is what the matrix cores really do'},
    }
    if args.workload == 'resnet50':
        ex = RESNET50_FACTOR_EXECUTED_FLOP / f_ms / 1e9
        out['roofline']['executed_tflops'] = round(ex, 2)
        out['roofline']['executed_frac'] = round(ex / PEAK_FP32_MFMA_TFLOPS, 4)
    if not args.no_cpu_baseline:
        cpu_ms, cores, sample = run_cpu_baseline(specs, batch)
        out['cpu_baseline'] = {'value': round(cpu_ms, 1), 'unit': 'ms', 'cores': cores,
                               'kind': 'port', 'sample': sample}
        out['speedup_vs_cpu'] = round(cpu_ms / ms, 1)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
