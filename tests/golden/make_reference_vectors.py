"""Writes golden vectors for the host sequencing of the K-FAC step by running the
reference implementation itself (cybertronai/pytorch-sso mounted read-only at
/root/reference) on its CPU path.

Run once, in the development container only (the reference does not exist on
the GPU box):

    python tests/golden/make_reference_vectors.py

What it pins (behaviour that is convention rather than mathematics, so that a
restatement could silently disagree): the order of operations inside
SecondOrderOptimizer.step when l2_reg, damping, momentum and weight decay
interact (momentum type, gradient EMA, bias correction, LARS, weight normalisation,
accumulation over micro-steps, running max); what the hooks take as layer input /
output gradient on current torch; the accumulation scales of VIOptimizer's MC loop.  The numerical kernels
themselves are pinned by mathematics in tests/test_oracle.py.

The reference imports `chainer` at module level for its multi-GPU communicator
(torchsso/utils/chainer_communicators/_utility.py:11), which is out of scope and
not installed; empty placeholder modules are put in sys.modules before the
import so that the single-process classes load.  No reference file is modified
or copied; only inputs and outputs (arrays) are saved.

VIOptimizer's posterior sampling with Kronecker curvature cannot be produced
this way: the reference's `torchsso.utils.cholesky` exists for CuPy only
(utils/cholesky_cupy.py:9-14).  The Kronecker VI case below therefore uses
prior_variance=0 (no sampling, std_scale=0).  With diagonal curvature (VOGN) the
std is an element-wise square root, so that case samples, and pins the order in
which the generator is consumed (valid for CPU tensors only: a GPU generator
yields other numbers).

    python tests/golden/make_reference_vectors.py [case ...]     (default: all)
"""
import os
import sys
import types
import warnings

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = '/root/reference'


def _import_reference():
    for name in ('chainer', 'chainer.backends', 'chainer.backends.cuda'):
        sys.modules.setdefault(name, types.ModuleType(name))
    sys.modules['chainer'].backends = sys.modules['chainer.backends']
    sys.modules['chainer.backends'].cuda = sys.modules['chainer.backends.cuda']
    sys.path.insert(0, REFERENCE)
    import torchsso  # noqa: the reference package
    assert os.path.realpath(torchsso.__file__).startswith(REFERENCE), torchsso.__file__
    return torchsso


def build_mlp(torch, nn):
    torch.manual_seed(1)
    return nn.Sequential(nn.Linear(12, 16), nn.ReLU(), nn.Linear(16, 10), nn.ReLU(),
                         nn.Linear(10, 5))


def build_convnet(torch, nn):
    torch.manual_seed(1)
    return nn.Sequential(
        nn.Conv2d(2, 4, 3, padding=1), nn.BatchNorm2d(4), nn.ReLU(),
        nn.Conv2d(4, 6, 3, stride=2, bias=False), nn.ReLU(),
        nn.Flatten(), nn.Linear(6 * 3 * 3, 5))


def snapshot(optimizer, out, tag):
    for gi, group in enumerate(optimizer.param_groups):
        curv = group['curv']
        for pi, p in enumerate(group['params']):
            out['%s.g%d.param%d' % (tag, gi, pi)] = p.detach().numpy().copy()
            out['%s.g%d.grad%d' % (tag, gi, pi)] = p.grad.detach().numpy().copy()
        for name in ('ema', 'inv'):
            val = getattr(curv, name)
            if val is None:          # a micro-step of an accumulation: nothing updated yet
                continue
            for k, t in enumerate(val):
                out['%s.g%d.%s%d' % (tag, gi, name, k)] = t.detach().numpy().copy()
        out['%s.g%d.damping' % (tag, gi)] = np.float64(curv.damping)


def run_case(torchsso, torch, nn, F, name, model, x, y, opt_cls, opt_args, steps):
    if len(sys.argv) > 1 and name not in sys.argv[1:]:
        return
    out = {'x': x.numpy().copy(), 'y': y.numpy().copy()}
    for k, v in model.state_dict().items():
        out['init.' + k] = v.numpy().copy()
    optimizer = opt_cls(model, **opt_args)

    def closure():
        model.zero_grad()
        output = model(x)
        loss = F.cross_entropy(output, y)
        loss.backward()
        return loss, output

    for s in range(steps):
        ret = optimizer.step(closure=closure)
        loss = ret[0]
        out['step%d.loss' % s] = np.float64(loss.item())
        snapshot(optimizer, out, 'step%d' % s)
    path = os.path.join(HERE, name + '.npz')
    np.savez_compressed(path, **out)
    print('wrote', path, os.path.getsize(path), 'bytes')


def main():
    warnings.simplefilter('ignore')
    torchsso = _import_reference()
    import torch
    import torch.nn as nn
    import torch.nn.functional as F
    torch.set_num_threads(1)

    # 1. MLP, Kron curvature for every Linear, all interacting options on
    torch.manual_seed(0)
    x = torch.randn(8, 12)
    y = torch.randint(0, 5, (8,))
    run_case(torchsso, torch, nn, F, 'ref_mlp_kfac', build_mlp(torch, nn), x, y,
             torchsso.optim.SecondOrderOptimizer,
             dict(curv_type='Cov', curv_shapes={'Linear': 'Kron'},
                  curv_kwargs={'damping': 1e-3, 'ema_decay': 0.95},
                  lr=0.05, momentum=0.9, l2_reg=1e-3, weight_decay=1e-3), steps=3)

    # 2. Conv + BatchNorm (diagonal) + strided bias-free conv + Linear
    torch.manual_seed(0)
    x = torch.randn(6, 2, 8, 8)
    y = torch.randint(0, 5, (6,))
    run_case(torchsso, torch, nn, F, 'ref_convnet_kfac', build_convnet(torch, nn), x, y,
             torchsso.optim.SecondOrderOptimizer,
             dict(curv_type='Cov',
                  curv_shapes={'Linear': 'Kron', 'Conv2d': 'Kron', 'BatchNorm2d': 'Diag'},
                  curv_kwargs={'damping': 1e-2, 'ema_decay': 0.9},
                  lr=0.02, momentum=0.5, momentum_type='raw', l2_reg=1e-4), steps=2)

    # 3. VI sequencing without sampling (prior_variance=0 -> l2_reg=0, std_scale=0)
    torch.manual_seed(0)
    x = torch.randn(8, 12)
    y = torch.randint(0, 5, (8,))
    run_case(torchsso, torch, nn, F, 'ref_mlp_vi_nosample', build_mlp(torch, nn), x, y,
             torchsso.optim.VIOptimizer,
             dict(dataset_size=100, curv_type='Cov', curv_shapes={'Linear': 'Kron'},
                  curv_kwargs={'damping': 1e-3, 'ema_decay': 0.95},
                  lr=0.05, momentum=0.9, num_mc_samples=3, prior_variance=0), steps=2)

    # 4. VOGN: diagonal curvature for Conv2d / BatchNorm2d / Linear, with sampling
    torch.manual_seed(0)
    x = torch.randn(6, 2, 8, 8)
    y = torch.randint(0, 5, (6,))
    run_case(torchsso, torch, nn, F, 'ref_convnet_vogn', build_convnet(torch, nn), x, y,
             torchsso.optim.VOGN,
             dict(dataset_size=60, lr=0.01, num_mc_samples=2, warmup_kl_weighting_steps=None,
                  curv_kwargs={'ema_decay': 0.1, 'damping': 1e-3}), steps=3)

    # 5. the same without sampling (prior_variance=0), for runs on a GPU generator
    torch.manual_seed(0)
    x = torch.randn(6, 2, 8, 8)
    y = torch.randint(0, 5, (6,))
    run_case(torchsso, torch, nn, F, 'ref_convnet_vogn_nosample', build_convnet(torch, nn), x, y,
             torchsso.optim.VOGN,
             dict(dataset_size=60, lr=0.01, num_mc_samples=2, warmup_kl_weighting_steps=None,
                  prior_variance=0, curv_kwargs={'ema_decay': 0.1, 'damping': 1e-3}), steps=3)

    # 6. the tails of the update: gradient EMA on the preconditioned gradient, bias
    #    correction, LARS, weight normalisation, no regularisation for BatchNorm, running
    #    max of the curvature (orders of operations that no formula fixes)
    torch.manual_seed(0)
    x = torch.randn(6, 2, 8, 8)
    y = torch.randint(0, 5, (6,))
    run_case(torchsso, torch, nn, F, 'ref_convnet_kfac_tails', build_convnet(torch, nn), x, y,
             torchsso.optim.SecondOrderOptimizer,
             dict(curv_type='Cov',
                  curv_shapes={'Linear': 'Kron', 'Conv2d': 'Kron', 'BatchNorm2d': 'Diag'},
                  curv_kwargs={'damping': 1e-2, 'ema_decay': 0.9, 'use_max_ema': True},
                  lr=0.02, momentum=0.5, grad_ema_decay=0.8, grad_ema_type='preconditioned',
                  l2_reg=1e-4, weight_decay=1e-3, bias_correction=True, lars=True,
                  normalizing_weights=True, non_reg_for_bn=True), steps=3)

    # 7. accumulation over 2 micro-steps, raw momentum, LARS on the raw gradient, a
    #    fixed weight scale; 6 calls = 3 updates
    torch.manual_seed(0)
    x = torch.randn(8, 12)
    y = torch.randint(0, 5, (8,))
    run_case(torchsso, torch, nn, F, 'ref_mlp_kfac_accumulate', build_mlp(torch, nn), x, y,
             torchsso.optim.SecondOrderOptimizer,
             dict(curv_type='Cov', curv_shapes={'Linear': 'Kron'},
                  curv_kwargs={'damping': 1e-3, 'ema_decay': 0.95},
                  lr=0.05, momentum=0.9, momentum_type='raw', l2_reg=1e-3, acc_steps=2,
                  lars=True, lars_type='raw', normalizing_weights=True, weight_scale=1.5),
             steps=6)

    # 8. diagonal curvature everywhere with the square root of the running average, a
    #    gradient EMA on the raw gradient and bias correction: the Adam-like setting
    torch.manual_seed(0)
    x = torch.randn(6, 2, 8, 8)
    y = torch.randint(0, 5, (6,))
    run_case(torchsso, torch, nn, F, 'ref_convnet_diag_sqrt', build_convnet(torch, nn), x, y,
             torchsso.optim.SecondOrderOptimizer,
             dict(curv_type='Cov',
                  curv_shapes={'Linear': 'Diag', 'Conv2d': 'Diag', 'BatchNorm2d': 'Diag'},
                  curv_kwargs={'damping': 1e-8, 'ema_decay': 0.001, 'use_sqrt_ema': True},
                  lr=1e-3, grad_ema_decay=0.1, grad_ema_type='raw', bias_correction=True),
             steps=4)

    # 10. VOGN with a KL warm-up, a prior variance other than 1 and an initial precision:
    #     the l2 / std scale bookkeeping of VIOptimizer, with sampling from the first step
    torch.manual_seed(0)
    x = torch.randn(6, 2, 8, 8)
    y = torch.randint(0, 5, (6,))
    run_case(torchsso, torch, nn, F, 'ref_convnet_vogn_warmup', build_convnet(torch, nn), x, y,
             torchsso.optim.VOGN,
             dict(dataset_size=60, lr=0.01, num_mc_samples=2, warmup_kl_weighting_steps=3,
                  warmup_kl_weighting_init=0.1, kl_weighting=0.5, prior_variance=2,
                  init_precision=8e-3, curv_kwargs={'ema_decay': 0.1, 'damping': 1e-3}), steps=5)

    # 9. the iteration-based learning-rate schedules (host arithmetic only)
    if len(sys.argv) == 1 or 'ref_lr_schedules' in sys.argv[1:]:
        L = torchsso.optim.lr_scheduler
        out = {}

        def sgd(lr=0.4, momentum=0.9):
            return torch.optim.SGD(nn.Linear(3, 2).parameters(), lr=lr, momentum=momentum)

        def run(tag, opt, sched, steps):
            lrs, moms = [], []
            for _ in range(steps):
                sched.step()
                lrs.append(opt.param_groups[0]['lr'])
                moms.append(opt.param_groups[0]['momentum'])
            out[tag + '.lr'] = np.array(lrs, dtype=np.float64)
            out[tag + '.momentum'] = np.array(moms, dtype=np.float64)

        opt = sgd()
        run('poly_start2', opt, L.PolynomialDecayIterLR(opt, rate=2, max_count=10, start_iter=2), 12)
        opt = sgd()
        run('poly_target', opt, L.PolynomialDecayIterLR(opt, rate=1, max_count=10, target=0.1), 10)
        opt = sgd()
        run('poly_negative_rate', opt,
            L.PolynomialDecayIterLR(opt, rate=-0.5, max_count=10, target=0.8), 9)
        opt = sgd()
        run('warmup_momentum', opt,
            L.MomentumCorrectionLR(L.GradualWarmupIterLR(opt, initial_lr=0.1, max_count=4)), 7)
        opt = sgd()
        opt.param_groups[0]['initial_lr'] = 0.4
        run('poly_resumed', opt,
            L.PolynomialDecayIterLR(opt, rate=2, max_count=10, last_iter=5), 4)
        path = os.path.join(HERE, 'ref_lr_schedules.npz')
        np.savez_compressed(path, **out)
        print('wrote', path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
