"""One step of bench.py's own workloads (BASELINE config 3: the ResNet-50 layer set at
batch 32; config 4: AlexNet fc6-fc8 at batch 256) checked at full size: for a sample of
layers, the largest included, the running average after the first step, the pi-damped
inverses and the preconditioned gradient are recomputed in float64 on the device with
library routines (unfold, matmul, torch.linalg.inv).  The inverses of config 4 and of the
largest ResNet-50 factors are also put beside the reference's own float32 result on the same
damped matrix (scipy.linalg.inv through the oracle), with the condition number: where even
that is further than 1e-4 from float64, the device result may be at most 1.5 x as far.
Nothing in the timed step is skipped or cached."""
import os
import sys

import pytest
import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu
TOL = 1e-4


def rel(a, b):
    return ((a.double() - b).norm() / b.norm()).item()


def inverse_error(X, shift, Y):
    """Relative error of Y as the inverse of X + shift*I, in float64 on the device:
    against torch.linalg.inv up to 3000 rows, beyond that (where the library routine
    can run out of workspace here) through one Newton step,
    Y_true = Y + Y (I - X Y) + O(|I - X Y|^2)."""
    n = X.shape[0]
    Xd = X + torch.eye(n, dtype=torch.float64, device=X.device) * shift
    Yd = Y.double()
    if n <= 3000:
        ref = torch.linalg.inv(Xd)
        return ((Yd - ref).norm() / ref.norm()).item()
    R = torch.eye(n, dtype=torch.float64, device=X.device) - Xd @ Yd
    return ((Yd @ R).norm() / Yd.norm()).item()


def conv_a_float64(x, s):
    """sum over the batch of unfold(x) unfold(x)^T / n, image by image."""
    k = s['k']
    d = s['cin'] * k * k
    A = torch.zeros(d, d, dtype=torch.float64, device=x.device)
    for i in range(x.shape[0]):
        u = F.unfold(x[i:i + 1].double(), k, padding=s['pad'], stride=s['stride'])[0]
        A += u @ u.t()
    return A / x.shape[0]


def norm2(M, iters=40):
    """Largest singular value of a symmetric float64 matrix by power iteration."""
    v = torch.ones(M.shape[0], dtype=torch.float64, device=M.device)
    v /= v.norm()
    lam = 0.
    for _ in range(iters):
        w = M @ v
        lam = w.norm().item()
        v = w / lam
    return lam


def inverse_record(name, X, shift, Y):
    """The device's float32 inverse Y of X + shift*I next to the reference's own float32
    result on the same matrix: torchsso.utils.inv on a CPU tensor is scipy.linalg.inv in
    float32 (torchsso/utils/inv_cupy.py:32-34), which is what the oracle's float32 path calls.
    Returns (condition number, device vs float64, reference float32 vs float64, device vs
    reference float32); everything but the scipy call runs in float64 on the device."""
    from oracle import kfac_oracle as O
    ref32 = O.damped_inverse(X.float().cpu(), float(shift), torch.float32).to(X.device)
    cond = norm2(X + torch.eye(X.shape[0], dtype=torch.float64, device=X.device) * shift) * \
        norm2(Y.double())
    e_dev = inverse_error(X, shift, Y)
    e_ref = inverse_error(X, shift, ref32)
    d = rel(Y, ref32.double())
    print('%-22s n=%5d cond %.2e | device fp32 vs fp64 %.2e | reference fp32 (scipy) vs fp64 %.2e '
          '| device vs reference fp32 %.2e' % (name, X.shape[0], cond, e_dev, e_ref, d), flush=True)
    return cond, e_dev, e_ref, d, ref32


def newton_inverse(X, shift, Y0, steps=8):
    """The float64 inverse of X + shift*I on the device, from a float32 inverse Y0 by Newton
    steps  Y <- Y + Y (I - X Y)  (the residual I - X Y squares each time); no library
    factorisation, no workspace.  Returns (inverse, rms entry of the last residual)."""
    n = X.shape[0]
    eye = torch.eye(n, dtype=torch.float64, device=X.device)
    Xd = X + eye * shift
    Y = Y0.double()
    res = None
    for _ in range(steps):
        R = eye - Xd @ Y
        res = (R.norm() / n ** 0.5).item()
        if res < 1e-12:
            break
        Y = Y + Y @ R
    return Y, res


PICKED = {
    'resnet50': ['conv1', 'layer1.0.conv1', 'layer1.0.conv2', 'layer2.0.conv2',
                 'layer3.0.downsample', 'layer4.0.conv2', 'layer4.2.conv2', 'layer4.2.conv3', 'fc',
                 'layer3.1.bn2'],
    'alexnet_fc': ['fc6', 'fc7', 'fc8'],
}
# layers whose inverses are also put beside the reference's float32 result
BESIDE_REFERENCE = {'resnet50': ['layer4.2.conv2', 'fc'], 'alexnet_fc': ['fc6', 'fc7', 'fc8']}


@pytest.mark.parametrize('workload', ['resnet50', 'alexnet_fc'])
def test_benchmark_step_at_full_size_against_float64_on_device(workload):
    import bench
    dev = torch.device('cuda:0')
    specs, batch, _ = bench.WORKLOADS[workload]
    specs = specs()
    if workload == 'alexnet_fc':
        for s in specs:
            s['relu_input'] = True      # as bench.py runs it: a = clamp(N(0,1), min=0)
    ls = bench.LayerSet(specs, batch, dev)
    raw = ls.flat_raw.clone()
    ls.step()
    torch.cuda.synchronize()
    names = [s['name'] for s in specs]
    picked = PICKED[workload]
    offs = {}
    total = 0
    for m in ls.model:
        for p in m.parameters():
            offs[id(p)] = total
            total += (p.numel() + 63) // 64 * 64
    worst = {}
    inverse_bounds = {}     # entry of `worst` -> bound tied to the reference's own float32 error
    for name in picked:
        i = names.index(name)
        s, m, curv, x, g = specs[i], ls.model[i], ls.curvs[i], ls.inputs[i], ls.gouts[i]
        n = x.shape[0]
        if s['kind'] == 'bn':
            xhat = (x.double() - m.bias.detach().double().view(1, -1, 1, 1)) / \
                m.weight.detach().double().view(1, -1, 1, 1)
            sx = (xhat * xhat).sum((2, 3))
            sg = (g.double() ** 2).sum((2, 3))
            want = [(sx * sg).mean(0) * n * n, sg.mean(0) * n * n]
            for k in range(2):
                worst['bn ema'] = max(worst.get('bn ema', 0.), rel(curv.ema[k], want[k]))
                worst['bn inv'] = max(worst.get('bn inv', 0.),
                                      rel(curv.inv[k], 1. / (curv.ema[k].double() + 1e-3)))
            continue
        if s['kind'] == 'conv':
            A = conv_a_float64(x, s)
            hw = g.shape[2] * g.shape[3]
            gm = g.double().permute(1, 0, 2, 3).reshape(g.shape[1], -1)
            G = gm @ gm.t() * (float(n) / hw)
        else:
            xa = torch.cat([x.double(), torch.ones(n, 1, dtype=torch.float64, device=dev)], 1)
            A = xa.t() @ xa / n
            G = g.double().t() @ g.double() * float(n)
        worst['A'] = max(worst.get('A', 0.), rel(curv.ema[0], A))
        worst['G'] = max(worst.get('G', 0.), rel(curv.ema[1], G))
        del A, G
        # pi-damped inverses of the running averages the step produced
        eA, eG = curv.ema[0].double(), curv.ema[1].double()
        pi = ((eA.diagonal().sum() / eA.shape[0]) / (eG.diagonal().sum() / eG.shape[0])).sqrt()
        r = 1e-3 ** 0.5
        chain = {}
        if name in BESIDE_REFERENCE[workload]:
            for tag, X, shift, Y in (('A', eA, r * pi, curv.inv[0]), ('G', eG, r / pi, curv.inv[1])):
                key = '%s %s inverse' % (name, tag)
                _, e_dev, e_ref, d, ref32 = inverse_record(key, X, shift.item(), Y)
                worst[key] = e_dev
                # two float32 inverses of one matrix are no further apart than their
                # distances from the float64 inverse add up to
                assert d <= 1.001 * (e_dev + e_ref), (key, d, e_dev, e_ref)
                truth, res = newton_inverse(X, shift.item(), Y)
                assert res < 1e-11, (key, res)
                chain[tag] = (truth, ref32)
                # 1e-4 where the reference's float32 inverse meets it too; where even
                # scipy.linalg.inv in float32 is further than that from float64 (error of
                # any float32 inverse ~ cond * 2^-24), at most 1.5 x the reference's error
                inverse_bounds[key] = max(TOL, 1.5 * e_ref)
        else:
            worst['A inverse'] = max(worst.get('A inverse', 0.), inverse_error(eA, r * pi, curv.inv[0]))
            worst['G inverse'] = max(worst.get('G inverse', 0.), inverse_error(eG, r / pi, curv.inv[1]))
        assert curv.info.cpu().tolist() == [0, 0]
        # preconditioned gradient (first step: the momentum buffer equals it)
        ps = list(m.parameters())
        V = raw[offs[id(ps[0])]:offs[id(ps[0])] + ps[0].numel()].view(ps[0].shape[0], -1).double()
        got = ps[0].grad.reshape(ps[0].shape[0], -1).double()
        if len(ps) > 1:
            V = torch.cat([V, raw[offs[id(ps[1])]:offs[id(ps[1])] + ps[1].numel()].double()[:, None]], 1)
            got = torch.cat([got, ps[1].grad.double()[:, None]], 1)
        want = curv.inv[1].double() @ V @ curv.inv[0].double()
        worst['preconditioned gradient'] = max(worst.get('preconditioned gradient', 0.), rel(got, want))
        if chain:
            # End to end: G^-1 [grad W | grad b] A^-1 with the float64 inverses of the SAME
            # damped running averages, beside (i) what the device wrote and (ii) the
            # reference's own float32 chain (scipy float32 inverses, two float32 products:
            # torchsso/utils/inv_cupy.py:32-34, curv/cov/linear.py:69-84).  Where the
            # condition number puts any float32 result further than 1e-4 from float64, the
            # device may be at most 1.5 x as far as the reference.
            truth = chain['G'][0] @ V @ chain['A'][0]
            ref_chain = (chain['G'][1] @ V.float() @ chain['A'][1]).double()
            e_dev, e_ref = rel(got, truth), rel(ref_chain, truth)
            print('%-22s preconditioned gradient end to end: device vs float64 %.2e | reference '
                  'float32 chain vs float64 %.2e | device vs reference %.2e | device vs its own '
                  'inverses in float64 %.2e' % (name, e_dev, e_ref, rel(got, ref_chain),
                                               rel(got, want)), flush=True)
            key = '%s preconditioned gradient end to end' % name
            worst[key] = e_dev
            inverse_bounds[key] = max(TOL, 1.5 * e_ref)
            del truth, ref_chain
        del eA, eG, chain
    print(workload, 'step at full size, worst rel. Frobenius errors:',
          {k: '%.2e' % v for k, v in worst.items()}, flush=True)
    for k, v in worst.items():
        bound = inverse_bounds.get(k, TOL)
        assert v <= bound, (k, v, bound)
