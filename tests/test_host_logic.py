"""Host-side logic of the torchsso package without a GPU.

The engine calls (torchsso._ops) are replaced, for these tests only, by the
oracle-backed stand-in from kfac_testlib, so that the optimizers' sequencing --
group construction, hook timing, accumulation, phase order, update rule -- can
be checked on CPU tensors against the golden vectors the reference wrote.
The product itself has no CPU path: the last tests check that it refuses."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import torchsso
from torchsso import _hip, _ops
import kfac_testlib as T
from oracle import kfac_oracle as O


# rows from which update_inv keeps an inverse as its triangular factor: the library's
# default (beyond every test network: all inverses explicit), every factor, and a value
# that splits the test networks' layers into sides of both kinds
@pytest.fixture(params=[None, 1, 20], ids=['explicit', 'factored', 'mixed'])
def oracle_ops(monkeypatch, request):
    from torchsso.curv.curvature import KronCurvature
    if request.param is not None:
        monkeypatch.setattr(KronCurvature, 'factored_inverse_min_dim', request.param)
    fake = T.OracleOps()
    for name in dir(fake):
        if not name.startswith('_') and callable(getattr(fake, name)) and hasattr(_ops, name):
            monkeypatch.setattr(_ops, name, getattr(fake, name))
    return fake


def _closure(model, x, y):
    def closure():
        model.zero_grad()
        out = model(x)
        loss = F.cross_entropy(out, y)
        loss.backward()
        return loss, out
    return closure


def test_second_order_optimizer_matches_reference_mlp(oracle_ops):
    gold = T.load_golden('ref_mlp_kfac')
    model = T.load_init(T.build_mlp(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.SecondOrderOptimizer(
        model, 'Cov', {'Linear': 'Kron'}, {'damping': 1e-3, 'ema_decay': 0.95},
        lr=0.05, momentum=0.9, l2_reg=1e-3, weight_decay=1e-3)
    snaps = []
    for s in range(3):
        loss, _ = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-4
        snaps.append(T.snapshot_optimizer(opt))
        assert abs(opt.param_groups[0]['curv'].damping - float(gold['step%d.g0.damping' % s])) < 1e-12
    T.compare_with_golden(snaps, gold)
    assert opt.optim_state == {'step': 3, 'acc_step': 0}


def test_second_order_optimizer_matches_reference_convnet(oracle_ops):
    gold = T.load_golden('ref_convnet_kfac')
    model = T.load_init(T.build_convnet(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.SecondOrderOptimizer(
        model, 'Cov', {'Linear': 'Kron', 'Conv2d': 'Kron', 'BatchNorm2d': 'Diag'},
        {'damping': 1e-2, 'ema_decay': 0.9}, lr=0.02, momentum=0.5, momentum_type='raw', l2_reg=1e-4)
    names = [type(g['curv']).__name__ for g in opt.param_groups]
    assert names == ['KronCovConv2d', 'DiagCovBatchNorm2d', 'KronCovConv2d', 'KronCovLinear']
    snaps = []
    for s in range(2):
        opt.step(closure=_closure(model, x, y))
        snaps.append(T.snapshot_optimizer(opt))
    T.compare_with_golden(snaps, gold)


TAILS_ARGS = dict(curv_type='Cov',
                  curv_shapes={'Linear': 'Kron', 'Conv2d': 'Kron', 'BatchNorm2d': 'Diag'},
                  curv_kwargs={'damping': 1e-2, 'ema_decay': 0.9, 'use_max_ema': True},
                  lr=0.02, momentum=0.5, grad_ema_decay=0.8, grad_ema_type='preconditioned',
                  l2_reg=1e-4, weight_decay=1e-3, bias_correction=True, lars=True,
                  normalizing_weights=True, non_reg_for_bn=True)
ACCUMULATE_ARGS = dict(curv_type='Cov', curv_shapes={'Linear': 'Kron'},
                       curv_kwargs={'damping': 1e-3, 'ema_decay': 0.95},
                       lr=0.05, momentum=0.9, momentum_type='raw', l2_reg=1e-3, acc_steps=2,
                       lars=True, lars_type='raw', normalizing_weights=True, weight_scale=1.5)


def test_update_tails_match_reference(oracle_ops):
    """Gradient EMA on the preconditioned gradient, bias correction, LARS, weight
    normalisation, no regularisation for BatchNorm, running max of the curvature."""
    gold = T.load_golden('ref_convnet_kfac_tails')
    model = T.load_init(T.build_convnet(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.SecondOrderOptimizer(model, **TAILS_ARGS)
    snaps = []
    for s in range(3):
        loss, _ = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-4
        snaps.append(T.snapshot_optimizer(opt))
    # the conv bias in front of the BatchNorm has a zero gradient (rounding noise, which
    # LARS then scales up to the norm of the bias)
    T.compare_with_golden(snaps, gold, skip={(0, 'grad', 1), (0, 'param', 1)})


def test_accumulation_with_raw_momentum_and_lars_matches_reference(oracle_ops):
    """acc_steps = 2: the odd calls only accumulate, the even ones update."""
    gold = T.load_golden('ref_mlp_kfac_accumulate')
    model = T.load_init(T.build_mlp(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.SecondOrderOptimizer(model, **ACCUMULATE_ARGS)
    snaps = []
    for s in range(6):
        loss, _ = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-4
        snaps.append(T.snapshot_optimizer(opt))
        assert opt.optim_state == {'step': (s + 1) // 2, 'acc_step': (s + 1) % 2}
    T.compare_with_golden(snaps, gold)


DIAG_SQRT_ARGS = dict(curv_type='Cov',
                      curv_shapes={'Linear': 'Diag', 'Conv2d': 'Diag', 'BatchNorm2d': 'Diag'},
                      curv_kwargs={'damping': 1e-8, 'ema_decay': 0.001, 'use_sqrt_ema': True},
                      lr=1e-3, grad_ema_decay=0.1, grad_ema_type='raw', bias_correction=True)


def test_diagonal_sqrt_curvature_with_bias_correction_matches_reference(oracle_ops):
    """The Adam-like setting: diagonal curvature, sqrt of the running average, gradient
    EMA on the raw gradient, bias correction with the square root."""
    gold = T.load_golden('ref_convnet_diag_sqrt')
    model = T.load_init(T.build_convnet(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.SecondOrderOptimizer(model, **DIAG_SQRT_ARGS)
    snaps = []
    for s in range(4):
        loss, _ = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-4
        snaps.append(T.snapshot_optimizer(opt))
    # the conv bias in front of the BatchNorm has a zero gradient: g / sqrt(g^2) of rounding noise
    T.compare_with_golden(snaps, gold,
                          skip={(0, k, 1) for k in ('grad', 'param', 'ema', 'inv')})


def test_vi_optimizer_accumulation_matches_reference(oracle_ops):
    gold = T.load_golden('ref_mlp_vi_nosample')
    model = T.load_init(T.build_mlp(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.VIOptimizer(
        model, 100, 'Cov', {'Linear': 'Kron'}, {'damping': 1e-3, 'ema_decay': 0.95},
        lr=0.05, momentum=0.9, num_mc_samples=3, prior_variance=0)
    assert all(g['std_scale'] == 0 for g in opt.param_groups)
    snaps = []
    for s in range(2):
        loss, prob = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-4
        # prob is accumulated with 1/acc_steps per MC sample (reference quirk, vi.py:209)
        assert abs(prob.sum().item() - 3 * x.shape[0]) < 1e-3
        snaps.append(T.snapshot_optimizer(opt))
    T.compare_with_golden(snaps, gold)


def test_vogn_matches_reference_with_sampling(oracle_ops):
    """VOGN (diagonal curvature everywhere) against the vectors the reference wrote
    on CPU, posterior sampling included: pins the diagonal Conv2d/Linear/BatchNorm
    curvature, the element-wise std and the order and shape in which the
    generator is consumed (one draw per parameter, in param_group order)."""
    gold = T.load_golden('ref_convnet_vogn')
    model = T.load_init(T.build_convnet(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.VOGN(model, 60, lr=0.01, num_mc_samples=2,
                              warmup_kl_weighting_steps=None,
                              curv_kwargs={'ema_decay': 0.1, 'damping': 1e-3})
    names = [type(g['curv']).__name__ for g in opt.param_groups]
    assert names == ['DiagCovConv2d', 'DiagCovBatchNorm2d', 'DiagCovConv2d', 'DiagCovLinear']
    snaps = []
    for s in range(3):
        loss, _ = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-3 * max(1, abs(loss.item()))
        snaps.append(T.snapshot_optimizer(opt))
    # the raw gradient of the conv bias in front of the BatchNorm is zero up to rounding
    # noise (1e-9), which the diagonal inverse (1 / damping = 1e3 for a curvature of g^2 ~
    # 1e-18) scales up next to the prior term l2_reg * bias: that one entry carries the noise
    # of two different summation orders and gets a named, wider bound
    T.compare_with_golden(snaps, gold, label='ref_convnet_vogn', exceptions={
        (0, 'grad', 1): (2e-4, 'zero raw gradient in front of BatchNorm, noise / damping')})


def test_vogn_kl_warmup_prior_and_initial_precision_match_reference(oracle_ops):
    """KL warm-up over 3 steps, prior variance 2, initial precision: the l2_reg /
    std_scale bookkeeping of VIOptimizer (optim/vi.py:77-78, 98-106, 141-162), with a
    posterior to sample from before the first step."""
    gold = T.load_golden('ref_convnet_vogn_warmup')
    model = T.load_init(T.build_convnet(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.VOGN(model, 60, lr=0.01, num_mc_samples=2, warmup_kl_weighting_steps=3,
                              warmup_kl_weighting_init=0.1, kl_weighting=0.5, prior_variance=2,
                              init_precision=8e-3,
                              curv_kwargs={'ema_decay': 0.1, 'damping': 1e-3})
    snaps = []
    for s in range(5):
        loss, _ = opt.step(closure=_closure(model, x, y))
        assert abs(loss.item() - float(gold['step%d.loss' % s])) < 1e-3 * max(1, abs(loss.item()))
        snaps.append(T.snapshot_optimizer(opt))
        for gi, g in enumerate(opt.param_groups):
            assert abs(g['curv'].damping - float(gold['step%d.g%d.damping' % (s, gi)])) < 1e-9
    # the bias of the conv in front of the BatchNorm has a zero gradient (rounding noise
    # over its tiny curvature); everything else, sampled parameters included, must agree
    T.compare_with_golden(snaps, gold, skip={(0, 'grad', 1)})


def test_kl_rate_follows_the_stateful_warmup_of_the_reference():
    """The reference keeps l2_reg / std_scale in the param groups and moves them in
    adjust_kl_weighting after every update (optim/vi.py:150-172): nothing while
    step > warmup_steps, else rate = (init + step / warmup * (target - init)) / init.
    Simulated here as that loop, against the closed function of the step."""
    import math
    from torchsso.optim.vi import kl_rate
    for warmup, init, target in ((3, 0.1, 0.5), (1000, 0.01, 1.), (2.5, 0.2, 0.1), (0.5, 0.1, 1.),
                                 (1, 0.3, 0.3)):
        rate = 1.                                   # what the groups hold, relative to the start
        for step in range(1, 12):
            if not warmup < step:
                rate = (init + step / warmup * (target - init)) / init
            assert kl_rate(step, warmup, init, target) == rate, (warmup, step)
    assert kl_rate(7, None, 0.01, 1.) == 1.
    assert kl_rate(0, 5, 0.01, 1.) == 1.
    # and the optimizer applies it to the groups that have a prior term only
    model = nn.Sequential(nn.Linear(4, 3), nn.BatchNorm1d(3))
    opt = torchsso.optim.VIOptimizer(model, 50, 'Cov', {'Linear': 'Kron', 'BatchNorm1d': 'Diag'},
                                     {}, non_reg_for_bn=True, warmup_kl_weighting_steps=4,
                                     warmup_kl_weighting_init=0.1, kl_weighting=0.5, prior_variance=2)
    lin, bn = opt.param_groups
    assert lin['l2_reg'] == 0.1 / 50 / 2 and lin['std_scale'] == math.sqrt(0.1 / 50)
    assert bn['l2_reg'] == 0 and bn['std_scale'] == 0
    opt.optim_state['step'] = 2
    opt.adjust_kl_weighting()
    r = kl_rate(2, 4, 0.1, 0.5)
    assert lin['l2_reg'] == r * (0.1 / 50 / 2) and lin['std_scale'] == math.sqrt(r) * math.sqrt(0.1 / 50)
    assert bn['l2_reg'] == 0 and bn['std_scale'] == 0
    opt.optim_state['step'] = 9
    lin['l2_reg'] = 123.                           # past the warm-up nothing is touched
    opt.adjust_kl_weighting()
    assert lin['l2_reg'] == 123.


def test_check_spd_raises_and_names_the_layer(oracle_ops, monkeypatch):
    """check_spd=True: the status words of the inversion are read once per step and a
    factor that was not positive definite raises, naming the layer, instead of the
    reference's silent NaNs (utils/inv_cupy.py:124,130 never read dev_info)."""
    from torchsso.curv.curvature import NotPositiveDefiniteError
    torch.manual_seed(2)
    model = nn.Sequential(nn.Linear(4, 3), nn.ReLU(), nn.Linear(3, 2))
    x, y = torch.randn(8, 4), torch.randint(0, 2, (8,))
    opt = torchsso.optim.SecondOrderOptimizer(model, 'Cov', {'Linear': 'Kron'}, {'damping': 1e-3},
                                              check_spd=True)
    opt.step(closure=_closure(model, x, y))        # healthy factors: no complaint
    real, real_fac = oracle_ops.pi_damped_inverse_batched, oracle_ops.pi_damped_inverse_factored_batched

    def failing(As, Gs, dampings, A_invs=None, G_invs=None, info=None):
        a, g, info = real(As, Gs, dampings, A_invs, G_invs, info)
        info[3] = 2                                 # layer 1, factor G, leading minor 2
        return a, g, info

    def failing_factored(*args, **kwargs):
        info = real_fac(*args, **kwargs)
        info[3] = 2
        return info
    monkeypatch.setattr(_ops, 'pi_damped_inverse_batched', failing)
    monkeypatch.setattr(_ops, 'pi_damped_inverse_factored_batched', failing_factored)
    with pytest.raises(NotPositiveDefiniteError, match=r'layer 1 \(Linear\): inverse of factor G.*order 2'):
        opt.step(closure=_closure(model, x, y))
    opt.check_spd = False                           # the default: nothing is read
    opt.step(closure=_closure(model, x, y))


def test_vi_sampling_consumes_generator_in_group_order(oracle_ops):
    """With a std present, params = mean + std_scale * U_G E U_A with E drawn by
    torch.randn in param_group order after manual_seed(step + seed)."""
    torch.manual_seed(3)
    model = nn.Sequential(nn.Linear(6, 5), nn.ReLU(), nn.Linear(5, 3))
    x, y = torch.randn(16, 6), torch.randint(0, 3, (16,))
    opt = torchsso.optim.VIOptimizer(model, 200, 'Cov', {'Linear': 'Kron'},
                                     {'damping': 1e-2, 'ema_decay': 0.9}, lr=0.01,
                                     num_mc_samples=2, seed=5)
    opt.step(closure=_closure(model, x, y))          # first step: no std yet -> mean only
    assert all(g['curv'].std is not None for g in opt.param_groups)
    means = [[m.clone() for m in g['mean']] for g in opt.param_groups]
    opt.set_random_seed()
    opt.sample_params()
    torch.manual_seed(opt.optim_state['step'] + 5)
    from oracle import kfac_oracle as O
    for g, mean in zip(opt.param_groups, means):
        A_ic, G_ic = g['curv'].std
        E = torch.randn(G_ic.shape[0], A_ic.shape[0])
        w, b = O.sample(mean[0], mean[1], G_ic, A_ic, E, g['std_scale'])
        assert torch.allclose(g['params'][0].data, w, atol=1e-6)
        assert torch.allclose(g['params'][1].data, b, atol=1e-6)
    assert abs(opt.defaults['l2_reg'] - 1 / 200) < 1e-12
    assert abs(opt.param_groups[0]['std_scale'] - (1 / 200) ** 0.5) < 1e-12


def test_accumulation_steps_average_gradients_and_factors(oracle_ops):
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(4, 3))
    xs = [torch.randn(5, 4) for _ in range(2)]
    ys = [torch.randint(0, 3, (5,)) for _ in range(2)]
    opt = torchsso.optim.SecondOrderOptimizer(model, 'Cov', {'Linear': 'Kron'},
                                              {'damping': 1e-2, 'ema_decay': 1.}, acc_steps=2)
    w0 = model[0].weight.detach().clone()
    opt.step(closure=_closure(model, xs[0], ys[0]))
    assert torch.equal(model[0].weight.detach(), w0)          # no update yet
    assert opt.optim_state == {'step': 0, 'acc_step': 1}
    A0 = opt.param_groups[0]['curv'].A.clone()
    seen = {}
    inner = _closure(model, xs[1], ys[1])

    def second():
        ret = inner()
        seen['A1'] = opt.param_groups[0]['curv'].A.clone()    # this pass's factor
        return ret
    opt.step(closure=second)
    A1 = seen['A1']
    assert opt.optim_state == {'step': 1, 'acc_step': 0}
    assert not torch.equal(model[0].weight.detach(), w0)
    assert torch.allclose(opt.param_groups[0]['curv'].ema[0], 0.5 * (A0 + A1), atol=1e-6)


def test_vi_forward_pass_between_micro_steps_leaves_the_accumulators_alone(oracle_ops):
    """acc_steps = 2: a prediction() (or any forward pass) between the two micro-steps must
    not add its input factor to the accumulated curvature; the reference only adds curv.data
    inside its MC loop (vi.py:211-220)."""
    def run(predict_between, fail_first=False):
        torch.manual_seed(0)
        model = nn.Sequential(nn.Linear(4, 3))
        xs = [torch.randn(5, 4) for _ in range(3)]
        ys = [torch.randint(0, 3, (5,)) for _ in range(2)]
        opt = torchsso.optim.VIOptimizer(model, 100, 'Cov', {'Linear': 'Kron'},
                                         {'damping': 1e-2, 'ema_decay': 1.}, num_mc_samples=2,
                                         prior_variance=0, acc_steps=2)
        if fail_first:
            def broken():
                model(xs[2])
                raise RuntimeError('closure failed')
            with pytest.raises(RuntimeError):
                opt.step(closure=broken)
            curv = opt.param_groups[0]['curv']
            assert curv._acc_into is None
            model(xs[2])               # a pass after the failure is not accumulated either
            return None
        opt.step(closure=_closure(model, xs[0], ys[0]))
        assert opt.optim_state == {'step': 0, 'acc_step': 1}
        if predict_between:
            opt.prediction(xs[2])
            model(xs[2])
        opt.step(closure=_closure(model, xs[1], ys[1]))
        assert opt.optim_state == {'step': 1, 'acc_step': 0}
        return [e.clone() for e in opt.param_groups[0]['curv'].ema]
    plain, disturbed = run(False), run(True)
    for a, b in zip(plain, disturbed):
        assert torch.equal(a, b)
    run(False, fail_first=True)


def test_checkpoint_is_tensor_only_and_resumes_exactly(oracle_ops, tmp_path):
    import copy
    gold = T.load_golden('ref_convnet_kfac')
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])

    def make(model):
        return torchsso.optim.SecondOrderOptimizer(
            model, 'Cov', {'Linear': 'Kron', 'Conv2d': 'Kron', 'BatchNorm2d': 'Diag'},
            {'damping': 1e-2, 'ema_decay': 0.9}, lr=0.02, momentum=0.5, l2_reg=1e-4)

    model = T.load_init(T.build_convnet(), gold)
    opt = make(model)
    for _ in range(2):
        opt.step(closure=_closure(model, x, y))
    path = str(tmp_path / 'ckpt.pt')
    torch.save({'model': model.state_dict(), 'optimizer': opt.state_dict()}, path)
    # nothing but tensors, numbers, strings and containers: the safe loader accepts it
    ckpt = torch.load(path, weights_only=True)

    model2 = T.build_convnet()
    model2.load_state_dict(ckpt['model'])
    opt2 = make(model2)
    opt2.param_groups[0]['lr'] = 123.          # overwritten by the checkpoint
    opt2.load_state_dict(ckpt['optimizer'])
    assert opt2.optim_state == opt.optim_state and opt2.param_groups[0]['lr'] == 0.02
    for g, g2 in zip(opt.param_groups, opt2.param_groups):
        assert g2['curv'].damping == g['curv'].damping
        for a, b in zip(g['curv'].ema, g2['curv'].ema):
            assert torch.equal(a, b) and a.data_ptr() != b.data_ptr()
    opt.step(closure=_closure(model, x, y))
    opt2.step(closure=_closure(model2, x, y))
    for p, q in zip(model.parameters(), model2.parameters()):
        assert torch.equal(p, q)

    # VI: the posterior means and their momentum buffers travel too
    vm = T.load_init(T.build_mlp(), T.load_golden('ref_mlp_vi_nosample'))
    vx, vy = torch.randn(8, 12), torch.randint(0, 5, (8,))
    vargs = dict(curv_kwargs={'damping': 1e-3, 'ema_decay': 0.95}, lr=0.05, momentum=0.9,
                 num_mc_samples=2)
    vopt = torchsso.optim.VIOptimizer(vm, 100, 'Cov', {'Linear': 'Kron'}, **vargs)
    vopt.step(closure=_closure(vm, vx, vy))
    sd = copy.deepcopy(vopt.state_dict())
    vm2 = T.build_mlp()
    vm2.load_state_dict(vm.state_dict())
    vopt2 = torchsso.optim.VIOptimizer(vm2, 100, 'Cov', {'Linear': 'Kron'}, **vargs)
    vopt2.load_state_dict(sd)
    la, _ = vopt.step(closure=_closure(vm, vx, vy))
    lb, _ = vopt2.step(closure=_closure(vm2, vx, vy))
    assert la.item() == lb.item()
    for g, g2 in zip(vopt.param_groups, vopt2.param_groups):
        for a, b in zip(g['mean'], g2['mean']):
            assert torch.equal(a, b)


def test_iteration_lr_schedules():
    from torchsso.optim import lr_scheduler as L
    model = nn.Linear(3, 2)
    opt = torch.optim.SGD(model.parameters(), lr=0.4, momentum=0.9)
    with pytest.raises(TypeError):
        L.PolynomialDecayIterLR(model, rate=2, max_count=10)
    sched = L.PolynomialDecayIterLR(opt, rate=2, max_count=10, start_iter=2)
    lrs = []
    for _ in range(12):
        sched.step()
        lrs.append(opt.param_groups[0]['lr'])
    # iterations 0, 1: untouched; from 2 on: 0.4 * (1 - (t - 2) / 8)^2, clamped at 0
    want = [0.4, 0.4] + [0.4 * max(1 - (t - 2) / 8, 0) ** 2 for t in range(2, 12)]
    assert lrs == pytest.approx(want, abs=1e-15)
    assert sched.state_dict()['last_iter'] == 11 and 'optimizer' not in sched.state_dict()

    opt = torch.optim.SGD(model.parameters(), lr=0.4, momentum=0.9)
    sched = L.PolynomialDecayIterLR(opt, rate=1, max_count=10, target=0.1)
    seen = []
    for _ in range(9):
        sched.step()
        seen.append(opt.param_groups[0]['lr'])
    assert seen == pytest.approx([max(0.4 * (1 - t / 10), 0.1) for t in range(9)], abs=1e-15)

    opt = torch.optim.SGD(model.parameters(), lr=0.4, momentum=0.9)
    warm = L.MomentumCorrectionLR(L.GradualWarmupIterLR(opt, initial_lr=0.1, max_count=4))
    assert opt.param_groups[0]['init_momentum'] == 0.9 and warm.max_count == 4
    lrs, moms = [], []
    for _ in range(6):
        warm.step()
        lrs.append(opt.param_groups[0]['lr'])
        moms.append(opt.param_groups[0]['momentum'])
    assert lrs == pytest.approx([0.1, 0.175, 0.25, 0.325, 0.4, 0.4], abs=1e-15)
    # momentum follows lr / previous lr (first step: no previous rate)
    assert moms[0] == 0.9 and moms[2] == pytest.approx(0.9 * 0.25 / 0.175)
    assert moms[5] == pytest.approx(0.9)
    # resuming needs initial_lr in the groups
    fresh = torch.optim.SGD(model.parameters(), lr=0.4)
    with pytest.raises(KeyError):
        L.GradualWarmupIterLR(fresh, 0.0, 4, last_iter=3)


def test_iteration_lr_schedules_match_reference():
    """The same schedules, stepped by the reference itself (golden sequences)."""
    from torchsso.optim import lr_scheduler as L
    gold = T.load_golden('ref_lr_schedules')

    def sgd():
        return torch.optim.SGD(nn.Linear(3, 2).parameters(), lr=0.4, momentum=0.9)

    def check(tag, opt, sched):
        want_lr, want_m = gold[tag + '.lr'], gold[tag + '.momentum']
        for k in range(len(want_lr)):
            sched.step()
            assert opt.param_groups[0]['lr'] == pytest.approx(want_lr[k], rel=1e-14, abs=1e-300), (tag, k)
            assert opt.param_groups[0]['momentum'] == pytest.approx(want_m[k], rel=1e-14), (tag, k)

    opt = sgd()
    check('poly_start2', opt, L.PolynomialDecayIterLR(opt, rate=2, max_count=10, start_iter=2))
    opt = sgd()
    sched = L.PolynomialDecayIterLR(opt, rate=1, max_count=10, target=0.1)
    check('poly_target', opt, sched)
    with pytest.raises(ZeroDivisionError):      # the reference divides by the decayed rate
        sched.step()
    opt = sgd()
    check('poly_negative_rate', opt, L.PolynomialDecayIterLR(opt, rate=-0.5, max_count=10, target=0.8))
    opt = sgd()
    check('warmup_momentum', opt,
          L.MomentumCorrectionLR(L.GradualWarmupIterLR(opt, initial_lr=0.1, max_count=4)))
    opt = sgd()
    opt.param_groups[0]['initial_lr'] = 0.4
    check('poly_resumed', opt, L.PolynomialDecayIterLR(opt, rate=2, max_count=10, last_iter=5))


def test_running_average_written_by_the_factor_kernels(oracle_ops):
    """With acc_steps == 1 the hooks build beta*factor + (1-beta)*ema straight into
    a second buffer and update_ema swaps buffers.  Same numbers as the unfused
    sequence; `data` is rebuilt on demand; a step without new factors re-applies
    the previous ones, as the reference's persistent `data` does."""
    gold = T.load_golden('ref_convnet_kfac')
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])

    def make(fuse):
        model = T.load_init(T.build_convnet(), gold)
        opt = torchsso.optim.SecondOrderOptimizer(
            model, 'Cov', {'Linear': 'Kron', 'Conv2d': 'Kron', 'BatchNorm2d': 'Diag'},
            {'damping': 1e-2, 'ema_decay': 0.9}, lr=0.02, momentum=0.5, l2_reg=1e-4)
        kron = [g['curv'] for g in opt.param_groups if g['curv'].kind == 'kron']
        assert all(c.fuse_ema for c in kron)
        if not fuse:
            for c in kron:
                c.fuse_ema = False
        return model, opt, kron

    (ma, oa, ka), (mb, ob, kb) = make(True), make(False)
    for step in range(3):
        seen = {}

        def closure_a():
            ret = _closure(ma, x, y)()
            seen['raw'] = [[d.clone() for d in c.data] for c in ka]
            seen['stored'] = [c._A is None and c._G is None for c in ka]
            return ret
        oa.step(closure=closure_a)
        ob.step(closure=_closure(mb, x, y))
        # first step: no average yet, the raw factors are stored; afterwards they are not
        assert seen['stored'] == [step > 0] * len(ka)
        for ca, cb, raw in zip(ka, kb, seen['raw']):
            for ea, eb, ra, rb in zip(ca.ema, cb.ema, raw, cb.data):
                assert O.rel_fro(ea, eb) < 1e-6
                assert O.rel_fro(ra, rb) < 1e-5          # rebuilt from the two averages
            assert abs(ca.damping - cb.damping) < 1e-12
    for p, q in zip(ma.parameters(), mb.parameters()):
        assert O.rel_fro(p.detach(), q.detach()) < 1e-6
    # a step with no forward/backward in between: the last factors enter again
    for m in (ma, mb):
        for p in m.parameters():
            p.grad = torch.ones_like(p) * 1e-3
    oa.step()
    ob.step()
    for ca, cb in zip(ka, kb):
        for ea, eb in zip(ca.ema, cb.ema):
            assert O.rel_fro(ea, eb) < 1e-5
    # accumulation over micro-steps and VI keep the raw factors
    m2 = T.load_init(T.build_convnet(), gold)
    o2 = torchsso.optim.SecondOrderOptimizer(m2, 'Cov', {'Linear': 'Kron', 'Conv2d': 'Kron'},
                                             {'damping': 1e-2, 'ema_decay': 0.9}, acc_steps=2)
    assert not any(getattr(g['curv'], 'fuse_ema', False) for g in o2.param_groups)
    m3 = T.build_mlp()
    o3 = torchsso.optim.VIOptimizer(m3, 100, 'Cov', {'Linear': 'Kron'},
                                    {'damping': 1e-3, 'ema_decay': 0.95}, num_mc_samples=2)
    assert not any(g['curv'].fuse_ema for g in o3.param_groups)


def test_packer_and_extractors_lay_out_the_wire_buffer(oracle_ops):
    from torchsso.utils import packer as P
    gold = T.load_golden('ref_mlp_kfac')
    model = T.load_init(T.build_mlp(), gold)
    x, y = torch.from_numpy(gold['x']), torch.from_numpy(gold['y'])
    opt = torchsso.optim.SecondOrderOptimizer(model, 'Cov', {'Linear': 'Kron'},
                                              {'damping': 1e-3, 'ema_decay': 0.95}, lr=0.05)
    opt.step(closure=_closure(model, x, y))
    # two rank blocks (layers 0-1 | layer 2): gradients whole, running averages as triangles
    extractors = [P.extract_attr_from_params('grad'), P.extract_attr_from_curv('ema', True)]
    arrays = P.extract(opt.param_groups, [[0, 1], [2]], extractors)
    assert [len(a) for a in arrays] == [8, 4]
    assert [tri for _, tri in arrays[0]] == [False, False, True, True] * 2
    n = P.get_nelems(arrays)
    want = 0
    for g in opt.param_groups:
        want += sum(p.numel() for p in g['params'])
        want += sum(e.shape[0] * (e.shape[0] + 1) // 2 for e in g['curv'].ema)
    assert n == want
    buf = torch.zeros(n + 7)
    packer = P.Packer()
    assert packer.pack(arrays, buf, offset=7) == n + 7
    first = opt.param_groups[0]
    assert torch.equal(buf[7:7 + first['params'][0].numel()], first['params'][0].grad.reshape(-1))
    # a reduced buffer coming back: unpack restores full symmetric matrices
    saved = [[t.clone() for t, _ in a] for a in arrays]
    for a in arrays:
        for t, _ in a:
            t.zero_()
    packer.unpack(arrays, buf, offset=7)
    for a, sv in zip(arrays, saved):
        for (t, tri), ref in zip(a, sv):
            assert torch.equal(t, ref)
    with pytest.raises(RuntimeError):          # 'non square matrix', as the reference raises
        _ops._pack_lists([(torch.zeros(2, 3), True)])


def test_constructor_validation_and_class_lookup():
    model = nn.Sequential(nn.Linear(4, 3))
    kw = dict(curv_type='Cov', curv_shapes={'Linear': 'Kron'}, curv_kwargs={'damping': 1e-3})
    for bad in (dict(lr=-1), dict(momentum=-1), dict(momentum=0.9, momentum_type='x'),
                dict(grad_ema_decay=2), dict(l2_reg=-1), dict(weight_decay=-1), dict(acc_steps=0),
                dict(lars=True, lars_type='x')):
        with pytest.raises(ValueError):
            torchsso.optim.SecondOrderOptimizer(model, **kw, **bad)
    for bad in ({'ema_decay': 1.5}, {'damping': -1e-3}, {'pi_type': 'other'}):
        with pytest.raises(ValueError):
            torchsso.optim.SecondOrderOptimizer(model, 'Cov', {'Linear': 'Kron'}, bad)
    with pytest.raises(AssertionError):
        torchsso.optim.SecondOrderOptimizer(model, 'Nope', {'Linear': 'Kron'}, {})
    for bad in (dict(dataset_size=-1), dict(dataset_size=10, num_mc_samples=0),
                dict(dataset_size=10, kl_weighting=-1), dict(dataset_size=10, prior_variance=-1)):
        with pytest.raises(ValueError):
            torchsso.optim.VIOptimizer(model, curv_type='Cov', curv_shapes={'Linear': 'Kron'},
                                       curv_kwargs={}, **bad)
    opt = torchsso.optim.SecondOrderOptimizer(model, **kw, momentum=0.9)
    g = opt.param_groups[0]
    for key in ('params', 'curv', 'acc_curv', 'acc_grads', 'lr', 'momentum', 'damping'):
        assert key in g
    assert g['curv'].shape == ((5, 5), (3, 3)) and g['curv'].bias
    st = opt.state[g['params'][0]]
    assert set(st) == {'momentum_buffer', 'grad_ema_buffer'}
    # Kron element_wise_init puts sqrt(value) on both diagonals
    g['curv'].element_wise_init(4.0)
    assert torch.equal(g['curv'].A, 2 * torch.eye(5)) and torch.equal(g['curv'].G, 2 * torch.eye(3))


def test_product_has_no_cpu_path():
    """Without the stand-in, CPU tensors are refused loudly."""
    model = nn.Sequential(nn.Linear(4, 3))
    torchsso.optim.SecondOrderOptimizer(model, 'Cov', {'Linear': 'Kron'}, {})
    with pytest.raises(_hip.KfacHipError):
        model(torch.randn(2, 4))
    with pytest.raises(_hip.KfacHipError):
        torchsso.utils.inv(torch.eye(3))
    acc = torchsso.utils.TensorAccumulator()
    with pytest.raises(AssertionError):
        acc.update([1.0, 2.0])


def test_factor_side_streams_host_logic():
    """The stream count is validated, and tensors that are not on a HIP device never
    reach a side stream (the launch runs where it is and raises there)."""
    from torchsso import _lanes
    before = torchsso.factor_streams()
    try:
        for bad in (-1, 9):
            with pytest.raises(ValueError):
                torchsso.set_factor_streams(bad)
        torchsso.set_factor_streams(2)
        assert torchsso.factor_streams() == 2
        calls = []
        out = _lanes.run(torch.device('cpu'), 5, (torch.zeros(1),), lambda st: calls.append(st) or 'out')
        assert out == 'out' and calls == [None]
        torchsso.join_factor_streams()        # nothing pending: no device is touched
    finally:
        torchsso.set_factor_streams(before)
    assert torchsso.factor_streams() == 2     # the default


def test_factor_mode_host_logic():
    """Grouped / eager mode and the flush threshold are validated on the host; a tensor that
    is not on a HIP device is never queued (its product runs, and raises, where it is)."""
    from torchsso import _lanes
    assert torchsso.factor_mode() == 'grouped'       # the default
    before_work = _lanes.flush_work()
    try:
        with pytest.raises(ValueError):
            torchsso.set_factor_mode('deferred')
        torchsso.set_factor_mode('eager')
        assert torchsso.factor_mode() == 'eager'
        torchsso.set_factor_mode('grouped')
        for bad in (0, -1.):
            with pytest.raises(ValueError):
                torchsso.set_factor_flush_work(bad)
        torchsso.set_factor_flush_work(None)
        assert _lanes.flush_work() is None
        torchsso.set_factor_flush_work(5e9)
        assert _lanes.flush_work() == 5e9
        assert _lanes.deferred_count() == 0
        lin = torch.nn.Linear(3, 2)
        curv = torchsso.KronCovLinear(lin)
        with pytest.raises(torchsso._hip.KfacHipError):
            lin(torch.randn(4, 3))                   # CPU input: no queue, no CPU path
        assert _lanes.deferred_count() == 0
        del curv
    finally:
        torchsso.set_factor_mode('grouped')
        torchsso.set_factor_flush_work(before_work)


def test_fisher_closure_exact_and_mc(oracle_ops):
    """Exact Fisher: the G factor of the logits layer equals mean_n(diag(p) - p p^T);
    every layer (also the first) gets a G factor; gradients are those of the true
    loss.  MC Fisher with many samples approaches the exact one."""
    torch.manual_seed(5)

    class Net(nn.Module):
        num_classes = 4

        def __init__(self):
            super().__init__()
            self.l1 = nn.Linear(6, 5)
            self.l2 = nn.Linear(5, 4)

        def forward(self, x):
            return self.l2(F.relu(self.l1(x)))

    model = Net()
    x, y = torch.randn(10, 6), torch.randint(0, 4, (10,))
    import copy
    plain = copy.deepcopy(model)      # no curvature hooks on this one
    opt = torchsso.optim.SecondOrderOptimizer(model, 'Fisher', {'Linear': 'Kron'},
                                              {'damping': 1e-3, 'ema_decay': 1.}, lr=0.0)
    assert type(opt.param_groups[0]['curv']).__name__ == 'KronFisherLinear'
    ref_grads = torch.autograd.grad(F.cross_entropy(plain(x), y), list(plain.parameters()))
    p = torch.softmax(plain(x), 1).detach()
    closed = sum(torch.diag(p[i]) - torch.outer(p[i], p[i]) for i in range(10)) / 10
    raw = {}

    def closure():
        ret = torchsso.get_closure_for_fisher(opt, model, x, y)()
        raw['g'] = [q.grad.clone() for q in model.parameters()]
        raw['G'] = [g['curv'].G.clone() for g in opt.param_groups]
        return ret
    opt.step(closure=closure)
    for got, ref in zip(raw['g'], ref_grads):
        assert torch.allclose(got, ref, atol=1e-6)
    assert torch.allclose(raw['G'][1], closed, atol=1e-5)
    assert raw['G'][0].abs().sum() > 0 and all(q.requires_grad for q in model.parameters())
    exact_first = raw['G'][0]
    torch.manual_seed(0)
    mc = torchsso.get_closure_for_fisher(opt, model, x, y, approx_type='mc', num_mc=4000)
    mc()
    assert torch.allclose(opt.param_groups[1]['curv'].G, closed, atol=0.02)
    assert (opt.param_groups[0]['curv'].G - exact_first).norm() / exact_first.norm() < 0.15
    with pytest.raises(ValueError):
        torchsso.get_closure_for_fisher(opt, model, x, y, approx_type='bogus')()


def test_layers_are_sorted_into_classes_by_the_length_of_their_factorisation():
    """curvature.chain_classes: which layers keep the caller's stream in the curvature phase
    (those holding a factor of more than half the largest dimension) and which go to the
    side stream; one class where the largest factor is small or nothing would be left."""
    from torchsso.curv.curvature import chain_classes
    # ResNet-50-like: three 4608-row layers, 2304 / 2048-row ones, small ones, BatchNorm (0)
    dims = [147, 0, 576, 4608, 2304, 0, 2048, 4608, 1024, 2049, 4608]
    assert chain_classes(dims, 2048, 2) == [[3, 7, 10], [0, 1, 2, 4, 5, 6, 8, 9]]
    # exactly half the largest dimension belongs to the second class, one more row does not
    assert chain_classes([4608, 2304, 2305], 2048, 2) == [[0, 2], [1]]
    # AlexNet's classifier: fc6 against fc7 / fc8
    assert chain_classes([9217, 4097, 4097], 2048, 2) == [[0], [1, 2]]
    # three classes when allowed
    assert chain_classes([9217, 4097, 1000, 0], 2048, 3) == [[0], [1], [2, 3]]
    # small factors, a single class, or only layers without factors left: one stream
    assert chain_classes([1001, 1000, 11], 2048, 2) is None
    assert chain_classes([4608, 4000], 2048, 2) is None
    assert chain_classes([4608, 0, 0], 2048, 2) is None
    assert chain_classes([4608, 100], None, 2) is None
    assert chain_classes([4608, 100], 2048, 1) is None
