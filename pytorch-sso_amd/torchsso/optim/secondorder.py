"""SecondOrderOptimizer: K-FAC style preconditioned SGD driven by per-layer
curvature objects.

Same constructor, param_group layout, `step(closure)` contract and update rule
as torchsso/optim/secondorder.py:15-330 of the reference.  The per-layer loop
of the reference (secondorder.py:195-209) is regrouped by phase -- layers are
independent, so the results are the same -- and every phase is one batched call
into the HIP engine:

    raw phase            grad += l2_reg * p                    (axpby kernel)
    curvature phase      EMA, pi-damped inverses of all layers (batched Cholesky)
    precondition phase   G^-1 [dW|db] A^-1 for all layers      (two MFMA launches)
    update phase         weight decay, momentum, p -= lr * g   (one fused kernel)

Raw-gradient momentum, gradient EMA and bias correction run on the same
element-wise kernels in the reference's order; LARS and weight normalisation
need tensor norms on the host and use torch's norm() for them.
"""
import math

import numpy as np
import torch
import torch.nn as nn
from torch.optim import Optimizer

import torchsso
from torchsso import _ops
from torchsso.curv import curvature as _curv
from torchsso.utils import TensorAccumulator


class SecondOrderOptimizer(Optimizer):
    r"""Optimizer that preconditions each layer's gradient with the inverse of
    that layer's curvature.

    Args (as the reference, secondorder.py:23-49):
        model (torch.nn.Module): model with parameters to be trained
        curv_type (str): 'Cov' (this package builds the 'Cov' curvatures)
        curv_shapes (dict): curvature shape per module class name, e.g.
            {"Conv2d": "Kron", "Linear": "Kron", "BatchNorm2d": "Diag"}
        curv_kwargs (dict): keyword arguments of torchsso.Curvature.__init__
        lr, momentum, momentum_type ('raw' | 'preconditioned'),
        grad_ema_decay, grad_ema_type, l2_reg, weight_decay,
        normalizing_weights, weight_scale, acc_steps, non_reg_for_bn,
        bias_correction, lars, lars_type, update_inv, precondition_grad
        check_spd (bool, not in the reference): raise NotPositiveDefiniteError when the
            inversion of a step met a factor that is not positive definite
    """

    def __init__(self, model: nn.Module, curv_type: str, curv_shapes: dict, curv_kwargs: dict,
                 lr=0.01, momentum=0., momentum_type='preconditioned',
                 grad_ema_decay=1., grad_ema_type='raw', l2_reg=0., weight_decay=0.,
                 normalizing_weights=False, weight_scale=None,
                 acc_steps=1, non_reg_for_bn=False, bias_correction=False,
                 lars=False, lars_type='preconditioned', update_inv=True, precondition_grad=True,
                 check_spd=False):

        if lr < 0:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if momentum < 0:
            raise ValueError("Invalid momentum: {}".format(momentum))
        if momentum > 0 and momentum_type not in ['raw', 'preconditioned']:
            raise ValueError("Invalid momentum type: {}".format(momentum_type))
        if grad_ema_decay < 0 or 1 < grad_ema_decay:
            raise ValueError("Invalid grad_ema value: {}".format(grad_ema_decay))
        if grad_ema_decay > 0 and grad_ema_type not in ['raw', 'preconditioned']:
            raise ValueError("Invalid grad_ema type: {}".format(grad_ema_type))
        if l2_reg < 0:
            raise ValueError("Invalid l2_reg value: {}".format(l2_reg))
        if weight_decay < 0:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        if acc_steps < 1:
            raise ValueError("Invalid acc_steps: {}".format(acc_steps))
        if lars and lars_type not in ['raw', 'preconditioned']:
            raise ValueError("Invalid LARS type: {}".format(lars_type))
        if normalizing_weights and weight_scale is not None and weight_scale <= 0:
            raise ValueError("Invalid weight scale for LARS: {}".format(weight_scale))

        self.model = model
        defaults = {'lr': lr, 'momentum': momentum, 'momentum_type': momentum_type,
                    'grad_ema_decay': grad_ema_decay, 'grad_ema_type': grad_ema_type,
                    'l2_reg': l2_reg, 'weight_decay': weight_decay,
                    'normalizing_weights': normalizing_weights, 'weight_scale': weight_scale,
                    'acc_steps': acc_steps, 'bias_correction': bias_correction,
                    'lars': lars, 'lars_type': lars_type}
        defaults.update(curv_kwargs)

        self.curv_type = curv_type
        self.curv_shapes = {} if curv_shapes is None else curv_shapes
        self.update_inv = update_inv
        self.precondition_grad = precondition_grad
        # opt-in (not in the reference): after the inversion of a step, read the solver's
        # status words once (a host synchronisation) and raise if a factor was not
        # positive definite; may also be switched on later as an attribute
        self.check_spd = bool(check_spd)
        self.optim_state = {'step': 0, 'acc_step': 0}

        # one param_group per leaf module that owns parameters
        groups = []
        bn_groups = []
        for module in model.modules():
            if len(list(module.children())) > 0:
                continue
            params = list(module.parameters())
            if len(params) == 0:
                continue
            curv_class = self.get_curv_class(module)
            curvature = curv_class(module, **curv_kwargs)
            group = {'params': params, 'curv': curvature,
                     'acc_curv': TensorAccumulator(), 'acc_grads': TensorAccumulator()}
            groups.append(group)
            if non_reg_for_bn and isinstance(module, (nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d)):
                bn_groups.append(group)
        if len(groups) == 0:
            raise ValueError("model has no parameters to optimize")

        # torch's base class fills every group with the defaults and sets up
        # `state`; the reference assigns those fields by hand instead
        # (secondorder.py:94-106), which current torch no longer tolerates.
        super(SecondOrderOptimizer, self).__init__(groups, defaults)

        # Without accumulation over micro-steps nothing reads the raw Kronecker
        # factors between the hooks and step(): the factor kernels then write the
        # running average themselves (curvature.py, KronCurvature.fuse_ema).
        if acc_steps == 1 and self._fuse_running_average:
            for group in self.param_groups:
                if type(group['curv']) in (torchsso.KronCovLinear, torchsso.KronCovConv2d):
                    group['curv'].fuse_ema = True

        for group in self.param_groups:
            self.init_buffer(group['params'])
        for group in bn_groups:
            group['l2_reg'] = 0
            group['weight_decay'] = 0
            group['normalizing_weights'] = False

    _fuse_running_average = True     # VIOptimizer accumulates over MC samples: off there

    def init_buffer(self, params):
        for p in params:
            state = self.state[p]
            state['momentum_buffer'] = torch.zeros_like(p.data)
            state['grad_ema_buffer'] = torch.zeros_like(p.data)

    @property
    def local_param_groups(self):
        return self.param_groups

    def get_curv_class(self, module):
        """Class looked up by name on the package namespace: shape + type + module
        class, e.g. 'Kron' + 'Cov' + 'Linear' (reference: secondorder.py:148-156)."""
        module_name = module.__class__.__name__
        curv_shape = self.curv_shapes.get(module_name, '')
        curv_name = curv_shape + self.curv_type + module_name
        curv_class = getattr(torchsso, curv_name, None)

        assert curv_class is not None, f"Failed to lookup Curvature class {curv_name} for {module}."

        return curv_class

    # ----------------------------------------------------------- checkpointing

    _GROUP_OBJECTS = ('params', 'curv', 'acc_curv', 'acc_grads', 'mean')

    def state_dict(self):
        """Checkpoint of tensors, numbers and strings only (loadable with
        torch.load(..., weights_only=True)): the step counters and, per param
        group, its options (lr, momentum, ...), the curvature's ema / inv / std, the
        momentum and gradient-EMA buffers and, for VI, the posterior means.
        torch's default would pickle the Curvature objects held in param_groups, as
        the reference's checkpoints do."""
        groups = []
        for group in self.param_groups:
            entry = {'options': {k: v for k, v in group.items() if k not in self._GROUP_OBJECTS}}
            curv = group['curv']
            entry['curvature'] = None if curv is None else curv.state_dict()
            for target in ('params', 'mean'):
                if target not in group:
                    continue
                entry[target + '_buffers'] = [
                    {k: v.detach().clone() for k, v in self.state[t].items() if torch.is_tensor(v)}
                    for t in group[target]]
            if 'mean' in group:
                entry['mean'] = [m.detach().clone() for m in group['mean']]
            groups.append(entry)
        return {'optim_state': dict(self.optim_state), 'groups': groups}

    def load_state_dict(self, state_dict):
        groups = state_dict['groups']
        if len(groups) != len(self.param_groups):
            raise ValueError('checkpoint has %d param groups, the optimizer has %d'
                             % (len(groups), len(self.param_groups)))
        for group, entry in zip(self.param_groups, groups):
            group.update(entry['options'])
            curv = group['curv']
            if curv is not None and entry['curvature'] is not None:
                curv.load_state_dict(entry['curvature'])
            for target in ('params', 'mean'):
                bufs = entry.get(target + '_buffers')
                if bufs is None or target not in group:
                    continue
                if len(bufs) != len(group[target]):
                    raise ValueError('checkpoint group has %d %s, the optimizer has %d'
                                     % (len(bufs), target, len(group[target])))
                for t, saved in zip(group[target], bufs):
                    for k, v in saved.items():
                        self.state[t][k] = v.detach().to(device=t.device, dtype=t.dtype).clone()
            if 'mean' in entry and 'mean' in group:
                for m, saved in zip(group['mean'], entry['mean']):
                    m.data.copy_(saved)
        self.optim_state = dict(state_dict['optim_state'])

    # ------------------------------------------------------------------ step

    def step(self, closure=None):
        """One optimization step.  `closure` runs forward and backward and returns
        the loss or (loss, output); its return value is passed through."""
        n = self.defaults['acc_steps']
        loss = None

        if closure is not None:
            loss = closure()

            if n > 1:
                self._accumulate(1 / n)

            self.optim_state['acc_step'] += 1
            if self.optim_state['acc_step'] < n:
                return loss
            self.optim_state['acc_step'] = 0

            if n > 1:
                self.backward_postprocess()
            # n == 1: the accumulated values are the gradients and factors
            # themselves (scale 1), so they are used where they lie

        self.optim_state['step'] += 1
        self._update_groups(self.local_param_groups, target='params',
                            update_inv=self.update_inv, update_std=False,
                            precondition=self.precondition_grad)
        return loss

    def _begin_accumulation(self, weight):
        """Before forward / backward passes whose factors will be accumulated with `weight`:
        the Kronecker curvatures add their factors to the group's accumulator in the factor
        products themselves (KronCurvature.accumulate_into), so `_accumulate` has only the
        gradients and the diagonal curvatures left.  Used where no user code runs between the
        passes that could ask for a single pass's factor (the MC loop of VIOptimizer.step);
        accumulation over micro-steps, between which the caller has the floor, adds up stored
        factors as the reference does."""
        for group in self.param_groups:
            curv = group['curv']
            if curv is not None and curv.kind == 'kron' and not curv.fuse_ema:
                curv.accumulate_into(group['acc_curv'], weight)

    def _end_accumulation(self):
        """The hooks store their factors again (the accumulators keep what they hold)."""
        for group in self.param_groups:
            curv = group['curv']
            if curv is not None and curv.kind == 'kron':
                curv.accumulate_into(None, 0.)

    def _accumulate(self, weight):
        """Adds weight * (current gradients, current curvature data) of every group to the
        group's accumulators (reference: secondorder.py:175-182, vi.py:211-220)."""
        accs, datas = [], []
        for group in self.param_groups:
            accs.append(group['acc_grads'])
            datas.append([p.grad.data for p in group['params']])
            curv = group['curv']
            if curv is not None and getattr(curv, '_acc_into', None) is None:
                accs.append(group['acc_curv'])
                datas.append(curv.data)
        TensorAccumulator.update_many(accs, datas, scale=weight)   # one launch for all layers

    def _update_groups(self, groups, target, update_inv, update_std, precondition):
        self._l2_all(groups, target)        # grad += l2_reg * p, one launch per distinct l2_reg
        for group in groups:
            self.update_preprocess(group, target=target, grad_type='raw', l2_done=True)

        def finish(sub):
            """Everything behind the preconditioning, for the groups in `sub`."""
            fused = []
            for group in sub:
                if self._can_fuse_update(group):
                    fused.append(group)
                else:
                    self.update_preprocess(group, target=target, grad_type='preconditioned')
                    self.update(group, target=target)
            self._fused_update(fused, target)
            for group in sub:
                self.update_postprocess(group, target=target)

        with_curv = [g for g in groups if g['curv'] is not None]
        curvs = [g['curv'] for g in with_curv]
        if curvs:
            if isinstance(update_std, (list, tuple)):
                update_std = [u for g, u in zip(groups, update_std) if g['curv'] is not None]
            pairs = [(g['curv'], g[target]) for g in with_curv]
            by_curv = {id(g['curv']): g for g in with_curv}
            finish_pairs = lambda sub: finish([by_curv[id(c)] for c, _ in sub])
            if getattr(self, 'check_spd', False):
                _curv.step_all(curvs, update_std=update_std, update_inv=update_inv)
                _curv.check_spd_all(curvs)       # (before anything is preconditioned)
                if precondition:
                    _curv.precondition_all(pairs)
                finish(with_curv)
            else:
                # (the layers are independent: where the curvature phase runs on two
                # streams, each part's update follows its preconditioning on its stream)
                _curv.step_and_precondition_all(pairs, update_std=update_std,
                                                update_inv=update_inv, precondition=precondition,
                                                then=finish_pairs)
        finish([g for g in groups if g['curv'] is None])

    def backward_postprocess(self, target='params'):
        """Accumulated gradients and factors become the current ones
        (reference: secondorder.py:213-223)."""
        for group in self.param_groups:
            acc_grads = group['acc_grads'].get()
            for p, acc_grad in zip(group[target], acc_grads):
                p.grad = acc_grad
            curv = group['curv']
            if curv is not None:
                curv.data = group['acc_curv'].get()
                if curv.kind == 'kron':
                    curv.accumulate_into(None, 0.)

    # ------------------------------------------------------------ update tail

    @staticmethod
    def _can_fuse_update(group):
        """The fused kernel covers weight decay, momentum on the preconditioned
        gradient and the parameter update."""
        # (momentum on the raw gradient was already applied in the raw phase)
        if group['grad_ema_decay'] != 1 and group['grad_ema_type'] == 'preconditioned':
            return False
        if group['bias_correction']:
            return False
        if group['lars'] and group['lars_type'] == 'preconditioned':
            return False
        return True

    def _fused_update(self, groups, target):
        ps, gs, bufs, lrs, moms, wds = [], [], [], [], [], []
        for group in groups:
            mom = group['momentum'] if group['momentum_type'] == 'preconditioned' else 0.
            for p in group[target]:
                grad = p.grad
                if grad is None:
                    continue
                if not grad.is_contiguous():
                    p.grad = grad = grad.contiguous()
                ps.append(p.data)
                gs.append(grad)
                bufs.append(self.state[p]['momentum_buffer'] if mom != 0 else None)
                lrs.append(group['lr'])
                moms.append(mom)
                wds.append(group['weight_decay'])
        _ops.sgd_update_batched(ps, gs, bufs, lrs, moms, wds)

    def update(self, group, target='params'):
        """p -= lr * grad (reference: secondorder.py:225-231)."""
        ps, gs = [], []
        for p in group[target]:
            if p.grad is None:
                continue
            ps.append(p.data)
            gs.append(p.grad)
        if ps:
            _ops.axpby_batched(gs, ps, -group['lr'], 1.)

    def _l2_all(self, groups, target):
        """The l2 term of the raw phase for all groups at once (reference:
        secondorder.py:238-243, per group): grad += l2_reg * p, and the curvature learns
        the coefficient (it enters the damping through its running average)."""
        by_coeff = {}
        for group in groups:
            if group['l2_reg'] == 0:
                continue
            params = [p for p in group[target] if p.grad is not None]
            for p in params:
                if p.grad.is_sparse:
                    raise RuntimeError(
                        "l2 regularization option is not compatible with sparse gradients")
            ps, gs = by_coeff.setdefault(group['l2_reg'], ([], []))
            ps.extend(p.data for p in params)
            gs.extend(p.grad for p in params)
            if params and group['curv'] is not None:
                group['curv'].l2_reg = group['l2_reg']
        for coeff, (ps, gs) in by_coeff.items():
            _ops.axpby_batched(ps, gs, coeff, 1.)

    def update_preprocess(self, group, target='params', grad_type='raw', l2_done=False):
        """Gradient transformations before ('raw') and after ('preconditioned')
        preconditioning, in the reference's order (secondorder.py:233-312)."""
        assert grad_type in ['raw', 'preconditioned'], 'Invalid grad type: {}.'.format(grad_type)
        params = [p for p in group[target] if p.grad is not None]
        if not params:
            return
        state = self.state

        if grad_type == 'raw' and group['l2_reg'] != 0 and not l2_done:
            for p in params:
                if p.grad.is_sparse:
                    raise RuntimeError(
                        "l2 regularization option is not compatible with sparse gradients")
            _ops.axpby_batched([p.data for p in params], [p.grad for p in params],
                               group['l2_reg'], 1.)
            curv = group['curv']
            if curv is not None:
                curv.l2_reg = group['l2_reg']

        if grad_type == 'preconditioned' and group['weight_decay'] != 0:
            for p in params:
                if p.grad.is_sparse:
                    raise RuntimeError(
                        "weight_decay option is not compatible with sparse gradients")
            _ops.axpby_batched([p.data for p in params], [p.grad for p in params],
                               group['weight_decay'], 1.)

        if group['momentum_type'] == grad_type and group['momentum'] != 0:
            bufs = [state[p]['momentum_buffer'] for p in params]
            grads = [p.grad for p in params]
            _ops.axpby_batched(grads, bufs, 1., group['momentum'])      # buf = m*buf + g
            _ops.axpby_batched(bufs, grads, 1., 0.)                     # g = buf

        if group['grad_ema_type'] == grad_type and group['grad_ema_decay'] != 1:
            decay = group['grad_ema_decay']
            bufs = [state[p]['grad_ema_buffer'] for p in params]
            grads = [p.grad for p in params]
            _ops.axpby_batched(grads, bufs, decay, 1 - decay)           # buf = (1-d)*buf + d*g
            _ops.axpby_batched(bufs, grads, 1., 0.)

        if grad_type == 'preconditioned' and group['bias_correction']:
            curv = group['curv']
            beta1 = 1 - group['grad_ema_decay']
            beta2 = 1 - curv.ema_decay
            bias_correction1 = 1 - beta1 ** self.optim_state['step']
            bias_correction2 = 1 - beta2 ** self.optim_state['step']
            if getattr(curv, 'use_sqrt_ema', False):
                bias_correction2 = math.sqrt(bias_correction2)
            grads = [p.grad for p in params]
            _ops.axpby_batched(grads, grads, bias_correction2 / bias_correction1, 0.)

        if group['lars_type'] == grad_type and group['lars']:
            thr, eps = 1e-2, 1e-9
            for p in params:
                d_norm = p.data.norm()
                if d_norm > thr:
                    g_norm = p.grad.norm()
                    p.grad.mul_(d_norm / (g_norm + eps))

    def update_postprocess(self, group, target='params'):
        """Optional weight normalisation (reference: secondorder.py:314-330)."""
        if not group['normalizing_weights']:
            return
        curv = group['curv']
        thr, eps = 1e-2, 1e-9
        for p, _p in zip(group[target], group['params']):
            w = getattr(curv.module, 'weight', None)
            if w is not None and w is _p:
                d_norm = p.data.norm()
                if d_norm > thr:
                    scale = group['weight_scale']
                    if scale is None:
                        scale = np.sqrt(2.0 * w.data.shape[0])
                    p.data.div_(d_norm + eps).mul_(scale)
