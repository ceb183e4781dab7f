"""True-Fisher curvatures: the output-gradient factor is weighted per sample by a
probability and summed over the classes (exact) or over labels sampled from the
model's own predictive distribution (Monte Carlo).

Mirrors torchsso/curv/fisher/__init__.py, fisher/linear.py:38-63,
fisher/conv.py:50-69 and fisher/batchnorm.py:5-32 of the reference.  On the
engine side the weighting is sqrt(prob) applied to the output gradient
(kfac_scale_rows) followed by the ordinary symmetric factor kernel, and the sum
over the extra backward passes is that kernel's accumulate epilogue (beta = 1),
so no per-pass factor is ever materialised.
"""
import torch
import torch.nn.functional as F

from torchsso import _ops
from torchsso.curv.cov.batchnorm import DiagCovBatchNorm2d
from torchsso.curv.cov.conv import DiagCovConv2d, KronCovConv2d
from torchsso.curv.cov.linear import DiagCovLinear, KronCovLinear


class Fisher(object):
    """State shared by the Fisher curvatures (reference: fisher/__init__.py:7-31)."""

    def __init__(self):
        self.prob = None
        self._do_backward = True
        self._acc = None        # running sum over the weighted backward passes

    @property
    def do_backward(self):
        return self._do_backward

    def turn_on_backward(self):
        self._do_backward = True

    def turn_off_backward(self):
        self._do_backward = False

    def finalize(self):
        acc, self._acc = self._acc, None
        return acc

    def update_as_presoftmax(self, prob):
        raise NotImplementedError('This method supports only torchsso.KronFisherLinear.')


class _DiagFisher(Fisher):
    """Diagonal Fisher of a Linear / Conv2d layer: the per-sample gradients are
    weighted by sqrt(prob) through the output gradient, so their squares carry
    prob (reference: fisher/linear.py:5-35, fisher/conv.py:6-47)."""

    def update_in_backward(self, grad_output):
        if self.do_backward:
            assert self.prob is not None
            n = grad_output.shape[0]
            pg = _ops.scale_rows(grad_output, self.prob.reshape(n), True)
            data = self._diag_data(pg)
            if self._acc is None:
                self._acc = data
            else:
                _ops.axpby_batched([d.reshape(-1) for d in data],
                                   [a.reshape(-1) for a in self._acc], 1., 1.)
            self._data = self._acc
        else:
            self._data = self.finalize()


class DiagFisherLinear(_DiagFisher, DiagCovLinear):

    def __init__(self, *args, **kwargs):
        DiagCovLinear.__init__(self, *args, **kwargs)
        Fisher.__init__(self)


class DiagFisherConv2d(_DiagFisher, DiagCovConv2d):

    def __init__(self, *args, **kwargs):
        DiagCovConv2d.__init__(self, *args, **kwargs)
        Fisher.__init__(self)


class KronFisherLinear(KronCovLinear, Fisher):

    def __init__(self, *args, **kwargs):
        KronCovLinear.__init__(self, *args, **kwargs)
        Fisher.__init__(self)

    def update_in_backward(self, grad_output):
        if self.do_backward:
            assert self.prob is not None
            n = grad_output.shape[0]
            # G += (1/n) sum_k prob[k] g_k g_k^T, times n^2 (curvature.py:154-155)
            pg = _ops.scale_rows(grad_output.reshape(n, -1), self.prob.reshape(n), True)
            first = self._acc is None
            self._acc = _ops.factor_linear(pg, False, float(n), out=self._acc,
                                           beta=0. if first else 1.)
            self._G = self._acc
        else:
            self._G = self.finalize()

    def update_as_presoftmax(self, prob):
        """Closed form for the layer that produces the logits:
        G = (diag(sum_n p_n) - P^T P / n) / n   (reference: fisher/linear.py:58-63)."""
        n, dim = prob.shape
        cov = _ops.factor_linear(prob.detach(), False, 1.0 / n)
        self._G = (torch.diag(prob.detach().sum(dim=0)) - cov) / n


class KronFisherConv2d(KronCovConv2d, Fisher):

    def __init__(self, *args, **kwargs):
        KronCovConv2d.__init__(self, *args, **kwargs)
        Fisher.__init__(self)

    def update_in_backward(self, grad_output):
        if self.do_backward:
            assert self.prob is not None
            n, c, h, w = grad_output.shape
            pg = _ops.scale_rows(grad_output, self.prob.reshape(n), True)
            first = self._acc is None
            self._acc = _ops.factor_conv_g(pg, float(n) / (h * w), out=self._acc,
                                           beta=0. if first else 1.)
            self._G = self._acc
        else:
            self._G = self.finalize()


class DiagFisherBatchNorm2d(DiagCovBatchNorm2d, Fisher):

    def __init__(self, *args, **kwargs):
        DiagCovBatchNorm2d.__init__(self, *args, **kwargs)
        Fisher.__init__(self)

    def update_in_backward(self, grad_out):
        if self.do_backward:
            assert self.prob is not None
            n = grad_out.shape[0]
            sg = _ops.rowsq_sum(grad_out, self._module.num_features)
            sg = _ops.scale_rows(sg, self.prob.reshape(n), False)      # prob * sum_hw g^2
            w, b = _ops.bn_diag_combine(self._sx, sg, float(n), self.bias)
            data = [w] if b is None else [w, b]
            if self._acc is None:
                self._acc = data
            else:
                _ops.axpby_batched(data, self._acc, 1., 1.)
            self._data = self._acc
        else:
            self._data = self.finalize()


def get_closure_for_fisher(optimizer, model, data, target, approx_type=None, num_mc=1):
    """Closure for `optimizer.step` that fills the Fisher curvatures (reference:
    fisher/__init__.py:34-90).  approx_type None: exact sum over the classes,
    each backward pass weighted by that class's predicted probability; 'mc':
    `num_mc` labels drawn from the predictive distribution, weight 1/num_mc.
    During those passes the parameters do not require grad (only the curvature
    hooks see gradients); a final ordinary backward pass yields the loss
    gradients.  A floating-point input is made to require grad during the extra
    passes so that the first layer's output gradient exists as well."""
    _APPROX_TYPE_MC = 'mc'

    def set_param_grad(flag):
        for group in optimizer.param_groups:
            if flag:
                group['curv'].turn_off_backward()
            else:
                group['curv'].turn_on_backward()
            for param in group['params']:
                param.requires_grad = flag

    def closure():
        for group in optimizer.param_groups:
            assert isinstance(group['curv'], Fisher), f"Invalid Curvature type: {type(group['curv'])}."
        if approx_type is not None and approx_type != _APPROX_TYPE_MC:
            raise ValueError('Invalid approx type: {}'.format(approx_type))

        optimizer.zero_grad()
        x = data
        if torch.is_floating_point(data) and not data.requires_grad:
            x = data.detach().requires_grad_(True)
        output = model(x)
        prob = F.softmax(output, dim=1)

        set_param_grad(False)
        if approx_type == _APPROX_TYPE_MC:
            dist = torch.distributions.Categorical(prob)
            _target = dist.sample((num_mc,))
            for group in optimizer.param_groups:
                group['curv'].prob = torch.ones_like(prob[:, 0]).div(num_mc)
            for i in range(num_mc):
                loss = F.cross_entropy(output, _target[i])
                loss.backward(retain_graph=True)
        else:
            for i in range(model.num_classes):
                for group in optimizer.param_groups:
                    group['curv'].prob = prob[:, i].detach()
                loss = F.cross_entropy(output, torch.ones_like(target).mul(i))
                loss.backward(retain_graph=True)
        set_param_grad(True)

        loss = F.cross_entropy(output, target)
        loss.backward()

        return loss, output

    return closure
