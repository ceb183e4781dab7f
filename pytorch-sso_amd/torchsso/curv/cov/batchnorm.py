"""Diagonal curvature of BatchNorm layers.

Mirrors torchsso/curv/cov/batchnorm.py:10-49 of the reference:
    w_curv[c] = mean_n[(sum_hw x_hat^2)(sum_hw g^2)],  b_curv[c] = mean_n[sum_hw g^2]
followed by the n^2 rescale (curvature.py:154-158), where
x_hat = (out - bias) / weight is the normalised input (curvature.py:123-134).
sum_hw x_hat^2 is reduced straight from the layer output in the forward hook
(before an in-place activation can touch it) and x_hat itself is never stored.
"""
import torch
import torch.nn as nn

from torchsso import _lanes, _ops
from torchsso.curv.curvature import Curvature, DiagCurvature


class CovBatchNorm1d(Curvature):

    def update_in_backward(self, grad_output_data):
        pass


class CovBatchNorm2d(Curvature):

    def update_in_backward(self, grad_output):
        pass


class _DiagCovBatchNorm(DiagCurvature):

    # set to True (on the class or an instance) to have the forward hook store the
    # normalised input x_hat = (out - bias) / weight as module.data_input
    expose_normalized_input = False

    def forward_postprocess(self, module, input, output):
        assert self._module == module
        bn = module
        if not isinstance(bn, (nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d)):
            raise TypeError('expected a BatchNorm module, got %s' % type(bn).__name__)
        out = output.detach()
        # [n, c] sums over the spatial positions of ((out - bias) / weight)^2
        self._sx = _ops.rowsq_sum(out, bn.num_features, bn.weight.detach(), bn.bias.detach())
        # module.data_input: x_hat, as the reference keeps it (curvature.py:123-136), only
        # on request: it costs a pass over the activation and a tensor of its size that
        # nothing here reads
        if self.expose_normalized_input:
            shape = (1, -1) + (1,) * (out.dim() - 2)
            x_hat = (out - bn.bias.detach().view(shape)) / bn.weight.detach().view(shape)
        else:
            x_hat = None
        setattr(module, 'data_input', x_hat)
        setattr(module, 'data_output', output)
        if output.requires_grad:
            output.register_hook(self._on_grad_output)

    # In grouped mode the backward reduction is only queued by the hook (the output gradient
    # stays referenced) and runs with those of the other BatchNorm layers in ONE launch when
    # the queue runs (torchsso._lanes); whoever reads `data` first has it run.
    _queued = False

    @property
    def data(self):
        if self._queued:
            self._queued = False
            _lanes.join()
        return self._data

    @data.setter
    def data(self, value):
        if self._queued:            # (the queued reduction writes the tensors it was given)
            self._queued = False
            _lanes.join()
        self._data = value

    def adjust_data_scale(self, scale):
        self.data                   # (runs a queued reduction first)
        super(_DiagCovBatchNorm, self).adjust_data_scale(scale)

    def update_in_backward(self, grad_output):
        n = grad_output.shape[0]
        channels = self._module.num_features
        device = grad_output.device
        if (_lanes.mode() == 'grouped' and device.type == 'cuda'
                and n <= _ops.BN_BATCH_MAX_ROWS):
            g = grad_output.contiguous()
            w = torch.empty(channels, dtype=torch.float32, device=device)
            b = torch.empty(channels, dtype=torch.float32, device=device) if self.bias else None
            _lanes.defer_bn(device, (id(self), 'bn'), (g, channels, self._sx, float(n), w, b))
            self._data = [w] if b is None else [w, b]
            self._queued = True
            return
        w, b = _ops.bn_diag_cov(grad_output, channels, self._sx, float(n), self.bias)   # n^2 / n
        self._data = [w] if b is None else [w, b]


class DiagCovBatchNorm1d(_DiagCovBatchNorm):
    pass


class DiagCovBatchNorm2d(_DiagCovBatchNorm):
    pass
