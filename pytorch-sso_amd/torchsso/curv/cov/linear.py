"""Curvature of nn.Linear from the covariance of per-sample gradients.

KronCovLinear mirrors torchsso/curv/cov/linear.py:48-114 of the reference; the
factors come from the HIP factor kernel, with the bias column (LAST) synthesised
in the kernel and the 1/n and n^2 scalings folded into its scale factor.
DiagCovLinear mirrors cov/linear.py:28-45: one product of the squared output
gradient with the squared input, the operands squared inside the kernel.
"""
from torchsso import _ops
from torchsso.curv.curvature import Curvature, DiagCurvature, KronCurvature


class CovLinear(Curvature):
    """Full (dense) covariance of a Linear layer: named by the reference
    (cov/linear.py:5-25) but not part of the K-FAC path; not implemented here."""

    def update_in_backward(self, grad_output):
        raise NotImplementedError('CovLinear (dense curvature) is outside the K-FAC path')

    def precondition_grad(self, params):
        pass


class DiagCovLinear(DiagCurvature):

    def _diag_data(self, grad_output):
        # W[i][j] = mean_b g[b][i]^2 a[b][j]^2, b[i] = mean_b g[b][i]^2, both * n^2
        # (reference: linear.py:30-45, curvature.py:154-158)
        data_input = getattr(self._module, 'data_input', None)
        assert data_input is not None
        n = data_input.shape[0]
        a = data_input.reshape(n, -1)
        g = grad_output.reshape(n, -1)
        w, b = _ops.diag_cov_linear(g, a, self.bias, float(n))
        return [w] if b is None else [w, b]

    def update_in_backward(self, grad_output):
        self._data = self._diag_data(grad_output)


class KronCovLinear(KronCurvature):

    def update_in_forward(self, input_data):
        # A = [a,1]^T [a,1] / n                       (reference: linear.py:50-59)
        a = input_data.reshape(-1, input_data.shape[-1]) if input_data.dim() != 2 else input_data
        a = a.contiguous()
        n = input_data.shape[0]
        self._build_factor(0, a, 'linear', 1. / n, add_bias=self.bias)

    def update_in_backward(self, grad_output):
        # G = g^T g / n, then * n^2                   (reference: linear.py:61-67,
        #                                              curvature.py:154-155,299-300)
        g = grad_output.reshape(-1, grad_output.shape[-1]) if grad_output.dim() != 2 else grad_output
        g = g.contiguous()
        n = grad_output.shape[0]
        self._build_factor(1, g, 'linear', float(n))

    def _get_shape(self):
        f_out, f_in = self._module.weight.shape
        d_a = f_in + 1 if self.bias else f_in
        return (d_a, d_a), (f_out, f_out)
