"""Curvature of nn.Conv2d.

KronCovConv2d mirrors torchsso/curv/cov/conv.py:45-123 of the reference.  The
A factor is built by the implicit-im2col HIP kernel (patches gathered into LDS,
no unfold tensor in memory), the G factor reads grad_output in place as
[c_out, n*h*w].
"""
from torchsso import _ops
from torchsso.curv.curvature import Curvature, KronCurvature


class CovConv2d(Curvature):
    """Placeholder, as in the reference (cov/conv.py:6-12)."""

    def update_in_backward(self, grad_output):
        pass


class KronCovConv2d(KronCurvature):

    def update_in_forward(self, data_input):
        # A = M M^T / n, M = im2col(x) with a trailing row of ones for the bias;
        # divided by n only                              (reference: conv.py:47-67)
        conv2d = self._module
        n = data_input.shape[0]
        self._A = _ops.factor_conv_a(data_input, conv2d.kernel_size, conv2d.stride,
                                     conv2d.padding, conv2d.dilation, self.bias, 1.0 / n)

    def update_in_backward(self, grad_output):
        # G = m m^T / (n h w), then * n^2                (reference: conv.py:69-74,
        #                                                 curvature.py:154-155,299-300)
        n, c, h, w = grad_output.shape
        self._G = _ops.factor_conv_g(grad_output, float(n) / (h * w))

    def _get_shape(self):
        c_out, c_in, k_h, k_w = self._module.weight.shape
        dim = c_in * k_h * k_w + (1 if self.bias else 0)
        return (dim, dim), (c_out, c_out)
