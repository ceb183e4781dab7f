"""Curvature of nn.Conv2d.

KronCovConv2d mirrors torchsso/curv/cov/conv.py:45-123 of the reference.  The
A factor is built by the implicit-im2col HIP kernel (patches gathered into LDS,
no unfold tensor in memory), the G factor reads grad_output in place as
[c_out, n*h*w].  DiagCovConv2d mirrors cov/conv.py:15-42: the batch mean of the
squared per-sample weight gradients, accumulated tile by tile in registers.
"""
from torchsso import _ops
from torchsso.curv.curvature import Curvature, DiagCurvature, KronCurvature


class CovConv2d(Curvature):
    """Placeholder, as in the reference (cov/conv.py:6-12)."""

    def update_in_backward(self, grad_output):
        pass


class DiagCovConv2d(DiagCurvature):

    def _diag_data(self, grad_output):
        # W = mean_b (g_b M_b^T)^2 reshaped to the weight; bias = mean_b sum_hw g_b^2
        # (the sum of squares, not the square of the sum), both * n^2
        # (reference: conv.py:17-42, curvature.py:154-158)
        conv2d = self._module
        data_input = getattr(conv2d, 'data_input', None)
        assert data_input is not None
        n, c_out, h, w = grad_output.shape
        data_w = _ops.diag_cov_conv2d(grad_output, data_input, conv2d.kernel_size, conv2d.stride,
                                      conv2d.padding, conv2d.dilation, float(n))
        data = [data_w.reshape(c_out, -1, *conv2d.kernel_size)]
        if self.bias:
            sg = _ops.rowsq_sum(grad_output, c_out)                # [n, c_out] sums over h*w
            _, data_b = _ops.bn_diag_combine(sg, sg, float(n), True)
            data.append(data_b)
        return data

    def update_in_backward(self, grad_output):
        self._data = self._diag_data(grad_output)


class KronCovConv2d(KronCurvature):

    def update_in_forward(self, data_input):
        # A = M M^T / n, M = im2col(x) with a trailing row of ones for the bias;
        # divided by n only                              (reference: conv.py:47-67)
        conv2d = self._module
        n = data_input.shape[0]
        data_input = data_input.contiguous()
        self._build_factor(0, data_input, 'conv_a', 1. / n, add_bias=self.bias,
                           kernel_size=conv2d.kernel_size, stride=conv2d.stride,
                           padding=conv2d.padding, dilation=conv2d.dilation)

    def update_in_backward(self, grad_output):
        # G = m m^T / (n h w), then * n^2                (reference: conv.py:69-74,
        #                                                 curvature.py:154-155,299-300)
        n, c, h, w = grad_output.shape
        grad_output = grad_output.contiguous()
        self._build_factor(1, grad_output, 'conv_g', n / (h * w))

    def _get_shape(self):
        c_out, c_in, k_h, k_w = self._module.weight.shape
        dim = c_in * k_h * k_w + (1 if self.bias else 0)
        return (dim, dim), (c_out, c_out)
