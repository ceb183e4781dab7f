"""Tensor-level wrappers over the C ABI (one function per entry point).

Each wrapper checks shapes on the host before anything is launched, brings the
scratch the entry point asks for, and enqueues on torch's current stream.
"""
import torch

from torchsso import _hip


def _pair(v):
    if isinstance(v, (tuple, list)):
        return int(v[0]), int(v[1])
    return int(v), int(v)


def _out_square(out, d, like, beta):
    if out is None:
        if beta != 0:
            raise _hip.KfacHipError('beta != 0 needs an existing output to accumulate into')
        out = torch.empty((d, d), dtype=torch.float32, device=like.device)
    elif tuple(out.shape) != (d, d):
        raise _hip.KfacHipError('output has shape %s, expected (%d, %d)' % (tuple(out.shape), d, d))
    return out


def factor_linear(x, add_bias, alpha, out=None, beta=0.):
    """out = alpha * [x,1]^T [x,1] + beta * out for x of shape [rows, f]."""
    lib = _hip.load()
    if x.dim() != 2:
        x = x.reshape(-1, x.shape[-1])
    x = x.contiguous()
    rows, f = x.shape
    d = f + (1 if add_bias else 0)
    out = _out_square(out, d, x, beta)
    ws, ws_bytes = _hip.workspace(x.device, lib.kfac_factor_workspace_bytes(d, rows))
    st = lib.kfac_factor_linear(_hip.dev_ptr(x, 'input'), rows, f, f, int(bool(add_bias)),
                                float(alpha), float(beta), _hip.dev_ptr(out, 'factor'),
                                None if ws is None else ws.data_ptr(), ws_bytes,
                                _hip.stream_ptr(x.device))
    _hip.check(st, 'kfac_factor_linear')
    return out


def factor_conv_a(x, kernel_size, stride, padding, dilation, add_bias, alpha, out=None, beta=0.):
    """out = alpha * M M^T + beta * out, M = implicit im2col of x [n, c, H, W]."""
    lib = _hip.load()
    if x.dim() != 4:
        raise _hip.KfacHipError('conv input must be [n, c, H, W], got %s' % (tuple(x.shape),))
    x = x.contiguous()
    n, c, H, W = x.shape
    kh, kw = _pair(kernel_size)
    sh, sw = _pair(stride)
    ph, pw = _pair(padding)
    dh, dw = _pair(dilation)
    oh = (H + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (W + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    if oh <= 0 or ow <= 0:
        raise _hip.KfacHipError('conv geometry gives an empty output')
    d = c * kh * kw + (1 if add_bias else 0)
    out = _out_square(out, d, x, beta)
    ws, ws_bytes = _hip.workspace(x.device, lib.kfac_factor_workspace_bytes(d, n * oh * ow))
    st = lib.kfac_factor_conv_a(_hip.dev_ptr(x, 'input'), n, c, H, W, kh, kw, sh, sw, ph, pw,
                                dh, dw, int(bool(add_bias)), float(alpha), float(beta),
                                _hip.dev_ptr(out, 'factor'),
                                None if ws is None else ws.data_ptr(), ws_bytes,
                                _hip.stream_ptr(x.device))
    _hip.check(st, 'kfac_factor_conv_a')
    return out


def factor_conv_g(g, alpha, out=None, beta=0.):
    """out = alpha * m m^T + beta * out, m = g [n, c, h, w] viewed as [c, n*h*w]."""
    lib = _hip.load()
    if g.dim() != 4:
        raise _hip.KfacHipError('conv output gradient must be [n, c, h, w]')
    g = g.contiguous()
    n, c, h, w = g.shape
    out = _out_square(out, c, g, beta)
    ws, ws_bytes = _hip.workspace(g.device, lib.kfac_factor_workspace_bytes(c, n * h * w))
    st = lib.kfac_factor_conv_g(_hip.dev_ptr(g, 'grad_output'), n, c, h, w, float(alpha),
                                float(beta), _hip.dev_ptr(out, 'factor'),
                                None if ws is None else ws.data_ptr(), ws_bytes,
                                _hip.stream_ptr(g.device))
    _hip.check(st, 'kfac_factor_conv_g')
    return out
