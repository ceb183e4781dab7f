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


def _out_square(out, d, like, beta, prev=None):
    if out is None:
        if beta != 0 and prev is None:
            raise _hip.KfacHipError('beta != 0 needs an existing output to accumulate into')
        out = torch.empty((d, d), dtype=torch.float32, device=like.device)
    elif tuple(out.shape) != (d, d):
        raise _hip.KfacHipError('output has shape %s, expected (%d, %d)' % (tuple(out.shape), d, d))
    if prev is not None and tuple(prev.shape) != (d, d):
        raise _hip.KfacHipError('prev has shape %s, expected (%d, %d)' % (tuple(prev.shape), d, d))
    return out


def _prev_ptr(prev):
    return None if prev is None else _hip.dev_ptr(prev, 'previous factor')


def _contiguous_for(x, stream, what):
    """x.contiguous(); with an explicit stream the copy would run on another stream than
    the kernels that read it, so the caller has to bring a contiguous tensor."""
    if stream is not None and not x.is_contiguous():
        raise _hip.KfacHipError('%s must be contiguous when a stream is given' % what)
    return x.contiguous()


def factor_linear(x, add_bias, alpha, out=None, beta=0., prev=None, stream=None):
    """out = alpha * [x,1]^T [x,1] + beta * (prev if given else out) for x of shape [rows, f].
    `stream`: a torch.cuda.Stream to enqueue on instead of the current one (the caller
    orders it after the producers of x / prev and before the readers of out)."""
    lib = _hip.load()
    if x.dim() != 2:
        x = x.reshape(-1, x.shape[-1])
    x = _contiguous_for(x, stream, 'input')
    rows, f = x.shape
    d = f + (1 if add_bias else 0)
    out = _out_square(out, d, x, beta, prev)
    ws, ws_bytes = _hip.workspace(x.device, lib.kfac_factor_workspace_bytes(d, rows), stream)
    st = lib.kfac_factor_linear(_hip.dev_ptr(x, 'input'), rows, f, f, int(bool(add_bias)),
                                float(alpha), float(beta), _prev_ptr(prev),
                                _hip.dev_ptr(out, 'factor'),
                                None if ws is None else ws.data_ptr(), ws_bytes,
                                _hip.stream_ptr(x.device, stream))
    _hip.check(st, 'kfac_factor_linear')
    return out


def factor_conv_a(x, kernel_size, stride, padding, dilation, add_bias, alpha, out=None, beta=0.,
                  prev=None, stream=None):
    """out = alpha * M M^T + beta * (prev if given else out), M = implicit im2col of x [n, c, H, W]."""
    lib = _hip.load()
    if x.dim() != 4:
        raise _hip.KfacHipError('conv input must be [n, c, H, W], got %s' % (tuple(x.shape),))
    x = _contiguous_for(x, stream, 'input')
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
    out = _out_square(out, d, x, beta, prev)
    ws, ws_bytes = _hip.workspace(x.device, lib.kfac_factor_conv_a_workspace_bytes(
        n, c, H, W, kh, kw, sh, sw, ph, pw, dh, dw, int(bool(add_bias))), stream)
    st = lib.kfac_factor_conv_a(_hip.dev_ptr(x, 'input'), n, c, H, W, kh, kw, sh, sw, ph, pw,
                                dh, dw, int(bool(add_bias)), float(alpha), float(beta),
                                _prev_ptr(prev), _hip.dev_ptr(out, 'factor'),
                                None if ws is None else ws.data_ptr(), ws_bytes,
                                _hip.stream_ptr(x.device, stream))
    _hip.check(st, 'kfac_factor_conv_a')
    return out


def factor_conv_g(g, alpha, out=None, beta=0., prev=None, stream=None):
    """out = alpha * m m^T + beta * (prev if given else out), m = g [n, c, h, w] as [c, n*h*w]."""
    lib = _hip.load()
    if g.dim() != 4:
        raise _hip.KfacHipError('conv output gradient must be [n, c, h, w]')
    g = _contiguous_for(g, stream, 'grad_output')
    n, c, h, w = g.shape
    out = _out_square(out, c, g, beta, prev)
    ws, ws_bytes = _hip.workspace(g.device, lib.kfac_factor_workspace_bytes(c, n * h * w), stream)
    st = lib.kfac_factor_conv_g(_hip.dev_ptr(g, 'grad_output'), n, c, h, w, float(alpha),
                                float(beta), _prev_ptr(prev), _hip.dev_ptr(out, 'factor'),
                                None if ws is None else ws.data_ptr(), ws_bytes,
                                _hip.stream_ptr(g.device, stream))
    _hip.check(st, 'kfac_factor_conv_g')
    return out


def factor_job(kind, x, alpha, out, beta=0., prev=None, add_bias=False, kernel_size=1,
               stride=1, padding=0, dilation=1):
    """A `_hip.FactorJob` describing  out = alpha * P^T P + beta * (prev if given else out)
    for kfac_factor_grouped: kind 'linear' (x [rows, f]), 'conv_a' (x [n, c, H, W] and the
    geometry of the convolution) or 'conv_g' (x = grad_output [n, c, h, w]).  The tensors
    must stay alive until factor_grouped has run."""
    job = _hip.FactorJob()
    if kind == 'linear':
        if x.dim() != 2:
            raise _hip.KfacHipError('linear factor input must be [rows, f], got %s' % (tuple(x.shape),))
        rows, c = x.shape
        d = c + (1 if add_bias else 0)
        job.kind, job.H, job.W = _hip.FACTOR_LINEAR, 1, 1
    else:
        if x.dim() != 4:
            raise _hip.KfacHipError('conv factor input must be [n, c, H, W], got %s' % (tuple(x.shape),))
        rows, c, H, W = x.shape
        job.H, job.W = H, W
        if kind == 'conv_a':
            job.kind = _hip.FACTOR_CONV_A
            job.kh, job.kw = _pair(kernel_size)
            job.sh, job.sw = _pair(stride)
            job.ph, job.pw = _pair(padding)
            job.dh, job.dw = _pair(dilation)
            d = c * job.kh * job.kw + (1 if add_bias else 0)
        elif kind == 'conv_g':
            job.kind = _hip.FACTOR_CONV_G
            d = c
        else:
            raise _hip.KfacHipError('unknown factor kind %r' % (kind,))
    if tuple(out.shape) != (d, d) or (prev is not None and tuple(prev.shape) != (d, d)):
        raise _hip.KfacHipError('factor buffers must be (%d, %d)' % (d, d))
    if beta != 0 and prev is None:
        prev = out
    job.add_bias = int(bool(add_bias))
    job.x = _hip.dev_ptr(x, 'input')
    job.rows, job.c = rows, c
    job.alpha, job.beta = float(alpha), float(beta)
    job.C_prev = _prev_ptr(prev)
    job.C = _hip.dev_ptr(out, 'factor')
    return job


def factor_job_update(job, x, alpha, out, beta=0., prev=None):
    """Points an existing job (same kind, shapes and geometry) at new tensors."""
    if beta != 0 and prev is None:
        prev = out
    job.x = _hip.dev_ptr(x, 'input')
    job.alpha, job.beta = float(alpha), float(beta)
    job.C_prev = _prev_ptr(prev)
    job.C = _hip.dev_ptr(out, 'factor')


def conv_output_positions(x, kernel_size=1, stride=1, padding=0, dilation=1):
    """Output positions per image of a convolution over x [n, c, H, W]."""
    kh, kw = _pair(kernel_size)
    sh, sw = _pair(stride)
    ph, pw = _pair(padding)
    dh, dw = _pair(dilation)
    oh = (x.shape[2] + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (x.shape[3] + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    return max(oh, 0) * max(ow, 0)


def factor_grouped(jobs, device, stream=None):
    """Runs a list of `factor_job`s in one engine call (a handful of launches for all of them)."""
    lib = _hip.load()
    if len(jobs) == 0:
        return
    arr = (_hip.FactorJob * len(jobs))(*jobs)
    ws, ws_bytes = _hip.workspace(device, lib.kfac_factor_grouped_workspace_bytes(len(jobs), arr),
                                  stream)
    st = lib.kfac_factor_grouped(len(jobs), arr, _ws_ptr(ws), ws_bytes,
                                 _hip.stream_ptr(device, stream))
    _hip.check(st, 'kfac_factor_grouped')


def factor_grouped_executed_flops(jobs):
    lib = _hip.load()
    if len(jobs) == 0:
        return 0.
    arr = (_hip.FactorJob * len(jobs))(*jobs)
    return lib.kfac_factor_grouped_executed_flops(len(jobs), arr)


def _ws_ptr(ws):
    return None if ws is None else ws.data_ptr()


def _square_dims(mats, what):
    dims = []
    for i, m in enumerate(mats):
        if m.dim() != 2 or m.shape[0] != m.shape[1]:
            raise _hip.KfacHipError('%s %d is not square: %s' % (what, i, tuple(m.shape)))
        dims.append(m.shape[0])
    return dims


def pi_damped_inverse_batched(As, Gs, dampings, A_invs=None, G_invs=None, info=None):
    """A_inv, G_inv = (A + sqrt(d)*pi*I)^-1, (G + sqrt(d)/pi*I)^-1 for every layer.

    Returns (A_invs, G_invs, info) with info a device int32 tensor of 2*layers
    (nothing is synchronised; read it when you want to know)."""
    lib = _hip.load()
    layers = len(As)
    if layers == 0:
        return [], [], None
    dev = As[0].device
    dA = _square_dims(As, 'A')
    dG = _square_dims(Gs, 'G')
    if A_invs is None:
        A_invs = [torch.empty_like(a) for a in As]
    if G_invs is None:
        G_invs = [torch.empty_like(g) for g in Gs]
    if info is None:
        info = torch.empty(2 * layers, dtype=torch.int32, device=dev)
    dims = []
    for a, g in zip(dA, dG):
        dims += [a, g]
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_inverse_workspace_bytes(len(dims), _hip.int_array(dims)))
    st = lib.kfac_pi_damped_inverse_batched(
        layers, _hip.int_array(dA), _hip.int_array(dG), _hip.ptr_array(As, 'A'),
        _hip.ptr_array(Gs, 'G'), _hip.f32_array(dampings), _hip.ptr_array(A_invs, 'A_inv'),
        _hip.ptr_array(G_invs, 'G_inv'), info.data_ptr(), _ws_ptr(ws), ws_bytes,
        _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_pi_damped_inverse_batched')
    return A_invs, G_invs, info


def _pi_inverse_two_outputs(entry, As, Gs, dampings, A_invs, G_invs, A_others, G_others, info,
                            check):
    """Common part of the pi-damped inversions that write up to two results per matrix."""
    lib = _hip.load()
    layers = len(As)
    if layers == 0:
        return None
    dev = As[0].device
    dA = _square_dims(As, 'A')
    dG = _square_dims(Gs, 'G')
    for what, srcs, invs, others in (('A', As, A_invs, A_others), ('G', Gs, G_invs, G_others)):
        for l, (x, i, o) in enumerate(zip(srcs, invs, others)):
            check(l, what, i, o)
            if any(t is not None and t.shape != x.shape for t in (i, o)):
                raise _hip.KfacHipError('layer %d: output buffers of %s have the wrong shape' % (l, what))
    if info is None:
        info = torch.empty(2 * layers, dtype=torch.int32, device=dev)
    dims = []
    for a, g in zip(dA, dG):
        dims += [a, g]
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_inverse_workspace_bytes(len(dims), _hip.int_array(dims)))
    st = getattr(lib, entry)(
        layers, _hip.int_array(dA), _hip.int_array(dG), _hip.ptr_array(As, 'A'),
        _hip.ptr_array(Gs, 'G'), _hip.f32_array(dampings), _hip.ptr_array(A_invs, 'A_inv', True),
        _hip.ptr_array(G_invs, 'G_inv', True), _hip.ptr_array(A_others, 'A output', True),
        _hip.ptr_array(G_others, 'G output', True), info.data_ptr(), _ws_ptr(ws), ws_bytes,
        _hip.stream_ptr(dev))
    _hip.check(st, entry)
    return info


def pi_damped_inverse_std_batched(As, Gs, dampings, A_invs, G_invs, A_stds, G_stds, info=None):
    """pi_damped_inverse_batched that also writes, for the matrices whose A_stds / G_stds entry
    is a tensor (None: no std for it), the upper Cholesky factor of the inverse
    (std^T std = inverse), read off the triangular inverse instead of a second factorisation."""
    def check(l, what, inv, std):
        if inv is None:
            raise _hip.KfacHipError('layer %d: no buffer for the inverse of %s' % (l, what))
    return _pi_inverse_two_outputs('kfac_pi_damped_inverse_std_batched', As, Gs, dampings,
                                   A_invs, G_invs, A_stds, G_stds, info, check)


def pi_damped_inverse_factored_batched(As, Gs, dampings, A_invs, G_invs, A_facs, G_facs, info=None):
    """The pi-damped inverses, each in exactly one of two forms: the matrix itself (a tensor in
    A_invs / G_invs, None in A_facs / G_facs) or only its upper-triangular factor Y with
    Y Y^T = inverse (the other way round), for which the explicit inverse is never formed."""
    def check(l, what, inv, fac):
        if (inv is None) == (fac is None):
            raise _hip.KfacHipError('layer %d: exactly one of inverse and factor must be asked for %s'
                                    % (l, what))
    return _pi_inverse_two_outputs('kfac_pi_damped_inverse_factored_batched', As, Gs, dampings,
                                   A_invs, G_invs, A_facs, G_facs, info, check)


def precondition_factored_batched(G_ops, A_ops, grad_ws, grad_bs, g_factored=None, a_factored=None):
    """[gW | gb] <- G^-1 [gW | gb] A^-1 in place for every layer (gb may be None), with the
    inverses given by their upper-triangular factors (Y Y^T = inverse) where the flag of that
    side is true (no flag list: all of them), and as the explicit matrices elsewhere."""
    lib = _hip.load()
    layers = len(G_ops)
    if layers == 0:
        return
    dev = G_ops[0].device
    _square_dims(G_ops, 'G operand')
    _square_dims(A_ops, 'A operand')
    dG, dA = _kron_dims(G_ops, A_ops, grad_ws, grad_bs, 'precondition')
    dGa, dAa = _hip.int_array(dG), _hip.int_array(dA)
    flags = [None if f is None else _hip.int_array([int(bool(v)) for v in f])
             for f in (g_factored, a_factored)]
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_precondition_factored_workspace_bytes(layers, dGa, dAa))
    st = lib.kfac_precondition_factored_batched(
        layers, dGa, dAa, _hip.ptr_array(G_ops, 'G operand'), _hip.ptr_array(A_ops, 'A operand'),
        flags[0], flags[1], _hip.ptr_array(grad_ws, 'weight grad'),
        _hip.ptr_array(grad_bs, 'bias grad', True), _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_precondition_factored_batched')


def damped_inverse_batched(mats, damps=None, outs=None, info=None):
    """outs[i] = (mats[i] + damps[i]*I)^-1."""
    lib = _hip.load()
    count = len(mats)
    if count == 0:
        return [], None
    dev = mats[0].device
    dims = _square_dims(mats, 'matrix')
    if outs is None:
        outs = [torch.empty_like(m) for m in mats]
    if info is None:
        info = torch.empty(count, dtype=torch.int32, device=dev)
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_inverse_workspace_bytes(count, _hip.int_array(dims)))
    st = lib.kfac_damped_inverse_batched(
        count, _hip.int_array(dims), _hip.ptr_array(mats, 'matrix'),
        None if damps is None else _hip.f32_array(damps), _hip.ptr_array(outs, 'inverse'),
        info.data_ptr(), _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_damped_inverse_batched')
    return outs, info


def cholesky_upper_batched(mats, outs=None, info=None):
    """outs[i] = U upper triangular with mats[i] = U^T U."""
    lib = _hip.load()
    count = len(mats)
    if count == 0:
        return [], None
    dev = mats[0].device
    dims = _square_dims(mats, 'matrix')
    if outs is None:
        outs = [torch.empty_like(m) for m in mats]
    if info is None:
        info = torch.empty(count, dtype=torch.int32, device=dev)
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_inverse_workspace_bytes(count, _hip.int_array(dims)))
    st = lib.kfac_cholesky_upper_batched(
        count, _hip.int_array(dims), _hip.ptr_array(mats, 'matrix'), _hip.ptr_array(outs, 'factor'),
        info.data_ptr(), _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_cholesky_upper_batched')
    return outs, info


def _kron_dims(Ls, Rs, Ws, bs, what):
    dG, dA = [], []
    for l, (L, R, W, b) in enumerate(zip(Ls, Rs, Ws, bs)):
        g, a = L.shape[0], R.shape[0]
        aw = a - (0 if b is None else 1)
        if W.numel() != g * aw or W.shape[0] != g:
            raise _hip.KfacHipError('%s layer %d: weight-shaped tensor %s does not match factors '
                                    '(%d, %d)' % (what, l, tuple(W.shape), g, a))
        if b is not None and b.numel() != g:
            raise _hip.KfacHipError('%s layer %d: bias-shaped tensor has %d elements, expected %d'
                                    % (what, l, b.numel(), g))
        dG.append(g)
        dA.append(a)
    return dG, dA


def precondition_batched(G_invs, A_invs, grad_ws, grad_bs):
    """[gW | gb] <- G_inv [gW | gb] A_inv in place for every layer (gb may be None)."""
    lib = _hip.load()
    layers = len(G_invs)
    if layers == 0:
        return
    dev = G_invs[0].device
    _square_dims(G_invs, 'G_inv')
    _square_dims(A_invs, 'A_inv')
    dG, dA = _kron_dims(G_invs, A_invs, grad_ws, grad_bs, 'precondition')
    dGa, dAa = _hip.int_array(dG), _hip.int_array(dA)
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_precondition_workspace_bytes(layers, dGa, dAa))
    st = lib.kfac_precondition_batched(
        layers, dGa, dAa, _hip.ptr_array(G_invs, 'G_inv'), _hip.ptr_array(A_invs, 'A_inv'),
        _hip.ptr_array(grad_ws, 'weight grad'), _hip.ptr_array(grad_bs, 'bias grad', True),
        _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_precondition_batched')


def sample_batched(U_Gs, U_As, noises, mean_ws, mean_bs, param_ws, param_bs, std_scale):
    """[pW | pb] = [mW | mb] + std_scale * U_G @ noise @ U_A for every layer."""
    lib = _hip.load()
    layers = len(U_Gs)
    if layers == 0:
        return
    dev = U_Gs[0].device
    _square_dims(U_Gs, 'U_G')
    _square_dims(U_As, 'U_A')
    dG, dA = _kron_dims(U_Gs, U_As, param_ws, param_bs, 'sample')
    for l, e in enumerate(noises):
        if tuple(e.shape) != (dG[l], dA[l]):
            raise _hip.KfacHipError('noise %d has shape %s, expected (%d, %d)'
                                    % (l, tuple(e.shape), dG[l], dA[l]))
    dGa, dAa = _hip.int_array(dG), _hip.int_array(dA)
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_precondition_workspace_bytes(layers, dGa, dAa))
    st = lib.kfac_sample_batched(
        layers, dGa, dAa, _hip.ptr_array(U_Gs, 'U_G'), _hip.ptr_array(U_As, 'U_A'),
        _hip.ptr_array(noises, 'noise'), _hip.ptr_array(mean_ws, 'mean weight'),
        _hip.ptr_array(mean_bs, 'mean bias', True), _hip.ptr_array(param_ws, 'weight'),
        _hip.ptr_array(param_bs, 'bias', True), float(std_scale), _ws_ptr(ws), ws_bytes,
        _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_sample_batched')


def _vec_args(lib, tensors):
    dev = tensors[0].device
    numel = _hip.i64_array([t.numel() for t in tensors])
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_vector_workspace_bytes(len(tensors)))
    return dev, numel, ws, ws_bytes


def _check_same_numel(xs, ys, what):
    for i, (x, y) in enumerate(zip(xs, ys)):
        if x.numel() != y.numel():
            raise _hip.KfacHipError('%s %d: %d vs %d elements' % (what, i, x.numel(), y.numel()))


def axpby_batched(xs, ys, a, b):
    """ys[i] = a*xs[i] + b*ys[i] in place."""
    lib = _hip.load()
    if len(xs) == 0:
        return
    _check_same_numel(xs, ys, 'axpby')
    dev, numel, ws, ws_bytes = _vec_args(lib, xs)
    st = lib.kfac_axpby_batched(len(xs), numel, _hip.ptr_array(xs, 'x'), _hip.ptr_array(ys, 'y'),
                                float(a), float(b), _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_axpby_batched')


def diag_inverse_batched(emas, invs, dampings, use_sqrt):
    lib = _hip.load()
    if len(emas) == 0:
        return
    _check_same_numel(emas, invs, 'diag inverse')
    dev, numel, ws, ws_bytes = _vec_args(lib, emas)
    st = lib.kfac_diag_inverse_batched(len(emas), numel, _hip.ptr_array(emas, 'ema'),
                                       _hip.ptr_array(invs, 'inv'), _hip.f32_array(dampings),
                                       int(bool(use_sqrt)), _ws_ptr(ws), ws_bytes,
                                       _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_diag_inverse_batched')


def diag_precondition_batched(invs, grads):
    lib = _hip.load()
    if len(invs) == 0:
        return
    _check_same_numel(invs, grads, 'diag precondition')
    dev, numel, ws, ws_bytes = _vec_args(lib, invs)
    st = lib.kfac_diag_precondition_batched(len(invs), numel, _hip.ptr_array(invs, 'inv'),
                                            _hip.ptr_array(grads, 'grad'), _ws_ptr(ws), ws_bytes,
                                            _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_diag_precondition_batched')


def sqrt_batched(xs, ys):
    """ys[i] = sqrt(xs[i])."""
    lib = _hip.load()
    if len(xs) == 0:
        return
    _check_same_numel(xs, ys, 'sqrt')
    dev, numel, ws, ws_bytes = _vec_args(lib, xs)
    st = lib.kfac_sqrt_batched(len(xs), numel, _hip.ptr_array(xs, 'x'), _hip.ptr_array(ys, 'y'),
                               _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_sqrt_batched')


def max_batched(xs, ys):
    """ys[i] = max(xs[i], ys[i]) in place."""
    lib = _hip.load()
    if len(xs) == 0:
        return
    _check_same_numel(xs, ys, 'max')
    dev, numel, ws, ws_bytes = _vec_args(lib, xs)
    st = lib.kfac_max_batched(len(xs), numel, _hip.ptr_array(xs, 'x'), _hip.ptr_array(ys, 'y'),
                              _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_max_batched')


def diag_sample_batched(means, stds, noise_to_params, std_scales):
    """noise_to_params[i] = means[i] + std_scales[i] * noise_to_params[i] * stds[i] in place."""
    lib = _hip.load()
    if len(means) == 0:
        return
    _check_same_numel(means, stds, 'diag sample (std)')
    _check_same_numel(means, noise_to_params, 'diag sample (param)')
    dev, numel, ws, ws_bytes = _vec_args(lib, means)
    st = lib.kfac_diag_sample_batched(len(means), numel, _hip.ptr_array(means, 'mean'),
                                      _hip.ptr_array(stds, 'std'),
                                      _hip.ptr_array(noise_to_params, 'param'),
                                      _hip.f32_array(std_scales), _ws_ptr(ws), ws_bytes,
                                      _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_diag_sample_batched')


def diag_cov_linear(g, a, add_bias, alpha):
    """(W, b): W[i][j] = alpha * sum_k g[k,i]^2 a[k,j]^2 ; b[i] = alpha * sum_k g[k,i]^2 (or None)."""
    lib = _hip.load()
    if g.dim() != 2 or a.dim() != 2 or g.shape[0] != a.shape[0]:
        raise _hip.KfacHipError('diag_cov_linear: g %s vs a %s' % (tuple(g.shape), tuple(a.shape)))
    g, a = g.contiguous(), a.contiguous()
    n, fout = g.shape
    fin = a.shape[1]
    W = torch.empty((fout, fin), dtype=torch.float32, device=g.device)
    b = torch.empty(fout, dtype=torch.float32, device=g.device) if add_bias else None
    st = lib.kfac_diag_cov_linear(_hip.dev_ptr(g, 'output gradient'), _hip.dev_ptr(a, 'input'), n,
                                  fout, fin, int(bool(add_bias)), float(alpha), W.data_ptr(),
                                  None if b is None else b.data_ptr(), _hip.stream_ptr(g.device))
    _hip.check(st, 'kfac_diag_cov_linear')
    return W, b


def diag_cov_conv2d(g, x, kernel_size, stride, padding, dilation, alpha):
    """[cout, c*kh*kw] tensor alpha * sum_b (g_b M_b^T)^2 of squared per-sample weight gradients."""
    lib = _hip.load()
    if g.dim() != 4 or x.dim() != 4 or g.shape[0] != x.shape[0]:
        raise _hip.KfacHipError('diag_cov_conv2d: g %s vs x %s' % (tuple(g.shape), tuple(x.shape)))
    g, x = g.contiguous(), x.contiguous()
    n, c, H, W = x.shape
    cout = g.shape[1]
    kh, kw = _pair(kernel_size)
    sh, sw = _pair(stride)
    ph, pw = _pair(padding)
    dh, dw = _pair(dilation)
    oh = (H + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (W + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    if (oh, ow) != tuple(g.shape[2:]):
        raise _hip.KfacHipError('diag_cov_conv2d: output gradient is %s, geometry gives %s'
                                % (tuple(g.shape[2:]), (oh, ow)))
    out = torch.empty((cout, c * kh * kw), dtype=torch.float32, device=g.device)
    ws, ws_bytes = _hip.workspace(g.device,
                                  lib.kfac_diag_cov_conv2d_workspace_bytes(n, cout, c, kh, kw))
    st = lib.kfac_diag_cov_conv2d(_hip.dev_ptr(g, 'output gradient'), _hip.dev_ptr(x, 'input'), n,
                                  cout, c, H, W, kh, kw, sh, sw, ph, pw, dh, dw, float(alpha),
                                  out.data_ptr(), _ws_ptr(ws), ws_bytes, _hip.stream_ptr(g.device))
    _hip.check(st, 'kfac_diag_cov_conv2d')
    return out


def sgd_update_batched(params, grads, bufs, lrs, momenta, weight_decays):
    """g += wd*p; buf = m*buf + g, g = buf (if m); p -= lr*g  for every tensor."""
    lib = _hip.load()
    if len(params) == 0:
        return
    _check_same_numel(params, grads, 'update')
    for i, (p, buf, m) in enumerate(zip(params, bufs, momenta)):
        if m != 0 and (buf is None or buf.numel() != p.numel()):
            raise _hip.KfacHipError('update %d: momentum buffer missing or of wrong size' % i)
    dev, numel, ws, ws_bytes = _vec_args(lib, params)
    st = lib.kfac_sgd_update_batched(
        len(params), numel, _hip.ptr_array(params, 'param'), _hip.ptr_array(grads, 'grad'),
        _hip.ptr_array(bufs, 'momentum buffer', True), _hip.f32_array(lrs),
        _hip.f32_array(momenta), _hip.f32_array(weight_decays), _ws_ptr(ws), ws_bytes,
        _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_sgd_update_batched')


def rowsq_sum(x, channels, scale=None, shift=None):
    """[n, c] tensor of sum over the trailing dims of ((x - shift[c]) / scale[c])^2."""
    lib = _hip.load()
    x = x.contiguous()
    n = x.shape[0]
    if x.shape[1] != channels:
        raise _hip.KfacHipError('expected %d channels, got %s' % (channels, tuple(x.shape)))
    length = x.numel() // (n * channels)
    out = torch.empty((n, channels), dtype=torch.float32, device=x.device)
    st = lib.kfac_rowsq_sum(_hip.dev_ptr(x, 'input'), n * channels, channels, length,
                            None if scale is None else _hip.dev_ptr(scale, 'scale'),
                            None if shift is None else _hip.dev_ptr(shift, 'shift'),
                            out.data_ptr(), _hip.stream_ptr(x.device))
    _hip.check(st, 'kfac_rowsq_sum')
    return out


def bn_diag_combine(sx, sg, alpha, bias):
    lib = _hip.load()
    n, c = sx.shape
    if tuple(sg.shape) != (n, c):
        raise _hip.KfacHipError('bn_diag_combine: %s vs %s' % (tuple(sx.shape), tuple(sg.shape)))
    w = torch.empty(c, dtype=torch.float32, device=sx.device)
    b = torch.empty(c, dtype=torch.float32, device=sx.device) if bias else None
    st = lib.kfac_bn_diag_combine(_hip.dev_ptr(sx, 'sx'), _hip.dev_ptr(sg, 'sg'), n, c,
                                  float(alpha), w.data_ptr(), None if b is None else b.data_ptr(),
                                  _hip.stream_ptr(sx.device))
    _hip.check(st, 'kfac_bn_diag_combine')
    return w, b


def bn_diag_cov(grad_output, channels, sx, alpha, bias):
    """(w_curv, b_curv) of a BatchNorm layer from the output gradient and the forward
    hook's [n, c] sums sx: alpha * sum_n sx * sum_hw g^2 and alpha * sum_n sum_hw g^2."""
    lib = _hip.load()
    g = grad_output.contiguous()
    n = g.shape[0]
    if g.shape[1] != channels or tuple(sx.shape) != (n, channels):
        raise _hip.KfacHipError('bn_diag_cov: grad_output %s, sums %s, %d channels'
                                % (tuple(g.shape), tuple(sx.shape), channels))
    length = g.numel() // (n * channels)
    w = torch.empty(channels, dtype=torch.float32, device=g.device)
    b = torch.empty(channels, dtype=torch.float32, device=g.device) if bias else None
    # the row sums of long rows pass through memory
    ws = (torch.empty((n, channels), dtype=torch.float32, device=g.device)
          if length > 256 or n > 2048 else None)
    st = lib.kfac_bn_diag_cov(_hip.dev_ptr(g, 'grad_output'), n, channels, length,
                              _hip.dev_ptr(sx, 'sx'), float(alpha), w.data_ptr(),
                              None if b is None else b.data_ptr(),
                              None if ws is None else ws.data_ptr(),
                              0 if ws is None else ws.numel() * 4, _hip.stream_ptr(g.device))
    _hip.check(st, 'kfac_bn_diag_cov')
    return w, b


BN_BATCH_MAX_ROWS = 2048     # samples per layer the batched BatchNorm call takes


def bn_diag_cov_batched(jobs, device, stream=None):
    """bn_diag_cov for a list of layers in one launch.  jobs: (grad_output, channels, sx,
    alpha, w, b) with grad_output contiguous [n, c, ...], sx [n, c], and w, b (b may be
    None) the [c] outputs, written in place."""
    if not jobs:
        return
    lib = _hip.load()
    gs, ns, cs, ls, sxs, alphas, ws_, bs = [], [], [], [], [], [], [], []
    for g, channels, sx, alpha, w, b in jobs:
        n = g.shape[0]
        if g.shape[1] != channels or tuple(sx.shape) != (n, channels) or n > BN_BATCH_MAX_ROWS:
            raise _hip.KfacHipError('bn_diag_cov_batched: grad_output %s, sums %s, %d channels'
                                    % (tuple(g.shape), tuple(sx.shape), channels))
        gs.append(g)
        ns.append(n)
        cs.append(channels)
        ls.append(g.numel() // (n * channels))
        sxs.append(sx)
        alphas.append(alpha)
        ws_.append(w)
        bs.append(b)
    count = len(jobs)
    ws, ws_bytes = _hip.workspace(device, lib.kfac_bn_diag_cov_batched_workspace_bytes(count), stream)
    st = lib.kfac_bn_diag_cov_batched(
        count, _hip.ptr_array(gs, 'grad_output'), _hip.int_array(ns), _hip.int_array(cs),
        _hip.int_array(ls), _hip.ptr_array(sxs, 'sx'), _hip.f32_array(alphas),
        _hip.ptr_array(ws_, 'w_curv'), _hip.ptr_array(bs, 'b_curv', allow_none=True),
        _ws_ptr(ws), ws_bytes, _hip.stream_ptr(device, stream))
    _hip.check(st, 'kfac_bn_diag_cov_batched')


def scale_rows(x, w, use_sqrt):
    """x[r] * (sqrt(w[r]) if use_sqrt else w[r]) for every row r = index along dim 0 (new tensor)."""
    lib = _hip.load()
    x = x.contiguous()
    rows = x.shape[0]
    if w.numel() != rows:
        raise _hip.KfacHipError('scale_rows: %d weights for %d rows' % (w.numel(), rows))
    out = torch.empty_like(x)
    st = lib.kfac_scale_rows(_hip.dev_ptr(x, 'input'), _hip.dev_ptr(w.contiguous(), 'weights'), rows,
                             x.numel() // rows, int(bool(use_sqrt)), out.data_ptr(),
                             _hip.stream_ptr(x.device))
    _hip.check(st, 'kfac_scale_rows')
    return out


def _pack_lists(arrays):
    """arrays: list of (tensor, triangular).  Returns tensors, numel, dims, flags."""
    tensors, numel, dims, flags = [], [], [], []
    for i, (t, tri) in enumerate(arrays):
        if tri and (t.dim() != 2 or t.shape[0] != t.shape[1]):
            raise RuntimeError('non square matrix')
        if not t.is_contiguous():
            raise _hip.KfacHipError('pack/unpack: array %d is not contiguous' % i)
        tensors.append(t)
        numel.append(t.numel())
        dims.append(t.shape[0] if tri else 0)
        flags.append(1 if tri else 0)
    return tensors, numel, dims, flags


def packed_numel(arrays):
    """Length in elements of the packed form of a list of (tensor, triangular)."""
    return sum(t.shape[0] * (t.shape[0] + 1) // 2 if tri else t.numel() for t, tri in arrays)


def pack_batched(arrays, buf, offset=0):
    """Packs a list of (tensor, triangular) into the flat buffer `buf` from element
    `offset` on; returns the offset behind the last array."""
    return _pack_call(arrays, buf, offset, False)


def unpack_batched(arrays, buf, offset=0):
    """Inverse of pack_batched: fills the tensors (both triangles of a symmetric one)."""
    return _pack_call(arrays, buf, offset, True)


def _pack_call(arrays, buf, offset, unpack):
    lib = _hip.load()
    if len(arrays) == 0:
        return offset
    tensors, numel, dims, flags = _pack_lists(arrays)
    total = packed_numel(arrays)
    if buf.dim() != 1 or not buf.is_contiguous() or offset < 0 or offset + total > buf.numel():
        raise _hip.KfacHipError('pack/unpack: buffer of %d elements cannot hold %d from offset %d'
                                % (buf.numel(), total, offset))
    dev = buf.device
    ws, ws_bytes = _hip.workspace(dev, lib.kfac_pack_workspace_bytes(len(tensors)))
    fn = lib.kfac_unpack_batched if unpack else lib.kfac_pack_batched
    st = fn(len(tensors), _hip.ptr_array(tensors, 'array'), _hip.i64_array(numel),
            _hip.int_array(dims), _hip.int_array(flags), _hip.dev_ptr(buf, 'buffer'), int(offset),
            _ws_ptr(ws), ws_bytes, _hip.stream_ptr(dev))
    _hip.check(st, 'kfac_unpack_batched' if unpack else 'kfac_pack_batched')
    return offset + total
