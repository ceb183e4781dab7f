"""CPU oracle for the K-FAC hot path of cybertronai/pytorch-sso.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module; it is the checker that tests, the smoke run and the CPU-baseline leg of
the benchmark compare the HIP kernels against.

Every function restates, from the mathematics, what one reference function
computes on CPU tensors, and cites the reference file:line it follows.  The
arithmetic type is selectable: ``dtype=torch.float32`` follows the reference's
CPU path operation by operation (torch CPU einsum / unfold / mm and SciPy's
LU-based ``linalg.inv``), ``dtype=torch.float64`` is the high-precision truth
that both the fp32 oracle and the GPU results are compared with.

Pinning (what each function is checked against in tests/test_oracle.py, none of
which retypes the formula):
  factor_linear_*      brute-force loops, A[-1,-1]==1, A[-1,:-1]==mean(a)
  factor_conv_a        7-nested-loop patch extraction, 1x1-conv == linear case,
                       autograd weight.grad identity (row order c,kh,kw)
  factor_conv_g        autograd identity, linear special case
  ema / accumulate     hand-computed two-step recursion, beta==1 copy
  pi_damped_inverse    scalar-identity special case, residual X·X^-1 == I,
                       2x2 by hand
  precondition         Kronecker identity via torch.kron
  bn_diag              per-sample gradient identity through autograd
  diag_cov_linear/conv per-sample gradients taken one sample at a time through autograd
                       (the bias entry of diag_cov_conv2d, a sum of squares where the
                       per-sample gradient would give the square of a sum, is pinned
                       by brute-force loops instead)
  fisher_*             prob == 1 reduces to the Cov factor; the exact sum over classes at the
                       logits layer equals mean_n(diag(p_n) - p_n p_n^T) (closed form);
                       fisher_conv_g and fisher_bn_diag by explicit per-sample loops with
                       prob != 1 on a 2x3x2x2 input, the h = w = 1 reduction to the linear
                       case and linearity in prob
  cholesky_upper       U^T U == X, U upper, diag > 0
  sample               injected-noise Kronecker identity
  tri_pack / unpack    the reference's own index formula evaluated by loops
                       (utils/chainer_communicators/_utility.py:19-31), round trip
  kfac_step / vi_step  golden vectors written by the reference itself
                       (tests/golden/*.npz) and torch.optim.SGD equivalence
The reference ships no golden vectors or known-answer tests for this path.
"""
import math

import numpy as np
import scipy.linalg
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# factors
# --------------------------------------------------------------------------

def factor_linear_a(a, bias=True, dtype=torch.float32):
    """A = [a,1]^T [a,1] / n   (torchsso/curv/cov/linear.py:50-59).

    a: [n, f_in].  The ones column is the LAST column (linear.py:52-55)."""
    a = a.to(dtype)
    n = a.shape[0]
    if bias:
        a = torch.cat((a, a.new_ones((n, 1))), 1)
    return (a.t() @ a) / n


def factor_linear_g(g, dtype=torch.float32, scale_by_batch=True):
    """G = g^T g / n, then *= n^2   (torchsso/curv/cov/linear.py:61-67 followed by
    torchsso/curv/curvature.py:154-155,299-300)."""
    g = g.to(dtype)
    n = g.shape[0]
    G = (g.t() @ g) / n
    if scale_by_batch:
        G = G * float(n ** 2)
    return G


def factor_conv_a(x, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
                  bias=True, dtype=torch.float32):
    """A = M M^T / n with M = unfold(x) as [c_in*kh*kw (+1), n*h_out*w_out]
    (torchsso/curv/cov/conv.py:47-67).  Divides by n only (conv.py:66); the ones
    ROW is last (conv.py:60-62); row order is (c_in, kh, kw) as F.unfold."""
    x = x.to(dtype)
    n = x.shape[0]
    u = F.unfold(x, kernel_size=kernel_size, stride=stride, padding=padding,
                 dilation=dilation)                       # n x a x L'
    m = u.transpose(0, 1).reshape(u.shape[1], -1)         # a x (n L')
    if bias:
        m = torch.cat((m, m.new_ones((1, m.shape[1]))), 0)
    return (m @ m.t()) / n


def factor_conv_g(g, dtype=torch.float32, scale_by_batch=True):
    """G = m m^T / (n h w), m = grad_out as [c_out, n*h*w], then *= n^2
    (torchsso/curv/cov/conv.py:69-74; curvature.py:154-155,299-300)."""
    g = g.to(dtype)
    n, c, h, w = g.shape
    m = g.transpose(0, 1).reshape(c, -1)
    G = (m @ m.t()) / (n * h * w)
    if scale_by_batch:
        G = G * float(n ** 2)
    return G


def bn_diag(xhat, g, bias=True, dtype=torch.float32, scale_by_batch=True):
    """Diagonal curvature of BatchNorm (torchsso/curv/cov/batchnorm.py:12-25 for
    [n,f], :36-49 for [n,c,h,w]); every data tensor is then multiplied by n^2
    (curvature.py:154-158)."""
    xhat = xhat.to(dtype)
    g = g.to(dtype)
    n = g.shape[0]
    if g.dim() == 4:
        in_in = (xhat * xhat).sum(dim=(2, 3))
        gg = (g * g).sum(dim=(2, 3))
    else:
        in_in = xhat * xhat
        gg = g * g
    out = [(in_in * gg).mean(dim=0)]
    if bias:
        out.append(gg.mean(dim=0))
    if scale_by_batch:
        out = [o * float(n ** 2) for o in out]
    return out


def diag_cov_linear(a, g, bias=True, prob=None, dtype=torch.float32, scale_by_batch=True):
    """Diagonal covariance of a Linear layer: W = (g^2)^T (a^2) / n, b = mean_n g^2
    (torchsso/curv/cov/linear.py:28-45), times n^2 (curvature.py:154-158).  With
    `prob`, one weighted pass of DiagFisherLinear: g^2 is replaced by prob * g^2
    (fisher/linear.py:11-33)."""
    a, g = a.to(dtype), g.to(dtype)
    n = a.shape[0]
    gg = g * g
    if prob is not None:
        gg = gg * prob.to(dtype).reshape(n, 1)
    out = [(gg.t() @ (a * a)) / n]
    if bias:
        out.append(gg.mean(dim=0))
    return [o * float(n ** 2) for o in out] if scale_by_batch else out


def diag_cov_conv2d(x, g, kernel_size, stride=(1, 1), padding=(0, 0), dilation=(1, 1), bias=True,
                    prob=None, dtype=torch.float32, scale_by_batch=True):
    """Diagonal covariance of a Conv2d layer: the batch mean of the squared
    per-sample weight gradients g_b M_b^T (M_b = unfold of sample b), shaped like
    the weight; the bias entry is mean_n sum_hw g^2 -- the sum of the squares,
    as the reference computes it (torchsso/curv/cov/conv.py:15-42), times n^2
    (curvature.py:154-158).  With `prob`, one weighted pass of DiagFisherConv2d
    (fisher/conv.py:12-45)."""
    x, g = x.to(dtype), g.to(dtype)
    n, c_out, h, w = g.shape
    kh, kw = kernel_size
    m = F.unfold(x, kernel_size=kernel_size, stride=stride, padding=padding, dilation=dilation)
    g2d = g.reshape(n, c_out, -1)
    grad_in = torch.bmm(g2d, m.transpose(1, 2))                    # n x c_out x (c kh kw)
    sq = grad_in * grad_in
    gg = (g2d * g2d).sum(dim=2)                                    # n x c_out
    if prob is not None:
        sq = sq * prob.to(dtype).reshape(n, 1, 1)
        gg = gg * prob.to(dtype).reshape(n, 1)
    out = [sq.mean(dim=0).reshape(c_out, -1, kh, kw)]
    if bias:
        out.append(gg.mean(dim=0))
    return [o * float(n ** 2) for o in out] if scale_by_batch else out


def fisher_linear_g(g, prob, dtype=torch.float32, scale_by_batch=True):
    """One weighted pass of KronFisherLinear: G = (prob * g)^T g / n, then *= n^2
    (torchsso/curv/fisher/linear.py:47-54; curvature.py:154-155).  The passes of one
    step are summed (Fisher.accumulate_cov, fisher/__init__.py:24-28)."""
    g = g.to(dtype)
    n = g.shape[0]
    G = ((g * prob.to(dtype).reshape(n, 1)).t() @ g) / n
    return G * float(n ** 2) if scale_by_batch else G


def fisher_conv_g(g, prob, dtype=torch.float32, scale_by_batch=True):
    """One weighted pass of KronFisherConv2d (torchsso/curv/fisher/conv.py:61-70)."""
    g = g.to(dtype)
    n, c, h, w = g.shape
    pm = (g * prob.to(dtype).reshape(n, 1, 1, 1)).transpose(0, 1).reshape(c, -1)
    m = g.transpose(0, 1).reshape(c, -1)
    G = (pm @ m.t()) / (n * h * w)
    return G * float(n ** 2) if scale_by_batch else G


def fisher_bn_diag(xhat, g, prob, bias=True, dtype=torch.float32, scale_by_batch=True):
    """One weighted pass of DiagFisherBatchNorm2d (torchsso/curv/fisher/batchnorm.py:11-30)."""
    xhat, g = xhat.to(dtype), g.to(dtype)
    n = g.shape[0]
    gg = (g * prob.to(dtype).reshape(n, 1, 1, 1) * g).sum(dim=(2, 3))
    in_in = (xhat * xhat).sum(dim=(2, 3))
    out = [(in_in * gg).mean(dim=0)]
    if bias:
        out.append(gg.mean(dim=0))
    return [o * float(n ** 2) for o in out] if scale_by_batch else out


def bn_restore_input(out, weight, bias):
    """x_hat = (out - bias) / weight   (torchsso/curv/curvature.py:123-134)."""
    shape = (1, -1) + (1,) * (out.dim() - 2)
    return (out - bias.view(shape)) / weight.view(shape)


# --------------------------------------------------------------------------
# accumulate / EMA
# --------------------------------------------------------------------------

def accumulate(acc, data, scale):
    """acc = scale*data on first use else acc + scale*data
    (torchsso/utils/accumulator.py:23-38)."""
    if acc is None:
        return [d * scale for d in data]
    return [a + scale * d for a, d in zip(acc, data)]


def ema_update(data, ema, beta):
    """First call or beta == 1: copy.  Else ema = beta*data + (1-beta)*ema_old;
    ``beta`` weighs the NEW data (torchsso/curv/curvature.py:174-187)."""
    if ema is None or beta == 1:
        return [d.clone() for d in data]
    return [d * beta + (1 - beta) * e for d, e in zip(data, ema)]


def l2_reg_ema_update(l2_reg, l2_reg_ema, beta, first):
    """Scalar recursion next to the factor EMA (curvature.py:183,187)."""
    if first or beta == 1:
        return l2_reg
    return l2_reg * beta + l2_reg_ema * (1 - beta)


# --------------------------------------------------------------------------
# inverse
# --------------------------------------------------------------------------

def _inv(m):
    """torchsso.utils.inv on CPU = scipy.linalg.inv, general LU
    (torchsso/utils/inv_cupy.py:32-34).  fp64 input gives the truth."""
    return torch.from_numpy(scipy.linalg.inv(m.numpy()))


def pi_and_damping(A, G, damping):
    """pi = sqrt((trA/dA)/(trG/dG)); r = sqrt(damping); shifts r*pi and r/pi
    (torchsso/curv/curvature.py:302-312)."""
    pi = math.sqrt((A.trace().item() / A.shape[0]) / (G.trace().item() / G.shape[0]))
    r = damping ** 0.5
    return pi, r * pi, r / pi


def pi_damped_inverse(A, G, damping, dtype=torch.float32):
    """A^-1 = (A + r*pi*I)^-1, G^-1 = (G + r/pi*I)^-1
    (curvature.py:302-312, add_value_to_diagonal :334-340, inv_cupy.py:27-34)."""
    A = A.to(dtype)
    G = G.to(dtype)
    _, da, dg = pi_and_damping(A, G, damping)
    Ad = A + torch.eye(A.shape[0], dtype=dtype) * da
    Gd = G + torch.eye(G.shape[0], dtype=dtype) * dg
    return _inv(Ad), _inv(Gd)


def damped_inverse(X, value, dtype=torch.float32):
    """(X + value*I)^-1 for one matrix (Curvature._inv, curvature.py:197-200)."""
    X = X.to(dtype)
    return _inv(X + torch.eye(X.shape[0], dtype=dtype) * value)


def diag_inverse(X, damping, use_sqrt_ema=False):
    """DiagCurvature._inv: 1 / (X(+sqrt) + damping)  (curvature.py:226-232)."""
    if use_sqrt_ema:
        X = X.sqrt()
    return 1 / (X + damping)


def cholesky_upper(X, dtype=torch.float32):
    """torchsso.utils.cholesky(X, upper=True): U = (lower Cholesky factor)^T so
    X = U^T U  (torchsso/utils/cholesky_cupy.py:9-14).  The reference has no CPU
    implementation (cupy only); torch.linalg.cholesky is the library stand-in."""
    return torch.linalg.cholesky(X.to(dtype)).mT.contiguous()


# --------------------------------------------------------------------------
# precondition / sampling
# --------------------------------------------------------------------------

def precondition(G_inv, A_inv, grad_w, grad_b=None, dtype=torch.float32):
    """U = G^-1 [dW | db] A^-1, split back into dW (same shape as given) and db
    (torchsso/curv/cov/linear.py:69-84, cov/conv.py:76-92)."""
    oc = grad_w.shape[0]
    g2 = grad_w.reshape(oc, -1).to(dtype)
    if grad_b is not None:
        g2 = torch.cat((g2, grad_b.to(dtype).view(-1, 1)), 1)
    u = G_inv.to(dtype) @ g2 @ A_inv.to(dtype)
    if grad_b is not None:
        return u[:, :-1].reshape(grad_w.shape), u[:, -1].clone()
    return u.reshape(grad_w.shape), None


def sample(mean_w, mean_b, U_G, U_A, noise, std_scale, dtype=torch.float32):
    """P = [mean_W | mean_b] + std_scale * U_G @ noise @ U_A with U = upper
    Cholesky factors of the inverses; ``noise`` is what randn_like(m) returned
    (torchsso/curv/cov/linear.py:86-100, cov/conv.py:94-108)."""
    oc = mean_w.shape[0]
    m = mean_w.reshape(oc, -1).to(dtype)
    if mean_b is not None:
        m = torch.cat((m, mean_b.to(dtype).view(-1, 1)), 1)
    p = m + std_scale * (U_G.to(dtype) @ noise.to(dtype) @ U_A.to(dtype))
    if mean_b is not None:
        return p[:, :-1].reshape(mean_w.shape), p[:, -1].clone()
    return p.reshape(mean_w.shape), None


# --------------------------------------------------------------------------
# straight-line optimizer steps (host sequencing)
# --------------------------------------------------------------------------

class LayerState(object):
    """EMA / inverse / momentum state of one layer as Curvature and the
    optimizer keep it (curvature.py:37-48, secondorder.py:138-142)."""

    def __init__(self, kind, bias):
        self.kind = kind          # 'kron' or 'diag'
        self.bias = bias
        self.ema = None
        self.inv = None
        self.std = None
        self.l2_reg = 0.
        self.l2_reg_ema = 0.
        self.momentum = None      # one buffer per parameter


def curvature_step(state, data, damping, ema_decay, dtype=torch.float32, update_std=False):
    """Curvature.step: EMA of the data and of l2_reg, then the inverse with
    damping + l2_reg_ema -- pi-split for a Kron layer, element-wise for a
    diagonal one -- then optionally std (curvature.py:166-191,226-232,302-321)."""
    first = state.ema is None
    state.ema = ema_update([d.to(dtype) for d in data], state.ema, ema_decay)
    state.l2_reg_ema = l2_reg_ema_update(state.l2_reg, state.l2_reg_ema, ema_decay, first)
    damp = damping + state.l2_reg_ema
    if state.kind == 'kron':
        state.inv = list(pi_damped_inverse(state.ema[0], state.ema[1], damp, dtype))
        if update_std:
            state.std = [cholesky_upper(X, dtype) for X in state.inv]
    else:
        state.inv = [diag_inverse(e, damp) for e in state.ema]
        if update_std:
            state.std = [i.sqrt() for i in state.inv]
    return state


def layer_step(state, params, grads, data, *, lr, damping, ema_decay, l2_reg=0., momentum=0.,
               momentum_type='preconditioned', weight_decay=0., dtype=torch.float32,
               update_std=False):
    """The per-group body of SecondOrderOptimizer.step (secondorder.py:195-209):
       raw:   g += l2_reg*p (and curv.l2_reg = l2_reg), momentum if type 'raw'
       curv.step(); curv.precondition_grad()
       preconditioned: g += weight_decay*p, momentum if type 'preconditioned'
       p -= lr*g
    params/grads: [w, b] or [w]; returns (new params, final grads)."""
    params = [p.to(dtype) for p in params]
    grads = [g.to(dtype) for g in grads]
    if state.momentum is None:
        state.momentum = [torch.zeros_like(p) for p in params]

    def apply_momentum(gs):
        if momentum == 0:
            return gs
        state.momentum = [b * momentum + g for b, g in zip(state.momentum, gs)]
        return [b.clone() for b in state.momentum]

    if l2_reg != 0:
        grads = [g + l2_reg * p for g, p in zip(grads, params)]
        state.l2_reg = l2_reg
    if momentum_type == 'raw':
        grads = apply_momentum(grads)
    curvature_step(state, data, damping, ema_decay, dtype, update_std)
    if state.kind == 'kron':
        gw, gb = precondition(state.inv[1], state.inv[0], grads[0],
                              grads[1] if state.bias else None, dtype)
        grads = [gw, gb] if state.bias else [gw]
    else:
        grads = [i * g for i, g in zip(state.inv, grads)]
    if weight_decay != 0:
        grads = [g + weight_decay * p for g, p in zip(grads, params)]
    if momentum_type == 'preconditioned':
        grads = apply_momentum(grads)
    params = [p - lr * g for p, g in zip(params, grads)]
    return params, grads


def sgd_tail(p, grad, buf, lr, momentum=0., weight_decay=0.):
    """Preconditioned-gradient tail for one tensor: g += wd*p; buf = m*buf + g;
    g = buf; p -= lr*g  (secondorder.py:248-261,225-231)."""
    if weight_decay != 0:
        grad = grad + weight_decay * p
    if momentum != 0:
        buf = buf * momentum + grad
        grad = buf.clone()
    return p - lr * grad, grad, buf


# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------

def tri_pack(mat):
    """Upper triangle of a square matrix, row by row: the packed form in which the
    reference sends symmetric factors (cuBLAS strttp with FILL_MODE_LOWER on the
    row-major array, torchsso/utils/chainer_communicators/_utility.py:59-86)."""
    n = mat.shape[0]
    iu = torch.triu_indices(n, n)
    return mat[iu[0], iu[1]]


def tri_unpack(vec, n):
    """Symmetric n x n matrix from its packed upper triangle: element (y, x) and
    (x, y) are vec[n*y - y*(y+1)/2 + x] for x >= y (_utility.py:19-31)."""
    out = torch.empty(n, n, dtype=vec.dtype)
    iu = torch.triu_indices(n, n)
    out[iu[0], iu[1]] = vec
    out[iu[1], iu[0]] = vec
    return out


def pack_arrays(arrays):
    """Flat buffer of a list of (tensor, triangular): arrays back to back, symmetric
    ones as triangles (Packer.pack, _utility.py:33-44)."""
    return torch.cat([tri_pack(t) if tri else t.reshape(-1) for t, tri in arrays])


def rel_fro(x, ref):
    """||x - ref||_F / ||ref||_F in float64."""
    x = torch.as_tensor(x).double().cpu()
    ref = torch.as_tensor(ref).double().cpu()
    d = (x - ref).norm().item()
    r = ref.norm().item()
    return d / r if r > 0 else d


def conv_out_size(size, k, s, p, d):
    return (size + 2 * p - d * (k - 1) - 1) // s + 1


def np_seeded(shape, seed, scale=1.0):
    rng = np.random.RandomState(seed)
    return torch.from_numpy((rng.standard_normal(shape) * scale).astype(np.float32))
