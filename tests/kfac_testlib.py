"""Shared helpers for the test-suite: model builders, a plain-torch capture of
per-layer inputs / output gradients, a straight-line K-FAC replay on the CPU
oracle, and an oracle-backed stand-in for torchsso._ops used to exercise the
host logic of the optimizers where no GPU exists."""
import os

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import kfac_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def load_golden(name):
    return dict(np.load(os.path.join(GOLDEN, name + '.npz')))


# models of the golden fixtures (same definitions as tests/golden/make_reference_vectors.py)
def build_mlp():
    torch.manual_seed(1)
    return nn.Sequential(nn.Linear(12, 16), nn.ReLU(), nn.Linear(16, 10), nn.ReLU(),
                         nn.Linear(10, 5))


def build_convnet():
    torch.manual_seed(1)
    return nn.Sequential(
        nn.Conv2d(2, 4, 3, padding=1), nn.BatchNorm2d(4), nn.ReLU(),
        nn.Conv2d(4, 6, 3, stride=2, bias=False), nn.ReLU(),
        nn.Flatten(), nn.Linear(6 * 3 * 3, 5))


def load_init(model, golden):
    sd = {k[5:]: torch.from_numpy(v) for k, v in golden.items() if k.startswith('init.')}
    model.load_state_dict(sd)
    return model


def leaf_modules(model):
    return [m for m in model.modules()
            if len(list(m.children())) == 0 and len(list(m.parameters())) > 0]


def capture(model, x, y):
    """One forward/backward with plain torch hooks: per leaf module the input,
    the output (detached copy) and the gradient w.r.t. the output."""
    rec = {}
    handles = []

    def fwd(mod, inp, out):
        rec[mod] = {'input': inp[0].detach().clone(), 'output': out.detach().clone()}
        out.register_hook(lambda g, mod=mod: rec[mod].__setitem__('grad_output', g.detach().clone()))

    for m in leaf_modules(model):
        handles.append(m.register_forward_hook(fwd))
    model.zero_grad()
    out = model(x)
    loss = F.cross_entropy(out, y)
    loss.backward()
    for h in handles:
        h.remove()
    return loss.detach(), out.detach(), rec


def oracle_factors(mod, r, dtype):
    """Curvature data of one layer from the captured tensors, via the oracle."""
    if isinstance(mod, nn.Linear):
        return 'kron', [O.factor_linear_a(r['input'], mod.bias is not None, dtype),
                        O.factor_linear_g(r['grad_output'], dtype)]
    if isinstance(mod, nn.Conv2d):
        return 'kron', [O.factor_conv_a(r['input'], mod.kernel_size, mod.stride, mod.padding,
                                        mod.dilation, mod.bias is not None, dtype),
                        O.factor_conv_g(r['grad_output'], dtype)]
    if isinstance(mod, (nn.BatchNorm1d, nn.BatchNorm2d)):
        xhat = O.bn_restore_input(r['output'].to(dtype), mod.weight.detach().to(dtype),
                                  mod.bias.detach().to(dtype))
        return 'diag', O.bn_diag(xhat, r['grad_output'], mod.bias is not None, dtype)
    raise TypeError(type(mod))


def oracle_kfac_run(model, x, y, steps, *, lr, damping, ema_decay, l2_reg=0., momentum=0.,
                    momentum_type='preconditioned', weight_decay=0., dtype=torch.float32,
                    num_mc_samples=None):
    """Straight-line replay of SecondOrderOptimizer (or, with num_mc_samples, of
    VIOptimizer without sampling) on the CPU oracle.  Returns a list (per step)
    of lists (per layer) of dicts with params / grads / ema / inv."""
    mods = leaf_modules(model)
    states = {}
    history = []
    for _ in range(steps):
        reps = 1 if num_mc_samples is None else num_mc_samples
        acc = {m: None for m in mods}
        accg = {m: None for m in mods}
        for _r in range(reps):
            _, _, rec = capture(model, x, y)
            for m in mods:
                kind, data = oracle_factors(m, rec[m], dtype)
                grads = [p.grad.detach().to(dtype) for p in m.parameters()]
                acc[m] = O.accumulate(acc[m], data, 1.0 / reps)
                accg[m] = O.accumulate(accg[m], grads, 1.0 / reps)
                if m not in states:
                    states[m] = O.LayerState(kind, m.bias is not None)
        snap = []
        for m in mods:
            params = [p.detach() for p in m.parameters()]
            new_params, grads = O.layer_step(
                states[m], params, accg[m], acc[m], lr=lr, damping=damping, ema_decay=ema_decay,
                l2_reg=l2_reg, momentum=momentum, momentum_type=momentum_type,
                weight_decay=weight_decay, dtype=dtype)
            with torch.no_grad():
                for p, q in zip(m.parameters(), new_params):
                    p.copy_(q.to(p.dtype))
            snap.append({'params': new_params, 'grads': grads, 'ema': states[m].ema,
                         'inv': states[m].inv, 'damping': damping + states[m].l2_reg_ema})
        history.append(snap)
    return history


def compare_with_golden(history_or_optimizer_snapshots, golden, tol=1e-4,
                        what=('param', 'grad', 'ema', 'inv'), skip=(), exceptions=None, label=''):
    """Relative Frobenius error of every stored array against the golden arrays; prints the
    worst entry and asserts each one <= tol (1e-4, the bar of the parity tests).
    `skip` lists (group, name, index) entries that are mathematically zero, whose
    stored value is rounding noise (e.g. the gradient of a bias in front of a
    BatchNorm layer).  `exceptions` maps (group, name, index) to (bound, reason) for an
    entry that is allowed a named, wider bound; every use is printed."""
    worst, worst_at = 0., None
    exceptions = exceptions or {}
    for s, snap in enumerate(history_or_optimizer_snapshots):
        for gi, layer in enumerate(snap):
            for key, name in (('params', 'param'), ('grads', 'grad'), ('ema', 'ema'), ('inv', 'inv')):
                if name not in what:
                    continue
                for k, t in enumerate(layer[key]):
                    if (gi, name, k) in skip:
                        continue
                    ref = golden['step%d.g%d.%s%d' % (s, gi, name, k)]
                    err = O.rel_fro(torch.as_tensor(t).reshape(ref.shape), torch.from_numpy(ref))
                    where = 'step %d layer %d %s%d' % (s, gi, name, k)
                    bound = tol
                    if (gi, name, k) in exceptions:
                        bound, reason = exceptions[(gi, name, k)]
                        print('golden %s: %s held to %.1e instead of %.1e (%s): %.3e'
                              % (label, where, bound, tol, reason, err))
                    assert err <= bound, '%s: rel err %.3e > %.1e' % (where, err, bound)
                    if err > worst:
                        worst, worst_at = err, where
    print('golden %s: worst rel. Frobenius error %.3e at %s (bar %.0e)' % (label, worst, worst_at, tol))
    return worst


def snapshot_optimizer(optimizer, target='params'):
    """Per-layer dicts in the same layout as oracle_kfac_run, from a torchsso optimizer."""
    snap = []
    for group in optimizer.param_groups:
        curv = group['curv']
        snap.append({'params': [p.detach().cpu().clone() for p in group['params']],
                     'grads': [p.grad.detach().cpu().clone() for p in group['params']],
                     'ema': [e.detach().cpu().clone() for e in (curv.ema or [])],
                     'inv': [i.detach().cpu().clone() for i in (curv.inv or [])]})
    return snap


# ---------------------------------------------------------------------------
# oracle-backed stand-in for torchsso._ops (host-logic tests without a GPU)
# ---------------------------------------------------------------------------

class OracleOps(object):
    """Same function names and argument meaning as torchsso._ops, computed on CPU
    tensors by the oracle.  Lives in tests/ only."""

    dtype = torch.float32

    def factor_linear(self, x, add_bias, alpha, out=None, beta=0., prev=None, stream=None):
        n = x.shape[0]
        r = O.factor_linear_a(x, add_bias, self.dtype) * (n * alpha)
        return self._emit(r, out, beta, prev)

    def factor_conv_a(self, x, kernel_size, stride, padding, dilation, add_bias, alpha, out=None, beta=0.,
                      prev=None, stream=None):
        n = x.shape[0]
        r = O.factor_conv_a(x, kernel_size, stride, padding, dilation, add_bias, self.dtype) * (n * alpha)
        return self._emit(r, out, beta, prev)

    def factor_conv_g(self, g, alpha, out=None, beta=0., prev=None, stream=None):
        n, c, h, w = g.shape
        r = O.factor_conv_g(g, self.dtype, scale_by_batch=False) * (n * h * w * alpha)
        return self._emit(r, out, beta, prev)

    @staticmethod
    def _emit(r, out, beta, prev=None):
        old = out if prev is None else prev
        if beta != 0:
            r = r + beta * old
        if out is None:
            return r
        out.copy_(r)
        return out

    def pi_damped_inverse_batched(self, As, Gs, dampings, A_invs=None, G_invs=None, info=None):
        ra, rg = [], []
        for i, (A, G, d) in enumerate(zip(As, Gs, dampings)):
            a, g = O.pi_damped_inverse(A, G, d, self.dtype)
            if A_invs is not None:
                A_invs[i].copy_(a)
                G_invs[i].copy_(g)
            ra.append(a)
            rg.append(g)
        return (A_invs or ra), (G_invs or rg), torch.zeros(2 * len(As), dtype=torch.int32)

    def pi_damped_inverse_std_batched(self, As, Gs, dampings, A_invs, G_invs, A_stds, G_stds,
                                      info=None):
        _, _, info = self.pi_damped_inverse_batched(As, Gs, dampings, A_invs, G_invs)
        for inv, std in list(zip(A_invs, A_stds)) + list(zip(G_invs, G_stds)):
            if std is not None:
                std.copy_(O.cholesky_upper(inv, self.dtype))
        return info

    def pi_damped_inverse_factored_batched(self, As, Gs, dampings, A_invs, G_invs, A_facs, G_facs,
                                           info=None):
        ra, rg, info = self.pi_damped_inverse_batched(As, Gs, dampings)
        for res, invs, facs in ((ra, A_invs, A_facs), (rg, G_invs, G_facs)):
            for r, inv, fac in zip(res, invs, facs):
                assert (inv is None) != (fac is None)
                if inv is not None:
                    inv.copy_(r)
                else:
                    # the upper Y with Y Y^T = r: the lower Cholesky factor of r with rows
                    # and columns reversed, reversed back
                    low = torch.linalg.cholesky(r.double().flip(0, 1))
                    fac.copy_(low.flip(0, 1).to(r.dtype))
        return info

    def precondition_factored_batched(self, G_ops, A_ops, grad_ws, grad_bs, g_factored=None,
                                      a_factored=None):
        def explicit(ops, flags):
            return [op @ op.t() if flags is None or flags[l] else op for l, op in enumerate(ops)]
        self.precondition_batched(explicit(G_ops, g_factored), explicit(A_ops, a_factored),
                                  grad_ws, grad_bs)

    def damped_inverse_batched(self, mats, damps=None, outs=None, info=None):
        res = [O.damped_inverse(m, 0. if damps is None else damps[i], self.dtype)
               for i, m in enumerate(mats)]
        if outs is not None:
            for o, r in zip(outs, res):
                o.copy_(r)
            res = outs
        return res, torch.zeros(len(mats), dtype=torch.int32)

    def cholesky_upper_batched(self, mats, outs=None, info=None):
        res = [O.cholesky_upper(m, self.dtype) for m in mats]
        if outs is not None:
            for o, r in zip(outs, res):
                o.copy_(r)
            res = outs
        return res, torch.zeros(len(mats), dtype=torch.int32)

    def precondition_batched(self, G_invs, A_invs, grad_ws, grad_bs):
        for Gi, Ai, gw, gb in zip(G_invs, A_invs, grad_ws, grad_bs):
            w, b = O.precondition(Gi, Ai, gw, gb, self.dtype)
            gw.copy_(w)
            if gb is not None:
                gb.copy_(b)

    def sample_batched(self, U_Gs, U_As, noises, mean_ws, mean_bs, param_ws, param_bs, std_scale):
        for ug, ua, e, mw, mb, pw, pb in zip(U_Gs, U_As, noises, mean_ws, mean_bs, param_ws, param_bs):
            w, b = O.sample(mw, mb, ug, ua, e, std_scale, self.dtype)
            pw.copy_(w)
            if pb is not None:
                pb.copy_(b)

    def axpby_batched(self, xs, ys, a, b):
        for x, y in zip(xs, ys):
            y.copy_(a * x + (b * y if b != 0 else 0))

    def diag_inverse_batched(self, emas, invs, dampings, use_sqrt):
        for e, i, d in zip(emas, invs, dampings):
            i.copy_(O.diag_inverse(e, d, use_sqrt))

    def diag_precondition_batched(self, invs, grads):
        for i, g in zip(invs, grads):
            g.mul_(i)

    def sgd_update_batched(self, params, grads, bufs, lrs, momenta, weight_decays):
        for p, g, b, lr, m, wd in zip(params, grads, bufs, lrs, momenta, weight_decays):
            np_, ng, nb = O.sgd_tail(p, g, b, lr, m, wd)
            p.copy_(np_)
            g.copy_(ng)
            if m != 0:
                b.copy_(nb)

    def rowsq_sum(self, x, channels, scale=None, shift=None):
        if scale is not None:
            x = O.bn_restore_input(x, scale, shift)
        return (x * x).reshape(x.shape[0], channels, -1).sum(dim=2)

    def bn_diag_combine(self, sx, sg, alpha, bias):
        w = alpha * (sx * sg).sum(dim=0)
        b = alpha * sg.sum(dim=0) if bias else None
        return w, b

    def bn_diag_cov(self, grad_output, channels, sx, alpha, bias):
        return self.bn_diag_combine(sx, self.rowsq_sum(grad_output, channels), alpha, bias)


def _oracle_sqrt_batched(self, xs, ys):
    for x, y in zip(xs, ys):
        y.copy_(x.sqrt())


def _oracle_max_batched(self, xs, ys):
    for x, y in zip(xs, ys):
        y.copy_(torch.max(x, y))


def _oracle_diag_sample_batched(self, means, stds, noise_to_params, std_scales):
    for m, s, p, sc in zip(means, stds, noise_to_params, std_scales):
        p.copy_(m + sc * p * s)


def _oracle_diag_cov_linear(self, g, a, add_bias, alpha):
    n = g.shape[0]
    out = O.diag_cov_linear(a, g, add_bias, None, self.dtype, scale_by_batch=False)
    return out[0] * (n * alpha), (out[1] * (n * alpha) if add_bias else None)


def _oracle_diag_cov_conv2d(self, g, x, kernel_size, stride, padding, dilation, alpha):
    n, c_out = g.shape[:2]
    out = O.diag_cov_conv2d(x, g, tuple(kernel_size), stride, padding, dilation, False, None,
                            self.dtype, scale_by_batch=False)
    return out[0].reshape(c_out, -1) * (n * alpha)


def _oracle_pack_batched(self, arrays, buf, offset=0):
    flat = O.pack_arrays(arrays)
    buf[offset:offset + flat.numel()] = flat
    return offset + flat.numel()


def _oracle_unpack_batched(self, arrays, buf, offset=0):
    for t, tri in arrays:
        n = t.shape[0] * (t.shape[0] + 1) // 2 if tri else t.numel()
        seg = buf[offset:offset + n]
        t.copy_(O.tri_unpack(seg, t.shape[0]) if tri else seg.reshape(t.shape))
        offset += n
    return offset


def _oracle_packed_numel(self, arrays):
    return sum(t.shape[0] * (t.shape[0] + 1) // 2 if tri else t.numel() for t, tri in arrays)


OracleOps.pack_batched = _oracle_pack_batched
OracleOps.unpack_batched = _oracle_unpack_batched
OracleOps.packed_numel = _oracle_packed_numel
OracleOps.sqrt_batched = _oracle_sqrt_batched
OracleOps.max_batched = _oracle_max_batched
OracleOps.diag_sample_batched = _oracle_diag_sample_batched
OracleOps.diag_cov_linear = _oracle_diag_cov_linear
OracleOps.diag_cov_conv2d = _oracle_diag_cov_conv2d


def _oracle_scale_rows(self, x, w, use_sqrt):
    s = w.reshape((-1,) + (1,) * (x.dim() - 1))
    return x * (s.sqrt() if use_sqrt else s)


OracleOps.scale_rows = _oracle_scale_rows
