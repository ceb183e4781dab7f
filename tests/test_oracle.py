"""Pins the CPU oracle (oracle/kfac_oracle.py) without a GPU: against the golden
vectors written by the reference itself (tests/golden/*.npz) and against what
the mathematics fixes -- brute force on tiny inputs, closed forms, special cases
and invariants chosen so that a dropped term, a wrong index order or a
transposed operand fails."""
import math

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import kfac_oracle as O
import kfac_testlib as T

D = torch.float64


# ---- factors ---------------------------------------------------------------

def test_linear_a_bruteforce_and_bias_invariants():
    torch.manual_seed(0)
    a = torch.randn(7, 4, dtype=D)
    A = O.factor_linear_a(a, True, D)
    assert A.shape == (5, 5)
    ref = torch.zeros(5, 5, dtype=D)
    for n in range(7):
        row = list(a[n]) + [1.0]
        for i in range(5):
            for j in range(5):
                ref[i, j] += row[i] * row[j] / 7
    assert torch.allclose(A, ref, atol=1e-12)
    assert abs(A[-1, -1].item() - 1) < 1e-12            # ones column is LAST
    assert torch.allclose(A[-1, :-1], a.mean(0), atol=1e-12)
    assert O.factor_linear_a(a, False, D).shape == (4, 4)


def test_linear_g_scale_is_n_times_sum_outer():
    torch.manual_seed(1)
    g = torch.randn(6, 3, dtype=D)
    G = O.factor_linear_g(g, D)
    ref = sum(torch.outer(g[n], g[n]) for n in range(6)) * 6    # (1/n) * n^2
    assert torch.allclose(G, ref, atol=1e-12)


def _bruteforce_conv_a(x, kh, kw, sh, sw, ph, pw, dh, dw, bias):
    n, c, H, W = x.shape
    oh = (H + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    ow = (W + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    d = c * kh * kw + (1 if bias else 0)
    A = torch.zeros(d, d, dtype=D)
    for b in range(n):
        for y in range(oh):
            for xx in range(ow):
                patch = []
                for ci in range(c):
                    for i in range(kh):
                        for j in range(kw):
                            yy = y * sh - ph + i * dh
                            xj = xx * sw - pw + j * dw
                            inside = 0 <= yy < H and 0 <= xj < W
                            patch.append(x[b, ci, yy, xj].item() if inside else 0.0)
                if bias:
                    patch.append(1.0)
                v = torch.tensor(patch, dtype=D)
                A += torch.outer(v, v)
    return A / n, oh * ow


@pytest.mark.parametrize('geom', [
    (3, 3, 1, 1, 1, 1, 1, 1, True),
    (3, 2, 2, 1, 0, 1, 1, 1, False),
    (2, 3, 1, 2, 2, 0, 2, 1, True),
    (1, 1, 1, 1, 0, 0, 1, 1, True),
])
def test_conv_a_against_nested_loops(geom):
    kh, kw, sh, sw, ph, pw, dh, dw, bias = geom
    torch.manual_seed(2)
    x = torch.randn(2, 3, 6, 7, dtype=D)
    A = O.factor_conv_a(x, (kh, kw), (sh, sw), (ph, pw), (dh, dw), bias, D)
    ref, npos = _bruteforce_conv_a(x, kh, kw, sh, sw, ph, pw, dh, dw, bias)
    assert torch.allclose(A, ref, atol=1e-10)
    if bias:
        assert abs(A[-1, -1].item() - npos) < 1e-9      # divided by n only, not n*h*w


def test_conv_1x1_equals_linear_case():
    torch.manual_seed(3)
    x = torch.randn(3, 5, 4, 4, dtype=D)
    A = O.factor_conv_a(x, (1, 1), bias=False, dtype=D)
    flat = x.permute(0, 2, 3, 1).reshape(-1, 5)
    assert torch.allclose(A, flat.t() @ flat / 3, atol=1e-12)
    g = torch.randn(3, 5, 4, 4, dtype=D)
    G = O.factor_conv_g(g, D, scale_by_batch=False)
    gf = g.permute(0, 2, 3, 1).reshape(-1, 5)
    assert torch.allclose(G, gf.t() @ gf / (3 * 16), atol=1e-12)


def test_conv_row_order_matches_weight_layout_via_autograd():
    """dL/dW (as [c_out, c_in*kh*kw]) == m_G M^T for a sum-reduced loss: this fixes
    the (c, kh, kw) row order of M and the [c_out, n*h*w] layout of m_G."""
    torch.manual_seed(4)
    conv = nn.Conv2d(3, 4, 3, stride=2, padding=1, bias=True).double()
    x = torch.randn(2, 3, 7, 7, dtype=D)
    out = conv(x)
    gout = torch.randn_like(out)
    (out * gout).sum().backward()
    u = F.unfold(x, 3, stride=2, padding=1)
    M = u.transpose(0, 1).reshape(27, -1)
    mG = gout.transpose(0, 1).reshape(4, -1)
    assert torch.allclose(conv.weight.grad.reshape(4, -1), mG @ M.t(), atol=1e-10)
    # and the two factors are the Gram matrices of exactly these M and m_G
    assert torch.allclose(O.factor_conv_a(x, (3, 3), (2, 2), (1, 1), bias=False, dtype=D),
                          M @ M.t() / 2, atol=1e-10)
    assert torch.allclose(O.factor_conv_g(gout, D, scale_by_batch=False),
                          mG @ mG.t() / mG.shape[1], atol=1e-12)


def test_batch_rescale_undoes_mean_reduction():
    """G built from the gradients of a mean-reduced loss, times n^2, equals
    n * sum of outer products of the sum-reduced loss gradients."""
    torch.manual_seed(5)
    lin = nn.Linear(4, 3).double()
    x = torch.randn(5, 4, dtype=D)
    y = torch.randint(0, 3, (5,))
    out = lin(x)
    out.retain_grad()
    F.cross_entropy(out, y, reduction='mean').backward()
    g_mean = out.grad.clone()
    out2 = lin(x)
    out2.retain_grad()
    F.cross_entropy(out2, y, reduction='sum').backward()
    g_sum = out2.grad
    assert torch.allclose(O.factor_linear_g(g_mean, D), g_sum.t() @ g_sum / 5, atol=1e-12)


def test_bn_diag_is_mean_of_squared_per_sample_grads():
    torch.manual_seed(6)
    n, c = 4, 3
    bn = nn.BatchNorm2d(c).double()
    with torch.no_grad():
        bn.weight.uniform_(0.5, 1.5)
        bn.bias.normal_()
    x = torch.randn(n, c, 5, 5, dtype=D)
    out = bn(x)
    gout = torch.randn_like(out)
    xhat = O.bn_restore_input(out.detach(), bn.weight.detach(), bn.bias.detach())
    mu = x.mean(dim=(0, 2, 3), keepdim=True)
    var = x.var(dim=(0, 2, 3), unbiased=False, keepdim=True)
    assert torch.allclose(xhat, (x - mu) / torch.sqrt(var + bn.eps), atol=1e-9)
    w_curv, b_curv = O.bn_diag(xhat, gout, True, D, scale_by_batch=False)
    # per-sample gradients of weight/bias are sum_hw(xhat*g) and sum_hw(g); the
    # reference uses (sum xhat^2)(sum g^2) and sum g^2 instead: check those literally
    ref_w = torch.stack([(xhat[i] ** 2).sum((1, 2)) * (gout[i] ** 2).sum((1, 2)) for i in range(n)]).mean(0)
    ref_b = torch.stack([(gout[i] ** 2).sum((1, 2)) for i in range(n)]).mean(0)
    assert torch.allclose(w_curv, ref_w, atol=1e-10) and torch.allclose(b_curv, ref_b, atol=1e-10)
    w2, _ = O.bn_diag(xhat, gout, True, D)
    assert torch.allclose(w2, ref_w * n * n, atol=1e-8)


def test_diag_cov_is_mean_of_squared_per_sample_grads():
    """DiagCovLinear / DiagCovConv2d: with the layer's real output gradient of a
    mean-reduced loss, n^2-rescaled data == mean over samples of the squared gradient
    of that sample's own loss, taken sample by sample through autograd.  The conv
    bias entry is the reference's sum of squares (not the squared sum that the
    per-sample bias gradient would give), checked by loops."""
    torch.manual_seed(12)
    n = 5
    lin = nn.Linear(7, 4).double()
    x = torch.randn(n, 7, dtype=D)
    y = torch.randint(0, 4, (n,))
    out = lin(x)
    out.retain_grad()
    F.cross_entropy(out, y).backward()
    w, b = O.diag_cov_linear(x, out.grad, True, None, D)
    ref_w, ref_b = torch.zeros_like(lin.weight), torch.zeros_like(lin.bias)
    for i in range(n):
        gw, gb = torch.autograd.grad(F.cross_entropy(lin(x[i:i + 1]), y[i:i + 1]), [lin.weight, lin.bias])
        ref_w += gw ** 2 / n
        ref_b += gb ** 2 / n
    assert torch.allclose(w, ref_w, atol=1e-12) and torch.allclose(b, ref_b, atol=1e-12)
    # prob weighting scales each sample's squared gradient
    prob = torch.rand(n, dtype=D)
    wp, bp = O.diag_cov_linear(x, out.grad, True, prob, D)
    ref_w.zero_()
    for i in range(n):
        gw, = torch.autograd.grad(F.cross_entropy(lin(x[i:i + 1]), y[i:i + 1]), [lin.weight])
        ref_w += prob[i] * gw ** 2 / n
    assert torch.allclose(wp, ref_w, atol=1e-12)

    conv = nn.Conv2d(3, 4, (3, 2), stride=(2, 1), padding=(1, 0), dilation=(1, 2)).double()
    xc = torch.randn(n, 3, 9, 8, dtype=D)
    oc = conv(xc)
    oc.retain_grad()
    head = torch.randn(oc[0].numel(), 4, dtype=D)
    F.cross_entropy(oc.reshape(n, -1) @ head, y).backward()
    w, b = O.diag_cov_conv2d(xc, oc.grad, (3, 2), (2, 1), (1, 0), (1, 2), True, None, D)
    assert w.shape == conv.weight.shape
    ref_w = torch.zeros_like(conv.weight)
    for i in range(n):
        li = F.cross_entropy(conv(xc[i:i + 1]).reshape(1, -1) @ head, y[i:i + 1])
        gw, = torch.autograd.grad(li, [conv.weight])
        ref_w += gw ** 2 / n
    assert torch.allclose(w, ref_w, atol=1e-12)
    g = oc.grad
    ref_b = torch.zeros(4, dtype=D)
    for i in range(n):
        for c in range(4):
            for r in range(g.shape[2]):
                for q in range(g.shape[3]):
                    ref_b[c] += g[i, c, r, q] ** 2
    assert torch.allclose(b, ref_b * n, atol=1e-12)          # mean over n, times n^2


# ---- EMA / accumulate -------------------------------------------------------

def test_ema_weights_new_data_and_first_call_copies():
    d1, d2 = [torch.tensor([2.0])], [torch.tensor([10.0])]
    e = O.ema_update(d1, None, 0.95)
    assert e[0].item() == 2.0
    e = O.ema_update(d2, e, 0.95)
    assert abs(e[0].item() - (0.95 * 10 + 0.05 * 2)) < 1e-6
    assert O.ema_update(d2, e, 1)[0].item() == 10.0
    assert O.l2_reg_ema_update(1e-3, 0., 0.95, True) == 1e-3
    assert abs(O.l2_reg_ema_update(1e-3, 5e-4, 0.95, False) - (0.95e-3 + 0.05 * 5e-4)) < 1e-12
    acc = O.accumulate(None, d1, 0.5)
    acc = O.accumulate(acc, d2, 0.5)
    assert acc[0].item() == 6.0


# ---- inverse ----------------------------------------------------------------

def test_pi_damping_scalar_identity_case():
    A = torch.eye(3, dtype=D) * 4.0
    G = torch.eye(2, dtype=D) * 0.25
    pi, da, dg = O.pi_and_damping(A, G, 1e-2)
    assert abs(pi - 4.0) < 1e-12 and abs(da - 0.4) < 1e-12 and abs(dg - 0.025) < 1e-12
    Ai, Gi = O.pi_damped_inverse(A, G, 1e-2, D)
    assert torch.allclose(Ai, torch.eye(3, dtype=D) / 4.4, atol=1e-12)
    assert torch.allclose(Gi, torch.eye(2, dtype=D) / 0.275, atol=1e-12)


def test_inverse_2x2_by_hand_and_residual():
    X = torch.tensor([[2.0, 1.0], [1.0, 3.0]], dtype=D)
    inv = O.damped_inverse(X, 1.0, D)            # (X + I)^-1 = [[3,1],[1,4]]^-1
    ref = torch.tensor([[4.0, -1.0], [-1.0, 3.0]], dtype=D) / 11
    assert torch.allclose(inv, ref, atol=1e-12)
    torch.manual_seed(7)
    m = torch.randn(40, 30, dtype=D)
    S = m.t() @ m / 40
    inv = O.damped_inverse(S, 0.1, D)
    assert torch.allclose((S + 0.1 * torch.eye(30, dtype=D)) @ inv, torch.eye(30, dtype=D), atol=1e-9)
    assert O.rel_fro(O.damped_inverse(S, 0.1, torch.float32), inv) < 1e-5
    assert torch.allclose(O.diag_inverse(torch.tensor([4.0, 9.0]), 1.0), torch.tensor([0.2, 0.1]))
    assert torch.allclose(O.diag_inverse(torch.tensor([4.0, 9.0]), 1.0, True), torch.tensor([1 / 3, 0.25]))


def test_cholesky_upper_properties():
    torch.manual_seed(8)
    m = torch.randn(30, 12, dtype=D)
    S = m.t() @ m / 30 + 0.1 * torch.eye(12, dtype=D)
    U = O.cholesky_upper(S, D)
    assert torch.allclose(U.t() @ U, S, atol=1e-10)
    assert torch.equal(U, torch.triu(U)) and (U.diagonal() > 0).all()


# ---- precondition / sample --------------------------------------------------

def test_precondition_kronecker_identity():
    torch.manual_seed(9)
    dG, dA = 3, 5
    Gi = torch.randn(dG, dG, dtype=D); Gi = Gi @ Gi.t()
    Ai = torch.randn(dA, dA, dtype=D); Ai = Ai @ Ai.t()
    gw = torch.randn(dG, dA - 1, dtype=D)
    gb = torch.randn(dG, dtype=D)
    pw, pb = O.precondition(Gi, Ai, gw, gb, D)
    V = torch.cat((gw, gb.view(-1, 1)), 1)
    ref = (torch.kron(Gi, Ai) @ V.reshape(-1)).reshape(dG, dA)     # row-major vec
    assert torch.allclose(pw, ref[:, :-1], atol=1e-9) and torch.allclose(pb, ref[:, -1], atol=1e-9)
    # conv-shaped weight gradient keeps its shape
    gw4 = torch.randn(dG, 2, 1, 2, dtype=D)
    pw4, _ = O.precondition(Gi, Ai[:4, :4], gw4, None, D)
    assert pw4.shape == gw4.shape
    assert torch.allclose(pw4.reshape(dG, -1), Gi @ gw4.reshape(dG, -1) @ Ai[:4, :4], atol=1e-9)


def test_sample_with_injected_noise():
    torch.manual_seed(10)
    dG, dA = 3, 4
    UG = torch.triu(torch.randn(dG, dG, dtype=D))
    UA = torch.triu(torch.randn(dA, dA, dtype=D))
    mw = torch.randn(dG, dA - 1, dtype=D); mb = torch.randn(dG, dtype=D)
    E = torch.randn(dG, dA, dtype=D)
    pw, pb = O.sample(mw, mb, UG, UA, E, 0.5, D)
    M = torch.cat((mw, mb.view(-1, 1)), 1)
    ref = M + 0.5 * (torch.kron(UG, UA.t().contiguous()) @ E.reshape(-1)).reshape(dG, dA)
    assert torch.allclose(torch.cat((pw, pb.view(-1, 1)), 1), ref, atol=1e-10)
    pw0, _ = O.sample(mw, mb, UG, UA, E, 0.0, D)
    assert torch.equal(pw0, mw)


# ---- host sequencing against the reference's own golden vectors ---------------

def test_sgd_equivalence_without_preconditioning():
    """With identity curvature inverses the step is plain SGD with momentum and
    weight decay, i.e. torch.optim.SGD."""
    torch.manual_seed(11)
    w0 = torch.randn(3, 4, dtype=D)
    g = [torch.randn(3, 4, dtype=D) for _ in range(3)]
    p = nn.Parameter(w0.clone())
    sgd = torch.optim.SGD([p], lr=0.1, momentum=0.9, weight_decay=1e-2)
    w, buf = w0.clone(), torch.zeros_like(w0)
    for k in range(3):
        p.grad = g[k].clone()
        sgd.step()
        w, _, buf = O.sgd_tail(w, g[k], buf, 0.1, 0.9, 1e-2)
        assert torch.allclose(w, p.detach(), atol=1e-12)


def test_oracle_step_matches_reference_mlp():
    gold = T.load_golden('ref_mlp_kfac')
    model = T.load_init(T.build_mlp(), gold)
    hist = T.oracle_kfac_run(model, torch.from_numpy(gold['x']), torch.from_numpy(gold['y']), 3,
                             lr=0.05, damping=1e-3, ema_decay=0.95, l2_reg=1e-3, momentum=0.9,
                             weight_decay=1e-3)
    worst = T.compare_with_golden(hist, gold)
    # effective damping = damping + EMA of l2_reg (curvature.py:102-104)
    for s in range(3):
        assert abs(hist[s][0]['damping'] - float(gold['step%d.g0.damping' % s])) < 1e-12
    assert worst < 1e-4


def test_oracle_step_matches_reference_convnet_bn_raw_momentum():
    gold = T.load_golden('ref_convnet_kfac')
    model = T.load_init(T.build_convnet(), gold)
    hist = T.oracle_kfac_run(model, torch.from_numpy(gold['x']), torch.from_numpy(gold['y']), 2,
                             lr=0.02, damping=1e-2, ema_decay=0.9, l2_reg=1e-4, momentum=0.5,
                             momentum_type='raw')
    T.compare_with_golden(hist, gold)


def test_oracle_vi_accumulation_matches_reference():
    gold = T.load_golden('ref_mlp_vi_nosample')
    model = T.load_init(T.build_mlp(), gold)
    hist = T.oracle_kfac_run(model, torch.from_numpy(gold['x']), torch.from_numpy(gold['y']), 2,
                             lr=0.05, damping=1e-3, ema_decay=0.95, momentum=0.9, num_mc_samples=3)
    T.compare_with_golden(hist, gold)


# ---- Fisher weighting ---------------------------------------------------------

def test_fisher_factors_reduce_to_cov_and_match_the_presoftmax_closed_form():
    torch.manual_seed(12)
    n, c = 6, 4
    g = torch.randn(n, c, dtype=D)
    ones = torch.ones(n, dtype=D)
    assert torch.allclose(O.fisher_linear_g(g, ones, D), O.factor_linear_g(g, D), atol=1e-12)
    g4 = torch.randn(n, c, 3, 3, dtype=D)
    assert torch.allclose(O.fisher_conv_g(g4, ones, D), O.factor_conv_g(g4, D), atol=1e-12)
    xh = torch.randn(n, c, 3, 3, dtype=D)
    a, b = O.fisher_bn_diag(xh, g4, ones, True, D), O.bn_diag(xh, g4, True, D)
    assert all(torch.allclose(u, v, atol=1e-12) for u, v in zip(a, b))
    # exact Fisher at the logits: sum over classes of p_c * grad_c grad_c^T, with
    # grad_c = (p - e_c)/n the gradient of the mean cross entropy for label c
    logits = torch.randn(n, c, dtype=D)
    p = torch.softmax(logits, 1)
    G = torch.zeros(c, c, dtype=D)
    for k in range(c):
        grad_k = (p - torch.eye(c, dtype=D)[k]) / n
        G += O.fisher_linear_g(grad_k, p[:, k], D)
    closed = sum(torch.diag(p[i]) - torch.outer(p[i], p[i]) for i in range(n)) / n
    assert torch.allclose(G, closed, atol=1e-12)


def test_fisher_conv_and_batchnorm_weighting_with_nontrivial_prob():
    """G = sum_n prob[n] * (sum_hw g_n g_n^T) / (n h w)  (torchsso/curv/fisher/conv.py:61-70) and
    the BatchNorm diagonal  mean_n[(sum_hw xhat^2) * prob[n] * (sum_hw g^2)]
    (fisher/batchnorm.py:11-30), written as explicit per-sample loops on a 2x3x2x2 input with
    prob != 1: a prob^2 weighting, a weight along the channel axis or a weight applied to
    xhat as well would all fail here.  The batch^2 rescale is left out (scale_by_batch=False)
    so that the loops state the reference formula literally."""
    torch.manual_seed(13)
    n, c, h, w = 2, 3, 2, 2
    g = torch.randn(n, c, h, w, dtype=D)
    xh = torch.randn(n, c, h, w, dtype=D)
    prob = torch.tensor([0.3, 0.9], dtype=D)
    G = torch.zeros(c, c, dtype=D)
    for b in range(n):
        for i in range(c):
            for j in range(c):
                for y in range(h):
                    for x in range(w):
                        G[i, j] += prob[b] * g[b, i, y, x] * g[b, j, y, x]
    G /= n * h * w
    assert torch.allclose(O.fisher_conv_g(g, prob, D, scale_by_batch=False), G, atol=1e-13)
    assert torch.allclose(O.fisher_conv_g(g, prob, D), G * n * n, atol=1e-12)
    wcurv, bcurv = torch.zeros(c, dtype=D), torch.zeros(c, dtype=D)
    for b in range(n):
        for i in range(c):
            gg = sum(prob[b] * g[b, i, y, x] ** 2 for y in range(h) for x in range(w))
            xx = sum(xh[b, i, y, x] ** 2 for y in range(h) for x in range(w))
            wcurv[i] += xx * gg / n
            bcurv[i] += gg / n
    got = O.fisher_bn_diag(xh, g, prob, True, D, scale_by_batch=False)
    assert torch.allclose(got[0], wcurv, atol=1e-13) and torch.allclose(got[1], bcurv, atol=1e-13)
    got = O.fisher_bn_diag(xh, g, prob, False, D)
    assert len(got) == 1 and torch.allclose(got[0], wcurv * n * n, atol=1e-12)
    # h = w = 1 reduces the conv factor to the Linear one, which the closed form at the
    # logits pins (test above)
    g1 = torch.randn(5, c, 1, 1, dtype=D)
    p5 = torch.rand(5, dtype=D)
    assert torch.allclose(O.fisher_conv_g(g1, p5, D), O.fisher_linear_g(g1.reshape(5, c), p5, D),
                          atol=1e-12)
    # and the weight is linear in prob, not quadratic
    assert torch.allclose(O.fisher_conv_g(g, 2 * prob, D), 2 * O.fisher_conv_g(g, prob, D), atol=1e-12)
    a2 = O.fisher_bn_diag(xh, g, 2 * prob, True, D)
    a1 = O.fisher_bn_diag(xh, g, prob, True, D)
    assert all(torch.allclose(u, 2 * v, atol=1e-12) for u, v in zip(a2, a1))


def test_triangular_wire_format_matches_the_reference_index_formula():
    """mat[i] = vec[n*y - y*(y+1)/2 + x] with (y, x) = sorted(i // n, i % n): the
    reference's unpack kernel, evaluated literally."""
    torch.manual_seed(21)
    for n in (1, 2, 5, 9):
        a = torch.randn(n, n, dtype=D)
        sym = a + a.t()
        vec = O.tri_pack(sym)
        assert vec.numel() == n * (n + 1) // 2
        back = torch.empty(n * n, dtype=D)
        for i in range(n * n):
            x, y = i % n, i // n
            if x < y:
                x, y = y, x
            back[i] = vec[n * y - y * (y + 1) // 2 + x]
        assert torch.equal(back.reshape(n, n), sym)
        assert torch.equal(O.tri_unpack(vec, n), sym)
        # packing walks the rows from the diagonal to the right (what strttp writes)
        k = 0
        for y in range(n):
            for x in range(y, n):
                assert vec[k] == sym[y, x]
                k += 1
    g = torch.randn(3, 4, dtype=D)
    buf = O.pack_arrays([(sym, True), (g, False)])
    assert buf.numel() == 45 + 12 and torch.equal(buf[45:], g.reshape(-1))
