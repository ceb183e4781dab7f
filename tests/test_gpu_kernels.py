"""Parity of every HIP kernel with the CPU oracle, called through the C ABI
(torchsso._ops is a ctypes shim over libkfac_hip.so).  Bar: relative Frobenius
error <= 1e-4 in fp32 against the float64 oracle."""
import pytest
import torch

from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-4
D = torch.float64


@pytest.fixture(scope='module')
def ops():
    from torchsso import _ops
    return _ops


@pytest.fixture(scope='module')
def dev():
    return torch.device('cuda:0')


def spd(n, L=None, seed=0):
    g = torch.Generator().manual_seed(seed + n)
    L = L or max(2 * n, 64)
    x = torch.randn(L, n, dtype=D, generator=g)
    return ((x.t() @ x) / L).float()


@pytest.mark.parametrize('n,f,bias', [(1, 1, True), (1, 1, False), (8, 5, True), (128, 784, True),
                                      (128, 1000, False), (37, 129, True), (300, 130, True),
                                      (5000, 64, False), (20000, 200, True), (256, 2048, True)])
def test_factor_linear(ops, dev, n, f, bias):
    torch.manual_seed(n + f)
    x = torch.randn(n, f)
    out = ops.factor_linear(x.to(dev), bias, 1.0 / n)
    assert O.rel_fro(out, O.factor_linear_a(x, bias, D)) < TOL
    assert torch.equal(out, out.t())
    # G convention: alpha = n
    g = torch.randn(n, f) * 1e-2
    outg = ops.factor_linear(g.to(dev), False, float(n))
    assert O.rel_fro(outg, O.factor_linear_g(g, D)) < TOL


def test_factor_linear_fused_running_average(ops, dev):
    torch.manual_seed(0)
    for n, f in [(64, 300), (9000, 70)]:     # single pass and split-k paths
        x = torch.randn(n, f)
        old = spd(f + 1)
        out = ops.factor_linear(x.to(dev), True, 0.95 / n, out=old.to(dev).clone(), beta=0.05)
        ref = 0.95 * O.factor_linear_a(x, True, D) + 0.05 * old.double()
        assert O.rel_fro(out, ref) < TOL
        # the same into a second buffer: the previous average stays untouched
        prev = old.to(dev).clone()
        nxt = torch.full_like(prev, float('nan'))
        ops.factor_linear(x.to(dev), True, 0.95 / n, out=nxt, beta=0.05, prev=prev)
        assert O.rel_fro(nxt, ref) < TOL and torch.equal(prev.cpu(), old)


@pytest.mark.parametrize('shape,k,s,p,d,bias', [
    ((2, 3, 8, 8), (3, 3), (1, 1), (1, 1), (1, 1), True),
    ((4, 3, 32, 32), (5, 5), (1, 1), (0, 0), (1, 1), True),
    ((3, 5, 9, 11), (3, 3), (2, 2), (1, 1), (1, 1), False),
    ((2, 4, 12, 12), (3, 3), (1, 1), (2, 2), (2, 2), True),
    ((2, 3, 10, 9), (3, 2), (2, 1), (1, 0), (1, 2), True),
    ((8, 64, 14, 14), (3, 3), (1, 1), (1, 1), (1, 1), False),
    ((4, 16, 8, 8), (1, 1), (1, 1), (0, 0), (1, 1), True),
    ((2, 3, 30, 30), (7, 7), (2, 2), (3, 3), (1, 1), False),
    ((1, 1, 1, 1), (1, 1), (1, 1), (0, 0), (1, 1), True),
    ((16, 32, 28, 28), (3, 3), (2, 2), (1, 1), (1, 1), False),
    # pointwise without bias (read like an output gradient), with padding, with stride
    ((4, 48, 8, 8), (1, 1), (1, 1), (0, 0), (1, 1), False),
    ((3, 300, 7, 7), (1, 1), (1, 1), (0, 0), (1, 1), False),
    ((3, 20, 7, 7), (1, 1), (1, 1), (1, 1), (1, 1), False),
    ((3, 20, 8, 8), (1, 1), (2, 2), (0, 0), (1, 1), False),
])
def test_factor_conv_a(ops, dev, shape, k, s, p, d, bias):
    torch.manual_seed(sum(shape))
    x = torch.randn(*shape)
    out = ops.factor_conv_a(x.to(dev), k, s, p, d, bias, 1.0 / shape[0])
    ref = O.factor_conv_a(x, k, s, p, d, bias, D)
    assert out.shape == ref.shape
    assert O.rel_fro(out, ref) < TOL
    assert torch.equal(out, out.t())


# stride 1, no bias, 2..9 taps, an even channel count >= 16: the A factor is assembled
# from spatial correlations of the input instead of the im2col product (and falls
# back to it when the geometry needs too many pieces, e.g. 3x3 without padding)
@pytest.mark.parametrize('shape,k,p,d', [
    ((3, 16, 7, 9), (3, 3), (1, 1), (1, 1)),
    ((2, 130, 9, 8), (3, 3), (2, 2), (2, 2)),
    ((2, 18, 6, 7), (2, 3), (1, 0), (1, 2)),
    ((2, 16, 5, 5), (3, 3), (2, 1), (1, 1)),
    ((2, 32, 3, 3), (3, 3), (1, 1), (1, 1)),
    ((2, 16, 2, 2), (3, 3), (1, 1), (1, 1)),
    ((2, 20, 10, 10), (1, 5), (0, 2), (1, 1)),
    ((2, 16, 6, 6), (3, 3), (3, 3), (1, 1)),
    ((2, 16, 7, 7), (3, 3), (0, 0), (1, 1)),
    ((4, 256, 14, 14), (3, 3), (1, 1), (1, 1)),
    ((2, 512, 7, 7), (3, 3), (1, 1), (1, 1)),
    ((5, 66, 28, 28), (3, 3), (1, 1), (1, 1)),
])
def test_factor_conv_a_by_correlations(ops, dev, shape, k, p, d):
    torch.manual_seed(sum(shape) + k[1])
    x = torch.randn(*shape)
    ref = O.factor_conv_a(x, k, (1, 1), p, d, False, D)
    out = ops.factor_conv_a(x.to(dev), k, (1, 1), p, d, False, 1.0 / shape[0])
    assert out.shape == ref.shape
    assert O.rel_fro(out, ref) < TOL
    assert torch.equal(out, out.t())
    # running-average epilogue on the same path
    old = spd(ref.shape[0])
    out = ops.factor_conv_a(x.to(dev), k, (1, 1), p, d, False, 0.9 / shape[0],
                            out=old.to(dev).clone(), beta=0.1)
    assert O.rel_fro(out, 0.9 * ref + 0.1 * old.double()) < TOL
    prev = old.to(dev).clone()
    nxt = ops.factor_conv_a(x.to(dev), k, (1, 1), p, d, False, 0.9 / shape[0], beta=0.1, prev=prev)
    assert O.rel_fro(nxt, 0.9 * ref + 0.1 * old.double()) < TOL and torch.equal(prev.cpu(), old)


# the last three: few k-splits over many tiles (tile-wise reduction, mirrored blocks
# through LDS), with a ragged last tile in one of them
@pytest.mark.parametrize('shape', [(1, 1, 1, 1), (2, 3, 4, 4), (8, 64, 7, 7), (4, 130, 14, 14),
                                   (16, 64, 56, 56), (3, 257, 5, 3), (32, 1024, 14, 14),
                                   (32, 2048, 7, 7), (8, 1500, 10, 10),
                                   # small factors over long reductions, ragged sizes
                                   (32, 128, 28, 28), (24, 100, 30, 31), (20, 40, 30, 31),
                                   (6, 64, 112, 112)])
def test_factor_conv_g(ops, dev, shape):
    torch.manual_seed(sum(shape))
    g = torch.randn(*shape) * 1e-2
    n, c, h, w = shape
    out = ops.factor_conv_g(g.to(dev), float(n) / (h * w))
    assert O.rel_fro(out, O.factor_conv_g(g, D)) < TOL
    old = spd(c)
    prev = old.to(dev).clone()
    nxt = ops.factor_conv_g(g.to(dev), 0.5 * float(n) / (h * w), beta=0.5, prev=prev)
    assert O.rel_fro(nxt, 0.5 * O.factor_conv_g(g, D) + 0.5 * old.double()) < TOL
    assert torch.equal(prev.cpu(), old)


DIMS = [1, 2, 31, 32, 33, 64, 96, 97, 127, 128, 129, 255, 256, 257, 300, 513, 785]


def test_damped_inverse_batched_mixed_sizes(ops, dev):
    mats = [spd(n) for n in DIMS]
    damps = [0.05 + 0.01 * i for i in range(len(DIMS))]
    outs, info = ops.damped_inverse_batched([m.to(dev) for m in mats], damps)
    assert info.cpu().tolist() == [0] * len(DIMS)
    for m, d, o in zip(mats, damps, outs):
        assert O.rel_fro(o, O.damped_inverse(m, d, D)) < TOL
        assert torch.equal(o, o.t())


def test_pi_damped_inverse_pairs(ops, dev):
    As = [spd(785), spd(76), spd(1601), spd(10)]
    Gs = [spd(1000) * 3, spd(64) * 0.01, spd(128) * 0.5, spd(129) * 40]
    damp = [1e-3, 1e-2, 1e-3, 5e-3]
    Ai, Gi, info = ops.pi_damped_inverse_batched([a.to(dev) for a in As], [g.to(dev) for g in Gs], damp)
    assert info.cpu().tolist() == [0] * 8
    for a, g, d, ai, gi in zip(As, Gs, damp, Ai, Gi):
        ra, rg = O.pi_damped_inverse(a, g, d, D)
        assert O.rel_fro(ai, ra) < TOL and O.rel_fro(gi, rg) < TOL


def test_inverse_reports_non_spd_and_leaves_others_intact(ops, dev):
    bad = spd(300)
    bad[150, 150] = -5.0
    good = spd(40)
    outs, info = ops.damped_inverse_batched([bad.to(dev), good.to(dev)], [0.0, 0.0])
    info = info.cpu().tolist()
    assert info[0] == 151 and info[1] == 0
    assert O.rel_fro(outs[1], O.damped_inverse(good, 0.0, D)) < TOL


def test_cholesky_upper_batched(ops, dev):
    mats = [spd(n) + 0.1 * torch.eye(n) for n in DIMS]
    outs, info = ops.cholesky_upper_batched([m.to(dev) for m in mats])
    assert info.cpu().tolist() == [0] * len(DIMS)
    for m, o in zip(mats, outs):
        assert O.rel_fro(o, O.cholesky_upper(m, D)) < TOL
        assert torch.equal(o, torch.triu(o))


def test_inverse_and_cholesky_of_random_ragged_batches(ops, dev):
    """Batches of one to seven matrices of random sizes up to 1500 (last blocks of every
    width, few-tile launches of every shape) against float64 on the device."""
    gen = torch.Generator().manual_seed(7)
    for trial in range(10):
        count = int(torch.randint(1, 7, (1,), generator=gen))
        sizes = [int(torch.randint(1, 1500, (1,), generator=gen)) for _ in range(count)]
        if trial % 3 == 0:   # a size next to a multiple of the block size
            sizes.append(max(1, 128 * int(torch.randint(1, 12, (1,), generator=gen))
                             + int(torch.randint(0, 3, (1,), generator=gen)) - 1))
        mats = []
        for n in sizes:
            a = torch.randn(n, n + 8, generator=gen).to(dev)
            mats.append(a @ a.t() / (n + 8) + 0.1 * torch.eye(n, device=dev))
        outs, info = ops.damped_inverse_batched(mats, [1e-3] * len(mats))
        chol, info2 = ops.cholesky_upper_batched(mats)
        assert int(info.abs().sum()) == 0 and int(info2.abs().sum()) == 0, sizes
        for m, o, u in zip(mats, outs, chol):
            n = m.shape[0]
            m64 = m.double()
            ref = torch.linalg.inv(m64 + 1e-3 * torch.eye(n, device=dev, dtype=torch.float64))
            assert ((o.double() - ref).norm() / ref.norm()).item() < TOL, (sizes, n)
            assert ((u.double().t() @ u.double() - m64).norm() / m64.norm()).item() < 1e-5, (sizes, n)
            assert torch.equal(u, torch.triu(u)), (sizes, n)


def test_inverse_with_posterior_std_from_the_same_factorisation(ops, dev):
    """kfac_pi_damped_inverse_std_batched: for the layers that ask for it, the upper Cholesky
    factor W of each inverse (W^T W = inverse: what torchsso.utils.cholesky of the inverse
    gives, utils/cholesky_cupy.py:9-14) comes out of the inversion itself, which factors those
    matrices back to front.  Ragged sizes (1 .. 1500, block-size neighbours), layers with and
    without std mixed in one call; everything against float64 on the device."""
    gen = torch.Generator().manual_seed(11)
    pairs = [(1, 3), (33, 64), (129, 127), (700, 10), (385, 192), (1500, 256), (128, 1025)]
    As, Gs = [], []
    for dA, dG in pairs:
        for n, lst in ((dA, As), (dG, Gs)):
            a = torch.randn(n, n + 8, generator=gen).to(dev)
            lst.append((a @ a.t() / (n + 8)).contiguous())
    damp = [1e-3 * (l + 1) for l in range(len(pairs))]
    want_std = [l % 3 != 1 for l in range(len(pairs))]
    Ai = [torch.full_like(a, float('nan')) for a in As]
    Gi = [torch.full_like(g, float('nan')) for g in Gs]
    Astd = [torch.full_like(a, float('nan')) if w else None for a, w in zip(As, want_std)]
    Gstd = [torch.full_like(g, float('nan')) if w else None for g, w in zip(Gs, want_std)]
    info = ops.pi_damped_inverse_std_batched(As, Gs, damp, Ai, Gi, Astd, Gstd)
    plainA, plainG, info0 = ops.pi_damped_inverse_batched(As, Gs, damp)
    assert info.cpu().tolist() == [0] * (2 * len(pairs)) and int(info0.abs().sum()) == 0
    eye = lambda n: torch.eye(n, dtype=D, device=dev)
    worst = {'inverse': 0., 'std': 0., 'std^T std vs inverse': 0.}
    for l, (a, g) in enumerate(zip(As, Gs)):
        pi = ((a.double().diagonal().sum() / a.shape[0]) / (g.double().diagonal().sum() / g.shape[0])).sqrt()
        r = damp[l] ** 0.5
        for X, shift, inv, plain, std in ((a, r * pi, Ai[l], plainA[l], Astd[l]),
                                          (g, r / pi, Gi[l], plainG[l], Gstd[l])):
            n = X.shape[0]
            ref = torch.linalg.inv(X.double() + shift * eye(n))
            worst['inverse'] = max(worst['inverse'], ((inv.double() - ref).norm() / ref.norm()).item())
            assert torch.equal(inv, inv.t())
            if std is None:
                assert torch.equal(inv, plain)              # untouched by the others' reversal
                continue
            W = std.double()
            assert torch.equal(std, torch.triu(std)) and bool((std.diagonal() > 0).all())
            refW = torch.linalg.cholesky(ref).mT
            worst['std'] = max(worst['std'], ((W - refW).norm() / refW.norm()).item())
            worst['std^T std vs inverse'] = max(worst['std^T std vs inverse'],
                                                ((W.t() @ W - inv.double()).norm() / inv.double().norm()).item())
    print('inverse + std in one factorisation, worst rel. Frobenius errors:',
          {k: '%.2e' % v for k, v in worst.items()})
    assert worst['inverse'] < TOL and worst['std'] < TOL and worst['std^T std vs inverse'] < 1e-5


def test_inverse_in_factored_form(ops, dev):
    """kfac_pi_damped_inverse_factored_batched: per matrix either the inverse or only its
    upper-triangular factor Y (Y Y^T = inverse, zeros below the diagonal), for which no
    explicit inverse is formed.  Every combination per layer in one call; Y against the
    inverse of the float64 Cholesky factor, Y Y^T and the explicit inverses against the
    float64 inverse; ragged sizes around the 128-blocks."""
    gen = torch.Generator().manual_seed(12)
    pairs = [(1, 2), (64, 33), (127, 129), (10, 700), (192, 385), (1025, 128), (257, 1500), (300, 513)]
    As, Gs = [], []
    for dA, dG in pairs:
        for n, lst in ((dA, As), (dG, Gs)):
            a = torch.randn(n, n + 8, generator=gen).to(dev)
            lst.append((a @ a.t() / (n + 8)).contiguous())
    damp = [1e-3 * (l + 1) for l in range(len(pairs))]
    nan = lambda x: torch.full_like(x, float('nan'))
    # per layer: the form asked for A and for G ('f' factor, 'i' inverse)
    plan = ['ff', 'fi', 'if', 'ff', 'fi', 'ff', 'ii', 'if']
    Ai = [nan(a) if p[0] == 'i' else None for a, p in zip(As, plan)]
    Gi = [nan(g) if p[1] == 'i' else None for g, p in zip(Gs, plan)]
    Af = [nan(a) if p[0] == 'f' else None for a, p in zip(As, plan)]
    Gf = [nan(g) if p[1] == 'f' else None for g, p in zip(Gs, plan)]
    info = ops.pi_damped_inverse_factored_batched(As, Gs, damp, Ai, Gi, Af, Gf)
    assert info.cpu().tolist() == [0] * (2 * len(pairs))
    eye = lambda n: torch.eye(n, dtype=D, device=dev)
    worst = {'factor': 0., 'Y Y^T vs inverse': 0., 'inverse': 0.}
    for l, (a, g) in enumerate(zip(As, Gs)):
        pi = ((a.double().diagonal().sum() / a.shape[0]) / (g.double().diagonal().sum() / g.shape[0])).sqrt()
        r = damp[l] ** 0.5
        for X, shift, inv, y in ((a, r * pi, Ai[l], Af[l]), (g, r / pi, Gi[l], Gf[l])):
            Xd = X.double() + shift * eye(X.shape[0])
            ref = torch.linalg.inv(Xd)
            if inv is not None:
                assert torch.equal(inv, inv.t())
                worst['inverse'] = max(worst['inverse'], ((inv.double() - ref).norm() / ref.norm()).item())
            else:
                assert torch.equal(y, torch.triu(y)) and bool((y.diagonal() > 0).all())
                refY = torch.linalg.inv(torch.linalg.cholesky(Xd).mT)     # X = R^T R, Y = R^-1
                Y = y.double()
                worst['factor'] = max(worst['factor'], ((Y - refY).norm() / refY.norm()).item())
                worst['Y Y^T vs inverse'] = max(worst['Y Y^T vs inverse'],
                                                ((Y @ Y.t() - ref).norm() / ref.norm()).item())
    print('factored inverse, worst rel. Frobenius errors:', {k: '%.2e' % v for k, v in worst.items()})
    assert max(worst.values()) < TOL
    with pytest.raises(Exception, match='exactly one of inverse and factor'):
        ops.pi_damped_inverse_factored_batched(As[:1], Gs[:1], damp[:1], [None], [nan(Gs[0])],
                                               [None], [None])


def test_precondition_with_factored_inverses(ops, dev):
    """kfac_precondition_factored_batched: G^-1 [gW | gb] A^-1 with each side given either by
    its upper-triangular factor Y (Y Y^T = inverse, applied twice) or by the explicit inverse,
    all four combinations, against the float64 product with the explicit inverses; with and
    without bias column, sizes on both sides of the 128-tiles, more layers than one table
    chunk holds.  The strict lower triangles of the factor buffers hold zeros, as the
    inversion leaves them."""
    torch.manual_seed(21)
    shapes = SHAPES + [(257, 640, True), (385, 129, False), (1100, 300, True), (640, 900, True)] \
        + [(1 + (13 * i) % 140, 2 + (29 * i) % 260, i % 2 == 0) for i in range(135)]
    Gy = [torch.triu(torch.randn(g, g) / g ** 0.5 + torch.eye(g)) for g, a, b in shapes]
    Ay = [torch.triu(torch.randn(a, a) / a ** 0.5 + torch.eye(a)) for g, a, b in shapes]
    gfac = [i % 4 in (0, 1) for i in range(len(shapes))]
    afac = [i % 4 in (0, 2) for i in range(len(shapes))]
    Ginv = [y.double() @ y.double().t() for y in Gy]
    Ainv = [y.double() @ y.double().t() for y in Ay]
    Gop = [(y if f else i.float()).to(dev) for y, i, f in zip(Gy, Ginv, gfac)]
    Aop = [(y if f else i.float()).to(dev) for y, i, f in zip(Ay, Ainv, afac)]
    gws = [torch.randn(g, a - (1 if b else 0)) for g, a, b in shapes]
    gbs = [torch.randn(g) if b else None for g, a, b in shapes]
    for flags in ((gfac, afac), (None, None)):
        dgw = [x.to(dev).clone() for x in gws]
        dgb = [None if x is None else x.to(dev).clone() for x in gbs]
        if flags[0] is None:        # no flag arrays: every operand is a factor
            ops.precondition_factored_batched([y.to(dev) for y in Gy], [y.to(dev) for y in Ay], dgw, dgb)
        else:
            ops.precondition_factored_batched(Gop, Aop, dgw, dgb, gfac, afac)
        worst = 0.
        for i in range(len(shapes)):
            rw, rb = O.precondition(Ginv[i], Ainv[i], gws[i], gbs[i], D)
            errs = [O.rel_fro(dgw[i], rw)] + ([] if rb is None else [O.rel_fro(dgb[i], rb)])
            worst = max([worst] + errs)
            assert max(errs) < TOL, (shapes[i], gfac[i], afac[i])
        print('factored preconditioning over %d layers (%s): worst rel. Frobenius error %.2e'
              % (len(shapes), 'mixed' if flags[0] else 'all factored', worst))


SHAPES = [(10, 193, True), (64, 76, True), (1000, 785, True), (128, 1601, True),
          (512, 1152, False), (1, 2, True), (3, 1, False), (64, 64, False), (130, 257, True)]


def test_precondition_batched(ops, dev):
    torch.manual_seed(1)
    Gis = [spd(g) for g, a, b in SHAPES]
    Ais = [spd(a) for g, a, b in SHAPES]
    gws = [torch.randn(g, a - (1 if b else 0)) for g, a, b in SHAPES]
    gbs = [torch.randn(g) if b else None for g, a, b in SHAPES]
    dgw = [x.to(dev).clone() for x in gws]
    dgb = [None if x is None else x.to(dev).clone() for x in gbs]
    ops.precondition_batched([x.to(dev) for x in Gis], [x.to(dev) for x in Ais], dgw, dgb)
    for i in range(len(SHAPES)):
        rw, rb = O.precondition(Gis[i], Ais[i], gws[i], gbs[i], D)
        assert O.rel_fro(dgw[i], rw) < TOL
        if rb is not None:
            assert O.rel_fro(dgb[i], rb) < TOL


def test_more_than_128_matrices_and_layers_in_one_call(ops, dev):
    """The batched launches list their work 128 matrices / layers at a time: 150 of
    mixed sizes must come out the same as one by one."""
    dims = [1 + (37 * i) % 300 for i in range(150)]
    mats = [spd(n, seed=i) for i, n in enumerate(dims)]
    outs, info = ops.damped_inverse_batched([m.to(dev) for m in mats], [0.05] * len(mats))
    assert info.cpu().tolist() == [0] * len(mats)
    for m, o in zip(mats, outs):
        assert O.rel_fro(o, O.damped_inverse(m, 0.05, D)) < TOL
    torch.manual_seed(9)
    shapes = [(1 + (13 * i) % 140, 2 + (29 * i) % 260, i % 2 == 0) for i in range(140)]
    Gis = [spd(g, seed=1) for g, a, b in shapes]
    Ais = [spd(a, seed=2) for g, a, b in shapes]
    gws = [torch.randn(g, a - (1 if b else 0)) for g, a, b in shapes]
    gbs = [torch.randn(g) if b else None for g, a, b in shapes]
    dgw = [x.to(dev).clone() for x in gws]
    dgb = [None if x is None else x.to(dev).clone() for x in gbs]
    ops.precondition_batched([x.to(dev) for x in Gis], [x.to(dev) for x in Ais], dgw, dgb)
    for i in range(len(shapes)):
        rw, rb = O.precondition(Gis[i], Ais[i], gws[i], gbs[i], D)
        assert O.rel_fro(dgw[i], rw) < TOL
        if rb is not None:
            assert O.rel_fro(dgb[i], rb) < TOL


def test_precondition_conv_shaped_gradient(ops, dev):
    torch.manual_seed(2)
    Gi, Ai = spd(6), spd(4 * 3 * 3 + 1)
    gw, gb = torch.randn(6, 4, 3, 3), torch.randn(6)
    dw, db = gw.to(dev).clone(), gb.to(dev).clone()
    ops.precondition_batched([Gi.to(dev)], [Ai.to(dev)], [dw], [db])
    rw, rb = O.precondition(Gi, Ai, gw, gb, D)
    assert dw.shape == gw.shape and O.rel_fro(dw, rw) < TOL and O.rel_fro(db, rb) < TOL


def test_sample_batched(ops, dev):
    torch.manual_seed(3)
    UG = [O.cholesky_upper(spd(g) + 0.1 * torch.eye(g)) for g, a, b in SHAPES]
    UA = [O.cholesky_upper(spd(a) + 0.1 * torch.eye(a)) for g, a, b in SHAPES]
    noise = [torch.randn(g, a) for g, a, b in SHAPES]
    mws = [torch.randn(g, a - (1 if b else 0)) for g, a, b in SHAPES]
    mbs = [torch.randn(g) if b else None for g, a, b in SHAPES]
    pw = [torch.empty_like(x).to(dev) for x in mws]
    pb = [None if x is None else torch.empty_like(x).to(dev) for x in mbs]
    ops.sample_batched([x.to(dev) for x in UG], [x.to(dev) for x in UA], [x.to(dev) for x in noise],
                       [x.to(dev) for x in mws], [None if x is None else x.to(dev) for x in mbs],
                       pw, pb, 0.37)
    for i in range(len(SHAPES)):
        rw, rb = O.sample(mws[i], mbs[i], UG[i], UA[i], noise[i], 0.37, D)
        assert O.rel_fro(pw[i], rw) < TOL
        if rb is not None:
            assert O.rel_fro(pb[i], rb) < TOL


def test_elementwise_tails(ops, dev):
    torch.manual_seed(4)
    sizes = [1, 100, 5000, 785000]
    xs = [torch.randn(n) for n in sizes]
    ys = [torch.randn(n) for n in sizes]
    dys = [y.to(dev).clone() for y in ys]
    ops.axpby_batched([x.to(dev) for x in xs], dys, 0.95, 0.05)
    for d, x, y in zip(dys, xs, ys):
        assert O.rel_fro(d, 0.95 * x.double() + 0.05 * y.double()) < 1e-6
    lrs, moms, wds = [0.1, 0.2, 0.3], [0.9, 0.0, 0.5], [0.0, 1e-2, 1e-3]
    ps = [torch.randn(n) for n in [7, 4097, 300000]]
    gs = [torch.randn(n) for n in [7, 4097, 300000]]
    bs = [torch.randn(n) for n in [7, 4097, 300000]]
    dp = [p.to(dev).clone() for p in ps]
    dg = [g.to(dev).clone() for g in gs]
    db = [b.to(dev).clone() for b in bs]
    ops.sgd_update_batched(dp, dg, [db[0], None, db[2]], lrs, moms, wds)
    for i in range(3):
        rp, rg, rb = O.sgd_tail(ps[i].double(), gs[i].double(), bs[i].double(), lrs[i], moms[i], wds[i])
        assert O.rel_fro(dp[i], rp) < 1e-6 and O.rel_fro(dg[i], rg) < 1e-6
        assert O.rel_fro(db[i], rb) < 1e-6
    ema = torch.rand(50) + 0.1
    inv = [torch.empty(50, device=dev)]
    ops.diag_inverse_batched([ema.to(dev)], inv, [1e-3], False)
    assert O.rel_fro(inv[0], O.diag_inverse(ema.double(), 1e-3)) < 1e-6
    ops.diag_inverse_batched([ema.to(dev)], inv, [1e-3], True)
    assert O.rel_fro(inv[0], O.diag_inverse(ema.double(), 1e-3, True)) < 1e-6
    g = torch.randn(50)
    dgr = [g.to(dev).clone()]
    ops.diag_precondition_batched(inv, dgr)
    assert O.rel_fro(dgr[0], g.double() * inv[0].cpu().double()) < 1e-6


# row lengths: 1 (BatchNorm1d), up to 64 / 128 / 256 loads per row with and without
# float4 alignment, the ResNet-50 shapes 7x7, 14x14 and 28x28, a ragged channel count,
# rows beyond 1024 elements and a batch beyond 2048 samples (general kernels)
@pytest.mark.parametrize('shape', [(6, 10, 5, 5), (4, 3, 1, 1), (32, 64, 56, 56), (16, 7),
                                   (32, 96, 7, 7), (32, 130, 14, 14), (8, 70, 28, 28),
                                   (5, 33, 10, 13), (3, 300, 9, 9), (7, 18, 16, 20),
                                   (2, 9, 33, 33), (40, 6, 2, 2), (2100, 3, 2, 2)])
@pytest.mark.parametrize('bias', [True, False])
def test_batchnorm_diag(ops, dev, shape, bias):
    torch.manual_seed(5)
    c = shape[1]
    out = torch.randn(*shape)
    w = torch.rand(c) + 0.5
    b = torch.randn(c)
    g = torch.randn(*shape) * 1e-2
    ref = O.bn_diag(O.bn_restore_input(out.double(), w.double(), b.double()), g, bias, D)
    sx = ops.rowsq_sum(out.to(dev), c, w.to(dev), b.to(dev))
    xhat = O.bn_restore_input(out.double(), w.double(), b.double())
    assert O.rel_fro(sx, (xhat * xhat).reshape(shape[0], c, -1).sum(2)) < TOL
    sg = ops.rowsq_sum(g.to(dev), c)
    wc, bc = ops.bn_diag_combine(sx, sg, float(shape[0]), bias)
    assert O.rel_fro(wc, ref[0]) < TOL and (not bias or O.rel_fro(bc, ref[1]) < TOL)
    # the backward half in one call
    wf, bf = ops.bn_diag_cov(g.to(dev), c, sx, float(shape[0]), bias)
    assert O.rel_fro(wf, ref[0]) < TOL and (not bias or O.rel_fro(bf, ref[1]) < TOL)
    assert (bf is None) == (not bias)


def test_batchnorm_diag_of_many_layers_in_one_launch(ops, dev):
    """kfac_bn_diag_cov_batched: every row-length class in one call (1 element, rows with
    and without float4 alignment in the three load counts, rows beyond 1024 elements), with
    and without a bias output, against the float64 oracle; the short-row layers give the
    bits of the single-layer call (same code), and a second call the same bits."""
    torch.manual_seed(6)
    shapes = [(6, 10, 5, 5), (4, 3, 1, 1), (8, 16, 56, 56), (16, 7), (32, 96, 7, 7),
              (32, 130, 14, 14), (8, 70, 28, 28), (5, 33, 10, 13), (3, 300, 9, 9),
              (7, 18, 16, 20), (2, 9, 33, 33), (40, 6, 2, 2), (4, 5, 112, 112), (3, 4, 41, 37)]
    jobs, refs, singles = [], [], []
    for k, shape in enumerate(shapes):
        c, n, bias = shape[1], shape[0], k % 3 != 0
        out = torch.randn(*shape)
        w, b = torch.rand(c) + 0.5, torch.randn(c)
        g = (torch.randn(*shape) * 1e-2).to(dev)
        refs.append(O.bn_diag(O.bn_restore_input(out.double(), w.double(), b.double()), g.cpu(), bias, D))
        sx = ops.rowsq_sum(out.to(dev), c, w.to(dev), b.to(dev))
        wo = torch.full((c,), float('nan'), device=dev)
        bo = torch.full((c,), float('nan'), device=dev) if bias else None
        jobs.append((g, c, sx, float(n), wo, bo))
        singles.append(ops.bn_diag_cov(g, c, sx, float(n), bias))
    ops.bn_diag_cov_batched(jobs, dev)
    first = [(j[4].clone(), None if j[5] is None else j[5].clone()) for j in jobs]
    ops.bn_diag_cov_batched(jobs, dev)
    for shape, job, ref, one, again in zip(shapes, jobs, refs, singles, first):
        wo, bo = job[4], job[5]
        assert O.rel_fro(wo, ref[0]) < TOL, shape
        assert bo is None or O.rel_fro(bo, ref[1]) < TOL, shape
        assert torch.equal(wo, again[0]) and (bo is None or torch.equal(bo, again[1])), shape
        if job[0].numel() // (shape[0] * shape[1]) <= 256:
            assert torch.equal(wo, one[0]) and (bo is None or torch.equal(bo, one[1])), shape


# ---- size-independent properties at the benchmark's sizes ---------------------

def test_large_inverse_at_benchmark_sizes(ops, dev):
    """4608 (largest ResNet-50 factor, batch 32) and 9217 (AlexNet fc6, batch
    256, rank-deficient before damping).  The error of the float32 result Y is
    measured in float64 on the device through one Newton step,
    Y_true = Y + Y (I - X Y) + O(|I - X Y|^2), and for 4608 also against
    torch.linalg.inv in float64 (a library routine).  The 9217 matrix has a condition
    number of about 7e2, where the error of ANY float32 inverse (cond * 2^-24 times a
    modest factor) sits right at 1e-4: the reference's own float32 result on the same
    matrix (scipy.linalg.inv, torchsso/utils/inv_cupy.py:32-34, through the oracle) is
    measured beside it and the bound is 1e-4 or 1.5 x that error, whichever is larger.
    The residual X Y - I scales with the condition number and gets a looser bound."""
    from test_gpu_bench_step import inverse_record
    for n, L in [(4608, 1568), (9217, 256)]:
        g = torch.Generator(device='cpu').manual_seed(n)
        x = torch.randn(L, n, generator=g).to(dev)
        X = ops.factor_linear(x, False, 1.0 / L)
        damp = 0.05 * X.diagonal().mean().item()
        outs, info = ops.damped_inverse_batched([X], [damp])
        assert info.cpu().tolist() == [0]
        Xd = X.double()
        _, err, err_ref, _, _ = inverse_record('random rank-%d factor' % L, Xd, damp, outs[0])
        Xd.diagonal().add_(damp)
        Y = outs[0].double()
        R = torch.eye(n, device=dev, dtype=D) - Xd @ Y
        res = R.norm().item() / n ** 0.5
        print('n=%d rel err %.2e (reference fp32: %.2e) residual %.2e' % (n, err, err_ref, res))
        assert res < 1e-3, (n, res)
        assert err <= max(TOL, 1.5 * err_ref), (n, err, err_ref)
        if n == 4608:
            assert err < TOL
            ref = torch.linalg.inv(Xd)
            assert ((Y - ref).norm() / ref.norm()).item() < TOL
            del ref
        assert torch.equal(outs[0], outs[0].t())
        del Xd, Y, R


def test_cholesky_factor_at_benchmark_size(ops, dev):
    """std = upper Cholesky factor of a 4608^2 inverse (posterior of the largest
    ResNet-50 factor): U^T U reproduces the matrix (float64 product on the device), U is
    upper triangular with a positive diagonal, and agrees with torch.linalg.cholesky in
    float64 (a library routine)."""
    n = 4608
    g = torch.Generator(device='cpu').manual_seed(n)
    x = torch.randn(1568, n, generator=g).to(dev)
    X = ops.factor_linear(x, False, 1.0 / 1568)
    X.diagonal().add_(0.05 * X.diagonal().mean().item())
    outs, info = ops.cholesky_upper_batched([X])
    assert info.cpu().tolist() == [0]
    U = outs[0]
    assert torch.equal(U, torch.triu(U)) and (U.diagonal() > 0).all()
    Ud = U.double()
    assert ((Ud.t() @ Ud - X.double()).norm() / X.double().norm()).item() < 1e-5
    ref = torch.linalg.cholesky(X.double()).t()
    assert ((Ud - ref).norm() / ref.norm()).item() < TOL


def test_precondition_at_benchmark_sizes_against_float64_on_device(ops, dev):
    """G^-1 [dW | db] A^-1 for the largest layers of configs 3 and 4 (ResNet-50
    layer4 3x3 conv: 512 x 4608, no bias; AlexNet fc6: 4096 x 9216 + bias) against
    the same product in float64 on the device (torch.matmul, a library routine)."""
    for dg, da, bias in [(512, 4608, False), (4096, 9217, True)]:
        g = torch.Generator(device='cpu').manual_seed(dg + da)
        Gi = torch.randn(dg, dg, generator=g).to(dev)
        Gi = Gi @ Gi.t() / dg + torch.eye(dg, device=dev)
        Ai = torch.randn(da, da // 4, generator=g).to(dev)
        Ai = Ai @ Ai.t() / (da // 4) + torch.eye(da, device=dev)
        W = torch.randn(dg, da - (1 if bias else 0), generator=g).to(dev)
        b = torch.randn(dg, generator=g).to(dev) if bias else None
        V = W.double() if b is None else torch.cat([W.double(), b.double()[:, None]], 1)
        ref = Gi.double() @ V @ Ai.double()
        gw, gb = W.clone(), None if b is None else b.clone()
        ops.precondition_batched([Gi], [Ai], [gw], [gb])
        got = gw.double() if gb is None else torch.cat([gw.double(), gb.double()[:, None]], 1)
        err = ((got - ref).norm() / ref.norm()).item()
        print('precondition %d x %d: rel err %.2e' % (dg, da, err))
        assert err < TOL
        del Gi, Ai, V, ref, got


def test_factor_linearity_at_full_size(ops, dev):
    """factor(x stacked with y) = factor(x) + factor(y) (sums of outer products),
    on the ResNet-50 layer1 3x3 shape (c=64, 56x56, batch 32)."""
    torch.manual_seed(6)
    x = torch.randn(32, 64, 56, 56, device=dev)
    full = ops.factor_conv_a(x, (3, 3), (1, 1), (1, 1), (1, 1), False, 1.0)
    a = ops.factor_conv_a(x[:16].contiguous(), (3, 3), (1, 1), (1, 1), (1, 1), False, 1.0)
    b = ops.factor_conv_a(x[16:].contiguous(), (3, 3), (1, 1), (1, 1), (1, 1), False, 1.0)
    assert O.rel_fro(full, (a.double() + b.double())) < 1e-5
    # and against F.unfold on the device in float64 for one image (library routine)
    u = torch.nn.functional.unfold(x[:1].double(), 3, padding=1)[0]
    one = ops.factor_conv_a(x[:1].contiguous(), (3, 3), (1, 1), (1, 1), (1, 1), False, 1.0)
    assert O.rel_fro(one, u @ u.t()) < TOL


@pytest.mark.parametrize('c,hw,stride', [(128, 28, 1), (256, 14, 1), (512, 7, 1), (256, 28, 2)])
def test_conv_a_at_resnet50_shapes_against_unfold_on_device(ops, dev, c, hw, stride):
    """The 3x3 layers of BASELINE config 3 at batch 32 (d = 1152 / 2304 / 4608, both the
    correlation path and the strided im2col path) against F.unfold + matmul in float64
    on the device (library routines)."""
    torch.manual_seed(c + hw)
    x = torch.randn(32, c, hw, hw, device=dev)
    out = ops.factor_conv_a(x, (3, 3), (stride, stride), (1, 1), (1, 1), False, 1.0 / 32)
    ref = torch.zeros(9 * c, 9 * c, dtype=D, device=dev)
    for i in range(0, 32, 4):
        u = torch.nn.functional.unfold(x[i:i + 4].double(), 3, padding=1, stride=stride)
        u = u.transpose(0, 1).reshape(9 * c, -1)
        ref += u @ u.t()
    ref /= 32
    assert O.rel_fro(out, ref) < TOL
    assert torch.equal(out, out.t())
    ev = torch.linalg.eigvalsh(out.double())
    assert ev.min().item() > -1e-4 * ev.max().item()       # a Gram matrix: positive semi-definite


# ---- wire format ----------------------------------------------------------------------

def test_pack_and_unpack_against_the_oracle(ops, dev):
    torch.manual_seed(31)
    arrays = []
    for n in (1, 2, 63, 64, 65, 130, 1000):
        a = torch.randn(n, n)
        arrays.append((a + a.t(), True))
        arrays.append((torch.randn(n, 3), False))
    arrays.append((torch.randn(5000), False))
    total = ops.packed_numel(arrays)
    want = O.pack_arrays(arrays)
    assert total == want.numel()
    buf = torch.full((total + 11,), float('nan'), device=dev)
    end = ops.pack_batched([(t.to(dev), tri) for t, tri in arrays], buf, 11)
    assert end == total + 11
    assert torch.equal(buf[11:].cpu(), want) and torch.isnan(buf[:11]).all()
    outs = [(torch.full_like(t, float('nan')).to(dev), tri) for t, tri in arrays]
    ops.unpack_batched(outs, buf, 11)
    for (o, _), (t, _) in zip(outs, arrays):
        assert torch.equal(o.cpu(), t)
    # more arrays than one launch lists, and a factor of the largest benchmark size
    many = [(torch.randn(3 + i % 40, 3 + i % 40), i % 3 != 0) for i in range(150)]
    many = [((t + t.t()) if tri else t, tri) for t, tri in many]
    buf = torch.empty(ops.packed_numel(many), device=dev)
    ops.pack_batched([(t.to(dev), tri) for t, tri in many], buf)
    assert torch.equal(buf.cpu(), O.pack_arrays(many))
    big = torch.randn(4608, 4608, device=dev)
    big = big + big.t()
    buf = torch.empty(4608 * 4609 // 2, device=dev)
    ops.pack_batched([(big, True)], buf)
    back = torch.empty_like(big)
    ops.unpack_batched([(back, True)], buf)
    assert torch.equal(back, big)
    iu = torch.triu_indices(4608, 4608, device=dev)
    assert torch.equal(buf, big[iu[0], iu[1]])


# ---- diagonal covariance of Linear / Conv2d (VOGN) ------------------------------------

@pytest.mark.parametrize('n,fin,fout,bias', [(1, 1, 1, True), (7, 5, 3, False), (128, 784, 1000, True),
                                            (33, 130, 257, True), (256, 300, 10, False)])
def test_diag_cov_linear(ops, dev, n, fin, fout, bias):
    torch.manual_seed(n + fin)
    a, g = torch.randn(n, fin), torch.randn(n, fout) * 1e-2
    w, b = ops.diag_cov_linear(g.to(dev), a.to(dev), bias, float(n))
    ref = O.diag_cov_linear(a, g, bias, None, D)
    assert O.rel_fro(w, ref[0]) < TOL
    if bias:
        assert O.rel_fro(b, ref[1]) < TOL
    else:
        assert b is None


@pytest.mark.parametrize('shape,cout,k,s,p,d', [
    ((2, 3, 8, 8), 4, (3, 3), (1, 1), (1, 1), (1, 1)),
    ((5, 3, 9, 8), 4, (3, 2), (2, 1), (1, 0), (1, 2)),
    ((128, 3, 32, 32), 64, (5, 5), (1, 1), (0, 0), (1, 1)),       # config 2, conv1
    ((16, 64, 14, 14), 130, (5, 5), (1, 1), (0, 0), (1, 1)),      # several tiles, split over samples
    ((3, 200, 7, 7), 140, (3, 3), (2, 2), (1, 1), (1, 1)),
    ((1, 1, 1, 1), 1, (1, 1), (1, 1), (0, 0), (1, 1)),
])
def test_diag_cov_conv2d(ops, dev, shape, cout, k, s, p, d):
    torch.manual_seed(sum(shape) + cout)
    x = torch.randn(*shape)
    oh = O.conv_out_size(shape[2], k[0], s[0], p[0], d[0])
    ow = O.conv_out_size(shape[3], k[1], s[1], p[1], d[1])
    g = torch.randn(shape[0], cout, oh, ow) * 1e-2
    out = ops.diag_cov_conv2d(g.to(dev), x.to(dev), k, s, p, d, float(shape[0]))
    ref = O.diag_cov_conv2d(x, g, k, s, p, d, False, None, D)[0]
    assert O.rel_fro(out.reshape(ref.shape), ref) < TOL


def test_diag_element_wise_tails(ops, dev):
    torch.manual_seed(11)
    xs = [torch.rand(n) + 0.1 for n in (1, 7, 1000, 4097)]
    ys = [torch.empty(n, device=dev) for n in (1, 7, 1000, 4097)]
    ops.sqrt_batched([x.to(dev) for x in xs], ys)
    for x, y in zip(xs, ys):
        assert O.rel_fro(y, x.double().sqrt()) < 1e-6
    old = [torch.rand(n) for n in (1, 7, 1000, 4097)]
    ys = [o.to(dev) for o in old]
    ops.max_batched([x.to(dev) for x in xs], ys)
    for x, o, y in zip(xs, old, ys):
        assert torch.equal(y.cpu(), torch.max(x, o))
    means = [torch.randn(n) for n in (3, 1025)]
    stds = [torch.rand(n) for n in (3, 1025)]
    noise = [torch.randn(n) for n in (3, 1025)]
    ps = [e.to(dev) for e in noise]
    ops.diag_sample_batched([m.to(dev) for m in means], [s.to(dev) for s in stds], ps, [0.5, 2.0])
    for m, s, e, p, sc in zip(means, stds, noise, ps, (0.5, 2.0)):
        assert O.rel_fro(p, m.double() + sc * e.double() * s.double()) < 1e-6


# ---- Fisher weighting ---------------------------------------------------------------

def test_fisher_weighted_factors(ops, dev):
    torch.manual_seed(7)
    n, f = 96, 130
    g = torch.randn(n, f) * 1e-2
    passes = [torch.rand(n) for _ in range(3)]
    acc = None
    ref = torch.zeros(f, f, dtype=D)
    for k, prob in enumerate(passes):
        pg = ops.scale_rows(g.to(dev), prob.to(dev), True)
        acc = ops.factor_linear(pg, False, float(n), out=acc, beta=0. if k == 0 else 1.)
        ref += O.fisher_linear_g(g, prob, D)
    assert O.rel_fro(acc, ref) < TOL
    g4 = torch.randn(8, 70, 5, 6) * 1e-2
    prob = torch.rand(8)
    pg = ops.scale_rows(g4.to(dev), prob.to(dev), True)
    G = ops.factor_conv_g(pg, 8.0 / 30)
    assert O.rel_fro(G, O.fisher_conv_g(g4, prob, D)) < TOL
    # BatchNorm: prob * sum_hw g^2
    out = torch.randn(8, 70, 5, 6)
    w, b = torch.rand(70) + 0.5, torch.randn(70)
    sx = ops.rowsq_sum(out.to(dev), 70, w.to(dev), b.to(dev))
    sg = ops.scale_rows(ops.rowsq_sum(g4.to(dev), 70), prob.to(dev), False)
    wc, bc = ops.bn_diag_combine(sx, sg, 8.0, True)
    ref = O.fisher_bn_diag(O.bn_restore_input(out.double(), w.double(), b.double()), g4, prob, True, D)
    assert O.rel_fro(wc, ref[0]) < TOL and O.rel_fro(bc, ref[1]) < TOL
    # diagonal Fisher of Linear / Conv2d: sqrt(prob) on the output gradient, then the Cov kernels
    a = torch.randn(n, 50)
    prob = torch.rand(n)
    pg = ops.scale_rows(g.to(dev), prob.to(dev), True)
    dw, db = ops.diag_cov_linear(pg, a.to(dev), True, float(n))
    ref = O.diag_cov_linear(a, g, True, prob, D)
    assert O.rel_fro(dw, ref[0]) < TOL and O.rel_fro(db, ref[1]) < TOL
    x4 = torch.randn(8, 6, 7, 8)
    prob = torch.rand(8)
    pg = ops.scale_rows(g4.to(dev), prob.to(dev), True)
    dw = ops.diag_cov_conv2d(pg, x4.to(dev), (3, 3), (1, 1), (0, 0), (1, 1), 8.0)
    ref = O.diag_cov_conv2d(x4, g4, (3, 3), (1, 1), (0, 0), (1, 1), False, prob, D)[0]
    assert O.rel_fro(dw.reshape(ref.shape), ref) < TOL


def test_factor_input_above_one_gib_is_consumed_in_slices(ops, dev):
    """1.2 GB of rows: the entry point walks them in slices of at most 1 GiB that
    accumulate into the factor; checked by linearity against two half-size calls."""
    rows, f = 300000, 1024
    g = torch.Generator(device='cpu').manual_seed(3)
    x = torch.randn(rows, f, generator=g).to(dev)
    full = ops.factor_linear(x, True, 1.0 / rows)
    half = rows // 2
    a = ops.factor_linear(x[:half].contiguous(), True, 1.0 / rows)
    b = ops.factor_linear(x[half:].contiguous(), True, 1.0 / rows)
    assert O.rel_fro(full, a.double() + b.double()) < 1e-5
    assert abs(full[-1, -1].item() - 1.0) < 1e-5
