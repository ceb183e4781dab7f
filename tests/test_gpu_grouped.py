"""kfac_factor_grouped (the factor products of many layers in one engine call) against the
float64 oracle and against the single-product entry points, through the C ABI; and the
grouped mode of the hooks (products queued, run by the first reader) against the eager one."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

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


def spd(n, seed=0):
    g = torch.Generator().manual_seed(seed + n)
    x = torch.randn(2 * n + 8, n, dtype=D, generator=g)
    return ((x.t() @ x) / x.shape[0]).float()


# (kind, input shape, geometry (k, s, p, d) or None, bias)
CASES = [
    ('linear', (128, 784), None, True),
    ('linear', (37, 129), None, False),
    ('linear', (20000, 200), None, True),          # small factor, long reduction: many k-splits
    ('linear', (256, 2048), None, True),
    ('linear', (1, 1), None, True),
    ('conv_a', (4, 3, 32, 32), ((5, 5), (1, 1), (0, 0), (1, 1)), True),     # im2col
    ('conv_a', (3, 5, 9, 11), ((3, 3), (2, 2), (1, 1), (1, 1)), False),     # strided im2col
    ('conv_a', (16, 32, 28, 28), ((3, 3), (2, 2), (1, 1), (1, 1)), False),  # strided, 128-wide tiles
    ('conv_a', (2, 3, 30, 30), ((7, 7), (2, 2), (3, 3), (1, 1)), False),
    ('conv_a', (4, 48, 8, 8), ((1, 1), (1, 1), (0, 0), (1, 1)), False),     # pointwise: dense read
    ('conv_a', (3, 300, 7, 7), ((1, 1), (1, 1), (0, 0), (1, 1)), False),
    ('conv_a', (3, 20, 8, 8), ((1, 1), (2, 2), (0, 0), (1, 1)), False),     # pointwise with stride
    ('conv_a', (3, 6, 13, 10), ((3, 2), (3, 2), (2, 1), (1, 1)), True),     # strides that differ per axis
    ('conv_a', (2, 7, 12, 12), ((3, 3), (2, 2), (2, 2), (2, 2)), False),    # dilation = stride: one row phase read
    ('conv_a', (2, 5, 15, 14), ((3, 3), (2, 3), (0, 1), (3, 2)), True),     # dilated and strided
    ('conv_a', (3, 4, 17, 17), ((2, 2), (5, 5), (1, 1), (1, 1)), False),    # stride larger than the kernel
    ('conv_a', (3, 4, 17, 17), ((2, 7), (5, 1), (1, 3), (1, 1)), False),    # 35 planes: im2col with bounds tests instead
    ('conv_a', (4, 40, 10, 10), ((5, 5), (1, 1), (2, 2), (1, 1)), True),    # stride 1, padded copy, 128-wide tiles
    ('conv_a', (1, 1, 5, 5), ((3, 3), (2, 2), (1, 1), (1, 1)), True),       # one sample, one channel
    ('conv_a', (2, 3, 4, 9), ((4, 3), (1, 3), (0, 0), (1, 1)), False),      # one output row
    ('conv_a', (3, 2, 8, 3), ((2, 3), (2, 2), (0, 0), (1, 1)), True),       # one output column
    ('conv_a', (2, 2, 3, 3), ((5, 5), (1, 1), (2, 2), (1, 1)), True),       # kernel larger than the image
    ('conv_a', (5, 8, 6, 1), ((3, 1), (2, 1), (1, 0), (1, 1)), False),      # images one pixel wide
    ('conv_a', (8, 64, 14, 14), ((3, 3), (1, 1), (1, 1), (1, 1)), False),   # correlation kernels
    ('conv_a', (4, 256, 14, 14), ((3, 3), (1, 1), (1, 1), (1, 1)), False),
    ('conv_g', (16, 64, 56, 56), None, False),      # one 64-wide tile, very long reduction
    ('conv_g', (4, 130, 14, 14), None, False),
    ('conv_g', (32, 1024, 14, 14), None, False),    # few k-splits over many tiles
    ('conv_g', (32, 2048, 7, 7), None, False),      # no split
    ('conv_g', (24, 100, 30, 31), None, False),
    ('conv_g', (3, 257, 5, 3), None, False),
    ('conv_g', (1, 1, 1, 1), None, False),
]


def oracle_factor(kind, x, geo, bias):
    """(reference factor in float64, alpha that makes the kernel produce it)"""
    n = x.shape[0]
    if kind == 'linear':
        return O.factor_linear_a(x, bias, D), 1.0 / n
    if kind == 'conv_a':
        return O.factor_conv_a(x, *geo, bias, D), 1.0 / n
    return O.factor_conv_g(x, D), float(n) / (x.shape[2] * x.shape[3])


def make_job(ops, kind, xd, alpha, out, geo, bias, beta=0., prev=None):
    kw = {}
    if kind == 'conv_a':
        kw = dict(kernel_size=geo[0], stride=geo[1], padding=geo[2], dilation=geo[3])
    return ops.factor_job(kind, xd, alpha, out, beta=beta, prev=prev, add_bias=bias, **kw)


def single(ops, kind, xd, alpha, geo, bias, **kw):
    if kind == 'linear':
        return ops.factor_linear(xd, bias, alpha, **kw)
    if kind == 'conv_a':
        return ops.factor_conv_a(xd, geo[0], geo[1], geo[2], geo[3], bias, alpha, **kw)
    return ops.factor_conv_g(xd, alpha, **kw)


def test_grouped_against_oracle_and_single_products(ops, dev):
    """All cases in ONE call: plain products, running averages in place and into a second
    buffer; every result within 1e-4 of float64, symmetric to the bit, within rounding of the
    single-product entry point, and the same bits when the call is repeated."""
    torch.manual_seed(0)
    xs, refs, alphas = [], [], []
    for kind, shape, geo, bias in CASES:
        x = torch.randn(*shape)
        ref, alpha = oracle_factor(kind, x, geo, bias)
        xs.append(x.to(dev))
        refs.append(ref)
        alphas.append(alpha)

    def run(variant):
        outs, jobs, keep, want = [], [], [], []
        for (kind, shape, geo, bias), xd, ref, alpha in zip(CASES, xs, refs, alphas):
            d = ref.shape[0]
            if variant == 'plain':
                out = torch.full((d, d), float('nan'), device=dev)
                jobs.append(make_job(ops, kind, xd, alpha, out, geo, bias))
                want.append(ref)
            else:
                old = spd(d)
                want.append(0.9 * ref + 0.1 * old.double())
                if variant == 'in_place':
                    out = old.to(dev).clone()
                    jobs.append(make_job(ops, kind, xd, 0.9 * alpha, out, geo, bias, beta=0.1))
                else:
                    prev = old.to(dev).clone()
                    out = torch.full((d, d), float('nan'), device=dev)
                    jobs.append(make_job(ops, kind, xd, 0.9 * alpha, out, geo, bias, beta=0.1,
                                         prev=prev))
                    keep.append((prev, old))
            outs.append(out)
        ops.factor_grouped(jobs, dev)
        for prev, old in keep:
            assert torch.equal(prev.cpu(), old)       # the previous average stays untouched
        return outs, want

    worst = 0.
    for variant in ('plain', 'in_place', 'second_buffer'):
        outs, want = run(variant)
        for (kind, shape, geo, bias), out, ref in zip(CASES, outs, want):
            err = O.rel_fro(out, ref)
            worst = max(worst, err)
            assert err < TOL, (variant, kind, shape, err)
            assert torch.equal(out, out.t()), (variant, kind, shape)
    print('grouped factor products: worst rel. Frobenius error vs float64 %.2e' % worst)

    outs, _ = run('plain')
    again, _ = run('plain')
    for (kind, shape, geo, bias), xd, alpha, a, b in zip(CASES, xs, alphas, outs, again):
        assert torch.equal(a, b), (kind, shape)
        one = single(ops, kind, xd, alpha, geo, bias)
        assert O.rel_fro(a, one.double().cpu()) < 2e-6, (kind, shape)


def test_grouped_rejects_bad_lists(ops, dev):
    from torchsso import _hip
    x = torch.randn(8, 5, device=dev)
    out = torch.empty(5, 5, device=dev)
    j1 = ops.factor_job('linear', x, 1., out)
    j2 = ops.factor_job('linear', x, 2., out)
    with pytest.raises(_hip.KfacHipError):
        ops.factor_grouped([j1, j2], dev)             # two products into one buffer
    with pytest.raises(_hip.KfacHipError):
        ops.factor_job('linear', x, 1., torch.empty(6, 6, device=dev))
    with pytest.raises(_hip.KfacHipError):
        ops.factor_job('conv_g', x, 1., out)
    ops.factor_grouped([], dev)


class Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(3, 16, 3, padding=1)
        self.b1 = nn.BatchNorm2d(16)
        self.c2 = nn.Conv2d(16, 32, 3, padding=1, bias=False)
        self.c3 = nn.Conv2d(32, 32, 1, bias=False)
        self.c4 = nn.Conv2d(32, 24, 3, stride=2, padding=1)
        self.fc = nn.Linear(24 * 4 * 4, 10)

    def forward(self, x):
        x = F.relu(self.b1(self.c1(x)), inplace=True)
        x = F.relu(self.c2(x))
        x = x + self.c3(x)
        x = F.relu(self.c4(x))
        return self.fc(x.flatten(1))


def train(mode, steps=3):
    import torchsso
    before = torchsso.factor_mode()
    torchsso.set_factor_mode(mode)
    try:
        dev = torch.device('cuda:0')
        torch.manual_seed(3)
        model = Net().to(dev)
        opt = torchsso.optim.SecondOrderOptimizer(
            model, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron', 'BatchNorm2d': 'Diag'},
            {'damping': 1e-3, 'ema_decay': 0.95}, lr=0.01, momentum=0.9)
        x = torch.randn(16, 3, 8, 8, device=dev)
        y = torch.randint(0, 10, (16,), device=dev)
        mid = None
        for s in range(steps):
            def closure():
                model.zero_grad()
                loss = F.cross_entropy(model(x), y)
                loss.backward()
                return loss
            if s == steps - 1:
                # read the raw factors between backward and step: the queue runs here
                closure()
                mid = [t.clone() for g in opt.param_groups if g['curv'].kind == 'kron'
                       for t in g['curv'].data]
                opt.step()
            else:
                opt.step(closure=closure)
        torch.cuda.synchronize()
        return ([p.detach().clone() for p in model.parameters()],
                [t.clone() for g in opt.param_groups if g['curv'].kind == 'kron'
                 for t in g['curv'].ema], mid)
    finally:
        torchsso.set_factor_mode(before)


def test_grouped_mode_of_the_hooks_matches_eager_mode():
    import torchsso
    assert torchsso.factor_mode() == 'grouped'        # the default
    pe, ee, me = train('eager')
    pg, eg, mg = train('grouped')
    for a, b in zip(ee, eg):
        assert O.rel_fro(b, a.double().cpu()) < 1e-5
    for a, b in zip(me, mg):
        assert O.rel_fro(b, a.double().cpu()) < 1e-5
    for a, b in zip(pe, pg):
        assert O.rel_fro(b, a.double().cpu()) < 1e-4
    with pytest.raises(ValueError):
        torchsso.set_factor_mode('lazy')


def test_second_pass_before_a_read_runs_the_queue():
    """Two forward passes without a reader in between (evaluation with the hooks attached):
    the second product of a factor runs the queue first, so no more than one pass of
    inputs is ever kept alive, and the factor read afterwards is the one of the last pass."""
    import torchsso
    from torchsso import _lanes
    dev = torch.device('cuda:0')
    torch.manual_seed(5)
    lin = nn.Linear(6, 4).to(dev)
    curv = torchsso.KronCovLinear(lin, ema_decay=1.)
    x1, x2 = torch.randn(9, 6, device=dev), torch.randn(9, 6, device=dev)
    lin(x1)
    assert _lanes.deferred_count() == 1
    lin(x2)
    assert _lanes.deferred_count() == 1
    assert O.rel_fro(curv.A, O.factor_linear_a(x2.cpu(), True, D)) < TOL
    assert _lanes.deferred_count() == 0


def vi_run(mode, steps=3):
    import torchsso
    before = torchsso.factor_mode()
    torchsso.set_factor_mode(mode)
    try:
        dev = torch.device('cuda:0')
        torch.manual_seed(7)
        model = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(), nn.MaxPool2d(2),
                              nn.Conv2d(8, 16, 3), nn.ReLU(), nn.Flatten(),
                              nn.Linear(16 * 2 * 2, 10)).to(dev)
        x = torch.randn(12, 3, 8, 8, device=dev)
        y = torch.randint(0, 10, (12,), device=dev)
        opt = torchsso.optim.VIOptimizer(
            model, 1000, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron'},
            {'damping': 1e-3, 'ema_decay': 0.9}, lr=1e-2, momentum=0.9, num_mc_samples=3,
            prior_variance=1, kl_weighting=1, seed=3)
        seen = []

        def closure():
            model.zero_grad()
            out = model(x)
            loss = F.cross_entropy(out, y)
            loss.backward()
            return loss, out
        for _ in range(steps):
            opt.step(closure=closure)
            seen.append([t.clone() for g in opt.param_groups for t in g['curv'].ema])
        torch.cuda.synchronize()
        return [p.detach().clone() for p in model.parameters()], seen
    finally:
        torchsso.set_factor_mode(before)


def test_mc_loop_accumulates_in_the_factor_products():
    """VIOptimizer: the factors of the MC samples are added up in the epilogue of the factor
    products (nothing waits for them between the samples).  Same running averages and
    parameters in grouped and in eager mode over three steps with posterior sampling, and
    the running average after the first step is the mean over the samples of the factors an
    independent pass computes (float64 oracle)."""
    pg, eg = vi_run('grouped')
    pe, ee = vi_run('eager')
    for step, (a, b) in enumerate(zip(ee, eg)):
        for t_e, t_g in zip(a, b):
            assert O.rel_fro(t_g, t_e.double().cpu()) < 2e-5, step
    for a, b in zip(pe, pg):
        assert O.rel_fro(b, a.double().cpu()) < 1e-4
    # first step: no posterior yet, every MC sample sees the same parameters, so the mean
    # over the samples is the factor of one pass
    torch.manual_seed(7)
    model = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(), nn.MaxPool2d(2),
                          nn.Conv2d(8, 16, 3), nn.ReLU(), nn.Flatten(), nn.Linear(16 * 2 * 2, 10))
    x = torch.randn(12, 3, 8, 8, device='cuda:0').cpu()
    A0 = O.factor_conv_a(x, (3, 3), (1, 1), (1, 1), (1, 1), True, D)
    assert O.rel_fro(eg[0][0], A0) < TOL


def test_queue_runs_on_a_work_threshold_and_across_streams():
    """The queue also runs when the collected work passes the threshold (here: every product
    by itself), and products queued under another stream than the one that reads the factors
    wait for that stream's work: same factors as the eager mode either way."""
    import torchsso
    from torchsso import _lanes
    dev = torch.device('cuda:0')
    before = _lanes.flush_work()

    def factors(mode, work, side_stream):
        torchsso.set_factor_mode(mode)
        torchsso.set_factor_flush_work(work)
        torch.manual_seed(11)
        conv = nn.Conv2d(6, 10, 3, padding=1).to(dev)
        lin = nn.Linear(10 * 8 * 8, 7).to(dev)
        cc = torchsso.KronCovConv2d(conv, ema_decay=1.)
        cl = torchsso.KronCovLinear(lin, ema_decay=1.)
        x = torch.randn(16, 6, 8, 8, device=dev)
        torch.cuda.synchronize()
        if side_stream:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                # a slow producer in front of the layers: the products must wait for it
                big = torch.randn(4096, 4096, device=dev)
                for _ in range(6):
                    big = big @ big * 1e-3
                x2 = x + big[:1, :1].reshape(1, 1, 1, 1) * 0
                out = lin(conv(x2).flatten(1))
                out.sum().backward()
        else:
            out = lin(conv(x).flatten(1))
            out.sum().backward()
        res = [cc.A.clone(), cc.G.clone(), cl.A.clone(), cl.G.clone()]     # read on the default stream
        torch.cuda.synchronize()
        return res
    try:
        ref = factors('eager', before, False)
        for work, side in ((1., False), (None, False), (before, True), (1., True)):
            got = factors('grouped', work, side)
            for a, b in zip(ref, got):
                assert torch.isfinite(b).all()
                assert O.rel_fro(b, a.double().cpu()) < 1e-5, (work, side)
        assert _lanes.deferred_count() == 0
    finally:
        torchsso.set_factor_mode('grouped')
        torchsso.set_factor_flush_work(before)
