"""The side streams of the Kronecker factor products (torchsso._lanes): the results
are the same bits with and without them, and a reader of factor data right after
backward() sees the finished factors although the kernels run on other streams."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import bench
import kfac_testlib as T
import torchsso
from oracle import kfac_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def restore_stream_count():
    before = torchsso.factor_streams()
    yield
    torchsso.set_factor_streams(before)


def layer_set_state(count, specs, steps=3):
    torchsso.set_factor_streams(count)
    ls = bench.LayerSet(specs, 32, torch.device('cuda:0'), seed=3)
    for _ in range(steps):
        ls.step()
    torch.cuda.synchronize()
    out = [p.detach().clone() for p in ls.model.parameters()]
    for c in ls.curvs:
        out += [t.clone() for t in c.ema] + [t.clone() for t in c.inv]
    return out


@pytest.mark.parametrize('count', [1, 2, 3, 5])
def test_layer_set_step_is_bit_identical_with_side_streams(count):
    assert torchsso.factor_streams() == 2          # the default
    base = layer_set_state(0, bench.convnet_specs())
    got = layer_set_state(count, bench.convnet_specs())
    assert len(base) == len(got)
    for i, (a, b) in enumerate(zip(base, got)):
        assert torch.equal(a, b), 'tensor %d differs with %d streams' % (i, count)


def test_curvature_phase_on_two_streams_gives_the_same_step():
    """A layer with a factor of 2048 rows or more sends the layers whose factors are at
    most half as large to a side stream for their inversion and preconditioning
    (curvature.step_and_precondition_all).  Same parameters, running averages and
    inverses as on one stream: the running averages bit for bit, the rest to rounding
    (how a batched call groups its panel updates and cuts its reductions depends on the
    largest matrix of the call, so the order of the sums changes with the list)."""
    from torchsso.curv import curvature as C
    specs = [dict(kind='linear', name='wide', fin=2100, fout=300, bias=True),
             dict(kind='linear', name='mid', fin=900, fout=260, bias=True),
             bench.conv_spec('conv', 16, 32, 3, 1, 1, 12, bias=False),
             dict(kind='bn', name='bn', c=32, h=12),
             dict(kind='linear', name='small', fin=120, fout=10, bias=False)]
    before = C.two_stream_min_dim
    try:
        C.two_stream_min_dim = 2048
        ls = bench.LayerSet(specs, 32, torch.device('cuda:0'), seed=3)
        pairs = [(g['curv'], g['params']) for g in ls.opt.param_groups]
        late, early = C._chain_split(pairs)          # (two classes)
        assert [c.module.in_features for c, _ in late] == [2100] and len(early) == 4
        del ls
        two = layer_set_state(2, specs)
        C.two_stream_min_dim = None
        one = layer_set_state(2, specs)
    finally:
        C.two_stream_min_dim = before
    assert len(one) == len(two)
    worst = 0.
    for i, (a, b) in enumerate(zip(one, two)):
        err = ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30)).item()
        worst = max(worst, err)
        assert err <= 1e-4, 'tensor %d: one vs two curvature streams differ by %.3g' % (i, err)
    print('one vs two curvature streams: worst relative difference %.3g' % worst)
    n_params = sum(1 for _ in bench.LayerSet(specs, 32, torch.device('cuda:0')).model.parameters())
    k = n_params
    for c_specs in specs:                 # per curvature: ema tensors, then inverses
        n = 2
        for j in range(n):
            assert torch.equal(one[k + j], two[k + j]), 'running average %d differs' % (k + j)
        k += 2 * n


class Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.c1 = nn.Conv2d(16, 64, 3, padding=1)
        self.c2 = nn.Conv2d(64, 64, 3, padding=1, bias=False)
        self.c3 = nn.Conv2d(64, 128, 1, stride=2)
        self.fc = nn.Linear(128, 10)

    def forward(self, x):
        x = F.relu(self.c1(x))
        x = F.relu(self.c2(x))
        x = F.relu(self.c3(x))
        return self.fc(x.mean(dim=(2, 3)))


def test_factors_read_right_after_backward_are_complete():
    """56x56 inputs at batch 32: the factor kernels of the last hooks are still running
    when backward() returns.  `curv.data` must wait for them, and the memory of the
    output gradients (freed by autograd as soon as the hook returns) must not be handed
    out again under the kernels: fresh tensors are allocated and filled at once."""
    torch.manual_seed(0)
    dev = torch.device('cuda:0')
    model = Net().to(dev)
    opt = torchsso.optim.SecondOrderOptimizer(
        model, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron'}, {'damping': 1e-3, 'ema_decay': 1.},
        lr=1e-2)
    for g in opt.param_groups:
        g['curv'].fuse_ema = False
    x = torch.randn(32, 16, 56, 56, device=dev)
    y = torch.randint(0, 10, (32,), device=dev)
    model.zero_grad()
    loss = F.cross_entropy(model(x), y)
    loss.backward()
    junk = [torch.full((32, 64, 56, 56), float('nan'), device=dev) for _ in range(4)]
    got = {}
    for g in opt.param_groups:
        c = g['curv']
        got[c.module] = [t.clone() for t in c.data]
    torch.cuda.synchronize()
    del junk
    for mod, (A, G) in got.items():
        rec = {'input': mod.data_input.cpu(), 'grad_output': mod.grad_output.cpu()}
        _, (refA, refG) = T.oracle_factors(mod, rec, torch.float64)
        for name, mine, ref in (('A', A, refA), ('G', G, refG)):
            err = O.rel_fro(mine, ref)
            assert err < 1e-4, (type(mod).__name__, name, err)


def test_training_steps_match_single_stream_run():
    """Three optimizer steps of an autograd model, side streams against none.  The K-FAC
    kernels give the same bits either way (test above); the network's own backward
    kernels (MIOpen convolutions) are asked to be deterministic but are not bit-stable
    across runs on this stack, so the parameters and running averages are compared to
    1e-6 relative Frobenius, far below anything a misordered stream would leave."""
    dev = torch.device('cuda:0')
    det = torch.backends.cudnn.deterministic
    torch.backends.cudnn.deterministic = True
    try:
        runs = []
        for count in (0, 3):
            torchsso.set_factor_streams(count)
            torch.manual_seed(1)
            model = Net().to(dev)
            opt = torchsso.optim.SecondOrderOptimizer(
                model, 'Cov', {'Conv2d': 'Kron', 'Linear': 'Kron'},
                {'damping': 1e-3, 'ema_decay': 0.9}, lr=1e-2, momentum=0.9)
            gen = torch.Generator(device='cpu').manual_seed(5)
            for _ in range(3):
                x = torch.randn(16, 16, 28, 28, generator=gen).to(dev)
                y = torch.randint(0, 10, (16,), generator=gen).to(dev)

                def closure():
                    opt.zero_grad()
                    out = model(x)
                    loss = F.cross_entropy(out, y)
                    loss.backward()
                    return loss, out
                opt.step(closure=closure)
            torch.cuda.synchronize()
            runs.append([p.detach().clone() for p in model.parameters()]
                        + [t.clone() for g in opt.param_groups for t in g['curv'].ema])
        noise = max(((a - b).norm() / b.norm()).item() for a, b in zip(*runs))
        assert noise < 1e-6, noise
    finally:
        torch.backends.cudnn.deterministic = det


def test_stream_count_is_validated():
    with pytest.raises(ValueError):
        torchsso.set_factor_streams(-1)
    with pytest.raises(ValueError):
        torchsso.set_factor_streams(9)
