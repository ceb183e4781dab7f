"""Per-iteration learning-rate schedules for the torchsso optimizers.

Host-side glue with the interface of torchsso/optim/lr_scheduler.py of the
reference: schedulers are stepped once per optimizer iteration (not per epoch),
`state_dict()` holds every attribute but the optimizer, and
`MomentumCorrectionLR` rescales momentum by lr / previous lr whenever the
learning rate moves (reference: lr_scheduler.py:4-138).
"""
from torch.optim import Optimizer


class _IterLRScheduler(object):
    """Base class: `get_lr()` maps `self.last_iter` to one rate per param group
    (reference: lr_scheduler.py:4-48)."""

    scheduler_type = 'iter'

    def __init__(self, optimizer, last_iter=-1):
        if not isinstance(optimizer, Optimizer):
            raise TypeError('{} is not an Optimizer'.format(type(optimizer).__name__))
        self.optimizer = optimizer
        fresh = last_iter == -1
        for i, group in enumerate(optimizer.param_groups):
            if fresh:
                group.setdefault('initial_lr', group['lr'])
            elif 'initial_lr' not in group:
                raise KeyError("param 'initial_lr' is not specified "
                               "in param_groups[{}] when resuming an optimizer".format(i))
        self.base_lrs = [group['initial_lr'] for group in optimizer.param_groups]
        self.step(last_iter + 1)
        # as in the reference, the counter is put back after this first evaluation,
        # so that the first call of step() evaluates the same iteration again
        self.last_iter = last_iter
        self.scheduler_type = 'iter'

    def state_dict(self):
        return {k: v for k, v in self.__dict__.items() if k != 'optimizer'}

    def load_state_dict(self, state_dict):
        self.__dict__.update(state_dict)

    def get_lr(self):
        raise NotImplementedError

    def _current(self):
        return [group['lr'] for group in self.optimizer.param_groups]

    def step(self, iter=None):
        self.last_iter = self.last_iter + 1 if iter is None else iter
        for group, lr in zip(self.optimizer.param_groups, self.get_lr()):
            group['lr'] = lr


def polynomial_decay(base_lr, t, rate, max_count, start_iter=0, target=None):
    """base_lr * max(1 - (t - start) / (max_count - start), 0) ** rate, stopped at `target`
    when one is given: a decaying schedule (rate > 0) stops at it from above, a growing one
    (rate <= 0) from below.  Only defined from `start_iter` on."""
    remaining = max(1 - (t - start_iter) / (max_count - start_iter), 0)
    lr = base_lr * remaining ** rate
    if target is None:
        return lr
    # (the comparison is made on the quotient, as the reference makes it: a schedule with a
    # target that decays all the way to 0 raises ZeroDivisionError there too)
    quotient = target / lr
    passed = quotient > 1 if rate > 0 else quotient < 1
    return target if passed else lr


def linear_warmup(base_lr, t, initial_lr, max_count):
    """Point t / max_count of the way from `initial_lr` to `base_lr`."""
    alpha = t / max_count
    return initial_lr * (1 - alpha) + base_lr * alpha


class _FunctionOfIteration(_IterLRScheduler):
    """A schedule given as a function of (base rate, iteration), active on a range of
    iterations; outside of it the groups keep the rates they have."""

    def active(self, t):
        return True

    def rate_at(self, base_lr, t):
        raise NotImplementedError

    def get_lr(self):
        t = self.last_iter
        if not self.active(t):
            return self._current()
        return [self.rate_at(base, t) for base in self.base_lrs]


class PolynomialDecayIterLR(_FunctionOfIteration):
    """Polynomial decay from iteration `start_iter` on (reference: lr_scheduler.py:51-85)."""

    def __init__(self, optimizer, rate, max_count, target=None, start_iter=0, last_iter=-1):
        self.rate, self.max_count, self.target, self.start_iter = rate, max_count, target, start_iter
        super(PolynomialDecayIterLR, self).__init__(optimizer, last_iter)

    def active(self, t):
        return t >= self.start_iter

    def rate_at(self, base_lr, t):
        return polynomial_decay(base_lr, t, self.rate, self.max_count, self.start_iter, self.target)


class GradualWarmupIterLR(_FunctionOfIteration):
    """Linear ramp from `initial_lr` to the group's own rate over `max_count`
    iterations; unchanged afterwards (reference: lr_scheduler.py:88-108)."""

    def __init__(self, optimizer, initial_lr, max_count, last_iter=-1):
        self.initial_lr, self.max_count = initial_lr, max_count
        super(GradualWarmupIterLR, self).__init__(optimizer, last_iter)

    def active(self, t):
        return t <= self.max_count

    def rate_at(self, base_lr, t):
        return linear_warmup(base_lr, t, self.initial_lr, self.max_count)


class MomentumCorrectionLR(object):
    """Wraps a scheduler; after each step sets momentum = init_momentum * lr / lr_pre
    per group, lr_pre being the rate of the previous step (reference:
    lr_scheduler.py:111-138).  Every other attribute is the wrapped scheduler's."""

    def __init__(self, scheduler):
        object.__setattr__(self, 'scheduler', scheduler)
        for group in self.optimizer.param_groups:
            group['init_momentum'] = group['momentum']

    def step(self, count=None):
        self.scheduler.step(count)
        for group in self.optimizer.param_groups:
            previous = group.get('lr_pre', None)
            if previous is not None:
                group['momentum'] = group.get('init_momentum', 0) * group['lr'] / previous
            group['lr_pre'] = group['lr']

    def __getattr__(self, item):
        return getattr(self.scheduler, item)

    def __setattr__(self, key, value):
        setattr(self.scheduler, key, value)
