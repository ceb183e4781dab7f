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


class PolynomialDecayIterLR(_IterLRScheduler):
    """lr = initial_lr * max(1 - (t - start) / (max_count - start), 0) ** rate from
    iteration `start_iter` on, clipped at `target` when one is given
    (reference: lr_scheduler.py:51-85)."""

    def __init__(self, optimizer, rate, max_count, target=None, start_iter=0, last_iter=-1):
        self.rate = rate
        self.max_count = max_count
        self.target = target
        self.start_iter = start_iter
        super(PolynomialDecayIterLR, self).__init__(optimizer, last_iter)

    def get_lr(self):
        t = self.last_iter
        if t < self.start_iter:
            return self._current()
        span = self.max_count - self.start_iter
        decay = max(1 - (t - self.start_iter) / span, 0)
        lrs = []
        for base in self.base_lrs:
            lr = base * decay ** self.rate
            if self.target is not None:
                # a decaying schedule (rate > 0) stops at the target from above,
                # a growing one (rate <= 0) from below
                ratio = self.target / lr
                if (self.rate > 0 and ratio > 1) or (self.rate <= 0 and ratio < 1):
                    lr = self.target
            lrs.append(lr)
        return lrs


class GradualWarmupIterLR(_IterLRScheduler):
    """Linear ramp from `initial_lr` to the group's own rate over `max_count`
    iterations; unchanged afterwards (reference: lr_scheduler.py:88-108)."""

    def __init__(self, optimizer, initial_lr, max_count, last_iter=-1):
        self.initial_lr = initial_lr
        self.max_count = max_count
        super(GradualWarmupIterLR, self).__init__(optimizer, last_iter)

    def get_lr(self):
        if self.last_iter > self.max_count:
            return self._current()
        alpha = self.last_iter / self.max_count
        return [self.initial_lr * (1 - alpha) + base * alpha for base in self.base_lrs]


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
