"""Per-layer curvature state: data -> ema -> inv (-> std).

Host-side mirror of torchsso/curv/curvature.py of the reference (class names,
constructor arguments, attributes and error behaviour are the same); all
arithmetic runs in the HIP engine through torchsso._ops.  Differences in
mechanics, none in results:

* the per-layer methods (`step`, `update_ema`, `update_inv`, `update_std`,
  `precondition_grad`, `sample_params`) are thin wrappers over list-based
  functions at the bottom of this file (`step_all`, `precondition_all`,
  `sample_all`), which the optimizers call once for all layers so that every
  engine routine is launched once per step, not once per layer;
* `ema` is updated in place and `inv` / `std` buffers are reused from step to
  step (the reference allocates new tensors each time);
* the hooks queue the Kronecker factor products, and whoever reads factor data first has
  them all run in one grouped engine call on a side stream (torchsso._lanes; in eager mode
  every hook enqueues its own product on a side stream);
* the output gradient is taken with a tensor hook on the module output instead
  of the deprecated module backward hook (same tensor, and it also works with
  an in-place activation after the module).
"""
import math

import torch
import torch.nn as nn

from torchsso import _lanes, _ops

PI_TYPE_TRACENORM = 'tracenorm'


class Curvature(object):
    """Base class (reference: curvature.py:10-212)."""

    def __init__(self, module: nn.Module, ema_decay=1., damping=1e-7,
                 use_max_ema=False, use_sqrt_ema=False,
                 pi_type=PI_TYPE_TRACENORM):

        if ema_decay < 0 or 1 < ema_decay:
            raise ValueError("Invalid ema_decay: {}".format(ema_decay))
        if damping < 0:
            raise ValueError("Invalid damping: {}".format(damping))
        if pi_type not in [PI_TYPE_TRACENORM]:
            raise ValueError("Invalid pi_type: {}".format(pi_type))

        self._module = module
        self.ema_decay = ema_decay
        self._damping = damping
        self._l2_reg = 0
        self._l2_reg_ema = 0

        self._data = None
        self._acc_data = None
        self.ema = None
        self.ema_max = None
        self.inv = None
        self.std = None
        self.info = None       # device int32 status of the last inversion (0 = ok)
        self.std_info = None   # same for the last Cholesky factorisation of the inverses

        self.use_sqrt_ema = use_sqrt_ema
        self.use_max_ema = use_max_ema

        self.pi_type = pi_type

        module.register_forward_hook(self.forward_postprocess)

    # ---- attributes the optimizers and users read -------------------------

    @property
    def data(self):
        return self._data

    @data.setter
    def data(self, value):
        self._data = value

    @property
    def shape(self):
        if self._data is None:
            return self._get_shape()
        return tuple([d.shape for d in self._data])

    @property
    def device(self):
        return next(self._module.parameters()).device

    def _get_shape(self):
        size = sum(p.numel() for p in self._module.parameters())
        return tuple((size, size))

    def element_wise_init(self, value):
        self._data = [torch.diag(torch.full((s[0],), float(value), device=self.device))
                      for s in self.shape]

    @property
    def module(self):
        return self._module

    @property
    def bias(self):
        return getattr(self._module, 'bias', None) is not None

    @property
    def damping(self):
        return self._damping + self._l2_reg_ema

    @property
    def l2_reg(self):
        return self._l2_reg

    @l2_reg.setter
    def l2_reg(self, value):
        self._l2_reg = value

    @property
    def l2_reg_ema(self):
        return self._l2_reg_ema

    # ---- hooks ---------------------------------------------------------------

    def forward_postprocess(self, module, input, output):
        """Forward hook (reference: curvature.py:118-139)."""
        assert self._module == module
        data_input = input[0].detach()
        setattr(module, 'data_input', data_input)
        setattr(module, 'data_output', output)
        self.update_in_forward(data_input)
        if isinstance(output, torch.Tensor) and output.requires_grad:
            output.register_hook(self._on_grad_output)

    def _on_grad_output(self, grad_output):
        self.backward_postprocess(self._module, None, (grad_output,))

    def backward_postprocess(self, module, grad_input, grad_output):
        """Reference: curvature.py:141-155.  `module.grad_input` is None here: the
        gradient arrives through a tensor hook on the module output, which sees no
        gradient with respect to the module input (nothing on the K-FAC path reads
        it; the reference's value comes from the legacy module hook and may be None
        as well)."""
        assert self._module == module
        grad_output = grad_output[0].detach()
        if grad_input is not None:
            index = 1 if self.bias else 0
            grad_input = None if grad_input[index] is None else grad_input[index].detach()
        setattr(module, 'grad_input', grad_input)
        setattr(module, 'grad_output', grad_output)
        self.update_in_backward(grad_output)

    def adjust_data_scale(self, scale):
        """Multiply the current data by `scale` (reference: curvature.py:157-158).
        The hooks do not call it: the batch-size^2 rescale of curvature.py:154-155
        is folded into the scale factor of the factor kernels."""
        self._data = [d.mul_(scale) for d in self._data]

    def update_in_forward(self, data_input):
        pass

    def update_in_backward(self, grad_output):
        raise NotImplementedError

    # ---- checkpointing --------------------------------------------------------

    _STATE_LISTS = ('ema', 'ema_max', 'inv', 'std')

    def state_dict(self):
        """The running state as tensors and numbers only: ema, ema_max, inv, std
        (lists of tensors or None) and the two l2 scalars.  (The reference has no
        such method: its optimizer checkpoint pickles the Curvature objects, hooks
        and module included.)"""
        _lanes.join()
        out = {'l2_reg': float(self._l2_reg), 'l2_reg_ema': float(self._l2_reg_ema)}
        for name in self._STATE_LISTS:
            val = getattr(self, name)
            out[name] = None if val is None else [t.detach().clone() for t in val]
        return out

    def load_state_dict(self, state):
        _lanes.join()
        device = self.device
        self._l2_reg = state['l2_reg']
        self._l2_reg_ema = state['l2_reg_ema']
        for name in self._STATE_LISTS:
            val = state.get(name)
            setattr(self, name, None if val is None
                    else [t.detach().to(device=device, dtype=torch.float32).clone() for t in val])

    # ---- per-layer step (wrappers over the list-based engine calls) --------

    def step(self, update_std=False, update_inv=True):
        step_all([self], update_std=update_std, update_inv=update_inv)

    def update_ema(self):
        update_ema_all([self])

    def update_inv(self):
        update_inv_all([self])

    def update_std(self):
        update_std_all([self])

    def precondition_grad(self, params):
        precondition_all([(self, params)])

    def sample_params(self, params, mean, std_scale):
        sample_all([(self, params, mean, std_scale)])

    def std_norm(self):
        raise NotImplementedError

    # ---- what the list-based functions need from a subclass ---------------

    kind = 'full'   # 'kron' | 'diag' | 'full'

    def _inv_one(self, X):
        """Curvature._inv of the reference (curvature.py:197-200)."""
        outs, self.info = _ops.damped_inverse_batched([X], [self.damping])
        return outs[0]


class DiagCurvature(Curvature):
    """Element-wise curvature (reference: curvature.py:215-252)."""

    kind = 'diag'

    def _get_shape(self):
        return tuple(p.shape for p in self.module.parameters())

    def element_wise_init(self, value):
        self._data = [torch.full(tuple(s), float(value), device=self.device) for s in self.shape]

    def std_norm(self):
        if self.std is None:
            return 0
        return sum(std.norm().item() for std in self.std)


class KronCurvature(Curvature):
    """Kronecker-factored curvature A (x) G (reference: curvature.py:255-331).

    With `fuse_ema` set (SecondOrderOptimizer does it when no accumulation over
    micro-steps needs the raw factors) the factor kernels write the running
    average themselves: a hook builds  ema_decay * factor + (1 - ema_decay) * ema
    into a second buffer (`_next`) in the epilogue of the factor product, and
    `update_ema` just swaps the two buffers.  The raw factor is then never
    stored; `data`, `A` and `G` rebuild it on demand from the two averages."""

    kind = 'kron'
    _lanes_dealt = 0

    # update_inv keeps the inverse of a factor with at least this many rows as its
    # upper-triangular factor Y (Y Y^T = inverse) and preconditioning applies Y twice
    # instead of the inverse once: the same work there, and the inversion is spared the
    # product that forms the explicit inverse, a third of its work.  Below this size that
    # product is negligible and a triangular operand only wastes tile space.  `inv` forms
    # a missing inverse on first access.  None: update_inv forms every inverse explicitly.
    factored_inverse_min_dim = 256

    def __init__(self, *args, **kwargs):
        self._inv = None
        self._inv_factors = [None, None]
        super(KronCurvature, self).__init__(*args, **kwargs)
        self._A = None
        self._G = None
        self.fuse_ema = False
        self._lane = KronCurvature._lanes_dealt   # the side stream its factor products use
        KronCurvature._lanes_dealt += 1
        self._next = [None, None]        # receives the next running average
        self._jobs = [None, None]        # grouped mode: (signature, engine job, d, work) per factor
        self._acc_into = None            # (TensorAccumulator, weight): see accumulate_into
        self._fresh = [False, False]     # _next[i] holds the next average (hook ran since the last step)
        self._prev_ok = [False, False]   # _next[i] holds the average before the current one

    # ---- inverses ---------------------------------------------------------------

    @property
    def inv(self):
        """[A_inv, G_inv] (reference: curvature.py:302-312).  An inverse that update_inv kept
        in factored form is formed here, on first access, as Y Y^T."""
        if self._inv is not None:
            for k, y in enumerate(self._inv_factors):
                if self._inv[k] is None and y is not None:
                    self._inv[k] = _ops.factor_linear(y.t().contiguous(), False, 1.)
        return self._inv

    @inv.setter
    def inv(self, value):
        self._inv = None if value is None else list(value)
        self._inv_factors = [None, None]      # inverses given from outside have no factors

    def _inverse_outputs(self, with_std):
        """Output buffers for one update_inv of this layer, None where that output is not
        wanted: ([A_inv, G_inv], [A_fac, G_fac], [A_std, G_std]).  A side is kept either as
        the inverse or as its factor; with a posterior std to deliver (std^T std = inverse,
        another factor than Y) every inverse is explicit."""
        min_dim = None if with_std else self.factored_inverse_min_dim
        old_inv = self._inv or [None, None]
        old_std = self.std or [None, None]
        invs, facs, stds = [None, None], [None, None], [None, None]

        def reuse(t, like):
            return t if t is not None and t.shape == like.shape else torch.empty_like(like)
        for k, e in enumerate(self.ema):
            if min_dim is not None and e.shape[0] >= min_dim:
                facs[k] = reuse(self._inv_factors[k], e)
            else:
                invs[k] = reuse(old_inv[k], e)
                if with_std:
                    stds[k] = reuse(old_std[k], e)
        self._inv = list(invs)
        self._inv_factors = list(facs)
        if with_std:
            self.std = list(stds)
        return invs, facs, stds

    # ---- raw factors ------------------------------------------------------------

    def accumulate_into(self, accumulator, weight):
        """Until `accumulator` is None again, the hooks add `weight` times each new factor to
        the buffers of `accumulator` (a TensorAccumulator of [A, G]) in the epilogue of the
        factor product itself, instead of storing the raw factor for somebody to add up
        afterwards (the accumulation over MC samples or micro-steps of
        optim/secondorder.py:175-182 and optim/vi.py:211-220 of the reference): no pass over
        the factors, and nothing has to wait for the products before the running sum is
        used.  `data`, `A` and `G` are None while this is on."""
        self._acc_into = None if accumulator is None else (accumulator, float(weight))

    def _build_factor(self, idx, source, kind, scale, add_bias=False, **geometry):
        """Builds factor `idx` (0: A, 1: G) as  scale * P^T P  from the contiguous tensor
        `source` (`kind`: 'linear', 'conv_a' with the convolution's geometry, 'conv_g'):
        the raw factor or, in fused mode, the next running average.  In grouped mode the
        product is only queued here and runs with all others when factor data is first read
        (torchsso._lanes); in eager mode it runs now, on this layer's side stream."""
        beta = self.ema_decay
        device = source.device
        fused = self.fuse_ema and self.ema is not None and beta != 1
        if fused:
            prev = self.ema[idx]
            out = self._next[idx]
            if out is None or out.shape != prev.shape:
                out = torch.empty_like(prev)
            alpha, b = beta * scale, 1. - beta
        elif self._acc_into is not None:
            accumulator, weight = self._acc_into
            d = self._factor_dim(idx, source, kind, add_bias, geometry)
            out, fresh = accumulator.slot(idx, 2, (d, d), source)
            prev = None
            alpha, b = scale * weight, 0. if fresh else 1.
        else:
            prev, out = None, None
            alpha, b = scale, 0.
        accumulating = not fused and self._acc_into is not None
        if _lanes.mode() == 'grouped' and device.type == 'cuda':
            # (the job object of this factor is reused from pass to pass: the engine copies
            # it when the queue runs, and a second product of a queued factor runs the queue)
            _lanes.flush_if_queued(device, (id(self), idx))
            sig = (kind, tuple(source.shape), add_bias, tuple(sorted(geometry.items())))
            cached = self._jobs[idx]
            if cached is None or cached[0] != sig:
                d = self._factor_dim(idx, source, kind, add_bias, geometry)
                if out is None:
                    out = torch.empty((d, d), dtype=torch.float32, device=device)
                job = _ops.factor_job(kind, source, alpha, out, beta=b, prev=prev,
                                      add_bias=add_bias, **geometry)     # (checks the shapes)
                if kind == 'conv_a':
                    terms = source.shape[0] * _ops.conv_output_positions(source, **geometry)
                else:
                    terms = source.numel() // source.shape[1]
                cached = self._jobs[idx] = (sig, job, d, float(d) * d * terms)
            _, job, d, work = cached
            if out is None:
                out = torch.empty((d, d), dtype=torch.float32, device=device)
            _ops.factor_job_update(job, source, alpha, out, b, prev)
            _lanes.defer(device, (id(self), idx), job, (source, prev, out), work, backward=idx == 1)
        else:
            lane = 2 * self._lane + idx    # A and G of a layer on different lanes, each always on its own
            if kind == 'linear':
                build = lambda st: _ops.factor_linear(source, add_bias, alpha, out=out, beta=b,
                                                      prev=prev, stream=st)
            elif kind == 'conv_a':
                build = lambda st: _ops.factor_conv_a(
                    source, geometry['kernel_size'], geometry['stride'], geometry['padding'],
                    geometry['dilation'], add_bias, alpha, out=out, beta=b, prev=prev, stream=st)
            else:
                build = lambda st: _ops.factor_conv_g(source, alpha, out=out, beta=b, prev=prev,
                                                      stream=st)
            out = _lanes.run(device, lane, (source, prev), build)
        if fused:
            self._next[idx] = out
            self._fresh[idx] = True
            self._prev_ok[idx] = False
            raw = None
        elif accumulating:
            raw = None
            self._fresh[idx] = False
            self._prev_ok[idx] = False
        else:
            raw = out
            self._fresh[idx] = False
        if idx == 0:
            self._A = raw
        else:
            self._G = raw

    @staticmethod
    def _factor_dim(idx, source, kind, add_bias, geometry):
        if kind == 'conv_a':
            kh, kw = _ops._pair(geometry['kernel_size'])
            return source.shape[1] * kh * kw + (1 if add_bias else 0)
        return source.shape[1] + (1 if add_bias else 0)

    def _raw(self, idx):
        _lanes.join()
        t = self._A if idx == 0 else self._G
        if t is None and self.ema is not None and (self._fresh[idx] or self._prev_ok[idx]):
            # factor = (newer average - (1 - beta) * older average) / beta
            beta = self.ema_decay
            newer, older = ((self._next[idx], self.ema[idx]) if self._fresh[idx]
                            else (self.ema[idx], self._next[idx]))
            t = newer.clone()
            _ops.axpby_batched([older], [t], -(1. - beta) / beta, 1. / beta)
        return t

    @property
    def data(self):
        return [self._raw(0), self._raw(1)]

    @data.setter
    def data(self, value):
        self._A, self._G = value
        self._fresh = [False, False]

    @property
    def shape(self):
        if self._A is None or self._G is None:
            return self._get_shape()
        return self._A.shape, self._G.shape

    def _advance_average(self, xs, ys, stale):
        """update_ema in fused mode.  Factors whose next average is ready: swap the
        buffers.  Factors built the ordinary way go to the (xs, ys) lists of the
        axpby launch.  A factor that no hook has rebuilt since the last step
        enters again, as in the reference, where `data` simply persists:
        beta * factor + (1 - beta) * ema  with  factor = (ema - (1 - beta) * prev) / beta
        is (2 - beta) * ema - (1 - beta) * prev, written over prev (`stale` list)."""
        for idx in (0, 1):
            raw = self._A if idx == 0 else self._G
            if self._fresh[idx]:
                self.ema[idx], self._next[idx] = self._next[idx], self.ema[idx]
                self._fresh[idx] = False
                self._prev_ok[idx] = True
            elif raw is not None:
                xs.append(raw.contiguous())
                ys.append(self.ema[idx])
                self._prev_ok[idx] = False
            elif self._prev_ok[idx]:
                stale.append((self, idx))
            else:
                raise RuntimeError('update_ema: no factor has been built for %s'
                                   % type(self._module).__name__)

    def load_state_dict(self, state):
        super(KronCurvature, self).load_state_dict(state)
        self._next = [None, None]
        self._fresh = [False, False]
        self._prev_ok = [False, False]

    def _get_shape(self):
        raise NotImplementedError

    def element_wise_init(self, value):
        # sqrt(value) on each factor so that A (x) G has `value` on its diagonal
        super(KronCurvature, self).element_wise_init(math.sqrt(value))
        self._A, self._G = self._data

    @property
    def A(self):
        return self._raw(0)

    @property
    def G(self):
        return self._raw(1)

    def adjust_data_scale(self, scale):
        _lanes.join()
        self._G.mul_(scale)

    def std_norm(self):
        if self.std is None:
            return 0
        A_ic, G_ic = self.std
        return A_ic.norm().item() * G_ic.norm().item()

    # the 2-D [dG, dA(-1)] view of the weight-shaped tensor of this layer
    def _weight2d(self, w):
        return w.reshape(w.shape[0], -1)


def add_value_to_diagonal(X, value):
    """X + value*I as a new tensor (reference: curvature.py:334-340, which builds
    a Python list of n index pairs; here one strided in-place add on a copy)."""
    out = X.clone()
    out.diagonal().add_(value)
    return out


# ---------------------------------------------------------------------------
# list-based engine calls
# ---------------------------------------------------------------------------

def update_ema_all(curvs):
    """Curvature.update_ema for every curvature in the list
    (reference: curvature.py:174-191).  ema_decay weighs the NEW data."""
    _lanes.join()
    by_beta = {}
    stale = []
    for c in curvs:
        beta = c.ema_decay
        if c.kind == 'kron' and c.fuse_ema and c.ema is not None and beta != 1:
            xs, ys = by_beta.setdefault(beta, ([], []))
            c._advance_average(xs, ys, stale)
            c._l2_reg_ema = c._l2_reg * beta + c._l2_reg_ema * (1 - beta)
            continue
        data = c.data
        if c.ema is None or beta == 1:
            if c.ema is None:
                c.ema = [d.clone() for d in data]
            else:
                for e, d in zip(c.ema, data):
                    e.copy_(d)
            if c.use_max_ema and c.ema_max is None:
                c.ema_max = [e.clone() for e in c.ema]
            c._l2_reg_ema = c._l2_reg
        else:
            xs, ys = by_beta.setdefault(beta, ([], []))
            xs.extend(d.contiguous() for d in data)
            ys.extend(c.ema)
            c._l2_reg_ema = c._l2_reg * beta + c._l2_reg_ema * (1 - beta)
    for beta, (xs, ys) in by_beta.items():
        _ops.axpby_batched(xs, ys, beta, 1 - beta)
    for c, idx in stale:
        beta = c.ema_decay
        _ops.axpby_batched([c.ema[idx]], [c._next[idx]], 2. - beta, -(1. - beta))
        c.ema[idx], c._next[idx] = c._next[idx], c.ema[idx]
    xs, ys = [], []
    for c in curvs:
        if c.use_max_ema:
            xs.extend(c.ema)
            ys.extend(c.ema_max)
    _ops.max_batched(xs, ys)


def update_inv_all(curvs, with_std=()):
    """update_inv for every curvature: one batched pi-damped inversion for all
    Kronecker layers (reference: curvature.py:302-312), one element-wise launch
    for all diagonal layers (curvature.py:193-195,226-232).

    `with_std`: curvatures whose `std` will be asked for right after (update_std,
    curvature.py:317-321).  For the Kronecker ones among them the inversion delivers the
    Cholesky factors of the inverses as well (the engine factors those matrices back to
    front and reads the factor off the triangular inverse), so that update_std_all has
    nothing left to compute for them."""
    kron = [c for c in curvs if c.kind == 'kron']
    diag = [c for c in curvs if c.kind == 'diag']
    full = [c for c in curvs if c.kind == 'full']
    wanted = {id(c) for c in with_std}
    if kron:
        outs = [c._inverse_outputs(id(c) in wanted) for c in kron]
        column = lambda which, k: [o[which][k] for o in outs]
        args = ([c.ema[0] for c in kron], [c.ema[1] for c in kron], [c.damping for c in kron])
        if any(f is not None for _, facs, _ in outs for f in facs):
            # (a layer with a std to deliver has no factored side, but others may: its std
            # then takes a launch of its own below)
            info = _ops.pi_damped_inverse_factored_batched(*args, column(0, 0), column(0, 1),
                                                           column(1, 0), column(1, 1))
            for c in kron:
                c._info_reversed = False
                if id(c) in wanted:
                    c._std_current = False
        elif wanted:
            info = _ops.pi_damped_inverse_std_batched(*args, column(0, 0), column(0, 1),
                                                      column(2, 0), column(2, 1))
            for c in kron:
                if id(c) in wanted:
                    c._std_current = True      # update_std_all has nothing to do for it
                    c.std_info = None          # (a failure shows in `info`)
            for c in kron:
                c._info_reversed = id(c) in wanted
        else:
            _, _, info = _ops.pi_damped_inverse_batched(*args, column(0, 0), column(0, 1))
            for c in kron:
                c._info_reversed = False
        for i, c in enumerate(kron):
            c.info = info[2 * i:2 * i + 2]
    if diag:
        by_sqrt = {False: ([], [], []), True: ([], [], [])}
        for c in diag:
            ema = c.ema if not c.use_max_ema else c.ema_max
            if c.inv is None or any(i.shape != e.shape for i, e in zip(c.inv, ema)):
                c.inv = [torch.empty_like(e) for e in ema]
            emas, invs, damps = by_sqrt[bool(c.use_sqrt_ema)]
            emas.extend(ema)
            invs.extend(c.inv)
            damps.extend([c.damping] * len(ema))
        for use_sqrt, (emas, invs, damps) in by_sqrt.items():
            _ops.diag_inverse_batched(emas, invs, damps, use_sqrt)
    for c in full:
        ema = c.ema if not c.use_max_ema else c.ema_max
        c.inv = [c._inv_one(e) for e in ema]


def update_std_all(curvs):
    """update_std: upper Cholesky factors of the inverses for Kronecker layers
    (reference: curvature.py:317-321), sqrt of the inverse for diagonal ones
    (curvature.py:240-241)."""
    kron = []
    for c in curvs:
        if c.kind != 'kron':
            continue
        if getattr(c, '_std_current', False):
            c._std_current = False             # delivered with the inverses (update_inv_all)
        else:
            kron.append(c)
    mats, outs = [], []
    for c in kron:
        inv = c.inv                            # (forms an inverse kept in factored form)
        if c.std is None or any(s is None or s.shape != i.shape for s, i in zip(c.std, inv)):
            c.std = [torch.empty_like(i) for i in inv]
        mats.extend(inv)
        outs.extend(c.std)
    if mats:
        _, info = _ops.cholesky_upper_batched(mats, outs)
        for i, c in enumerate(kron):
            c.std_info = info[2 * i:2 * i + 2]
    xs, ys = [], []
    for c in curvs:
        if c.kind == 'diag':
            if c.std is None or any(s.shape != i.shape for s, i in zip(c.std, c.inv)):
                c.std = [torch.empty_like(i) for i in c.inv]
            xs.extend(c.inv)
            ys.extend(c.std)
        elif c.kind == 'full':
            raise NotImplementedError
    _ops.sqrt_batched(xs, ys)


class NotPositiveDefiniteError(RuntimeError):
    """A damped curvature factor (or its inverse, for the Cholesky factor of the
    posterior) had a non-positive pivot: its inverse / std holds garbage."""


def check_spd_all(curvs):
    """Reads the status words the batched inversion and Cholesky factorisation left on
    the device for every Kronecker curvature in the list (ONE device-to-host copy, which
    waits for the stream) and raises NotPositiveDefiniteError naming the layers whose
    factors were not positive definite.  The reference never looks at the solver's
    status (utils/inv_cupy.py:124,130) and carries NaNs forward instead."""
    words, owners = [], []
    for li, c in enumerate(curvs):
        if c.kind != 'kron':
            continue
        for what, info in (('inverse', c.info), ('Cholesky factor of the inverse', c.std_info)):
            if info is not None:
                words.append(info.reshape(-1))
                owners.append((li, c, what))
    if not words:
        return
    flat = torch.cat(words).cpu().tolist()
    bad = []
    for k, (li, c, what) in enumerate(owners):
        for side, code in zip(('A', 'G'), flat[2 * k:2 * k + 2]):
            if code != 0:
                # (a factor inverted together with its std is factored back to front: the
                # status word then counts a leading minor of the matrix with its rows and
                # columns reversed, i.e. a trailing minor of the factor)
                which = ('trailing' if what == 'inverse' and getattr(c, '_info_reversed', False)
                         else 'leading')
                bad.append('layer %d (%s): %s of factor %s failed, %s minor of order %d is '
                           'not positive' % (li, type(c.module).__name__, what, side, which, code))
    if bad:
        raise NotPositiveDefiniteError(
            'curvature factors that are not positive definite (raise `damping`):\n  '
            + '\n  '.join(bad))


def step_all(curvs, update_std=False, update_inv=True):
    """Curvature.step for a list (reference: curvature.py:166-172).
    `update_std` may be a bool or a list of bools, one per curvature."""
    update_ema_all(curvs)
    if isinstance(update_std, (list, tuple)):
        sel = [c for c, u in zip(curvs, update_std) if u]
    else:
        sel = list(curvs) if update_std else []
    if update_inv:
        update_inv_all(curvs, with_std=sel)
    if sel:
        update_std_all(sel)


# The blocked Cholesky factorisation of the largest factors is a chain of small launches
# (two per 128 rows) that leaves most of the chip idle; smaller factors ride along in the
# same launches for nothing, but their triangular inverses and the preconditioning of
# their layers would still queue up behind the end of that chain.  When the largest factor
# has at least this many rows, the layers whose factors are at most half its size take
# their whole curvature phase (running average, inversion, preconditioning) to a side
# stream, where their dense launches fill the chip beside the chain.  None: one stream.
two_stream_min_dim = 2048


# (classes of layers that get a stream each; with three, the smaller factors no longer ride
# along in the launches of the middle ones and the step is as slow as on one stream)
curvature_streams_max = 2


def chain_classes(dims, min_dim, max_classes):
    """Indices of the layers in classes by the length of their longest factorisation,
    longest first: `dims[i]` is the largest factor dimension of layer i (0 for a layer
    without Kronecker factors).  A class is split off while the largest dimension left is
    at least `min_dim`: it takes the layers with a factor of more than half that size, and
    the rest must still hold a Kronecker layer.  None where one class (one stream) serves."""
    if min_dim is None:
        return None
    classes = []
    rest = list(range(len(dims)))
    while rest and len(classes) + 1 < max_classes:
        dmax = max(dims[i] for i in rest)
        if dmax < min_dim:
            break
        head = [i for i in rest if 2 * dims[i] > dmax]
        tail = [i for i in rest if 2 * dims[i] <= dmax]
        if not any(dims[i] > 0 for i in tail):
            break
        classes.append(head)
        rest = tail
    if not classes:
        return None
    classes.append(rest)
    return classes


def _chain_split(pairs):
    """The (curvature, params) pairs in the classes of `chain_classes`, or None."""
    if two_stream_min_dim is None or len(pairs) < 2:
        return None
    dims, devices = [], set()
    for c, params in pairs:
        w = params[0]
        if not w.is_cuda:
            return None
        devices.add(w.device)
        dims.append(max(w.shape[0], w[0].numel() + (1 if c.bias else 0))
                    if c.kind == 'kron' else 0)
    if len(devices) != 1:
        return None
    classes = chain_classes(dims, two_stream_min_dim, curvature_streams_max)
    return None if classes is None else [[pairs[i] for i in cls] for cls in classes]


def step_and_precondition_all(pairs, update_std=False, update_inv=True, precondition=True,
                              then=None):
    """step_all for the curvatures of `pairs` (a list of (curvature, params)), then
    precondition_all(pairs) if asked; on several streams where that pays (see
    `two_stream_min_dim`): the layers are independent of one another, so the results are
    those of one stream.  `then(sub_pairs)`: called for every part of the list right behind
    its preconditioning, on the stream that did it (the parameter update of those layers);
    when this function returns, the caller's stream has been made to wait for all of it."""
    curvs = [c for c, _ in pairs]
    plain_std = not isinstance(update_std, (list, tuple)) and not update_std
    split = _chain_split(pairs) if (update_inv and precondition and plain_std) else None
    if split is None:
        step_all(curvs, update_std=update_std, update_inv=update_inv)
        if precondition:
            precondition_all(pairs)
        if then is not None:
            then(pairs)
        return
    device = pairs[0][1][0].device
    _lanes.join()                       # (on the caller's stream: the side streams inherit it)
    cur = torch.cuda.current_stream(device)
    sides = [_lanes.curvature_stream(device, k) for k in range(len(split) - 1)]
    for side in sides:
        side.wait_stream(cur)
    for part, stream in zip(split, [cur] + sides):
        with torch.cuda.stream(stream):
            step_all([c for c, _ in part])
            precondition_all(part)
            if then is not None:
                then(part)
    for side in sides:
        cur.wait_stream(side)


def precondition_all(pairs):
    """precondition_grad for a list of (curvature, params): grads are replaced
    in place by G^-1 [dW|db] A^-1 (reference: cov/linear.py:69-84,
    cov/conv.py:76-92) or inv * grad (curvature.py:234-238)."""
    kron = ([], [], [], [], [], [])     # G operand, A operand, gW, gb, G is a factor, A is a factor
    dinv, dgrad = [], []
    for c, params in pairs:
        if c.kind == 'kron':
            w = params[0]
            if not w.grad.is_contiguous():
                w.grad = w.grad.contiguous()
            gb = None
            if c.bias:
                b = params[1]
                if not b.grad.is_contiguous():
                    b.grad = b.grad.contiguous()
                gb = b.grad
            fa, fg = c._inv_factors
            for lst, v in zip(kron, (fg if fg is not None else c._inv[1],
                                     fa if fa is not None else c._inv[0],
                                     w.grad, gb, fg is not None, fa is not None)):
                lst.append(v)
        elif c.kind == 'diag':
            for p, inv in zip(params, c.inv):
                if not p.grad.is_contiguous():
                    p.grad = p.grad.contiguous()
                dinv.append(inv)
                dgrad.append(p.grad)
        # 'full' curvatures do not precondition (reference: cov/linear.py:24-25)
    if any(kron[4]) or any(kron[5]):
        # one call for all layers, explicit ones included: every product is then one launch
        _ops.precondition_factored_batched(*kron)
    elif kron[0]:
        _ops.precondition_batched(*kron[:4])
    if dinv:
        _ops.diag_precondition_batched(dinv, dgrad)


def sample_all(items):
    """sample_params for a list of (curvature, params, mean, std_scale).

    The standard-normal noise is drawn with torch.randn_like in list order, one
    [dG, dA] matrix per Kronecker layer and one tensor per parameter of a
    diagonal layer, which is the order and shape in which the reference consumes
    the generator (cov/linear.py:92-93, cov/conv.py:100-101,
    curvature.py:243-246); the products run batched afterwards."""
    by_scale = {}
    d_mean, d_std, d_param, d_scale = [], [], [], []
    for c, params, mean, std_scale in items:
        if c.kind == 'kron':
            A_ic, G_ic = c.std
            dG, dA = G_ic.shape[0], A_ic.shape[0]
            noise = torch.randn((dG, dA), dtype=mean[0].dtype, device=mean[0].device)
            lst = by_scale.setdefault(float(std_scale), [])
            w = params[0].data
            if not w.is_contiguous():
                params[0].data = w = w.contiguous()
            pb = None
            mb = None
            if c.bias:
                pb = params[1].data
                mb = mean[1].contiguous()
            lst.append((G_ic, A_ic, noise, mean[0].contiguous(), mb, w, pb))
        elif c.kind == 'diag':
            for p, m, std in zip(params, mean, c.std):
                if not p.data.is_contiguous():
                    p.data = p.data.contiguous()
                # the noise is drawn straight into the parameter (same generator
                # consumption as randn_like(m)) and turned into the sample in place
                p.data.normal_()
                d_mean.append(m.contiguous())
                d_std.append(std)
                d_param.append(p.data)
                d_scale.append(float(std_scale))
        else:
            raise NotImplementedError
    _ops.diag_sample_batched(d_mean, d_std, d_param, d_scale)
    for std_scale, lst in by_scale.items():
        _ops.sample_batched([x[0] for x in lst], [x[1] for x in lst], [x[2] for x in lst],
                            [x[3] for x in lst], [x[4] for x in lst], [x[5] for x in lst],
                            [x[6] for x in lst], std_scale)
