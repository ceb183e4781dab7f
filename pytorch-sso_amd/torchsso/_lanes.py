"""Side streams ("lanes") for the Kronecker factor kernels.

A factor product depends only on the layer input (or output gradient) the hook
was handed, and nothing reads it before the optimizer step.  The hooks therefore
enqueue it on one of a few library-owned HIP streams instead of the caller's:
the product then runs beside the network's own forward / backward kernels and
beside the factor products of other layers, and the drain of one launch is
covered by the next.  (Back to back on one stream, every launch waits for the
last workgroup of the one before; the 226 launches of a ResNet-50 factor pass
lose about a millisecond to that.)

Ordering rules, all enforced here:
* a lane waits for everything the caller's stream has enqueued so far before it
  runs a product (the input exists, earlier readers of the output buffer are done);
* the tensors a product reads are marked as used by the lane
  (`Tensor.record_stream`), so the caching allocator does not hand their memory
  out again while the lane still reads it;
* a layer always uses the same lane, so the products of one layer stay in order;
* `join()` makes the caller's current stream wait for all lanes; every reader of
  factor data calls it first (`KronCurvature.data`, `update_ema_all`, ...).

All default-priority streams.  `set_count(0)` puts every product back on the
caller's stream.  The results do not depend on the setting: the kernels are
deterministic and each stream has its own scratch.

Grouped mode (`set_mode('grouped')`, the default) goes one step further: a hook only
describes its product (`defer`) and keeps the tensor it reads alive; the first reader of
factor data (`join()`, as before) hands all products collected so far to ONE engine call,
which runs them as a handful of launches holding the work items of all layers.  The queue
also runs at the first backward hook of a pass (the input factors then run beside the
backward pass), when a factor that is still queued gets a second product, and when the
collected work passes `flush_work()`; the engine calls take turns on the side streams, and
calls in flight that touch the same buffer are ordered by an event.  `set_mode('eager')`
runs every product in its hook, on the side streams, as described above.
"""
import atexit
import threading

import torch

_count = 2
_mode = 'grouped'
_lock = threading.Lock()
_flush_work = 2.5e11
# queued BatchNorm reductions run once the output gradients they keep alive reach this size
_BN_FLUSH_BYTES = 4e8


class _Queue(object):
    """Factor products of one device waiting for their engine call."""
    __slots__ = ('keys', 'items', 'work', 'forward', 'bn', 'bn_bytes')

    def __init__(self):
        self.keys = set()
        self.items = []      # (job, tensors kept alive, stream of the hook)
        self.work = 0.
        self.forward = False    # holds products queued by forward hooks
        self.bn = []         # BatchNorm backward reductions: (job tuple, stream of the hook)
        self.bn_bytes = 0    # output gradients those keep alive


_deferred = {}     # device index -> _Queue
_calls = {}        # device index -> engine calls made so far (deals them to the side streams)
_inflight = {}     # device index -> list of (event, items, addresses written) of calls the side streams may still run
_streams = {}      # device index -> list of (torch.cuda.Stream, torch.cuda.Event for the fork)
_pending = {}      # device index -> set of lane indices with work since the last join


def set_count(n):
    """Number of side streams for factor products (0: none, use the caller's stream)."""
    global _count
    n = int(n)
    if n < 0 or n > 8:
        raise ValueError('factor lanes: expected 0..8, got %d' % n)
    join()
    _count = n


def count():
    return _count


def set_mode(mode):
    """'grouped': hooks collect their factor products and the first reader of factor data
    runs them all in one engine call; 'eager': every product runs in its hook."""
    global _mode
    if mode not in ('grouped', 'eager'):
        raise ValueError("factor mode: expected 'grouped' or 'eager', got %r" % (mode,))
    join()
    _mode = mode


def mode():
    return _mode


def set_flush_work(work):
    """Grouped mode: the queue of a device also runs as soon as the products collected
    amount to `work` multiply-adds (d^2 * K summed over them), so that the engine starts on
    the first layers of a pass while the hooks of the later ones are still being called; a
    pass then takes a few engine calls instead of one.  None: only readers run the queue."""
    global _flush_work
    if work is not None and work <= 0:
        raise ValueError('flush work must be positive or None')
    _flush_work = work


def flush_work():
    return _flush_work


def defer(device, key, job, keep, work=0., backward=False):
    """Queues one factor product (a `_hip.FactorJob` whose pointers refer to the tensors in
    `keep`, which stay referenced until the product has been enqueued).  `key` names the
    factor: a second product for a key that is still queued runs the queue first, so at
    most one pass of products is ever pending.  `work`: its multiply-adds.  `backward`: the
    product belongs to a backward hook; the first of those runs what the forward hooks have
    queued, so that the input factors are computed beside the backward pass."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    stream = torch.cuda.current_stream(device)
    with _lock:
        q = _deferred.get(idx)
        if q is None:
            q = _deferred[idx] = _Queue()
        run_first = key in q.keys or (backward and q.forward)
    if run_first:
        _run_deferred(idx)
    with _lock:
        q = _deferred[idx]
        q.keys.add(key)
        q.forward = q.forward or not backward
        q.items.append((job, keep, stream))
        q.work += work
        full = _flush_work is not None and q.work >= _flush_work
    if full:
        _run_deferred(idx)


def defer_bn(device, key, job):
    """Queues the backward half of a BatchNorm layer's diagonal curvature: `job` =
    (grad_output, channels, sx, alpha, w, b) as `_ops.bn_diag_cov_batched` takes them (its
    tensors stay referenced until the reduction has been enqueued).  All queued layers run
    in ONE launch on the caller's stream when the queue runs.  A backward hook: the first
    one of a pass runs what the forward hooks have queued."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    stream = torch.cuda.current_stream(device)
    with _lock:
        q = _deferred.get(idx)
        if q is None:
            q = _deferred[idx] = _Queue()
        run_first = key in q.keys or q.forward
    if run_first:
        _run_deferred(idx)
    with _lock:
        q = _deferred[idx]
        q.keys.add(key)
        q.bn.append((job, stream))
        q.bn_bytes += job[0].numel() * 4
        full = q.bn_bytes >= _BN_FLUSH_BYTES
    if full:
        # (the reductions alone: the factor products keep waiting for their own trigger)
        _run_deferred(idx, bn_only=True)


def flush_if_queued(device, key):
    """Runs the queue of `device` if it holds a product for `key` (the caller is about to
    reuse that product's job object or output buffer)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    with _lock:
        q = _deferred.get(idx)
        dup = q is not None and key in q.keys
    if dup:
        _run_deferred(idx)


def deferred_count():
    """Products queued and not yet handed to the engine (all devices)."""
    with _lock:
        return sum(len(q.items) + len(q.bn) for q in _deferred.values())


def _run_deferred(only=None, bn_only=False):
    from torchsso import _ops
    with _lock:
        todo = []
        for i, q in _deferred.items():
            if bn_only:
                if q.bn and only == i:
                    todo.append((i, [], q.bn))
                    q.keys.difference_update(key for key in list(q.keys) if key[1] == 'bn')
                    q.bn, q.bn_bytes = [], 0
            elif (q.items or q.bn) and (only is None or only == i):
                todo.append((i, q.items, q.bn))
                _deferred[i] = _Queue()
    for i, items, bn in todo:
        device = torch.device('cuda', i)
        cur = torch.cuda.current_stream(i)
        if bn:
            # the BatchNorm reductions stay on the caller's stream (one launch for all queued
            # layers): they are bound by memory and run beside the factor products of the
            # side streams; whoever reads their outputs does so on this stream, behind them
            waited = []
            for job, st in bn:
                if st != cur:
                    if st not in waited:
                        waited.append(st)
                        cur.wait_stream(st)
                    for t in (job[0], job[2]) + tuple(job[4:]):
                        if t is not None:
                            t.record_stream(cur)
            _ops.bn_diag_cov_batched([job for job, _ in bn], device)
        if not items:
            continue
        side = None
        if _count > 0:
            # the engine call goes to a side stream (the calls of a pass take turns), so
            # that it runs beside whatever the caller's stream does next
            _, lst = _lane_streams(device)
            with _lock:
                lane = _calls.get(i, 0) % _count
                _calls[i] = _calls.get(i, 0) + 1
            side, fork = lst[lane]
            if side == cur:
                side = None
        target = cur if side is None else side
        # a product queued under another stream: its input is complete once that stream
        # has run what it held at the time of the hook (all of it, to keep this simple)
        others = []
        for _, keep, st in items:
            if st != cur:
                if st not in others and st != target:
                    others.append(st)
                for t in keep:
                    if t is not None:
                        t.record_stream(target)
        jobs = [job for job, _, _ in items]
        if side is not None:
            with _lock:
                fork.record(cur)
                side.wait_event(fork)
                # a call still in flight on ANOTHER side stream that writes a buffer this
                # call reads or adds to (factors accumulated over MC samples): wait for it
                touched = set()
                for job in jobs:
                    touched.add(job.C)
                    if job.C_prev:
                        touched.add(job.C_prev)
                for done, _, written in _inflight.get(i, []):
                    if not touched.isdisjoint(written):
                        side.wait_event(done)
        for st in others:
            target.wait_stream(st)
        # (the call's workspace is the cached scratch of the stream it runs on; a pass under
        # no_grad leaves its inputs referenced in the queue, or in `_inflight`, until the
        # next flush or join)
        _ops.factor_grouped(jobs, device, stream=side)
        if side is not None:
            # the tensors stay referenced until the caller's stream has been made to wait
            # for the side stream (join), or until the side stream is seen to have passed
            done = torch.cuda.Event()
            done.record(side)
            with _lock:
                held = [h for h in _inflight.get(i, []) if not h[0].query()]
                held.append((done, items, set(job.C for job in jobs)))
                _inflight[i] = held
                _pending.setdefault(i, set()).add(lane)


def _lane_streams(device):
    idx = device.index if device.index is not None else torch.cuda.current_device()
    lst = _streams.get(idx)
    if lst is None or len(lst) < _count:
        with _lock:
            lst = _streams.setdefault(idx, [])
            while len(lst) < _count:
                # (default priority; the event is re-recorded before every product)
                lst.append((torch.cuda.Stream(device=device), torch.cuda.Event()))
    return idx, lst


def run(device, key, reads, launch):
    """Runs `launch(stream)` on lane `key % count` of `device`: `launch` enqueues its
    kernels on the torch.cuda.Stream it is given (None: torch's current stream) and
    returns the output tensor, allocated on the current stream.  `reads`: the
    tensors the kernels read."""
    if _count == 0 or device.type != 'cuda':
        return launch(None)
    idx, lst = _lane_streams(device)
    lane = key % _count
    side, fork = lst[lane]
    cur = torch.cuda.current_stream(device)
    if side == cur:
        return launch(None)
    # the lane waits for what the caller's stream holds now (a later record of the
    # same event does not change what this wait refers to)
    with _lock:   # (hooks of two host threads may share a lane)
        fork.record(cur)
        side.wait_event(fork)
    out = launch(side)
    for t in reads:
        if t is not None:
            t.record_stream(side)
    out.record_stream(side)
    with _lock:
        _pending.setdefault(idx, set()).add(lane)
    return out


_curvature_streams = {}    # (device index, k) -> torch.cuda.Stream


def curvature_stream(device, k=0):
    """The k-th library-owned default-priority stream for the parts of the curvature phase
    (inversion, preconditioning) that run beside the caller's stream."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    with _lock:
        st = _curvature_streams.get((idx, k))
        if st is None:
            st = _curvature_streams[(idx, k)] = torch.cuda.Stream(device=idx)
    return st


def join(device=None):
    """The current stream of `device` (all devices if None) waits for the factor
    products enqueued so far."""
    if _deferred:
        _run_deferred(None if device is None or device.index is None else device.index)
    if not _pending:
        return
    with _lock:
        todo = [(i, sorted(l)) for i, l in _pending.items()
                if l and (device is None or device.index is None or device.index == i)]
        for i, _ in todo:
            _pending[i].clear()
    for i, lanes in todo:
        cur = torch.cuda.current_stream(i)
        for lane in lanes:
            cur.wait_stream(_streams[i][lane][0])
        with _lock:
            held = _inflight.pop(i, None) or []
        # What these calls read may be freed from here on, and the allocator hands a freed
        # block out again on the stream it was allocated under: a hook that ran under
        # another stream than this one has that stream wait for the call too.
        for done, items, _ in held:
            waited = []
            for _, _, st in items:
                if st != cur and st not in waited:
                    waited.append(st)
                    st.wait_event(done)


def _at_exit():
    """Interpreter exit: wait for the side streams and drop them (and their events) while the
    HIP runtime is still whole."""
    try:
        for lst in _streams.values():
            for side, _ in lst:
                side.synchronize()
    except Exception:
        pass
    try:
        for st in _curvature_streams.values():
            st.synchronize()
    except Exception:
        pass
    _curvature_streams.clear()
    _pending.clear()
    _streams.clear()
    _deferred.clear()
    _inflight.clear()


atexit.register(_at_exit)
