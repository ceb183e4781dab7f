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
"""
import atexit
import threading

import torch

_count = 3
_lock = threading.Lock()
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


def join(device=None):
    """The current stream of `device` (all devices if None) waits for the factor
    products enqueued so far."""
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


def _at_exit():
    """Interpreter exit: wait for the side streams and drop them (and their events) while the
    HIP runtime is still whole."""
    try:
        for lst in _streams.values():
            for side, _ in lst:
                side.synchronize()
    except Exception:
        pass
    _pending.clear()
    _streams.clear()


atexit.register(_at_exit)
