"""Running sum of tensors (gradients, curvature factors) across accumulation steps.

Same interface as the reference's torchsso/utils/accumulator.py:4-56:
``update(data, scale)`` adds ``scale * data`` (a Tensor or a list of Tensors),
``get(clear=True)`` hands the sum out.  On HIP tensors the additions are one
batched launch of the engine's axpby kernel into buffers this object owns, so
``get`` can hand the buffers over without another copy.
"""
from torch import Tensor

from torchsso import _ops


class TensorAccumulator(object):

    def __init__(self):
        self._accumulation = None

    def check_type(self, data):
        ok = 'the type of data has to be list of torch.Tensor or torch.Tensor'
        if isinstance(data, list):
            assert type(data[0]) == Tensor, ok
        else:
            assert type(data) == Tensor, ok
        acc = self._accumulation
        if acc is not None:
            assert type(data) == type(acc), \
                'the type of data ({}) is different from the type of the accumulation ({})'.format(
                    type(data), type(acc))

    @staticmethod
    def _add(acc, data, scale):
        """acc (None or list) + scale * data (list) -> list"""
        if data[0].is_cuda:
            src = [d.detach().contiguous() for d in data]
            if acc is None:
                acc = [d.new_empty(d.shape) for d in src]
                _ops.axpby_batched(src, acc, scale, 0.)
            else:
                _ops.axpby_batched(src, acc, scale, 1.)
            return acc
        # host tensors (losses, probabilities kept on the CPU by a caller)
        if acc is None:
            return [d * scale for d in data]
        return [a + scale * d for a, d in zip(acc, data)]

    @classmethod
    def update_many(cls, accumulators, datas, scale=1.):
        """accumulators[i].update(datas[i], scale) for every i, with ONE batched launch for
        all HIP tensors of all accumulators (an optimizer step accumulates the gradients
        and the curvature factors of every layer at once)."""
        srcs, dsts_new, dsts_old = [], [], []
        for acc, data in zip(accumulators, datas):
            acc.check_type(data)
            as_list = data if isinstance(data, list) else [data]
            if not as_list[0].is_cuda:
                acc.update(data, scale)
                continue
            src = [d.detach().contiguous() for d in as_list]
            have = acc._accumulation
            if have is None:
                new = [d.new_empty(d.shape) for d in src]
                acc._accumulation = new if isinstance(data, list) else new[0]
                srcs.extend(src)
                dsts_new.extend(new)
            else:
                dsts_old.append((src, have if isinstance(have, list) else [have]))
        if dsts_new:
            _ops.axpby_batched(srcs, dsts_new, scale, 0.)
        if dsts_old:
            _ops.axpby_batched([x for src, _ in dsts_old for x in src],
                               [y for _, have in dsts_old for y in have], scale, 1.)

    def slot(self, index, count, shape, like):
        """(buffer, fresh) for tensor `index` of a list accumulation of `count` tensors whose
        producers add into it themselves (a factor kernel with an accumulating epilogue):
        `fresh` tells the producer that the buffer is new and must be written, not added to.
        Every slot has to be filled before `get`."""
        if self._accumulation is None:
            self._accumulation = [None] * count
        acc = self._accumulation
        assert isinstance(acc, list) and len(acc) == count, 'accumulation of another shape exists'
        buf = acc[index]
        fresh = buf is None
        if fresh:
            buf = acc[index] = like.new_empty(shape)
        else:
            assert tuple(buf.shape) == tuple(shape)
        return buf, fresh

    def update(self, data, scale=1.):
        self.check_type(data)
        if isinstance(data, list):
            self._accumulation = self._add(self._accumulation, data, scale)
        else:
            acc = None if self._accumulation is None else [self._accumulation]
            self._accumulation = self._add(acc, [data], scale)[0]

    def get(self, clear=True):
        acc = self._accumulation
        if acc is None:
            return
        if clear:
            # the buffers are ours alone: hand them over instead of cloning
            self._accumulation = None
            return acc
        if isinstance(acc, list):
            return [a.clone() for a in acc]
        return acc.clone()

    def clear(self):
        self._accumulation = None
