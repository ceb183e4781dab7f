"""Wire format of factors and gradients: the flat buffer that the reference's
communicators reduce and gather (torchsso/utils/chainer_communicators/_utility.py:16-138).

A buffer holds, rank block after rank block, the arrays of that block back to
back: a symmetric matrix (Kronecker factor, inverse) as its upper triangle row
by row, anything else whole.  Packing and unpacking of a whole list is one
engine launch each.  Only the format lives here; this build runs on one GPU and
has no collectives.
"""
from torchsso import _ops


class Packer(object):
    """pack / unpack of `arrays` = list (one entry per rank block) of lists of
    (tensor, triangular) into / from a flat fp32 device tensor, starting at element
    `offset` (reference: Packer, _utility.py:16-104; there the buffer is a CuPy
    DeviceMemory addressed in bytes on an explicit stream, here a torch tensor on
    the current stream)."""

    def pack(self, arrays, buf, offset=0):
        for local_arrays in arrays:
            offset = _ops.pack_batched(list(local_arrays), buf, offset)
        return offset

    def unpack(self, arrays, buf, offset=0):
        for local_arrays in arrays:
            offset = _ops.unpack_batched(list(local_arrays), buf, offset)
        return offset

    @staticmethod
    def packed_numel(arrays):
        return sum(_ops.packed_numel(list(local_arrays)) for local_arrays in arrays)


def get_nelems(arrays):
    """Number of elements of the packed form (reference: _utility.py:195-207)."""
    return Packer.packed_numel(arrays)


def extract(param_groups, indices, extractors):
    """Lists of (array, triangular) per rank block: `indices` is a list of lists of
    param_group indices, each extractor maps a param_group to an iterable of
    (array, triangular) (reference: _utility.py:119-138)."""
    arrays = []
    for local_indices in indices:
        local_arrays = []
        for index in local_indices:
            for extractor in extractors:
                local_arrays.extend(extractor(param_groups[index]))
        arrays.append(local_arrays)
    return arrays


def extract_attr_from_params(attr, target='params', triangular=False):
    """Extractor of p.<attr> for every parameter of a group (reference:
    _utility.py:141-157)."""
    def _extract(group):
        out = []
        for p in group[target]:
            t = getattr(p, attr, None)
            if t is not None:
                out.append((t, triangular))
        return out
    return _extract


def extract_attr_from_curv(attr, triangular=False):
    """Extractor of curv.<attr> (a tensor or a list of tensors) of a group; only
    2-D square tensors are sent as triangles (reference: _utility.py:160-192)."""
    def _extract(group):
        curv = group['curv']
        if curv is None:
            return []
        target = getattr(curv, attr, None)
        if target is None:
            if curv.data is not None:
                zeros = [d.new_zeros(d.shape) for d in curv.data]
                setattr(curv, attr, zeros)
                target = getattr(curv, attr)
            else:
                return []
        items = target if isinstance(target, (list, tuple)) else [target]
        return [(t, triangular and t.dim() == 2 and t.shape[0] == t.shape[1]) for t in items]
    return _extract
