"""Padding up to a multiple along chosen dims (src/utils/padding.py:6-25)."""
import torch.nn.functional as F


def pad_to_multiple(tensor, multiple, dims=-1, value=0):
    """`tensor` with every dim in `dims` (an int or an iterable of ints) extended at its end to the
    next multiple of `multiple`, filled with `value`; the tensor itself when nothing is missing."""
    wanted = {d % tensor.ndim for d in ([dims] if isinstance(dims, int) else dims)}
    missing = [(-tensor.size(d)) % multiple if d in wanted else 0 for d in range(tensor.ndim)]
    if not any(missing):
        return tensor
    # F.pad lists (before, after) pairs from the last dim backwards
    spec = tuple(x for extra in reversed(missing) for x in (0, extra))
    return F.pad(tensor, spec, value=value)
