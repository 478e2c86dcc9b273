"""Zero padding to a multiple along chosen dims (src/utils/padding.py:6-25)."""
import torch.nn.functional as F


def pad_to_multiple(tensor, multiple, dims=-1, value=0):
    try:
        dims = list(dims)
    except TypeError:
        dims = [dims]
    dims = [d if d >= 0 else tensor.ndim + d for d in dims]
    padding = [0] * (2 * tensor.ndim)
    for d in dims:
        remainder = tensor.size(d) % multiple
        if remainder != 0:
            padding[2 * (tensor.ndim - d - 1) + 1] = multiple - remainder
    if not any(padding):
        return tensor
    return F.pad(tensor, tuple(padding), value=value)
