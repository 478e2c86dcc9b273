"""Mask types handed to the attention layers (boundary types of the reference:
src/models/modules/masking.py:23-199).  True / 1 marks a position that is kept."""
import torch


class BaseMask:
    """Interface: subclasses provide ``bool_matrix``; everything else is derived and cached."""

    @property
    def bool_matrix(self):
        raise NotImplementedError()

    def _cached(self, name, make):
        if not hasattr(self, name):
            with torch.no_grad():
                setattr(self, name, make())
        return getattr(self, name)

    @property
    def float_matrix(self):
        return self._cached('_float_matrix', lambda: self.bool_matrix.float())

    @property
    def lengths(self):
        """Number of kept positions per row; raises ValueError unless every row is a prefix of
        ones (masking.py:41-58)."""
        def make():
            m = self.bool_matrix
            lengths = m.long().sum(dim=-1)
            prefix = torch.arange(m.shape[-1], device=m.device) < lengths.unsqueeze(-1)
            if not torch.equal(prefix, m):
                raise ValueError('The mask is not a length mask')
            return lengths
        return self._cached('_lengths', make)

    @property
    def shape(self):
        return self.bool_matrix.shape

    @property
    def additive_matrix(self):
        """0 where kept, -inf where masked (masking.py:66-74)."""
        return self._cached('_additive_matrix', lambda: torch.log(self.bool_matrix.float()))

    @property
    def additive_matrix_finite(self):
        """0 where kept, -1e24 where masked (masking.py:76-84)."""
        return self._cached('_additive_matrix_finite', lambda: (~self.bool_matrix).float() * (-1e24))

    @property
    def all_ones(self):
        return self._cached('_all_ones', lambda: torch.all(self.bool_matrix))

    @property
    def lower_triangular(self):
        def make():
            try:
                lengths = self.lengths
            except ValueError:
                return False
            if lengths.dim() != 1:
                return False
            target = torch.arange(1, len(lengths) + 1, device=lengths.device)
            return bool(torch.all(lengths == target))
        return self._cached('_lower_triangular', make)


class FullMask(BaseMask):
    """Arbitrary boolean (N, M) mask.  ``FullMask(mask)``, ``FullMask(N)``, ``FullMask(N, M)`` or
    keyword forms, as in masking.py:111-156."""

    def __init__(self, mask=None, N=None, M=None, device='cpu'):
        if isinstance(mask, torch.Tensor):
            if mask.dtype != torch.bool:
                raise ValueError('FullMask expects the mask to be bool')
            with torch.no_grad():
                self._mask = mask.clone()
            return
        if mask is not None and M is None and isinstance(mask, int):
            M, N = N, mask
        if N is None:
            raise ValueError('Either mask or N should be provided')
        M = M or N
        self._mask = torch.ones(N, M, dtype=torch.bool, device=device)
        self._all_ones = True

    @property
    def bool_matrix(self):
        return self._mask


class LengthMask(BaseMask):
    """Rows of ones followed by zeros, given by their lengths (masking.py:159-186).  ``max_len``
    defaults to the largest length; ``device`` to the device of ``lengths``."""

    def __init__(self, lengths, max_len=None, device=None):
        self._device = lengths.device if device is None else device
        self._lengths = lengths.detach().clone().to(self._device)
        self._max_len = self._lengths.max() if not max_len else max_len
        self._all_ones = bool((self._lengths == self._max_len).all())
        self._bool_matrix = None

    @property
    def bool_matrix(self):
        if self._bool_matrix is None:
            positions = torch.arange(self._max_len, device=self._device)
            self._bool_matrix = positions.unsqueeze(0) < self._lengths.unsqueeze(-1)
        return self._bool_matrix


class TriangularCausalMask(LengthMask):
    """Lower-triangular (N, N) mask (masking.py:189-199)."""

    def __init__(self, N, device='cpu'):
        super().__init__(torch.arange(1, N + 1, device=device), N, device)
        self._lower_triangular = True


def pad_mask(mask, pad_length, left=True, value=True):
    """Extend a mask by pad_length key positions (src/models/attention/mask_utils.py:6-18)."""
    import torch.nn.functional as F
    assert value in [True, False]
    assert isinstance(mask, (FullMask, LengthMask))
    if isinstance(mask, FullMask):
        pad = (pad_length, 0) if left else (0, pad_length)
        return FullMask(F.pad(mask._mask, pad, value=value))
    lengths = mask._lengths + pad_length if value else mask._lengths
    return LengthMask(lengths, max_len=mask._max_len + pad_length, device=mask._lengths.device)
