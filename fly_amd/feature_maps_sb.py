"""Performer random features for Scatterbrain attention: the projection matrix and the module
that owns it (src/models/attention/projection_utils.py:8-28, feature_maps_sb.py:85-156).

Behind ``SBLocalAttention`` the feature values (feature_maps_sb.py:51-82) are computed inside
the HIP kernels and never reach the caller.  ``softmax_kernel`` / ``forward_queries`` /
``forward_keys`` give them as tensors for the layers that feed them to the block-sparse matmuls
(``SBBlockSparseAttention``).
"""
import math

import torch
import torch.nn as nn


def gaussian_orthogonal_random_matrix(nrows, ncols, scaling=0, device=None, dtype=None):
    """(nrows, ncols) matrix whose ncols-row blocks are Haar-orthogonal, with rows rescaled to
    chi-distributed norms (scaling=0) or to sqrt(ncols) (scaling=1) -- projection_utils.py:8-28.
    Unlike the reference, which draws the row norms on the target device (:23), every random
    number comes from the CPU generator so that a seed gives the same matrix on any machine."""
    nblocks = int(math.ceil(nrows / ncols))
    gauss = torch.randn((nblocks, ncols, ncols), device='cpu')
    q, r = torch.linalg.qr(gauss)
    q = q * torch.sign(torch.diagonal(r, dim1=-2, dim2=-1)).unsqueeze(-2)
    rows = q.transpose(-1, -2).reshape(nblocks * ncols, ncols)[:nrows]
    if scaling == 0:
        norms = torch.randn((nrows, ncols), device='cpu').norm(dim=1)
        rows = norms.unsqueeze(-1) * rows
    elif scaling == 1:
        rows = math.sqrt(ncols) * rows
    else:
        raise ValueError(f'Invalid scaling {scaling}')
    return rows.to(device=device, dtype=dtype)


def softmax_kernel(data, *, projection_matrix, is_query, softmax_temp=None, eps=0., cosh=True,
                   return_log=False):
    """Positive random features of `data` (..., S, D) with their log-scale (feature_maps_sb.py:51-82):
    features = exp(+-sqrt(t) P x - stabiliser), where queries are stabilised per row (and the
    log-scale carries -t|x|^2/2 + rowmax - log(m)/2) and keys by one maximum over the last two
    dimensions.  Returns (features or their logs, in the dtype of `data`; log_scale)."""
    if return_log and eps != 0:
        raise NotImplementedError('return_log is not compatible with nonzero eps')
    if not cosh:
        raise NotImplementedError('only the cosh (two-sided) feature map is implemented')
    d = data.shape[-1]
    m = 2 * projection_matrix.shape[0]
    if softmax_temp is None:
        softmax_temp = 1 / math.sqrt(d)
    normalizer = math.sqrt(softmax_temp)
    dash = torch.matmul(data, (normalizer * projection_matrix.type_as(data)).t())
    dash = torch.cat([dash, -dash], dim=-1)
    diag = data.square().sum(dim=-1, keepdim=True) / 2 * softmax_temp
    if is_query:
        row_max = torch.amax(dash, dim=-1, keepdim=True)
        log_scale = -diag + row_max - math.log(m) / 2
        dash_log = dash - row_max
    else:
        shifted = dash - diag - math.log(m) / 2
        log_scale = torch.amax(shifted, dim=(-1, -2), keepdim=True)
        dash_log = shifted - log_scale
    if return_log:
        return dash_log.type_as(data), log_scale
    return (torch.exp(dash_log) + eps / math.sqrt(m)).type_as(data), log_scale


class SBPerformerFeatures(nn.Module):
    """Holder of the random projection (feature_maps_sb.py:85-156).

    ``n_features`` defaults to int(E ln E); the cosh feature map uses n_features // 2 projection
    rows and produces 2 * (n_features // 2) features.  ``new_feature_map`` draws the matrix on the
    first call only (the reference sets ``redraw = pi`` so that ``calls % redraw == 0`` just once,
    :119,135-137).  The buffer ``projection_matrix`` has shape (n_features // 2, query_dims); a
    matrix loaded from a state dict or assigned by the caller is used as is when
    ``freeze_projection()`` has been called.
    """

    def __init__(self, query_dims, n_features=None, ortho_scaling=0, softmax_temp=None,
                 orthogonal=False, cosh=True, redraw=1, deterministic_eval=False, eps=0.0,
                 device=None, dtype=None):
        super().__init__()
        if not cosh:
            raise NotImplementedError('only the cosh (two-sided) feature map is implemented')
        if n_features is None or n_features == 0:
            n_features = int(query_dims * math.log(query_dims))
        if softmax_temp is None:
            softmax_temp = query_dims ** -0.5
        # `orthogonal` and `redraw` are accepted and ignored like in the reference, which fixes the redraw
        # period to an irrational number: only call number 0 is a multiple of it
        vars(self).update(query_dims=query_dims, n_features=n_features, ortho_scaling=ortho_scaling,
                          softmax_temp=softmax_temp, orthogonal=orthogonal, cosh=cosh, redraw=math.pi,
                          deterministic_eval=deterministic_eval, eps=eps,
                          factory_kwargs=dict(device=device, dtype=dtype), _calls=-1)
        self.register_buffer('projection_matrix', torch.zeros(self.projection_rows, query_dims, device=device, dtype=dtype))

    @property
    def projection_rows(self):
        """Rows of the projection: each gives an exp(+.) and an exp(-.) feature."""
        return self.n_features // 2

    def freeze_projection(self):
        """Keep the current ``projection_matrix`` (e.g. one loaded from a checkpoint or set by a
        test) instead of drawing a new one on the first forward."""
        self._calls = 0

    def new_feature_map(self, device):
        """Called once per forward by the attention layers; draws the projection when a redraw is due."""
        if self.deterministic_eval and not self.training:
            return
        self._calls += 1
        due = math.fmod(self._calls, self.redraw) == 0
        if due:
            self.projection_matrix = gaussian_orthogonal_random_matrix(
                self.projection_rows, self.query_dims, scaling=self.ortho_scaling, device=device,
                dtype=self.factory_kwargs['dtype'])

    def _features(self, x, is_query, return_log):
        return softmax_kernel(x, projection_matrix=self.projection_matrix, is_query=is_query,
                              softmax_temp=self.softmax_temp, eps=self.eps, cosh=self.cosh, return_log=return_log)

    def forward_queries(self, x, return_log=False):
        return self._features(x, True, return_log)

    def forward_keys(self, x, return_log=False):
        return self._features(x, False, return_log)
