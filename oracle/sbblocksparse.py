"""CPU restatement of Scatterbrain attention on a block-sparse support -- TEST INFRASTRUCTURE ONLY
(imported by tests/; never by fly_amd).

`sbblocksparse_attention` follows the op sequence of
src/models/attention/sbblocksparse_attention.py:161-212 on dense masked matrices (features with
log-scales, support logsumexp, overlap sum, clamp, joint normalisation, weights, output).
`dense_closed_form` evaluates the same quantity straight from the mathematics in float64 -- exact
softmax weights on the support, positive-random-feature weights elsewhere, one normalisation --
with no stabilisers and no subtraction of the overlap; tests/test_oracle_sbblocksparse.py pins the
former against the latter, against explicit loops on a tiny case, and against the Scatterbrain-local
oracle on a layout whose support is exactly a band.
"""
import math

import torch

from . import blocksparse as ob
from . import sblocal as osb


def support_mask(layout, block):
    """(H, T, S) boolean: the nonzero blocks of the layout, expanded to elements."""
    if layout.dim() == 2:
        layout = layout.unsqueeze(0)
    return layout.bool().repeat_interleave(block, dim=1).repeat_interleave(block, dim=2)


def sbblocksparse_attention(query, key, value, projection_matrix, layout, block, softmax_temp=None,
                            dropout_multiplier=None):
    """query (B,T,H,E), key (B,S,H,E), value (B,S,H,D) -> out (B,T,H,D), log_normalization (B,H,T,1).
    Same op sequence as the reference layer (sbblocksparse_attention.py:161-212), dense.
    dropout_multiplier: None, or (B,H,T,S) -- the mask of nn.Dropout times 1 / (1 - p); it multiplies
    exp(QK - log_normalization) and nothing else (:196-200)."""
    B, T, H, E = query.shape
    t = softmax_temp or 1 / math.sqrt(E)
    q = query.permute(0, 2, 1, 3)
    k = key.permute(0, 2, 1, 3)
    v = value.permute(0, 2, 1, 3)
    qp, q_ls = osb.softmax_kernel(q, projection_matrix, True, softmax_temp=t)        # :165-166
    kp, k_ls = osb.softmax_kernel(k, projection_matrix, False, softmax_temp=t)
    prime_log_scale = q_ls + k_ls                                                     # :168
    qk1 = osb.linear_attention_normalization(qp, kp)                                  # :174
    qkv = osb.linear_attention(qp, kp, v)                                             # :175
    mask = support_mask(layout, block).unsqueeze(0)                                   # (1,H,T,S)
    QK = t * (q @ k.transpose(-1, -2))                                                # :181 on the support
    dots_prime = (qp @ kp.transpose(-1, -2)) * mask                                   # :182
    QK_lse = torch.logsumexp(QK.masked_fill(~mask, float('-inf')), dim=-1, keepdim=True)    # :187
    QK_lse = torch.where(torch.isinf(QK_lse), torch.zeros_like(QK_lse), QK_lse)       # empty rows give 0
    dots_prime_sum = dots_prime.sum(-1, keepdim=True)                                 # :188
    lr_log_norm = torch.log((qk1.unsqueeze(-1) - dots_prime_sum).clamp_min(1e-24)) + prime_log_scale   # :189-190
    log_norm = torch.logaddexp(QK_lse, lr_log_norm)                                   # :191
    prime_scale = torch.exp(prime_log_scale - log_norm)                               # :193
    exact = torch.exp(QK - log_norm)
    if dropout_multiplier is not None:
        exact = exact * dropout_multiplier
    dots = (exact - dots_prime * prime_scale) * mask                                  # :200
    out = dots @ v + qkv * prime_scale                                                # :203-204
    return out.permute(0, 2, 1, 3), log_norm


def dense_closed_form(query, key, value, projection_matrix, layout, block, softmax_temp=None):
    """From the mathematics, float64: A_ij = exp(t q_i.k_j) on the support, phi(q_i).phi(k_j) elsewhere;
    out = A v / rowsum(A), log_normalization = log rowsum(A)."""
    B, T, H, E = query.shape
    t = softmax_temp or 1 / math.sqrt(E)
    q = query.permute(0, 2, 1, 3).double()
    k = key.permute(0, 2, 1, 3).double()
    v = value.permute(0, 2, 1, 3).double()
    W = projection_matrix.double() * math.sqrt(t)
    m = 2 * W.shape[0]

    def phi(x):
        proj = x @ W.t()
        sq = (x * x).sum(-1, keepdim=True) * t / 2
        return torch.exp(torch.cat([proj, -proj], -1) - sq) / math.sqrt(m)

    lowrank = phi(q) @ phi(k).transpose(-1, -2)
    exact = torch.exp(t * (q @ k.transpose(-1, -2)))
    A = torch.where(support_mask(layout, block).unsqueeze(0), exact, lowrank)
    Z = A.sum(-1, keepdim=True)
    return ((A @ v) / Z).permute(0, 2, 1, 3), torch.log(Z)
