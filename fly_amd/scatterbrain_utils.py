"""Low-rank (linear attention) reductions of Scatterbrain on feature tensors
(src/models/attention/scatterbrain_utils.py:18-22, 48-52): plain library GEMMs."""
import torch


def linear_attention_normalization(q, k, causal=False):
    """q' . sum_s k'_s per query: (..., T, m), (..., S, m) -> (..., T)."""
    if causal:
        raise NotImplementedError('causal linear attention is not part of this build')
    return torch.einsum('...nm,...m->...n', q, k.sum(dim=-2))


def linear_attention(q, k, v, need_weights=False):
    """q' (k'^T v): returns ((..., T, D), attention weights or None)."""
    k_v = torch.einsum('...nm,...nd->...md', k, v)
    q_k_v = torch.einsum('...nm,...md->...nd', q, k_v)
    attn = None if not need_weights else torch.einsum('...im,...jm->...ij', q, k)
    return q_k_v, attn
