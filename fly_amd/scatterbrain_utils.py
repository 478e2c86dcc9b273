"""Low-rank (linear attention) reductions of Scatterbrain on feature tensors
(src/models/attention/scatterbrain_utils.py:18-22, 48-52): plain library GEMMs."""
import torch


def linear_attention_normalization(q, k, causal=False):
    """q' . sum_s k'_s per query: q (..., T, m), k (..., S, m) -> (..., T)."""
    if causal:
        raise NotImplementedError('causal linear attention is not part of this build')
    key_total = k.sum(dim=-2).unsqueeze(-1)                   # (..., m, 1)
    return torch.matmul(q, key_total).squeeze(-1)


def linear_attention(q, k, v, need_weights=False):
    """q' (k'^T v) without forming the (T, S) weights unless asked for: returns ((..., T, D), weights or None)."""
    summary = torch.matmul(k.transpose(-1, -2), v)            # (..., m, D)
    weights = torch.matmul(q, k.transpose(-1, -2)) if need_weights else None
    return torch.matmul(q, summary), weights
