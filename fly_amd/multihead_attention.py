"""Multi-head wrapper around a pluggable attention layer: the caller of the attention layers of
this package in the reference's transformer models (src/models/modules/multihead_attention.py:21-258).

Same constructor, parameter names and ``forward(attention_layer, query, key, value,
key_padding_mask=None, need_weights=False, attn_mask=None)`` as the reference, so state dicts
are interchangeable: ``in_proj_weight`` (rows q | k | v, or qk | v with ``shared_qk``) or the
separate ``q_proj_weight`` / ``k_proj_weight`` / ``v_proj_weight`` when kdim != vdim,
``in_proj_bias``, ``out_proj.{weight,bias}``, ``bias_k`` / ``bias_v``, and the aliases of the input
projection under ``in_proj_container.*`` that the reference's state dict carries
(multihead_attention.py:100-102).  As in the reference, query / key / value all have last dimension
``embed_dim`` and are projected to kdim, kdim, vdim (multihead_attention.py:51-58).

The projections are library GEMMs; the attention itself is whatever layer is handed in
(SBLocalAttention, LocalAttention, BlockSparseAttention, SBBlockSparseAttention ...), called with
(B, T, H, head_dim) tensors and the mask objects of ``fly_amd.masking``."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from .masking import FullMask, LengthMask, pad_mask


class InProjContainer(nn.Module):
    """Holds the input-projection parameters of a MultiheadAttention (the same Parameter objects)
    and applies them (multihead_attention.py:261-352).  Self-attention (q is k is v) and
    encoder-decoder attention (k is v) use one GEMM for the tensors that coincide."""

    def __init__(self, q_proj_weight, k_proj_weight, v_proj_weight, in_proj_weight, in_proj_bias, shared_qk=False):
        super().__init__()
        self.q_proj_weight = q_proj_weight
        self.k_proj_weight = k_proj_weight
        self.v_proj_weight = v_proj_weight
        self.in_proj_weight = in_proj_weight
        self.in_proj_bias = in_proj_bias
        self.packed_weight = in_proj_weight is not None
        self.shared_qk = shared_qk

    def _sizes(self):
        """Row counts (q, k, v) of the projections inside the packed weight / bias."""
        if self.packed_weight:
            e = self.in_proj_weight.shape[0] // (2 if self.shared_qk else 3)
            return e, e, e
        kd = self.q_proj_weight.shape[0]
        return kd, kd, self.v_proj_weight.shape[0]

    def forward(self, q, k, v):
        nq, nk, nv = self._sizes()
        b = self.in_proj_bias
        if self.packed_weight:
            w = self.in_proj_weight
            if self.shared_qk:                       # rows: qk | v
                w_q, w_k, w_v = w[:nq], w[:nq], w[nq:]
                b_q, b_k, b_v = (None,) * 3 if b is None else (b[:nq], b[:nq], b[nq:])
            else:                                    # rows: q | k | v
                w_q, w_k, w_v = w[:nq], w[nq:nq + nk], w[nq + nk:]
                b_q, b_k, b_v = (None,) * 3 if b is None else (b[:nq], b[nq:nq + nk], b[nq + nk:])
            if q is k and k is v:
                if self.shared_qk:
                    qk, vv = F.linear(q, w, b).split([nq, nv], dim=-1)
                    return qk, qk, vv
                return tuple(F.linear(q, w, b).split([nq, nk, nv], dim=-1))
            if k is v and not self.shared_qk:
                kv = F.linear(k, w[nq:], None if b is None else b[nq:])
                return (F.linear(q, w_q, b_q),) + tuple(kv.split([nk, nv], dim=-1))
            if k is v:
                kk, vv = F.linear(k, w, b).split([nq, nv], dim=-1)
                return F.linear(q, w_q, b_q), kk, vv
            return F.linear(q, w_q, b_q), F.linear(k, w_k, b_k), F.linear(v, w_v, b_v)
        w_q = self.q_proj_weight
        w_k = self.q_proj_weight if self.shared_qk else self.k_proj_weight
        w_v = self.v_proj_weight
        assert w_q is not None and w_k is not None and w_v is not None, 'separate projection weights missing'
        if b is None:
            b_q = b_k = b_v = None
        elif self.shared_qk:                         # bias: qk | v
            b_q, b_k, b_v = b[:nq], b[:nq], b[nq:]
        else:
            b_q, b_k, b_v = b[:nq], b[nq:nq + nk], b[nq + nk:]
        return F.linear(q, w_q, b_q), F.linear(k, w_k, b_k), F.linear(v, w_v, b_v)


class MultiheadAttention(nn.Module):
    """``MultiheadAttention(embed_dim, num_heads, bias=True, add_bias_kv=False, add_zero_attn=False,
    kdim=None, vdim=None, batch_first=False, shared_qk=False, device=None, dtype=None)``
    (multihead_attention.py:64-112)."""
    __constants__ = ['batch_first']

    def __init__(self, embed_dim, num_heads, bias=True, add_bias_kv=False, add_zero_attn=False,
                 kdim=None, vdim=None, batch_first=False, shared_qk=False, device=None, dtype=None):
        fk = {'device': device, 'dtype': dtype}
        super().__init__()
        self.embed_dim = embed_dim
        self.kdim = kdim if kdim is not None else embed_dim
        self.vdim = vdim if vdim is not None else embed_dim
        self._qkv_same_dim = self.kdim == self.vdim
        self.num_heads = num_heads
        self.batch_first = batch_first
        assert self.kdim % num_heads == 0, 'self.kdim must be divisible by num_heads'
        assert self.vdim % num_heads == 0, 'self.vdim must be divisible by num_heads'
        self.shared_qk = shared_qk
        if self._qkv_same_dim:
            self.in_proj_weight = nn.Parameter(torch.empty(((2 if shared_qk else 3) * self.kdim, embed_dim), **fk))
            for name in ('q_proj_weight', 'k_proj_weight', 'v_proj_weight'):
                self.register_parameter(name, None)
        else:
            self.q_proj_weight = nn.Parameter(torch.empty((self.kdim, embed_dim), **fk))
            if shared_qk:
                self.register_parameter('k_proj_weight', None)
            else:
                self.k_proj_weight = nn.Parameter(torch.empty((self.kdim, embed_dim), **fk))
            self.v_proj_weight = nn.Parameter(torch.empty((self.vdim, embed_dim), **fk))
            self.register_parameter('in_proj_weight', None)
        if bias:
            self.in_proj_bias = nn.Parameter(torch.empty((1 if shared_qk else 2) * self.kdim + self.vdim, **fk))
        else:
            self.register_parameter('in_proj_bias', None)
        self.in_proj_container = InProjContainer(self.q_proj_weight, self.k_proj_weight, self.v_proj_weight,
                                                 self.in_proj_weight, self.in_proj_bias, shared_qk=shared_qk)
        self.out_proj = nn.Linear(self.vdim, embed_dim, bias=bias, **fk)
        if add_bias_kv:
            self.bias_k = nn.Parameter(torch.empty((1, 1, self.kdim), **fk))
            self.bias_v = nn.Parameter(torch.empty((1, 1, self.vdim), **fk))
        else:
            self.bias_k = self.bias_v = None
        self.add_zero_attn = add_zero_attn
        self._reset_parameters()

    def _reset_parameters(self):
        """Xavier-uniform projections, zero biases, Xavier-normal bias_k / bias_v
        (multihead_attention.py:114-130)."""
        for w in (self.in_proj_weight, self.q_proj_weight, self.k_proj_weight, self.v_proj_weight):
            if w is not None:
                nn.init.xavier_uniform_(w)
        if self.in_proj_bias is not None:
            nn.init.constant_(self.in_proj_bias, 0.)
            nn.init.constant_(self.out_proj.bias, 0.)
        for bkv in (self.bias_k, self.bias_v):
            if bkv is not None:
                nn.init.xavier_normal_(bkv)

    def forward(self, attention_layer, query, key, value, key_padding_mask=None, need_weights=False,
                attn_mask=None):
        """query (T, B, embed_dim), key / value (S, B, embed_dim) -- (B, T|S, embed_dim) with
        ``batch_first``; ``attn_mask`` a FullMask (T, S) or LengthMask (T), ``key_padding_mask`` a
        mask object over (B, S).  Returns (output in the layout of query, attention weights or None)
        (multihead_attention.py:132-258)."""
        if self.batch_first:
            bsz, tgt_len, embed_dim = query.shape
            src_len = key.shape[1]
        else:
            tgt_len, bsz, embed_dim = query.shape
            src_len = key.shape[0]
        assert embed_dim == self.embed_dim, f'was expecting embedding dimension of {self.embed_dim}, but got {embed_dim}'
        assert key.shape == value.shape, f'key shape {key.shape} does not match value shape {value.shape}'

        q, k, v = self.in_proj_container(query, key, value)
        if not self.batch_first:                     # batch first from here on
            q, k, v = (x.transpose(0, 1) for x in (q, k, v))

        if attn_mask is not None:
            assert isinstance(attn_mask, (FullMask, LengthMask))
            if isinstance(attn_mask, FullMask):
                if tuple(attn_mask.bool_matrix.shape) != (tgt_len, src_len):
                    raise RuntimeError(f'The shape of the 2D attn_mask is {tuple(attn_mask.bool_matrix.shape)}, '
                                       f'but should be {(tgt_len, src_len)}.')
            elif tuple(attn_mask._lengths.shape) != (tgt_len,):
                raise RuntimeError(f'The length of the 2D attn_mask is {tuple(attn_mask._lengths.shape)}, '
                                   f'but should be {(tgt_len,)}.')

        # The extra key positions go in FRONT of the keys (the reference's choice, so that a length-type
        # key_padding_mask stays a prefix-of-ones mask, multihead_attention.py:213-241); bias first, then
        # the zero position in front of it.
        extra = []
        if self.bias_k is not None and self.bias_v is not None:
            extra.append((self.bias_k.expand(bsz, 1, -1), self.bias_v.expand(bsz, 1, -1)))
        if self.add_zero_attn:
            extra.append((k.new_zeros(bsz, 1, self.kdim), v.new_zeros(bsz, 1, self.vdim)))
        for ek, ev in extra:
            k = torch.cat([ek.to(k.dtype), k], dim=1)
            v = torch.cat([ev.to(v.dtype), v], dim=1)
            if attn_mask is not None:
                attn_mask = pad_mask(attn_mask, 1, left=True)
            if key_padding_mask is not None:
                key_padding_mask = pad_mask(key_padding_mask, 1, left=True)

        H = self.num_heads
        q, k, v = (x.reshape(x.shape[0], x.shape[1], H, x.shape[2] // H) for x in (q, k, v))
        out, weights = attention_layer(q, k, v, attn_mask=attn_mask, key_padding_mask=key_padding_mask,
                                       need_weights=need_weights)
        out = self.out_proj(out.reshape(bsz, tgt_len, -1))
        if not self.batch_first:
            out = out.transpose(0, 1)
        return out, (weights if need_weights else None)
