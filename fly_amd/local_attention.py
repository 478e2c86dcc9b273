"""Plain local (banded) softmax attention on the HIP kernel: drop-in for ``LocalAttention``
(src/models/attention/local_attention.py:12-108)."""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from .sblocal_attention import _HEAD_DIMS, _round_up_choice, _vector_ready
from .sblocal_backward import BandWindows, _band_kernel_dims, _band_terms_hip


def _additive_mask(attn_mask, T, S, device):
    """The (T, S) additive matrix as the kernels read it: float32, contiguous, on the device; finite entries only
    (the reference hands over additive_matrix_finite, 0 / -1e24, local_attention.py:53-56)."""
    if attn_mask is None:
        return None
    if tuple(attn_mask.shape) != (T, S):
        raise ValueError(f'attn_mask must have shape ({T}, {S}), got {tuple(attn_mask.shape)}')
    return attn_mask.to(device=device, dtype=torch.float32).contiguous()


def local_forward(query, key, value, local_context, softmax_temp=None, key_lengths=None, return_lse=False,
                  dropout=(0.0, 0), attn_mask=None):
    """query (B,T,H,E), key (B,S,H,E), value (B,S,H,D) float32, bfloat16 or float16 GPU tensors ->
    out (B,T,H,D): query i attends to keys j with -(local_context // 2) <= j - i < (local_context + 1) // 2
    and j < key_lengths[b] (local_attention.py:68-92 for attn_mask=None).  With return_lse
    also the log of every query's softmax denominator, (B,H,T) float32 (0 for a query without keys).
    dropout = (p, seed) with p > 0: the weights are dropped after the softmax with probability p and the kept ones
    scaled by 1 / (1 - p) (local_attention.py:91, `self.dropout(torch.softmax(...))`), by a hash of (seed, batch,
    head, query, key) formed inside the kernel instead of a stored mask.
    attn_mask: None or a (T, S) float tensor added to q.k before the temperature (local_attention.py:53-56, 68-75:
    additive_matrix_finite, 0 / -1e24).  -1e24 absorbs the product in float32, so a query whose visible keys are all
    masked weighs each position of its band 1 / local_context, the positions outside the keys included (they add
    nothing to the output; :76-81 leaves such rows as they are); its lse entry is -inf."""
    _lib.require_gpu(query, key, value, key_lengths, attn_mask)
    if query.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise NotImplementedError(f'the local attention kernel supports float32, bfloat16 and float16, got {query.dtype}')
    if key.dtype != query.dtype or value.dtype != query.dtype:
        raise ValueError('query, key and value must share a dtype')
    B, T, H, E = query.shape
    Bk, S, Hk, Ek = key.shape
    Bv, Sv, Hv, D = value.shape
    if (Bk, Hk, Ek) != (B, H, E) or (Bv, Sv, Hv) != (B, S, H):
        raise ValueError(f'inconsistent shapes q{tuple(query.shape)} k{tuple(key.shape)} v{tuple(value.shape)}')
    if local_context < 1:
        raise ValueError('local_context must be >= 1')
    t = softmax_temp or 1 / math.sqrt(E)
    dim = _round_up_choice(max(E, D), _HEAD_DIMS, 'head dimension')

    def prep(x):
        if x.shape[-1] != dim:
            x = F.pad(x, (0, dim - x.shape[-1]))      # zero columns change no dot product
        # (2-byte rows are loaded 8 elements at a time: strides in multiples of 8)
        ready = _vector_ready(x) and (x.element_size() == 4 or all(st % 8 == 0 for st in x.stride()[:-1]))
        return x if ready else x.contiguous()
    q, k, v = prep(query), prep(key), prep(value)
    lens = None
    if key_lengths is not None:
        lens = key_lengths.to(device=query.device, dtype=torch.int64).contiguous()
        if lens.shape != (B,):
            raise ValueError(f'key_lengths must have shape ({B},)')
    out = torch.empty(B, T, H, dim, dtype=query.dtype, device=query.device)
    lse = torch.empty(B, H, T, dtype=torch.float32, device=query.device) if return_lse else None
    add = _additive_mask(attn_mask, T, S, query.device)
    with torch.cuda.device(query.device):
        _lib.call('flyhip_local_fwd_masked', q.data_ptr(), k.data_ptr(), v.data_ptr(), _lib.ptr(lens), _lib.ptr(add),
                  out.data_ptr(), _lib.ptr(lse), B, H, T, S, dim, dim, local_context,
                  q.stride(0), q.stride(2), q.stride(1), k.stride(0), k.stride(2), k.stride(1),
                  v.stride(0), v.stride(2), v.stride(1), out.stride(0), out.stride(2), out.stride(1),
                  t, _lib.dtype_code(q), float(dropout[0]), int(dropout[1]), _lib.stream_ptr(query.device))
    return (out[..., :D], lse) if return_lse else out[..., :D]


def local_backward(query, key, value, local_context, softmax_temp, key_lengths, grad_out, chunk=256,
                   max_elements=1 << 27, out=None, lse=None, dropout=(0.0, 0), attn_mask=None):
    """Gradients of local attention with respect to query, key and value (the reference takes them from
    autograd through fast_transformers.local_product, local_attention.py:68-92).  The band softmax is
    evaluated again for all chunks of queries at once against the windows of keys their bands touch
    (sblocal_backward.BandWindows); with
    P = softmax over the band, g = d out and delta_i = sum_s P_is g_i.v_s:
    d v_s = sum_i P_is g_i,  d(t q_i.k_s) = P_is (g_i.v_s - delta_i).  Queries without any visible
    key get zero gradients.  bfloat16 and float16 GPU tensors with the forward's out and lse, no attn_mask and no
    dropout: flyhip_local_bwd, on the matrix pipe of the input type (_local_backward_2byte).  Otherwise, given the
    forward's out and lse (local_forward(..., return_lse=True)), GPU tensors
    and head dims <= 64, the sums run in float32 on the backward band kernel of
    Scatterbrain-local attention with its feature operands zero (flyhip_sblocal_bwd_band: P_is =
    exp(t q_i.k_s - lse_i), delta_i = g_i.out_i); otherwise as batched library products on the GPU (host tensors are
    accepted in float64 only: the check of these formulas against autograd).  dropout = (p, seed) of the forward:
    with M the kept / (1 - p) mask, d v_s = sum_i M_is P_is g_i and d(t q_i.k_s) = P_is (M_is g_i.v_s - delta_i),
    delta_i = g_i.out_i as before; on the band kernel only.  attn_mask: the forward's additive matrix (the scores are
    t (q.k + mask); a query with lse = -inf weighs its visible keys 1 / local_context each); on the band kernel only."""
    B, T, H, E = query.shape
    S, D = key.shape[1], value.shape[3]
    t = softmax_temp or 1 / math.sqrt(E)
    if (query.dtype in (torch.bfloat16, torch.float16) and query.is_cuda and out is not None and lse is not None
            and attn_mask is None and dropout[0] == 0 and max(E, D) <= _HEAD_DIMS[-1]):
        return _local_backward_2byte(query, key, value, local_context, t, key_lengths, grad_out, out, lse)
    wdt = torch.float64 if query.dtype == torch.float64 else torch.float32

    def bh(x):                                   # (B,L,H,C) -> (B*H, L, C)
        return x.permute(0, 2, 1, 3).reshape(B * H, x.shape[1], x.shape[3]).to(wdt)
    Q, K, V, G = bh(query), bh(key), bh(value), bh(grad_out)

    def back(x, like):                           # (B*H, L, C) -> (B,L,H,C)
        # (in the inputs' own memory order: autograd then accumulates the gradient without another copy)
        return x.reshape(B, H, x.shape[1], x.shape[2]).permute(0, 2, 1, 3).to(like.dtype, memory_format=torch.contiguous_format)
    if not Q.is_cuda and wdt != torch.float64:
        # host tensors are accepted for one purpose: checking the written-out gradient formulas in float64 against autograd
        raise NotImplementedError('local_backward runs on the GPU; host tensors only in float64 (the check of the formulas)')
    dims = _band_kernel_dims(E, D, 0)
    if out is not None and lse is not None and Q.is_cuda and wdt == torch.float32 and dims is not None:
        zq, zk = Q.new_zeros(B * H, T, dims[1]), Q.new_zeros(B * H, S, dims[1])
        delta = (G * bh(out)).sum(-1, keepdim=True)
        lens_b = None if key_lengths is None else key_lengths.to(device=Q.device, dtype=torch.int64).contiguous()
        dQ, _, dK, _, dV = _band_terms_hip(Q, K, V, G, zq, zk, lse.reshape(B * H, T, 1), delta, lens_b, H,
                                           local_context, t, dims, dropout, _additive_mask(attn_mask, T, S, Q.device))
        return back(dQ, query), back(dK, key), back(dV, value)
    if attn_mask is not None:
        raise NotImplementedError('the gradients of local attention with an attn_mask run on the band kernel only: '
                                  'float32 or bfloat16 GPU tensors, head dims <= 64, the forward\'s out and lse given')
    if dropout[0] > 0:
        raise NotImplementedError('the gradients of dropped local attention run on the band kernel only: float32 or '
                                  'bfloat16 GPU tensors, head dims <= 64, the forward\'s out and lse given')
    lens = None
    if key_lengths is not None:
        lens = key_lengths.to(Q.device).repeat_interleave(H).view(B * H, 1, 1)
    band = BandWindows(T, S, local_context, chunk, Q.device, lens, max_elements)
    Qc, Gc = band.chunks(Q), band.chunks(G)
    acc_k, acc_v = band.key_accumulator(B * H, E, wdt), band.key_accumulator(B * H, D, wdt)
    dQc = torch.zeros_like(Qc)
    Kw, Vw = band.windows(K), band.windows(V)
    for j0, j1 in band.groups(B * H):
        sl = slice(j0, j1)
        ks, vs = Kw[:, sl], Vw[:, sl]
        scores = (t * (Qc[:, sl] @ ks.transpose(2, 3))).masked_fill(~band.mask(j0, j1), -math.inf)
        p = torch.softmax(scores, dim=-1).nan_to_num(0.0)          # rows without a visible key: zeros
        dp = Gc[:, sl] @ vs.transpose(2, 3)
        ds = p * (dp - (p * dp).sum(-1, keepdim=True))
        dQc[:, sl] = t * (ds @ ks)
        band.add_windows(acc_k, j0, t * (ds.transpose(2, 3) @ Qc[:, sl]))
        band.add_windows(acc_v, j0, p.transpose(2, 3) @ Gc[:, sl])
    dQ, dK, dV = band.unchunk(dQc), band.fold(acc_k), band.fold(acc_v)
    return back(dQ, query), back(dK, key), back(dV, value)


def _local_backward_2byte(query, key, value, local_context, t, key_lengths, grad_out, out, lse):
    """local_backward for bfloat16 / float16 GPU tensors on flyhip_local_bwd: the band softmax is formed again from the
    forward's lse on the matrix pipe of the input type; delta_i = g_i . out_i is formed by the first launch."""
    B, T, H, E = query.shape
    S, D = key.shape[1], value.shape[3]
    dim = _round_up_choice(max(E, D), _HEAD_DIMS, 'head dimension')

    def prep(x):
        if x.shape[-1] != dim:
            x = F.pad(x, (0, dim - x.shape[-1]))      # zero columns change no dot product
        ready = _vector_ready(x) and all(st % 8 == 0 for st in x.stride()[:-1])
        return x if ready else x.contiguous()
    q, k, v, g, o = prep(query), prep(key), prep(value), prep(grad_out.to(query.dtype)), prep(out.to(query.dtype))
    delta = torch.empty(B, H, T, dtype=torch.float32, device=query.device)     # g . out per query, filled by the kernels
    lse_ = lse.reshape(B, H, T).float().contiguous()
    lens = None if key_lengths is None else key_lengths.to(device=query.device, dtype=torch.int64).contiguous()
    dq = torch.empty(B, T, H, dim, dtype=query.dtype, device=query.device)
    dk = torch.empty(B, S, H, dim, dtype=query.dtype, device=query.device)
    dv = torch.empty(B, S, H, dim, dtype=query.dtype, device=query.device)

    def strides(x):
        return x.stride(0), x.stride(2), x.stride(1)
    with torch.cuda.device(query.device):
        _lib.call('flyhip_local_bwd', q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr(),
                  lse_.data_ptr(), _lib.ptr(lens), delta.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                  B, H, T, S, dim, local_context, *strides(q), *strides(k), *strides(v), *strides(o), *strides(g),
                  *strides(dq), *strides(dk), *strides(dv), t, _lib.dtype_code(q), _lib.stream_ptr(query.device))
    return dq[..., :E], dk[..., :E], dv[..., :D]


class _LocalFn(torch.autograd.Function):
    """Forward on the fused kernel, gradients from local_backward."""

    @staticmethod
    def forward(ctx, query, key, value, local_context, softmax_temp, key_lengths, dropout=(0.0, 0), attn_mask=None):
        out, lse = local_forward(query, key, value, local_context, softmax_temp=softmax_temp, key_lengths=key_lengths,
                                 return_lse=True, dropout=dropout, attn_mask=attn_mask)
        ctx.save_for_backward(query, key, value, key_lengths, out, lse, attn_mask)
        ctx.local_context, ctx.softmax_temp, ctx.dropout = local_context, softmax_temp, dropout
        return out

    @staticmethod
    def backward(ctx, grad_out):
        query, key, value, key_lengths, out, lse, attn_mask = ctx.saved_tensors
        dq, dk, dv = local_backward(query, key, value, ctx.local_context, ctx.softmax_temp, key_lengths, grad_out,
                                    out=out, lse=lse, dropout=ctx.dropout, attn_mask=attn_mask)
        return dq, dk, dv, None, None, None, None, None


def local_attention_fn(query, key, value, local_context, softmax_temp=None, key_lengths=None, dropout=(0.0, 0),
                       attn_mask=None):
    """local_forward that autograd can differentiate (no gradient reaches attn_mask)."""
    return _LocalFn.apply(query, key, value, local_context, softmax_temp, key_lengths, dropout, attn_mask)


class LocalAttention(nn.Module):
    """Softmax attention in which query i only sees keys j with
    -(local_context // 2) <= j - i < (local_context + 1) // 2.  Same constructor and forward signature
    as the reference class.  Covered on the GPU: optional attn_mask (its additive_matrix_finite is added inside the
    kernels), optional length-style key_padding_mask, attention dropout in training mode (inside the kernels);
    anything else raises NotImplementedError.  need_weights=True also returns the dense
    (B,H,T,S) matrix (local_attention.py:94-106), exp(t q.k - lse) on the band with the kernel's own
    log-denominators, as ordinary tensor algebra: an inspection path for problems of up to
    max_weight_elements entries."""

    def __init__(self, local_context, softmax_temp=None, attention_dropout=0.0, device=None, dtype=None):
        super().__init__()
        self.local_context = local_context
        self.softmax_temp = softmax_temp
        self.dropout = nn.Dropout(attention_dropout)
        self.max_weight_elements = 1 << 26

    def forward(self, query, key, value, attn_mask=None, key_padding_mask=None, need_weights=False):
        additive = None
        if attn_mask is not None and not bool(attn_mask.all_ones):
            additive = attn_mask.additive_matrix_finite.to(query.device)    # local_attention.py:53-56
        # training-mode dropout (local_attention.py:91) runs inside the kernels: the mask is a hash of (seed, batch,
        # head, query, key); the seed is drawn per call from torch's CPU generator and kept in last_dropout_seed
        dropout = (0.0, 0)
        self.last_dropout_seed = None
        if self.training and self.dropout.p > 0.0:
            if not self.dropout.p < 1.0:
                raise NotImplementedError('attention dropout with p = 1 is not implemented in the fused kernel')
            if need_weights:
                raise NotImplementedError('need_weights with active attention dropout is not implemented')
            dropout = (float(self.dropout.p), int(torch.randint(0, 2 ** 62, (1,)).item()))
            self.last_dropout_seed = dropout[1]
        lengths = None
        if key_padding_mask is not None and not bool(key_padding_mask.all_ones):
            lengths = key_padding_mask.lengths
        if not need_weights:
            out = local_attention_fn(query, key, value, self.local_context, softmax_temp=self.softmax_temp,
                                     key_lengths=lengths, dropout=dropout, attn_mask=additive)
            return out, None
        B, T, H, E = query.shape
        S = key.shape[1]
        if B * H * T * S > self.max_weight_elements:
            raise NotImplementedError(f'need_weights=True materialises the (B,H,T,S) matrix: {B * H * T * S} entries '
                                      f'exceed max_weight_elements = {self.max_weight_elements}')
        out, lse = local_forward(query, key, value, self.local_context, softmax_temp=self.softmax_temp,
                                 key_lengths=lengths, return_lse=True, attn_mask=additive)
        t = self.softmax_temp or 1 / math.sqrt(E)
        scores = torch.einsum('bthe,bshe->bhts', query.float(), key.float())
        if additive is not None:
            scores = scores + additive.to(scores)
        scores = t * scores
        idx = torch.arange(S, device=query.device).view(1, S) - torch.arange(T, device=query.device).view(T, 1)
        band = ((idx >= -(self.local_context // 2)) & (idx < (self.local_context + 1) // 2)).view(1, 1, T, S)
        if lengths is not None:
            band = band & (torch.arange(S, device=query.device).view(1, 1, 1, S) < lengths.view(B, 1, 1, 1))
        attn = torch.where(band, torch.exp(scores - lse.unsqueeze(-1)), scores.new_zeros(()))
        if additive is not None:         # every visible key masked (lse = -inf): equal weights over the packed band
            attn = torch.where(torch.isinf(lse).unsqueeze(-1), band.to(attn.dtype) / self.local_context, attn)
        return out, attn
