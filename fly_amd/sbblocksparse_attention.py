"""Scatterbrain attention on a block-sparse support: drop-in for ``SBBlockSparseAttention``
(src/models/attention/sbblocksparse_attention.py:31-213).

Exact softmax weights on the nonzero blocks of the layout, the Performer low-rank estimate
everywhere else, one joint normalisation.  The block-sparse products (Q K^T and Q' K'^T on the
support, weights x V), the row logsumexp / row sum and the fused weight formula run on the HIP
kernels of this package; the feature maps and the global low-rank reductions are library GEMMs.
"""
import math

import torch
import torch.nn as nn
from torch import distributed as dist

from .blocksparse_attention import instantiate
from .blocksparse_matmul import matmul
from .blocksparse_softmax import blocksparse_sum, logsumexp
from .blocksparse_utils import (densify_tensor, sparsify_broadcast_tensor, tile_mask_table, union_heavy, union_order,
                                union_table)
from .sblocal_attention import ScratchCache, sbblocksparse_forward, sbblocksparse_forward_supported
from .feature_maps_sb import SBPerformerFeatures
from .padding import pad_to_multiple
from .scatterbrain_utils import linear_attention, linear_attention_normalization


def fused_tables(layout, device, block=32):
    """Index tables of the fused forward for a (H, T/block, S/block) layout of 16 x 16 or 32 x 32 blocks: per
    64-query tile the 32-key tiles on its support with the masks of its four groups of 16 queries
    (blocksparse_utils.tile_mask_table), the tiles' start order (longest list first), and the tiles whose lists are long
    enough to be walked in parts -- (ptr, inner, mask, order, heavy, parts), tensors on `device`."""
    ptr, inner, mask = tile_mask_table(layout, block)
    H = layout.shape[0]
    order = union_order(ptr, H)
    heavy, parts = union_heavy(ptr, mask - 1)        # (mask 0 = absent, as a block id of -1)
    if heavy.numel():
        groups = order.numel() // H
        marked = order.reshape(H, groups).clone()
        is_heavy = torch.zeros(H * groups, dtype=torch.bool)
        is_heavy[heavy.long()] = True
        flat = torch.arange(H).unsqueeze(1) * groups + marked.long()
        marked[is_heavy[flat]] = -1 - marked[is_heavy[flat]]
        order = marked.reshape(-1).contiguous()
    return tuple(x.to(device) for x in (ptr, inner, mask, order, heavy)) + (parts,)


def backward_tables(layout, device, transposed=False, n_heavy_min=32, entries_per_part=12, max_parts=16, block=32):
    """Index tables of one pass of the backward kernels for a (H, T/block, S/block) layout of 16 x 16 or 32 x 32 blocks:
    the lists of the 64-row outer tiles (queries, or with transposed=True keys) with the masks of their four groups of 16
    rows (blocksparse_utils.tile_mask_table), a flag per tile for the lists long enough to be walked in parts, those
    tiles, and the number of parts -- (ptr, inner, mask, skip, heavy, parts), tensors on `device`."""
    ptr, inner, blk = tile_mask_table(layout, block, transposed=transposed)
    counts = (ptr[1:] - ptr[:-1]).long()
    skip = (counts >= n_heavy_min).to(torch.int32)
    heavy = skip.nonzero().flatten().to(torch.int32)
    parts = max(2, min(max_parts, int(counts.max()) // entries_per_part)) if heavy.numel() else 1
    return tuple(x.to(device) for x in (ptr, inner, blk, skip, heavy)) + (parts,)


class _SBBlockSparseFn(torch.autograd.Function):
    """The fused forward with gradients for query, key and value: the backward of Scatterbrain-local attention with
    the band replaced by the layout's blocks (sblocal_backward.sblocal_backward, support=...)."""

    @staticmethod
    def forward(ctx, query, key, value, projection_matrix, tables, support, softmax_temp, cache=None, dropout=(0.0, 0)):
        out, log_norm = sbblocksparse_forward(query, key, value, projection_matrix, tables, softmax_temp, cache=cache,
                                              dropout_p=dropout[0], dropout_seed=dropout[1])
        ctx.save_for_backward(query, key, value, projection_matrix, out, log_norm)
        ctx.support, ctx.softmax_temp, ctx.dropout = support, softmax_temp, dropout
        ctx.mark_non_differentiable(log_norm)
        return out, log_norm

    @staticmethod
    def backward(ctx, grad_out, _grad_log_norm):
        from .sblocal_backward import sblocal_backward
        query, key, value, projection_matrix, out, log_norm = ctx.saved_tensors
        dq, dk, dv = sblocal_backward(query, key, value, projection_matrix, 1, ctx.softmax_temp, None, out, log_norm,
                                      grad_out, support=ctx.support, dropout=ctx.dropout)
        return dq, dk, dv, None, None, None, None, None, None


class SBBlockSparseAttention(nn.Module):
    """sparsity_config: an object with ``.block`` and ``.make_layout(seq_len) -> (H, nb, nb)`` or a
    mapping with ``_target_``.  forward(query (B,T,H,E), key (B,S,H,E), value (B,S,H,D)) returns
    (out (B,T,H,D), attn or None).  Like the reference (its assertion at :181) the layer takes no
    masks, which also means sequence lengths that are multiples of the block."""

    def __init__(self, sparsity_config, dim_heads, nb_features=None, ortho_scaling=0,
                 causal=False, softmax_temp=None, attention_dropout=0.0, softmax_eps=0.0,
                 max_seq_length=2048):
        super().__init__()
        if causal:
            raise NotImplementedError('causal Scatterbrain attention is not part of this build '
                                      '(the reference marks it unchecked, sbblocksparse_attention.py:147)')
        self.sparsity_config = instantiate(sparsity_config)
        self.feature_map = SBPerformerFeatures(dim_heads, nb_features, ortho_scaling=ortho_scaling,
                                               softmax_temp=softmax_temp, eps=softmax_eps)
        self.causal = causal
        self.softmax_temp = softmax_temp
        self.dropout = nn.Dropout(attention_dropout)
        self.softmax_eps = softmax_eps
        master_layout = self.sparsity_config.make_layout(max_seq_length)
        self.register_buffer("master_layout", master_layout)
        self._need_layout_synchronization = True
        self.ops_cache = dict()
        self._layout_cache = dict()
        self.fused_tables = dict()
        self.backward_tables = dict()
        # eligible forward passes run on the fused kernels; set to False to force the op-by-op path
        self.fuse = True
        # their device scratch (plan) and padded projection, kept between calls
        self._scratch_cache = ScratchCache()

    def get_layout(self, T, S=None):
        if S is None:
            S = T
        if self._need_layout_synchronization and dist.is_available() and dist.is_initialized():
            dist.broadcast(self.master_layout, src=0)
            self._need_layout_synchronization = False
        block = self.sparsity_config.block
        if (T % block != 0) or (S % block != 0):
            raise ValueError(f'Sequence lengths, {T} and {S}, needs to be divisible by block size {block}!')
        # one host copy per shape (keyed by the buffer's address and version counter): a device-to-host
        # copy per call would stall the stream
        key = (T, S, self.master_layout.data_ptr(), self.master_layout._version)
        if key not in self._layout_cache:
            layout = self.master_layout[..., :T // block, :S // block].cpu()
            self._layout_cache[key] = layout if layout.dim() == 3 else layout.unsqueeze(0)   # 2-D: one head
        return self._layout_cache[key]

    def get_ops(self, T, S=None):
        if S is None:
            S = T
        if (T, S) not in self.ops_cache:
            layout = self.get_layout(T, S)
            block = self.sparsity_config.block
            self.ops_cache[T, S] = (matmul(layout, block, 'sdd', trans_a=False, trans_b=True),
                                    matmul(layout, block, 'dsd', trans_a=False, trans_b=False),
                                    logsumexp(layout, block), blocksparse_sum(layout, block))
        return self.ops_cache[T, S]

    def forward(self, query, key, value, attn_mask=None, key_padding_mask=None, need_weights=False,
                return_attn_unnormalized=False):
        block = self.sparsity_config.block
        if attn_mask is not None or key_padding_mask is not None:
            raise NotImplementedError('SBBlockSparseAttention takes no masks (the reference asserts so, '
                                      'sbblocksparse_attention.py:181)')
        if query.shape[1] % block or key.shape[1] % block:
            # padding would create a key padding mask, which the reference then refuses (:135-138, 181)
            raise ValueError(f'Sequence lengths, {query.shape[1]} and {key.shape[1]}, needs to be divisible '
                             f'by block size {block}!')
        if query.shape[3] != self.feature_map.query_dims:
            raise ValueError(f'query has head dim {query.shape[3]}, the feature map was built for '
                             f'{self.feature_map.query_dims}')
        query = pad_to_multiple(query, block, dims=(1, 3))          # :125-127 (no-ops for the lengths)
        key = pad_to_multiple(key, block, dims=(1, 3))
        value = pad_to_multiple(value, block, dims=(1, 3))
        if query.shape[3] != self.feature_map.query_dims:
            raise ValueError(f'head dim {self.feature_map.query_dims} must be a multiple of the block '
                             f'size {block}: the padded queries no longer match the projection matrix')
        B, T, H, E = query.shape
        S = value.shape[1]
        softmax_temp = self.softmax_temp or 1 / math.sqrt(E)       # :131

        # blocks of 16 x 16 or 32 x 32, nothing but the output wanted: the whole forward on the fused kernels of
        # Scatterbrain-local attention, walking the layout's blocks instead of a band (with gradients: head dims and
        # feature counts of the backward kernels)
        self.feature_map.new_feature_map(query.device)
        layout = self.get_layout(T, S)
        needs_grad = torch.is_grad_enabled() and any(x.requires_grad for x in (query, key, value))
        from .sblocal_backward import _band_kernel_dims
        n_rows = self.feature_map.projection_matrix.shape[0]
        # training-mode dropout (:200: of the exact weights only) runs inside the kernels: the mask is a hash of (seed,
        # batch, head, query, key), the seed drawn per call from torch's CPU generator and kept in last_dropout_seed
        dropout = (0.0, 0)
        self.last_dropout_seed = None
        if self.training and 0 < self.dropout.p < 1:
            dropout = (float(self.dropout.p), int(torch.randint(0, 2 ** 62, (1,)).item()))
        if (self.fuse and not need_weights and not (self.training and self.dropout.p >= 1)
                and self.softmax_eps == 0
                and query.dtype in (torch.float32, torch.bfloat16, torch.float16)
                and sbblocksparse_forward_supported(block, torch.float32, E, value.shape[3], n_rows, layout.shape[0], H)
                # with gradients: the backward kernels' head dims and feature counts
                and (not needs_grad or _band_kernel_dims(E, value.shape[3], 2 * n_rows) is not None)):
            key_ = (T, S, query.device)
            if key_ not in self.fused_tables:
                self.fused_tables[key_] = fused_tables(layout, query.device, block)
            if not needs_grad:
                # 2-byte inputs go to the kernels as they are where the kernels on operand images run (they widen what
                # they load); otherwise they are widened here, as on the op-by-op path below
                native = sbblocksparse_forward_supported(block, query.dtype, E, value.shape[3], n_rows, layout.shape[0], H)
                qkv = (query, key, value) if native else (query.float(), key.float(), value.float())
                out, _ = sbblocksparse_forward(*qkv, self.feature_map.projection_matrix, self.fused_tables[key_], softmax_temp,
                                               cache=self._scratch_cache, dropout_p=dropout[0], dropout_seed=dropout[1])
                self.last_dropout_seed = dropout[1] if dropout[0] > 0 else None
                return out.to(query.dtype), None
            if key_ not in self.backward_tables:     # the support seen from the queries and from the keys
                self.backward_tables[key_] = (backward_tables(layout, query.device, block=block),
                                              backward_tables(layout, query.device, transposed=True, block=block))
            support = self.backward_tables[key_]
            # (with gradients 2-byte inputs are widened: the backward kernels take float32)
            out, _ = _SBBlockSparseFn.apply(query.float(), key.float(), value.float(), self.feature_map.projection_matrix,
                                            self.fused_tables[key_], support, softmax_temp, self._scratch_cache, dropout)
            self.last_dropout_seed = dropout[1] if dropout[0] > 0 else None
            return out.to(query.dtype), None

        # 2-byte inputs are widened: the scores pass through HBM between the stages, and a score kept
        # in bf16 (three significant digits, values of order 10) would cost percents in its exponential
        in_dtype = query.dtype
        query = query.permute(0, 2, 1, 3).float().contiguous()     # b h t e
        key = key.permute(0, 2, 1, 3).float().contiguous()
        value = value.permute(0, 2, 1, 3).float().contiguous()

        # op by op (:170-213): feature maps and the sums over all keys as library products, everything on the
        # support through the block-sparse operators.  Per query: Z = sum_support e^{t q.k} + max(phi(q).sum_all phi(k)
        # - sum_support phi(q).phi(k), 1e-24) e^{ls}; the weights on the support are e^{t q.k} / Z minus the feature
        # weight, which the all-keys term adds back; dropout touches the exact part only (:200).
        feat_q, ls_q = self.feature_map.forward_queries(query)
        feat_k, ls_k = self.feature_map.forward_keys(key)
        ls = (ls_q + ls_k).squeeze(-1)                                               # (b h t)
        mass_all = linear_attention_normalization(feat_q, feat_k)                    # phi(q) . sum_s phi(k_s)
        out_all, attn_prime = linear_attention(feat_q, feat_k, value, need_weights=need_weights)
        sdd_nt, dsd_nn, sparse_logsumexp, sparse_sum = self.get_ops(T, S)
        scores = sdd_nt(query, key).mul_(softmax_temp)
        overlap = sdd_nt(feat_q, feat_k)
        mass_off_support = (mass_all - sparse_sum(overlap)).clamp_min(1e-24)
        log_z = torch.logaddexp(sparse_logsumexp(scores), mass_off_support.log() + ls)
        feat_weight = (ls - log_z).exp()

        def per_block(rows):                     # a (b h t) vector spread over the columns of the support's blocks
            return sparsify_broadcast_tensor(rows, layout, block)
        dots = self.dropout((scores - per_block(log_z)).exp()) - overlap * per_block(feat_weight)
        out = (dsd_nn(dots, value) + out_all * feat_weight.unsqueeze(-1)).to(in_dtype)

        attn = None
        if need_weights:
            attn = densify_tensor(dots, layout) + attn_prime * feat_weight.unsqueeze(-1)
            if return_attn_unnormalized:
                attn = (attn, attn * log_z.exp().unsqueeze(-1), attn_prime * ls.exp().unsqueeze(-1))
        return out.permute(0, 2, 1, 3), attn
