"""Block-sparse softmax attention on the HIP kernels: drop-in for
src/models/attention/blocksparse_attention.py:23-166 (SDD -> block softmax -> DSD)."""
import importlib
import math

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import distributed as dist

from .blocksparse_fused import fused_attention
from .blocksparse_matmul import matmul
from .blocksparse_softmax import softmax
from .blocksparse_utils import densify_tensor
from .masking import FullMask, LengthMask, pad_mask
from .padding import pad_to_multiple


def _cut(out, seqlen, dim):
    """out[:, :seqlen, :, :dim] -- sliced only where something is cut off: under autograd every slice, also one that
    keeps everything, costs a zero-fill and a copy of the whole tensor in the backward pass."""
    if out.shape[1] != seqlen:
        out = out[:, :seqlen]
    if out.shape[3] != dim:
        out = out[..., :dim]
    return out


class _AttentionCoreFn(torch.autograd.Function):
    """softmax(scale * q k^T + masks) v on the nonzero blocks, for calls that need gradients.  With masks
    the forward is the reference's three ops (blocksparse_attention.py:134-160; the probabilities are
    kept for the backward); without, the one-kernel attention, which keeps one log-denominator per row,
    and the backward forms the probabilities again.  The backward runs four kernels instead of the
    op-by-op chain's six plus elementwise passes:
    dV = P^T dO, dS = scale * P * (dO V^T - rowsum(dO * O)) in one kernel (the sdd fused with the softmax
    gradient), dQ = dS K, dK = dS^T Q.  32x32 blocks of bf16 / fp16 with shared-tile tables only.
    After the one-kernel forward with head dims up to 64 the backward is flyhip_bs_attn_bwd: two
    launches (query-major for dQ, key-major for dK and dV) that form P and dS per block and never write them.
    ``dropout=(p, seed)`` (one-kernel forward only): the dropout of blocksparse_attention.py:160 with the mask
    a hash of (seed, batch, head, query, key) that the backward kernel forms again: it writes M * P for dV and
    dS = scale * P * (M * dO V^T - rowsum(dO * O)), M = kept / (1 - p)."""

    @staticmethod
    def forward(ctx, q, k, v, sdd, dsd, sm, scale, kpm, am, fused, dropout=(0.0, 0)):
        ctx.ops, ctx.scale, ctx.dropout = (sdd, dsd), scale, dropout
        masked = kpm is not None or am is not None
        if dropout[0] > 0 and not (fused is not None and not masked):
            raise NotImplementedError('dropout inside the kernels needs the one-kernel forward without masks')
        ctx.masks = (None, None)
        if fused is not None and (not masked or (dropout[0] == 0 and q.shape[3] in (32, 64))):
            # the one-kernel forward; it keeps the rows' log-denominators instead of the probabilities, which the
            # backward forms again.  With masks (head dims up to 64, no dropout) the backward kernels read them too.
            out, lse2 = fused(q, k, v, scale, kpm, return_lse=True, attn_mask=am, dropout=dropout)
            ctx.save_for_backward(q, k, v, out, lse2)
            ctx.masks = (kpm, am)
            ctx.recompute = True
            return out
        p = sm(sdd._run('sdd', q, k, False, True, False), scale=scale, key_padding_mask=kpm, attn_mask=am,
               key_padding_mask_mode='add', attn_mask_mode='add')
        if kpm is not None or am is not None:
            p.nan_to_num_()
        out = dsd._run('dsd', p, v, False, False, False)
        ctx.save_for_backward(q, k, v, p, out)
        ctx.recompute = False
        return out

    @staticmethod
    def backward(ctx, dout):
        from . import _lib
        sdd, dsd = ctx.ops
        H, rows, cols = sdd.spdims
        uni_ptr, uni_inner, uni_blk = sdd._table('union', dout.device)

        def vec(x):          # 16-byte loads: last dim contiguous, other strides multiples of 8
            ok = x.stride(3) == 1 and all(s_ % 8 == 0 for s_ in x.stride()[:3]) and x.data_ptr() % 16 == 0
            return x if ok else x.contiguous()
        dout = vec(dout)
        if ctx.recompute and ctx.saved_tensors[0].shape[3] in (32, 64):
            # head dims up to 64: both orientations on one kernel that keeps neither P nor dS (a dropout mask is formed again)
            q, k, v, out, lse2 = ctx.saved_tensors
            col_tabs = sdd._table('union_t', dout.device)
            if len(col_tabs) == 3:
                qq, kk, vv, oo = vec(q), vec(k), vec(v), vec(out)
                # (in the layout of the inputs -- (B, T, H, E) seen as (B, H, T, E) -- so that autograd hands them on as they are)
                dq, dk, dv = (torch.empty_like(x) for x in (qq, kk, vv))
                delta = torch.empty_like(lse2)
                kpm, am = ctx.masks
                kpm = None if kpm is None else kpm.to(device=q.device, dtype=torch.float32).contiguous()
                am = None if am is None else am.to(device=q.device, dtype=torch.float32).contiguous()

                def st3(x):
                    return x.stride(0), x.stride(1), x.stride(2)
                with torch.cuda.device(q.device):
                    _lib.call('flyhip_bs_attn_bwd', qq.data_ptr(), kk.data_ptr(), vv.data_ptr(), oo.data_ptr(),
                              dout.data_ptr(), lse2.data_ptr(), delta.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                              dv.data_ptr(), uni_ptr.data_ptr(), uni_inner.data_ptr(), uni_blk.data_ptr(),
                              col_tabs[0].data_ptr(), col_tabs[1].data_ptr(), col_tabs[2].data_ptr(),
                              H, rows, cols, q.shape[0], q.shape[3], *st3(qq), *st3(kk), *st3(vv), *st3(oo), *st3(dout),
                              *st3(dq), *st3(dk), *st3(dv), float(ctx.scale), _lib.dtype_code(q),
                              float(ctx.dropout[0]), int(ctx.dropout[1]), _lib.ptr(kpm), 0 if kpm is None else kpm.stride(0),
                              _lib.ptr(am), 0 if am is None else am.stride(0), _lib.stream_ptr(q.device))
                return dq, dk, dv, None, None, None, None, None, None, None, None
            if ctx.masks != (None, None):
                raise NotImplementedError('the backward with masks needs the shared-tile tables of the transposed layout')
        if ctx.recompute:
            # probabilities, score gradient, dq and the rows' delta = rowsum(d out * out) from one kernel: both
            # products (q k^T, d out v^T) per block
            q, k, v, out, lse2 = ctx.saved_tensors
            nnz = int(sdd.layout.sum())
            p = torch.empty((q.shape[0], nnz, 32, 32), dtype=q.dtype, device=q.device)
            ds = torch.empty_like(p)
            qq, kk, vv, oo = vec(q), vec(k), vec(v), vec(out)
            dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
            with torch.cuda.device(q.device):
                _lib.call('flyhip_bs_sdd_prob_dsoftmax_dropout', dout.data_ptr(), vv.data_ptr(), qq.data_ptr(), kk.data_ptr(),
                          None, oo.data_ptr(), lse2.data_ptr(), ds.data_ptr(), p.data_ptr(), dq.data_ptr(),
                          uni_ptr.data_ptr(), uni_inner.data_ptr(), uni_blk.data_ptr(),
                          nnz, H, rows, q.shape[0], q.shape[3], 32,
                          dout.stride(0), dout.stride(1), dout.stride(2), vv.stride(0), vv.stride(1), vv.stride(2),
                          qq.stride(0), qq.stride(1), qq.stride(2), kk.stride(0), kk.stride(1), kk.stride(2),
                          dq.stride(0), dq.stride(1), dq.stride(2), oo.stride(0), oo.stride(1), oo.stride(2),
                          float(ctx.scale), _lib.dtype_code(q), float(ctx.dropout[0]), int(ctx.dropout[1]),
                          _lib.stream_ptr(q.device))
            dv = dsd._run('dsd', p, dout, True, False, False)
        else:
            dq = None
            q, k, v, p, out = ctx.saved_tensors
            dv = dsd._run('dsd', p, dout, True, False, False)
            delta = (dout.float() * out.float()).sum(-1).contiguous()
            ds = torch.empty_like(p)
            vv = vec(v)
            with torch.cuda.device(q.device):
                _lib.call('flyhip_bs_sdd_dsoftmax', dout.data_ptr(), vv.data_ptr(), p.data_ptr(), delta.data_ptr(),
                          ds.data_ptr(), uni_ptr.data_ptr(), uni_inner.data_ptr(), uni_blk.data_ptr(),
                          p.shape[1], H, rows, q.shape[0], v.shape[3], 32,
                          dout.stride(0), dout.stride(1), dout.stride(2), vv.stride(0), vv.stride(1), vv.stride(2),
                          float(ctx.scale), _lib.dtype_code(q), _lib.stream_ptr(q.device))
        if dq is None:
            dq = dsd._run('dsd', ds, k, False, False, False)
        dk = dsd._run('dsd', ds, q, True, False, False)
        return dq, dk, dv, None, None, None, None, None, None, None, None

    @staticmethod
    def supports(sdd, block, dtype, head_dim, device):
        return (block == 32 and dtype in (torch.bfloat16, torch.float16) and head_dim % 32 == 0
                and head_dim <= 128 and len(sdd._table('union', device)) == 3)


def instantiate(cfg, *args, **kwargs):
    """Resolve a plugin description the way the reference's hydra.utils.instantiate call sites do
    (blocksparse_attention.py:39, blocksparse_linear.py:49, fastlinear.py:789): a mapping with a
    ``_target_`` dotted path plus keyword arguments becomes an object; anything else is taken to be
    the object itself."""
    if isinstance(cfg, dict) or (hasattr(cfg, 'keys') and '_target_' in cfg):
        cfg = dict(cfg)
        target = cfg.pop('_target_')
        cfg.pop('_recursive_', None)
        module, _, name = target.rpartition('.')
        # reference paths resolve to this package's drop-ins
        module = {'src.models.layers.blocksparse_linear': 'fly_amd.blocksparse_linear',
                  'src.models.layers.fastlinear': 'fly_amd.fastlinear',
                  'src.models.attention.sblocal_attention': 'fly_amd.sblocal_attention',
                  'src.models.attention.local_attention': 'fly_amd.local_attention',
                  'src.models.attention.blocksparse_attention': 'fly_amd.blocksparse_attention',
                  'src.models.attention.sbblocksparse_attention': 'fly_amd.sbblocksparse_attention',
                  'src.models.layers.mlp': 'fly_amd.t2t_vit',
                  }.get(module, module)
        return getattr(importlib.import_module(module), name)(*args, **{**cfg, **kwargs})
    return cfg


class BlockSparseAttention(nn.Module):
    """Softmax attention restricted to the nonzero blocks of ``sparsity_config.make_layout``.

    sparsity_config: an object with ``.block`` and ``.make_layout(seq_len) -> (H, nb, nb)`` or a
    mapping with ``_target_``.  Same forward convention as the reference: query (B,T,H,E), key
    (B,S,H,E), value (B,S,H,D), optional FullMask attn_mask and key_padding_mask, returns
    (out (B,T,H,D), attn or None)."""

    def __init__(self, sparsity_config, softmax_temp=None, attention_dropout=0.1, max_seq_length=2048):
        super().__init__()
        self.sparsity_config = instantiate(sparsity_config)
        self.softmax_temp = softmax_temp
        self.dropout = nn.Dropout(attention_dropout)
        master_layout = self.sparsity_config.make_layout(max_seq_length)
        self.register_buffer("master_layout", master_layout)
        self._need_layout_synchronization = True
        self.ops_cache = dict()
        self.fused_cache = dict()
        self._layout_cache = dict()
        # forward passes that need neither gradients nor attention weights run as ONE kernel (no score
        # tensor in memory), dropout included; set to False to force the three ops
        self.fuse = True

    def get_layout(self, T, S=None):
        if S is None:
            S = T
        if self._need_layout_synchronization and dist.is_available() and dist.is_initialized():
            dist.broadcast(self.master_layout, src=0)
            self._need_layout_synchronization = False
        block = self.sparsity_config.block
        if (T % block != 0) or (S % block != 0):
            raise ValueError(f'Sequence lengths, {T} and {S}, needs to be divisible by block size {block}!')
        # the host copy is made once per shape: the master layout does not change after construction
        # (and synchronisation; the key carries its address and version counter in case it is replaced or
        # loaded into), and a device-to-host copy per call would stall the stream
        key = (T, S, self.master_layout.data_ptr(), self.master_layout._version)
        if key not in self._layout_cache:
            self._layout_cache[key] = self.master_layout[..., :T // block, :S // block].cpu()
        return self._layout_cache[key]

    def get_ops(self, T, S=None):
        if S is None:
            S = T
        if (T, S) not in self.ops_cache:
            layout = self.get_layout(T, S)
            block = self.sparsity_config.block
            self.ops_cache[T, S] = (matmul(layout, block, 'sdd', trans_a=False, trans_b=True),
                                    matmul(layout, block, 'dsd', trans_a=False, trans_b=False),
                                    softmax(layout, block))
        return self.ops_cache[T, S]

    def forward(self, query, key, value, attn_mask=None, key_padding_mask=None, need_weights=False):
        block = self.sparsity_config.block
        _, q_seqlen_og, n_head, q_dim_og = query.shape
        k_seqlen_og = key.shape[1]
        v_dim_og = value.shape[3]
        query = pad_to_multiple(query, block, dims=(1, 3))          # :107-109
        key = pad_to_multiple(key, block, dims=(1, 3))
        value = pad_to_multiple(value, block, dims=(1, 3))
        B, T, H, E = query.shape
        S = value.shape[1]
        softmax_temp = self.softmax_temp or 1 / math.sqrt(q_dim_og)  # :114

        if S > k_seqlen_og:                                          # :117-123
            if key_padding_mask is None:
                key_padding_mask = LengthMask(key.new_full((key.shape[0],), k_seqlen_og, dtype=torch.long),
                                              max_len=S)
            else:
                key_padding_mask = pad_mask(key_padding_mask, pad_length=S - k_seqlen_og, left=False,
                                            value=False)
        if attn_mask is not None and (S > k_seqlen_og or T > q_seqlen_og):   # :125-127
            attn_mask = FullMask(F.pad(attn_mask._mask, (0, S - k_seqlen_og, 0, T - q_seqlen_og), value=False))

        # the kernels read (B,T,H,E) through strides: no permuted copies (the reference makes
        # contiguous (B,H,T,E) tensors at :130-132)
        q, k, v = (x.permute(0, 2, 1, 3) for x in (query, key, value))
        layout = self.get_layout(T, S)
        needs_grad = torch.is_grad_enabled() and any(x.requires_grad for x in (query, key, value))
        # training-mode dropout (:160) runs inside the kernels: the mask is a hash of (seed, batch, head, query, key),
        # the seed drawn per call from torch's CPU generator (torch.manual_seed makes it repeatable) and kept in
        # last_dropout_seed
        dropout = (0.0, 0)
        if self.training and self.dropout.p > 0:
            dropout = (float(self.dropout.p), int(torch.randint(0, 2 ** 62, (1,)).item()))
        self.last_dropout_seed = None                       # set where a kernel uses the seed
        if (self.fuse and not need_weights and not needs_grad and dropout[0] < 1.0
                and fused_attention.supports(block, query.dtype, E, value.shape[3])):
            if (T, S) not in self.fused_cache:
                self.fused_cache[T, S] = fused_attention(layout, block)
            key_mask = add_mask = None
            if key_padding_mask is not None and not key_padding_mask.all_ones:
                key_mask = key_padding_mask.additive_matrix
            if attn_mask is not None and not attn_mask.all_ones:
                add_mask = attn_mask.additive_matrix        # (T, S), read per nonzero block inside the kernel
            out = self.fused_cache[T, S](q, k, v, softmax_temp, key_mask, attn_mask=add_mask, dropout=dropout)
            self.last_dropout_seed = dropout[1] if dropout[0] > 0 else None
            return _cut(out.permute(0, 2, 1, 3), q_seqlen_og, v_dim_og), None
        sdd_nt, dsd_nn, sparse_softmax = self.get_ops(T, S)
        unmasked = ((key_padding_mask is None or key_padding_mask.all_ones)
                    and (attn_mask is None or attn_mask.all_ones))
        one_kernel = self.fuse and fused_attention.supports(block, query.dtype, E, value.shape[3])
        if one_kernel and not unmasked:
            # with masks: the backward kernels that read them take head dims up to 64 and no dropout (with masks AND
            # dropout a training step stays on the three ops below)
            one_kernel = (needs_grad and dropout[0] == 0.0 and E in (32, 64)
                          and len(sdd_nt._table('union_t', query.device)) == 3)
        if (needs_grad and not need_weights and (dropout[0] == 0.0 or (one_kernel and dropout[0] < 1.0))
                and E == value.shape[3] and _AttentionCoreFn.supports(sdd_nt, block, query.dtype, E, query.device)):
            fused = None
            if one_kernel:
                if (T, S) not in self.fused_cache:
                    self.fused_cache[T, S] = fused_attention(layout, block)
                fused = self.fused_cache[T, S]
            self.last_dropout_seed = dropout[1] if dropout[0] > 0 else None
            out = _AttentionCoreFn.apply(
                q, k, v, sdd_nt, dsd_nn, sparse_softmax, softmax_temp,
                None if unmasked or key_padding_mask is None else key_padding_mask.additive_matrix,
                None if unmasked or attn_mask is None else attn_mask.additive_matrix, fused, dropout)
            return _cut(out.permute(0, 2, 1, 3), q_seqlen_og, v_dim_og), None
        qk = sdd_nt(q, k)
        attn = sparse_softmax(qk, scale=softmax_temp,
                              key_padding_mask=None if key_padding_mask is None else key_padding_mask.additive_matrix,
                              attn_mask=None if attn_mask is None else attn_mask.additive_matrix,
                              key_padding_mask_mode='add', attn_mask_mode='add')
        if ((key_padding_mask is not None and not key_padding_mask.all_ones)
                or (attn_mask is not None and not attn_mask.all_ones)):
            # :156-158: fully masked rows -> 0 (out of place under autograd: the softmax keeps its
            # output for the backward pass)
            attn = attn.nan_to_num() if attn.requires_grad else attn.nan_to_num_()
        out = dsd_nn(self.dropout(attn), v)
        weights = None
        if need_weights:
            weights = densify_tensor(attn, layout)[:, :, :q_seqlen_og, :k_seqlen_og]
        return _cut(out.permute(0, 2, 1, 3), q_seqlen_og, v_dim_og), weights
