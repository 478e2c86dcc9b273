"""Fused block-sparse attention on the HIP kernel: the SDD -> block softmax -> DSD sequence of
src/models/attention/blocksparse_attention.py:134-160 as one launch that never materialises the
(Z, nnz, block, block) score / probability tensor."""
import torch

from . import _lib
from .blocksparse_utils import _as_layout3, union_table


class fused_attention:
    """``fused_attention(layout, block)(q, k, v, scale, key_mask=None, attn_mask=None)`` with q (Z,H,rows,D),
    k / v (Z,H,cols,D) (any batch / head / row strides, D contiguous) returns
    softmax(scale * q k^T + key_mask[z, col] + attn_mask[row, col]) v over the nonzero blocks of `layout`, shaped
    (Z,H,rows,D) over memory laid out (Z,rows,H,D).  key_mask: fp32 (Z, cols), attn_mask: fp32 (rows, cols), both
    additive (0 / -inf from the mask classes, blocksparse_attention.py:146-152).  ``dropout=(p, seed)`` with p > 0
    drops probabilities the way ``self.dropout(attn)`` of blocksparse_attention.py:160 does -- after the softmax,
    kept ones scaled by 1 / (1 - p) -- with the mask a hash of (seed, batch, head, query, key) formed inside the
    kernel instead of a stored tensor.  Forward only, 32x32 blocks of bf16 / fp16, D in {32,64,128}: `supports()`
    says whether a call qualifies."""

    def __init__(self, layout, block, rows_per_group=8):
        self.layout = _as_layout3(layout)
        self.spdims = self.layout.shape
        self.block = block
        self.rows_per_group = rows_per_group
        self.lut_cache = dict()

    @staticmethod
    def supports(block, dtype, q_dim, v_dim):
        return (block == 32 and dtype in (torch.bfloat16, torch.float16) and q_dim == v_dim
                and q_dim in (32, 64, 128))

    def make_lut(self, device):
        if device not in self.lut_cache:
            self.lut_cache[device] = tuple(t.to(device) for t in union_table(self.layout, self.rows_per_group))
        return self.lut_cache[device]

    def __call__(self, q, k, v, scale, key_mask=None, return_lse=False, attn_mask=None, dropout=(0.0, 0)):
        _lib.require_gpu(q, k, v)
        H, p, r = self.spdims
        Z, D = q.shape[0], q.shape[3]
        if not self.supports(self.block, q.dtype, D, v.shape[3]) or k.dtype != q.dtype or v.dtype != q.dtype:
            raise NotImplementedError('fused block-sparse attention needs 32x32 blocks, bf16 / fp16 inputs of one '
                                      'dtype and equal head dims in {32,64,128}')
        if (tuple(q.shape) != (Z, H, p * 32, D) or tuple(k.shape) != (Z, H, r * 32, D)
                or tuple(v.shape) != (Z, H, r * 32, D)):
            raise ValueError(f'operands {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)} do not match layout '
                             f'{tuple(self.spdims)} with block 32')

        def aligned(x):          # 16-byte vector loads: D contiguous, other strides multiples of 8
            ok = x.stride(3) == 1 and all(s % 8 == 0 for s in x.stride()[:3]) and x.data_ptr() % 16 == 0
            return x if ok else x.contiguous()
        q, k, v = aligned(q), aligned(k), aligned(v)
        km, km_stride = None, 0
        if key_mask is not None:
            if tuple(key_mask.shape) != (Z, r * 32):
                raise ValueError(f'key_mask must have shape ({Z}, {r * 32}), got {tuple(key_mask.shape)}')
            key_mask = key_mask.to(device=q.device, dtype=torch.float32).contiguous()
            km, km_stride = key_mask.data_ptr(), key_mask.stride(0)
        am, am_stride = None, 0
        if attn_mask is not None:
            if tuple(attn_mask.shape) != (p * 32, r * 32):
                raise ValueError(f'attn_mask must have shape ({p * 32}, {r * 32}), got {tuple(attn_mask.shape)}')
            attn_mask = attn_mask.to(device=q.device, dtype=torch.float32).contiguous()
            am, am_stride = attn_mask.data_ptr(), attn_mask.stride(0)
        uni_ptr, uni_inner, uni_blk = self.make_lut(q.device)
        if uni_inner.numel() == 0:                      # a layout without blocks: every row is empty
            out = torch.zeros((Z, p * 32, H, D), dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)
            lse2 = torch.full((Z, H, p * 32), float('inf'), dtype=torch.float32, device=q.device)
            return (out, lse2) if return_lse else out
        out = torch.empty((Z, p * 32, H, D), dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)
        # base-2 log of every row's softmax denominator (+inf for a row without a finite score): what a
        # backward pass needs to form the probabilities again
        lse2 = torch.empty((Z, H, p * 32), dtype=torch.float32, device=q.device) if return_lse else None
        drop_p, drop_seed = float(dropout[0]), int(dropout[1])
        if not 0.0 <= drop_p < 1.0:
            raise ValueError(f'dropout probability {drop_p} not in [0, 1)')
        with torch.cuda.device(q.device):
            common = (q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _lib.ptr(lse2),
                      uni_ptr.data_ptr(), uni_inner.data_ptr(), uni_blk.data_ptr(), self.rows_per_group,
                      km, km_stride, am, am_stride, Z, H, p, D, 32,
                      q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
                      v.stride(0), v.stride(1), v.stride(2), out.stride(0), out.stride(1), out.stride(2),
                      float(scale), _lib.dtype_code(q))
            if drop_p > 0.0:
                _lib.call('flyhip_bs_attn_dropout', *common, drop_p, drop_seed, _lib.stream_ptr(q.device))
            else:
                _lib.call('flyhip_bs_attn_masks', *common, _lib.stream_ptr(q.device))
        return (out, lse2) if return_lse else out
