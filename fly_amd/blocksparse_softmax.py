"""Row operations over block-sparse matrices on the HIP kernels.

`softmax` replaces the third-party ``triton.ops.blocksparse.softmax`` the reference imports
(src/models/attention/blocksparse_attention.py:14, call :146-152); `logsumexp` and
`blocksparse_sum` replace src/models/attention/blocksparse_logsumexp.py:161-184 and
blocksparse_sum.py:156-179.
"""
import torch

from . import _lib
from .blocksparse_utils import _as_layout3, row_table


class _RowOp:
    def __init__(self, layout, block, bench=False):
        self.layout = _as_layout3(layout)
        self.spdims = self.layout.shape
        self.block = block
        self.bench = bench
        self.lut_cache = dict()

    def make_lut(self, device):
        """(row_ptr, row_blk, row_col, max_row_nnz) on `device`, cached per device."""
        key = (device,)
        if key not in self.lut_cache:
            ptr, blk, col, max_nnz = row_table(self.layout)
            self.lut_cache[key] = (ptr.to(device), blk.to(device), col.to(device), max_nnz)
        return self.lut_cache[key]

    def _check(self, x):
        if not x.is_cuda:
            raise ValueError('Only GPU devices are supported for now')
        nnz = int(self.layout.sum())
        if x.dim() != 4 or tuple(x.shape[1:]) != (nnz, self.block, self.block):
            raise ValueError(f'expected a sparse tensor (Z, {nnz}, {self.block}, {self.block}), got {tuple(x.shape)}')


def _mask_arg(mask, mode, rows, cols, name, device):
    if mask is None:
        return None, 0, 0
    if mode not in ('add', 'mul'):
        raise ValueError(f'{name}_mode must be "add" or "mul"')
    if tuple(mask.shape) != (rows, cols):
        raise ValueError(f'{name} must have shape ({rows}, {cols}), got {tuple(mask.shape)}')
    mask = mask.to(device=device, dtype=torch.float32).contiguous()
    return mask, mask.stride(0), int(mode == 'mul')


class softmax(_RowOp):
    """``softmax(layout, block)(x, scale=1., rpe=None, key_padding_mask=None, attn_mask=None,
    key_padding_mask_mode='add', attn_mask_mode='add')`` -- IN PLACE row softmax over the nonzero
    blocks of x*scale + key_padding_mask[z, col] + attn_mask[row, col]; returns x.  Rows without any
    finite entry become NaN like in the kernel it replaces (the attention layer clears them)."""

    def __call__(self, x, scale=1., rpe=None, key_padding_mask=None, attn_mask=None,
                 key_padding_mask_mode='add', attn_mask_mode='add'):
        if rpe is not None:
            raise NotImplementedError('relative position embeddings are not supported')
        self._check(x)
        if not x.is_contiguous():
            raise ValueError('the sparse tensor must be contiguous (it is updated in place)')
        H, p, r = self.spdims
        Z = x.shape[0]
        kpm, kpm_stride, kpm_mul = _mask_arg(key_padding_mask, key_padding_mask_mode, Z, r * self.block,
                                             'key_padding_mask', x.device)
        am, am_stride, am_mul = _mask_arg(attn_mask, attn_mask_mode, p * self.block, r * self.block,
                                          'attn_mask', x.device)
        ptr, blk, col, max_nnz = self.make_lut(x.device)
        with torch.cuda.device(x.device):
            _lib.call('flyhip_bs_softmax', x.data_ptr(), ptr.data_ptr(), blk.data_ptr(), col.data_ptr(),
                      H * p, p, max_nnz, Z, self.block, x.stride(0), float(scale),
                      _lib.ptr(kpm), kpm_stride, kpm_mul, _lib.ptr(am), am_stride, am_mul,
                      _lib.dtype_code(x), _lib.stream_ptr(x.device))
        return x


class _Reduce(_RowOp):
    op_code = None

    def __call__(self, x):
        self._check(x)
        x = x.contiguous()
        H, p, r = self.spdims
        Z = x.shape[0]
        ptr, blk, col, _ = self.make_lut(x.device)
        out = torch.empty((Z, H, p * self.block), dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            _lib.call('flyhip_bs_rowreduce', x.data_ptr(), out.data_ptr(), ptr.data_ptr(), blk.data_ptr(),
                      H * p, Z, self.block, x.stride(0), self.op_code, _lib.dtype_code(x),
                      _lib.stream_ptr(x.device))
        return out


class logsumexp(_Reduce):
    """Row logsumexp over the nonzero blocks -> (Z, H, M); 0 for rows of empty block-rows."""
    op_code = 0


class blocksparse_sum(_Reduce):
    """Row sum over the nonzero blocks -> (Z, H, M)."""
    op_code = 1
