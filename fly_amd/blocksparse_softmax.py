"""Row operations over block-sparse matrices on the HIP kernels.

`softmax` replaces the third-party ``triton.ops.blocksparse.softmax`` the reference imports
(src/models/attention/blocksparse_attention.py:14, call :146-152); `logsumexp` and
`blocksparse_sum` replace src/models/attention/blocksparse_logsumexp.py:161-184 and
blocksparse_sum.py:156-179.
"""
import torch

from . import _lib
from .blocksparse_utils import _as_layout3, row_table, sparsify_broadcast_tensor


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
        return _SoftmaxFn.apply(x, self, float(scale), (kpm, kpm_stride, kpm_mul), (am, am_stride, am_mul))

    def _launch(self, x, scale, kpm_args, am_args):
        H, p, r = self.spdims
        kpm, kpm_stride, kpm_mul = kpm_args
        am, am_stride, am_mul = am_args
        ptr, blk, col, max_nnz = self.make_lut(x.device)
        with torch.cuda.device(x.device):
            _lib.call('flyhip_bs_softmax', x.data_ptr(), ptr.data_ptr(), blk.data_ptr(), col.data_ptr(),
                      H * p, p, max_nnz, x.shape[0], self.block, x.stride(0), scale,
                      _lib.ptr(kpm), kpm_stride, kpm_mul, _lib.ptr(am), am_stride, am_mul,
                      _lib.dtype_code(x), _lib.stream_ptr(x.device))


class _SoftmaxFn(torch.autograd.Function):
    """In-place block softmax y = softmax(scale * x + masks); backward dx = scale * y * (dy - rowsum(dy * y))
    with the row sums on the row-reduction kernel (the kernel it replaces differentiates the same way)."""

    @staticmethod
    def forward(ctx, x, op, scale, kpm_args, am_args):
        op._launch(x, scale, kpm_args, am_args)
        ctx.mark_dirty(x)
        ctx.save_for_backward(x)
        ctx.op, ctx.scale = op, scale
        ctx.masked = kpm_args[0] is not None or am_args[0] is not None
        return x

    @staticmethod
    def backward(ctx, dy):
        (y,) = ctx.saved_tensors
        op = ctx.op
        if ctx.masked:
            # a row whose every entry was masked came out as NaN; it has no gradient (the caller has
            # replaced it by zeros, blocksparse_attention.py:156-158), and 0 * NaN must not leak into dx
            y = y.nan_to_num()
        ptr, blk, col, max_nnz = op.make_lut(y.device)
        if (op.block == 32 and y.dtype in (torch.bfloat16, torch.float16) and max_nnz <= 64
                and y.stride(0) % 8 == 0):
            dy = dy.contiguous()
            dx = torch.empty_like(y)
            H, p, r = op.spdims
            with torch.cuda.device(y.device):
                _lib.call('flyhip_bs_softmax_bwd', y.data_ptr(), dy.data_ptr(), dx.data_ptr(), ptr.data_ptr(),
                          blk.data_ptr(), H * p, max_nnz, y.shape[0], 32, y.stride(0), ctx.scale,
                          _lib.dtype_code(y), _lib.stream_ptr(y.device))
            return dx, None, None, None, None
        dyy = (dy * y).contiguous()
        rows = _reduce_rows(op, dyy, 1)                                   # (Z, H, M)
        dx = (dyy - y * sparsify_broadcast_tensor(rows, op.layout, op.block)) * ctx.scale
        return dx, None, None, None, None


def _reduce_rows(op, x, op_code):
    H, p, r = op.spdims
    Z = x.shape[0]
    ptr, blk, col, _ = op.make_lut(x.device)
    out = torch.empty((Z, H, p * op.block), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _lib.call('flyhip_bs_rowreduce', x.data_ptr(), out.data_ptr(), ptr.data_ptr(), blk.data_ptr(),
                  H * p, Z, op.block, x.stride(0), op_code, _lib.dtype_code(x), _lib.stream_ptr(x.device))
    return out


class _Reduce(_RowOp):
    op_code = None

    def __call__(self, x):
        self._check(x)
        return _ReduceFn.apply(x.contiguous(), self)


class _ReduceFn(torch.autograd.Function):
    """Row logsumexp / sum with their gradients (blocksparse_logsumexp.py:63-102, blocksparse_sum.py):
    d logsumexp = exp(x - lse[row]) * dout[row], d sum = dout[row], on the nonzero blocks."""

    @staticmethod
    def forward(ctx, x, op):
        out = _reduce_rows(op, x, op.op_code)
        ctx.save_for_backward(x, out)
        ctx.op = op
        return out

    @staticmethod
    def backward(ctx, dout):
        x, out = ctx.saved_tensors
        op = ctx.op
        d_rows = sparsify_broadcast_tensor(dout.contiguous(), op.layout, op.block)
        if op.op_code == 1:
            return d_rows.expand_as(x).contiguous(), None
        return torch.exp(x - sparsify_broadcast_tensor(out, op.layout, op.block)) * d_rows, None


class logsumexp(_Reduce):
    """Row logsumexp over the nonzero blocks -> (Z, H, M); 0 for rows of empty block-rows."""
    op_code = 0


class blocksparse_sum(_Reduce):
    """Row sum over the nonzero blocks -> (Z, H, M)."""
    op_code = 1
