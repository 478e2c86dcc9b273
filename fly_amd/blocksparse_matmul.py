"""Block-sparse matmul operator on the HIP kernels: drop-in for the `matmul` class of
src/models/attention/blocksparse_matmul.py:590-719 (modes 'sdd', 'dsd', 'dds')."""
import torch

from . import _lib
from .blocksparse_utils import group_table, sdd_table, segment_table, union_table

# Sharing the dense operand's tiles among four block-rows pays when the rows have columns in
# common: the union tables are passed to the kernels when the layout has at least this many
# (row, column) pairs per union column on average.
UNION_MIN_SHARING = 1.5
# sdd with both operands contraction-major (a^T b) takes the split-K kernel from this contraction length on
KMAJOR_MIN_K = 512

_BLOCKS = (16, 32, 64, 128)


def _aligned(x):
    return x.data_ptr() % 16 == 0 and all(s % 4 == 0 for s, n in zip(x.stride(), x.shape) if n > 1 and s != 1)


def _dense_operand(x):
    """Dense operands are read through strides; fall back to a contiguous copy only when neither of
    the two matrix dims is unit-stride or vector alignment fails."""
    if (x.stride(-1) == 1 or x.stride(-2) == 1) and _aligned(x):
        return x
    return x.contiguous()


class _MatmulFn(torch.autograd.Function):
    """c = op(a) @ op(b) with one sparse participant; backward re-uses the same three kernels with
    permuted roles exactly as blocksparse_matmul.py:562-587 does."""

    @staticmethod
    def forward(ctx, a, b, op):
        ctx.save_for_backward(a, b)
        ctx.op = op
        return op._run(op.mode, a, b, op.trans_a, op.trans_b, False)

    @staticmethod
    def backward(ctx, dc):
        a, b = ctx.saved_tensors
        op = ctx.op
        mode = op.mode
        da = db = None
        if ctx.needs_input_grad[0]:
            mode_da = mode[1] + mode[0] + mode[2]
            da = op._run(mode_da, dc, b, False, not op.trans_b, op.trans_a)
        if ctx.needs_input_grad[1]:
            mode_db = mode[2] + mode[1] + mode[0]
            db = op._run(mode_db, a, dc, not op.trans_a, False, op.trans_b)
        return da, db, None


class matmul:
    """``matmul(layout, block, mode, trans_a=False, trans_b=False)(a, b)``.

    mode 'sdd': sparse = op(a) @ op(b), a, b dense (Z,H,.,.)           -> (Z, nnz, blk, blk)
    mode 'dsd': dense  = op(a) @ op(b), a sparse (Z,nnz,blk,blk)       -> (Z, H, M, N)
    mode 'dds': dense  = op(a) @ op(b), b sparse                       -> (Z, H, M, N)
    layout (H, rows, cols) of 0/1 (2-D means one head).  Shape, device and dtype problems raise
    ValueError before anything is launched, as the reference's _validate_inputs does (:678-702).
    """

    def __init__(self, layout, block, mode, trans_a=False, trans_b=False):
        if mode not in ['sdd', 'dsd', 'dds']:
            raise NotImplementedError('Supported modes are: sdd, dsd, dds')
        if block not in _BLOCKS:
            raise NotImplementedError(f'block size {block} not in {_BLOCKS}')
        assert layout.ndim in (2, 3), "Layout should be a 2 or 3 dimensional tensor of 0s and 1s"
        self.block, self.mode, self.trans_a, self.trans_b = block, mode, trans_a, trans_b
        self.lut_cache = dict()
        self.layout = _as_heads(layout)            # (H, block-rows, block-cols), integral; 2-D means one head
        self.spdims = self.layout.shape
        if mode != 'sdd':
            # The contraction runs over one axis of the sparse operand's layout and one dim of the dense
            # operand: sparse first ('dsd') contracts its columns unless transposed, and meets dim -2 of
            # op(b); dense first ('dds') contracts dim -1 of op(a) with the sparse operand's rows.
            if mode == 'dsd':
                layout_axis, self.dense_inner_dim = (-2 if trans_a else -1), (-1 if trans_b else -2)
            else:
                layout_axis, self.dense_inner_dim = (-1 if trans_b else -2), (-2 if trans_a else -1)
            self.dense_inner_size = self.layout.shape[layout_axis] * block
            self.sparse_shape = (int(self.layout.sum()), block, block)

    # ------------------------------------------------------------------ tables
    def _table(self, kind, device):
        key = (kind, device)
        if key not in self.lut_cache:
            if kind == 'sdd':
                tabs = (sdd_table(self.layout),)
            elif kind in ('grp_rows', 'grp_cols'):
                tabs = group_table(self.layout, by_rows=(kind == 'grp_rows'))
            elif kind in ('union', 'union_t'):
                tabs = union_table(self.layout, transposed=(kind == 'union_t'))
                if int(self.layout.sum()) < UNION_MIN_SHARING * tabs[1].numel():
                    tabs = ()
            else:
                tabs = segment_table(self.layout, by_rows=(kind == 'rows'))
            self.lut_cache[key] = tuple(t.to(device) for t in tabs)
        return self.lut_cache[key]

    def make_lut(self, dtype, device):
        """Build (and cache) the index tables this op needs on `device`; dtype is accepted for
        signature compatibility (:591) -- the tables do not depend on it."""
        if self.mode == 'sdd':
            return self._table('sdd', device)
        by_rows = (not self.trans_a) if self.mode == 'dsd' else self.trans_b
        return self._table('rows' if by_rows else 'cols', device)

    # ------------------------------------------------------------------ call
    def __call__(self, a, b):
        original_dims = max(a.ndim, b.ndim)
        a, b = self._validate_inputs(a, b)
        c = _MatmulFn.apply(a, b, self)
        for _ in range(c.ndim - original_dims):
            c = c.squeeze(0)
        return c

    def _validate_inputs(self, a, b):
        """Device, dtype and shape checks with the reference's messages (:678-702); returns both
        operands as 4-D views (leading singleton dims added)."""
        if a.device != b.device:
            raise ValueError(f"Inputs must be on the same device; got {a.device} for tensor A "
                             f"and {b.device} for tensor B")
        if not a.is_cuda:
            raise ValueError("Only GPU devices are supported for now")
        if torch.is_autocast_enabled():            # like torch.matmul under autocast
            a, b = a.half(), b.half()
        elif a.dtype != b.dtype:
            raise ValueError(f"Inputs must be the same dtype; got {a.dtype} for A and {b.dtype} for B")
        if self.mode != 'sdd':
            (dense, dense_name), (sparse, sparse_name) = ((a, 'A'), (b, 'B')) if self.mode == 'dds' else ((b, 'B'), (a, 'A'))
            got = dense.shape[self.dense_inner_dim]
            if got != self.dense_inner_size:
                raise ValueError(f"Expected tensor {dense_name} to have size {self.dense_inner_size} at dim "
                                 f"{self.dense_inner_dim % dense.ndim}, got {got}.")
            if tuple(sparse.shape[-3:]) != self.sparse_shape:
                raise ValueError(f"Expected tensor with trailing dimensions of shape {self.sparse_shape} for argument "
                                 f"{sparse_name}, got {sparse.shape}")
        for x in (a, b):
            if x.ndim > 4:
                raise ValueError("Tensors with more than 4 dimensions are not currently supported")
        return tuple(x.reshape((1,) * (4 - x.ndim) + tuple(x.shape)) if x.ndim < 4 else x for x in (a, b))

    # ------------------------------------------------------------------ kernels
    def _run(self, mode, a, b, trans_a, trans_b, trans_c):
        return {'sdd': self._sdd, 'dsd': self._dsd, 'dds': self._dds}[mode](a, b, trans_a, trans_b, trans_c)

    def _sdd(self, a, b, trans_a, trans_b, trans_c):
        if trans_c:                                  # (A B)^T = B^T A^T   (:281-283)
            a, b = b, a
            trans_a, trans_b = not trans_b, not trans_a
        a, b = _dense_operand(a), _dense_operand(b)
        a_dim, b_dim = (-2 if trans_a else -1), (-1 if trans_b else -2)
        K, Kb = a.shape[a_dim], b.shape[b_dim]
        if K != Kb:
            raise ValueError(f"Size of tensor A along the {_dim_to_name(a_dim)} dim ({K}) must match size "
                             f"of tensor B along the {_dim_to_name(b_dim)} dim ({Kb})")
        if K % 16 != 0:
            raise ValueError('Reduction size for SDD must be a multiple of 16')
        H, p, r = self.spdims
        Z = a.shape[0]
        M = a.shape[3 if trans_a else 2]
        N = b.shape[2 if trans_b else 3]
        if a.shape[1] != H or b.shape[1] != H or b.shape[0] != Z or M != p * self.block or N != r * self.block:
            raise ValueError(f'SDD operands {tuple(a.shape)}, {tuple(b.shape)} do not match layout '
                             f'{tuple(self.spdims)} with block {self.block}')
        if int(self.layout.sum()) == 0:              # a layout without blocks: nothing to compute or launch
            return torch.empty((Z, 0, self.block, self.block), dtype=a.dtype, device=a.device)
        if (trans_a and not trans_b and self.block == 32 and a.dtype in (torch.bfloat16, torch.float16)
                and K >= KMAJOR_MIN_K and a.stride(3) == 1 and b.stride(3) == 1
                and all(s % 8 == 0 for s in a.stride()[:3] + b.stride()[:3])):
            return self._sdd_kmajor(a, b, Z, K)
        (lut,) = self._table('sdd', a.device)
        row_ptr, row_blk, row_col = self._table('rows', a.device)
        uni = [t.data_ptr() for t in self._table('union', a.device)] or [None] * 3
        nnz = lut.shape[0]
        c = torch.empty((Z, nnz, self.block, self.block), dtype=a.dtype, device=a.device)
        a_sm, a_sk = (a.stride(3), a.stride(2)) if trans_a else (a.stride(2), a.stride(3))
        b_sn, b_sk = (b.stride(2), b.stride(3)) if trans_b else (b.stride(3), b.stride(2))
        with torch.cuda.device(a.device):
            _lib.call('flyhip_bs_sdd', a.data_ptr(), b.data_ptr(), c.data_ptr(), lut.data_ptr(), nnz,
                      row_ptr.data_ptr(), row_blk.data_ptr(), row_col.data_ptr(), H * p, p, *uni,
                      Z, K, self.block, a.stride(0), a.stride(1), a_sm, a_sk,
                      b.stride(0), b.stride(1), b_sn, b_sk, _lib.dtype_code(a), _lib.stream_ptr(a.device))
        return c

    def _sdd_kmajor(self, a, b, Z, K):
        """sparse = a^T b with the contraction index slowest in both operands and long (the weight
        gradient of a block-sparse linear layer: K = tokens): split over K, accumulated in fp32."""
        H, p, r = self.spdims
        row_ptr, row_blk, row_col = self._table('rows', a.device)
        grp_row0, grp_n = self._table('grp_rows', a.device)
        nnz = int(self.layout.sum())
        max_row_nnz = int(self.layout.sum(-1).max())
        tiles = grp_row0.shape[0] * ((max_row_nnz + 3) // 4) * Z
        slices = max(1, min(K // 256, -(-2048 // tiles)))       # about eight workgroups per CU
        k_slice = -(-(-(-K // slices)) // 32) * 32
        c32 = torch.zeros((Z, nnz, 32, 32), dtype=torch.float32, device=a.device)
        with torch.cuda.device(a.device):
            _lib.call('flyhip_bs_sdd_kmajor', a.data_ptr(), b.data_ptr(), c32.data_ptr(),
                      row_ptr.data_ptr(), row_blk.data_ptr(), row_col.data_ptr(),
                      grp_row0.data_ptr(), grp_n.data_ptr(), grp_row0.shape[0], max_row_nnz,
                      p, nnz, Z, K, k_slice, 32, a.stride(0), a.stride(1), a.stride(2),
                      b.stride(0), b.stride(1), b.stride(2), _lib.dtype_code(a), _lib.stream_ptr(a.device))
        return c32.to(a.dtype)

    def _dsd(self, a, b, trans_a, trans_b, trans_c):
        b = _dense_operand(b)
        a = a.contiguous()
        H, p, r = self.spdims
        by_rows = not trans_a
        seg_ptr, seg_blk, seg_inner = self._table('rows' if by_rows else 'cols', b.device)
        uni = [t.data_ptr() for t in self._table('union' if by_rows else 'union_t', b.device)] or [None] * 3
        per_head = p if by_rows else r
        M = per_head * self.block
        Z = b.shape[0]
        N = b.shape[2 if trans_b else 3]
        b_sk, b_sn = (b.stride(3), b.stride(2)) if trans_b else (b.stride(2), b.stride(3))
        c = torch.empty((Z, H, N, M) if trans_c else (Z, H, M, N), dtype=b.dtype, device=b.device)
        c_sm, c_sn = (c.stride(3), c.stride(2)) if trans_c else (c.stride(2), c.stride(3))
        with torch.cuda.device(b.device):
            _lib.call('flyhip_bs_dsd', a.data_ptr(), b.data_ptr(), c.data_ptr(),
                      seg_ptr.data_ptr(), seg_blk.data_ptr(), seg_inner.data_ptr(), *uni,
                      H * per_head, per_head, Z, N, self.block, int(trans_a), a.stride(0),
                      b.stride(0), b.stride(1), b_sk, b_sn, c.stride(0), c.stride(1), c_sm, c_sn,
                      _lib.dtype_code(b), _lib.stream_ptr(b.device))
        return c

    def _dds(self, a, b, trans_a, trans_b, trans_c):
        if trans_a and trans_c and not trans_b:
            # (a^T b)^T = b^T a: the same numbers as a dsd with the sparse operand transposed, which has
            # a tiled kernel (this is the gradient of the second operand of an sdd, e.g. dK = dS^T Q)
            return self._dsd(b, a, True, False, False)
        a = _dense_operand(a)
        b = b.contiguous()
        H, p, r = self.spdims
        by_rows = trans_b
        seg_ptr, seg_blk, seg_inner = self._table('rows' if by_rows else 'cols', a.device)
        grp_row0, grp_n = self._table('grp_rows' if by_rows else 'grp_cols', a.device)
        per_head = p if by_rows else r
        N = per_head * self.block
        Z = a.shape[0]
        M = a.shape[3 if trans_a else 2]
        a_sm, a_sk = (a.stride(3), a.stride(2)) if trans_a else (a.stride(2), a.stride(3))
        c = torch.empty((Z, H, N, M) if trans_c else (Z, H, M, N), dtype=a.dtype, device=a.device)
        c_sm, c_sn = (c.stride(3), c.stride(2)) if trans_c else (c.stride(2), c.stride(3))
        with torch.cuda.device(a.device):
            _lib.call('flyhip_bs_dds', a.data_ptr(), b.data_ptr(), c.data_ptr(),
                      seg_ptr.data_ptr(), seg_blk.data_ptr(), seg_inner.data_ptr(),
                      grp_row0.data_ptr(), grp_n.data_ptr(), grp_row0.shape[0],
                      int(self.layout.sum(-1 if by_rows else -2).max()),
                      H * per_head, per_head, Z, M, self.block, int(trans_b),
                      a.stride(0), a.stride(1), a_sm, a_sk, b.stride(0),
                      c.stride(0), c.stride(1), c_sm, c_sn, _lib.dtype_code(a), _lib.stream_ptr(a.device))
        return c


def _as_heads(layout):
    return (layout.unsqueeze(0) if layout.ndim == 2 else layout).long()


def _dim_to_name(x):
    return "last" if x == -1 else "second to last"
