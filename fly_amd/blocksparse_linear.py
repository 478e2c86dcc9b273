"""Pixelfly block-sparse linear layer on the HIP kernels: drop-in for
src/models/layers/blocksparse_linear.py (BlockSparseLinear :35-172,
FlatBlockButterflySparsityConfig :175-211)."""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn import init

from .blocksparse_attention import instantiate
from .blocksparse_matmul import matmul
from .blocksparse_utils import densify_tensor


class FlatBlockButterflySparsityConfig:
    """Sparsity pattern = sum of the first ``n_factors`` butterfly factors of size ``butterfly_size``
    ("flat butterfly"), stretched to the weight shape and reduced to blocks.

    Entry (i, j) of butterfly factor k (stride 2^k, all-ones twiddle) is nonzero iff j == i or
    j == i xor 2^k (src/ops/butterfly_factor.py:8-26), so the flat pattern is
    ``j in {i} U {i xor 2^k : k < n_factors}``; that closed form is evaluated directly here."""

    def __init__(self, butterfly_size, n_factors, block=32, global_size=0, shuffle=False):
        levels = butterfly_size.bit_length() - 1
        if butterfly_size < 2 or butterfly_size != 1 << levels:
            raise NotImplementedError(f'butterfly_size={butterfly_size}: only powers of two (>= 2) have butterfly factors')
        if n_factors < 1 or n_factors > levels:
            raise NotImplementedError(f'n_factors={n_factors}: a butterfly of size {butterfly_size} has factors 1..{levels}')
        self.butterfly_size, self.n_factors = butterfly_size, n_factors
        self.block, self.global_size, self.shuffle = block, global_size, shuffle

    def make_layout(self, out_features, in_features=None):
        """int32 (out_features/block, in_features/block) layout (:191-211).  A single argument means
        a square (seq, seq) attention layout."""
        if in_features is None:
            in_features = out_features
        if out_features % self.block or in_features % self.block:
            raise AssertionError(f'({out_features}, {in_features}) is not a whole number of {self.block}-blocks')
        n = self.butterfly_size
        i = torch.arange(n).view(n, 1)
        j = torch.arange(n).view(1, n)
        diff = i ^ j
        pattern = diff == 0
        for k in range(self.n_factors):
            pattern = pattern | (diff == (1 << k))
        if self.shuffle:                                   # channel shuffle of the columns (:196-200)
            ngroups = 2 ** (int(math.log2(n)) - self.n_factors)
            cols = torch.arange(n)
            dest = (cols % (n // ngroups)) * ngroups + cols // (n // ngroups)
            shuffled = torch.zeros_like(pattern)
            shuffled[:, dest] = pattern
            pattern = shuffled
        rows = torch.arange(out_features) // (out_features // n)      # butterfly cell of every row
        cols = torch.arange(in_features) // (in_features // n)
        dense = pattern[rows][:, cols]
        if self.global_size > 0:
            dense[:self.global_size] = True
            dense[:, :self.global_size] = True
        p, r = out_features // self.block, in_features // self.block
        return dense.view(p, self.block, r, self.block).any(dim=3).any(dim=1).int()


class BlockSparseLinear(nn.Module):
    """y = x W^T + b with W block-sparse.  `weight` holds the nonzero blocks in (out-block, in-block)
    row-major order, block content [out_local, in_local]: (1, nnz, blk, blk) for backend 'triton' (the
    name kept from the reference; it selects the HIP kernel, a DDS product with the sparse operand
    transposed), (nnz, blk, blk) for backend 'dense' (a library GEMM on the densified weight).
    'huggingface' (third-party pytorch_block_sparse) is not available.

    Attribute, buffer and parameter names, the initial distribution and the order of the random draws
    follow blocksparse_linear.py:41-109; the forward computes what :134-172 computes."""

    _BACKENDS = ('triton', 'dense')

    def __init__(self, in_features, out_features, sparsity_config, bias=True,
                 backend='triton', weight_decay=True):
        super().__init__()
        backend = 'triton' if backend is None else backend
        if backend == 'huggingface':
            raise ImportError('backend huggingface (pytorch_block_sparse) is not available in this build')
        if backend not in self._BACKENDS:
            raise NotImplementedError(f'backend {backend} not supported')
        self.backend = backend
        self.in_features, self.out_features = in_features, out_features
        self.sparsity_config = instantiate(sparsity_config)
        blk = self.block_size = self.sparsity_config.block
        self.in_features_extended = -(-in_features // blk) * blk
        self.out_features_extended = -(-out_features // blk) * blk
        self.register_buffer('layout', self.sparsity_config.make_layout(self.out_features_extended,
                                                                         self.in_features_extended))
        self.nnz_blocks = int(self.layout.sum())
        lead = (1,) if backend == 'triton' else ()
        self.weight = nn.Parameter(torch.empty(*lead, self.nnz_blocks, blk, blk))
        self.bias = nn.Parameter(torch.empty(out_features)) if bias else None
        self.reset_parameters()
        if not weight_decay:
            self.weight._no_weight_decay = True
        self.ops_cache = dict()

    def reset_parameters(self) -> None:
        """Kaiming-uniform(a = sqrt 5) on the dense matrix, then the bias from U(+-1/sqrt(fan_in)) with the
        padded fan-in (:91-96)."""
        self.set_weights_from_dense_init(dense_init_fn_=lambda w: init.kaiming_uniform_(w, a=math.sqrt(5)))
        if self.bias is not None and self.in_features_extended > 0:
            init.uniform_(self.bias, -self.in_features_extended ** -0.5, self.in_features_extended ** -0.5)

    def set_weights_from_dense_init(self, dense_init_fn_):
        """Draw a dense (out, in) matrix with `dense_init_fn_`, give every block-row the gain
        sqrt(#block-columns / #nonzero block-columns) so that the output variance survives the mask, and keep
        the nonzero blocks (:98-109)."""
        blk, layout = self.block_size, self.layout
        n_brow, n_bcol = layout.shape
        dense = self.weight.new_empty(self.out_features_extended, self.in_features_extended)
        dense_init_fn_(dense)
        gain = (n_bcol / layout.sum(dim=1).to(dense.dtype)).sqrt().to(dense.device)         # (n_brow,)
        tiles = dense.view(n_brow, blk, n_bcol, blk) * gain.view(n_brow, 1, 1, 1)
        brow, bcol = layout.to(dense.device).nonzero(as_tuple=True)                          # row-major order
        with torch.no_grad():
            self.weight.copy_(tiles.permute(0, 2, 1, 3)[brow, bcol].reshape(self.weight.shape))

    @property
    def saving(self):
        """Fraction of the dense layer's parameters that is stored."""
        return self.nnz_blocks * self.block_size ** 2 / (self.in_features * self.out_features)

    def get_ops(self):
        """The DDS operator of the 'triton' backend (None for 'dense'), created on first use."""
        try:
            return self.ops_cache[self.backend]
        except KeyError:
            op = None
            if self.backend == 'triton':
                op = matmul(self.layout.cpu(), self.block_size, 'dds', trans_a=False, trans_b=True)
            self.ops_cache[self.backend] = op
            return op

    def forward(self, x):
        """x (..., in_features) -> (..., out_features)."""
        if self.backend == 'dense':
            pad_in = self.in_features_extended - x.shape[-1]
            dense = densify_tensor(self.weight.view(1, self.nnz_blocks, self.block_size, self.block_size),
                                   self.layout.unsqueeze(0))[0, 0]
            y = F.linear(F.pad(x, (0, pad_in)) if pad_in > 0 else x, dense)
        else:
            if not x.is_cuda:
                raise NotImplementedError('Backend triton only supports GPU tensors')
            lead = x.shape[:-1]
            tokens = x.reshape(-1, x.shape[-1])
            n_tok = tokens.shape[0]
            # one zero-padding for both axes: features up to the padded fan-in, tokens up to whole blocks
            pad_in = max(self.in_features_extended - tokens.shape[1], 0)
            pad_tok = -n_tok % self.block_size
            if pad_in or pad_tok:
                tokens = F.pad(tokens, (0, pad_in, 0, pad_tok))
            # (views only, and slices only where something is cut off: under autograd a select or a slice of the
            #  result, also one that keeps everything, costs a zero-fill and a copy of the whole tensor on the way back)
            y = self.get_ops()(tokens.view(1, 1, *tokens.shape), self.weight)
            y = y.view(y.shape[2], y.shape[3])
            if pad_tok:
                y = y[:n_tok]
            y = y.reshape(*lead, y.shape[-1])
        if y.shape[-1] != self.out_features:
            y = y[..., :self.out_features]
        # the bias joins in the dtype of the product (under autocast the product is half precision)
        return y if self.bias is None else y + self.bias.to(y.dtype)
