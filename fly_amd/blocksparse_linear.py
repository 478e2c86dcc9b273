"""Pixelfly block-sparse linear layer on the HIP kernels: drop-in for
src/models/layers/blocksparse_linear.py (BlockSparseLinear :35-172,
FlatBlockButterflySparsityConfig :175-211)."""
import math
from functools import partial

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn import init

from .blocksparse_attention import instantiate
from .blocksparse_matmul import matmul
from .blocksparse_utils import densify_tensor, sparsify_tensor
from .padding import pad_to_multiple


class FlatBlockButterflySparsityConfig:
    """Sparsity pattern = sum of the first ``n_factors`` butterfly factors of size ``butterfly_size``
    ("flat butterfly"), stretched to the weight shape and reduced to blocks.

    Entry (i, j) of butterfly factor k (stride 2^k, all-ones twiddle) is nonzero iff j == i or
    j == i xor 2^k (src/ops/butterfly_factor.py:8-26), so the flat pattern is
    ``j in {i} U {i xor 2^k : k < n_factors}``; that closed form is evaluated directly here."""

    def __init__(self, butterfly_size, n_factors, block=32, global_size=0, shuffle=False):
        self.block = block
        log_n = int(math.log2(butterfly_size))
        if butterfly_size != 2 ** log_n or butterfly_size < 2:
            raise NotImplementedError('butterfly_size must be a power of 2')
        if not (1 <= n_factors <= log_n):
            raise NotImplementedError('n_factors must be a between 1 and log_2(butterfly_size)')
        self.butterfly_size = butterfly_size
        self.n_factors = n_factors
        self.global_size = global_size
        self.shuffle = shuffle

    def make_layout(self, out_features, in_features=None):
        """int32 (out_features/block, in_features/block) layout (:191-211).  A single argument means
        a square (seq, seq) attention layout."""
        if in_features is None:
            in_features = out_features
        assert out_features % self.block == 0 and in_features % self.block == 0
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
    """y = x W^T + b with W block-sparse.  `weight` is stored as (1, nnz, blk, blk) blocks in
    (out-block, in-block) row-major order, block content [out_local, in_local]; the product runs as
    DDS with the sparse operand transposed.  backend 'triton' (the name kept from the reference)
    selects the HIP kernel; 'dense' multiplies by the densified weight with a library GEMM;
    'huggingface' is not available."""

    def __init__(self, in_features, out_features, sparsity_config, bias=True,
                 backend='triton', weight_decay=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.sparsity_config = instantiate(sparsity_config)
        self.block_size = self.sparsity_config.block
        self.in_features_extended = int(math.ceil(in_features / self.block_size)) * self.block_size
        self.out_features_extended = int(math.ceil(out_features / self.block_size)) * self.block_size
        layout = self.sparsity_config.make_layout(self.out_features_extended, self.in_features_extended)
        self.register_buffer("layout", layout)
        self.nnz_blocks = self.layout.sum().item()
        if backend is None:
            backend = 'triton'
        if backend == 'huggingface':
            raise ImportError('backend huggingface (pytorch_block_sparse) is not available in this build')
        if backend not in ['triton', 'dense']:
            raise NotImplementedError(f'backend {backend} not supported')
        self.backend = backend
        self.weight = nn.Parameter(torch.empty(self.nnz_blocks, self.block_size, self.block_size))
        if bias:
            self.bias = nn.Parameter(torch.empty(out_features))
        else:
            self.register_parameter('bias', None)
        self.reset_parameters()
        if self.backend == 'triton':
            self.weight = nn.Parameter(self.weight.detach().unsqueeze(0))     # (1, nnz, blk, blk)
        if not weight_decay:
            self.weight._no_weight_decay = True
        self.ops_cache = dict()

    def reset_parameters(self) -> None:
        self.set_weights_from_dense_init(dense_init_fn_=partial(init.kaiming_uniform_, a=math.sqrt(5)))
        fan_in = self.in_features_extended
        if self.bias is not None:
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            init.uniform_(self.bias, -bound, bound)

    def set_weights_from_dense_init(self, dense_init_fn_):
        """Initialise a dense (out, in) matrix, rescale each block-row by sqrt(#cols / #nonzero cols)
        to keep the output variance, and keep the nonzero blocks (:98-109)."""
        dense_weight = torch.empty(self.out_features_extended, self.in_features_extended,
                                   device=self.weight.device, dtype=self.weight.dtype)
        dense_init_fn_(dense_weight)
        ncol = self.layout.shape[-1]
        n_nonzero_cols = self.layout.sum(dim=-1, keepdim=True)
        scaling = torch.sqrt(ncol / n_nonzero_cols)
        dense_weight *= scaling.repeat_interleave(self.block_size, dim=0).to(dense_weight.device)
        with torch.no_grad():
            blocks = sparsify_tensor(dense_weight.unsqueeze(0), self.layout.unsqueeze(0))
            self.weight.copy_(blocks.reshape(self.weight.shape))

    @property
    def saving(self):
        return self.nnz_blocks * self.block_size ** 2 / (self.in_features * self.out_features)

    def get_ops(self):
        if self.backend not in self.ops_cache:
            self.ops_cache[self.backend] = None if self.backend == 'dense' else \
                matmul(self.layout.cpu(), self.block_size, 'dds', trans_a=False, trans_b=True)
        return self.ops_cache[self.backend]

    def forward(self, x):
        """x (..., in_features) -> (..., out_features)."""
        if not x.is_cuda and self.backend != 'dense':
            raise NotImplementedError('Backend triton only supports GPU tensors')
        if x.shape[-1] < self.in_features_extended:
            x = F.pad(x, (0, self.in_features_extended - x.shape[-1]))
        if self.backend == 'triton':
            dds = self.get_ops()
            batch_shape = x.shape[:-1]
            x = x.reshape(-1, x.shape[-1])
            rows = x.shape[0]
            x = pad_to_multiple(x, multiple=self.block_size, dims=0)
            output = dds(x.view(1, 1, *x.shape), self.weight).view(x.shape[0], -1)
            if output.shape[0] > rows:
                output = output[:rows, :]
            output = output.reshape(batch_shape + (output.shape[-1],))
        else:
            weight = densify_tensor(self.weight.reshape(1, self.nnz_blocks, self.block_size, self.block_size),
                                    self.layout.unsqueeze(0))[0, 0]
            output = F.linear(x, weight)
        if output.shape[-1] > self.out_features:
            output = output[..., :self.out_features]
        return (output + self.bias.to(dtype=output.dtype)) if self.bias is not None else output
