"""fly_amd -- MI355X (gfx950) implementation of the Scatterbrain / Pixelfly hot path of
HazyResearch/fly: SBLocalAttention and the block-sparse matmul / softmax family, as hand-written
HIP kernels behind the reference's module interfaces.  The kernels live in ``libflyhip.so``
(built from ``csrc/`` by ``python -m fly_amd.build``); nothing here falls back to a CPU path."""
from .masking import FullMask, LengthMask, TriangularCausalMask
from .feature_maps_sb import SBPerformerFeatures, gaussian_orthogonal_random_matrix
from .sblocal_attention import SBLocalAttention, sblocal_forward, sblocal_attention_fn
from .sblocal_backward import sblocal_backward
from .local_attention import LocalAttention, local_forward, local_attention_fn, local_backward
from .blocksparse_utils import sparsify_tensor, densify_tensor, mask_tensor, sparsify_broadcast_tensor
from .blocksparse_matmul import matmul
from .blocksparse_softmax import softmax, logsumexp, blocksparse_sum
from .blocksparse_fused import fused_attention
from .blocksparse_attention import BlockSparseAttention
from .sbblocksparse_attention import SBBlockSparseAttention
from .blocksparse_linear import BlockSparseLinear, FlatBlockButterflySparsityConfig
from .fastlinear import LowRank, SparseLRLinear
from .t2t_vit import (T2T_ViT, T2T_module, T2TAttention, Token_transformer, MlpCustom, t2t_vit_t_14,
                      convert_t2t_vit_state_dict)
from .multihead_attention import MultiheadAttention

__all__ = ['FullMask', 'LengthMask', 'TriangularCausalMask', 'SBPerformerFeatures',
           'gaussian_orthogonal_random_matrix', 'SBLocalAttention', 'sblocal_forward', 'sblocal_attention_fn', 'sblocal_backward', 'LocalAttention', 'local_forward', 'local_attention_fn', 'local_backward',
           'sparsify_tensor', 'densify_tensor', 'mask_tensor', 'sparsify_broadcast_tensor',
           'matmul', 'softmax', 'logsumexp', 'blocksparse_sum', 'BlockSparseAttention', 'fused_attention',
           'SBBlockSparseAttention',
           'BlockSparseLinear', 'FlatBlockButterflySparsityConfig', 'LowRank', 'SparseLRLinear',
           'T2T_ViT', 'T2T_module', 'T2TAttention', 'Token_transformer', 'MlpCustom', 't2t_vit_t_14',
           'convert_t2t_vit_state_dict', 'MultiheadAttention']
