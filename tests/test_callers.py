"""CPU checks of the restated callers (T2T-ViT, MlpCustom): module graph, shapes, the temperature
handed to the attention plugin, dense-attention equivalence.  No kernels run here."""
import math

import torch
import torch.nn as nn

import fly_amd
from fly_amd.t2t_vit import T2TAttention, T2T_module, Token_transformer, MlpCustom


class _Recorder(nn.Module):
    """Stand-in attention plugin: records the temperature and the layout it is called with."""
    def __init__(self, softmax_temp=None, tag=None):
        super().__init__()
        self.softmax_temp, self.tag, self.shapes = softmax_temp, tag, None

    def forward(self, q, k, v):
        self.shapes = (tuple(q.shape), tuple(k.shape), tuple(v.shape))
        t = self.softmax_temp
        att = torch.softmax(torch.einsum('bthe,bshe->bhts', q, k) * t, dim=-1)
        return torch.einsum('bhts,bshd->bthd', att, v), None


def test_t2t_attention_temperature_layout_and_dense_equivalence():
    torch.manual_seed(0)
    cfg = {'_target_': 'tests.test_callers._Recorder', 'tag': 'x'}
    import sys
    sys.modules.setdefault('tests.test_callers', sys.modules[__name__])
    plug = T2TAttention(dim=147, num_heads=1, in_dim=64, attn_cfg=cfg)
    dense = T2TAttention(dim=147, num_heads=1, in_dim=64, attn_cfg=None)
    dense.load_state_dict({k: v for k, v in plug.state_dict().items() if not k.startswith('attention_layer')})
    assert plug.attention_layer.softmax_temp == 147 ** -0.5          # from the INPUT dim, not 64
    x = torch.randn(2, 50, 147)
    y = plug(x)
    assert plug.attention_layer.shapes == ((2, 50, 1, 64),) * 3      # (B, N, heads, head_dim)
    assert torch.allclose(y, dense(x), atol=1e-5)
    # skip connection from v: zero the output projection -> the layer returns v
    with torch.no_grad():
        dense.proj.weight.zero_(); dense.proj.bias.zero_()
    v = dense.qkv(x).chunk(3, dim=-1)[2]
    assert torch.allclose(dense(x), v)


def test_t2t_module_shape_walk_through():
    torch.manual_seed(0)
    mod = T2T_module(img_size=224, embed_dim=384, token_dim=64)
    x = torch.randn(1, 3, 224, 224)
    t0 = mod.soft_split0(x).transpose(1, 2)
    assert t0.shape == (1, 3136, 147)
    t1 = mod.soft_split1(mod._to_image(mod.attention1(t0))).transpose(1, 2)
    assert t1.shape == (1, 784, 576)
    t2 = mod.soft_split2(mod._to_image(mod.attention2(t1))).transpose(1, 2)
    assert t2.shape == (1, 196, 576)
    assert mod(x).shape == (1, 196, 384) and mod.num_patches == 196
    assert mod.attention2.attn.scale == 576 ** -0.5


def test_t2t_vit_t_14_structure():
    torch.manual_seed(0)
    model = fly_amd.t2t_vit_t_14()
    n = sum(p.numel() for p in model.parameters())
    assert abs(n - 21.5e6) < 0.2e6                                   # the published size of T2T-ViT-t-14
    sd = model.state_dict()
    for key in ['cls_token', 'pos_embed.pe', 'patch_embed.attention1.attn.qkv.weight', 'patch_embed.project.weight',
                'blocks.13.mlp.fc2.bias', 'norm.weight', 'head.weight']:
        assert key in sd
    assert sd['pos_embed.pe'].shape == (1, 197, 384) and sd['blocks.0.attn.qkv.weight'].shape == (1152, 384)
    assert sd['blocks.0.mlp.fc1.weight'].shape == (1152, 384)        # mlp_ratio 3
    assert float(sd['head.bias'].abs().max()) == 0 and float(sd['norm.weight'].min()) == 1
    pe = sd['pos_embed.pe'][0]
    assert torch.allclose(pe[5, 0::2], torch.sin(5 * torch.exp(-math.log(10000.0) * torch.arange(0.0, 384, 2.0) / 384)))
    with_attn = fly_amd.t2t_vit_t_14(
        t2tattn1_cfg={'_target_': 'src.models.attention.sblocal_attention.SBLocalAttention', 'local_context': 256,
                      'dim_heads': 64, 'nb_features': 128},
        t2tattn2_cfg={'_target_': 'src.models.attention.sblocal_attention.SBLocalAttention', 'local_context': 256,
                      'dim_heads': 64, 'nb_features': 128})
    a1 = with_attn.patch_embed.attention1.attn.attention_layer
    a2 = with_attn.patch_embed.attention2.attn.attention_layer
    assert isinstance(a1, fly_amd.SBLocalAttention) and a1.softmax_temp == 147 ** -0.5 and a2.softmax_temp == 576 ** -0.5
    assert 'patch_embed.attention1.attn.attention_layer.feature_map.projection_matrix' in with_attn.state_dict()


def test_mlp_custom_with_plugin_linears():
    torch.manual_seed(0)
    cfg = fly_amd.FlatBlockButterflySparsityConfig(8, 2, block=32)
    lin = {'_target_': 'src.models.layers.fastlinear.SparseLRLinear',
           'sparse_cfg': {'_target_': 'src.models.layers.blocksparse_linear.BlockSparseLinear',
                          'sparsity_config': cfg, 'backend': 'dense'},
           'rank': 8}
    mlp = MlpCustom(256, 512, linear1_cfg=lin, linear2_cfg=lin)
    assert isinstance(mlp.fc1, fly_amd.SparseLRLinear) and mlp.fc2.out_features == 256
    x = torch.randn(3, 7, 256)
    want = mlp.fc2(torch.nn.functional.gelu(mlp.fc1(x)))
    assert torch.allclose(mlp(x), want)
    plain = MlpCustom(16, 32)
    assert isinstance(plain.fc1, nn.Linear) and plain(torch.randn(2, 16)).shape == (2, 16)


def test_published_checkpoint_names_convert_and_load():
    """A state dict under the names of the published T2T-ViT checkpoints ('tokens_to_token.*', a bare
    'pos_embed', everything under 'state_dict_ema') loads after conversion, strictly
    (scripts/convert_checkpoint_t2t_vit.py:19-31)."""
    torch.manual_seed(0)
    small = dict(embed_dim=64, depth=1, num_heads=2, mlp_ratio=1., token_dim=16, num_classes=10)
    src = fly_amd.T2T_ViT(**small)
    published = {}
    for k, v in src.state_dict().items():
        k = 'pos_embed' if k == 'pos_embed.pe' else k
        k = 'tokens_to_token.' + k[len('patch_embed.'):] if k.startswith('patch_embed.') else k
        published[k] = v.clone()
    assert 'pos_embed' in published and any(k.startswith('tokens_to_token.attention1') for k in published)
    converted = fly_amd.convert_t2t_vit_state_dict({'state_dict_ema': published})
    assert set(converted) == set(src.state_dict())
    dst = fly_amd.T2T_ViT(**small)
    dst.load_state_dict(converted, strict=True)
    x = torch.randn(2, 3, 224, 224)
    assert torch.equal(src.eval()(x), dst.eval()(x))
    assert fly_amd.convert_t2t_vit_state_dict(converted).keys() == converted.keys()      # idempotent


def test_vit_initialisation_reaches_the_pixelfly_layers():
    """T2T_ViT._init_weights (t2t_vit.py:88-99): with Pixelfly linears plugged into the blocks' MLPs the
    biases are zero and the weights come from a truncated normal(0.02) dense draw -- block-sparse weights
    rescaled per block-row, low-rank factors from its projection -- not from the layers' own defaults."""
    torch.manual_seed(0)
    cfg = fly_amd.FlatBlockButterflySparsityConfig(4, 2, block=16)
    lin = {'_target_': 'src.models.layers.fastlinear.SparseLRLinear',
           'sparse_cfg': {'_target_': 'src.models.layers.blocksparse_linear.BlockSparseLinear',
                          'sparsity_config': cfg, 'backend': 'dense'},
           'rank': 4, 'gating': True}
    mlp_cfg = {'_target_': 'src.models.layers.mlp.MlpCustom', 'linear1_cfg': lin, 'linear2_cfg': lin}
    model = fly_amd.T2T_ViT(embed_dim=64, depth=1, num_heads=2, mlp_ratio=1., token_dim=16, num_classes=10,
                            mlp_cfg=mlp_cfg)
    fc1 = model.blocks[0].mlp.fc1
    assert isinstance(fc1, fly_amd.SparseLRLinear)
    assert float(fc1.bias.detach().abs().max()) == 0.0 and float(fc1.gate.bias.detach().abs().max()) == 0.0
    # normal with std 0.02, block-rows rescaled by sqrt(cols / nonzero cols) = sqrt(4 / 3): std 0.0231
    # (the layer's own default, uniform(+-1/8) times the same factor, has std 0.083)
    w = fc1.sparse.weight.detach()
    assert 0.021 < float(w.std()) < 0.025
    # the low-rank factors reproduce a rank-4 matrix whose entries are of the dense draw's size
    lr = (fc1.low_rank.lr_weight2 @ fc1.low_rank.lr_weight1).detach()
    assert lr.shape == (64, 64) and float(lr.std()) < 0.02
