"""T2T-ViT with pluggable tokens-to-token attention: the caller of SBLocalAttention in the
reference (src/models/modules/token_transformer.py:20-86, src/models/modules/t2t.py:20-82,
src/models/vit/t2t_vit.py:54-128,197-206, src/models/modules/vision_common.py:16-105,
src/models/modules/seq_common.py:114-169), restated with plain nn.Modules and the reference's
attribute names so that its (converted) checkpoints load.  Everything outside the two T2T attention
layers is ordinary dense PyTorch; dropouts / stochastic depth are identities (rates 0, as in the
reference's T2T-ViT configs)."""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .blocksparse_attention import instantiate


class Mlp(nn.Module):
    """fc1 -> GELU -> fc2."""

    def __init__(self, in_features, hidden_features=None, out_features=None, act_layer=nn.GELU):
        super().__init__()
        out_features = out_features or in_features
        hidden_features = hidden_features or in_features
        self.fc1 = nn.Linear(in_features, hidden_features)
        self.act = act_layer()
        self.fc2 = nn.Linear(hidden_features, out_features)

    def forward(self, x):
        return self.fc2(self.act(self.fc1(x)))


class MlpCustom(nn.Module):
    """fc1 -> act -> drop -> fc2 -> drop with either linear taken from a plugin description
    (src/models/layers/mlp.py:24-68); this is how the Pixelfly SparseLRLinear enters MLP-Mixer."""

    def __init__(self, in_features, hidden_features=None, out_features=None, act_layer=nn.GELU,
                 act_fn=None, drop=0., drop_btw_fcs=True, linear1_cfg=None, linear2_cfg=None):
        super().__init__()
        out_features = out_features or in_features
        hidden_features = hidden_features or in_features
        self.fc1 = nn.Linear(in_features, hidden_features) if linear1_cfg is None else \
            instantiate(linear1_cfg, in_features, hidden_features)
        self.act = act_layer() if act_fn is None else act_fn
        self.fc2 = nn.Linear(hidden_features, out_features) if linear2_cfg is None else \
            instantiate(linear2_cfg, hidden_features, out_features)
        self.drop = nn.Dropout(drop)
        self.drop_btw_fcs = drop_btw_fcs

    def forward(self, x):
        x = self.act(self.fc1(x))
        if self.drop_btw_fcs:
            x = self.drop(x)
        return self.drop(self.fc2(x))


class T2TAttention(nn.Module):
    """qkv projection -> attention over (B, N, heads, in_dim/heads) -> proj, skip connection from v.
    The temperature handed to the attention layer comes from the INPUT dim: (dim // heads)^-0.5
    (token_transformer.py:26-27,36)."""

    def __init__(self, dim, num_heads=8, in_dim=None, qkv_bias=False, qk_scale=None, attn_cfg=None):
        super().__init__()
        self.num_heads = num_heads
        self.in_dim = in_dim if in_dim is not None else dim
        self.scale = qk_scale or (dim // num_heads) ** -0.5
        self.qkv = nn.Linear(dim, self.in_dim * 3, bias=qkv_bias)
        self.proj = nn.Linear(self.in_dim, self.in_dim)
        self.attention_layer = None if attn_cfg is None else instantiate(attn_cfg, softmax_temp=self.scale)

    def forward(self, x):
        B, N, _ = x.shape
        q, k, v = self.qkv(x).chunk(3, dim=-1)
        v_og = v
        q, k, v = (t.reshape(B, N, self.num_heads, -1) for t in (q, k, v))
        if self.attention_layer is None:                       # dense softmax attention
            qh, kh, vh = (t.transpose(1, 2) for t in (q, k, v))
            attn = ((qh * self.scale) @ kh.transpose(-2, -1)).softmax(dim=-1)
            out = (attn @ vh).transpose(1, 2)
        else:
            out, _ = self.attention_layer(q, k, v)
        return v_og + self.proj(out.reshape(B, N, -1))


class Token_transformer(nn.Module):
    def __init__(self, dim, in_dim, num_heads, mlp_ratio=1., qkv_bias=False, qk_scale=None, attn_cfg=None):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn = T2TAttention(dim, in_dim=in_dim, num_heads=num_heads, qkv_bias=qkv_bias,
                                 qk_scale=qk_scale, attn_cfg=attn_cfg)
        self.norm2 = nn.LayerNorm(in_dim)
        self.mlp = Mlp(in_features=in_dim, hidden_features=int(in_dim * mlp_ratio), out_features=in_dim)

    def forward(self, x):
        x = self.attn(self.norm1(x))
        return x + self.mlp(self.norm2(x))


class T2T_module(nn.Module):
    """Unfold 7x7/4 -> attention1 -> Unfold 3x3/2 -> attention2 -> Unfold 3x3/2 -> Linear
    ('transformer' tokens type of src/models/modules/t2t.py:28-38,61-82)."""

    def __init__(self, img_size=224, in_chans=3, embed_dim=768, token_dim=64, attn1_cfg=None, attn2_cfg=None):
        super().__init__()
        self.soft_split0 = nn.Unfold(kernel_size=(7, 7), stride=(4, 4), padding=(2, 2))
        self.soft_split1 = nn.Unfold(kernel_size=(3, 3), stride=(2, 2), padding=(1, 1))
        self.soft_split2 = nn.Unfold(kernel_size=(3, 3), stride=(2, 2), padding=(1, 1))
        self.attention1 = Token_transformer(dim=in_chans * 7 * 7, in_dim=token_dim, num_heads=1,
                                            mlp_ratio=1.0, attn_cfg=attn1_cfg)
        self.attention2 = Token_transformer(dim=token_dim * 3 * 3, in_dim=token_dim, num_heads=1,
                                            mlp_ratio=1.0, attn_cfg=attn2_cfg)
        self.project = nn.Linear(token_dim * 3 * 3, embed_dim)
        self.num_patches = (img_size // 16) * (img_size // 16)

    @staticmethod
    def _to_image(x):
        B, L, C = x.shape
        side = int(math.sqrt(L))
        return x.transpose(1, 2).reshape(B, C, side, side)

    def forward(self, x):
        x = self.soft_split0(x).transpose(1, 2)                 # (B, 3136, 147) at 224 x 224
        x = self.soft_split1(self._to_image(self.attention1(x))).transpose(1, 2)   # (B, 784, 576)
        x = self.soft_split2(self._to_image(self.attention2(x))).transpose(1, 2)   # (B, 196, 576)
        return self.project(x)


class PositionalEncoding(nn.Module):
    """Fixed sinusoidal table added to the tokens (seq_common.py:114-169, batch_first)."""

    def __init__(self, d_model, max_len=5000):
        super().__init__()
        position = torch.arange(0.0, max_len).unsqueeze(1)
        div_term = torch.exp(-math.log(10000.0) * torch.arange(0.0, d_model, 2.0) / d_model)
        pe = torch.empty(max_len, d_model)
        pe[:, 0::2] = torch.sin(position * div_term)
        pe[:, 1::2] = torch.cos(position * div_term)
        self.register_buffer('pe', pe.unsqueeze(0))

    def forward(self, x):
        return x + self.pe[:, :x.size(1)]


class AttentionSimple(nn.Module):
    """Dense self-attention with a packed qkv projection (vision_common.py:16-81)."""

    def __init__(self, dim, num_heads=8, qkv_bias=False, qk_scale=None):
        super().__init__()
        self.num_heads = num_heads
        self.scale = qk_scale or (dim // num_heads) ** -0.5
        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.proj = nn.Linear(dim, dim)

    def forward(self, x):
        B, N, C = x.shape
        qkv = self.qkv(x).reshape(B, N, 3, self.num_heads, C // self.num_heads).permute(2, 0, 3, 1, 4)
        q, k, v = qkv[0], qkv[1], qkv[2]
        attn = F.softmax((q @ k.transpose(-2, -1)) * self.scale, dim=-1)
        return self.proj((attn @ v).transpose(1, 2).reshape(B, N, C))


class Block(nn.Module):
    def __init__(self, dim, num_heads, mlp_ratio=4., qkv_bias=False, qk_scale=None, mlp_cfg=None):
        super().__init__()
        self.norm1 = nn.LayerNorm(dim)
        self.attn = AttentionSimple(dim, num_heads=num_heads, qkv_bias=qkv_bias, qk_scale=qk_scale)
        self.norm2 = nn.LayerNorm(dim)
        hidden = int(dim * mlp_ratio)
        self.mlp = Mlp(in_features=dim, hidden_features=hidden) if mlp_cfg is None else \
            instantiate(mlp_cfg, in_features=dim, hidden_features=hidden)

    def forward(self, x):
        x = x + self.attn(self.norm1(x))
        return x + self.mlp(self.norm2(x))


class T2T_ViT(nn.Module):
    def __init__(self, img_size=224, in_chans=3, num_classes=1000, embed_dim=768, depth=12, num_heads=12,
                 mlp_ratio=4., qkv_bias=False, qk_scale=None, token_dim=64,
                 t2tattn1_cfg=None, t2tattn2_cfg=None, mlp_cfg=None):
        super().__init__()
        self.num_classes = num_classes
        self.num_features = self.embed_dim = embed_dim
        self.patch_embed = T2T_module(img_size=img_size, in_chans=in_chans, embed_dim=embed_dim,
                                      token_dim=token_dim, attn1_cfg=t2tattn1_cfg, attn2_cfg=t2tattn2_cfg)
        self.cls_token = nn.Parameter(torch.zeros(1, 1, embed_dim))
        self.pos_embed = PositionalEncoding(embed_dim, max_len=self.patch_embed.num_patches + 1)
        self.blocks = nn.Sequential(*[Block(embed_dim, num_heads, mlp_ratio, qkv_bias, qk_scale, mlp_cfg)
                                      for _ in range(depth)])
        self.norm = nn.LayerNorm(embed_dim)
        self.head = nn.Linear(embed_dim, num_classes) if num_classes > 0 else nn.Identity()
        nn.init.trunc_normal_(self.cls_token, std=.02)
        self.apply(self._init_weights)                          # t2t_vit.py:88-99

    @staticmethod
    def _init_weights(m):
        """Truncated-normal(0.02) weights and zero biases for every linear-like layer, the Pixelfly ones
        (block-sparse, low-rank, sparse + low-rank) through their dense-initialisation hooks; unit / zero
        LayerNorm affine parameters (t2t_vit.py:88-99)."""
        from .blocksparse_linear import BlockSparseLinear
        from .fastlinear import LowRank, SparseLRLinear
        if isinstance(m, nn.LayerNorm):
            nn.init.ones_(m.weight)
            nn.init.zeros_(m.bias)
            return
        if not isinstance(m, (nn.Linear, BlockSparseLinear, LowRank, SparseLRLinear)):
            return
        if m.bias is not None:
            nn.init.zeros_(m.bias)

        def small_normal_(w):
            return nn.init.trunc_normal_(w, std=.02)
        if isinstance(m, nn.Linear):
            small_normal_(m.weight)
        elif isinstance(m, (BlockSparseLinear, LowRank)):     # (SparseLRLinear's two halves are visited as children)
            m.set_weights_from_dense_init(small_normal_)

    def forward_features(self, x):
        x = self.patch_embed(x)
        x = torch.cat((self.cls_token.expand(x.shape[0], -1, -1), x), dim=1)
        x = self.norm(self.blocks(self.pos_embed(x)))
        return x[:, 0]

    def forward(self, x):
        return self.head(self.forward_features(x))


def t2t_vit_t_14(**kwargs):
    """T2T-ViT-t-14: transformer tokens-to-token, embed 384, depth 14, 6 heads, mlp_ratio 3
    (t2t_vit.py:197-206)."""
    return T2T_ViT(embed_dim=384, depth=14, num_heads=6, mlp_ratio=3., **kwargs)


def convert_t2t_vit_state_dict(state_dict):
    """State dict of a published T2T-ViT checkpoint -> the names of this model (the mapping of the
    reference's conversion script, scripts/convert_checkpoint_t2t_vit.py:19-31, and the unwrapping of
    its loader, src/eval.py:22-32): the weights may sit under the single key 'state_dict_ema';
    'pos_embed' becomes 'pos_embed.pe' and the 'tokens_to_token.' prefix 'patch_embed.'.  Returns a
    new dict; the tensors are not copied.  Already converted dicts come back unchanged."""
    if set(state_dict.keys()) == {'state_dict_ema'}:
        state_dict = state_dict['state_dict_ema']

    def rename(key):
        if key == 'pos_embed':
            return 'pos_embed.pe'
        if key.startswith('tokens_to_token.'):
            return 'patch_embed.' + key[len('tokens_to_token.'):]
        return key

    return {rename(k): v for k, v in state_dict.items()}
