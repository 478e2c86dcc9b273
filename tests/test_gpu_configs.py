"""BASELINE configs 3, 4 and 5 on the GPU against the oracle (GPU box only)."""
import copy
import math

import pytest
import torch
import torch.nn as nn

from conftest import rel_err
from oracle import sblocal as osb
from oracle import blocksparse as ob

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'


class OracleSBLocal(nn.Module):
    """Attention plugin that evaluates the CPU oracle with a given projection matrix."""
    def __init__(self, P, lc, temp):
        super().__init__()
        self.P, self.lc, self.temp = P, lc, temp

    def forward(self, q, k, v):
        out, _ = osb.sblocal_attention(q, k, v, self.P, self.lc, softmax_temp=self.temp)
        return out, None


def _sb_cfg():
    return {'_target_': 'src.models.attention.sblocal_attention.SBLocalAttention', 'local_context': 256,
            'dim_heads': 64, 'nb_features': 128}


def test_config3_t2t_vit_logits_parity():
    """T2T-ViT-t-14, both T2T layers on SBLocalAttention (window 256, 128 features, temperatures
    147^-0.5 and 576^-0.5): logits of the HIP-attention model on the GPU against the same weights
    with oracle attention on the CPU (batch 2 for the CPU side), then the full batch of 64 on the GPU."""
    import fly_amd
    torch.manual_seed(0)
    model = fly_amd.t2t_vit_t_14(t2tattn1_cfg=_sb_cfg(), t2tattn2_cfg=_sb_cfg()).eval()
    layers = [model.patch_embed.attention1.attn, model.patch_embed.attention2.attn]
    for lay in layers:                                   # fixed seeded projection per layer
        lay.attention_layer.feature_map.new_feature_map('cpu')
    ref = copy.deepcopy(model)
    for lay_ref, lay in zip([ref.patch_embed.attention1.attn, ref.patch_embed.attention2.attn], layers):
        P = lay.attention_layer.feature_map.projection_matrix.clone()
        assert P.shape == (64, 64) and float(P.abs().sum()) > 0
        lay_ref.attention_layer = OracleSBLocal(P, 256, lay.scale)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 3, 224, 224, generator=g)
    with torch.no_grad():
        want = ref(x[:2])
        gpu = model.to(DEV)
        got = gpu(x[:2].to(DEV)).cpu()
        print('logits rel err', rel_err(got, want), 'max elementwise rel',
              float(((got - want).abs() / want.abs().clamp_min(1e-3)).max()), flush=True)
        assert got.shape == (2, 1000)
        assert rel_err(got, want) <= 1e-4
        full = gpu(x.to(DEV))
        torch.cuda.synchronize()
        assert full.shape == (64, 1000) and bool(torch.isfinite(full).all())
        assert rel_err(full[:2].cpu(), want) <= 1e-4


def atol_needed(got, ref, rtol=1e-4):
    """The smallest atol with which torch.allclose(got, ref, rtol, atol) holds (negative: rtol alone suffices)."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return float(((got - ref).abs() - rtol * ref.abs()).max())


@pytest.mark.parametrize('L,dim', [(3136, 147), (784, 576)])
def test_config3_attention_layers_parity(L, dim):
    """Both Scatterbrain-local layers of T2T-ViT at their real size (batch 4): 1e-4 of the tensor's maximum, and
    elementwise rtol 1e-4 with a stated atol.  The outputs are of order one here (unscaled N(0,1) values), so an atol
    of 1e-6 is float32 resolution: the float32 oracle itself needs 5e-7.  The fp32-pipe kernels hold 1e-6; the default
    kernels (bf16 pieces, V rounded to 16 bits) need 2e-6 .. 4.2e-6 and are held to 6e-6 -- the measured values are
    printed."""
    from fly_amd import sblocal_forward
    g = torch.Generator().manual_seed(L)
    q, k, v = (torch.randn(4, L, 1, 64, generator=g) for _ in range(3))
    P = osb.gaussian_orthogonal_random_matrix(64, 64, generator=g)
    t = dim ** -0.5
    ref_out, ref_ln = osb.sblocal_attention(q.double(), k.double(), v.double(), P.double(), 256, softmax_temp=t)
    for exact, atol in ((False, 6e-6), (True, 1e-6)):
        out, ln = sblocal_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), 256, softmax_temp=t, exact_fp32=exact)
        need = atol_needed(out, ref_out)
        print('exact_fp32', exact, 'out', rel_err(out, ref_out), 'log-normaliser', rel_err(ln, ref_ln),
              'atol needed at rtol 1e-4', need, flush=True)
        assert rel_err(out, ref_out) <= 1e-4 and rel_err(ln, ref_ln) <= 1e-4
        assert need <= atol, need
        assert torch.allclose(ln.double().cpu(), ref_ln, rtol=1e-4, atol=1e-6)


def test_config4_pixelfly_mlp_bf16():
    """MLP-Mixer-B channel MLP 768 -> 3072 -> 768 in bf16: SparseLRLinear = flat butterfly (8, 2) block 32
    sparse term (HIP DDS kernel) + rank 96 low-rank term + sigmoid gate, on 256 x 196 tokens."""
    import fly_amd
    torch.manual_seed(0)
    cfg = fly_amd.FlatBlockButterflySparsityConfig(8, 2, block=32)
    lin = {'_target_': 'src.models.layers.fastlinear.SparseLRLinear',
           'sparse_cfg': {'_target_': 'src.models.layers.blocksparse_linear.BlockSparseLinear', 'sparsity_config': cfg},
           'rank': 96, 'gating': True}
    mlp = fly_amd.MlpCustom(768, 3072, linear1_cfg=lin, linear2_cfg=lin)
    assert int(mlp.fc1.sparse.layout.sum()) == 864 and int(mlp.fc2.sparse.layout.sum()) == 864
    g = torch.Generator().manual_seed(1)
    x = torch.randn(256 * 196, 768, generator=g).bfloat16()
    gpu = copy.deepcopy(mlp).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        y = gpu(x.to(DEV))
        torch.cuda.synchronize()
        assert y.shape == (256 * 196, 768) and y.dtype == torch.bfloat16

        def slr_ref(mod, inp):        # oracle: fp32 math on the bf16-rounded weights and inputs
            w = lambda p: p.detach().bfloat16().float()
            sp = ob.blocksparse_linear(inp, w(mod.sparse.weight), mod.sparse.layout, 32, None, mod.out_features)
            return ob.sparse_lr_linear(inp, sp, w(mod.low_rank.lr_weight1), w(mod.low_rank.lr_weight2),
                                       w(mod.gate.weight), w(mod.gate.bias), w(mod.bias))
        n = 4096                                       # oracle on a slice of the tokens
        xs = x[:n].float()
        h_gpu = gpu.fc1(x[:n].to(DEV)).float().cpu()
        h_ref = slr_ref(mlp.fc1, xs)
        assert rel_err(h_gpu, h_ref) <= 2e-2
        ref = slr_ref(mlp.fc2, torch.nn.functional.gelu(h_ref.bfloat16().float()).bfloat16().float())
        assert rel_err(y[:n].float().cpu(), ref) <= 2e-2
        # the sparse term alone, all tokens, fc1 shape: DDS against the dense formula
        s_gpu = gpu.fc1.sparse(x.to(DEV)).float().cpu()
        s_ref = ob.blocksparse_linear(x.float(), mlp.fc1.sparse.weight.detach().bfloat16().float(),
                                      mlp.fc1.sparse.layout, 32, None, 3072)
        assert rel_err(s_gpu, s_ref) <= 2e-2


def test_config5_long_sequence_bf16():
    """B=1, H=16, L=16384, d=64, window 1024, 256 features, bf16 inputs with 5 % of the key rows
    scaled by 8.  The GPU runs all 16 heads; the oracle (fp32 on the bf16-rounded inputs) checks two."""
    from fly_amd import sblocal_forward
    g = torch.Generator().manual_seed(0)
    B, L, H, E = 1, 16384, 16, 64
    q = torch.randn(B, L, H, E, generator=g)
    k = torch.randn(B, L, H, E, generator=g)
    v = torch.randn(B, L, H, E, generator=g)
    idx = torch.randperm(L, generator=g)[: L // 20]
    k[:, idx] *= 8
    P = osb.gaussian_orthogonal_random_matrix(128, 64, generator=g)
    qb, kb, vb = q.bfloat16(), k.bfloat16(), v.bfloat16()
    out, ln = sblocal_forward(qb.to(DEV), kb.to(DEV), vb.to(DEV), P.to(DEV), 1024)
    torch.cuda.synchronize()
    assert out.shape == (B, L, H, E) and out.dtype == torch.bfloat16 and bool(torch.isfinite(out.float()).all())
    heads = [3, 12]
    sel = lambda t: t[:, :, heads].float()
    ref_out, ref_ln = osb.sblocal_attention(sel(qb), sel(kb), sel(vb), P, 1024, chunk=512)
    assert rel_err(out[:, :, heads], ref_out) <= 2e-2
    assert rel_err(ln[:, heads], ref_ln) <= 2e-2
    # normalisation identity at full size: values of one give outputs of one
    ones, _ = sblocal_forward(qb.to(DEV), kb.to(DEV), torch.ones_like(vb).to(DEV), P.to(DEV), 1024)
    assert float((ones.float() - 1).abs().max()) <= 1e-2


def test_matmul_backward_matches_dense_autograd():
    """Gradients of the three modes against autograd through the dense formula (the reference's
    backward re-uses its kernels with permuted roles, blocksparse_matmul.py:562-587)."""
    from fly_amd import matmul
    from fly_amd.blocksparse_utils import densify_tensor, sparsify_tensor
    g = torch.Generator().manual_seed(0)
    block, Z, H, p, r = 32, 2, 2, 3, 4
    layout = (torch.rand(H, p, r, generator=g) < 0.6).long()
    nnz = int(layout.sum())
    a = torch.randn(Z, H, p * block, 48, generator=g).to(DEV).requires_grad_()
    b = torch.randn(Z, H, r * block, 48, generator=g).to(DEV).requires_grad_()
    c = matmul(layout, block, 'sdd', trans_b=True)(a, b)
    w = torch.randn(c.shape, generator=g).to(DEV)
    (c * w).sum().backward()
    a2, b2 = a.detach().clone().requires_grad_(), b.detach().clone().requires_grad_()
    (sparsify_tensor(a2 @ b2.transpose(-1, -2), layout) * w).sum().backward()
    assert rel_err(a.grad, a2.grad) <= 1e-5 and rel_err(b.grad, b2.grad) <= 1e-5

    sp = torch.randn(Z, nnz, block, block, generator=g).to(DEV).requires_grad_()
    d = torch.randn(Z, H, r * block, 48, generator=g).to(DEV).requires_grad_()   # SDD in the backward needs K % 16 == 0
    out = matmul(layout, block, 'dsd')(sp, d)
    w = torch.randn(out.shape, generator=g).to(DEV)
    (out * w).sum().backward()
    sp2, d2 = sp.detach().clone().requires_grad_(), d.detach().clone().requires_grad_()
    ((densify_tensor(sp2, layout) @ d2) * w).sum().backward()
    assert rel_err(sp.grad, sp2.grad) <= 1e-5 and rel_err(d.grad, d2.grad) <= 1e-5

    x = torch.randn(1, 1, 64, r * block, generator=g).to(DEV).requires_grad_()
    wsp = torch.randn(1, int(layout[0].sum()), block, block, generator=g).to(DEV).requires_grad_()
    y = matmul(layout[0], block, 'dds', trans_b=True)(x, wsp)
    w = torch.randn(y.shape, generator=g).to(DEV)
    (y * w).sum().backward()
    x2, w2 = x.detach().clone().requires_grad_(), wsp.detach().clone().requires_grad_()
    ((x2 @ densify_tensor(w2, layout[:1]).transpose(-1, -2)) * w).sum().backward()
    assert rel_err(x.grad, x2.grad) <= 1e-5 and rel_err(wsp.grad, w2.grad) <= 1e-5


def test_row_ops_backward_match_dense_autograd():
    """Gradients of the block softmax (with scale and an additive key-padding mask), logsumexp and row sum
    against autograd through the dense formulas on -inf / zero filled matrices
    (the reference's own checks: tests/models/attention/test_blocksparse_logsumexp.py:25-33)."""
    from fly_amd import softmax, logsumexp, blocksparse_sum
    from fly_amd.blocksparse_utils import densify_tensor, sparsify_tensor
    g = torch.Generator().manual_seed(3)
    block, Z, H, p, r = 16, 2, 2, 3, 4
    layout = (torch.rand(H, p, r, generator=g) < 0.6).long()
    layout[:, :, 0] = 1                                   # no empty block-row: every row has a finite entry
    nnz = int(layout.sum())
    x0 = torch.randn(Z, nnz, block, block, generator=g).to(DEV)
    w = torch.randn(Z, nnz, block, block, generator=g).to(DEV)
    kpm = torch.zeros(Z, r * block)
    kpm[1, -5:] = float('-inf')
    for name in ('softmax', 'logsumexp', 'sum'):
        print('case', name, flush=True)
        x = x0.clone().requires_grad_()
        xd = x0.clone().requires_grad_()
        if name == 'softmax':
            y = softmax(layout, block)(x * 1.0, scale=0.7, key_padding_mask=kpm.to(DEV))
            dense = densify_tensor(xd * 0.7, layout, float('-inf')) + kpm.to(DEV)[:, None, None, :]
            ref = sparsify_tensor(torch.softmax(dense, dim=-1), layout)
            (y * w).sum().backward()
            (ref * w).sum().backward()
        else:
            op = logsumexp(layout, block) if name == 'logsumexp' else blocksparse_sum(layout, block)
            y = op(x)
            wr = torch.randn(y.shape, generator=g).to(DEV)
            if name == 'logsumexp':
                ref = torch.logsumexp(densify_tensor(xd, layout, float('-inf')), dim=-1)
            else:
                ref = densify_tensor(xd, layout, 0.0).sum(-1)
            (y * wr).sum().backward()
            (ref * wr).sum().backward()
        assert rel_err(y, ref) <= 1e-5
        assert rel_err(x.grad, xd.grad) <= 1e-5, name


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('p,r', [(4, 6), (3, 40), (5, 61)])
def test_softmax_backward_kernel_matches_dense_autograd(p, r, dtype):
    """The one-pass gradient kernel of the block softmax (32x32 blocks, 2-byte types; 4 / 13 / 16
    register slots) against autograd through the dense softmax on the same rounded inputs."""
    from fly_amd import softmax
    from fly_amd.blocksparse_utils import densify_tensor, sparsify_tensor
    print('case', p, r, dtype, flush=True)
    g = torch.Generator().manual_seed(10 * p + r)
    block, Z, H = 32, 2, 2
    layout = (torch.rand(H, p, r, generator=g) < 0.7).long()
    layout[:, :, 0] = 1
    layout[0, 1, :] = 1                                   # a full block-row: the longest column list
    nnz = int(layout.sum())
    x0 = torch.randn(Z, nnz, block, block, generator=g).to(dtype).to(DEV)
    w = torch.randn(Z, nnz, block, block, generator=g).to(dtype).to(DEV)
    kpm = torch.zeros(Z, r * block)
    kpm[1, -37:] = float('-inf')
    x = x0.clone().requires_grad_()
    y = softmax(layout, block)(x * 1.0, scale=0.3, key_padding_mask=kpm.to(DEV))
    (y.float() * w.float()).sum().backward()
    xd = x0.float().clone().requires_grad_()
    dense = densify_tensor(xd * 0.3, layout, float('-inf')) + kpm.to(DEV)[:, None, None, :]
    ref = sparsify_tensor(torch.softmax(dense, dim=-1), layout)
    (ref * w.float()).sum().backward()
    assert x.grad.dtype == dtype
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    assert rel_err(x.grad.float(), xd.grad) <= tol, rel_err(x.grad.float(), xd.grad)


def test_bf16_gradients_on_the_tiled_kernels():
    """The gradient paths of the 2-byte tiled kernels against autograd through the dense formulas on the
    same rounded inputs: dQ / dK (dsd, transposed dsd), dP (sdd), dV (transposed dsd) of an attention-like
    sdd -> dsd chain on a band layout, and dx (dds on untransposed blocks) / dW (split-K sdd over 1024
    tokens) of a block-sparse linear layer."""
    from fly_amd import matmul
    from fly_amd.blocksparse_utils import densify_tensor, sparsify_tensor
    g = torch.Generator().manual_seed(1)
    block, Z, H, nb, d = 32, 2, 2, 12, 64
    r_ = torch.arange(nb)
    layout = ((r_.view(-1, 1) - r_.view(1, -1)).abs() <= 2).long().unsqueeze(0).repeat(H, 1, 1)
    bf = torch.bfloat16
    q, k, v = (torch.randn(Z, H, nb * block, d, generator=g).to(bf).to(DEV).requires_grad_() for _ in range(3))
    s = matmul(layout, block, 'sdd', trans_b=True)(q, k)
    o = matmul(layout, block, 'dsd')(s * 0.05, v)
    w = torch.randn(o.shape, generator=g).to(DEV)
    (o.float() * w).sum().backward()
    q2, k2, v2 = (x.detach().float().requires_grad_() for x in (q, k, v))
    s2 = sparsify_tensor(q2 @ k2.transpose(-1, -2), layout)
    o2 = densify_tensor(s2 * 0.05, layout) @ v2
    (o2 * w).sum().backward()
    for got, ref, name in ((q.grad, q2.grad, 'dq'), (k.grad, k2.grad, 'dk'), (v.grad, v2.grad, 'dv')):
        assert rel_err(got.float(), ref) <= 3e-2, (name, rel_err(got.float(), ref))

    lay1 = layout[0]
    x = torch.randn(1, 1, 1024, nb * block, generator=g).to(bf).to(DEV).requires_grad_()
    wsp = (torch.randn(1, int(lay1.sum()), block, block, generator=g) * 0.1).to(bf).to(DEV).requires_grad_()
    y = matmul(lay1, block, 'dds', trans_b=True)(x, wsp)
    wy = torch.randn(y.shape, generator=g).to(bf).to(DEV)
    y.backward(wy)
    x2, w2 = x.detach().float().requires_grad_(), wsp.detach().float().requires_grad_()
    (x2 @ densify_tensor(w2, lay1.unsqueeze(0)).transpose(-1, -2)).backward(wy.float())
    assert rel_err(x.grad.float(), x2.grad) <= 2e-2 and rel_err(wsp.grad.float(), w2.grad) <= 2e-2
